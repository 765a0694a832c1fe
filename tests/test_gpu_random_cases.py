"""Seeded random shapes and hyper-parameters: update-only bit-exact against the oracle, the fused
step bit-exact given the GPU's own contraction, the accumulator-resident fused step equal to the
two-kernel one, forward / input gradient within tolerance of a double-precision product."""
import numpy as np
import pytest
import torch

from tests import synth
from tests.test_gpu_parity import dev, host, ops  # noqa: F401  (fixture)

pytestmark = pytest.mark.gpu
F = np.float32


def random_hypers(rng):
    return dict(lr=float(10 ** rng.uniform(-4, 0)), lr_scale=float(rng.choice([0.0, 0.0, 0.01, 0.05])),
                rms_beta=float(rng.choice([0.0, 0.5, 0.9, 0.99])), rms_eps=float(10 ** rng.uniform(-8, -2)))


def dense_cases():
    rng = np.random.default_rng(2024)
    cases = []
    for i in range(36):
        n_in = 4 * int(rng.integers(1, 5000)) if i % 3 else 4 * int(rng.integers(1, 64))
        n_out = int(rng.integers(1, max(2, 400000 // n_in)))
        cases.append((i, n_out, n_in, int(rng.integers(1, 12))))
    return cases


@pytest.mark.parametrize("case", dense_cases(), ids=lambda c: "i%d_out%d_in%d_C%d" % c)
def test_random_update_only_cases_are_bit_exact(ops, oracle, case):
    i, n_out, n_in, C = case
    rng = np.random.default_rng(1000 + i)
    hp = random_hypers(rng)
    g_sigma = float(10 ** rng.uniform(-6, 1))
    _, state, G, scale, v = synth.counter_case(500 + i, n_out, n_in, C, g_sigma, full_range=bool(i % 5 == 0),
                                               oracle=oracle)
    if i % 7 == 0:
        G[rng.random(G.shape) < 0.3] = 0.0          # exact zeros among the gradients
    d = [dev(state), dev(scale), dev(v)]
    seed = int(rng.integers(0, 2 ** 32))
    ops.apply_update_dense(*d, dev(G), C, hp["lr"], hp["lr_scale"], hp["rms_beta"], hp["rms_eps"], seed)
    exp = oracle.update_dense(state, scale, v, G, C, hp["lr"], hp["lr_scale"], hp["rms_beta"], hp["rms_eps"], seed)
    for got, want, name in zip(d, exp, ("state", "scale", "v")):
        assert np.array_equal(host(got), want), name


def fused_cases():
    rng = np.random.default_rng(7)
    return [(i, int(rng.integers(1, 700)), 4 * int(rng.integers(1, 300)), int(rng.integers(1, 500)),
             int(rng.integers(1, 12))) for i in range(12)]


@pytest.mark.parametrize("case", fused_cases(), ids=lambda c: "i%d_N%d_in%d_out%d_C%d" % c)
def test_random_fused_cases(ops, oracle, case):
    i, n, n_in, n_out, C = case
    rng = np.random.default_rng(2000 + i)
    hp = random_hypers(rng)
    _, state, _, scale, v = synth.counter_case(600 + i, n_out, n_in, C, oracle=oracle)
    x, dy = synth.activations(700 + i, n, n_in, n_out, 0.7, 0.05)
    d = [dev(state), dev(scale), dev(v)]
    ws = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, n), dtype=torch.uint8, device="cuda")
    ops.apply_update_fused(*d, dev(dy), dev(x), ws, C, hp["lr"], hp["lr_scale"], hp["rms_beta"], hp["rms_eps"], 99 + i)
    g_gpu = host(ws.view(torch.float32)[: n_out * n_in].view(n_out, n_in))
    g_ref = dy.astype(np.float64).T @ x.astype(np.float64)
    assert np.abs(g_gpu - g_ref).max() <= 1e-4 * max(np.abs(g_ref).max(), 1e-30)
    exp = oracle.update_dense(state, scale, v, g_gpu, C, hp["lr"], hp["lr_scale"], hp["rms_beta"], hp["rms_eps"], 99 + i)
    for got, want in zip(d, exp):
        assert np.array_equal(host(got), want)


def strip_cases():
    rng = np.random.default_rng(11)
    return [(i, int(rng.integers(1, 400)), 128 * int(rng.integers(1, 20)), 128 * int(rng.integers(1, 8)),
             int(rng.integers(1, 12))) for i in range(10)]


@pytest.mark.parametrize("case", strip_cases(), ids=lambda c: "i%d_N%d_in%d_out%d_C%d" % c)
def test_random_strip_cases_equal_the_two_kernel_path(ops, oracle, case):
    i, n, n_in, n_out, C = case
    rng = np.random.default_rng(3000 + i)
    hp = random_hypers(rng)
    _, state, _, scale, v = synth.counter_case(800 + i, n_out, n_in, C, full_range=bool(i % 2), oracle=oracle)
    x, dy = synth.activations(900 + i, n, n_in, n_out, 0.7, 0.05)
    dx, ddy = dev(x), dev(dy)
    results = []
    for nbytes in (ops.fused_workspace_nbytes(n_in, n_out, n), ops.fused_strip_workspace_nbytes(n_in, n_out, n)):
        d = [dev(state), dev(scale), dev(v)]
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        ops.apply_update_fused(*d, ddy, dx, ws, C, hp["lr"], 0.0, hp["rms_beta"], hp["rms_eps"], 5 + i)
        ops.fused_check(ws, n_in, n_out, n)
        results.append([host(t) for t in d])
    for a, b in zip(*results):
        assert np.array_equal(a, b)


def linear_cases():
    rng = np.random.default_rng(13)
    return [(i, int(rng.integers(1, 600)), 4 * int(rng.integers(1, 400)), int(rng.integers(1, 600)),
             int(rng.integers(1, 12))) for i in range(12)]


@pytest.mark.parametrize("case", linear_cases(), ids=lambda c: "i%d_N%d_in%d_out%d_C%d" % c)
def test_random_forward_and_input_gradient_cases(ops, oracle, case):
    i, n, n_in, n_out, C = case
    _, state, _, scale, _ = synth.counter_case(1100 + i, n_out, n_in, C, full_range=bool(i % 2), oracle=oracle)
    x, dy = synth.activations(1200 + i, n, n_in, n_out, 0.8, 0.9)
    w = oracle.decode_weight(state, scale, C, n_in, n_out).astype(np.float64)
    y = host(ops.forward(dev(x), dev(state), dev(scale), C, n_out))
    y_ref = x.astype(np.float64) @ w.T
    assert np.abs(y - y_ref).max() <= 2e-5 * max(1.0, np.abs(y_ref).max())
    gx = host(ops.backward_input(dev(dy), dev(state), dev(scale), C, n_in))
    gx_ref = dy.astype(np.float64) @ w
    assert np.abs(gx - gx_ref).max() <= 2e-5 * max(1.0, np.abs(gx_ref).max())
