"""The optional split-bf16 form of the weight-gradient contraction: accuracy against a
double-precision product no worse than the fp32 matrix instruction's, the fused step still
bit-exact given the gradient it produced, and silent fallback on shapes it does not take."""
import numpy as np
import pytest
import torch

from tests import synth
from tests.test_gpu_parity import dev, host, ops  # noqa: F401  (fixture)

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture()
def bf16x6(ops):
    ops.set_contraction_mode(ops.CONTRACTION_BF16X6)
    yield ops
    ops.set_contraction_mode(ops.CONTRACTION_FP32)


def test_mode_is_validated_and_readable(ops):
    from motifcl_amd.lib import MccError
    assert ops.get_contraction_mode() == ops.CONTRACTION_FP32
    with pytest.raises(MccError, match="unknown contraction mode"):
        ops.set_contraction_mode(7)
    assert ops.get_contraction_mode() == ops.CONTRACTION_FP32


@pytest.mark.parametrize("shape", [(512, 256, 384), (4096, 128, 128), (2048, 1024, 512), (8192, 256, 256)],
                         ids=lambda s: "K%d_M%d_N%d" % s)
def test_split_contraction_is_as_accurate_as_the_fp32_instruction(ops, shape):
    k, m, n = shape
    rng = np.random.default_rng(k + m)
    a = (rng.standard_normal((k, m)) * np.exp2(rng.integers(-8, 8, (k, m)))).astype(F)
    b = (rng.standard_normal((k, n)) * np.exp2(rng.integers(-8, 8, (k, n)))).astype(F)
    ref = a.astype(np.float64).T @ b.astype(np.float64)
    errs = []
    for mode in (ops.CONTRACTION_FP32, ops.CONTRACTION_BF16X6):
        ops.set_contraction_mode(mode)
        try:
            c = host(ops.matmul_transpose_a(dev(a), dev(b)))
        finally:
            ops.set_contraction_mode(ops.CONTRACTION_FP32)
        errs.append(np.abs(c - ref).max() / np.abs(ref).max())
    print("max error / max|G|: fp32 instruction %.2e, split bf16 %.2e" % tuple(errs))
    assert errs[1] <= 2.0 * errs[0] + 1e-7
    assert errs[1] <= 1e-5


def test_fused_step_with_split_contraction(bf16x6, oracle):
    ops = bf16x6
    n, n_in, n_out, C = 1024, 512, 256, 11   # whole tiles; the token range is split into chunks of 256
    _, state, _, scale, v = synth.counter_case(3, n_out, n_in, C, oracle=oracle)
    x, dy = synth.activations(4, n, n_in, n_out)
    d = [dev(state), dev(scale), dev(v)]
    ws = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, n), dtype=torch.uint8, device="cuda")
    ops.apply_update_fused(*d, dev(dy), dev(x), ws, C, 3e-3, 0.0, 0.9, 1e-3, 321)
    g_gpu = host(ws.view(torch.float32)[: n_out * n_in].view(n_out, n_in))
    e_state, e_scale, e_v, g_seq = oracle.update_fused(state, scale, v, dy, x, C, 3e-3, 0.0, 0.9, 1e-3, 321)
    assert np.abs(g_gpu - g_seq).max() <= 1e-4 * np.abs(g_seq).max()
    exp = oracle.update_dense(state, scale, v, g_gpu, C, 3e-3, 0.0, 0.9, 1e-3, 321)
    for got, want in zip(d, exp):
        assert np.array_equal(host(got), want)   # bit-exact given the gradient it produced
    flips = float((oracle.unpack_codes(host(d[0])) != oracle.unpack_codes(e_state)).mean())
    print("split contraction: counter-flip mismatch vs sequential-sum oracle %.3e" % flips)
    assert flips <= 2e-3


def test_shapes_it_does_not_take_fall_back_to_the_fp32_instruction(ops):
    k, m, n = 300, 288, 288
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal((k, m)).astype(F), rng.standard_normal((k, n)).astype(F)
    c0 = host(ops.matmul_transpose_a(dev(a), dev(b)))
    ops.set_contraction_mode(ops.CONTRACTION_BF16X6)
    try:
        c1 = host(ops.matmul_transpose_a(dev(a), dev(b)))
    finally:
        ops.set_contraction_mode(ops.CONTRACTION_FP32)
    assert np.array_equal(c0, c1)
