"""The fused step for a list of tensors in a handful of launches (grouped contraction, grouped
slice sum, batched update): state, scale and v must be the bytes the per-tensor entry point
produces, whatever mix of shapes shares the launches."""
import numpy as np
import pytest
import torch

from tests import synth
from tests.test_gpu_parity import dev, host, ops  # noqa: F401  (fixture; oracle comes from conftest)

pytestmark = pytest.mark.gpu
HP = dict(C=11, lr=3e-3, lr_scale=0.0, rms_beta=0.9, rms_eps=1e-3)

# (out, in, tokens): small-tile and large-tile plans, ragged edges, token counts that split and
# that do not, a shape that is not grouped (unaligned width), one that fills the device alone
MIXES = {
    "layer_15m": [(288, 288, 2048)] * 4 + [(768, 288, 2048)] * 2 + [(288, 768, 2048)],
    "mixed": [(256, 256, 512), (2048, 768, 1024), (132, 260, 300), (64, 64, 64), (768, 2048, 512), (35, 68, 37)],
    "with_large": [(288, 288, 1024), (4096, 4096, 256), (768, 768, 1024)],
}


def build(ops, oracle, shapes, seed):
    tensors = []
    for i, (n_out, n_in, tokens) in enumerate(shapes):
        codes, state, _, scale, v = synth.counter_case(seed + i, n_out, n_in, HP["C"], oracle=oracle)
        x, dy = synth.activations(seed + 100 + i, tokens, n_in, n_out)
        tensors.append((state, scale, v, dy, x))
    return tensors


@pytest.mark.parametrize("name", sorted(MIXES))
@pytest.mark.parametrize("lr_scale", [0.0, 1e-3])
def test_batched_fused_step_matches_the_per_tensor_entry_point(ops, oracle, name, lr_scale):
    shapes = MIXES[name]
    host_tensors = build(ops, oracle, shapes, 7)
    seeds = [12345 + 17 * i for i in range(len(shapes))]
    # per tensor, full workspace
    expect = []
    for (state, scale, v, dy, x), seed, (n_out, n_in, tokens) in zip(host_tensors, seeds, shapes):
        d = [dev(t) for t in (state, scale, v, dy, x)]
        ws = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, tokens), dtype=torch.uint8, device="cuda")
        ops.apply_update_fused(*d, ws, HP["C"], HP["lr"], lr_scale, HP["rms_beta"], HP["rms_eps"], seed)
        expect.append([host(t) for t in d[:3]])
    # the list at once
    d_all = [[dev(t) for t in tensor] for tensor in host_tensors]
    batch = ops.FusedBatch([tuple(d) for d in d_all], HP["lr"], seeds)
    need = batch.workspace_nbytes()
    assert need >= sum(ops.fused_workspace_nbytes(n_in, n_out, tokens) for (n_out, n_in, tokens) in shapes)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    for step in range(2):  # twice through the same workspace; the second step from the updated state
        ops.apply_update_fused_batched(batch, ws, HP["C"], lr_scale, HP["rms_beta"], HP["rms_eps"])
        if step == 0:
            for d, e in zip(d_all, expect):
                for got, want in zip(d[:3], e):
                    np.testing.assert_array_equal(host(got), want)
    torch.cuda.synchronize()


def layer_shapes(dim, hidden, layers, tokens):
    return ([(dim, dim, tokens)] * 4 + [(hidden, dim, tokens)] * 2 + [(dim, hidden, tokens)]) * layers


@pytest.fixture()
def span_mode():
    """Test aid of the equal-spans contraction: polls before a taker gives up, takers first."""
    import motifcl_amd
    L = motifcl_amd.load()
    yield lambda polls, start_first: L.mcc_contraction_spans_set_test_mode(polls, start_first)
    L.mcc_contraction_spans_set_test_mode(0xFFFFFFFF, 0)


# the 110M-shaped model (12 layers of 768 / 2048: 1296 tiles of 256 x 256) runs as equal spans of the
# whole list; with 64 tokens the per-tensor call does not chunk either, so the bytes must be equal
@pytest.mark.parametrize("mode", ["default", "every_hand_off_abandoned", "takers_first"])
@pytest.mark.parametrize("lr_scale", [0.0, 1e-3])
def test_list_of_256_multiple_layers_runs_as_equal_spans_with_the_same_bytes(ops, oracle, span_mode, mode, lr_scale):
    shapes = layer_shapes(768, 2048, 12, 64)
    host_tensors = build(ops, oracle, shapes, 21)
    seeds = [999 + 3 * i for i in range(len(shapes))]
    expect = []
    for (state, scale, v, dy, x), seed, (n_out, n_in, tokens) in zip(host_tensors, seeds, shapes):
        d = [dev(t) for t in (state, scale, v, dy, x)]
        ws = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, tokens), dtype=torch.uint8, device="cuda")
        ops.apply_update_fused(*d, ws, HP["C"], HP["lr"], lr_scale, HP["rms_beta"], HP["rms_eps"], seed)
        expect.append([host(t) for t in d[:3]])
    d_all = [[dev(t) for t in tensor] for tensor in host_tensors]
    batch = ops.FusedBatch([tuple(d) for d in d_all], HP["lr"], seeds)
    need = batch.workspace_nbytes()
    assert need == sum((o * i * 4 + 255) // 256 * 256 for (o, i, _) in shapes) + 1024   # a gradient per tensor, no slices
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    if mode == "every_hand_off_abandoned":
        span_mode(0, 1)
    elif mode == "takers_first":
        span_mode(0xFFFFFFFF, 1)
    print("equal spans over a list,", mode, flush=True)
    ops.apply_update_fused_batched(batch, ws, HP["C"], lr_scale, HP["rms_beta"], HP["rms_eps"])
    torch.cuda.synchronize()
    for d, e in zip(d_all, expect):
        for got, want in zip(d[:3], e):
            np.testing.assert_array_equal(host(got), want)


@pytest.mark.parametrize("model", [(768, 2048, 12), (288, 768, 6)], ids=["110m_equal_spans", "15m_small_tiles"])
def test_equal_spans_over_a_list_against_the_oracle(ops, oracle, model):
    # 1024 tokens: the per-tensor call would split them into chunks; the list's gradients are the
    # unchunked sums (equal spans of 256 x 256 tiles for the 110M shapes; for the 15M shapes the
    # list's 1680 small tiles fill the device, so nothing is chunked either).  Each gradient within
    # 1e-4 of the oracle's sequential sum, state / scale / v exact for the GPU's gradient, counter
    # flips against the sequential-sum oracle counted.
    shapes = layer_shapes(*model, 1024)
    host_tensors = build(ops, oracle, shapes, 33)
    seeds = [4000 + i for i in range(len(shapes))]
    d_all = [[dev(t) for t in tensor] for tensor in host_tensors]
    batch = ops.FusedBatch([tuple(d) for d in d_all], HP["lr"], seeds)
    ws = torch.empty(batch.workspace_nbytes(), dtype=torch.uint8, device="cuda")
    ops.apply_update_fused_batched(batch, ws, HP["C"], 0.0, HP["rms_beta"], HP["rms_eps"])
    torch.cuda.synchronize()
    offset, n_flip, n_all = 0, 0, 0
    for (state, scale, v, dy, x), seed, (n_out, n_in, tokens), d in zip(host_tensors, seeds, shapes, d_all):
        g_gpu = ws[offset: offset + n_out * n_in * 4].view(torch.float32).view(n_out, n_in).cpu().numpy()
        # a tensor's region of the workspace: its gradient alone under equal spans, else what its own call asks for
        region = n_out * n_in * 4 if model[0] % 256 == 0 else ops.fused_workspace_nbytes(n_in, n_out, tokens)
        offset += (region + 255) // 256 * 256
        e_state, e_scale, e_v, g_seq = oracle.update_fused(state, scale, v, dy, x, HP["C"], HP["lr"], 0.0,
                                                          HP["rms_beta"], HP["rms_eps"], seed)
        assert np.abs(g_gpu - g_seq).max() <= 1e-4 * np.abs(g_seq).max()
        x_state, x_scale, x_v = oracle.update_dense(state, scale, v, g_gpu, HP["C"], HP["lr"], 0.0, HP["rms_beta"],
                                                    HP["rms_eps"], seed)
        np.testing.assert_array_equal(host(d[0]), x_state)
        np.testing.assert_array_equal(host(d[1]), x_scale)
        np.testing.assert_array_equal(host(d[2]), x_v)
        diff = oracle.unpack_codes(x_state) != oracle.unpack_codes(e_state)
        n_flip += int(diff.sum())
        n_all += diff.size
    print("%d tensors at 1024 tokens, unchunked: counter-flip fraction vs the sequential-sum oracle %.2e" % (len(shapes), n_flip / n_all))
    assert n_flip / n_all <= 1e-4


def test_batched_fused_step_validates_its_arguments(ops, oracle):
    from motifcl_amd.lib import MccError
    shapes = [(64, 64, 64), (32, 128, 16)]
    d_all = [[dev(t) for t in tensor] for tensor in build(ops, oracle, shapes, 3)]
    batch = ops.FusedBatch([tuple(d) for d in d_all], HP["lr"], [1, 2])
    ws = torch.empty(batch.workspace_nbytes(), dtype=torch.uint8, device="cuda")
    with pytest.raises(MccError, match="workspace is too small"):
        ops.apply_update_fused_batched(batch, ws[:-256], HP["C"], 0.0, 0.9, 1e-3)
    with pytest.raises(MccError, match="256-byte aligned"):
        ops.apply_update_fused_batched(batch, torch.empty(len(ws) + 256, dtype=torch.uint8, device="cuda")[16:],
                                       HP["C"], 0.0, 0.9, 1e-3)
    batch.array[1].x_nbytes -= 4
    with pytest.raises(MccError, match="tensor 1: .*activation buffer is too small"):
        ops.apply_update_fused_batched(batch, ws, HP["C"], 0.0, 0.9, 1e-3)
    batch.array[1].x_nbytes += 4
    with pytest.raises(MccError, match="rms_eps"):
        ops.apply_update_fused_batched(batch, ws, HP["C"], 0.0, 0.9, -1.0)


def test_batched_fused_step_under_the_split_bf16_mode_goes_tensor_by_tensor(ops, oracle):
    shapes = [(128, 128, 256), (256, 128, 512)]
    host_tensors = build(ops, oracle, shapes, 11)
    seeds = [5, 6]
    ops.set_contraction_mode(ops.CONTRACTION_BF16X6)
    try:
        expect = []
        for (state, scale, v, dy, x), seed, (n_out, n_in, tokens) in zip(host_tensors, seeds, shapes):
            d = [dev(t) for t in (state, scale, v, dy, x)]
            ws = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, tokens), dtype=torch.uint8, device="cuda")
            ops.apply_update_fused(*d, ws, HP["C"], HP["lr"], 0.0, HP["rms_beta"], HP["rms_eps"], seed)
            expect.append([host(t) for t in d[:3]])
        d_all = [[dev(t) for t in tensor] for tensor in host_tensors]
        batch = ops.FusedBatch([tuple(d) for d in d_all], HP["lr"], seeds)
        ws = torch.empty(batch.workspace_nbytes(), dtype=torch.uint8, device="cuda")
        ops.apply_update_fused_batched(batch, ws, HP["C"], 0.0, HP["rms_beta"], HP["rms_eps"])
        for d, e in zip(d_all, expect):
            for got, want in zip(d[:3], e):
                np.testing.assert_array_equal(host(got), want)
    finally:
        ops.set_contraction_mode(ops.CONTRACTION_FP32)
