"""The contraction of shapes that are more than two but not whole rounds of 256 x 256 tiles
(11008 x 4096: 688 tiles on 256 CUs) runs as one launch of equal spans in which neighbouring
workgroups hand a partly summed tile on.  It must give the bytes of the undivided tiles -- which is
what the same entry point computes when the workspace has no room for the hand-off words -- also
when every hand-off falls back to computing the tile alone."""
import numpy as np
import pytest
import torch

from tests.test_gpu_parity import ops  # noqa: F401  (fixture)

pytestmark = pytest.mark.gpu

SHAPES = [  # (tokens, out, in)
    (64, 11008, 4096),
    (48, 4096, 11008),
    (160, 8448, 4096),   # 33 x 16 tiles: 528 = two rounds and a sixteenth
    (4096, 11008, 4096),
]


@pytest.fixture()
def spans_mode():
    from motifcl_amd import lib
    L = lib.load()
    yield lambda polls, start_first: L.mcc_contraction_spans_set_test_mode(polls, start_first)
    L.mcc_contraction_spans_set_test_mode(0xFFFFFFFF, 0)


def fused(ops, tokens, n_out, n_in, ws_nbytes, seed=5):
    """One fused update from a fixed start; returns (state, scale, v, G) as host arrays."""
    x = ops.fill_normal(torch.empty(tokens, n_in, device="cuda"), 11, 1.0)
    dy = ops.fill_normal(torch.empty(tokens, n_out, device="cuda"), 12, 0.01)
    state = ops.fill_counter_state(torch.empty(n_out * n_in // 4 * 3, dtype=torch.uint8, device="cuda"), 13, 63)
    scale = torch.full((n_out,), 0.02, device="cuda")
    v = torch.zeros(n_out, device="cuda")
    ws = torch.zeros(ws_nbytes, dtype=torch.uint8, device="cuda")
    ops.apply_update_fused(state, scale, v, dy, x, ws, 11, 3e-3, 0.05, 0.9, 1e-3, seed)
    torch.cuda.synchronize()
    g = ws[: n_out * n_in * 4].view(torch.float32).view(n_out, n_in)
    return state.cpu().numpy(), scale.cpu().numpy(), v.cpu().numpy(), g.cpu().numpy(), (x, dy)


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "N%d_out%d_in%d" % s)
def test_spans_give_the_bytes_of_undivided_tiles(ops, spans_mode, shape):
    tokens, n_out, n_in = shape
    full = ops.fused_workspace_nbytes(n_in, n_out, tokens)
    plain = n_out * n_in * 4
    assert full == plain + 1024, "this shape is meant to use the hand-off words"
    ref = fused(ops, tokens, n_out, n_in, plain)       # no room for the words: tiles one by one
    got = fused(ops, tokens, n_out, n_in, full)
    for a, b in zip(ref[:4], got[:4]):
        assert np.array_equal(a, b)
    # every taker arrives before its owner and gives up at once: all tiles computed alone
    spans_mode(0, 1)
    alone = fused(ops, tokens, n_out, n_in, full)
    for a, b in zip(ref[:4], alone[:4]):
        assert np.array_equal(a, b)
    # takers arrive first but wait: all tiles handed on late
    spans_mode(1 << 24, 1)
    late = fused(ops, tokens, n_out, n_in, full)
    for a, b in zip(ref[:4], late[:4]):
        assert np.array_equal(a, b)
    # against a double-precision product on a few rows
    x, dy = ref[4]
    rows = torch.arange(0, n_out, n_out // 7, device="cuda")[:7]
    want = (dy[:, rows].double().t() @ x.double()).cpu().numpy()
    rel = np.abs(got[3][rows.cpu().numpy()] - want).max() / np.abs(want).max()
    assert rel < 1e-5


def test_plain_contraction_uses_spans_and_matches(ops, spans_mode):
    tokens, m, n = 96, 11008, 4096
    a = ops.fill_normal(torch.empty(tokens, m, device="cuda"), 21, 0.01)
    b = ops.fill_normal(torch.empty(tokens, n, device="cuda"), 22, 1.0)
    c1 = torch.empty(m, n, device="cuda")
    ops.matmul_transpose_a(a, b, c1)
    spans_mode(0, 1)
    c2 = torch.empty(m, n, device="cuda")
    ops.matmul_transpose_a(a, b, c2)
    torch.cuda.synchronize()
    assert torch.equal(c1, c2)
    want = a.double().t() @ b.double()
    assert float((c1.double() - want).abs().max() / want.abs().max()) < 1e-5


@pytest.mark.parametrize("tokens", [16, 32, 48, 64, 80, 96, 112, 128, 144, 272])
def test_wide_tiles_with_few_slabs_match_the_small_tiles(ops, tokens):
    """The 256 x 256 tile loop keeps four 16-token slabs in flight and runs four slabs per
    iteration; token counts below and around that depth must give the bits of the 128 x 128 tiles,
    which a 4096 x 2048 product (half a round of wide tiles) still uses."""
    m = n = 4096
    a = ops.fill_normal(torch.empty(tokens, m, device="cuda"), 31, 0.01)
    b = ops.fill_normal(torch.empty(tokens, n, device="cuda"), 32, 1.0)
    c = torch.empty(m, n, device="cuda")
    ops.matmul_transpose_a(a, b, c)
    for half in range(2):
        bh = b[:, half * 2048:(half + 1) * 2048].contiguous()
        ch = torch.empty(m, 2048, device="cuda")
        ops.matmul_transpose_a(a, bh, ch)
        assert torch.equal(c[:, half * 2048:(half + 1) * 2048], ch)
    want = a.double().t() @ b.double()
    assert float((c.double() - want).abs().max() / want.abs().max()) < 1e-5
