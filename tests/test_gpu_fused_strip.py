"""Accumulator-resident fused step against the two-kernel fused step (same bytes wherever the latter
contracts the tokens in one chunk) and the oracle."""
import numpy as np
import pytest
import torch

from tests import synth
from tests.test_gpu_parity import dev, host, ops  # noqa: F401  (fixture)

pytestmark = pytest.mark.gpu
F = np.float32

HP = dict(lr=3e-3, lr_scale=0.0, rms_beta=0.9, rms_eps=1e-3)

# (N, in, out, C)
STRIP_SHAPES = [
    (64, 128, 128, 11),     # one tile: a strip of a single column tile (odd chains stay empty)
    (100, 256, 128, 11),    # one strip, one tile per parity; token count not a multiple of the slab
    (96, 384, 256, 3),      # odd number of tiles per strip
    (257, 1024, 384, 11),
    (64, 768, 2048, 11),    # BASELINE cfg2 shapes, few tokens
    (64, 2048, 768, 8),
    (32, 4096, 4096, 11),   # 1024 tiles: the whole grid in one pass
    (32, 11008, 4096, 11),  # 86 tiles per strip, several passes of the persistent grid
    (32, 4096, 11008, 11),
]


def strip_nbytes(ops, n_in, n_out, n, grid_cap=0):
    """Strip workspace size; with the test aid's grid cap, the size a capped launch needs (the
    public size query never depends on the cap)."""
    if not grid_cap:
        return ops.fused_strip_workspace_nbytes(n_in, n_out, n)
    import motifcl_amd
    return int(motifcl_amd.load().mcc_compact_counter_fused_strip_workspace_nbytes_for_grid(n_in, n_out, n, grid_cap))


def run_both(ops, n, n_in, n_out, C, seed, lr=HP["lr"], lr_scale=HP["lr_scale"], grid_cap=0):
    _, _, _, scale, v = synth.counter_case(seed, n_out, n_in, C, oracle=None)
    rng = np.random.default_rng(seed + 1)
    hi = 3 * (2 * C - 1)
    # every 6-bit code inside the reachable range
    codes = rng.integers(0, hi, (n_out, n_in)).astype(np.uint32).reshape(-1, 4)
    word = codes[:, 0] | (codes[:, 1] << 6) | (codes[:, 2] << 12) | (codes[:, 3] << 18)
    state = np.stack([word & 255, (word >> 8) & 255, (word >> 16) & 255], axis=1).astype(np.uint8).reshape(-1)
    x, dy = synth.activations(seed + 2, n, n_in, n_out)
    dx, ddy = dev(x), dev(dy)
    out = []
    for nbytes in (ops.fused_workspace_nbytes(n_in, n_out, n), strip_nbytes(ops, n_in, n_out, n, grid_cap)):
        assert nbytes > 0
        d = [dev(state), dev(scale), dev(v)]
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        ops.apply_update_fused(*d, ddy, dx, ws, C, lr, lr_scale, HP["rms_beta"], HP["rms_eps"], 4242)
        ops.fused_check(ws, n_in, n_out, n)
        out.append([host(t) for t in d])
    return state, scale, v, x, dy, out


@pytest.fixture()
def tile_mode():
    """Selects the strip step's tiles: 0 by shape, 1 the 256 x 256 tiles wherever possible, 2 never;
    grid_cap holds the 256 x 256 kernel to that many workgroups."""
    import motifcl_amd
    L = motifcl_amd.load()
    yield lambda mode, grid_cap=0: L.mcc_compact_counter_fused_strip_set_tile_mode(mode, grid_cap)
    L.mcc_compact_counter_fused_strip_set_tile_mode(0, 0)


# (N, in, out, C): sides that are multiples of 256 and whole 16-token slabs, which the wide tiles take
WIDE_STRIP_SHAPES = [
    (16, 256, 256, 11),     # one tile
    (48, 512, 256, 3),      # one strip of two tiles, three slabs
    (96, 1024, 512, 11),
    (64, 768, 2048, 11),    # BASELINE cfg2 shapes, few tokens
    (64, 2048, 768, 8),
    (32, 4096, 4096, 11),   # one round of 16 strips of 16 tiles
    (32, 4096, 2816, 11),   # 11 strips: one round that does not fill the device
    (32, 11008, 1536, 11),  # 43 tiles per strip: five strips a round, two rounds
]


@pytest.mark.parametrize("lr_scale", [0.0, 0.05])
@pytest.mark.parametrize("shape", WIDE_STRIP_SHAPES, ids=lambda s: "N%d_in%d_out%d_C%d" % s)
def test_wide_strip_tiles_match_small_tiles_and_two_kernel_path(ops, tile_mode, shape, lr_scale):
    n, n_in, n_out, C = shape
    print("wide strip case", shape, lr_scale, flush=True)
    tile_mode(2)
    state, scale, v, _, _, (full, small) = run_both(ops, n, n_in, n_out, C, seed=n_in + n_out, lr_scale=lr_scale)
    tile_mode(1)
    _, _, _, _, _, (_, wide) = run_both(ops, n, n_in, n_out, C, seed=n_in + n_out, lr_scale=lr_scale)
    assert not np.array_equal(full[0], state)
    for a, b, c in zip(wide, small, full):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
        assert np.array_equal(a.view(np.uint8), c.view(np.uint8))


# (N, in, out, C, workgroups): the grid held so small that strips straddle its passes
PARKING_CASES = [
    (48, 2048, 2048, 11, 44),   # 8 tiles a strip: four tiles parked in pass 0 by workgroups without a second tile
    (48, 2048, 2048, 11, 12),   # ... parked tiles finished after the owner's next tile, several times
    (32, 2048, 2048, 3, 10),    # workgroups 8 and 9 park in two passes running
    (32, 1280, 1536, 11, 7),    # 5 tiles a strip, 30 tiles in passes of 7
    (32, 11008, 768, 11, 50),   # 43 tiles a strip: 43 + 7 parked, ...
]


@pytest.mark.parametrize("lr_scale", [0.0, 0.05])
@pytest.mark.parametrize("case", PARKING_CASES, ids=lambda s: "N%d_in%d_out%d_C%d_wgs%d" % s)
def test_wide_strip_tiles_parked_between_passes(ops, tile_mode, case, lr_scale):
    n, n_in, n_out, C, wgs = case
    print("parking case", case, lr_scale, flush=True)
    tile_mode(2)
    plain = ops.fused_strip_workspace_nbytes(n_in, n_out, n)
    state, scale, v, _, _, (full, small) = run_both(ops, n, n_in, n_out, C, seed=n_in + wgs, lr_scale=lr_scale)
    tile_mode(1, wgs)
    assert ops.fused_strip_workspace_nbytes(n_in, n_out, n) == plain   # the public size ignores the test aid
    assert strip_nbytes(ops, n_in, n_out, n, wgs) > plain              # slots for the parked tiles
    from motifcl_amd.lib import MccError
    with pytest.raises(MccError):  # a capped launch without room for its parked tiles is rejected
        run_both(ops, n, n_in, n_out, C, seed=n_in + wgs, lr_scale=lr_scale)
    _, _, _, _, _, (_, wide) = run_both(ops, n, n_in, n_out, C, seed=n_in + wgs, lr_scale=lr_scale, grid_cap=wgs)
    assert not np.array_equal(full[0], state)
    for a, b, c in zip(wide, small, full):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
        assert np.array_equal(a.view(np.uint8), c.view(np.uint8))


@pytest.mark.parametrize("shape", STRIP_SHAPES, ids=lambda s: "N%d_in%d_out%d_C%d" % s)
def test_strip_path_matches_two_kernel_path(ops, shape):
    n, n_in, n_out, C = shape
    print("strip case", shape, flush=True)
    assert ops.fused_strip_workspace_nbytes(n_in, n_out, n) < ops.fused_workspace_nbytes(n_in, n_out, n)
    state, scale, v, _, _, (full, strip) = run_both(ops, n, n_in, n_out, C, seed=n_in + n_out)
    assert not np.array_equal(full[0], state)
    assert np.array_equal(strip[1], full[1])  # scale
    assert np.array_equal(strip[2], full[2])  # v
    assert np.array_equal(strip[0], full[0])  # state bytes


@pytest.mark.parametrize("shape", [(1024, 1536, 2176, 11), (700, 896, 640, 11), (2048, 768, 2560, 5)],
                         ids=lambda s: "N%d_in%d_out%d_C%d" % s)
def test_strip_and_split_contraction_differ_only_by_rounding(ops, shape):
    # 512 tokens or more on a layer of fewer than 1024 tiles: the two-kernel path contracts the
    # tokens in chunks and adds the chunk sums, the accumulator-resident one sums straight through.
    # Same terms, another order: v and scale agree to rounding and few counters land differently.
    n, n_in, n_out, C = shape
    assert ops.fused_workspace_nbytes(n_in, n_out, n) > 4 * n_in * n_out  # more than one slice
    state, scale, v, x, dy, (full, strip) = run_both(ops, n, n_in, n_out, C, seed=n_in)
    np.testing.assert_allclose(strip[2], full[2], rtol=1e-5)
    np.testing.assert_array_equal(strip[1], full[1])  # lr_scale == 0: the scale does not move
    flips = (strip[0] != full[0]).mean()
    assert flips < 1e-3, flips
    # under 512 tokens the same layer is contracted in one chunk and the bytes are the same
    _, _, _, _, _, (full_s, strip_s) = run_both(ops, 300, n_in, n_out, C, seed=n_in)
    assert all(np.array_equal(a, b) for a, b in zip(full_s, strip_s))


def test_strip_path_against_oracle(ops, oracle):
    n, n_in, n_out, C = 192, 512, 256, 11
    state, scale, v, x, dy, (_, strip) = run_both(ops, n, n_in, n_out, C, seed=5)
    e_state, e_scale, e_v, _ = oracle.update_fused(state, scale, v, dy, x, C, HP["lr"], HP["lr_scale"],
                                                   HP["rms_beta"], HP["rms_eps"], 4242)
    flips = np.mean(oracle.unpack_codes(strip[0]) != oracle.unpack_codes(e_state))
    print("strip vs oracle: counter-flip mismatch %.3e" % flips)
    assert flips <= 2e-3
    assert np.allclose(strip[2], e_v, rtol=1e-5, atol=0)
    assert np.array_equal(strip[1], e_scale)


@pytest.mark.parametrize("shape", [(64, 768, 256, 11), (96, 1024, 384, 3), (32, 4096, 4096, 11), (32, 11008, 4096, 11)],
                         ids=lambda s: "N%d_in%d_out%d_C%d" % s)
def test_strip_path_with_scale_learning_matches_two_kernel_path(ops, oracle, shape):
    # lr_scale != 0: the row sums of g * t travel through the strip beside the sums of squares
    n, n_in, n_out, C = shape
    state, scale, v, x, dy, (full, strip) = run_both(ops, n, n_in, n_out, C, seed=n_in + n_out + 1, lr_scale=0.05)
    assert not np.array_equal(full[1], scale)  # the scale moved
    for a, b in zip(strip, full):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    if n_in * n_out <= 1 << 20:
        g = host(ops.matmul_transpose_a(dev(dy), dev(x)))
        exp = oracle.update_dense(state, scale, v, g, C, HP["lr"], 0.05, HP["rms_beta"], HP["rms_eps"], 4242)
        for a, b in zip(strip, exp):
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8))


# (N, in, out, C): layers too small or too oddly shaped for the strips run band by band
BANDED_SHAPES = [(64, 256, 256, 11),   # tests/test_memory_truth_gate.cpp:34
                 (64, 288, 288, 11), (300, 260, 35, 3), (37, 68, 35, 3), (8, 64, 40, 3), (128, 512, 1000, 11)]


@pytest.mark.parametrize("shape", BANDED_SHAPES, ids=lambda s: "N%d_in%d_out%d_C%d" % s)
@pytest.mark.parametrize("lr_scale", [0.0, 0.05])
def test_banded_small_workspace_matches_two_kernel_path(ops, oracle, shape, lr_scale):
    # under 512 tokens neither way splits the tokens: the gradients are the same bits and so is the state
    n, n_in, n_out, C = shape
    small, full_n = ops.fused_strip_workspace_nbytes(n_in, n_out, n), ops.fused_workspace_nbytes(n_in, n_out, n)
    assert 0 < small < full_n
    if n_out >= 20:
        assert small < n_in * n_out  # a quarter of the dense gradient (tests/test_memory_truth_gate.cpp:109-113)
    state, scale, v, x, dy, (full, banded) = run_both(ops, n, n_in, n_out, C, seed=n_in + 7, lr_scale=lr_scale)
    assert not np.array_equal(full[0], state)
    for a, b in zip(banded, full):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    g = host(ops.matmul_transpose_a(dev(dy), dev(x)))
    exp = oracle.update_dense(state, scale, v, g, C, HP["lr"], lr_scale, HP["rms_beta"], HP["rms_eps"], 4242)
    for a, b in zip(banded, exp):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))


def test_banded_small_workspace_with_token_chunks_differs_only_by_rounding(ops, oracle):
    # BASELINE config 0: 4096 tokens are contracted in chunks, differently cut for a band than for
    # the whole layer; same terms, another order
    n, n_in, n_out, C = 4096, 288, 288, 11
    state, scale, v, x, dy, (full, banded) = run_both(ops, n, n_in, n_out, C, seed=3, lr_scale=0.05)
    np.testing.assert_allclose(banded[2], full[2], rtol=1e-5)
    np.testing.assert_allclose(banded[1], full[1], rtol=1e-4)  # the sum of g * t cancels: a few more ulps
    assert (banded[0] != full[0]).mean() < 1e-3
    e_state = oracle.update_fused(state, scale, v, dy, x, C, HP["lr"], 0.05, HP["rms_beta"], HP["rms_eps"], 4242)[0]
    flips = np.mean(oracle.unpack_codes(banded[0]) != oracle.unpack_codes(e_state))
    print("banded vs oracle: counter-flip mismatch %.3e" % flips)
    assert flips <= 2e-3


def test_small_workspace_rules(ops):
    assert ops.fused_strip_workspace_nbytes(128, 64, 64) > 0        # banded
    assert ops.fused_strip_workspace_nbytes(6, 64, 64) == 0         # in_features not a multiple of 4
    n, n_in, n_out, C = 64, 1024, 128, 11
    _, _, _, scale, v = synth.counter_case(1, n_out, n_in, C)
    state = np.zeros(n_out * n_in // 4 * 3, dtype=np.uint8)
    x, dy = synth.activations(2, n, n_in, n_out)
    ws = torch.empty(ops.fused_strip_workspace_nbytes(n_in, n_out, n), dtype=torch.uint8, device="cuda")
    from motifcl_amd.lib import MccError
    with pytest.raises(MccError, match="too small"):
        ops.apply_update_fused(dev(state), dev(scale), dev(v), dev(dy), dev(x), ws[:-16], C, 3e-3, 0.0, 0.9, 1e-3, 1)


def test_strip_steps_on_two_streams_are_ordered_on_the_device(ops):
    # tiles of a strip wait for each other on the device, so two such launches must not share the
    # GPU: a step on another stream is ordered behind the previous one by the library.  Steps of one
    # tensor alternate between two streams with no synchronisation of the caller's: the bytes must be
    # those of the same steps on one stream.
    n, n_in, n_out, C = 2048, 4096, 4096, 11
    rng = np.random.default_rng(0)
    state = dev(rng.integers(0, 63, n_out * n_in // 4 * 3).astype(np.uint8))
    scale = torch.full((n_out,), 0.02, device="cuda")
    v = torch.zeros(n_out, device="cuda")
    state2, scale2, v2 = state.clone(), scale.clone(), v.clone()
    x = torch.randn(n, n_in, device="cuda")
    dy = torch.randn(n, n_out, device="cuda") * 0.01
    nbytes = ops.fused_strip_workspace_nbytes(n_in, n_out, n)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    for step in range(6):
        ops.apply_update_fused(state, scale, v, dy, x, ws, C, 3e-3, 0.0, 0.9, 1e-3, 1 + step)
    torch.cuda.synchronize()
    ops.fused_check(ws, n_in, n_out, n)
    for step in range(6):
        if step % 2:
            with torch.cuda.stream(side):
                ops.apply_update_fused(state2, scale2, v2, dy, x, ws, C, 3e-3, 0.0, 0.9, 1e-3, 1 + step)
        else:
            ops.apply_update_fused(state2, scale2, v2, dy, x, ws, C, 3e-3, 0.0, 0.9, 1e-3, 1 + step)
    torch.cuda.synchronize()
    ops.fused_check(ws, n_in, n_out, n)
    assert torch.equal(state, state2) and torch.equal(scale, scale2) and torch.equal(v, v2)


@pytest.mark.parametrize("wide", [0, 1, 20], ids=["tiles128", "tiles256", "tiles256_parked"])
def test_given_up_wait_is_reported_and_leaves_whole_strips_untouched(ops, tile_mode, wide):
    # a spin budget of one poll makes waits fail from the host side; the kernel must still drain,
    # the failure must surface through fused_check -- also after another layer has used the same
    # workspace -- and every strip (128 or 256 rows) must be either fully updated or untouched
    import motifcl_amd
    # wide == 20: the 32 wide tiles run on 20 workgroups, four tiles of the second strip are parked
    tile_mode(1 if wide else 2, wide if wide > 1 else 0)
    strip_rows = 256 if wide else 128
    from motifcl_amd.lib import MccError
    L = motifcl_amd.load()
    n, n_in, n_out, C = 32, 4096, 512, 11
    rng = np.random.default_rng(4)
    state = rng.integers(0, 63, n_out * n_in // 4 * 3).astype(np.uint8)
    scale = np.full(n_out, 0.05, dtype=F)
    v = np.zeros(n_out, dtype=F)
    x, dy = synth.activations(3, n, n_in, n_out)
    ws = torch.empty(strip_nbytes(ops, n_in, n_out, n, wide if wide > 1 else 0), dtype=torch.uint8, device="cuda")
    ref = [dev(state), dev(scale), dev(v)]
    full = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, n), dtype=torch.uint8, device="cuda")
    ops.apply_update_fused(*ref, dev(dy), dev(x), full, C, 3e-3, 0.0, 0.9, 1e-3, 5)
    ref = [host(t) for t in ref]
    L.mcc_compact_counter_fused_strip_set_spin_limit(1)
    try:
        d = [dev(state), dev(scale), dev(v)]
        ops.apply_update_fused(*d, dev(dy), dev(x), ws, C, 3e-3, 0.0, 0.9, 1e-3, 5)
        torch.cuda.synchronize()
    finally:
        L.mcc_compact_counter_fused_strip_set_spin_limit(0)
    # a second layer's step (two-kernel path) through memory that overlaps the first one's workspace
    other = [dev(state[:256 * 256 // 4 * 3]), dev(scale[:256]), dev(v[:256])]
    ops.apply_update_fused(*other, dev(dy[:, :256]), dev(x[:, :256]), full, 11, 3e-3, 0.0, 0.9, 1e-3, 6)
    with pytest.raises(MccError, match="gave up waiting"):
        ops.fused_check(ws, n_in, n_out, n)
    ops.fused_check(ws, n_in, n_out, n)  # reported once
    got = [host(t) for t in d]
    row_bytes = n_in // 4 * 3
    untouched = 0
    for s0 in range(0, n_out, strip_rows):
        rows = slice(s0, s0 + strip_rows)
        st = slice(s0 * row_bytes, (s0 + strip_rows) * row_bytes)
        if np.array_equal(got[0][st], state[st]):
            untouched += 1
            assert np.array_equal(got[1][rows], scale[rows]) and np.array_equal(got[2][rows], v[rows])
        else:
            assert np.array_equal(got[0][st], ref[0][st]), "strip %d is half-updated" % (s0 // strip_rows)
            assert np.array_equal(got[1][rows], ref[1][rows]) and np.array_equal(got[2][rows], ref[2][rows])
    assert untouched >= 1
    # with the default budget the same call completes and matches the two-kernel path
    d = [dev(state), dev(scale), dev(v)]
    ops.apply_update_fused(*d, dev(dy), dev(x), ws, C, 3e-3, 0.0, 0.9, 1e-3, 5)
    ops.fused_check(ws, n_in, n_out, n)
    for a, b in zip(d, ref):
        assert np.array_equal(host(a), b)
