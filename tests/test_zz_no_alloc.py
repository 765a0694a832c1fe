"""The fused step on the library's static workspace (mcc_compact_counter_apply_update_fused_static)
against mcc_compact_counter_apply_update_fused with a lent workspace: identical bytes, on two calls
in a row through the shared array, the second with a smaller input; both workspace kinds (full and
strip) and the size limit."""
import numpy as np
import pytest
import torch

from tests import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import motifcl_amd
    motifcl_amd.load()
    from motifcl_amd import ops as _ops
    assert torch.cuda.is_available()
    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _case(oracle, seed, N, n_in, n_out, C):
    _, state, _, scale, v = synth.counter_case(seed, n_out, n_in, C, oracle=oracle)
    x, dy = synth.activations(seed + 1, N, n_in, n_out)
    return state, scale, v, dev(dy), dev(x)


def _lent(ops, case, N, n_in, n_out, C, hp, seed, strip):
    state, scale, v, dy, x = case
    d = [dev(state), dev(scale), dev(v)]
    nbytes = ops.fused_strip_workspace_nbytes(n_in, n_out, N) if strip else ops.fused_workspace_nbytes(n_in, n_out, N)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    ops.apply_update_fused(*d, dy, x, ws, C, hp[0], hp[1], 0.9, 1e-3, seed)
    if strip:
        ops.fused_check(ws, n_in, n_out, N)
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in d]


def _static(ops, case, C, hp, seed):
    state, scale, v, dy, x = case
    d = [dev(state), dev(scale), dev(v)]
    ops.apply_update_fused_static(*d, dy, x, C, hp[0], hp[1], 0.9, 1e-3, seed)
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in d]


def _same(a, b):
    for p, q in zip(a, b):
        assert np.array_equal(p.view(np.uint8), q.view(np.uint8))


def test_static_workspace_matches_lent_workspace_twice_in_a_row(ops, oracle):
    C = 11
    # first a tensor whose token chunks fill most of the array, then a smaller one, then the first again
    big = (4096, 768, 768, (3e-3, 0.01))    # N, in, out: full workspace, several token chunks
    small = (300, 288, 96, (0.05, 0.0))
    assert 0 < ops.fused_workspace_nbytes(big[1], big[2], big[0]) <= ops.NOALLOC_WORKSPACE_NBYTES
    for i, (N, n_in, n_out, hp) in enumerate((big, small, big)):
        case = _case(oracle, 100 + i, N, n_in, n_out, C)
        exp = _lent(ops, case, N, n_in, n_out, C, hp, 7 + i, strip=False)
        got = _static(ops, case, C, hp, 7 + i)
        _same(got, exp)
        assert not np.array_equal(got[0], case[0])  # the step did something


def test_static_workspace_takes_the_strip_path_for_large_layers(ops, oracle):
    C = 11
    # 4096 x 4096 needs 64 MiB of full workspace: beyond the array, so the strip path runs (with and
    # without scale learning); then a smaller full-workspace tensor through the same array
    N, n_in, n_out = 64, 4096, 4096
    assert ops.fused_workspace_nbytes(n_in, n_out, N) > ops.NOALLOC_WORKSPACE_NBYTES
    case = _case(oracle, 200, N, n_in, n_out, C)
    exp_s = _lent(ops, case, N, n_in, n_out, C, (3e-3, 0.02), 10, strip=True)
    _same(_static(ops, case, C, (3e-3, 0.02), 10), exp_s)
    exp = _lent(ops, case, N, n_in, n_out, C, (3e-3, 0.0), 11, strip=True)
    _same(_static(ops, case, C, (3e-3, 0.0), 11), exp)
    case2 = _case(oracle, 201, 128, 1024, 512, C)
    exp2 = _lent(ops, case2, 128, 1024, 512, C, (3e-3, 0.0), 12, strip=False)
    _same(_static(ops, case2, C, (3e-3, 0.0), 12), exp2)
    # and against the oracle: given its own gradient the strip step is the dense step
    state, scale, v, dy, x = case
    g = ops.matmul_transpose_a(dy, x).cpu().numpy()
    o = oracle.update_dense(state, scale, v, g, C, 3e-3, 0.0, 0.9, 1e-3, 11)
    _same(exp, o)


def test_static_workspace_rejects_what_does_not_fit(ops, oracle):
    from motifcl_amd import lib as mlib
    # 8200 x 8200 is no multiple of 128: its smaller workspace is an eighth of 269 MB, beyond the array
    n, n_in, n_out = 16, 8200, 8200
    assert ops.fused_strip_workspace_nbytes(n_in, n_out, n) > ops.NOALLOC_WORKSPACE_NBYTES
    state = torch.zeros(n_out * n_in // 4 * 3, dtype=torch.uint8, device="cuda")
    scale = torch.full((n_out,), 0.02, device="cuda")
    v = torch.zeros(n_out, device="cuda")
    dy = torch.randn(n, n_out, device="cuda") * 0.01
    x = torch.randn(n, n_in, device="cuda")
    with pytest.raises(mlib.MccError) as e:
        ops.apply_update_fused_static(state, scale, v, dy, x, 11, 3e-3, 0.0, 0.9, 1e-3, 1)
    assert e.value.code == -1 and "static" in e.value.message
    torch.cuda.synchronize()
    assert int(state.max()) == 0  # nothing was enqueued
    # invalid arguments are reported as by the lent-workspace entry point
    with pytest.raises(mlib.MccError, match="divisible by 4"):
        ops.apply_update_fused_static(state, scale, v, dy[:, :6].contiguous(), x[:, :6].contiguous(), 11, 3e-3, 0.0, 0.9,
                                      1e-3, 1)
