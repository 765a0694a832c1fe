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
    # 4096 x 4096 needs 64 MiB of full workspace: beyond the array, so the strip path runs; then a
    # smaller strip-path-only... no: a smaller full-workspace tensor through the same array
    N, n_in, n_out = 64, 4096, 4096
    assert ops.fused_workspace_nbytes(n_in, n_out, N) > ops.NOALLOC_WORKSPACE_NBYTES
    case = _case(oracle, 200, N, n_in, n_out, C)
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
    # 4096 x 4096 with lr_scale != 0 has no strip path and 64 MiB of full workspace
    case = _case(oracle, 300, 16, 4096, 4096, 11)
    with pytest.raises(mlib.MccError) as e:
        _static(ops, case, 11, (3e-3, 0.01), 1)
    assert e.value.code == -1
    # a shape with neither: 4104 x 4096 (not a multiple of 128) at 67 MB
    case = _case(oracle, 301, 16, 4104, 4096, 11)
    with pytest.raises(mlib.MccError) as e:
        _static(ops, case, 11, (3e-3, 0.0), 1)
    assert e.value.code == -1 and "static" in e.value.message
