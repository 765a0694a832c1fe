"""The entry points only enqueue kernels on the caller's stream (no allocation, no
synchronisation, no memset node), so a caller may capture a step into a HIP graph.  A captured
sequence of fused and update-only steps is replayed several times, with eager work and
synchronisations between the replays, and every replay is checked against the eager result."""
import numpy as np
import pytest
import torch

from tests import synth
from tests.test_gpu_parity import dev, ops  # noqa: F401  (fixture)

pytestmark = pytest.mark.gpu
F = np.float32


def fresh(shape, seed):
    n, n_in, n_out, C = shape
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 3 * (2 * C - 1), (n_out, n_in)).astype(np.uint32).reshape(-1, 4)
    word = codes[:, 0] | (codes[:, 1] << 6) | (codes[:, 2] << 12) | (codes[:, 3] << 18)
    state = np.stack([word & 255, (word >> 8) & 255, (word >> 16) & 255], axis=1).astype(np.uint8).reshape(-1)
    scale = np.full(n_out, 0.05, dtype=F)
    v = np.zeros(n_out, dtype=F)
    x, dy = synth.activations(seed + 1, n, n_in, n_out)
    return state, scale, v, x, dy


SMALL = [(256, 512, 256, 11), (320, 256, 384, 11)]   # the first splits its token range
# 256 x 256 tiles: one round of them, then 688 tiles -- equal spans with hand-off words on the full
# workspace, three passes with parked tiles on the strip workspace
LARGE = [(32, 4096, 4096, 11), (32, 11008, 4096, 11)]


@pytest.mark.parametrize("shapes", [SMALL, LARGE], ids=["small", "large"])
@pytest.mark.parametrize("path", ["workspace", "strip"])
def test_captured_steps_replay_like_eager(ops, path, shapes):
    if path == "strip":
        nbytes = [ops.fused_strip_workspace_nbytes(s[1], s[2], s[0]) for s in shapes]
    else:
        nbytes = [ops.fused_workspace_nbytes(s[1], s[2], s[0]) for s in shapes]
    host = [fresh(s, 10 + i) for i, s in enumerate(shapes)]
    ws = torch.empty(max(nbytes), dtype=torch.uint8, device="cuda")
    gw = torch.randn(shapes[0][2], shapes[0][1], device="cuda") * 0.01

    def one_step(tensors):
        for (st, sc, v, x, dy), shape in zip(tensors, shapes):
            ops.apply_update_fused(st, sc, v, dy, x, ws[: nbytes[shapes.index(shape)]], shape[3], 3e-3, 0.0, 0.9,
                                   1e-3, 77)
        st, sc, v, _, _ = tensors[0]
        ops.apply_update_dense(st, sc, v, gw, 11, 3e-3, 0.0, 0.9, 1e-3, 78)

    def device_copy():
        return [[dev(a) for a in h] for h in host]

    # eager reference: three steps in a row
    eager = device_copy()
    snapshots = []
    for _ in range(3):
        one_step(eager)
        torch.cuda.synchronize()
        snapshots.append([[t.clone() for t in tensors[:3]] for tensors in eager])

    graphed = device_copy()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        one_step(graphed)              # warm-up on the capture stream, then restore the inputs
        torch.cuda.synchronize()
        for tensors, h in zip(graphed, host):
            for t, a in zip(tensors[:3], h[:3]):
                t.copy_(dev(a))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            one_step(graphed)
    torch.cuda.synchronize()
    for r in range(3):
        graph.replay()
        torch.cuda.synchronize()
        junk = torch.randn(1 << 16, device="cuda").sum().item()  # eager work between replays
        assert np.isfinite(junk)
        for tensors, snap in zip(graphed, snapshots[r]):
            for got, want in zip(tensors[:3], snap):
                assert torch.equal(got, want), "replay %d differs from the eager step" % r
    if path == "strip":
        ops.fused_check(ws[: nbytes[0]], shapes[0][1], shapes[0][2], shapes[0][0])


@pytest.mark.parametrize("shape", [(256, 512, 256, 11), (32, 4096, 4096, 11)], ids=["full", "strip"])
def test_static_workspace_step_is_capturable_and_allocates_nothing(ops, shape):
    # the entry point without a workspace argument, after one eager call on this GPU (the call that
    # resolves the static array's address): captured, replayed three times against eager steps, with
    # the device's free memory unchanged over capture and replays
    n, n_in, n_out, C = shape
    if shape[1] == 4096:  # 64 MiB of gradient do not fit the static array: the strip path runs
        assert ops.fused_workspace_nbytes(n_in, n_out, n) > (32 << 20)
    st, sc, v, x, dy = fresh(shape, 31)

    def step(t, seed):
        ops.apply_update_fused_static(t[0], t[1], t[2], t[4], t[3], C, 3e-3, 0.0, 0.9, 1e-3, seed)

    eager = [dev(a) for a in (st, sc, v, x, dy)]
    snapshots = []
    for r in range(3):
        step(eager, 5)
        torch.cuda.synchronize()
        snapshots.append([t.clone() for t in eager[:3]])
    graphed = [dev(a) for a in (st, sc, v, x, dy)]
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        warm = [dev(a) for a in (st, sc, v, x, dy)]
        step(warm, 5)                                   # the first call on the capture stream is eager
        torch.cuda.synchronize()
        del warm
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        with torch.cuda.graph(graph, stream=side):
            step(graphed, 5)
    torch.cuda.synchronize()
    for r in range(3):
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(graphed[:3], snapshots[r]):
            assert torch.equal(got, want), "replay %d differs from the eager step" % r
    # torch's own allocator may hand memory back meanwhile; the library must not have taken any
    assert torch.cuda.mem_get_info()[0] >= free_before
    ops.fused_check(None, n_in, n_out, n)
