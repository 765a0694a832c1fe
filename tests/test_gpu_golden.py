"""The HIP path against the committed fixtures (no oracle, no reference needed on the GPU box):
the reference's known-answer vectors and the frozen update vectors under tests/golden/."""
import numpy as np
import pytest
import torch

from tests import golden_cases as gc
from tests.test_gpu_parity import dev, host, ops  # noqa: F401  (fixture)

pytestmark = pytest.mark.gpu
F = np.float32


def _state(ka):
    codes = np.array([[gc.code_of(t, ka.get("counter", 0), ka["C"]) for t in row] for row in ka["ternary"]], dtype=np.uint8)
    return gc.pack_word_view(codes)


def test_reference_known_answers_on_the_gpu(ops):
    ka = gc.known_answers()
    d = ka["decode_weight"]
    w = host(ops.decode_weight(dev(_state(d)), dev(np.array(d["scale"], dtype=F)), d["C"], d["in_features"],
                               d["out_features"]))
    assert w.tolist() == d["weight"]
    b = ka["backward_input"]
    gx = host(ops.backward_input(dev(np.array(b["grad_out"], dtype=F)), dev(_state(b)), dev(np.array(b["scale"], dtype=F)),
                                 b["C"], b["in_features"]))
    assert gx.tolist() == b["grad_x"]  # every product and sum of this vector is exact in binary32
    f = ka["forward"]
    y = host(ops.forward(dev(np.array(f["x"], dtype=F)), dev(_state(f)), dev(np.array(f["scale"], dtype=F)), f["C"],
                         f["out_features"]))
    assert y.tolist() == f["y"]


def test_update_only_reproduces_the_frozen_vectors(ops):
    dense, _ = gc.update_vectors()
    for c in dense:
        st, sc, v = dev(c["state"]), dev(c["scale"]), dev(c["v"])
        ops.apply_update_dense(st, sc, v, dev(c["G"]), c["C"], c["lr"], c["lr_scale"], c["rms_beta"], c["rms_eps"],
                               c["seed"])
        assert np.array_equal(host(st), c["state_new"]), (c["n_out"], c["n_in"])
        assert np.array_equal(host(sc), c["scale_new"]) and np.array_equal(host(v), c["v_new"])


def test_fused_step_against_the_frozen_vectors(ops):
    # the matrix cores sum the tokens in another order than the sequential sum the vectors were
    # made with: the gradient agrees to 1e-4 of its largest entry and few counters may flip
    _, fused = gc.update_vectors()
    for c in fused:
        g = host(ops.matmul_transpose_a(dev(c["dy"]), dev(c["x"])))
        assert np.abs(g - c["G_seq"]).max() <= 1e-4 * np.abs(c["G_seq"]).max()
        st, sc, v = dev(c["state"]), dev(c["scale"]), dev(c["v"])
        ws = torch.empty(ops.fused_workspace_nbytes(c["n_in"], c["n_out"], c["N"]), dtype=torch.uint8, device="cuda")
        ops.apply_update_fused(st, sc, v, dev(c["dy"]), dev(c["x"]), ws, c["C"], c["lr"], c["lr_scale"], c["rms_beta"],
                               c["rms_eps"], c["seed"])
        flips = (host(st) != c["state_new"]).mean()
        assert flips <= 0.01, flips
        np.testing.assert_allclose(host(v), c["v_new"], rtol=1e-4)
        np.testing.assert_allclose(host(sc), c["scale_new"], rtol=1e-4)
