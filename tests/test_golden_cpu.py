"""The CPU oracle against the committed fixtures: the reference's known-answer vectors
(tests/golden/reference_known_answers.json) and the frozen update vectors
(tests/golden/update_vectors.npz, written by tests/golden/make_update_vectors.py)."""
import numpy as np

from tests import golden_cases as gc

F = np.float32


def _state(ka, oracle):
    C = ka["C"]
    codes = np.array([[gc.code_of(t, ka.get("counter", 0), C) for t in row] for row in ka["ternary"]], dtype=np.uint8)
    state = gc.pack_word_view(codes)
    assert np.array_equal(oracle.pack_codes(codes), state)  # the oracle packs as the word view says
    return state


def test_reference_known_answers(oracle):
    ka = gc.known_answers()
    pv = ka["packed_word_view"]
    assert np.array_equal(gc.pack_word_view(pv["codes"]), np.array(pv["bytes"], dtype=np.uint8).reshape(-1))
    assert np.array_equal(oracle.pack_codes(np.array(pv["codes"], dtype=np.uint8)),
                          np.array(pv["bytes"], dtype=np.uint8).reshape(-1))
    d = ka["decode_weight"]
    w = oracle.decode_weight(_state(d, oracle), np.array(d["scale"], dtype=F), d["C"], d["in_features"], d["out_features"])
    assert w.tolist() == d["weight"]
    b = ka["backward_input"]
    gx = oracle.backward_input(np.array(b["grad_out"], dtype=F), _state(b, oracle), np.array(b["scale"], dtype=F), b["C"],
                               b["in_features"])
    assert gx.tolist() == b["grad_x"]
    f = ka["forward"]
    y = oracle.forward(np.array(f["x"], dtype=F), _state(f, oracle), np.array(f["scale"], dtype=F), f["C"],
                       f["out_features"])
    assert y.tolist() == f["y"]


def test_oracle_reproduces_the_frozen_update_vectors(oracle):
    dense, fused = gc.update_vectors()
    assert len(dense) >= 8 and len(fused) >= 3
    for c in dense:
        st, sc, v = oracle.update_dense(c["state"], c["scale"], c["v"], c["G"], c["C"], c["lr"], c["lr_scale"],
                                        c["rms_beta"], c["rms_eps"], c["seed"])
        assert np.array_equal(st, c["state_new"]) and np.array_equal(sc, c["scale_new"]) and np.array_equal(v, c["v_new"])
        assert not np.array_equal(st, c["state"])  # the case does something
    for c in fused:
        st, sc, v, g = oracle.update_fused(c["state"], c["scale"], c["v"], c["dy"], c["x"], c["C"], c["lr"],
                                           c["lr_scale"], c["rms_beta"], c["rms_eps"], c["seed"])
        assert np.array_equal(g, c["G_seq"])
        assert np.array_equal(st, c["state_new"]) and np.array_equal(sc, c["scale_new"]) and np.array_equal(v, c["v_new"])
