"""Writes tests/golden/update_vectors.npz: small update-only and fused cases with the outputs of the
CPU oracle (oracle/counter_oracle.c) frozen at the time of writing.

These are NOT outputs of MotifCL: its counter path only runs on an OpenCL or Vulkan device and
the reference tree holds no stored vector for it.  What the file pins is (1) that the oracle does
not drift -- tests/test_golden_cpu.py recomputes every case -- and (2) that the HIP kernels
reproduce the same bytes on the GPU box, where neither this script nor the reference need to be
present (tests/test_gpu_golden.py).  The oracle itself is pinned by tests/test_oracle_pins.py.

    python tests/golden/make_update_vectors.py        # from the repository root
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import counter_oracle as oracle  # noqa: E402
from tests import synth  # noqa: E402

F = np.float32
# (out, in, C, lr, lr_scale, rms_beta, rms_eps, seed, g_sigma, full_range)
DENSE = [
    (2, 8, 3, 0.05, 0.01, 0.9, 1e-8, 77, 0.5, False),       # tests/test_vulkan_backend.cpp:1183-1190 shape
    (35, 68, 3, 0.05, 0.01, 0.9, 1e-8, 4242, 0.05, False),  # tests/test_vulkan_counter_fused.cpp:57-60 shape
    (16, 256, 11, 3e-3, 0.0, 0.9, 1e-3, 12345, 0.01, False),
    (9, 516, 11, 3e-3, 1e-3, 0.9, 1e-3, 12346, 0.01, True),
    (5, 4096, 11, 3e-3, 0.0, 0.9, 1e-3, 99, 0.01, False),
    (3, 11008, 11, 3e-3, 0.0, 0.9, 1e-3, 100, 0.01, False),
    (3, 5124, 11, 1e-2, 0.0, 0.5, 1e-3, 101, 0.02, False),
    (4, 64, 1, 0.2, 0.0, 0.9, 1e-3, 5, 0.5, False),
]
# (tokens, in, out, C, lr, lr_scale, seed)
FUSED = [
    (2, 8, 2, 3, 0.05, 0.01, 3),
    (37, 68, 35, 3, 0.05, 0.01, 4),
    (64, 256, 32, 11, 3e-3, 0.0, 5),
]


def main():
    out = {}
    for i, (n_out, n_in, C, lr, lr_scale, beta, eps, seed, sigma, full) in enumerate(DENSE):
        codes, state, G, scale, v = synth.counter_case(1000 + i, n_out, n_in, C, g_sigma=sigma, full_range=full,
                                                       oracle=oracle)
        st, sc, vv = oracle.update_dense(state, scale, v, G, C, lr, lr_scale, beta, eps, seed)
        out["dense%d_hp" % i] = np.array([n_out, n_in, C, lr, lr_scale, beta, eps, seed], dtype=np.float64)
        for name, arr in (("state", state), ("scale", scale), ("v", v), ("G", G), ("state_new", st),
                          ("scale_new", sc), ("v_new", vv)):
            out["dense%d_%s" % (i, name)] = arr
    for i, (N, n_in, n_out, C, lr, lr_scale, seed) in enumerate(FUSED):
        codes, state, _, scale, v = synth.counter_case(2000 + i, n_out, n_in, C, oracle=oracle)
        x, dy = synth.activations(3000 + i, N, n_in, n_out)
        st, sc, vv, G = oracle.update_fused(state, scale, v, dy, x, C, lr, lr_scale, 0.9, 1e-3, seed)
        out["fused%d_hp" % i] = np.array([N, n_in, n_out, C, lr, lr_scale, 0.9, 1e-3, seed], dtype=np.float64)
        for name, arr in (("state", state), ("scale", scale), ("v", v), ("x", x), ("dy", dy), ("G_seq", G),
                          ("state_new", st), ("scale_new", sc), ("v_new", vv)):
            out["fused%d_%s" % (i, name)] = arr
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "update_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote %s (%d arrays, %d bytes)" % (path, len(out), os.path.getsize(path)))


if __name__ == "__main__":
    main()
