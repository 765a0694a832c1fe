"""Readers of the committed fixtures under tests/golden/ (shared by the CPU and the GPU test)."""
import json
import os

import numpy as np

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
F = np.float32


def known_answers():
    with open(os.path.join(HERE, "reference_known_answers.json")) as f:
        return json.load(f)


def code_of(t, c, C):
    return (t + 1) * (2 * C - 1) + (c + C - 1)


def pack_word_view(codes):
    """Bytes of rows of codes (multiples of 4 per row), by the 24-bit word rule of the fixture."""
    out = []
    flat = np.asarray(codes).reshape(-1, 4)
    for c in flat:
        w = int(c[0]) | int(c[1]) << 6 | int(c[2]) << 12 | int(c[3]) << 18
        out += [w & 255, (w >> 8) & 255, (w >> 16) & 255]
    return np.array(out, dtype=np.uint8)


def update_vectors():
    d = np.load(os.path.join(HERE, "update_vectors.npz"))  # plain arrays, no pickles
    dense, fused = [], []
    i = 0
    while "dense%d_hp" % i in d:
        hp = d["dense%d_hp" % i]
        dense.append(dict(n_out=int(hp[0]), n_in=int(hp[1]), C=int(hp[2]), lr=float(hp[3]), lr_scale=float(hp[4]),
                          rms_beta=float(hp[5]), rms_eps=float(hp[6]), seed=int(hp[7]),
                          **{k: d["dense%d_%s" % (i, k)] for k in
                             ("state", "scale", "v", "G", "state_new", "scale_new", "v_new")}))
        i += 1
    i = 0
    while "fused%d_hp" % i in d:
        hp = d["fused%d_hp" % i]
        fused.append(dict(N=int(hp[0]), n_in=int(hp[1]), n_out=int(hp[2]), C=int(hp[3]), lr=float(hp[4]),
                          lr_scale=float(hp[5]), rms_beta=float(hp[6]), rms_eps=float(hp[7]), seed=int(hp[8]),
                          **{k: d["fused%d_%s" % (i, k)] for k in
                             ("state", "scale", "v", "x", "dy", "G_seq", "state_new", "scale_new", "v_new")}))
        i += 1
    return dense, fused
