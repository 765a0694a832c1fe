"""Slow, literal numpy/float32 model of one counter update, for tiny shapes only.

Written independently of oracle/counter_oracle.c (different language, different
structure: explicit lane arrays, integer carry arithmetic) so that a mistake in
either shows up as a disagreement.  Follows kernels/compact_counter.cl:59-139.
"""
import numpy as np

F = np.float32
LANES = 64


def hash_u32(x):
    x &= 0xFFFFFFFF
    x ^= x >> 16
    x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15
    x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x


def uniform01(x):
    return F(hash_u32(x) & 0xFFFFFF) * F(1.0 / 16777216.0)


def unpack_state(state, n_codes):
    """24-bit little-endian word view: code k of group g = (word >> 6k) & 63."""
    b = np.asarray(state, dtype=np.uint32).reshape(-1, 3)
    word = b[:, 0] | (b[:, 1] << 8) | (b[:, 2] << 16)
    codes = np.stack([(word >> (6 * k)) & 0x3F for k in range(4)], axis=1).reshape(-1)
    assert codes.size == n_codes
    return codes.astype(np.int64)


def pack_state(codes):
    c = np.asarray(codes, dtype=np.uint32).reshape(-1, 4)
    word = c[:, 0] | (c[:, 1] << 6) | (c[:, 2] << 12) | (c[:, 3] << 18)
    out = np.stack([word & 0xFF, (word >> 8) & 0xFF, (word >> 16) & 0xFF], axis=1)
    return out.astype(np.uint8).reshape(-1)


def row_stats(codes_row, g_row, scale_row, v_row, C, lr_scale, beta, eps):
    """64 strided lane chains, then the s=32..1 tree; returns (v_new, scale_new, denom)."""
    n_in = g_row.size
    lv = 2 * C - 1
    gsq = np.zeros(LANES, dtype=F)
    gs = np.zeros(LANES, dtype=F)
    for lane in range(LANES):
        for g in range(lane, n_in // 4, LANES):
            for k in range(4):
                gw = F(g_row[4 * g + k])
                t = int(codes_row[4 * g + k]) // lv - 1
                gsq[lane] = F(gsq[lane] + F(gw * gw))
                gs[lane] = F(gs[lane] + F(gw * F(t)))
    s = LANES // 2
    while s > 0:
        gsq[:s] = gsq[:s] + gsq[s:2 * s]
        gs[:s] = gs[:s] + gs[s:2 * s]
        s //= 2
    mean_sq = F(gsq[0] / F(n_in))
    gsn = F(gs[0] / np.sqrt(F(n_in)))
    vv = F(F(F(beta) * F(v_row)) + F(F(F(1.0) - F(beta)) * mean_sq))
    denom = max(np.sqrt(vv), F(eps))
    sn = F(F(scale_row) - F(F(lr_scale) * gsn))
    scale_new = min(max(sn, F(1e-5)), F(10.0))
    return vv, F(scale_new), F(denom)


def draw_reference(seed, row, i, n_in):
    """The draw of kernels/compact_counter.cl:121,127: the element index row*in + i is hashed,
    xor-ed with the seed, and hashed again; the low 24 bits scale to [0, 1)."""
    elem = (row * n_in + i) & 0xFFFFFFFF
    return uniform01(seed ^ hash_u32(elem))


def tick(code, gw, s_old, s_new, dn, C, lr, rnd):
    """One stochastic-rounding tick for the draw `rnd`; the carry/remainder step is done on
    Python ints."""
    lv = 2 * C - 1
    t, c = code // lv - 1, code % lv - (C - 1)
    Cf = F(C)
    tk = F(F(F(-F(lr)) * F(F(gw) / F(dn))) * F(Cf / F(s_new)))
    val = F(F(F(c) * F(F(s_old) / F(s_new))) + tk)
    f = np.floor(val)
    total = int(f) + (1 if rnd < F(val - f) else 0)     # integer-valued ccv
    carry = abs(total) // C * (1 if total >= 0 else -1)  # truncation toward zero
    rem = total - carry * C
    nt = t + carry
    if nt > 1:
        nt, rem = 1, (C - 1 if total > 0 else (-(C - 1) if total < 0 else 0))
    elif nt < -1:
        nt, rem = -1, (C - 1 if total > 0 else (-(C - 1) if total < 0 else 0))
    return (nt + 1) * lv + rem + (C - 1)


def update_dense(state, scale, v, G, C, lr, lr_scale, beta, eps, seed, draw=draw_reference):
    """`draw(seed, row, i, n_in)` is the uniform variate of element (row, i); tests swap it to show
    that a wrong composition of seed, index and hash does not reproduce the frozen vectors."""
    n_out, n_in = G.shape
    codes = unpack_state(state, n_out * n_in).reshape(n_out, n_in)
    new_codes = np.zeros_like(codes)
    scale_out = np.zeros(n_out, dtype=F)
    v_out = np.zeros(n_out, dtype=F)
    for row in range(n_out):
        vv, sn, dn = row_stats(codes[row], G[row], scale[row], v[row], C, lr_scale, beta, eps)
        for i in range(n_in):
            new_codes[row, i] = tick(int(codes[row, i]), G[row, i], scale[row], sn, dn, C, lr,
                                     draw(seed, row, i, n_in))
        scale_out[row], v_out[row] = sn, vv
    return pack_state(new_codes), scale_out, v_out
