"""Pins the CPU oracle before anything is compared against it.

Sources of truth, in order: known-answer vectors held by the reference's own
tests, closed forms and invariants the mathematics fixes, and an independent
numpy model (tests/npmodel.py).  Each test names the mistake it would catch.
"""
import os
import re

import numpy as np
import pytest

from tests import npmodel

F = np.float32
REF_CL = "/root/reference/kernels/compact_counter.cl"


# --------------------------------------------------------------------------- codec
def _word_bytes(codes4):
    w = codes4[0] | (codes4[1] << 6) | (codes4[2] << 12) | (codes4[3] << 18)
    return [w & 0xFF, (w >> 8) & 0xFF, (w >> 16) & 0xFF]


def test_known_answer_decode_weight(oracle):
    # tests/test_vulkan_runtime_standalone.cpp:579-616: C=3, t = (1,0,-1,1),(0,1,1,-1), c = 0,
    # scales 0.5 / 2.0 -> {.5,0,-.5,.5, 0,2,2,-2}.  code(t) = (t+1)*5 + 2.
    code = lambda t: (t + 1) * 5 + 2
    rows = [[code(1), code(0), code(-1), code(1)], [code(0), code(1), code(1), code(-1)]]
    state = np.array(_word_bytes(rows[0]) + _word_bytes(rows[1]), dtype=np.uint8)
    # the oracle's packer must produce the same bytes as the 24-bit word view
    assert np.array_equal(oracle.pack_codes(np.array(rows, dtype=np.uint8)), state)
    w = oracle.decode_weight(state, np.array([0.5, 2.0], dtype=F), 3, 4, 2)
    assert w.tolist() == [[0.5, 0.0, -0.5, 0.5], [0.0, 2.0, 2.0, -2.0]]


def test_known_answer_grad_x(oracle):
    # tests/test_vulkan_runtime_standalone.cpp:1134-1160: closed form
    # grad_x[r,i] = go[r,0]*0.5*tern[i] + go[r,1]*2.0*tern[4+i].
    code = lambda t: (t + 1) * 5 + 2
    tern = [1, 0, -1, 1, 0, 1, 1, -1]
    state = oracle.pack_codes(np.array([code(t) for t in tern], dtype=np.uint8))
    go = np.array([[1.0, 2.0], [-1.0, 0.5]], dtype=F)
    gx = oracle.backward_input(go, state, np.array([0.5, 2.0], dtype=F), 3, 4)
    for r in range(2):
        for i in range(4):
            assert gx[r, i] == go[r, 0] * 0.5 * tern[i] + go[r, 1] * 2.0 * tern[4 + i]


def test_known_answer_forward(oracle):
    # tests/test_vulkan_backend.cpp:606-626: y[r,o] = sum_i x[r,i] * scale[o]*t[o,i]
    code = lambda t: (t + 1) * 5 + 2
    tern = np.array([[1, -1, 0, 1], [0, 1, 1, -1]])
    state = oracle.pack_codes(np.array([code(t) for t in tern.reshape(-1)], dtype=np.uint8))
    scale = np.array([0.25, 1.5], dtype=F)
    x = np.array([[1.0, 2.0, -1.0, 0.5], [-0.25, 0.75, 1.5, -2.0]], dtype=F)
    y = oracle.forward(x, state, scale, 3, 2)
    expect = x.astype(np.float64) @ (tern * scale[:, None].astype(np.float64)).T
    assert np.abs(y - expect).max() <= 1e-6


def test_pack_matches_word_view_exhaustively(oracle):
    # every 4-tuple of 6-bit codes: bytes == little-endian 24-bit word c0|c1<<6|c2<<12|c3<<18
    # (tests/test_vulkan_backend.cpp:582-592).  Catches a wrong shift or mask in pack/unpack.
    c = np.arange(64, dtype=np.uint8)
    codes = np.stack(np.meshgrid(c, c, c, c, indexing="ij"), axis=-1).reshape(-1, 4)
    state = oracle.pack_codes(codes)
    assert np.array_equal(state, npmodel.pack_state(codes))
    assert np.array_equal(oracle.unpack_codes(state).reshape(-1, 4), codes)


@pytest.mark.parametrize("C", list(range(1, 12)))
def test_codec_closed_form(oracle, C):
    lv = 2 * C - 1
    assert 3 * lv <= 64  # src/nn/compact_counter.cpp:61
    seen = set()
    for t in (-1, 0, 1):
        for c in range(-(C - 1), C):
            code = oracle.encode(t, c, C)
            assert code == (t + 1) * lv + (c + C - 1)
            assert oracle.decode(code, C) == (t, c)
            seen.add(code)
    assert seen == set(range(3 * lv))  # 63 reachable codes at C=11, code 63 never produced
    # codes beyond the reachable range still decode by the same formula (t = code/lv - 1)
    for code in range(3 * lv, 64):
        assert oracle.decode(code, C) == (code // lv - 1, code % lv - (C - 1))


# --------------------------------------------------------------------------- hash
def _unxorshift(x, s):
    y = x
    for _ in range(32 // s + 1):
        y = x ^ (y >> s)
    return y & 0xFFFFFFFF


def test_hash_is_the_invertible_lowbias32(oracle):
    # lowbias32 is a bijection: undo it with the modular inverses of its two multipliers.
    # A wrong shift, a swapped constant or a dropped step breaks the round trip.
    inv1 = pow(0x7FEB352D, -1, 1 << 32)
    inv2 = pow(0x846CA68B, -1, 1 << 32)
    assert (inv1, inv2) == (0x1D69E2A5, 0x43021123)  # published inverse constants
    rng = np.random.default_rng(1)
    for x in [0, 1, 2, 0xFFFFFFFF, 0x80000000] + rng.integers(0, 1 << 32, 2000).tolist():
        h = oracle.hash_u32(x)
        y = _unxorshift(h, 16)
        y = (y * inv2) & 0xFFFFFFFF
        y = _unxorshift(y, 15)
        y = (y * inv1) & 0xFFFFFFFF
        y = _unxorshift(y, 16)
        assert y == x
        assert h == npmodel.hash_u32(x)
    assert oracle.hash_u32(0) == 0


def test_hash_avalanche(oracle):
    # each input bit flips about half of the output bits (a degenerate mixer would not)
    rng = np.random.default_rng(2)
    xs = rng.integers(0, 1 << 32, 400).tolist()
    flips = [bin(oracle.hash_u32(x) ^ oracle.hash_u32(x ^ (1 << b))).count("1")
             for x in xs for b in range(32)]
    assert 15.0 < np.mean(flips) < 17.0


def test_uniform01_is_24_bits_of_the_hash(oracle):
    rng = np.random.default_rng(3)
    us = []
    for x in rng.integers(0, 1 << 32, 5000).tolist():
        u = oracle.uniform01(x)
        assert 0.0 <= u < 1.0
        assert u * 16777216.0 == float(oracle.hash_u32(x) & 0xFFFFFF)  # low 24 bits, exact
        us.append(u)
    assert abs(np.mean(us) - 0.5) < 0.02


@pytest.mark.skipif(not os.path.exists(REF_CL), reason="reference text not present")
def test_hash_constants_match_reference_text():
    text = open(REF_CL).read()
    body = text[text.index("cc_hash_u32"):text.index("cc_uniform01")]
    consts = [int(c, 16) for c in re.findall(r"0x([0-9a-fA-F]+)u", body)]
    shifts = [int(s) for s in re.findall(r">>\s*(\d+)", body)]
    assert consts == [0x7FEB352D, 0x846CA68B] and shifts == [16, 15, 16]


# --------------------------------------------------------------------------- row stats
def _random_case(rng, n_out, n_in, C, g_sigma=0.01, full_range=False):
    hi = 64 if full_range else 3 * (2 * C - 1)
    codes = rng.integers(0, hi, (n_out, n_in)).astype(np.uint8)
    G = (rng.standard_normal((n_out, n_in)) * g_sigma).astype(F)
    scale = (0.05 + rng.random(n_out)).astype(F)
    v = (rng.random(n_out) * g_sigma ** 2).astype(F)
    return codes, G, scale, v


@pytest.mark.parametrize("n_in", [4, 8, 68, 256, 260, 1028])
def test_row_stats_against_double_and_lane_model(oracle, n_in):
    rng = np.random.default_rng(n_in)
    C, n_out = 11, 3
    codes, G, scale, v = _random_case(rng, n_out, n_in, C)
    state = oracle.pack_codes(codes)
    v_new, s_new, dn = oracle.row_stats(state, scale, v, G, C, 0.01, 0.9, 1e-3)
    t = codes.astype(np.int64) // 21 - 1
    for row in range(n_out):
        # brute force in double: catches a dropped term, /in vs /sqrt(in), beta on the wrong side
        g = G[row].astype(np.float64)
        gsq = (g * g).sum() / n_in
        gs = (g * t[row]).sum() / np.sqrt(n_in)
        vv = 0.9 * float(v[row]) + (1.0 - float(F(0.9))) * gsq
        assert v_new[row] == pytest.approx(vv, rel=1e-5)
        assert dn[row] == pytest.approx(max(np.sqrt(vv), 1e-3), rel=1e-5)
        assert s_new[row] == pytest.approx(float(scale[row]) - 0.01 * gs, rel=1e-5, abs=1e-7)
        # literal 64-lane + tree emulation: exact
        mv, ms, md = npmodel.row_stats(codes[row], G[row], scale[row], v[row], C, 0.01, 0.9, 1e-3)
        assert (v_new[row], s_new[row], dn[row]) == (mv, ms, md)


def test_row_stats_closed_forms(oracle):
    C, n_in = 11, 64
    codes = np.full((4, n_in), oracle.encode(1, 0, C), dtype=np.uint8)
    state = oracle.pack_codes(codes)
    a = F(2.0 ** -7)
    G = np.full((4, n_in), a, dtype=F)
    G[1] *= -1
    scale = np.array([1.0, 1.0, 1e-5, 9.999], dtype=F)
    v = np.array([0.0, 4.0, 0.0, 0.0], dtype=F)
    # beta = 0.75: vv = 0.75*v + 0.25*a^2 exactly; sum G*t = +-64a, gs = +-8a
    v_new, s_new, dn = oracle.row_stats(state, scale, v, G, C, 0.5, 0.75, 1e-3)
    assert v_new[0] == F(0.25) * a * a and dn[0] == F(0.5) * a
    assert v_new[1] == F(3.0) + F(0.25) * a * a            # old moment decays by beta
    assert s_new[0] == F(1.0) - F(0.5) * (F(8.0) * a)      # aligned gradient shrinks the scale
    assert s_new[1] == F(1.0) + F(0.5) * (F(8.0) * a)
    assert s_new[2] == F(1e-5)                              # lower clamp
    G[3] *= -64                                              # big negative push: upper clamp
    assert oracle.row_stats(state, scale, v, G, C, 0.5, 0.75, 1e-3)[1][3] == F(10.0)
    # eps floor on the denominator
    assert oracle.row_stats(state, scale, v, G, C, 0.5, 0.75, 1.0)[2][0] == F(1.0)


# --------------------------------------------------------------------------- tick
def _integer_model(t, c, delta, C):
    """z = C*t + c moves by delta unless the ternary value saturates
    (docs/MEMORY_NATIVE_TRAINING_METHOD.md:48-55).  Returns (t', c')."""
    total = c + delta
    z = C * t + total
    # unique split with |c'| < C and c' carrying the sign of total (truncating carry)
    carry = abs(total) // C * (1 if total >= 0 else -1)
    nt, nc = t + carry, total - carry * C
    assert C * nt + nc == z
    if abs(nt) > 1:
        sgn = 1 if total > 0 else -1
        return sgn, sgn * (C - 1)
    return nt, nc


@pytest.mark.parametrize("C", [3, 4, 11])
def test_integer_ticks_are_rng_free_and_conserve_z(oracle, C):
    # rms_eps = 64 dominates the RMS so dn = 64; lr = 16; scale = C/4 so C/s_new = 4:
    # tick = -16 * (g/64) * 4 = -g exactly for integer g.  val is integral, so the
    # stochastic draw cannot matter and the new state has a closed form.
    # Catches: sign of the tick, C/s vs s/C, floor/trunc on negatives, remainder sign,
    # saturation value, clamp direction.
    lv = 2 * C - 1
    n_in = 4 * lv * 3
    gs = list(range(-4 * C - 1, 4 * C + 2))
    codes = np.tile(np.arange(3 * lv, dtype=np.uint8), n_in // (3 * lv) + 1)[:n_in]
    scale = np.full(len(gs), C / 4.0, dtype=F)
    v = np.zeros(len(gs), dtype=F)
    G = np.array([[g] * n_in for g in gs], dtype=F)
    state = oracle.pack_codes(np.tile(codes, (len(gs), 1)))
    outs = [oracle.update_dense(state, scale, v, G, C, 16.0, 0.0, 0.9, 64.0, seed)[0]
            for seed in (0, 777)]
    assert np.array_equal(outs[0], outs[1])  # integral ticks never consult the RNG
    new = oracle.unpack_codes(outs[0]).reshape(len(gs), n_in)
    for r, g in enumerate(gs):
        for i in range(n_in):
            t, c = oracle.decode(int(codes[i]), C)
            assert oracle.decode(int(new[r, i]), C) == _integer_model(t, c, -g, C), (g, t, c)


def test_hand_computed_ticks(oracle):
    # C=11, tick = +25 on (t=-1, c=3): total 28 -> carry 2, rem 6 -> (1, 6)
    assert oracle.decode(oracle.tick_code(oracle.encode(-1, 3, 11), -25.0, 11.0, 11.0, 1.0,
                                          11, 1.0, 0, 0), 11) == (1, 6)
    # tick = -25 on (t=0, c=3): total -22 -> carry -2 -> saturates at (-1, -10)
    assert oracle.decode(oracle.tick_code(oracle.encode(0, 3, 11), 25.0, 11.0, 11.0, 1.0,
                                          11, 1.0, 0, 0), 11) == (-1, -10)
    # tick = -5 on (t=1, c=2): total -3, no carry: the counter may go negative under t=+1
    assert oracle.decode(oracle.tick_code(oracle.encode(1, 2, 11), 5.0, 11.0, 11.0, 1.0,
                                          11, 1.0, 0, 0), 11) == (1, -3)


def test_rebase_uses_old_over_new_scale(oracle):
    # in=16, all t=+1, G = 1: sum G*t = 16, gs = 16/sqrt(16) = 4; lr_scale = 0.125 ->
    # scale_new = 1 - 0.5 = 0.5, ratio s_old/s_new = 2, C/s_new = 8 (C=4).
    # eps = 64 -> q = 1/64; lr = 8 -> tick = -8 * (1/64) * 8 = -1.  val = 2c - 1.
    # The inverse ratio (c/2 - 1) or C/s_old (tick -0.5) would give fractional values.
    C, n_in = 4, 16
    cs = [-3, -2, -1, 0, 1, 2, 3, 0] * 2
    codes = np.array([[oracle.encode(1, c, C) for c in cs]], dtype=np.uint8)
    state = oracle.pack_codes(codes)
    G = np.ones((1, n_in), dtype=F)
    ns, sc, vv = oracle.update_dense(state, np.ones(1, dtype=F), np.zeros(1, dtype=F), G,
                                     C, 8.0, 0.125, 0.9, 64.0, 5)
    assert sc[0] == F(0.5) and vv[0] == F(F(1.0) - F(0.9)) * F(1.0)
    new = oracle.unpack_codes(ns)
    for i, c in enumerate(cs):
        assert oracle.decode(int(new[i]), C) == _integer_model(1, 0, 2 * c - 1, C)


def test_zero_gradient_is_a_fixed_point(oracle):
    rng = np.random.default_rng(7)
    codes, _, scale, v = _random_case(rng, 5, 72, 11)
    state = oracle.pack_codes(codes)
    G = np.zeros((5, 72), dtype=F)
    ns, sc, vv = oracle.update_dense(state, scale, v, G, 11, 3e-3, 0.0, 0.9, 1e-3, 99)
    assert np.array_equal(ns, state)
    assert np.array_equal(sc, scale)
    assert np.array_equal(vv, F(0.9) * v)  # v <- beta*v exactly


def test_saturation_codes(oracle):
    C = 11
    rng = np.random.default_rng(8)
    codes, _, scale, v = _random_case(rng, 2, 64, C)
    state = oracle.pack_codes(codes)
    G = np.stack([np.full(64, -1e4, dtype=F), np.full(64, 1e4, dtype=F)])
    # the row RMS normalises |g|/dn to 1, so the tick is -+lr*C/scale: lr = 100 makes it >= 1000
    ns, _, _ = oracle.update_dense(state, scale, v, G, C, 100.0, 0.0, 0.0, 1e-3, 3)
    new = oracle.unpack_codes(ns).reshape(2, 64)
    assert (new[0] == 3 * 21 - 1).all()   # (t=+1, c=+10): negative gradient pushes up
    assert (new[1] == 0).all()            # (t=-1, c=-10)


def test_invariants_and_row_independence(oracle):
    C = 11
    rng = np.random.default_rng(9)
    codes, G, scale, v = _random_case(rng, 6, 132, C)
    state = oracle.pack_codes(codes)
    args = (C, 3e-3, 0.02, 0.9, 1e-3, 4242)
    ns, sc, vv = oracle.update_dense(state, scale, v, G, *args)
    new = oracle.unpack_codes(ns)
    assert new.max() < 63 and (new != codes.reshape(-1)).mean() > 0.05
    # rows are independent units and the RNG index is row*in + i, not tied to out_features:
    # updating the first 4 rows alone equals the first 4 rows of the full update
    rb = 132 // 4 * 3
    ns4, sc4, vv4 = oracle.update_dense(state[:4 * rb], scale[:4], v[:4], G[:4], *args)
    assert np.array_equal(ns4, ns[:4 * rb]) and np.array_equal(sc4, sc[:4]) and np.array_equal(vv4, vv[:4])
    # a different seed gives a different but equally valid state
    ns2, _, _ = oracle.update_dense(state, scale, v, G, C, 3e-3, 0.02, 0.9, 1e-3, 4243)
    assert not np.array_equal(ns2, ns)


@pytest.mark.parametrize("val", [0.3, -0.3, 2.75, -7.125])
def test_stochastic_rounding_is_unbiased(oracle, val):
    # E[ccv] = val: catches rnd < frac reversed, trunc instead of floor, frac taken from the
    # wrong side.  (t=0,c=0), C=11, s=11, dn=1, lr=1: tick = -g, so g = -val.
    C, n = 11, 20000
    tot = 0
    for seed in range(n):
        t, c = oracle.decode(oracle.tick_code(oracle.encode(0, 0, C), -val, 11.0, 11.0, 1.0,
                                              C, 1.0, seed, 12345), C)
        z = C * t + c
        assert z in (int(np.floor(val)), int(np.floor(val)) + 1)
        tot += z
    frac = val - np.floor(val)
    assert abs(tot / n - val) < 4.0 * np.sqrt(frac * (1 - frac) / n)


def test_draws_differ_across_elements_and_seeds(oracle):
    # same (code, g) at many element indices: a 0.5 fraction must split about evenly
    ups = sum(oracle.decode(oracle.tick_code(31, -0.5, 11.0, 11.0, 1.0, 11, 1.0, 1, e), 11)[1]
              for e in range(4000))
    assert 1800 < ups < 2200


# --------------------------------------------------------------------------- the draw's composition
REF_COMP = "/root/reference/kernels/vulkan/counter_apply_update_fused_f32.comp"


def _squash(text):
    return re.sub(r"\s+", "", text)


@pytest.mark.skipif(not (os.path.exists(REF_CL) and os.path.exists(REF_COMP)), reason="reference text not present")
def test_draw_call_site_matches_reference_text():
    # what the reference's three tick kernels write at the call site: the element index is
    # row*in + 4g + k, hashed, xor-ed with the seed, and cc_uniform01 hashes the result again and
    # keeps the LOW 24 bits.  Catches an oracle that follows a different reading of the text.
    cl = open(REF_CL).read()
    uni = _squash(cl[cl.index("cc_uniform01"):cl.index("cc_unpack4")])
    assert "(float)(cc_hash_u32(x)&0x00ffffffu)*(1.0f/16777216.0f)" in uni
    dense = _squash(cl[cl.index("void counter_apply_update_f32"):cl.index("void counter_row_stats_fused_f32")])
    fused = _squash(cl[cl.index("void counter_apply_update_fused_f32"):])
    draw = "floatrnd=cc_uniform01(seed^cc_hash_u32((uint)elem));"
    assert dense.count(draw) == 1 and fused.count(draw) == 1
    assert "intelem=row*in_features+g*4+k;" in dense
    assert "inti=g*4+k;intelem=row*in_features+i;" in fused
    for body in (dense, fused):
        assert "introw=gid/gpr;intg=gid-row*gpr;" in body and "intgpr=in_features/4;" in body
        assert "floatccv=f+(rnd<(val-f)?1.0f:0.0f);" in body
    comp = _squash(open(REF_COMP).read())
    assert "constfloatrnd=cc_uniform01(p.seed^cc_hash_u32(uint(elem)));" in comp
    assert "constinti=g*4+k;constintelem=row*p.in_features+i;" in comp
    assert "float(cc_hash_u32(h)&0x00ffffffu)*(1.0/16777216.0)" in comp


def _u01_low24(x):
    return npmodel.uniform01(x)


def _u01_high24(x):
    return F(npmodel.hash_u32(x) >> 8) * F(1.0 / 16777216.0)


# plausible wrong readings of the call site: (name, draw(seed, row, i, n_in))
_WRONG_DRAWS = [
    ("index not hashed", lambda s, r, i, n: _u01_low24(s ^ ((r * n + i) & 0xFFFFFFFF))),
    ("seed hashed instead of the index", lambda s, r, i, n: _u01_low24(npmodel.hash_u32(s) ^ ((r * n + i) & 0xFFFFFFFF))),
    ("xor of two hashes", lambda s, r, i, n: _u01_low24(npmodel.hash_u32(s) ^ npmodel.hash_u32((r * n + i) & 0xFFFFFFFF))),
    ("seed added, not xor-ed", lambda s, r, i, n: _u01_low24((s + npmodel.hash_u32((r * n + i) & 0xFFFFFFFF)) & 0xFFFFFFFF)),
    ("no second hash", lambda s, r, i, n: F((s ^ npmodel.hash_u32((r * n + i) & 0xFFFFFFFF)) & 0xFFFFFF) * F(1.0 / 16777216.0)),
    ("high 24 bits", lambda s, r, i, n: _u01_high24(s ^ npmodel.hash_u32((r * n + i) & 0xFFFFFFFF))),
    ("row dropped from the index", lambda s, r, i, n: _u01_low24(s ^ npmodel.hash_u32(i))),
    ("row stride in groups", lambda s, r, i, n: _u01_low24(s ^ npmodel.hash_u32((r * (n // 4) + i) & 0xFFFFFFFF))),
    ("column-major index", lambda s, r, i, n: _u01_low24(s ^ npmodel.hash_u32((i * 35 + r) & 0xFFFFFFFF))),
    ("group index instead of element index", lambda s, r, i, n: _u01_low24(s ^ npmodel.hash_u32((r * n + i) // 4))),
    ("code position swapped inside the group", lambda s, r, i, n: _u01_low24(s ^ npmodel.hash_u32((r * n + (i ^ 3)) & 0xFFFFFFFF))),
    ("one-based index", lambda s, r, i, n: _u01_low24(s ^ npmodel.hash_u32((r * n + i + 1) & 0xFFFFFFFF))),
]


def _frozen_case():
    from tests import golden_cases as gc
    dense, _ = gc.update_vectors()
    c = dense[1]  # 35 x 68, C = 3: the shape of tests/test_vulkan_counter_fused.cpp:57-60
    assert (c["n_out"], c["n_in"], c["C"]) == (35, 68, 3)
    return c


def _model_on(c, draw):
    return npmodel.update_dense(c["state"], c["scale"], c["v"], c["G"], c["C"], c["lr"], c["lr_scale"],
                                c["rms_beta"], c["rms_eps"], c["seed"], draw=draw)


def test_frozen_vector_is_the_reference_draw():
    # the committed vector is what the literal numpy model gives with the composition the
    # reference text shows (test above) ...
    c = _frozen_case()
    st, sc, v = _model_on(c, npmodel.draw_reference)
    assert np.array_equal(st, c["state_new"]) and np.array_equal(sc, c["scale_new"]) and np.array_equal(v, c["v_new"])


@pytest.mark.parametrize("name,draw", _WRONG_DRAWS, ids=[n.replace(" ", "_") for n, _ in _WRONG_DRAWS])
def test_frozen_vector_kills_wrong_draw_compositions(name, draw):
    # ... and every plausible other composition lands hundreds of counters elsewhere, so an
    # oracle or a kernel built on one of them cannot pass the frozen-vector tests
    c = _frozen_case()
    st, sc, v = _model_on(c, draw)
    assert np.array_equal(sc, c["scale_new"]) and np.array_equal(v, c["v_new"])  # statistics do not use the draw
    diff = (npmodel.unpack_state(st, 35 * 68) != npmodel.unpack_state(c["state_new"], 35 * 68)).sum()
    assert diff >= 50, (name, diff)


# --------------------------------------------------------------------------- whole update
@pytest.mark.parametrize("shape", [(2, 8, 3), (5, 68, 3), (3, 264, 11), (2, 4, 1)])
def test_update_dense_equals_numpy_model(oracle, shape):
    n_out, n_in, C = shape
    rng = np.random.default_rng(n_in)
    codes, G, scale, v = _random_case(rng, n_out, n_in, C, full_range=True)
    state = oracle.pack_codes(codes)
    for lr, lr_scale, eps in [(3e-3, 0.0, 1e-3), (0.05, 0.01, 1e-8), (1.0, 0.05, 1e-6)]:
        got = oracle.update_dense(state, scale, v, G, C, lr, lr_scale, 0.9, eps, 777)
        exp = npmodel.update_dense(state, scale, v, G, C, lr, lr_scale, 0.9, eps, 777)
        for a, b in zip(got, exp):
            assert np.array_equal(a, b)


def test_fused_equals_dense_on_sequential_gradient(oracle):
    # cfg of tests/test_vulkan_counter_fused.cpp:57-73: rows=37, in=68, out=35, C=3
    rng = np.random.default_rng(11)
    N, n_in, n_out, C = 37, 68, 35, 3
    x = (rng.standard_normal((N, n_in)) * 0.8).astype(F)
    dy = (rng.standard_normal((N, n_out)) * 0.9).astype(F)
    codes, _, scale, v = _random_case(rng, n_out, n_in, C)
    state = oracle.pack_codes(codes)
    # sequential-in-r fp32 accumulation, written as a numpy recurrence over r
    G = np.zeros((n_out, n_in), dtype=F)
    for r in range(N):
        G = (G + np.outer(dy[r], x[r]).astype(F)).astype(F)
    assert np.array_equal(oracle.grad_w_seq(dy, x), G)
    assert np.abs(G - dy.astype(np.float64).T @ x.astype(np.float64)).max() < 1e-4
    fused = oracle.update_fused(state, scale, v, dy, x, C, 1.0, 0.05, 0.9, 1e-6, 777)
    dense = oracle.update_dense(state, scale, v, G, C, 1.0, 0.05, 0.9, 1e-6, 777)
    for a, b in zip(fused[:3], dense):
        assert np.array_equal(a, b)
    assert not np.array_equal(fused[0], state) and not np.array_equal(fused[1], scale)


def test_init_state_matches_constructor_layout(oracle):
    # src/nn/compact_counter.cpp:64-84: c = 0, scale = gain*sqrt(3/(2 in)), v = 0
    tern = np.array([[1, 0, -1, 1, 0, 1, 1, -1]], dtype=np.int8)
    state, scale, v = oracle.init_state(tern, 3, 2.0)
    assert oracle.unpack_codes(state).tolist() == [(t + 1) * 5 + 2 for t in tern[0]]
    assert scale[0] == F(2.0) * np.sqrt(F(3.0) / (F(2.0) * F(8.0))) and v[0] == 0.0
