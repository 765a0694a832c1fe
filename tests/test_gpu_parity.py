"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle.

Bar: state bytes, scale and v bit-identical for the update-only step on the same fp32
gradient; for the fused step the contraction is held to a relative error of 1e-4 and the
fraction of counters that land on a different code is reported.
"""
import numpy as np
import pytest
import torch

from tests import synth

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def ops():
    import motifcl_amd
    motifcl_amd.load()  # fails loudly if the HIP library is missing
    from motifcl_amd import ops as _ops
    assert torch.cuda.is_available()
    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy()


HYPERS = [
    dict(lr=3e-3, lr_scale=0.0, rms_beta=0.9, rms_eps=1e-3),   # class defaults
    dict(lr=0.05, lr_scale=0.01, rms_beta=0.9, rms_eps=1e-8),  # tests/test_vulkan_backend.cpp:1185
    dict(lr=1.0, lr_scale=0.05, rms_beta=0.9, rms_eps=1e-6),   # tests/test_vulkan_counter_fused.cpp:68
]

# (out, in, C): reference test shapes, BASELINE shapes, every register-resident kernel
# variant (row length 64*ITERS groups and just below/above), and the generic fallback.
DENSE_SHAPES = [
    (2, 4, 3), (2, 8, 3), (35, 68, 3), (16, 16, 11), (256, 256, 11),
    (288, 288, 11), (768, 288, 11), (288, 768, 11), (96, 2048, 11), (48, 4096, 11),
    (12, 11008, 11), (5, 260, 11), (7, 1028, 8), (3, 3076, 11), (5, 6144, 11),
    (3, 8192, 4), (2, 11012, 11), (3, 16384, 11), (9, 516, 1),
    # long rows shared by four or eight cooperating waves in equal stretches: whole and ragged rows in
    # every class (up to 8192, 11264, 16384, 32768 weights), uneven last stretches, and beyond them
    # the rows one wave reads twice
    (4, 4352, 11), (3, 8448, 11), (3, 11268, 11), (2, 28672, 11), (2, 22532, 3),
    (3, 4100, 11), (2, 5120, 11), (2, 13824, 11), (2, 14336, 4), (2, 32768, 11), (2, 32772, 3), (1, 40960, 11),
]


def run_dense(ops, oracle, n_out, n_in, C, hp, seed, steps=1, full_range=False, g_sigma=0.01):
    _, state, G, scale, v = synth.counter_case(seed, n_out, n_in, C, g_sigma, full_range, oracle)
    d_state, d_scale, d_v = dev(state), dev(scale), dev(v)
    exp = (state, scale, v)
    for s in range(steps):
        Gs = np.roll(G, s, axis=1).copy()
        ops.apply_update_dense(d_state, d_scale, d_v, dev(Gs), C, hp["lr"], hp["lr_scale"],
                               hp["rms_beta"], hp["rms_eps"], 12345 + s)
        exp = oracle.update_dense(*exp, Gs, C, hp["lr"], hp["lr_scale"], hp["rms_beta"],
                                  hp["rms_eps"], 12345 + s)
    torch.cuda.synchronize()
    return (host(d_state), host(d_scale), host(d_v)), exp, state


def assert_bit_exact(got, exp):
    assert np.array_equal(got[0], exp[0]), "state bytes differ: %d of %d" % (
        (got[0] != exp[0]).sum(), exp[0].size)
    assert np.array_equal(got[1].view(np.uint32), exp[1].view(np.uint32)), "scale differs"
    assert np.array_equal(got[2].view(np.uint32), exp[2].view(np.uint32)), "v differs"


@pytest.mark.parametrize("shape", DENSE_SHAPES, ids=lambda s: "out%d_in%d_C%d" % s)
@pytest.mark.parametrize("hp", HYPERS, ids=["default", "lrscale", "lr1"])
def test_update_dense_bit_exact(ops, oracle, shape, hp):
    n_out, n_in, C = shape
    got, exp, state0 = run_dense(ops, oracle, n_out, n_in, C, hp, seed=n_in + n_out)
    assert_bit_exact(got, exp)
    if n_out * n_in >= 256:
        assert not np.array_equal(exp[0], state0)  # the case is not a no-op


def test_update_dense_several_steps_and_big_ticks(ops, oracle):
    hp = dict(lr=3e-3, lr_scale=0.002, rms_beta=0.9, rms_eps=1e-3)
    got, exp, _ = run_dense(ops, oracle, 64, 1024, 11, hp, seed=5, steps=4)
    assert_bit_exact(got, exp)
    # large gradients relative to the moment: carries of several levels and saturation
    got, exp, _ = run_dense(ops, oracle, 32, 512, 11, dict(lr=0.5, lr_scale=0.0, rms_beta=0.99, rms_eps=1e-3),
                            seed=6, g_sigma=1.0)
    assert_bit_exact(got, exp)
    codes = oracle.unpack_codes(exp[0])
    assert (codes == 0).any() and (codes == 62).any()


def test_update_dense_unreachable_codes_and_zero_gradient(ops, oracle):
    # codes 3*lv..63 never come out of an update but decode by the same formula
    got, exp, _ = run_dense(ops, oracle, 16, 256, 3, HYPERS[2], seed=7, full_range=True)
    assert_bit_exact(got, exp)
    _, state, G, scale, v = synth.counter_case(8, 8, 128, 11, oracle=oracle)
    d = [dev(state), dev(scale), dev(v)]
    ops.apply_update_dense(*d, dev(np.zeros_like(G)), 11, 3e-3, 0.0, 0.9, 1e-3, 1)
    assert np.array_equal(host(d[0]), state) and np.array_equal(host(d[1]), scale)
    assert np.array_equal(host(d[2]), F(0.9) * v)


def test_update_dense_misaligned_gradient_pointer(ops, oracle):
    # a gradient view that is only 4-byte aligned takes the generic kernel
    n_out, n_in, C = 6, 512, 11
    _, state, G, scale, v = synth.counter_case(9, n_out, n_in, C, oracle=oracle)
    buf = torch.empty(n_out * n_in + 1, dtype=torch.float32, device="cuda")
    gview = buf[1:].view(n_out, n_in)
    gview.copy_(dev(G))
    d = [dev(state), dev(scale), dev(v)]
    ops.apply_update_dense(*d, gview, C, 3e-3, 0.01, 0.9, 1e-3, 42)
    assert_bit_exact([host(t) for t in d], oracle.update_dense(state, scale, v, G, C, 3e-3, 0.01, 0.9, 1e-3, 42))


def test_update_dense_batched_matches_per_tensor_oracle(ops, oracle):
    # mixed row lengths (several kernel variants, the streamed fallback, a misaligned gradient)
    # and more tensors than one launch carries (64): every tensor must equal its own
    # single-tensor oracle result
    shapes = [(40, 288), (17, 4096), (9, 260), (6, 11008), (33, 768), (5, 16384), (12, 2048)]
    shapes += [(3 + (i % 5), 64 * (1 + i % 3)) for i in range(70)]
    C, hp = 11, dict(lr_scale=0.01, rms_beta=0.9, rms_eps=1e-3)
    cases, dev_tensors, lrs, seeds = [], [], [], []
    for i, (n_out, n_in) in enumerate(shapes):
        _, state, G, scale, v = synth.counter_case(1000 + i, n_out, n_in, C, oracle=oracle)
        if i == 2:  # 4-byte aligned gradient view
            buf = torch.empty(n_out * n_in + 1, dtype=torch.float32, device="cuda")
            g_dev = buf[1:].view(n_out, n_in)
            g_dev.copy_(dev(G))
        else:
            g_dev = dev(G)
        cases.append((state, scale, v, G))
        dev_tensors.append((dev(state), dev(scale), dev(v), g_dev))
        lrs.append(3e-3 * (1 + i % 3))
        seeds.append(777 + 13 * i)
    batch = ops.UpdateBatch(dev_tensors, lrs, seeds)
    ops.apply_update_dense_batched(batch, C, hp["lr_scale"], hp["rms_beta"], hp["rms_eps"])
    torch.cuda.synchronize()
    for i, (state, scale, v, G) in enumerate(cases):
        exp = oracle.update_dense(state, scale, v, G, C, lrs[i], hp["lr_scale"], hp["rms_beta"],
                                  hp["rms_eps"], seeds[i])
        assert_bit_exact([host(t) for t in dev_tensors[i][:3]], exp)


@pytest.mark.parametrize("n_in", [512, 4096, 11008, 10500, 5120], ids=lambda n: "in%d" % n)
def test_tiny_and_huge_gradients_take_the_exact_division(ops, oracle, n_in):
    # rows whose gradients leave the range of the reciprocal-based division (denormal and
    # 1e-30 entries next to ordinary ones; a row with a 1e25 entry) must still be bit-exact, and so
    # must rows with exact zeros, which hide the row's smallest magnitude from the cheap test --
    # in the one-wave kernels, the cooperating-wave kernel (11008, 10500) and the two-pass one
    n_out, C = 10, 11
    _, state, G, scale, v = synth.counter_case(31, n_out, n_in, C, oracle=oracle)
    G[0, ::3] = 1e-42
    G[1, ::5] = -3e-31
    G[2, 7] = 1e25
    G[3] *= 1e-20
    G[4] = 0.0
    G[5, ::2] = 0.0
    G[6, n_in - 1] = 0.0          # a single zero in the last wave's share
    G[7, ::7] = 0.0
    G[7, n_in // 2 + 1] = 1e-30   # zeros and a value too small for the reciprocal-based division
    G[8, 3] = 0.0
    G[8, n_in - 2] = -1e-41
    d = [dev(state), dev(scale), dev(v)]
    ops.apply_update_dense(*d, dev(G), C, 0.5, 0.0, 0.9, 0.0, 99)
    assert_bit_exact([host(t) for t in d], oracle.update_dense(state, scale, v, G, C, 0.5, 0.0, 0.9, 0.0, 99))


def test_integer_ticks_closed_form_on_gpu(ops, oracle):
    # tick = -g exactly (see tests/test_oracle_pins.py): z = C*t + c moves by -g or saturates
    C = 11
    lv = 2 * C - 1
    n_in = 4 * lv * 3
    gs = list(range(-4 * C - 1, 4 * C + 2))
    codes = np.tile(np.arange(3 * lv, dtype=np.uint8), n_in // (3 * lv) + 1)[:n_in]
    state = oracle.pack_codes(np.tile(codes, (len(gs), 1)))
    G = np.array([[g] * n_in for g in gs], dtype=F)
    d = [dev(state), dev(np.full(len(gs), C / 4.0, dtype=F)), dev(np.zeros(len(gs), dtype=F))]
    ops.apply_update_dense(*d, dev(G), C, 16.0, 0.0, 0.9, 64.0, 3)
    new = oracle.unpack_codes(host(d[0])).reshape(len(gs), n_in).astype(int)
    t0, c0 = codes.astype(int) // lv - 1, codes.astype(int) % lv - (C - 1)
    for r, g in enumerate(gs):
        total = c0 - g
        carry = np.sign(total) * (np.abs(total) // C)
        nt, nc = t0 + carry, total - carry * C
        sat = np.abs(nt) > 1
        nt = np.where(sat, np.sign(total), nt)
        nc = np.where(sat, np.sign(total) * (C - 1), nc)
        assert np.array_equal(new[r], (nt + 1) * lv + nc + C - 1)


GEMM_SHAPES = [(37, 35, 68), (2, 2, 8), (33, 7, 5), (4096, 288, 288), (1000, 768, 288),
               (512, 288, 768), (640, 300, 1028), (256, 1024, 2048),
               # 256 x 256 tiles: one whole round; two rounds of wide tiles + small tiles for the other
               # rows, and the same split by columns; 3.5 rounds
               (48, 4096, 4096), (32, 11008, 4096), (32, 4096, 11008), (16, 14336, 4096)]


@pytest.mark.parametrize("kmn", GEMM_SHAPES, ids=lambda s: "k%d_m%d_n%d" % s)
def test_matmul_transpose_a(ops, kmn):
    k, m, n = kmn
    rng = np.random.default_rng(k + m + n)
    a = rng.standard_normal((k, m)).astype(F)
    b = rng.standard_normal((k, n)).astype(F)
    c = host(ops.matmul_transpose_a(dev(a), dev(b)))
    ref = a.astype(np.float64).T @ b.astype(np.float64)
    rel = np.linalg.norm(c - ref) / np.linalg.norm(ref)
    assert rel <= 1e-5, rel  # tolerance: fp32 accumulation, relative Frobenius error
    assert np.abs(c - ref).max() <= 1e-4 * np.abs(ref).max()


@pytest.mark.parametrize("kmn", [(48, 4096, 4096), (32, 11008, 4096), (32, 4096, 11008)],
                         ids=lambda s: "k%d_m%d_n%d" % s)
def test_every_tile_shape_of_the_contraction_gives_the_same_bits(ops, kmn):
    # 256 x 256 tiles, the row / column split with small tiles on the rest, and the 64 x 64 tiles a
    # narrow block of the same operands gets: every output element sums its tokens in the same
    # order, so the overlapping blocks must agree bit for bit
    k, m, n = kmn
    rng = np.random.default_rng(m + n)
    a = rng.standard_normal((k, m)).astype(F)
    b = rng.standard_normal((k, n)).astype(F)
    full = host(ops.matmul_transpose_a(dev(a), dev(b)))
    for r0 in (0, (m // 2) // 128 * 128, m - 128):
        block = host(ops.matmul_transpose_a(dev(np.ascontiguousarray(a[:, r0:r0 + 128])), dev(b)))
        assert np.array_equal(block, full[r0:r0 + 128]), r0
    for c0 in (0, n - 128):
        block = host(ops.matmul_transpose_a(dev(a), dev(np.ascontiguousarray(b[:, c0:c0 + 128]))))
        assert np.array_equal(block, full[:, c0:c0 + 128]), c0


FUSED_SHAPES = [  # (N, in, out, C)
    (2, 8, 2, 3),        # tests/test_vulkan_backend.cpp:1183
    (37, 68, 35, 3),     # tests/test_vulkan_counter_fused.cpp:57-60
    (64, 256, 256, 11),  # tests/test_memory_truth_gate.cpp:34
    (4096, 288, 288, 11),  # BASELINE config 0
    (1024, 768, 288, 11), (1024, 288, 768, 11),
    # BASELINE config 2 (dim 768, hidden 2048): square, up and down projections
    (512, 768, 768, 11), (512, 768, 2048, 11), (512, 2048, 768, 11), (2048, 768, 2048, 11), (2048, 2048, 768, 11),
    # BASELINE config 4 (dim 4096, hidden 11008) at few tokens: one shape per tile plan of the
    # contraction (whole rounds of wide tiles; wide + small tiles split by rows, by columns)
    (64, 4096, 4096, 11), (512, 4096, 4096, 11), (32, 4096, 11008, 11), (32, 11008, 4096, 11),
]


@pytest.mark.parametrize("shape", FUSED_SHAPES, ids=lambda s: "N%d_in%d_out%d_C%d" % s)
def test_update_fused(ops, oracle, shape):
    N, n_in, n_out, C = shape
    hp = HYPERS[0] if C == 11 else HYPERS[1]
    _, state, _, scale, v = synth.counter_case(N, n_out, n_in, C, oracle=oracle)
    x, dy = synth.activations(N + 1, N, n_in, n_out)
    d = [dev(state), dev(scale), dev(v)]
    ws = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, N), dtype=torch.uint8, device="cuda")
    ops.apply_update_fused(*d, dev(dy), dev(x), ws, C, hp["lr"], hp["lr_scale"], hp["rms_beta"],
                           hp["rms_eps"], 777)
    torch.cuda.synchronize()
    got = [host(t) for t in d]
    g_gpu = host(ws.view(torch.float32)[: n_out * n_in].view(n_out, n_in))
    e_state, e_scale, e_v, g_seq = oracle.update_fused(state, scale, v, dy, x, C, hp["lr"], hp["lr_scale"],
                                                      hp["rms_beta"], hp["rms_eps"], 777)
    # tier 2: the contraction agrees with the reference's sequential fp32 sum to 1e-4 ...
    rel = np.abs(g_gpu - g_seq).max() / np.abs(g_seq).max()
    assert rel <= 1e-4, rel
    # ... and both sit within fp32 summation error of the exact product
    g_exact = dy.astype(np.float64).T @ x.astype(np.float64)
    assert np.abs(g_gpu - g_exact).max() <= np.abs(g_seq - g_exact).max() * 2 + 1e-7 * np.abs(g_exact).max()
    # given its own gradient, the fused step is the dense step, bit for bit
    assert_bit_exact(got, oracle.update_dense(state, scale, v, g_gpu, C, hp["lr"], hp["lr_scale"],
                                              hp["rms_beta"], hp["rms_eps"], 777))
    # counters that land on another code because the gradient differs in the last bits
    flips = (oracle.unpack_codes(got[0]) != oracle.unpack_codes(e_state)).mean()
    print("fused N=%d in=%d out=%d: max|dG|/max|G|=%.2e  counter-flip mismatch=%.3e" % (N, n_in, n_out, rel, flips))
    assert flips <= 2e-3
    assert np.allclose(got[1], e_scale, rtol=1e-5, atol=0) and np.allclose(got[2], e_v, rtol=1e-5, atol=0)


def test_two_identical_fused_updates_agree_exactly(ops, oracle):
    # tests/test_vulkan_counter_fused.cpp:120-133: same inputs and seed => identical bytes
    N, n_in, n_out, C = 37, 68, 35, 3
    _, state, _, scale, v = synth.counter_case(1, n_out, n_in, C, oracle=oracle)
    x, dy = synth.activations(2, N, n_in, n_out, 0.8, 0.9)
    res = []
    for _ in range(2):
        d = [dev(state), dev(scale), dev(v)]
        ws = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, N), dtype=torch.uint8, device="cuda")
        ops.apply_update_fused(*d, dev(dy), dev(x), ws, C, 1.0, 0.05, 0.9, 1e-6, 777)
        res.append([host(t) for t in d])
    for a, b in zip(*res):
        assert np.array_equal(a, b)
    assert not np.array_equal(res[0][0], state) and not np.array_equal(res[0][1], scale)


# (N, in, out, C): reference test shapes, slab tails (in or out not a multiple of 32, out not a
# multiple of 4), both tile sizes, and a full-range state (codes the update cannot produce)
LINEAR_SHAPES = [(2, 4, 2, 3), (37, 68, 35, 3), (64, 256, 256, 11), (100, 288, 768, 11),
                 (130, 768, 290, 11), (2048, 1024, 1280, 11), (1500, 2048, 1027, 4), (1, 4, 1, 11),
                 (128, 128, 128, 11), (256, 384, 256, 3), (128, 4096, 128, 11), (384, 160, 2048, 1),
                 (4096, 256, 2048, 11), (4096, 2048, 256, 11),  # 256-column tiles: forward, grad_x
                 # 256 such tiles and 16 slabs or more: the kernel whose waves either stage or multiply;
                 # 17 and 19 slabs leave a ragged end to its look-ahead, C = 1 is not ternary
                 (4096, 512, 2048, 11), (4096, 2048, 512, 11), (4096, 544, 2048, 3), (4096, 2048, 608, 4),
                 (4096, 640, 2048, 1), (2048, 4096, 1024, 1),
                 # a ragged token count over the same kernels: whole 128-row tiles, then the checked kernel
                 (4100, 512, 2048, 11), (4223, 2048, 512, 3), (200, 256, 128, 11)]


@pytest.mark.parametrize("shape", LINEAR_SHAPES, ids=lambda s: "N%d_in%d_out%d_C%d" % s)
def test_decode_forward_backward_input(ops, oracle, shape):
    N, n_in, n_out, C = shape
    _, state, _, scale, _ = synth.counter_case(N, n_out, n_in, C, full_range=(C == 4), oracle=oracle)
    x, dy = synth.activations(N, N, n_in, n_out, 0.8, 0.9)
    w = host(ops.decode_weight(dev(state), dev(scale), C, n_in, n_out))
    assert np.array_equal(w, oracle.decode_weight(state, scale, C, n_in, n_out))
    y = host(ops.forward(dev(x), dev(state), dev(scale), C, n_out))
    y_ref = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(y - y_ref).max() <= 2e-5 * max(1.0, np.abs(y_ref).max())  # tests/test_vulkan_counter_fused.cpp:107
    # against the sequential fp32 sum of the oracle as well: the matrix cores sum in another order
    assert np.abs(y - oracle.forward(x, state, scale, C, n_out)).max() <= 1e-4 * max(1.0, np.abs(y_ref).max())
    gx = host(ops.backward_input(dev(dy), dev(state), dev(scale), C, n_in))
    gx_ref = dy.astype(np.float64) @ w.astype(np.float64)
    # relative error of the whole gradient <= 1e-4 (tests/test_memory_truth_gate.cpp:86-92) and
    # elementwise within the forward tolerance
    assert np.linalg.norm(gx - gx_ref) <= 1e-4 * max(np.linalg.norm(gx_ref), 1e-30)
    assert np.abs(gx - gx_ref).max() <= 2e-5 * max(1.0, np.abs(gx_ref).max())
    assert np.abs(gx - oracle.backward_input(dy, state, scale, C, n_in)).max() <= 1e-4 * max(1.0, np.abs(gx_ref).max())


@pytest.mark.parametrize("shape", [(256, 4096, 512), (4096, 2048, 2048)], ids=lambda s: "N%d_in%d_out%d" % s)
def test_split_activation_products_keep_binary32_accuracy(ops, oracle, shape):
    # forward and grad_x run on the bf16 matrix cores with every activation split into three
    # bf16 terms whose products with the ternary weight are exact: the error against a
    # double-precision product must be that of an fp32 summation (the oracle's), not of bf16.
    # The second shape takes the kernel whose waves either stage or multiply.
    N, n_in, n_out = shape
    C = 11
    rng = np.random.default_rng(5)
    _, state, _, scale, _ = synth.counter_case(77, n_out, n_in, C, oracle=oracle)
    # activations over 12 binades, so that the low-order terms matter
    x = (rng.standard_normal((N, n_in)) * np.exp2(rng.integers(-6, 6, (N, n_in)))).astype(F)
    dy = (rng.standard_normal((N, n_out)) * np.exp2(rng.integers(-6, 6, (N, n_out)))).astype(F)
    w = oracle.decode_weight(state, scale, C, n_in, n_out).astype(np.float64)
    sample = slice(0, N, max(1, N // 256))  # the sequential sum of the oracle on 256 rows
    for name, got, ref, seq in (
            ("forward", host(ops.forward(dev(x), dev(state), dev(scale), C, n_out)), x.astype(np.float64) @ w.T,
             oracle.forward(np.ascontiguousarray(x[sample]), state, scale, C, n_out)),
            ("grad_x", host(ops.backward_input(dev(dy), dev(state), dev(scale), C, n_in)), dy.astype(np.float64) @ w,
             oracle.backward_input(np.ascontiguousarray(dy[sample]), state, scale, C, n_in))):
        err_gpu = np.abs(got - ref).max() / np.abs(ref).max()
        err_seq = np.abs(seq - ref[sample]).max() / np.abs(ref).max()
        print("%s: max error / max|.|  matrix cores %.2e, sequential fp32 sum %.2e" % (name, err_gpu, err_seq))
        assert err_gpu <= 2.0 * err_seq + 1e-7
        assert err_gpu <= 2e-6


def test_known_answer_vectors_on_gpu(ops, oracle):
    # tests/test_vulkan_runtime_standalone.cpp:579-638
    code = lambda t: (t + 1) * 5 + 2
    tern = [1, 0, -1, 1, 0, 1, 1, -1]
    state = oracle.pack_codes(np.array([code(t) for t in tern], dtype=np.uint8))
    scale = np.array([0.5, 2.0], dtype=F)
    w = host(ops.decode_weight(dev(state), dev(scale), 3, 4, 2))
    assert w.tolist() == [[0.5, 0.0, -0.5, 0.5], [0.0, 2.0, 2.0, -2.0]]
    go = np.array([[1.0, 2.0], [-1.0, 0.5]], dtype=F)
    gx = host(ops.backward_input(dev(go), dev(state), dev(scale), 3, 4))
    for r in range(2):
        for i in range(4):
            assert gx[r, i] == go[r, 0] * 0.5 * tern[i] + go[r, 1] * 2.0 * tern[4 + i]


@pytest.mark.gpu
def test_clock_probe_reports_a_plausible_shader_clock():
    # a measurement aid: one wave sleeps 20 ms of wall clock on a side stream and counts shader cycles
    import torch
    from motifcl_amd import ops
    probe = ops.ClockProbe(0.02)
    x = torch.randn(4096, 4096, device="cuda")
    for _ in range(10):
        x = x @ x * 1e-3
    torch.cuda.synchronize()
    mhz = probe.mhz()
    assert 100.0 < mhz < 3000.0, mhz
    with pytest.raises(RuntimeError):
        ops.ClockProbe(5.0)
