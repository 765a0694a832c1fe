#!/usr/bin/env python3
"""Benchmark of the compact-counter update on one MI355X.

Primary line (BASELINE config 4): the fused step of one 7B-shaped layer -- seven counter
tensors, 32768 tokens -- through mcc_compact_counter_apply_update_fused.  A "step" is one
fused update of all seven tensors.  The same JSON line carries, under "update_only",
BASELINE config 3: the update-only step over 224 7B-shaped tensors with precomputed
gradients (6.476 G counters, 25.9 GB of gradient, distinct buffer per tensor).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg0|cfg1|cfg2|cfg4]
                    [--no-update-only] [--no-cpu]

Inputs are synthetic and seeded (torch generator, seed 0): X ~ N(0,1), dY ~ N(0,0.01),
G ~ N(0,0.01), codes uniform on [0,62], scale = sqrt(3/(2 in)), v = 0, C = 11, lr = 3e-3,
lr_scale = 0, rms_beta = 0.9, rms_eps = 1e-3.  Everything is resident in HBM before the
timed region.  Kernel durations for the roofline come from HIP events recorded by the
library on the launch stream inside the timed region.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_BF16_TFLOPS = 2500.0  # dense bf16 MFMA
PEAK_MFMA_F32_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
C, LR, LR_SCALE, BETA, EPS = 11, 3e-3, 0.0, 0.9, 1e-3
BYTES_PER_PARAM = 5.5          # 4 (read G) + 0.75 (read state) + 0.75 (write state)

# HBM-side bytes per launch of the dominant kernels, measured offline with
# `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` on this same command (scaled by a plain
# 1 GiB copy; summaries and commands under profiles/).  They are reported, not re-measured
# here, and only for the default workloads they were measured on.
MEASURED_TRAFFIC_BYTES = {
    "cfg4/gemm_tn_f32": 8.94e9,       # average over the 7 contractions of a step (algorithmic 1.5 GB)
    "cfg4/fused_strip": 27.53e9,      # average over the 7 launches of a step, --fused-path strip
    "cfg3/update_rows": 36.16e9,      # the batched call of a step (algorithmic 35.64 GB)
}


def layer_shapes(dim, hidden):
    """(out, in) of the seven linears of one block: Wq Wk Wv Wo, W1 W3, W2."""
    return [(dim, dim)] * 4 + [(hidden, dim)] * 2 + [(dim, hidden)]


WORKLOADS = {
    # name: (description, [(out,in)...] per layer, layers, tokens)
    "cfg0": ("cfg0: single 288x288 counter linear, 4096 tokens, one fused update", [(288, 288)], 1, 4096),
    "cfg1": ("cfg1: stories15M-shaped full step (dim 288, hidden 768, 6 layers = 42 tensors), 8192 tokens",
             layer_shapes(288, 768), 6, 8192),
    "cfg2": ("cfg2: 110M-shaped step (dim 768, hidden 2048, 12 layers = 84 tensors), 16384 tokens",
             layer_shapes(768, 2048), 12, 16384),
    "cfg4": ("cfg4: 7B-shaped single-layer fused step (d=4096, hidden 11008, 7 linears), 32768 tokens",
             layer_shapes(4096, 11008), 1, 32768),
}


def pack_codes_torch(codes):
    """[out, in] uint8 codes -> packed state bytes, 4 codes per 3 bytes (little-endian word)."""
    import torch
    c = codes.view(-1, 4).to(torch.int32)
    w = c[:, 0] | (c[:, 1] << 6) | (c[:, 2] << 12) | (c[:, 3] << 18)
    b = torch.stack([w & 0xFF, (w >> 8) & 0xFF, (w >> 16) & 0xFF], dim=1)
    return b.to(torch.uint8).reshape(-1).contiguous()


def make_state(gen, n_out, n_in):
    import torch
    codes = torch.randint(0, 63, (n_out, n_in), dtype=torch.uint8, device="cuda", generator=gen)
    state = pack_codes_torch(codes)
    scale = torch.full((n_out,), math.sqrt(3.0 / (2.0 * n_in)), dtype=torch.float32, device="cuda")
    v = torch.zeros(n_out, dtype=torch.float32, device="cuda")
    return state, scale, v


def query(L, name):
    import ctypes
    ms, n = ctypes.c_double(), ctypes.c_uint64()
    rc = L.mcc_profiler_query(name.encode(), ctypes.byref(ms), ctypes.byref(n))
    assert rc == 0, L.mcc_last_error()
    return ms.value, n.value


def time_steps(step_fn, steps, warmup):
    import torch
    for i in range(warmup):
        step_fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step_fn(warmup + i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


PEAK_CLOCK_MHZ = 2400.0        # the engine clock the published matrix peaks are quoted at


CLOCK_PROBE = True   # --no-clock: counter runs want exactly steps + warmup launches


def clock_during(ops, fn, est_ms):
    """Shader clock (MHz) while fn() -- one unit of work of about est_ms -- runs back to back.

    A one-wave probe kernel on a side stream counts shader cycles against the constant-rate wall
    clock for 80 % of the stretch the repetitions take (at least 150 ms of work, at most 1.9 s)."""
    import torch
    if not CLOCK_PROBE:
        return None
    reps = max(1, int(math.ceil(150.0 / max(est_ms, 1e-3))))
    window = min(1.9, 0.8 * reps * est_ms * 1e-3)
    reps = min(reps, max(1, int(math.ceil(2.4 / max(est_ms * 1e-3, 1e-6)))))
    torch.cuda.synchronize()
    probe = ops.ClockProbe(window)
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    return probe.mhz()


def at_clock(roofline, mhz):
    """Adds the measured clock and the matrix peak scaled to it to a roofline object."""
    roofline["clock_mhz"] = mhz
    if mhz is None:
        return roofline
    roofline["peak_at_clock"] = roofline["peak"] * mhz / PEAK_CLOCK_MHZ
    roofline["frac_at_clock"] = roofline.get("executed", roofline["achieved"]) / roofline["peak_at_clock"]
    return roofline


def bench_fused(L, ops, name, steps, warmup, fused_path="workspace", graph=False, batched=False):
    import torch
    desc, shapes, layers, tokens = WORKLOADS[name]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    tensors = []
    ws_bytes = 0
    xs, dys = {}, {}
    for layer in range(layers):
        for (n_out, n_in) in shapes:
            # activations are shared by width inside a layer stack to bound memory on the small
            # configs; each 7B tensor still streams its own X/dY rows from HBM (>= 537 MB each)
            if n_in not in xs:
                xs[n_in] = torch.randn(tokens, n_in, device="cuda", generator=gen)
            if n_out not in dys:
                dys[n_out] = torch.randn(tokens, n_out, device="cuda", generator=gen) * 0.01
            tensors.append((make_state(gen, n_out, n_in), dys[n_out], xs[n_in], n_out, n_in))
            need = ops.fused_strip_workspace_nbytes(n_in, n_out, tokens) if fused_path == "strip" else 0
            # shapes the accumulator-resident step does not take fall back to the f32[out,in] workspace
            ws_bytes = max(ws_bytes, need or ops.fused_workspace_nbytes(n_in, n_out, tokens))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    params = sum(t[3] * t[4] for t in tensors)
    flops = sum(2.0 * tokens * t[3] * t[4] for t in tensors)

    def step(i):
        for k, ((state, scale, v), dy, x, n_out, n_in) in enumerate(tensors):
            ops.apply_update_fused(state, scale, v, dy, x, ws, C, LR, LR_SCALE, BETA, EPS,
                                   12345 + k + 1000 * i)

    if batched:
        # all tensors of the step in one call: grouped contraction, grouped slice sum, batched update
        fb = ops.FusedBatch([(st[0], st[1], st[2], dy, x) for (st, dy, x, _, _) in tensors], LR,
                            [12345 + k for k in range(len(tensors))])
        ws_bytes = fb.workspace_nbytes()
        del ws
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")

        def step(i):  # noqa: F811
            fb.set_seeds([12345 + k + 1000 * i for k in range(len(tensors))])
            ops.apply_update_fused_batched(fb, ws, C, LR_SCALE, BETA, EPS)

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    graph_ms = None
    if graph:
        # the same step captured once and replayed: what a launch-bound small model gains when the
        # host submits one graph instead of 3 launches per tensor (the seeds are baked in, so this
        # is a launch-cost measurement, not a training loop)
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            step(0)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                step(0)
        torch.cuda.synchronize()
        graph_ms = time_steps(lambda i: g.replay(), steps, 2)
    L.mcc_profiler_reset()
    L.mcc_profiler_enable(1)
    ms_per_step = time_steps(step, steps, 0)
    gemm_ms, gemm_n = query(L, "gemm_tn_f32")
    upd_ms, upd_n = query(L, "counter_update")
    strip_ms, strip_n = query(L, "fused_strip")
    kernel = "gemm_tn_f32"
    if strip_n and not gemm_n:
        kernel, gemm_ms, gemm_n = "fused_strip", strip_ms, strip_n
    L.mcc_profiler_enable(0)
    L.mcc_profiler_reset()
    # dominant kernel: the contraction.  One launch per tensor; flops per launch differ by
    # tensor, so achieved = (total algorithmic flops of the launches) / (their total duration).
    achieved = flops * steps / (gemm_ms * 1e-3) / 1e12
    out = {
        "value": params / (ms_per_step * 1e-3) / 1e9,
        "ms_per_step": ms_per_step,
        "config": {"workload": desc, "tensors": len(tensors), "params": params, "tokens": tokens,
                   "C": C, "lr": LR, "lr_scale": LR_SCALE, "rms_beta": BETA, "rms_eps": EPS},
        "roofline": {"bound": "mfma", "kernel": kernel, "achieved": achieved,
                     "peak": PEAK_MFMA_F32_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_MFMA_F32_TFLOPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(name + "/" + kernel),
                     "launches": gemm_n, "avg_launch_ms": gemm_ms / max(gemm_n, 1),
                     "algorithmic_flops_per_step": flops},
        "kernel_ms_per_step": {kernel: gemm_ms / steps, "counter_update": upd_ms / steps},
        "fused_path": fused_path, "batched_call": batched, "workspace_bytes": ws_bytes,
        "graph_replay_ms_per_step": graph_ms,
    }
    # the clock the dominant kernel runs at (the power limit holds it below the 2400 MHz of the
    # published peak): contraction alone on the two-kernel path, the whole step on the strip path
    if kernel == "gemm_tn_f32":
        gbuf = torch.empty(max(t[3] * t[4] for t in tensors), device="cuda")
        mats = [(t[1], t[2], gbuf[: t[3] * t[4]].view(t[3], t[4])) for t in tensors[:len(shapes)]]

        def contractions():
            for dy, x, g in mats:
                ops.matmul_transpose_a(dy, x, g)
        mhz = clock_during(ops, contractions, gemm_ms / steps / layers)
        del gbuf, mats
    else:
        mhz = clock_during(ops, lambda: step(0), ms_per_step)
    at_clock(out["roofline"], mhz)
    sample = tensors[0]
    del ws
    return out, sample, tokens


def bench_layer_products(L, ops, name, steps, warmup):
    """The other two contractions of a counter layer step (forward, input gradient) on the workload's shapes."""
    import torch
    desc, shapes, layers, tokens = WORKLOADS[name]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(2)
    out = {}
    xs, dys = {}, {}
    tensors = []
    for (n_out, n_in) in shapes:  # one layer's shapes: the products keep no state between calls
        if n_in not in xs:
            xs[n_in] = torch.randn(tokens, n_in, device="cuda", generator=gen)
        if n_out not in dys:
            dys[n_out] = torch.randn(tokens, n_out, device="cuda", generator=gen) * 0.01
        tensors.append((make_state(gen, n_out, n_in), n_out, n_in))
    flops = sum(2.0 * tokens * t[1] * t[2] for t in tensors)
    y = {n: torch.empty(tokens, n, device="cuda") for n in set(t[1] for t in tensors) | set(t[2] for t in tensors)}

    def step(_):
        for (state, scale, v), n_out, n_in in tensors:
            ops.forward(xs[n_in], state, scale, C, n_out, out=y[n_out])
            ops.backward_input(dys[n_out], state, scale, C, n_in, out=y[n_in])

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    L.mcc_profiler_reset()
    L.mcc_profiler_enable(1)
    time_steps(step, steps, 0)
    for kernel in ("counter_forward", "counter_backward_input"):
        ms, n = query(L, kernel)
        tf = flops * steps / (ms * 1e-3) / 1e12
        # three bf16 MFMA passes per product (the activation is split into three exact bf16 terms):
        # the matrix cores execute 3 x the algorithmic flops, priced against the dense bf16 peak
        out[kernel] = {"ms_per_step": ms / steps, "launches": n, "achieved": tf, "unit": "TFLOP/s",
                       "bound": "mfma", "executed": 3.0 * tf, "peak": PEAK_MFMA_BF16_TFLOPS,
                       "frac": 3.0 * tf / PEAK_MFMA_BF16_TFLOPS,
                       "algorithmic_rate_over_fp32_matrix_peak": tf / PEAK_MFMA_F32_TFLOPS}
    L.mcc_profiler_enable(0)
    L.mcc_profiler_reset()

    def forwards():
        for (state, scale, v), n_out, n_in in tensors:
            ops.forward(xs[n_in], state, scale, C, n_out, out=y[n_out])

    def backwards():
        for (state, scale, v), n_out, n_in in tensors:
            ops.backward_input(dys[n_out], state, scale, C, n_in, out=y[n_in])
    for kernel, fn in (("counter_forward", forwards), ("counter_backward_input", backwards)):
        at_clock(out[kernel], clock_during(ops, fn, out[kernel]["ms_per_step"]))
    out["tensors"] = len(tensors)
    out["tokens"] = tokens
    return out


def bench_side_optimizer(L, ops, steps, warmup):
    """Adam on one large FP32 tensor: 16 B read + 12 B written per element."""
    import torch
    n = 1 << 28  # 1 GiB per buffer
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    p = torch.randn(n, device="cuda", generator=gen)
    g = torch.randn(n, device="cuda", generator=gen) * 0.01
    m = torch.zeros(n, device="cuda")
    v = torch.zeros(n, device="cuda")
    for i in range(warmup):
        ops.adam_update(p, g, m, v, 3e-4, 0.9, 0.95, 1e-8, i + 1, 0.01)
    torch.cuda.synchronize()
    L.mcc_profiler_reset()
    L.mcc_profiler_enable(1)
    time_steps(lambda i: ops.adam_update(p, g, m, v, 3e-4, 0.9, 0.95, 1e-8, warmup + i + 1, 0.01), steps, 0)
    ms, launches = query(L, "adam_update")
    L.mcc_profiler_enable(0)
    L.mcc_profiler_reset()
    achieved = 28.0 * n * launches / (ms * 1e-3) / 1e9
    return {"workload": "adam_update_fast on one f32 tensor of 2^28 elements", "ms_per_launch": ms / launches,
            "value": n * launches / (ms * 1e-3) / 1e9, "unit": "Gparam/s",
            "roofline": {"bound": "hbm", "kernel": "adam_kernel", "achieved": achieved, "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS, "traffic": None,
                         "algorithmic_bytes_per_param": 28.0}}


def bench_update_only(L, ops, steps, warmup):
    import torch
    shapes = layer_shapes(4096, 11008)
    layers = 32
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    tensors = []
    for layer in range(layers):
        for (n_out, n_in) in shapes:
            g = torch.randn(n_out, n_in, device="cuda", generator=gen) * 0.01
            tensors.append((make_state(gen, n_out, n_in), g, n_out, n_in))
    params = sum(t[2] * t[3] for t in tensors)

    batch = ops.UpdateBatch([(st[0], st[1], st[2], g) for (st, g, _, _) in tensors], LR,
                            [12345 + k for k in range(len(tensors))])

    def step(i):
        # one call for the whole list: the optimizer step of the 224 tensors
        batch.set_seeds([12345 + k + 1000 * i for k in range(len(tensors))])
        ops.apply_update_dense_batched(batch, C, LR_SCALE, BETA, EPS)

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    L.mcc_profiler_reset()
    L.mcc_profiler_enable(1)
    ms_per_step = time_steps(step, steps, 0)
    upd_ms, upd_n = query(L, "counter_update")
    L.mcc_profiler_enable(0)
    L.mcc_profiler_reset()
    achieved = BYTES_PER_PARAM * params * steps / (upd_ms * 1e-3) / 1e9
    out = {
        "metric": "counter-synapse updates/s (Gparam/s), update-only",
        "value": params / (ms_per_step * 1e-3) / 1e9, "unit": "Gparam/s",
        "ms_per_step": ms_per_step, "steps": steps, "warmup": warmup,
        "config": {"workload": "cfg3: update-only, 224 7B-shaped tensors (32 layers x 7), "
                               "precomputed fp32 G, distinct buffer per tensor",
                   "tensors": len(tensors), "params": params},
        # one timed region per call = the launches that cover all 224 tensors
        "roofline": {"bound": "hbm", "kernel": "update_rows_kernel", "achieved": achieved,
                     "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS,
                     "traffic": MEASURED_TRAFFIC_BYTES["cfg3/update_rows"],
                     "launches": upd_n, "avg_launch_ms": upd_ms / max(upd_n, 1),
                     "algorithmic_bytes_per_param": BYTES_PER_PARAM,
                     "algorithmic_bytes_per_launch": BYTES_PER_PARAM * params},
    }
    out["roofline"]["clock_mhz"] = clock_during(ops, lambda: step(0), ms_per_step)
    sample = tensors[0]
    return out, sample, tensors


def cpu_baseline_fused(sample, tokens, rows, min_seconds=8.0):
    """Times the CPU oracle's fused update on the first `rows` rows of one tensor."""
    import numpy as np
    from oracle import counter_oracle as oracle
    (state, scale, v), dy, x, n_out, n_in = sample
    rows = min(rows, n_out)
    rb = n_in // 4 * 3
    h_state = state[: rows * rb].cpu().numpy().copy()
    h_scale, h_v = scale[:rows].cpu().numpy().copy(), v[:rows].cpu().numpy().copy()
    h_dy = np.ascontiguousarray(dy[:, :rows].cpu().numpy())
    h_x = x.cpu().numpy()
    t0 = time.perf_counter()
    passes = 0
    while passes == 0 or time.perf_counter() - t0 < min_seconds:
        oracle.update_fused(h_state, h_scale, h_v, h_dy, h_x, C, LR, LR_SCALE, BETA, EPS, 12345 + passes)
        passes += 1
    dt = time.perf_counter() - t0
    return {"value": passes * rows * n_in / dt / 1e9, "unit": "Gparam/s", "cores": oracle.num_threads(),
            "kind": "port", "seconds": dt,
            "sample": "CPU oracle (C, -O3 -mavx2 -ffp-contract=off, OpenMP) fused update of the first %d "
                      "rows of one [%d,%d] tensor at %d tokens (%.0f GFLOP per pass), %d passes; "
                      "extrapolates linearly in rows"
                      % (rows, n_out, n_in, tokens, 2.0 * tokens * rows * n_in / 1e9, passes)}


def cpu_baseline_dense(sample, min_seconds=4.0):
    from oracle import counter_oracle as oracle
    (state, scale, v), g, n_out, n_in = sample
    h = [t.cpu().numpy().copy() for t in (state, scale, v, g)]
    t0 = time.perf_counter()
    reps = 0
    while reps == 0 or time.perf_counter() - t0 < min_seconds:
        oracle.update_dense(h[0], h[1], h[2], h[3], C, LR, LR_SCALE, BETA, EPS, 12345 + reps)
        reps += 1
    dt = time.perf_counter() - t0
    return {"value": reps * n_out * n_in / dt / 1e9, "unit": "Gparam/s", "cores": oracle.num_threads(),
            "kind": "port", "seconds": dt,
            "sample": "CPU oracle update-only on one [%d,%d] tensor, %d passes" % (n_out, n_in, reps)}


def parity_leg(ops):
    """Correctness gates reported beside the speed figures: BASELINE config 0 (one 288x288
    tensor, 4096 tokens) on the GPU against the CPU oracle."""
    import numpy as np
    import torch
    from oracle import counter_oracle as oracle
    N, n_in, n_out = 4096, 288, 288
    rng = np.random.default_rng(0)
    state = oracle.pack_codes(rng.integers(0, 63, (n_out, n_in)).astype(np.uint8))
    scale = np.full(n_out, math.sqrt(3.0 / (2.0 * n_in)), dtype=np.float32)
    v = np.zeros(n_out, dtype=np.float32)
    x = rng.standard_normal((N, n_in)).astype(np.float32)
    dy = (rng.standard_normal((N, n_out)) * 0.01).astype(np.float32)
    d = [torch.from_numpy(a).cuda() for a in (state, scale, v)]
    ws = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, N), dtype=torch.uint8, device="cuda")
    ops.apply_update_fused(*d, torch.from_numpy(dy).cuda(), torch.from_numpy(x).cuda(), ws,
                           C, LR, LR_SCALE, BETA, EPS, 12345)
    torch.cuda.synchronize()
    g_gpu = ws.view(torch.float32)[: n_out * n_in].view(n_out, n_in).cpu().numpy()
    e_state, e_scale, e_v, g_seq = oracle.update_fused(state, scale, v, dy, x, C, LR, LR_SCALE, BETA, EPS, 12345)
    x_state, x_scale, x_v = oracle.update_dense(state, scale, v, g_gpu, C, LR, LR_SCALE, BETA, EPS, 12345)
    got = [t.cpu().numpy() for t in d]
    return {
        "workload": "cfg0: 288x288, 4096 tokens, one fused update, GPU vs CPU oracle",
        "state_scale_v_bit_exact_given_gpu_gradient": bool(
            np.array_equal(got[0], x_state) and np.array_equal(got[1], x_scale) and np.array_equal(got[2], x_v)),
        "max_abs_dG_over_max_abs_G_vs_sequential_sum": float(np.abs(g_gpu - g_seq).max() / np.abs(g_seq).max()),
        "counter_flip_mismatch_fraction_vs_sequential_sum": float(
            (oracle.unpack_codes(got[0]) != oracle.unpack_codes(e_state)).mean()),
        "counters_changed_fraction": float((oracle.unpack_codes(got[0]) != oracle.unpack_codes(state)).mean()),
    }


def parity_full_size_fused(ops, tokens=32768):
    """Size-independent properties at the cfg4 shapes: the two fused implementations (two-kernel and
    accumulator-resident) give the same bytes, and sampled rows of the contraction agree with a
    double-precision product."""
    import torch
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)
    out = {"tokens": tokens, "shapes": []}
    for (n_out, n_in) in [(4096, 4096), (11008, 4096), (4096, 11008)]:
        x = torch.randn(tokens, n_in, device="cuda", generator=gen)
        dy = torch.randn(tokens, n_out, device="cuda", generator=gen) * 0.01
        st0 = make_state(gen, n_out, n_in)
        results = []
        ws_full = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, tokens), dtype=torch.uint8, device="cuda")
        ws_strip = torch.empty(ops.fused_strip_workspace_nbytes(n_in, n_out, tokens), dtype=torch.uint8, device="cuda")
        for ws in (ws_full, ws_strip):
            d = [t.clone() for t in st0]
            ops.apply_update_fused(d[0], d[1], d[2], dy, x, ws, C, LR, LR_SCALE, BETA, EPS, 4242)
            ops.fused_check(ws, n_in, n_out, tokens)
            results.append(d)
        same = all(torch.equal(a, b) for a, b in zip(*results))
        rows = torch.arange(0, n_out, max(1, n_out // 8), device="cuda")[:8]
        g = ws_full.view(torch.float32)[: n_out * n_in].view(n_out, n_in)[rows].double()
        ref = dy[:, rows].double().t() @ x.double()
        rel = float((g - ref).abs().max() / ref.abs().max())
        changed = float((results[0][0] != st0[0]).float().mean())
        out["shapes"].append({"out": n_out, "in": n_in, "two_kernel_equals_accumulator_resident": bool(same),
                              "max_abs_dG_over_max_abs_G_vs_f64_on_8_rows": rel,
                              "state_bytes_changed_fraction": changed})
        del x, dy, ws_full, ws_strip, results, g, ref
        torch.cuda.empty_cache()
    return out


def parity_full_size_update_only(ops, tensors, picks=(0, 4, 6, 117, 223)):
    """cfg3 at full size: a sample of the 224 tensors, each updated on the GPU by the batched call
    and on the CPU by the oracle from the same snapshot; bytes must be identical."""
    import numpy as np
    import torch
    from oracle import counter_oracle as oracle
    picks = [k for k in picks if k < len(tensors)]
    before = {k: [t.cpu().numpy().copy() for t in tensors[k][0]] for k in picks}
    batch = ops.UpdateBatch([(st[0], st[1], st[2], g) for (st, g, _, _) in tensors], LR,
                            [777 + k for k in range(len(tensors))])
    ops.apply_update_dense_batched(batch, C, LR_SCALE, BETA, EPS)
    torch.cuda.synchronize()
    ok = []
    for k in picks:
        (st, g, n_out, n_in) = tensors[k]
        exp = oracle.update_dense(before[k][0], before[k][1], before[k][2], g.cpu().numpy(), C, LR, LR_SCALE,
                                  BETA, EPS, 777 + k)
        got = [t.cpu().numpy() for t in st]
        ok.append(bool(all(np.array_equal(a, b) for a, b in zip(got, exp))))
    return {"sampled_tensor_indices": picks, "shapes": [[tensors[k][2], tensors[k][3]] for k in picks],
            "state_scale_v_bit_exact": ok, "all_bit_exact": bool(all(ok))}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="cfg4", choices=sorted(WORKLOADS))
    ap.add_argument("--fused-path", default="workspace", choices=["workspace", "strip"],
                    help="workspace: contraction into a lent f32[out,in] buffer, then the update kernel; "
                         "strip: update applied from the contraction's accumulators, no weight-sized buffer")
    ap.add_argument("--graph", action="store_true",
                    help="also time the fused step captured into a HIP graph and replayed (reported beside "
                         "the eager figure, which stays the headline)")
    ap.add_argument("--batched", action="store_true",
                    help="fused leg through mcc_compact_counter_apply_update_fused_batched (one call per step)")
    ap.add_argument("--no-update-only", action="store_true", help="skip the cfg3 update-only leg")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-clock", action="store_true",
                    help="skip the shader-clock probes (they repeat each kernel outside the timed region)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run one plain 1 GiB device copy (torch copy_), the known-size kernel that "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by")
    ap.add_argument("--cpu-rows", type=int, default=4096, help="rows of one tensor for the CPU fused sample")
    args = ap.parse_args()
    global CLOCK_PROBE
    CLOCK_PROBE = not args.no_clock
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the path shards by output row with no "
                 "exchange); run with --gpus 1")
    if int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: launched with WORLD_SIZE > 1; this build measures one GPU only")

    import torch
    import motifcl_amd
    from motifcl_amd import ops
    L = motifcl_amd.load()  # raises if the HIP library is missing: there is no fallback
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    if args.traffic_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    fused, fused_sample, tokens = bench_fused(L, ops, args.workload, args.steps, args.warmup, args.fused_path, args.graph,
                                              args.batched)
    line = {
        "metric": "counter-synapse updates/s (Gparam/s)",
        "value": fused["value"], "unit": "Gparam/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": fused["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": fused["config"], "roofline": fused["roofline"],
        "kernel_ms_per_step": fused["kernel_ms_per_step"],
        "fused_path": fused["fused_path"], "fused_workspace_bytes": fused["workspace_bytes"],
        "graph_replay_ms_per_step": fused["graph_replay_ms_per_step"],
        "device": L.mcc_device_name().decode(),
    }
    if args.fused_path == "workspace":
        # the same step with the optional split-bf16 contraction (six bf16 matrix passes per
        # product, binary32 accuracy), reported beside the headline, which stays on the fp32
        # matrix instruction
        ops.set_contraction_mode(ops.CONTRACTION_BF16X6)
        try:
            alt, alt_sample, _ = bench_fused(L, ops, args.workload, max(3, args.steps // 2), 2, "workspace")
        finally:
            ops.set_contraction_mode(ops.CONTRACTION_FP32)
        del alt_sample
        tf = alt["roofline"]["achieved"]
        line["fused_split_bf16_contraction"] = {
            "ms_per_step": alt["ms_per_step"], "value": alt["value"], "unit": "Gparam/s",
            "roofline": {"bound": "mfma", "kernel": "gemm_tn_bf16x6", "achieved": tf, "executed": 6.0 * tf,
                         "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s", "frac": 6.0 * tf / PEAK_MFMA_BF16_TFLOPS,
                         "algorithmic_rate_over_fp32_matrix_peak": tf / PEAK_MFMA_F32_TFLOPS}}
        at_clock(line["fused_split_bf16_contraction"]["roofline"], alt["roofline"]["clock_mhz"])
        torch.cuda.empty_cache()
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_fused(fused_sample, tokens, args.cpu_rows)
        line["parity"] = parity_leg(ops)
        if args.workload == "cfg4":
            line["parity"]["full_size"] = parity_full_size_fused(ops)
    del fused_sample
    torch.cuda.empty_cache()
    line["side_optimizer"] = bench_side_optimizer(L, ops, max(3, args.steps), 2)
    torch.cuda.empty_cache()
    line["layer_products"] = bench_layer_products(L, ops, args.workload, max(2, args.steps // 2), 1)
    torch.cuda.empty_cache()
    if not args.no_update_only:
        uo, uo_sample, uo_tensors = bench_update_only(L, ops, args.steps, args.warmup)
        if not args.no_cpu:
            uo["cpu_baseline"] = cpu_baseline_dense(uo_sample)
            uo["parity_full_size"] = parity_full_size_update_only(ops, uo_tensors)
        del uo_tensors
        line["update_only"] = uo
    print(json.dumps(line))


if __name__ == "__main__":
    main()
