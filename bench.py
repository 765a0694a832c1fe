#!/usr/bin/env python3
"""Benchmark of the compact-counter update on one MI355X.

Primary line (BASELINE config 4): the fused step of one 7B-shaped layer -- seven counter
tensors, 32768 tokens -- through mcc_compact_counter_apply_update_fused.  A "step" is one
fused update of all seven tensors.  The same JSON line carries
  "update_only"    BASELINE config 3: the update-only step over 224 7B-shaped tensors with
                   precomputed gradients (6.476 G counters, 25.9 GB of gradient, a buffer per tensor),
  "small_configs"  BASELINE configs 0-2 (one 288x288 layer; the 15M- and the 110M-shaped steps):
                   fused step on the GPU, the same step on the CPU, and the share of counters that
                   land on a different code,
  "fused_strip"    the same cfg4 step with no weight-sized buffer (update applied from the
                   contraction's accumulators; 24 MB of workspace instead of 180 MB),
  "reference_microbench"  the reference's own published benchmark shape (in 1024, out 256, 8 tokens,
                   C = 3): wall p50 / min / p99 of 50 dispatch+wait runs after 5 warm-ups for the fused
                   update, decode and grad_x, beside the reference's RX 580 figures (context only: the
                   shape is launch-bound),
  "cpu_baseline"   the CPU restatement timed on this box's host cores on a bounded sample,
  "parity"         correctness gates measured in the same run.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg0|cfg1|cfg2|cfg4]
                    [--fused-path workspace|strip] [--batched] [--graph]
                    [--no-update-only] [--no-strip] [--no-small] [--no-by-row-length] [--no-cpu] [--no-clock]

Inputs are synthetic, from the library's counter-based generator (lowbias32 of element index
and stream id -> Box-Muller; mcc_fill_normal_f32 / mcc_fill_counter_state_u8), seed 0:
X ~ N(0,1), dY ~ N(0,0.01), G ~ N(0,0.01), codes uniform on [0,62], scale = sqrt(3/(2 in)),
v = 0, C = 11, lr = 3e-3, lr_scale = 0, rms_beta = 0.9, rms_eps = 1e-3; the update seed of
tensor k in step i is 12345 + k + 1000 i.  The CPU legs run on the very bytes the GPU generated.
Everything is resident in HBM before the timed region.  Kernel durations for the roofline come
from HIP events recorded by the library on the launch stream inside the timed region.
"""
import argparse
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_BF16_TFLOPS = 2500.0  # dense bf16 MFMA
PEAK_MFMA_F32_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
PEAK_CLOCK_MHZ = 2400.0        # the engine clock the published matrix peaks are quoted at
C, LR, LR_SCALE, BETA, EPS = 11, 3e-3, 0.0, 0.9, 1e-3
BYTES_PER_PARAM = 5.5          # 4 (read G) + 0.75 (read state) + 0.75 (write state)
SEED = 0

# HBM-side bytes per launch of the dominant kernels (for the fused step: the step's bytes over its
# seven contraction launches), from `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs of this
# same command (scaled by a plain 1 GiB copy).  They are reported with their source, not
# re-measured in the run.
MEASURED_TRAFFIC = {
    "cfg4/gemm_tn_f32": (1.140e10, "profiles/gemm_tn_f32__cfg4_fused_step.txt"),
    "cfg4/fused_strip": (1.438e10, "profiles/fused_strip__cfg4_fused_step.txt"),
    "cfg3/update_rows": (3.657e10, "profiles/update_rows__cfg3_update_only.txt"),
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
CLOCK_PROBE = True   # --no-clock: counter runs want exactly steps + warmup launches


# ------------------------------------------------------------------------------ inputs
_next_stream = [1]


def _stream_id():
    """A fresh generator stream per array: SEED picks the family, the counter the member."""
    _next_stream[0] += 1
    return (SEED * 0x9E3779B1 + _next_stream[0]) & 0xFFFFFFFF


def normal(ops, shape, sigma):
    import torch
    return ops.fill_normal(torch.empty(shape, dtype=torch.float32, device="cuda"), _stream_id(), sigma)


def make_state(ops, n_out, n_in):
    import torch
    state = ops.fill_counter_state(torch.empty(n_out * n_in // 4 * 3, dtype=torch.uint8, device="cuda"), _stream_id(), 63)
    scale = torch.full((n_out,), math.sqrt(3.0 / (2.0 * n_in)), dtype=torch.float32, device="cuda")
    v = torch.zeros(n_out, dtype=torch.float32, device="cuda")
    return state, scale, v


def cpu_model():
    """Everything /proc/cpuinfo says about the first processor's identity, and how many there are."""
    want = ("model name", "vendor_id", "cpu family", "model", "stepping", "cpu MHz", "cache size")
    got, count = {}, 0
    try:
        for line in open("/proc/cpuinfo"):
            if ":" not in line:
                continue
            key, val = [t.strip() for t in line.split(":", 1)]
            if key == "processor":
                count += 1
            elif key in want and key not in got:
                got[key] = val
    except OSError:
        return "unknown"
    if not got:
        return "unknown"
    return "%s (%s family %s model %s stepping %s, %s MHz, cache %s; %d logical processors visible)" % (
        got.get("model name", "?"), got.get("vendor_id", "?"), got.get("cpu family", "?"), got.get("model", "?"),
        got.get("stepping", "?"), got.get("cpu MHz", "?"), got.get("cache size", "?"), count)


# ------------------------------------------------------------------------------ timing
def query(L, name):
    import ctypes
    ms, n = ctypes.c_double(), ctypes.c_uint64()
    rc = L.mcc_profiler_query(name.encode(), ctypes.byref(ms), ctypes.byref(n))
    assert rc == 0, L.mcc_last_error()
    return ms.value, n.value


def time_steps(step_fn, steps, warmup):
    """`warmup` untimed steps, then exactly `steps` steps between two synchronisations.  Returns
    (mean ms per step by the host clock over the whole region, median of the per-step durations
    taken from events recorded between the steps on the launch stream)."""
    import torch
    for i in range(warmup):
        step_fn(i)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        step_fn(warmup + i)
        marks[i + 1].record()
    torch.cuda.synchronize()
    mean_ms = (time.perf_counter() - t0) * 1e3 / steps
    per_step = [marks[i].elapsed_time(marks[i + 1]) for i in range(steps)]
    return mean_ms, statistics.median(per_step)


def clock_during(ops, fn, est_ms):
    """Shader clock (MHz) while fn() -- one unit of work of about est_ms -- runs back to back.

    A one-wave probe kernel on a side stream counts shader cycles against the constant-rate wall
    clock for 80 % of the stretch the repetitions take (at least 150 ms of work, at most 1.9 s).
    Persistent kernels sized to fill the device run slower beside the probe, so this is done
    outside the timed region."""
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


def traffic_of(key):
    t = MEASURED_TRAFFIC.get(key)
    return (t[0], t[1]) if t else (None, None)


# ------------------------------------------------------------------------------ fused step
class FusedWorkload:
    """The tensors of one fused workload, resident on the GPU."""

    def __init__(self, ops, name, fused_path="workspace", batched=False):
        import torch
        self.ops, self.name, self.fused_path, self.batched = ops, name, fused_path, batched
        self.desc, shapes, self.layers, self.tokens = WORKLOADS[name]
        self.shapes = shapes
        self.tensors = []
        ws_bytes = 0
        xs, dys = {}, {}
        for layer in range(self.layers):
            for (n_out, n_in) in shapes:
                # activations are shared by width to bound memory; every tensor still streams its own
                # rows of them from HBM (at cfg4 each is 537 MB or more, far beyond the caches)
                if n_in not in xs:
                    xs[n_in] = normal(ops, (self.tokens, n_in), 1.0)
                if n_out not in dys:
                    dys[n_out] = normal(ops, (self.tokens, n_out), 0.01)
                self.tensors.append((make_state(ops, n_out, n_in), dys[n_out], xs[n_in], n_out, n_in))
                need = ops.fused_strip_workspace_nbytes(n_in, n_out, self.tokens) if fused_path == "strip" else 0
                ws_bytes = max(ws_bytes, need or ops.fused_workspace_nbytes(n_in, n_out, self.tokens))
        self.params = sum(t[3] * t[4] for t in self.tensors)
        self.flops = sum(2.0 * self.tokens * t[3] * t[4] for t in self.tensors)
        self.fb = None
        if batched:
            # all tensors of the step in one call: grouped contraction, grouped slice sum, batched update
            self.fb = ops.FusedBatch([(st[0], st[1], st[2], dy, x) for (st, dy, x, _, _) in self.tensors], LR,
                                     [12345 + k for k in range(len(self.tensors))])
            ws_bytes = self.fb.workspace_nbytes()
        self.ws_bytes = ws_bytes
        self.ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")

    def step(self, i):
        ops = self.ops
        if self.fb is not None:
            self.fb.set_seeds([12345 + k + 1000 * i for k in range(len(self.tensors))])
            ops.apply_update_fused_batched(self.fb, self.ws, C, LR_SCALE, BETA, EPS)
            return
        for k, ((state, scale, v), dy, x, n_out, n_in) in enumerate(self.tensors):
            ops.apply_update_fused(state, scale, v, dy, x, self.ws, C, LR, LR_SCALE, BETA, EPS, 12345 + k + 1000 * i)

    def snapshot(self):
        """Host copies of every tensor's state, scale and v."""
        return [[t.cpu().numpy().copy() for t in st] for (st, _, _, _, _) in self.tensors]

    def restore(self, snap):
        import torch
        for (st, _, _, _, _), h in zip(self.tensors, snap):
            for t, a in zip(st, h):
                t.copy_(torch.from_numpy(a))


def bench_fused(L, ops, name, steps, warmup, fused_path="workspace", graph=False, batched=False, keep=False):
    import torch
    w = FusedWorkload(ops, name, fused_path, batched)
    for i in range(warmup):
        w.step(i)
    torch.cuda.synchronize()
    graph_ms = None
    if graph:
        # the same step captured once and replayed: what a launch-bound small model gains when the
        # host submits one graph instead of 3 launches per tensor (the seeds are baked in, so this
        # is a launch-cost measurement, not a training loop)
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            w.step(0)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                w.step(0)
        torch.cuda.synchronize()
        graph_ms = time_steps(lambda i: g.replay(), steps, 2)[0]
    L.mcc_profiler_reset()
    L.mcc_profiler_enable(1)
    ms_per_step, median_ms = time_steps(lambda i: w.step(warmup + i), steps, 0)
    gemm_ms, gemm_n = query(L, "gemm_tn_f32")
    upd_ms, upd_n = query(L, "counter_update")
    strip_ms, strip_n = query(L, "fused_strip")
    kernel = "gemm_tn_f32"
    if strip_n and not gemm_n:
        kernel, gemm_ms, gemm_n = "fused_strip", strip_ms, strip_n
    L.mcc_profiler_enable(0)
    L.mcc_profiler_reset()
    if fused_path == "strip":
        ops.fused_check(w.ws, 4, 4, 1)  # raises if a strip step of the run gave up a wait
    # dominant kernel: the contraction.  One launch per tensor; flops per launch differ by
    # tensor, so achieved = (total algorithmic flops of the launches) / (their total duration).
    achieved = w.flops * steps / (gemm_ms * 1e-3) / 1e12
    traffic, traffic_source = traffic_of(name + "/" + kernel)
    out = {
        "value": w.params / (ms_per_step * 1e-3) / 1e9,
        "ms_per_step": ms_per_step, "median_ms_per_step": median_ms,
        "config": {"workload": w.desc, "tensors": len(w.tensors), "params": w.params, "tokens": w.tokens,
                   "C": C, "lr": LR, "lr_scale": LR_SCALE, "rms_beta": BETA, "rms_eps": EPS,
                   "inputs": "counter-based generator (lowbias32 -> Box-Muller), seed %d; activations shared "
                             "by width between the tensors of the workload" % SEED},
        "roofline": {"bound": "mfma", "kernel": kernel, "achieved": achieved,
                     "peak": PEAK_MFMA_F32_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_MFMA_F32_TFLOPS,
                     "traffic": traffic, "traffic_source": traffic_source,
                     "launches": gemm_n, "avg_launch_ms": gemm_ms / max(gemm_n, 1),
                     "algorithmic_flops_per_step": w.flops},
        "kernel_ms_per_step": {kernel: gemm_ms / steps, "counter_update": upd_ms / steps},
        "fused_path": fused_path, "batched_call": batched, "workspace_bytes": w.ws_bytes,
        "graph_replay_ms_per_step": graph_ms,
    }
    # the clock the dominant kernel runs at (the power limit holds it below the 2400 MHz of the
    # published peak): contraction alone on the two-kernel path, the whole step on the strip path
    if kernel == "gemm_tn_f32":
        gbuf = torch.empty(max(t[3] * t[4] for t in w.tensors), device="cuda")
        mats = [(t[1], t[2], gbuf[: t[3] * t[4]].view(t[3], t[4])) for t in w.tensors[:len(w.shapes)]]

        def contractions():
            for dy, x, g in mats:
                ops.matmul_transpose_a(dy, x, g)
        mhz = clock_during(ops, contractions, gemm_ms / steps / w.layers)
        del gbuf, mats
    else:
        mhz = clock_during(ops, lambda: w.step(0), ms_per_step)
    at_clock(out["roofline"], mhz)
    return (out, w) if keep else (out, None)


def bench_layer_products(L, ops, name, steps, warmup):
    """The other two contractions of a counter layer step (forward, input gradient) on the workload's shapes."""
    import torch
    desc, shapes, layers, tokens = WORKLOADS[name]
    out = {}
    xs, dys = {}, {}
    tensors = []
    for (n_out, n_in) in shapes:  # one layer's shapes: the products keep no state between calls
        if n_in not in xs:
            xs[n_in] = normal(ops, (tokens, n_in), 1.0)
        if n_out not in dys:
            dys[n_out] = normal(ops, (tokens, n_out), 0.01)
        tensors.append((make_state(ops, n_out, n_in), n_out, n_in))
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
    p = normal(ops, (n,), 1.0)
    g = normal(ops, (n,), 0.01)
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


# ------------------------------------------------------------------------------ update-only step
def bench_update_only(L, ops, steps, warmup, by_row_length=True):
    import torch
    shapes = layer_shapes(4096, 11008)
    layers = 32
    tensors = []
    for layer in range(layers):
        for (n_out, n_in) in shapes:
            g = normal(ops, (n_out, n_in), 0.01)
            tensors.append((make_state(ops, n_out, n_in), g, n_out, n_in))
    params = sum(t[2] * t[3] for t in tensors)

    batch = ops.UpdateBatch([(st[0], st[1], st[2], g) for (st, g, _, _) in tensors], LR,
                            [12345 + k for k in range(len(tensors))])

    def step(i):
        # one call for the whole list: the optimizer step of the 224 tensors
        batch.set_seeds([12345 + k + 1000 * i for k in range(len(tensors))])
        ops.apply_update_dense_batched(batch, C, LR_SCALE, BETA, EPS)

    # a call lasts under 7 ms and the clock takes a tenth of a second to settle under this kernel's
    # load: at least 30 untimed calls (0.2 s) before the timed ones
    warmup = max(warmup, 30)
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    L.mcc_profiler_reset()
    L.mcc_profiler_enable(1)
    ms_per_step, median_ms = time_steps(lambda i: step(warmup + i), steps, 0)
    upd_ms, upd_n = query(L, "counter_update")
    L.mcc_profiler_enable(0)
    L.mcc_profiler_reset()
    achieved = BYTES_PER_PARAM * params * steps / (upd_ms * 1e-3) / 1e9
    traffic, traffic_source = traffic_of("cfg3/update_rows")
    out = {
        "metric": "counter-synapse updates/s (Gparam/s), update-only",
        "value": params / (ms_per_step * 1e-3) / 1e9, "unit": "Gparam/s",
        "ms_per_step": ms_per_step, "median_ms_per_step": median_ms, "steps": steps, "warmup": warmup,
        "config": {"workload": "cfg3: update-only, 224 7B-shaped tensors (32 layers x 7), "
                               "precomputed fp32 G, distinct buffer per tensor",
                   "tensors": len(tensors), "params": params},
        # one timed region per call = the launches that cover all 224 tensors
        "roofline": {"bound": "hbm", "kernel": "update_rows_kernel", "achieved": achieved,
                     "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS,
                     "traffic": traffic, "traffic_source": traffic_source,
                     "launches": upd_n, "avg_launch_ms": upd_ms / max(upd_n, 1),
                     "algorithmic_bytes_per_param": BYTES_PER_PARAM,
                     "algorithmic_bytes_per_launch": BYTES_PER_PARAM * params},
    }
    # by row length: the 4096-wide rows (one wave per row) and the 11008-wide rows (four waves per row)
    by_width = {}
    for width in ((4096, 11008) if by_row_length else ()):
        sub = [(st[0], st[1], st[2], g) for (st, g, _, n_in) in tensors if n_in == width][:32]
        sub_params = sum(t[3].numel() for t in sub)
        sb = ops.UpdateBatch(sub, LR, list(range(len(sub))))
        for _ in range(2):
            ops.apply_update_dense_batched(sb, C, LR_SCALE, BETA, EPS)
        mean_ms, med_ms = time_steps(lambda i: ops.apply_update_dense_batched(sb, C, LR_SCALE, BETA, EPS), max(steps, 10), 0)
        by_width[str(width)] = {"tensors": len(sub), "ms_per_call": med_ms, "gparam_per_s": sub_params / (med_ms * 1e-3) / 1e9,
                                "hbm_frac": BYTES_PER_PARAM * sub_params / (med_ms * 1e-3) / 1e9 / PEAK_HBM_GBS}
    # row lengths of other model sizes (13B: 5120 / 13824, 70B: 8192 / 28672), outside cfg3: the classes of
    # cooperating waves that rows of 4097..32768 weights take
    for width in ((5120, 8192, 13824, 28672) if by_row_length else ()):
        sub = [(make_state(ops, 4096, width), normal(ops, (4096, width), 0.01)) for _ in range(8)]
        sub = [(st[0], st[1], st[2], g) for (st, g) in sub]
        sub_params = sum(t[3].numel() for t in sub)
        sb = ops.UpdateBatch(sub, LR, list(range(len(sub))))
        for _ in range(30):
            ops.apply_update_dense_batched(sb, C, LR_SCALE, BETA, EPS)
        mean_ms, med_ms = time_steps(lambda i: ops.apply_update_dense_batched(sb, C, LR_SCALE, BETA, EPS), max(steps, 10), 0)
        by_width[str(width)] = {"tensors": len(sub), "shape": [4096, width], "in_cfg3": False, "ms_per_call": med_ms,
                                "gparam_per_s": sub_params / (med_ms * 1e-3) / 1e9,
                                "hbm_frac": BYTES_PER_PARAM * sub_params / (med_ms * 1e-3) / 1e9 / PEAK_HBM_GBS}
        del sub, sb
    out["by_row_length"] = by_width
    out["roofline"]["clock_mhz"] = clock_during(ops, lambda: step(0), ms_per_step)
    return out, tensors


# ------------------------------------------------------------------------------ CPU legs and parity
def flips(oracle, a, b):
    return float((oracle.unpack_codes(a) != oracle.unpack_codes(b)).mean())


def cpu_and_parity_cfg4(ops, w, min_seconds=8.0):
    """One [4096,4096] tensor of the layer at the full 32768 tokens: the CPU restatement's fused update,
    timed, and its result against the GPU's on the same inputs (counter-flip mismatch fraction and
    gradient error at scale)."""
    import numpy as np
    import torch
    from oracle import counter_oracle as oracle
    (state, scale, v), dy, x, n_out, n_in = w.tensors[0]
    tokens = w.tokens
    # a fresh state for this comparison (the timed steps have moved the workload's own)
    st0 = make_state(ops, n_out, n_in)
    h0 = [t.cpu().numpy().copy() for t in st0]
    h_dy, h_x = dy.cpu().numpy(), x.cpu().numpy()
    t0 = time.perf_counter()
    e_state, e_scale, e_v, g_seq = oracle.update_fused(h0[0], h0[1], h0[2], h_dy, h_x, C, LR, LR_SCALE, BETA, EPS, 4242)
    passes, first = 1, time.perf_counter() - t0
    while time.perf_counter() - t0 < min_seconds:
        oracle.update_fused(h0[0], h0[1], h0[2], h_dy, h_x, C, LR, LR_SCALE, BETA, EPS, 4242 + passes)
        passes += 1
    dt = time.perf_counter() - t0
    ws = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, tokens), dtype=torch.uint8, device="cuda")
    ops.apply_update_fused(st0[0], st0[1], st0[2], dy, x, ws, C, LR, LR_SCALE, BETA, EPS, 4242)
    torch.cuda.synchronize()
    got = [t.cpu().numpy() for t in st0]
    g_gpu = ws.view(torch.float32)[: n_out * n_in].view(n_out, n_in).cpu().numpy()
    x_state, x_scale, x_v = oracle.update_dense(h0[0], h0[1], h0[2], g_gpu, C, LR, LR_SCALE, BETA, EPS, 4242)
    cpu = {"value": passes * n_out * n_in / dt / 1e9, "unit": "Gparam/s", "cores": oracle.num_threads(),
           "kind": "port", "seconds": dt, "cpu_model": cpu_model(),
           "sample": "CPU restatement (C, -O3 -mavx2 -ffp-contract=off, OpenMP) fused update of one [%d,%d] tensor "
                     "of the layer at %d tokens (%.0f GFLOP per pass), %d passes; the layer is 12.06 such tensors, "
                     "linear in the weight count" % (n_out, n_in, tokens, 2.0 * tokens * n_out * n_in / 1e9, passes)}
    par = {"workload": "one [%d,%d] tensor of cfg4 at %d tokens, one fused update, GPU vs CPU restatement" % (n_out, n_in, tokens),
           "state_scale_v_bit_exact_given_gpu_gradient": bool(
               np.array_equal(got[0], x_state) and np.array_equal(got[1], x_scale) and np.array_equal(got[2], x_v)),
           "max_abs_dG_over_max_abs_G_vs_sequential_sum": float(np.abs(g_gpu - g_seq).max() / np.abs(g_seq).max()),
           "counter_flip_mismatch_fraction_vs_sequential_sum": flips(oracle, got[0], e_state),
           "v_max_rel_diff_vs_sequential_sum": float(np.abs(got[2] - e_v).max() / np.abs(e_v).max()),
           "counters_changed_fraction": flips(oracle, got[0], h0[0])}
    del ws
    return cpu, par


def small_config(L, ops, name, steps, warmup, with_cpu):
    """One of BASELINE configs 0-2: the fused step per tensor and as one batched call on the GPU, and
    -- from the same initial state and inputs -- the whole step on the CPU restatement."""
    import numpy as np
    import torch
    out = {"workload": WORKLOADS[name][0]}
    for mode in ("per_tensor", "batched"):
        saved = _next_stream[0]
        _next_stream[0] = 1000 * (1 + sorted(WORKLOADS).index(name))  # the same inputs in both modes
        w = FusedWorkload(ops, name, "workspace", batched=(mode == "batched"))
        _next_stream[0] = saved
        if mode == "per_tensor" and with_cpu:
            from oracle import counter_oracle as oracle
            snap = w.snapshot()
            w.step(0)
            torch.cuda.synchronize()
            after = w.snapshot()
            w.restore(snap)
            host = {}

            def h(t):
                if t.data_ptr() not in host:
                    host[t.data_ptr()] = t.cpu().numpy()
                return host[t.data_ptr()]
            n_flip = n_all = 0
            worst_v = 0.0
            t0 = time.perf_counter()
            cpu_s = 0.0
            for k, (st, dy, x, n_out, n_in) in enumerate(w.tensors):
                hd, hx = h(dy), h(x)
                t1 = time.perf_counter()
                e_state, e_scale, e_v, _ = oracle.update_fused(snap[k][0], snap[k][1], snap[k][2], hd, hx, C, LR,
                                                               LR_SCALE, BETA, EPS, 12345 + k)
                cpu_s += time.perf_counter() - t1
                diff = oracle.unpack_codes(after[k][0]) != oracle.unpack_codes(e_state)
                n_flip += int(diff.sum())
                n_all += diff.size
                worst_v = max(worst_v, float(np.abs(after[k][2] - e_v).max() / max(np.abs(e_v).max(), 1e-30)))
            out["cpu"] = {"seconds_per_step": cpu_s, "gparam_per_s": w.params / cpu_s / 1e9, "threads": oracle.num_threads(),
                          "sample": "the whole step, every tensor, once"}
            out["counter_flip_mismatch_fraction_vs_cpu"] = n_flip / n_all
            out["v_max_rel_diff_vs_cpu"] = worst_v
            if name == "cfg0":
                st, dy, x, n_out, n_in = w.tensors[0]
                threads = oracle.num_threads()
                oracle.set_num_threads(1)
                try:
                    t1 = time.perf_counter()
                    oracle.update_fused(snap[0][0], snap[0][1], snap[0][2], h(dy), h(x), C, LR, LR_SCALE, BETA, EPS, 12345)
                    out["cpu_one_thread"] = {"seconds_per_step": time.perf_counter() - t1, "threads": 1}
                finally:
                    oracle.set_num_threads(threads)
        # timed with nothing else on the stream; the kernels' own durations come from a second pass
        # with the library's event bracketing on (at 50 us a step the events are not free)
        k_steps = max(steps, 10)
        mean_ms, med_ms = time_steps(w.step, k_steps, warmup)
        L.mcc_profiler_reset()
        L.mcc_profiler_enable(1)
        time_steps(w.step, k_steps, 0)
        gemm_ms, _ = query(L, "gemm_tn_f32")
        L.mcc_profiler_enable(0)
        L.mcc_profiler_reset()
        tf = w.flops * k_steps / (gemm_ms * 1e-3) / 1e12 if gemm_ms > 0 else None
        out[mode] = {"ms_per_step": mean_ms, "median_ms_per_step": med_ms, "gparam_per_s": w.params / (mean_ms * 1e-3) / 1e9,
                     "contraction_tflops": tf, "contraction_mfma_frac": tf / PEAK_MFMA_F32_TFLOPS if tf else None,
                     "step_mfma_frac": w.flops / (mean_ms * 1e-3) / 1e12 / PEAK_MFMA_F32_TFLOPS}
        out["params"], out["tensors"], out["tokens"] = w.params, len(w.tensors), w.tokens
        if mode == "batched":
            out["update_only"] = small_update_only(ops, w, steps, with_cpu)
        del w
        torch.cuda.empty_cache()
    return out


def small_update_only(ops, w, steps, with_cpu):
    """The update-only step of a small config: a precomputed G ~ N(0, 0.01) per tensor, one batched
    call on the GPU and the same step on the CPU restatement from the same snapshot."""
    import numpy as np
    import torch
    grads = [normal(ops, (n_out, n_in), 0.01) for (_, _, _, n_out, n_in) in w.tensors]
    batch = ops.UpdateBatch([(st[0], st[1], st[2], g) for (st, _, _, _, _), g in zip(w.tensors, grads)], LR,
                            [777 + k for k in range(len(w.tensors))])
    out = {}
    if with_cpu:
        from oracle import counter_oracle as oracle
        snap = w.snapshot()
        ops.apply_update_dense_batched(batch, C, LR_SCALE, BETA, EPS)
        torch.cuda.synchronize()
        after = w.snapshot()
        host_g = [g.cpu().numpy() for g in grads]
        t0 = time.perf_counter()
        exp = [oracle.update_dense(snap[k][0], snap[k][1], snap[k][2], host_g[k], C, LR, LR_SCALE, BETA, EPS, 777 + k)
               for k in range(len(w.tensors))]
        cpu_s = time.perf_counter() - t0
        out["cpu"] = {"seconds_per_step": cpu_s, "gparam_per_s": w.params / cpu_s / 1e9, "threads": oracle.num_threads(),
                      "sample": "the whole step, every tensor, once"}
        out["state_scale_v_bit_exact_vs_cpu"] = bool(all(
            np.array_equal(a, b) for k in range(len(w.tensors)) for a, b in zip(after[k], exp[k])))
    mean_ms, med_ms = time_steps(lambda i: ops.apply_update_dense_batched(batch, C, LR_SCALE, BETA, EPS), max(steps, 10), 2)
    out["gpu"] = {"ms_per_step": mean_ms, "median_ms_per_step": med_ms, "gparam_per_s": w.params / (mean_ms * 1e-3) / 1e9,
                  "hbm_frac": BYTES_PER_PARAM * w.params / (med_ms * 1e-3) / 1e9 / PEAK_HBM_GBS}
    return out


# ------------------------------------------------------------------------------ the reference's own benchmark shape
def reference_microbench(ops):
    """in 1024, out 256, 8 tokens, C = 3: wall time of one dispatch + wait, median of 50 runs after 5
    warm-ups, for the fused update, decode and grad_x -- the shape and method of the reference's
    published figures (benchmarks/bench_vulkan_perf.cpp:8-10,862-911).  Launch-bound: it says what a
    call costs, nothing about the kernels."""
    import torch
    n, n_in, n_out, c = 8, 1024, 256, 3
    state = ops.fill_counter_state(torch.empty(n_out * n_in // 4 * 3, dtype=torch.uint8, device="cuda"), _stream_id(), 15)
    scale = torch.full((n_out,), math.sqrt(3.0 / (2.0 * n_in)), dtype=torch.float32, device="cuda")
    v = torch.zeros(n_out, dtype=torch.float32, device="cuda")
    x = normal(ops, (n, n_in), 1.0)
    dy = normal(ops, (n, n_out), 0.01)
    ws = torch.empty(ops.fused_workspace_nbytes(n_in, n_out, n), dtype=torch.uint8, device="cuda")
    w_out = torch.empty(n_out, n_in, device="cuda")
    gx = torch.empty(n, n_in, device="cuda")
    seed = [0]

    def update():
        seed[0] += 1
        ops.apply_update_fused(state, scale, v, dy, x, ws, c, 3e-3, 0.0, 0.9, 1e-3, 12345 + seed[0])

    ops_by_name = {
        "fused_update": update,
        "decode_weight": lambda: ops.decode_weight(state, scale, c, n_in, n_out, out=w_out),
        "backward_input": lambda: ops.backward_input(dy, state, scale, c, n_in, out=gx),
    }
    published = {"fused_update": 608.6, "decode_weight": 188.3, "backward_input": 501.2}
    out = {"shape": "in1024_out256_N8, C=3", "method": "wall time of dispatch + wait, 50 runs after 5 warm-ups",
           "note": "the reference's figures are from one Radeon RX 580 (Vulkan wall p50, reports/vulkan-perf/*.json:7); "
                   "context only, the shape is launch-bound"}
    for name, fn in ops_by_name.items():
        for _ in range(5):
            fn()
            torch.cuda.synchronize()
        us = []
        for _ in range(50):
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            us.append((time.perf_counter() - t0) * 1e6)
        us.sort()
        out[name] = {"wall_us_p50": statistics.median(us), "wall_us_min": us[0], "wall_us_p99": us[-1],
                     "reference_rx580_wall_us_p50": published[name]}
    return out


def cpu_baseline_dense(tensor, min_seconds=4.0):
    from oracle import counter_oracle as oracle
    (state, scale, v), g, n_out, n_in = tensor
    h = [t.cpu().numpy().copy() for t in (state, scale, v, g)]
    t0 = time.perf_counter()
    reps = 0
    while reps == 0 or time.perf_counter() - t0 < min_seconds:
        oracle.update_dense(h[0], h[1], h[2], h[3], C, LR, LR_SCALE, BETA, EPS, 12345 + reps)
        reps += 1
    dt = time.perf_counter() - t0
    return {"value": reps * n_out * n_in / dt / 1e9, "unit": "Gparam/s", "cores": oracle.num_threads(),
            "kind": "port", "seconds": dt, "cpu_model": cpu_model(),
            "sample": "CPU restatement, update-only on one [%d,%d] tensor of the 224, %d passes" % (n_out, n_in, reps)}


def parity_full_size_fused(ops, tokens=32768):
    """Size-independent properties at the cfg4 shapes: the two fused implementations (two-kernel and
    accumulator-resident) give the same bytes, and sampled rows of the contraction agree with a
    double-precision product."""
    import torch
    out = {"tokens": tokens, "shapes": []}
    for (n_out, n_in) in [(4096, 4096), (11008, 4096), (4096, 11008)]:
        x = normal(ops, (tokens, n_in), 1.0)
        dy = normal(ops, (tokens, n_out), 0.01)
        st0 = make_state(ops, n_out, n_in)
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
    and on the CPU by the restatement from the same snapshot; bytes must be identical."""
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
                         "strip: no weight-sized buffer (update applied from the contraction's accumulators)")
    ap.add_argument("--graph", action="store_true",
                    help="also time the fused step captured into a HIP graph and replayed (reported beside "
                         "the eager figure, which stays the headline)")
    ap.add_argument("--batched", action="store_true",
                    help="fused leg through mcc_compact_counter_apply_update_fused_batched (one call per step)")
    ap.add_argument("--no-update-only", action="store_true", help="skip the cfg3 update-only leg")
    ap.add_argument("--no-strip", action="store_true", help="skip the strip-workspace leg of the cfg4 step")
    ap.add_argument("--no-small", action="store_true", help="skip the cfg0-cfg2 legs")
    ap.add_argument("--no-by-row-length", action="store_true",
                    help="skip the update-only sub-legs by row length (counter runs want the cfg3 launches only)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the legs beside the path (split-bf16 contraction, layer products, side optimizer)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU legs and the parity checks that need them")
    ap.add_argument("--no-clock", action="store_true",
                    help="skip the shader-clock probes (they repeat each kernel outside the timed region)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run one plain 1 GiB device copy (torch copy_), the known-size kernel that "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by")
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

    fused, w = bench_fused(L, ops, args.workload, args.steps, args.warmup, args.fused_path, args.graph, args.batched,
                           keep=True)
    line = {
        "metric": "counter-synapse updates/s (Gparam/s)",
        "value": fused["value"], "unit": "Gparam/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": fused["ms_per_step"], "median_ms_per_step": fused["median_ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": fused["config"], "roofline": fused["roofline"],
        "kernel_ms_per_step": fused["kernel_ms_per_step"],
        "fused_path": fused["fused_path"], "fused_workspace_bytes": fused["workspace_bytes"],
        "graph_replay_ms_per_step": fused["graph_replay_ms_per_step"],
        "device": L.mcc_device_name().decode(),
    }
    if not args.no_cpu:
        if args.workload == "cfg4":
            line["cpu_baseline"], line["parity"] = cpu_and_parity_cfg4(ops, w)
            del w
            torch.cuda.empty_cache()
            line["parity"]["full_size"] = parity_full_size_fused(ops)
        else:
            del w
            small = small_config(L, ops, args.workload, args.steps, args.warmup, True)
            line["cpu_baseline"] = {"value": small["cpu"]["gparam_per_s"], "unit": "Gparam/s", "cores": small["cpu"]["threads"],
                                    "kind": "port", "cpu_model": cpu_model(), "sample": small["cpu"]["sample"]}
            line["parity"] = {"counter_flip_mismatch_fraction_vs_sequential_sum": small["counter_flip_mismatch_fraction_vs_cpu"]}
    w = None
    torch.cuda.empty_cache()
    if args.fused_path == "workspace" and args.workload == "cfg4" and not args.no_strip:
        # the same step with no weight-sized buffer: same workload and seeds, its own roofline
        strip, _ = bench_fused(L, ops, args.workload, args.steps, args.warmup, "strip")
        line["fused_strip"] = {"ms_per_step": strip["ms_per_step"], "median_ms_per_step": strip["median_ms_per_step"],
                               "value": strip["value"], "unit": "Gparam/s", "roofline": strip["roofline"],
                               "workspace_bytes": strip["workspace_bytes"],
                               "fused_check": "ok: no strip step gave up a wait"}
        torch.cuda.empty_cache()
    if not args.no_extras:
        line["reference_microbench"] = reference_microbench(ops)
    if args.fused_path == "workspace" and not args.no_extras:
        # the same step with the optional split-bf16 contraction (six bf16 matrix passes per
        # product, binary32 accuracy), reported beside the headline, which stays on the fp32
        # matrix instruction
        ops.set_contraction_mode(ops.CONTRACTION_BF16X6)
        try:
            alt, _ = bench_fused(L, ops, args.workload, max(3, args.steps // 2), 2, "workspace")
        finally:
            ops.set_contraction_mode(ops.CONTRACTION_FP32)
        tf = alt["roofline"]["achieved"]
        line["fused_split_bf16_contraction"] = {
            "ms_per_step": alt["ms_per_step"], "value": alt["value"], "unit": "Gparam/s",
            "roofline": {"bound": "mfma", "kernel": "gemm_tn_bf16x6", "achieved": tf, "executed": 6.0 * tf,
                         "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s", "frac": 6.0 * tf / PEAK_MFMA_BF16_TFLOPS,
                         "algorithmic_rate_over_fp32_matrix_peak": tf / PEAK_MFMA_F32_TFLOPS}}
        at_clock(line["fused_split_bf16_contraction"]["roofline"], alt["roofline"]["clock_mhz"])
        torch.cuda.empty_cache()
    if not args.no_small and args.workload == "cfg4":
        line["small_configs"] = {name: small_config(L, ops, name, args.steps, args.warmup, not args.no_cpu)
                                 for name in ("cfg0", "cfg1", "cfg2")}
    if not args.no_extras:
        line["side_optimizer"] = bench_side_optimizer(L, ops, max(3, args.steps), 2)
        torch.cuda.empty_cache()
        line["layer_products"] = bench_layer_products(L, ops, args.workload, max(2, args.steps // 2), 1)
        torch.cuda.empty_cache()
    if not args.no_update_only:
        uo, uo_tensors = bench_update_only(L, ops, args.steps, args.warmup, not args.no_by_row_length)
        if not args.no_cpu:
            uo["cpu_baseline"] = cpu_baseline_dense(uo_tensors[0])
            uo["parity_full_size"] = parity_full_size_update_only(ops, uo_tensors)
        del uo_tensors
        line["update_only"] = uo
    print(json.dumps(line))


if __name__ == "__main__":
    main()
