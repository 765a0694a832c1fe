// The weight-gradient contraction c[m,n] = sum_k a[k,m] * b[k,n] on the fp32 matrix cores with
// 256 x 256 tiles: 8 waves (2 down x 4 across, 128 x 64 each), slabs of 16 tokens copied straight
// into one of four LDS buffers (global_load_lds_dwordx4).  Against the 128 x 128 tiles of
// gemm_tn_f32.hip a workgroup copies half as many operand bytes per flop.  Every output element
// still accumulates its tokens in the same order, two at a time, so the result is the same bits.
// Whole tiles and whole slabs only.
//
// Operand reads.  v_mfma_f32_32x32x2_f32 takes one float per lane from each operand; which matrix
// row a lane's float belongs to is the kernel's choice.  Here lane l of the wave's four 32-row
// blocks supplies rows 4 l .. 4 l + 3 (one per block) and columns 2 l, 2 l + 1, so a step's six
// operand floats are one 16-byte and one 8-byte LDS read instead of six 4-byte ones; the
// accumulators then hold a permuted tile, which the stores undo.
//
// Shapes of more than two rounds of tiles that are not whole rounds (11008 x 4096: 688 tiles on
// 256 CUs) run as one launch of one workgroup per CU in which every workgroup gets the same number
// of slabs of the (tile, slab) sequence: a partial tile at the end of its span, whole tiles, and a
// partial tile at the start.  The partial tile at the end is computed first and parked in c; the
// next workgroup, which owns the rest of that tile, takes it up last, loads the parked
// accumulators and carries on with the remaining slabs -- the same additions in the same order
// as an undivided tile, so the same bits, with no last round of idle CUs.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>

#include "gemm_tile.hpp"
#include "gemm_wide_tile.hpp"
#include "launch.hpp"

namespace mcc {
namespace {

// acc[i][j][r] is row wm0 + 4 (8 (r/4) + 4 half + r%4) + i, column wn0 + 2 l32 + j of the tile.
__device__ __forceinline__ void wide_store(float* __restrict__ c, int N, int m0, int n0, const WideAcc& acc,
                                           const WideLane& t) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = m0 + t.wm0 + 4 * (8 * (r / 4) + 4 * t.half + (r % 4)) + i;
            *reinterpret_cast<float2*>(&c[(size_t)row * N + n0 + t.wn0 + 2 * t.l32]) =
                make_float2(acc[i][0][r], acc[i][1][r]);
        }
}

MCC_WIDE_KERNEL void gemm_tn_wide_kernel(const float* __restrict__ a,
                                                                       const float* __restrict__ b,
                                                                       float* __restrict__ c, int K, int M, int N,
                                                                       int chunk) {
    __shared__ __attribute__((aligned(1024))) float lds[kWideBuffers * kWideSlabFloats];
    const WideLane t = wide_lane();
    const TileXY tile = xcd_tile(gridDim.x, gridDim.y, 4);
    const int m0 = tile.y * kWide, n0 = tile.x * kWide;
    const int k_begin = blockIdx.z * chunk;
    const int k_len = K - k_begin < chunk ? K - k_begin : chunk;
    WideAcc acc;
    wide_zero(acc);
    wide_accumulate(a + (size_t)k_begin * M + m0, b + (size_t)k_begin * N + n0, M, N, k_len, acc, lds, t);
    wide_store(c + (size_t)blockIdx.z * M * N, N, m0, n0, acc, t);
}

// ---------------------------------------------------------------------------- equal spans
// Hand-off word of workgroup j's parked tile: 0 nothing yet, kWriting the owner is storing it,
// kParked it is complete, kAbandoned the taker has given up waiting and computes the whole tile
// itself (the owner then skips its stores).  Every transition is a compare-and-swap from 0, so
// exactly one side wins; the parked accumulators cross the per-XCD L2 caches as device-scope atomic
// accesses, ordered by completion (the owner's stores are acknowledged before it raises the word,
// the taker loads after it has seen it).
constexpr int kWriting = 3, kParked = 1, kAbandoned = 2;

__device__ __forceinline__ int word_load(const int* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool word_claim(int* p, int desired) {
    int expected = 0;
    return __hip_atomic_compare_exchange_strong(p, &expected, desired, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
}

// The 65536 accumulators of a tile in the order (register, thread): element q * 512 + tid of the
// tile read row by row, so a wave moves whole 256-byte pieces.
__device__ __forceinline__ void wide_park(float* __restrict__ c, int N, int m0, int n0, const WideAcc& acc, int tid) {
#pragma unroll
    for (int q = 0; q < 128; ++q) {
        const int idx = q * kWideThreads + tid;
        __hip_atomic_store(&c[(size_t)(m0 + (idx >> 8)) * N + n0 + (idx & 255)], acc[q / 32][(q / 16) % 2][q % 16],
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
__device__ __forceinline__ void wide_take(const float* __restrict__ c, int N, int m0, int n0, WideAcc& acc, int tid) {
#pragma unroll
    for (int q = 0; q < 128; ++q) {
        const int idx = q * kWideThreads + tid;
        acc[q / 32][(q / 16) % 2][q % 16] = __hip_atomic_load(&c[(size_t)(m0 + (idx >> 8)) * N + n0 + (idx & 255)],
                                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Tiles in bands of four tile rows, column by column inside a band, so that workgroups with
// neighbouring spans work on tiles that share operand panels.
__device__ __forceinline__ TileXY band_tile(int t, int tiles_x, int tiles_y) {
    const int band_tiles = 4 * tiles_x;
    const int band = t / band_tiles, within = t - band * band_tiles;
    const int left = tiles_y - 4 * band;
    const int rows = left < 4 ? left : 4;
    TileXY r;
    r.x = within / rows;
    r.y = 4 * band + within % rows;
    return r;
}

MCC_WIDE_KERNEL void gemm_tn_wide_spans_kernel(
    const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ c, int K, int M, int N, int tiles_x,
    int tiles_y, int* words, unsigned spin_limit, int start_first, int classes, int order) {
    // One LDS object, read and written as floats only: a second LDS variable gives every LDS access
    // alias-scope metadata, and an access of another type loses the type-based one; with either
    // the compiler waits for the slab copies in flight (s_waitcnt vmcnt(0)) before the operand
    // reads of the slab at hand, which serialises copy and arithmetic.
    __shared__ __attribute__((aligned(1024))) float lds[kWideBuffers * kWideSlabFloats + 64];
    float& verdict = lds[kWideBuffers * kWideSlabFloats];
    const WideLane t = wide_lane();
    // Workgroups w, w + 8, ... share an XCD and its L2, which holds a few slabs of the panels in
    // use: two workgroups share a panel's fetches only while they are at the same token.  Spans
    // j, j + classes, j + 2 classes, ... begin whole tiles at the same moment (their first pieces
    // are equally long), so an XCD gets all spans of classes / 8 such families and the tile order
    // puts their tiles on one line of the tile grid (classes == 0: no such structure, neighbouring
    // spans per XCD).
    const int P = gridDim.x;
    int j = (int)blockIdx.x;
    if (classes > 0) {
        const int per_xcd = classes >> 3, local = (int)(blockIdx.x >> 3);
        j = (local / per_xcd) * classes + (int)(blockIdx.x & 7u) * per_xcd + local % per_xcd;
    } else if ((P & 7) == 0) {
        j = (int)(blockIdx.x & 7u) * (P >> 3) + (int)(blockIdx.x >> 3);
    }
    const long spt = K / kBK;  // slabs per tile
    const long total = (long)tiles_x * tiles_y * spt;
    const long base = total / P, rem = total % P;
    const long begin = j * base + (j < rem ? j : rem);
    const long end = begin + base + (j < rem ? 1 : 0);
    const int first_tile = (int)(begin / spt), last_tile = (int)((end - 1) / spt);
    const int s0 = (int)(begin - first_tile * spt);     // slabs of first_tile that belong to the span before
    const int e1 = (int)(end - (long)last_tile * spt);  // slabs of last_tile inside this span
    const bool has_start = s0 > 0, has_end = e1 < spt;  // the span is longer than two tiles: never the same tile
    WideAcc acc;

    auto tile_origin = [&](int tile, int& m0, int& n0) {
        TileXY xy;
        if (order == 1) { xy.y = tile % tiles_y; xy.x = tile / tiles_y; }
        else if (order == 2) { xy.x = tile % tiles_x; xy.y = tile / tiles_x; }
        else xy = band_tile(tile, tiles_x, tiles_y);
        m0 = xy.y * kWide;
        n0 = xy.x * kWide;
    };
    // the partial tile at the end of the span: slabs [0, e1), parked in c for workgroup j + 1
    auto run_end = [&]() {
        int m0, n0;
        tile_origin(last_tile, m0, n0);
        wide_zero(acc);
        __syncthreads();
        wide_accumulate(a + m0, b + n0, M, N, e1 * kBK, acc, lds, t);
        if (t.tid == 0) verdict = word_claim(&words[j], kWriting) ? 1.0f : 0.0f;
        __syncthreads();
        if (verdict != 0.0f) {  // else the taker has given up and computes the tile alone
            wide_park(c, N, m0, n0, acc, t.tid);
            __builtin_amdgcn_s_waitcnt(0);  // stores acknowledged
            __syncthreads();
            if (t.tid == 0) __hip_atomic_store(&words[j], kParked, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
    };
    auto run_whole = [&]() {
        for (int tile = first_tile + (has_start ? 1 : 0); tile <= last_tile - (has_end ? 1 : 0); ++tile) {
            int m0, n0;
            tile_origin(tile, m0, n0);
            wide_zero(acc);
            __syncthreads();
            wide_accumulate(a + m0, b + n0, M, N, K, acc, lds, t);
            wide_store(c, N, m0, n0, acc, t);
        }
    };
    // the partial tile at the start: slabs [s0, spt) on top of what workgroup j - 1 parked
    auto run_start = [&]() {
        int m0, n0;
        tile_origin(first_tile, m0, n0);
        if (t.tid == 0) {
            int* word = &words[j - 1];
            int got = 0;
            unsigned polls = 0;
            for (;;) {
                const int seen = word_load(word);
                if (seen == kParked) { got = 1; break; }
                // kWriting: the owner is running and about to finish, whatever the budget says
                if (seen == 0 && polls >= spin_limit && word_claim(word, kAbandoned)) break;
                __builtin_amdgcn_s_sleep(32);
                ++polls;
            }
            verdict = got ? 1.0f : 0.0f;
        }
        __syncthreads();
        const bool parked = verdict != 0.0f;
        if (parked) wide_take(c, N, m0, n0, acc, t.tid); else wide_zero(acc);
        const int from = parked ? s0 : 0;
        __syncthreads();
        wide_accumulate(a + (size_t)from * kBK * M + m0, b + (size_t)from * kBK * N + n0, M, N, (int)(spt - from) * kBK,
                        acc, lds, t);
        wide_store(c, N, m0, n0, acc, t);
    };
    if (!start_first) {
        if (has_end) run_end();
        run_whole();
        if (has_start) run_start();
    } else {  // test order: every taker arrives before its owner
        if (has_start) run_start();
        run_whole();
        if (has_end) run_end();
    }
}

// ---------------------------------------------------------------------------- equal spans over a list
// The same for a list of contractions (the layers of a model whose sides are multiples of 256):
// the (tile, slab) sequences of all jobs are laid end to end and every workgroup gets an equal
// span of the whole, so a list of mid-sized layers -- none of which fills the device with 256 x 256
// tiles on its own -- runs as one launch with no idle round, no token chunks and no slices to add
// up.  Every output element is still the sum of its tokens in token order.
struct SpanJob {
    const float* a;  // [K, M]
    const float* b;  // [K, N]
    float* c;        // [M, N]
    int K, M, N;
    int slab_begin;  // first slab of this job in the list's sequence
};
constexpr int kMaxSpanJobs = 96;
struct SpanGroupArgs {
    SpanJob job[kMaxSpanJobs];
    int n_jobs;
    int total_slabs;
    int* words;
    unsigned spin_limit;
    int start_first;
};
static_assert(sizeof(SpanGroupArgs) <= 4096, "kernel arguments are limited to 4 KiB");

// One piece of a tile: slabs [from, to) of tile `tile` of job `ji`.
struct SpanPiece {
    int ji, tile, from, to, spt;
};

MCC_WIDE_KERNEL void gemm_tn_wide_spans_group_kernel(SpanGroupArgs g) {
    __shared__ __attribute__((aligned(1024))) float lds[kWideBuffers * kWideSlabFloats + 64];
    float& verdict = lds[kWideBuffers * kWideSlabFloats];
    const WideLane t = wide_lane();
    const int P = gridDim.x;
    // neighbouring spans on one XCD: they work on neighbouring tiles, which share operand panels
    int j = (int)blockIdx.x;
    if ((P & 7) == 0) j = (int)(blockIdx.x & 7u) * (P >> 3) + (int)(blockIdx.x >> 3);
    const long total = g.total_slabs;
    const long base = total / P, rem = total % P;
    const int begin = (int)(j * base + (j < rem ? j : rem));
    const int end = (int)(begin + base + (j < rem ? 1 : 0));

    // the piece that holds slab `slab` (scalar: kernel arguments and blockIdx only)
    auto piece_at = [&](int slab, int ji) {
        while (ji + 1 < g.n_jobs && g.job[ji + 1].slab_begin <= slab) ++ji;
        SpanPiece p;
        p.ji = ji;
        p.spt = g.job[ji].K / kBK;
        const int local = slab - g.job[ji].slab_begin;
        p.tile = local / p.spt;
        p.from = local - p.tile * p.spt;
        p.to = p.spt;
        return p;
    };
    auto origin = [&](const SpanPiece& p, const SpanJob& job, int& m0, int& n0) {
        const TileXY xy = band_tile(p.tile, job.N / kWide, job.M / kWide);
        m0 = xy.y * kWide;
        n0 = xy.x * kWide;
    };
    SpanPiece first = piece_at(begin, 0);
    SpanPiece last = piece_at(end - 1, first.ji);
    last.to = end - g.job[last.ji].slab_begin - last.tile * last.spt;  // slabs of the last tile inside the span
    last.from = 0;
    // the host makes every span longer than two tiles, so the two are never the same tile
    const bool has_start = first.from > 0, has_end = last.to < last.spt;
    WideAcc acc;

    // the partial tile at the end of the span: slabs [0, to), parked in c for workgroup j + 1
    auto run_end = [&]() {
        const SpanJob job = g.job[last.ji];
        int m0, n0;
        origin(last, job, m0, n0);
        wide_zero(acc);
        __syncthreads();
        wide_accumulate(job.a + m0, job.b + n0, job.M, job.N, last.to * kBK, acc, lds, t);
        if (t.tid == 0) verdict = word_claim(&g.words[j], kWriting) ? 1.0f : 0.0f;
        __syncthreads();
        if (verdict != 0.0f) {  // else the taker has given up and computes the tile alone
            wide_park(job.c, job.N, m0, n0, acc, t.tid);
            __builtin_amdgcn_s_waitcnt(0);  // stores acknowledged
            __syncthreads();
            if (t.tid == 0) __hip_atomic_store(&g.words[j], kParked, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
    };
    auto run_whole = [&]() {
        // from the tile after a partial first one up to the tile before a partial last one
        int slab = begin + (has_start ? first.spt - first.from : 0);
        const int stop = has_end ? end - last.to : end;
        int ji = first.ji;
        while (slab < stop) {
            const SpanPiece p = piece_at(slab, ji);
            ji = p.ji;
            const SpanJob job = g.job[ji];
            int m0, n0;
            origin(p, job, m0, n0);
            wide_zero(acc);
            __syncthreads();
            wide_accumulate(job.a + m0, job.b + n0, job.M, job.N, job.K, acc, lds, t);
            wide_store(job.c, job.N, m0, n0, acc, t);
            slab += p.spt;
        }
    };
    // the partial tile at the start: slabs [from, spt) on top of what workgroup j - 1 parked
    auto run_start = [&]() {
        const SpanJob job = g.job[first.ji];
        int m0, n0;
        origin(first, job, m0, n0);
        if (t.tid == 0) {
            int* word = &g.words[j - 1];
            int got = 0;
            unsigned polls = 0;
            for (;;) {
                const int seen = word_load(word);
                if (seen == kParked) { got = 1; break; }
                // kWriting: the owner is running and about to finish, whatever the budget says
                if (seen == 0 && polls >= g.spin_limit && word_claim(word, kAbandoned)) break;
                __builtin_amdgcn_s_sleep(32);
                ++polls;
            }
            verdict = got ? 1.0f : 0.0f;
        }
        __syncthreads();
        const bool parked = verdict != 0.0f;
        if (parked) wide_take(job.c, job.N, m0, n0, acc, t.tid); else wide_zero(acc);
        const int from = parked ? first.from : 0;
        __syncthreads();
        wide_accumulate(job.a + (size_t)from * kBK * job.M + m0, job.b + (size_t)from * kBK * job.N + n0, job.M, job.N,
                        (first.spt - from) * kBK, acc, lds, t);
        wide_store(job.c, job.N, m0, n0, acc, t);
    };
    if (!g.start_first) {
        if (has_end) run_end();
        run_whole();
        if (has_start) run_start();
    } else {  // test order: every taker arrives before its owner
        if (has_start) run_start();
        run_whole();
        if (has_end) run_end();
    }
}

__global__ void clear_words_kernel(int* words, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) words[i] = 0;
}

// about 0.9 us per poll: 4 ms before a taker computes a tile alone
constexpr unsigned kDefaultSpanPolls = 4096;
// test aids of the calling thread (other threads keep the defaults)
thread_local unsigned g_span_polls = kDefaultSpanPolls;
thread_local int g_span_start_first = 0;
thread_local int g_span_order_override = -1;

int device_cus() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    int cus = cached[dev].load();
    if (cus == 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cached[dev].store(cus);
    }
    return cus;
}

}  // namespace

bool gemm_tn_wide_supports(const float* a, const float* b, int k, int m, int n, int chunk) {
    return m % kWide == 0 && n % kWide == 0 && k % kBK == 0 && chunk % kBK == 0 &&
           (reinterpret_cast<uintptr_t>(a) & 15u) == 0 && (reinterpret_cast<uintptr_t>(b) & 15u) == 0;
}

// tiles_x x tiles_y tiles starting at a, b, out; m and n are the row lengths of a / b and out
hipError_t launch_gemm_tn_wide(hipStream_t stream, const float* a, const float* b, float* out, int k, int m, int n,
                               int tiles_x, int tiles_y, int chunk, int splits) {
    const dim3 grid(tiles_x, tiles_y, splits);
    hipLaunchKernelGGL(gemm_tn_wide_kernel, grid, dim3(kWideThreads), 0, stream, a, b, out, k, m, n, chunk);
    return hipGetLastError();
}

bool gemm_tn_wide_spans_apply(int k, int m, int n) {
    if (m % kWide || n % kWide || k % kBK) return false;
    const long tiles = (long)(m / kWide) * (n / kWide);
    return tiles > 2 * kWideSpanWorkgroups && tiles % kWideSpanWorkgroups != 0;
}

hipError_t launch_gemm_tn_wide_spans(hipStream_t stream, const float* a, const float* b, float* out, int k, int m,
                                     int n, int* words) {
    // one workgroup per CU; on a device of another size the spans are simply longer or shorter
    int wgs = device_cus();
    if (wgs <= 0 || wgs > kWideSpanWorkgroups) wgs = kWideSpanWorkgroups;
    const long tiles = (long)(m / kWide) * (n / kWide);
    if (tiles < 2L * wgs) return hipErrorInvalidValue;
    hipLaunchKernelGGL(clear_words_kernel, dim3(1), dim3(kWideSpanWorkgroups), 0, stream, words, kWideSpanWorkgroups);
    // spans j and j + g start at the same slab of their tiles when g spans are a whole number of
    // tiles; with the tiles of such a family one line of the grid apart they share a panel
    const int tiles_x = n / kWide, tiles_y = m / kWide;
    const long spt = k / kBK, total = tiles * spt;
    int classes = 0, order = 0;
    if (total % wgs == 0 && wgs % 8 == 0) {
        const long base = total / wgs;
        long g = 1;
        while (g <= wgs && (base * g) % spt) ++g;
        const long step = base * g / spt;  // tiles between spans of a family
        if (g <= wgs && g % 8 == 0 && wgs % g == 0 && (step == tiles_y || step == tiles_x)) {
            classes = (int)g;
            order = step == tiles_y ? 1 : 2;
        }
    }
    if (g_span_order_override >= 0) { classes = 0; order = 0; }
    hipLaunchKernelGGL(gemm_tn_wide_spans_kernel, dim3(wgs), dim3(kWideThreads), 0, stream, a, b, out, k, m, n,
                       tiles_x, tiles_y, words, g_span_polls, g_span_start_first, classes, order);
    return hipGetLastError();
}

// Whether a list of contractions runs as one launch of equal spans: every job on whole 256 x 256
// tiles and whole slabs, at least two tiles per workgroup over the list, and -- so that a span never
// begins and ends inside one tile -- spans of at least two tiles of the job with the most tokens.
// A function of the shapes alone.
bool gemm_tn_spans_group_applies(const GemmTnJob* jobs, size_t n) {
    if (n == 0 || n > (size_t)kMaxSpanJobs) return false;
    long total = 0, tiles = 0, max_spt = 0;
    for (size_t i = 0; i < n; ++i) {
        const GemmTnJob& jb = jobs[i];
        if (jb.m % kWide || jb.n % kWide || jb.k % kBK || jb.k <= 0) return false;
        const long t = (long)(jb.m / kWide) * (jb.n / kWide), spt = jb.k / kBK;
        tiles += t;
        total += t * spt;
        if (spt > max_spt) max_spt = spt;
        if (total >= (1L << 31)) return false;
    }
    return tiles >= 2L * kWideSpanWorkgroups && total / kWideSpanWorkgroups >= 2 * max_spt;
}

hipError_t launch_gemm_tn_wide_spans_group(hipStream_t stream, const GemmTnJob* jobs, size_t n, int* words) {
    if (!gemm_tn_spans_group_applies(jobs, n)) return hipErrorInvalidValue;
    int wgs = device_cus();
    if (wgs <= 0 || wgs > kWideSpanWorkgroups) wgs = kWideSpanWorkgroups;
    SpanGroupArgs g;
    long total = 0;
    for (size_t i = 0; i < n; ++i) {
        const GemmTnJob& jb = jobs[i];
        if ((reinterpret_cast<uintptr_t>(jb.a) & 15u) || (reinterpret_cast<uintptr_t>(jb.b) & 15u) ||
            (reinterpret_cast<uintptr_t>(jb.out) & 15u))
            return hipErrorInvalidValue;
        g.job[i] = {jb.a, jb.b, jb.out, jb.k, jb.m, jb.n, (int)total};
        total += (long)(jb.m / kWide) * (jb.n / kWide) * (jb.k / kBK);
    }
    g.n_jobs = (int)n;
    g.total_slabs = (int)total;
    g.words = words;
    g.spin_limit = g_span_polls;
    g.start_first = g_span_start_first;
    hipLaunchKernelGGL(clear_words_kernel, dim3(1), dim3(kWideSpanWorkgroups), 0, stream, words, kWideSpanWorkgroups);
    hipLaunchKernelGGL(gemm_tn_wide_spans_group_kernel, dim3(wgs), dim3(kWideThreads), 0, stream, g);
    return hipGetLastError();
}

void set_gemm_tn_wide_spans_test_mode(unsigned polls, int start_first) {
    g_span_polls = polls == 0xffffffffu ? kDefaultSpanPolls : polls;
    g_span_start_first = start_first & 1;
    g_span_order_override = (start_first & 2) ? 0 : -1;
}

}  // namespace mcc
