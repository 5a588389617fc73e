// Token selection from float32 logits for gfx950: argmax, and the sampling pipeline
// repetition penalty -> temperature -> top-k -> softmax -> top-p -> renormalise -> inverse CDF
// (order of src/sampler/configurable_sampler.cpp:93-120 of the reference).
//
// Thresholds are exact selections, not the 16-step bisections of
// src/op/kernels/cuda/sampling_kernel.cu:202-296: a radix descent over the order-preserving
// integer image of a float finds the k-th largest logit (counts) and the smallest logit whose
// upper set still holds the mass top_p (sums).  Equal logits at a
// threshold are kept together.  The draw walks the kept tokens in vocabulary order and takes
// the first whose cumulative mass reaches u * total (src/op/kernels/cuda/sampling_kernel.cu:330-398);
// u in (0, 1] comes from the host, which derives it from (seed, tokens the request has generated so far).
#include "common.h"

#include <type_traits>

__device__ __forceinline__ uint32_t order_key(float f) {
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// argmax with the lowest index among equal values (src/op/kernels/cuda/argmax_kernel.cu:27).
__device__ __forceinline__ void better(float& v, int& i, float v2, int i2) {
    if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
}

// Stage one: ARGMAX_PARTS workgroups share a row, each finds the best of its slice (float4 loads
// when the row allows).  Stage two: one wavefront per row picks among the parts.
#define ARGMAX_PARTS 32
#define ARGMAX_THREADS 256

__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_part_kernel(const float* __restrict__ logits, float* __restrict__ part_val,
                                                                    int32_t* __restrict__ part_idx, int V) {
    __shared__ float s_val[ARGMAX_THREADS / WAVE];
    __shared__ int s_idx[ARGMAX_THREADS / WAVE];
    const int r = blockIdx.x, part = blockIdx.y;
    const float* row = logits + static_cast<size_t>(r) * V;
    const int per = ((V + ARGMAX_PARTS - 1) / ARGMAX_PARTS + 3) & ~3;      // a multiple of 4 elements
    const int lo = part * per, hi = min(V, lo + per);
    float best = -INFINITY;
    int idx = 0x7fffffff;
    if ((V & 3) == 0) {         // rows are 16-byte aligned: four logits a load
        for (int i = lo + threadIdx.x * 4; i < hi; i += ARGMAX_THREADS * 4) {
            const float4 v = *reinterpret_cast<const float4*>(row + i);
            better(best, idx, v.x, i);
            better(best, idx, v.y, i + 1);
            better(best, idx, v.z, i + 2);
            better(best, idx, v.w, i + 3);
        }
    } else {
        for (int i = lo + threadIdx.x; i < hi; i += ARGMAX_THREADS) better(best, idx, row[i], i);
    }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
        float v2 = __shfl_xor(best, off, WAVE);
        int i2 = __shfl_xor(idx, off, WAVE);
        better(best, idx, v2, i2);
    }
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    if (lane == 0) { s_val[wave] = best; s_idx[wave] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < ARGMAX_THREADS / WAVE; ++w) better(best, idx, s_val[w], s_idx[w]);
        part_val[r * ARGMAX_PARTS + part] = best;
        part_idx[r * ARGMAX_PARTS + part] = idx;
    }
}

__global__ void argmax_final_kernel(const float* __restrict__ part_val, const int32_t* __restrict__ part_idx,
                                    int32_t* __restrict__ out) {
    const int r = blockIdx.x;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    if (threadIdx.x < ARGMAX_PARTS) {
        best = part_val[r * ARGMAX_PARTS + threadIdx.x];
        idx = part_idx[r * ARGMAX_PARTS + threadIdx.x];
    }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
        float v2 = __shfl_xor(best, off, WAVE);
        int i2 = __shfl_xor(idx, off, WAVE);
        better(best, idx, v2, i2);
    }
    if (threadIdx.x == 0) out[r] = idx == 0x7fffffff ? 0 : idx;    // a row of NaN: the first token
}

// ---------------------------------------------------------------------------------------------
// The sampling pipeline.  A row of a large vocabulary is far too long for one workgroup (one
// compute unit draws a few per cent of the chip's bandwidth), so PARTS workgroups share a row, each
// with a contiguous slice, and the pipeline is a chain of short launches; whatever one launch
// decides for a row (a level of a radix descent, the mass of the kept tokens) every workgroup of
// the next launch works out again from the per-part results, in the same fixed order, so that all
// agree and no launch waits for another inside itself.  Per-part histograms and decisions of
// successive levels alternate between two buffers: a workgroup may still be reading the last
// level's while another writes the next one's.
//
// scratch, all sized by the host: work float [R, V]; part_max float / part_arg int32 [R, P];
// part_z, part_mass float / part_last int32 [R, P]; hist uint32 [2, R, P, 256] (counts, or the
// bits of float sums); state uint32 [R, 16]: words 2*l, 2*l + 1 = (prefix, remaining) after level
// l of the top-k descent (l = 0..3), words 8 + 2*l likewise for top-p (remaining as float bits).
struct SampleArgs {
    const float* logits; float* work;
    const float* temperature; const int32_t* top_k; const float* top_p; const float* penalty;
    int32_t* pen_ids; const int32_t* pen_off; int32_t* pen_count; const float* uniform; int32_t* out;
    float* part_max; int32_t* part_arg; float* part_z; float* part_mass; int32_t* part_last;
    uint32_t* hist; uint32_t* state;
    int R, V, P;
};

#define SP_THREADS 256
#define SP_WAVES (SP_THREADS / WAVE)

// Sweeps over a slice of a row.  A load that waits for the one before it costs a round trip to memory
// each, and a slice of some four thousand elements is sixteen of them for every thread: both sweeps ask
// for eight elements before the first is used (an element past the end is read from the last one and
// not used: no load is under a branch).
//   sweep_strided: thread t takes lo + t, lo + t + SP_THREADS, ...
//   sweep_run:     a thread's own run i0 .. i1 - 1, in order
#define SP_AHEAD 8
template <typename F>
__device__ __forceinline__ void sweep_strided(const float* __restrict__ p, int lo, int hi, int tid, F&& f) {
    for (int base = lo + tid; base < hi; base += SP_AHEAD * SP_THREADS) {
        float v[SP_AHEAD];
#pragma unroll
        for (int k = 0; k < SP_AHEAD; ++k) v[k] = p[min(base + k * SP_THREADS, hi - 1)];
#pragma unroll
        for (int k = 0; k < SP_AHEAD; ++k) {
            const int i = base + k * SP_THREADS;
            if (i < hi) f(v[k], i);
        }
    }
}
template <typename F>
__device__ __forceinline__ void sweep_run(const float* __restrict__ p, int i0, int i1, F&& f) {
    for (int base = i0; base < i1; base += SP_AHEAD) {
        float v[SP_AHEAD];
#pragma unroll
        for (int k = 0; k < SP_AHEAD; ++k) v[k] = p[min(base + k, i1 - 1)];
#pragma unroll
        for (int k = 0; k < SP_AHEAD; ++k)
            if (base + k < i1) f(v[k], base + k);
    }
}

struct Slice { int lo, hi; };
__device__ __forceinline__ Slice slice_of(int part, int V, int P) {
    const int per = ((V + P - 1) / P + 3) & ~3;
    const int lo = min(V, part * per);
    return Slice{lo, min(V, lo + per)};
}
__device__ __forceinline__ bool row_samples(const SampleArgs& a, int r) { return a.temperature[r] > 0.f; }
__device__ __forceinline__ bool row_top_k(const SampleArgs& a, int r) { return row_samples(a, r) && a.top_k[r] > 0 && a.top_k[r] < a.V; }
__device__ __forceinline__ bool row_top_p(const SampleArgs& a, int r) { return row_samples(a, r) && a.top_p[r] > 0.f && a.top_p[r] < 1.0f; }
__device__ __forceinline__ uint32_t* hist_of(const SampleArgs& a, int which, int r, int part) {
    return a.hist + ((static_cast<size_t>(which) * a.R + r) * a.P + part) * 256;
}

// One level of a radix descent, decided by every workgroup alike: the bins of all parts are summed in
// the order of the parts, then the highest bin b is found whose bins from b upwards hold at least
// `remaining`.  Returns b; `remaining` loses what the bins above b hold.  CT: uint32_t (counts) or float (sums).
template <typename CT>
__device__ int decide_level(const uint32_t* __restrict__ hist_row, int P, CT& remaining, CT* s_scan, int* s_bin) {
    const int tid = threadIdx.x;                      // SP_THREADS == 256: thread t owns bin 255 - t
    const int bin = 255 - tid;
    CT mine = 0;
    for (int p0 = 0; p0 < P; p0 += SP_AHEAD) {          // eight parts' bins asked for at a time, added in the order of the parts
        uint32_t raw[SP_AHEAD];
#pragma unroll
        for (int k = 0; k < SP_AHEAD; ++k) raw[k] = hist_row[static_cast<size_t>(min(p0 + k, P - 1)) * 256 + bin];
#pragma unroll
        for (int k = 0; k < SP_AHEAD; ++k) {
            if (p0 + k < P) {
                if constexpr (std::is_same<CT, float>::value) mine += __uint_as_float(raw[k]);
                else mine += raw[k];
            }
        }
    }
    // inclusive scan over the threads = sum of the bins from `bin` upwards
    CT incl = mine;
#pragma unroll
    for (int off = 1; off < WAVE; off <<= 1) {
        const CT o = __shfl_up(incl, off, WAVE);
        if ((tid % WAVE) >= off) incl += o;
    }
    const int wave = tid / WAVE, lane = tid % WAVE;
    __syncthreads();
    if (lane == WAVE - 1) s_scan[wave] = incl;
    if (tid == 0) *s_bin = 0;
    __syncthreads();
    CT before = 0;
    for (int w = 0; w < wave; ++w) before += s_scan[w];
    incl += before;
    if (incl >= remaining) atomicMax(s_bin, bin);
    __syncthreads();
    const int b = *s_bin;
    // what the bins above b hold: the exclusive value of bin b's thread
    __syncthreads();
    if (bin == b) s_scan[SP_WAVES] = incl - mine;
    __syncthreads();
    remaining -= s_scan[SP_WAVES];
    return b;
}

// Launch 1: penalty and temperature (src/op/kernels/cuda/sampling_kernel.cu:38-88), the slice's
// largest value, and the counts of the first radix level for top-k.  `plain`: no row of the batch asks for
// top-k or top-p, so every token is kept; the slice's sum of exp(w - its own maximum) is taken here as well,
// and the draw, which scales it to the row's maximum, is the only other launch.
__global__ __launch_bounds__(SP_THREADS) void sample_prepare_kernel(SampleArgs a, int plain) {
    __shared__ float s_val[SP_WAVES];
    __shared__ int s_idx[SP_WAVES];
    __shared__ uint32_t s_hist[256];
    __shared__ float s_red[16];
    const int r = blockIdx.x, part = blockIdx.y, tid = threadIdx.x;
    const Slice sl = slice_of(part, a.V, a.P);
    const float* lrow = a.logits + static_cast<size_t>(r) * a.V;
    float* w = a.work + static_cast<size_t>(r) * a.V;
    const float T = a.temperature[r];
    const float inv_t = (T <= 0.f || T == 1.0f) ? 1.0f : 1.0f / T;
    const float pen = a.penalty[r];
    const bool counts = row_top_k(a, r);
    float best = -INFINITY;
    int idx = 0x7fffffff;
    s_hist[tid] = 0;
    __syncthreads();
    auto consider = [&](float v, int i) {
        better(best, idx, v, i);
        if (counts) atomicAdd(&s_hist[order_key(v) >> 24], 1u);
    };
    if (pen == 1.0f) {
        sweep_strided(lrow, sl.lo, sl.hi, tid, [&](float l, int i) {
            const float v = l * inv_t;
            w[i] = v;
            consider(v, i);
        });
    } else {
        sweep_strided(lrow, sl.lo, sl.hi, tid, [&](float l, int i) { w[i] = l * inv_t; });
        __syncthreads();
        const int first = a.pen_off[r];
        const int n_pen = a.pen_count ? a.pen_count[r] : a.pen_off[r + 1] - first;
        for (int j = tid; j < n_pen; j += SP_THREADS) {
            const int id = a.pen_ids[first + j];
            if (id >= sl.lo && id < sl.hi) {
                float l = lrow[id];
                l = l > 0.f ? l / pen : l * pen;
                w[id] = l * inv_t;
            }
        }
        __syncthreads();
        sweep_strided(w, sl.lo, sl.hi, tid, consider);
    }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
        const float v2 = __shfl_xor(best, off, WAVE);
        const int i2 = __shfl_xor(idx, off, WAVE);
        better(best, idx, v2, i2);
    }
    const int wave = tid / WAVE, lane = tid % WAVE;
    if (lane == 0) { s_val[wave] = best; s_idx[wave] = idx; }
    __syncthreads();
    if (tid == 0) {
        for (int wv = 1; wv < SP_WAVES; ++wv) better(best, idx, s_val[wv], s_idx[wv]);
        a.part_max[r * a.P + part] = best;
        a.part_arg[r * a.P + part] = idx;
        s_val[0] = best;
    }
    if (counts) hist_of(a, 0, r, part)[tid] = s_hist[tid];
    if (plain && row_samples(a, r)) {
        __syncthreads();
        const float m = s_val[0];           // the slice's largest value (every thread reads back what the workgroup wrote)
        float z = 0.f;
        sweep_strided(w, sl.lo, sl.hi, tid, [&](float v, int) { z += expf(v - m); });
        z = block_sum(z, s_red);
        if (tid == 0) a.part_z[r * a.P + part] = z;
    }
}

// Launches 2 to 4 (level = 1, 2, 3): decide level `level` - 1 of the top-k descent from the counts the
// launch before left, then count the next eight bits of the keys that share the prefix so far.
__global__ __launch_bounds__(SP_THREADS) void sample_top_k_kernel(SampleArgs a, int level) {
    __shared__ uint32_t s_scan[SP_WAVES + 1];
    __shared__ int s_bin;
    __shared__ uint32_t s_hist[256];
    const int r = blockIdx.x, part = blockIdx.y, tid = threadIdx.x;
    if (!row_top_k(a, r)) return;
    uint32_t* st = a.state + static_cast<size_t>(r) * 16;
    uint32_t prefix = level == 1 ? 0u : st[2 * (level - 2)];
    uint32_t remaining = level == 1 ? static_cast<uint32_t>(a.top_k[r]) : st[2 * (level - 2) + 1];
    const int b = decide_level<uint32_t>(hist_of(a, (level - 1) & 1, r, 0), a.P, remaining, s_scan, &s_bin);
    const int decided_shift = 24 - 8 * (level - 1);
    prefix |= static_cast<uint32_t>(b) << decided_shift;
    if (part == 0 && tid == 0) { st[2 * (level - 1)] = prefix; st[2 * (level - 1) + 1] = remaining; }
    const int shift = decided_shift - 8;
    const uint32_t mask = 0xffffffffu << decided_shift;
    s_hist[tid] = 0;
    __syncthreads();
    const Slice sl = slice_of(part, a.V, a.P);
    const float* w = a.work + static_cast<size_t>(r) * a.V;
    sweep_strided(w, sl.lo, sl.hi, tid, [&](float v, int) {
        const uint32_t key = order_key(v);
        if ((key & mask) == prefix) atomicAdd(&s_hist[(key >> shift) & 255u], 1u);
    });
    __syncthreads();
    hist_of(a, level & 1, r, part)[tid] = s_hist[tid];
}

// The key of the k-th largest value once the counts of the last level are in (hist buffer 1), or 0.
__device__ uint32_t top_k_threshold(const SampleArgs& a, int r, uint32_t* s_scan, int* s_bin) {
    if (!row_top_k(a, r)) return 0u;
    const uint32_t* st = a.state + static_cast<size_t>(r) * 16;
    uint32_t remaining = st[5];
    const int b = decide_level<uint32_t>(hist_of(a, 1, r, 0), a.P, remaining, s_scan, s_bin);
    return st[4] | static_cast<uint32_t>(b);
}

// The row's largest value from the slices' (at most 32 of them: one load each by the first threads, met in LDS).
// Called by every thread of the workgroup.
__device__ float row_max(const SampleArgs& a, int r) {
    __shared__ float s_row_max;
    const int tid = threadIdx.x;
    if (tid < WAVE) {
        float m = tid < a.P ? a.part_max[r * a.P + tid] : -INFINITY;
#pragma unroll
        for (int off = WAVE / 2; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, WAVE));
        if (tid == 0) s_row_max = m;
    }
    __syncthreads();
    return s_row_max;
}

// Launch 5: the softmax mass of the slice's kept tokens, and the sums of the first radix level for top-p.
__global__ __launch_bounds__(SP_THREADS) void sample_mass_kernel(SampleArgs a) {
    __shared__ uint32_t s_scan[SP_WAVES + 1];
    __shared__ int s_bin;
    __shared__ float s_red[16];
    __shared__ float s_hist[256];
    const int r = blockIdx.x, part = blockIdx.y, tid = threadIdx.x;
    if (!row_samples(a, r)) return;
    const uint32_t thr = top_k_threshold(a, r, s_scan, &s_bin);
    if (part == 0 && tid == 0) a.state[static_cast<size_t>(r) * 16 + 6] = thr;
    const float M = row_max(a, r);
    const bool sums = row_top_p(a, r);
    s_hist[tid] = 0.f;
    __syncthreads();
    const Slice sl = slice_of(part, a.V, a.P);
    const float* w = a.work + static_cast<size_t>(r) * a.V;
    float z = 0.f;
    sweep_strided(w, sl.lo, sl.hi, tid, [&](float v, int) {
        const uint32_t key = order_key(v);
        if (key >= thr) {
            const float e = expf(v - M);
            z += e;
            if (sums) atomicAdd(&s_hist[key >> 24], e);
        }
    });
    z = block_sum(z, s_red);
    if (tid == 0) a.part_z[r * a.P + part] = z;
    if (sums) hist_of(a, 0, r, part)[tid] = __float_as_uint(s_hist[tid]);
}

// Launches 6 to 8 (level = 1, 2, 3): the same descent for top-p, over sums of exp(w - max) of the kept tokens.
__global__ __launch_bounds__(SP_THREADS) void sample_top_p_kernel(SampleArgs a, int level) {
    __shared__ float s_scan[SP_WAVES + 1];
    __shared__ int s_bin;
    __shared__ float s_hist[256];
    const int r = blockIdx.x, part = blockIdx.y, tid = threadIdx.x;
    if (!row_top_p(a, r)) return;
    uint32_t* st = a.state + static_cast<size_t>(r) * 16;
    uint32_t prefix;
    float remaining;
    if (level == 1) {
        float z = 0.f;
        for (int p = 0; p < a.P; ++p) z += a.part_z[r * a.P + p];
        prefix = 0u;
        remaining = a.top_p[r] * z;
    } else {
        prefix = st[8 + 2 * (level - 2)];
        remaining = __uint_as_float(st[8 + 2 * (level - 2) + 1]);
    }
    const int b = decide_level<float>(hist_of(a, (level - 1) & 1, r, 0), a.P, remaining, s_scan, &s_bin);
    const int decided_shift = 24 - 8 * (level - 1);
    prefix |= static_cast<uint32_t>(b) << decided_shift;
    if (part == 0 && tid == 0) { st[8 + 2 * (level - 1)] = prefix; st[8 + 2 * (level - 1) + 1] = __float_as_uint(remaining); }
    const int shift = decided_shift - 8;
    const uint32_t mask = 0xffffffffu << decided_shift;
    const uint32_t thr = st[6];
    const float M = row_max(a, r);
    s_hist[tid] = 0.f;
    __syncthreads();
    const Slice sl = slice_of(part, a.V, a.P);
    const float* w = a.work + static_cast<size_t>(r) * a.V;
    sweep_strided(w, sl.lo, sl.hi, tid, [&](float v, int) {
        const uint32_t key = order_key(v);
        if (key >= thr && (key & mask) == prefix) atomicAdd(&s_hist[(key >> shift) & 255u], expf(v - M));
    });
    __syncthreads();
    hist_of(a, level & 1, r, part)[tid] = __float_as_uint(s_hist[tid]);
}

// Launch 9: the final threshold, and per slice the mass of the tokens it keeps and the last of them.
__global__ __launch_bounds__(SP_THREADS) void sample_kept_kernel(SampleArgs a) {
    __shared__ float s_scan[SP_WAVES + 1];
    __shared__ int s_bin;
    __shared__ float s_red[16];
    __shared__ int s_last;
    const int r = blockIdx.x, part = blockIdx.y, tid = threadIdx.x;
    if (!row_samples(a, r)) return;
    uint32_t* st = a.state + static_cast<size_t>(r) * 16;
    uint32_t thr = st[6];
    if (row_top_p(a, r)) {
        float remaining = __uint_as_float(st[8 + 5]);
        const int b = decide_level<float>(hist_of(a, 1, r, 0), a.P, remaining, s_scan, &s_bin);
        thr = max(thr, st[8 + 4] | static_cast<uint32_t>(b));
    }
    if (part == 0 && tid == 0) st[7] = thr;
    if (tid == 0) s_last = -1;
    __syncthreads();
    const float M = row_max(a, r);
    const Slice sl = slice_of(part, a.V, a.P);
    const float* w = a.work + static_cast<size_t>(r) * a.V;
    // contiguous runs per thread, as the draw walks them
    const int seg = (sl.hi - sl.lo + SP_THREADS - 1) / SP_THREADS;
    const int i0 = min(sl.hi, sl.lo + tid * seg), i1 = min(sl.hi, i0 + seg);
    float mine = 0.f;
    int last_kept = -1;
    sweep_run(w, i0, i1, [&](float v, int i) {
        if (order_key(v) >= thr) { mine += expf(v - M); last_kept = i; }
    });
    if (last_kept >= 0) atomicMax(&s_last, last_kept);
    const float mass = block_sum(mine, s_red);
    if (tid == 0) { a.part_mass[r * a.P + part] = mass; a.part_last[r * a.P + part] = s_last; }
}

// Launch 10, one workgroup per row: the slice in which the cumulative mass reaches u * total, and in
// it the first token that does (src/op/kernels/cuda/sampling_kernel.cu:330-398); rows that do not
// sample take the largest (penalised) logit.  `plain` (see the first launch): every token is kept, and a
// slice's mass is its sum of exp(w - its own maximum) scaled to the row's maximum.
__global__ __launch_bounds__(SP_THREADS) void sample_draw_kernel(SampleArgs a, int plain) {
    __shared__ float s_red[SP_WAVES];
    __shared__ int s_pick;
    __shared__ float s_pmax[32], s_mass[32];
    __shared__ int s_parg[32], s_plast[32];
    const int r = blockIdx.x, tid = threadIdx.x;
    if (tid < a.P) { s_pmax[tid] = a.part_max[r * a.P + tid]; s_parg[tid] = a.part_arg[r * a.P + tid]; }
    __syncthreads();
    float best_v = -INFINITY;
    int best = 0x7fffffff;
    for (int p = 0; p < a.P; ++p) better(best_v, best, s_pmax[p], s_parg[p]);
    if (best == 0x7fffffff) best = 0;        // a row of NaN or -inf: the first token
    // with pen_count the chosen token joins the row's penalised tokens: the next draw of a run sees it
    auto choose = [&](int token) {
        a.out[r] = token;
        if (a.pen_count) {
            const int n = a.pen_count[r];
            a.pen_ids[a.pen_off[r] + n] = token;
            a.pen_count[r] = n + 1;
        }
    };
    if (!row_samples(a, r)) {
        if (tid == 0) choose(best);
        return;
    }
    const float M = best_v;
    const uint32_t thr = plain ? 0u : a.state[static_cast<size_t>(r) * 16 + 7];
    if (tid < a.P) {
        if (plain) {
            const Slice sp = slice_of(tid, a.V, a.P);
            s_mass[tid] = sp.hi > sp.lo ? a.part_z[r * a.P + tid] * expf(s_pmax[tid] - M) : 0.f;
            s_plast[tid] = sp.hi > sp.lo ? sp.hi - 1 : -1;
        } else {
            s_mass[tid] = a.part_mass[r * a.P + tid];
            s_plast[tid] = a.part_last[r * a.P + tid];
        }
    }
    if (tid == 0) s_pick = 0x7fffffff;
    __syncthreads();
    float total = 0.f;
    int last = -1;
    for (int p = 0; p < a.P; ++p) { total += s_mass[p]; last = max(last, s_plast[p]); }
    const float target = a.uniform[r] * total;
    // the first slice whose cumulative mass reaches the target
    int part = -1;
    float before_part = 0.f;
    {
        float cum = 0.f;
        for (int p = 0; p < a.P; ++p) {
            const float m = s_mass[p];
            if (m > 0.f && cum < target && target <= cum + m) { part = p; before_part = cum; break; }
            cum += m;
        }
    }
    if (part >= 0) {
        const Slice sl = slice_of(part, a.V, a.P);
        const float* w = a.work + static_cast<size_t>(r) * a.V;
        const int seg = (sl.hi - sl.lo + SP_THREADS - 1) / SP_THREADS;
        const int i0 = min(sl.hi, sl.lo + tid * seg), i1 = min(sl.hi, i0 + seg);
        float mine = 0.f;
        int last_kept = -1;
        // a thread's run is short where slices are (sixteen tokens at 128,256 of them in 32 slices): then the
        // weights of its kept tokens stay in registers for the walk below (0 for a token that is not kept)
        constexpr int KEEP = 16;
        float kept_e[KEEP];
#pragma unroll
        for (int k = 0; k < KEEP; ++k) kept_e[k] = 0.f;
        const bool in_registers = seg <= KEEP;
        if (in_registers) {
#pragma unroll
            for (int k = 0; k < KEEP; ++k) {
                const float v = w[min(i0 + k, sl.hi - 1)];
                if (i0 + k < i1 && order_key(v) >= thr) { kept_e[k] = expf(v - M); mine += kept_e[k]; last_kept = i0 + k; }
            }
        } else {
            sweep_run(w, i0, i1, [&](float v, int i) {
                if (order_key(v) >= thr) { mine += expf(v - M); last_kept = i; }
            });
        }
        float incl = mine;
#pragma unroll
        for (int off = 1; off < WAVE; off <<= 1) {
            const float o = __shfl_up(incl, off, WAVE);
            if ((tid % WAVE) >= off) incl += o;
        }
        const int wave = tid / WAVE, lane = tid % WAVE;
        if (lane == WAVE - 1) s_red[wave] = incl;
        __syncthreads();
        float before = before_part;
        for (int wv = 0; wv < wave; ++wv) before += s_red[wv];
        incl += before;
        const float excl = incl - mine;
        if (mine > 0.f && excl < target && target <= incl) {
            float cum = excl;
            int pick = last_kept;
            bool found = false;
            if (in_registers) {
#pragma unroll
                for (int k = 0; k < KEEP; ++k) {
                    // (a kept token's weight may round to zero: it is passed over, as a token of no mass is never drawn)
                    if (!found && kept_e[k] > 0.f) {
                        cum += kept_e[k];
                        if (cum >= target) { pick = i0 + k; found = true; }
                    }
                }
            } else {
                sweep_run(w, i0, i1, [&](float v, int i) {
                    if (!found && order_key(v) >= thr) {
                        cum += expf(v - M);
                        if (cum >= target) { pick = i; found = true; }
                    }
                });
            }
            atomicMin(&s_pick, pick);
        }
        __syncthreads();
    }
    // rounding may leave the target a hair past every running sum: then the last kept token of the slice, or of the row
    if (tid == 0) {
        int pick = s_pick;
        if (pick == 0x7fffffff && part >= 0) pick = s_plast[part] >= 0 ? s_plast[part] : 0x7fffffff;
        choose(pick != 0x7fffffff ? pick : (last >= 0 ? last : best));
    }
}

// part_val: float [R, 32], part_idx: int32 [R, 32] scratch
NI_EXPORT int ni_argmax(const void* logits, void* out, void* part_val, void* part_idx, int R, int V, hipStream_t stream) {
    if (R <= 0) return 0;
    argmax_part_kernel<<<dim3(R, ARGMAX_PARTS), ARGMAX_THREADS, 0, stream>>>((const float*)logits, (float*)part_val,
                                                                             (int32_t*)part_idx, V);
    int err = NI_LAUNCH_RESULT();
    if (err) return err;
    argmax_final_kernel<<<R, WAVE, 0, stream>>>((const float*)part_val, (const int32_t*)part_idx, (int32_t*)out);
    return NI_LAUNCH_RESULT();
}

// Workgroups that share a row, for R rows of V logits: enough to cover the chip, slices of at least 1,024 tokens.
NI_EXPORT int ni_sample_parts(int R, int V) {
    int P = 512 / (R > 0 ? R : 1);
    P = P < 1 ? 1 : P > 32 ? 32 : P;
    while (P > 1 && (V + P - 1) / P < 1024) --P;
    return P;
}

// Scratch (see SampleArgs): work float [R, V]; parts float [R, P, 5] (maximum, its index, mass before top-p,
// mass kept, last kept index: five arrays of R * P words one after another); hist uint32 [2, R, P, 256];
// state uint32 [R, 16].  P must be ni_sample_parts(R, V).  uses_top_k / uses_top_p: 0 if no row asks for
// it (their launches are skipped then).  Row r's penalised tokens are pen_ids[pen_off[r] .. pen_off[r + 1]),
// or with pen_count (int32 [R]) the first pen_count[r] of them; then the chosen token is appended and the
// count raised, for the next draw of the same rows (the caller leaves room).
NI_EXPORT int ni_sample(const void* logits, void* work, const void* temperature, const void* top_k, const void* top_p,
                        const void* penalty, void* pen_ids, const void* pen_off, void* pen_count, const void* uniform,
                        void* out, void* parts, void* hist, void* state, int R, int V, int P, int uses_top_k,
                        int uses_top_p, hipStream_t stream) {
    if (R <= 0) return 0;
    if (V < 1 || P != ni_sample_parts(R, V) || !parts || !hist || !state) return -1;
    SampleArgs a;
    a.logits = (const float*)logits; a.work = (float*)work;
    a.temperature = (const float*)temperature; a.top_k = (const int32_t*)top_k; a.top_p = (const float*)top_p;
    a.penalty = (const float*)penalty; a.pen_ids = (int32_t*)pen_ids; a.pen_off = (const int32_t*)pen_off;
    a.pen_count = (int32_t*)pen_count;
    a.uniform = (const float*)uniform; a.out = (int32_t*)out;
    float* pf = (float*)parts;
    const size_t n = static_cast<size_t>(R) * P;
    a.part_max = pf; a.part_arg = (int32_t*)(pf + n); a.part_z = pf + 2 * n; a.part_mass = pf + 3 * n;
    a.part_last = (int32_t*)(pf + 4 * n);
    a.hist = (uint32_t*)hist; a.state = (uint32_t*)state;
    a.R = R; a.V = V; a.P = P;
    const dim3 grid(R, P);
    int err;
#define SP_STEP(call) call; if ((err = NI_LAUNCH_RESULT()) != 0) return err;
    // no row asks for top-k or top-p: every token is kept, and two launches do (the first also sums the slices' masses)
    const int plain = !uses_top_k && !uses_top_p;
    if (P > 32) return -1;
    SP_STEP((sample_prepare_kernel<<<grid, SP_THREADS, 0, stream>>>(a, plain)))
    if (!plain) {
        if (uses_top_k)
            for (int level = 1; level <= 3; ++level) { SP_STEP((sample_top_k_kernel<<<grid, SP_THREADS, 0, stream>>>(a, level))) }
        SP_STEP((sample_mass_kernel<<<grid, SP_THREADS, 0, stream>>>(a)))
        if (uses_top_p)
            for (int level = 1; level <= 3; ++level) { SP_STEP((sample_top_p_kernel<<<grid, SP_THREADS, 0, stream>>>(a, level))) }
        SP_STEP((sample_kept_kernel<<<grid, SP_THREADS, 0, stream>>>(a)))
    }
    SP_STEP((sample_draw_kernel<<<R, SP_THREADS, 0, stream>>>(a, plain)))
#undef SP_STEP
    return 0;
}
