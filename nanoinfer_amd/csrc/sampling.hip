// Token selection from float32 logits for gfx950: argmax, and the sampling pipeline
// repetition penalty -> temperature -> top-k -> softmax -> top-p -> renormalise -> inverse CDF
// (order of src/sampler/configurable_sampler.cpp:93-120 of the reference).
//
// One workgroup of 1024 threads owns one row.  Thresholds are exact selections, not the
// 16-step bisections of src/op/kernels/cuda/sampling_kernel.cu:202-296: a radix descent over
// the order-preserving integer image of a float finds the k-th largest logit (counts) and the
// smallest logit whose upper set still holds the mass top_p (sums).  Equal logits at a
// threshold are kept together.  The draw walks the kept tokens in vocabulary order and takes
// the first whose cumulative mass reaches u * total (src/op/kernels/cuda/sampling_kernel.cu:330-398);
// u in (0, 1] comes from the host, which derives it from (seed, request, step).
#include "common.h"

#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / WAVE)

__device__ __forceinline__ uint32_t order_key(float f) {
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// argmax with the lowest index among equal values (src/op/kernels/cuda/argmax_kernel.cu:27).
__device__ __forceinline__ void better(float& v, int& i, float v2, int i2) {
    if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
}

__device__ int block_argmax(const float* __restrict__ row, int V, float* out_max, float* s_val, int* s_idx) {
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += blockDim.x) better(best, idx, row[i], i);
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
        float v2 = __shfl_xor(best, off, WAVE);
        int i2 = __shfl_xor(idx, off, WAVE);
        better(best, idx, v2, i2);
    }
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    __syncthreads();
    if (lane == 0) { s_val[wave] = best; s_idx[wave] = idx; }
    __syncthreads();
    const int nw = (blockDim.x + WAVE - 1) / WAVE;
    best = s_val[0]; idx = s_idx[0];
    for (int w = 1; w < nw; ++w) better(best, idx, s_val[w], s_idx[w]);
    if (idx == 0x7fffffff) idx = 0;  // a row of NaN or -inf: fall back to the first token
    *out_max = best;
    return idx;
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

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, float* __restrict__ work, const float* __restrict__ temperature,
    const int32_t* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ penalty,
    const int32_t* __restrict__ pen_ids, const int32_t* __restrict__ pen_off, const float* __restrict__ uniform,
    int32_t* __restrict__ out, int V) {
    __shared__ float s_val[SAMPLE_WAVES];
    __shared__ int s_idx[SAMPLE_WAVES];
    __shared__ float s_red[SAMPLE_WAVES];
    __shared__ float hist_f[256];
    __shared__ uint32_t hist_u[256];
    __shared__ uint32_t s_prefix;
    __shared__ float s_remaining_f;
    __shared__ uint32_t s_remaining_u;
    __shared__ int s_pick;
    __shared__ int s_last;

    const int r = blockIdx.x;
    const int tid = threadIdx.x;
    const float* lrow = logits + static_cast<size_t>(r) * V;
    float* w = work + static_cast<size_t>(r) * V;
    const float T = temperature[r];
    const float inv_t = (T <= 0.f || T == 1.0f) ? 1.0f : 1.0f / T;
    const float pen = penalty[r];

    // penalty and temperature (src/op/kernels/cuda/sampling_kernel.cu:38-88)
    for (int i = tid; i < V; i += SAMPLE_THREADS) w[i] = lrow[i] * inv_t;
    __syncthreads();
    if (pen != 1.0f) {
        for (int j = pen_off[r] + tid; j < pen_off[r + 1]; j += SAMPLE_THREADS) {
            const int id = pen_ids[j];
            if (id >= 0 && id < V) {
                float l = lrow[id];
                l = l > 0.f ? l / pen : l * pen;
                w[id] = l * inv_t;
            }
        }
        __syncthreads();
    }

    float M;
    const int best = block_argmax(w, V, &M, s_val, s_idx);
    if (T <= 0.f) {
        if (tid == 0) out[r] = best;
        return;
    }

    // top-k: the k-th largest key, by counts
    uint32_t thr = 0;
    const int k = top_k[r];
    if (k > 0 && k < V) {
        if (tid == 0) { s_prefix = 0; s_remaining_u = static_cast<uint32_t>(k); }
        for (int shift = 24; shift >= 0; shift -= 8) {
            if (tid < 256) hist_u[tid] = 0;
            __syncthreads();
            const uint32_t prefix = s_prefix;
            const uint32_t mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
            for (int i = tid; i < V; i += SAMPLE_THREADS) {
                const uint32_t key = order_key(w[i]);
                if ((key & mask) == prefix) atomicAdd(&hist_u[(key >> shift) & 255u], 1u);
            }
            __syncthreads();
            if (tid == 0) {
                uint32_t remaining = s_remaining_u, cum = 0;
                int b = 255;
                for (; b > 0; --b) {
                    if (cum + hist_u[b] >= remaining) break;
                    cum += hist_u[b];
                }
                s_remaining_u = remaining - cum;
                s_prefix = prefix | (static_cast<uint32_t>(b) << shift);
            }
            __syncthreads();
        }
        thr = s_prefix;
    }

    // softmax mass of the kept tokens
    float z = 0.f;
    for (int i = tid; i < V; i += SAMPLE_THREADS)
        if (order_key(w[i]) >= thr) z += expf(w[i] - M);
    z = block_sum(z, s_red);

    // top-p: the largest key whose upper set holds at least top_p of the mass, by sums
    const float p = top_p[r];
    if (p > 0.f && p < 1.0f) {
        __syncthreads();
        if (tid == 0) { s_prefix = 0; s_remaining_f = p * z; }
        for (int shift = 24; shift >= 0; shift -= 8) {
            if (tid < 256) hist_f[tid] = 0.f;
            __syncthreads();
            const uint32_t prefix = s_prefix;
            const uint32_t mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
            for (int i = tid; i < V; i += SAMPLE_THREADS) {
                const uint32_t key = order_key(w[i]);
                if (key >= thr && (key & mask) == prefix) atomicAdd(&hist_f[(key >> shift) & 255u], expf(w[i] - M));
            }
            __syncthreads();
            if (tid == 0) {
                float remaining = s_remaining_f, cum = 0.f;
                int b = 255;
                for (; b > 0; --b) {
                    if (cum + hist_f[b] >= remaining) break;
                    cum += hist_f[b];
                }
                s_remaining_f = remaining - cum;
                s_prefix = prefix | (static_cast<uint32_t>(b) << shift);
            }
            __syncthreads();
        }
        thr = max(thr, s_prefix);
    }

    // inverse CDF in vocabulary order over contiguous segments
    const int seg = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int i0 = min(V, tid * seg), i1 = min(V, i0 + seg);
    float mine = 0.f;
    int last_kept = -1;
    for (int i = i0; i < i1; ++i)
        if (order_key(w[i]) >= thr) { mine += expf(w[i] - M); last_kept = i; }
    // inclusive scan over threads
    float incl = mine;
#pragma unroll
    for (int off = 1; off < WAVE; off <<= 1) {
        float o = __shfl_up(incl, off, WAVE);
        if ((tid % WAVE) >= off) incl += o;
    }
    const int wave = tid / WAVE, lane = tid % WAVE;
    __syncthreads();
    if (tid == 0) { s_pick = 0x7fffffff; s_last = -1; }
    if (lane == WAVE - 1) s_red[wave] = incl;
    __syncthreads();
    float before = 0.f, total = 0.f;
    for (int wv = 0; wv < SAMPLE_WAVES; ++wv) {
        if (wv < wave) before += s_red[wv];
        total += s_red[wv];
    }
    incl += before;
    const float excl = incl - mine;
    const float target = uniform[r] * total;
    if (last_kept >= 0) atomicMax(&s_last, last_kept);
    if (mine > 0.f && excl < target && target <= incl) {
        float cum = excl;
        int pick = last_kept;
        for (int i = i0; i < i1; ++i) {
            if (order_key(w[i]) >= thr) {
                cum += expf(w[i] - M);
                if (cum >= target) { pick = i; break; }
            }
        }
        atomicMin(&s_pick, pick);
    }
    __syncthreads();
    if (tid == 0) out[r] = s_pick != 0x7fffffff ? s_pick : (s_last >= 0 ? s_last : best);
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

NI_EXPORT int ni_sample(const void* logits, void* work, const void* temperature, const void* top_k, const void* top_p,
                        const void* penalty, const void* pen_ids, const void* pen_off, const void* uniform, void* out,
                        int R, int V, hipStream_t stream) {
    if (R <= 0) return 0;
    sample_kernel<<<R, SAMPLE_THREADS, 0, stream>>>((const float*)logits, (float*)work, (const float*)temperature,
                                                    (const int32_t*)top_k, (const float*)top_p, (const float*)penalty,
                                                    (const int32_t*)pen_ids, (const int32_t*)pen_off,
                                                    (const float*)uniform, (int32_t*)out, V);
    return NI_LAUNCH_RESULT();
}
