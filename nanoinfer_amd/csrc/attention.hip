// Attention over the paged key/value cache, one query token at a time, for gfx950.
// Compiled once per head size (-DHEAD_DIM=n, a multiple of 16 up to 256).
//
// A work item is (query token, kv head, chunk of the query heads that share it, split of the
// key range).  The threads of a workgroup (256, or 512 when there are few work items: then one
// workgroup walks a whole key range with eight wavefronts and no second kernel has to merge
// splits) are arranged as key slots x dimension lanes:
// LPK consecutive lanes hold one key row between them (EPL dims each), so a wavefront reads
// 64/LPK whole rows per access, which are adjacent in a pool laid out
// [page, kv_head, slot_in_page, head_dim].  Every lane group keeps a running (max, sum, output)
// of its own for each query head; they are merged across the wave by shuffles, across waves
// through LDS, and across splits by a second, small kernel (letting the last workgroup of a split
// range do it needs device-wide fences, which cost more on this chip of eight L2 caches than the
// second launch does).
// Softmax and both products are float32; the bfloat16 instantiation takes exponentials with the
// hardware's exp2, the float32 one with the accurate library routine.
//
// Formula (reference: src/op/kernels/cuda/paged_attention_kernel.cu:111-199 for one token,
// src/op/kernels/cuda/prefill_attention_kernel.cu:66-141 for a chunk): the query at position P
// reads keys max(0, P+1-window)..P of its sequence through the block table, head h uses kv head
// h / (H/KVH), scores are scaled by `scale`, softmax subtracts the maximum and divides by the
// plain sum.  A prompt portion is handled as its tokens one by one: each reads the cache, which
// the step has already filled up to and including that token.
#include "common.h"
#include "attention_api.h"
#include <mutex>

#ifndef HEAD_DIM
#error "HEAD_DIM must be defined"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size: multiple of 16, at most 256");

#define ATT_THREADS 256        // threads of a workgroup
#define GT 4  // query heads handled together by one workgroup

template <typename T> struct Lanes {
    static constexpr int per16 = 16 / sizeof(T);                 // elements in a 16-byte access
    static constexpr int want = (HEAD_DIM + per16 - 1) / per16;  // lanes if each took 16 bytes
    static constexpr int LPK = want <= 1 ? 1 : want <= 2 ? 2 : want <= 4 ? 4 : want <= 8 ? 8 : 16;
    static constexpr int EPL = HEAD_DIM / LPK;
    static_assert(LPK * EPL == HEAD_DIM, "lanes x elements must cover a head");
};

// "minus infinity" that stays finite under subtraction: exp(NEG - x) is 0, never NaN
#define NEG_BIG (-1.0e30f)

template <bool FAST> __device__ __forceinline__ float ex(float x) {
    if constexpr (FAST) return __expf(x);
    else return expf(x);
}

template <typename T, bool POW2, int THREADS>
__global__ __launch_bounds__(THREADS) void token_attention_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ kpool, const T* __restrict__ vpool,
    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ positions, T* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    int H, int KVH, int page_size, int page_shift, int window, float scale, int nsplit) {
    using L = Lanes<T>;
    constexpr int LPK = L::LPK, EPL = L::EPL, HD = HEAD_DIM;
    constexpr int KPI = THREADS / LPK;           // keys per workgroup iteration
    constexpr int WAVES = THREADS / WAVE;
    constexpr bool FAST = sizeof(T) == 2;

    // (uncut key ranges of many tokens: a compute unit holds workgroups u and u + half the grid, the same x in the
    // lower and the upper half of y; the upper half takes the tokens from the far end, so that tokens that come in the
    // order of their contexts put a long and a short one on every unit)
    const int t = (gridDim.z == 1 && gridDim.y > 1 && 2 * blockIdx.y >= gridDim.y) ? gridDim.x - 1 - blockIdx.x : blockIdx.x;
    const int G = H / KVH;
    const int chunks = (G + GT - 1) / GT;
    const int g = blockIdx.y / chunks;
    const int chunk = blockIdx.y % chunks;
    const int h0 = g * G + chunk * GT;
    const int gc = min(GT, G - chunk * GT);
    const int split = blockIdx.z;

    const int pos = positions[t];
    const int seq = seq_of_token[t];
    const int hi = pos + 1;
    const int lo = window > 0 ? max(0, hi - window) : 0;
    const int per_split = (hi - lo + nsplit - 1) / nsplit;
    const int k0 = lo + split * per_split;
    const int k1 = min(hi, k0 + per_split);

    const int tid = threadIdx.x;
    const int sub = tid % LPK;
    const int kslot = tid / LPK;
    const int32_t* table = block_table + static_cast<size_t>(seq) * table_stride;

    float qreg[GT][EPL];
#pragma unroll
    for (int i = 0; i < GT; ++i) {
        if (i < gc) {
            VecIO<T, EPL>::load(q + static_cast<size_t>(t) * q_stride + static_cast<size_t>(h0 + i) * HD + sub * EPL, qreg[i]);
#pragma unroll
            for (int e = 0; e < EPL; ++e) qreg[i][e] *= scale;
        } else {
#pragma unroll
            for (int e = 0; e < EPL; ++e) qreg[i][e] = 0.f;
        }
    }

    float m[GT], l[GT], acc[GT][EPL];
#pragma unroll
    for (int i = 0; i < GT; ++i) {
        m[i] = NEG_BIG;
        l[i] = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[i][e] = 0.f;
    }

    // U keys per lane group and trip.  The loop is pipelined by hand: while trip t is being
    // multiplied, the rows of trip t+1 are in flight and the addresses of trip t+2 are being
    // worked out.  The running maximum moves once per trip: one rescaling of the output and
    // U + 1 exponentials per head and trip.
    constexpr int U = EPL <= 8 ? 4 : 2;
    auto page_of = [&](int j) { return POW2 ? (j >> page_shift) : j / page_size; };
    auto slot_of = [&](int j) { return POW2 ? (j & (page_size - 1)) : j % page_size; };

    // The block table of the key range is copied to LDS, a segment of TBL_MAX pages at a time
    // (one segment, unless the range is very long).  A table entry read from global memory
    // inside the loop would have to be waited for before the rows it points to can be asked
    // for, and that wait, being in order, would also drain every row load still in flight: one
    // full memory round trip per trip, whatever is prefetched.  With the table in LDS the row
    // loads of a trip depend on no other load, and stay in flight across the arithmetic.
    constexpr int TBL_MAX = 1024;
    __shared__ int32_t tbl[TBL_MAX];
    int s0 = k0, s1 = k0, lp0 = 0;     // keys s0..s1-1 are the current segment, its first page is lp0

    struct Where { size_t base[U]; bool valid[U]; };
    auto locate = [&](int it, Where& w) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = s0 + (it + u) * KPI + kslot;
            w.valid[u] = j < s1;
            const int jj = w.valid[u] ? j : s0;     // a key of this segment in any case: the address stays legal
            const int page = tbl[page_of(jj) - lp0];
            w.base[u] = ((static_cast<size_t>(page) * KVH + g) * page_size + slot_of(jj)) * HD + sub * EPL;
        }
    };
    struct Rows { RawRow<T, EPL> k[U], v[U]; bool valid[U]; };     // as loaded: converted when multiplied
    auto fetch = [&](const Where& w, Rows& r) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            r.k[u].load(kpool + w.base[u]);
            r.v[u].load(vpool + w.base[u]);
            r.valid[u] = w.valid[u];
        }
    };
    auto multiply = [&](const Rows& r) {
#pragma unroll
        for (int i = 0; i < GT; ++i) {
            float sc[U];
            float m_new = m[i];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float d = 0.f;
#pragma unroll
                for (int e = 0; e < EPL; ++e) d += qreg[i][e] * r.k[u].get(e);
#pragma unroll
                for (int o = LPK / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, WAVE);
                sc[u] = d;
                if (r.valid[u]) m_new = fmaxf(m_new, d);
            }
            const float corr = ex<FAST>(m[i] - m_new);
            float psum = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[i][e] *= corr;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float p = r.valid[u] ? ex<FAST>(sc[u] - m_new) : 0.f;
                psum += p;
#pragma unroll
                for (int e = 0; e < EPL; ++e) acc[i][e] += p * r.v[u].get(e);
            }
            l[i] = l[i] * corr + psum;
            m[i] = m_new;
        }
    };

    while (s1 < k1) {
        s0 = s1;
        lp0 = page_of(s0);
        s1 = min(k1, (lp0 + TBL_MAX) * page_size);
        __syncthreads();               // nobody still reads the previous segment's entries
        for (int i = tid; i <= page_of(s1 - 1) - lp0; i += THREADS) tbl[i] = table[lp0 + i];
        __syncthreads();
        const int iters = (s1 - s0 + KPI - 1) / KPI;

        // Two trips per turn of the loop, A and B, each with a place of its own in registers.
        // Rows past the end of the segment are loaded from a legal address and not used, so
        // that the loads are never under a branch.
        Where wa, wb;
        Rows ra, rb;
        locate(0, wa);
        locate(U, wb);
        fetch(wa, ra);
        for (int it = 0; it < iters; it += 2 * U) {
            fetch(wb, rb);
            locate(it + 2 * U, wa);
            multiply(ra);
            fetch(wa, ra);
            locate(it + 3 * U, wb);
            if (it + U < iters) multiply(rb);
        }
    }

    // merge the lane groups of a wave (lanes with equal `sub`)
#pragma unroll
    for (int o = LPK; o < WAVE; o <<= 1) {
#pragma unroll
        for (int i = 0; i < GT; ++i) {
            const float m_o = __shfl_xor(m[i], o, WAVE);
            const float l_o = __shfl_xor(l[i], o, WAVE);
            const float m_new = fmaxf(m[i], m_o);
            const float a = ex<FAST>(m[i] - m_new);
            const float b = ex<FAST>(m_o - m_new);
            l[i] = l[i] * a + l_o * b;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const float acc_o = __shfl_xor(acc[i][e], o, WAVE);
                acc[i][e] = acc[i][e] * a + acc_o * b;
            }
            m[i] = m_new;
        }
    }

    __shared__ float sm_m[WAVES][GT];
    __shared__ float sm_l[WAVES][GT];
    __shared__ float sm_acc[WAVES][GT][HD];
    const int wave = tid / WAVE;
    const int lane = tid % WAVE;
    if (lane < LPK) {
#pragma unroll
        for (int i = 0; i < GT; ++i) {
            if (lane == 0) { sm_m[wave][i] = m[i]; sm_l[wave][i] = l[i]; }
#pragma unroll
            for (int e = 0; e < EPL; ++e) sm_acc[wave][i][lane * EPL + e] = acc[i][e];
        }
    }
    __syncthreads();

    for (int idx = tid; idx < gc * HD; idx += THREADS) {
        const int i = idx / HD;
        const int dim = idx % HD;
        float M = sm_m[0][i];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) M = fmaxf(M, sm_m[w][i]);
        float Lsum = 0.f, O = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float f = ex<FAST>(sm_m[w][i] - M);
            Lsum += sm_l[w][i] * f;
            O += sm_acc[w][i][dim] * f;
        }
        const int h = h0 + i;
        if (nsplit == 1) {
            st(out + static_cast<size_t>(t) * H * HD + static_cast<size_t>(h) * HD + dim, O / Lsum);
        } else {
            const size_t p = (static_cast<size_t>(t) * H + h) * nsplit + split;
            part_o[p * HD + dim] = O;
            if (dim == 0) { part_ml[p * 2] = M; part_ml[p * 2 + 1] = Lsum; }
        }
    }
}

// Merge the partial (max, sum, output) of the splits of one (token, head).
template <typename T>
__global__ void merge_splits_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                    T* __restrict__ out, int H, int nsplit) {
    constexpr bool FAST = sizeof(T) == 2;
    const int t = blockIdx.x, h = blockIdx.y;
    const size_t p0 = (static_cast<size_t>(t) * H + h) * nsplit;
    float M = NEG_BIG;
    for (int s = 0; s < nsplit; ++s) M = fmaxf(M, part_ml[(p0 + s) * 2]);
    for (int dim = threadIdx.x; dim < HEAD_DIM; dim += blockDim.x) {
        float Lsum = 0.f, O = 0.f;
#pragma unroll 4
        for (int s = 0; s < nsplit; ++s) {
            const float f = ex<FAST>(part_ml[(p0 + s) * 2] - M);
            Lsum += part_ml[(p0 + s) * 2 + 1] * f;
            O += part_o[(p0 + s) * HEAD_DIM + dim] * f;
        }
        st(out + static_cast<size_t>(t) * H * HEAD_DIM + static_cast<size_t>(h) * HEAD_DIM + dim, O / Lsum);
    }
}

template <typename T>
static int launch(const void* q, int q_stride, const void* kpool, const void* vpool, const void* block_table,
                  int table_stride, const void* seq_of_token, const void* positions, void* out, void* part_o,
                  void* part_ml, int T_tokens, int H, int KVH, int page_size, int window, float scale,
                  int nsplit, hipStream_t stream) {
    const int G = H / KVH;
    const int chunks = (G + GT - 1) / GT;
    dim3 grid(T_tokens, KVH * chunks, nsplit);
    // a page size that is a power of two gets shifts and masks, any other divisions
    const bool pow2 = (page_size & (page_size - 1)) == 0;
    int page_shift = 0;
    while (pow2 && (1 << page_shift) < page_size) ++page_shift;
#define TA_ARGS                                                                                                    \
    (const T*)q, q_stride, (const T*)kpool, (const T*)vpool, (const int32_t*)block_table, table_stride,            \
        (const int32_t*)seq_of_token, (const int32_t*)positions, (T*)out, (float*)part_o, (float*)part_ml, H, KVH, \
        page_size, page_shift, window, scale, nsplit
    auto kernel = pow2 ? token_attention_kernel<T, true, ATT_THREADS> : token_attention_kernel<T, false, ATT_THREADS>;
    kernel<<<grid, ATT_THREADS, 0, stream>>>(TA_ARGS);
#undef TA_ARGS
    int err = NI_LAUNCH_RESULT();
    if (err || nsplit == 1) return err;
    merge_splits_kernel<T><<<dim3(T_tokens, H), 64, 0, stream>>>((const float*)part_o, (const float*)part_ml, (T*)out,
                                                                H, nsplit);
    return NI_LAUNCH_RESULT();
}

NI_EXPORT int ni_attention_head_dim() { return HEAD_DIM; }
NI_EXPORT int ni_attention_heads_per_group() { return GT; }

// part_o: float [T, H, nsplit, HEAD_DIM], part_ml: float [T, H, nsplit, 2]; unused when nsplit == 1.
NI_EXPORT int ni_token_attention(const void* q, int q_stride, const void* kpool, const void* vpool,
                                 const void* block_table, int table_stride, const void* seq_of_token,
                                 const void* positions, void* out, void* part_o, void* part_ml,
                                 int T_tokens, int H, int KVH, int page_size, int window, float scale, int nsplit,
                                 int dtype, hipStream_t stream) {
    if (T_tokens <= 0) return 0;
    if (H % KVH != 0 || nsplit < 1 || nsplit > 65535 || page_size < 1) return -1;
    if (nsplit > 1 && (!part_o || !part_ml)) return -2;
    if (dtype == 0)
        return launch<float>(q, q_stride, kpool, vpool, block_table, table_stride, seq_of_token, positions, out,
                             part_o, part_ml, T_tokens, H, KVH, page_size, window, scale, nsplit, stream);
    return launch<bf16_t>(q, q_stride, kpool, vpool, block_table, table_stride, seq_of_token, positions, out, part_o,
                          part_ml, T_tokens, H, KVH, page_size, window, scale, nsplit, stream);
}

// Merge of partial results in the layout above, for kernels of other libraries that split the keys.
NI_EXPORT int ni_merge_splits(const void* part_o, const void* part_ml, void* out, int T_tokens, int H, int nsplit,
                              int dtype, hipStream_t stream) {
    if (T_tokens <= 0) return 0;
    if (dtype == 0)
        merge_splits_kernel<float><<<dim3(T_tokens, H), 64, 0, stream>>>((const float*)part_o, (const float*)part_ml,
                                                                        (float*)out, H, nsplit);
    else
        merge_splits_kernel<bf16_t><<<dim3(T_tokens, H), 64, 0, stream>>>((const float*)part_o, (const float*)part_ml,
                                                                         (bf16_t*)out, H, nsplit);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- the entry point that allocates nothing
// The partial results of the key runs, held by the library itself.  In host code the array's
// name is only a handle for hipGetSymbolAddress: the address that kernels are given is asked for
// once per device and kept.
#define STATIC_SCRATCH_FLOATS (1L << 20)
#define STATIC_MAX_DEVICES 64
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];
static float* scratch_of_device[STATIC_MAX_DEVICES];
static std::mutex scratch_lock;

// Address of the current device's copy of the array (each GPU has its own), or null with *err set.
static float* static_scratch(int* err) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { *err = static_cast<int>(e); return nullptr; }
    if (dev < 0 || dev >= STATIC_MAX_DEVICES) { *err = -4; return nullptr; }
    std::lock_guard<std::mutex> hold(scratch_lock);
    if (!scratch_of_device[dev]) {
        float* ptr = nullptr;
        e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) { *err = e != hipSuccess ? static_cast<int>(e) : -5; return nullptr; }
        scratch_of_device[dev] = ptr;
    }
    return scratch_of_device[dev];
}

NI_EXPORT long ni_token_attention_static_floats(void) { return STATIC_SCRATCH_FLOATS; }

NI_EXPORT int ni_token_attention_static(const void* q, int q_stride, const void* kpool, const void* vpool,
                                        const void* block_table, int table_stride, const void* seq_of_token,
                                        const void* positions, void* out, int T_tokens, int H, int KVH,
                                        int page_size, int window, float scale, int nsplit, int dtype,
                                        hipStream_t stream) {
    if (T_tokens <= 0) return 0;
    if (H < 1 || KVH < 1 || H % KVH != 0 || nsplit < 1 || nsplit > 65535 || page_size < 1) return -1;
    float* part_o = nullptr;
    float* part_ml = nullptr;
    if (nsplit > 1) {
        const long long rows = static_cast<long long>(T_tokens) * H * nsplit;
        if (rows * (HEAD_DIM + 2) > STATIC_SCRATCH_FLOATS) return -3;      // more than the array holds
        int err = 0;
        float* base = static_scratch(&err);
        if (!base) return err;
        part_o = base;
        part_ml = base + rows * HEAD_DIM;
    }
    return ni_token_attention(q, q_stride, kpool, vpool, block_table, table_stride, seq_of_token, positions, out,
                              part_o, part_ml, T_tokens, H, KVH, page_size, window, scale, nsplit, dtype, stream);
}
