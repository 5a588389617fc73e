// Row-wise and element-wise kernels of a decoder step for gfx950: embedding gather,
// residual-add + RMSNorm, rotation table, rotation + paged key/value write, SwiGLU.
//
// Conventions shared by all of them:
//   * the residual stream is float32; activations that feed a matrix product are the
//     compute type (float or bfloat16); all arithmetic is float32;
//   * a key/value pool is laid out [page, kv_head, slot_in_page, head_dim];
//   * every entry point is extern "C", takes raw device pointers and a hipStream_t, and
//     returns 0 or the hipError_t of its launch.  Shapes are checked by the host wrapper.
#include "common.h"

#include <algorithm>

// ---------------------------------------------------------------- embedding
// out[t, :] = table[ids[t], :]   (src/op/kernels/cuda/embedding_kernel.cu:30-48 of the reference;
// ids are range-checked on the host before upload, an id outside the table never reaches here.)
template <typename T>
__global__ void embedding_kernel(const int32_t* __restrict__ ids, const T* __restrict__ table,
                                 float* __restrict__ out, int d, int vocab) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (id < 0 || id >= vocab) return;  // unreachable after the host check; never read out of bounds
    const T* row = table + static_cast<size_t>(id) * d;
    float* o = out + static_cast<size_t>(t) * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = ld(row + i);
}

// ---------------------------------------------------------------- add + RMSNorm
// v = h[row] + pending[row];  out = v * rsqrt(mean(v^2) + eps) * w
// Without `rows` the sum is written back to h (the residual stream moves on) and out has T rows.
// With `rows` (a gather before the output head) h is left alone and out row r comes from h[rows[r]].
// Formula: src/op/kernels/cuda/rmsnorm_kernel.cu:50-103 of the reference.
// Rows of up to NV * blockDim elements are held in registers: every load of the row is issued
// before anything waits, and the row is read from memory once.
template <typename TP, typename TO, int NV>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const TP* __restrict__ pending, int addends, size_t addend_stride,
                                   const float* __restrict__ w, TO* __restrict__ out,
                                   const int32_t* __restrict__ rows, int d, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
    float* hrow = h + src * d;
    const TP* prow = pending ? pending + src * d : nullptr;
    float v[NV], wv[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        v[j] = i < d ? hrow[i] : 0.f;
        wv[j] = i < d ? w[i] : 0.f;
    }
    if (prow) {
        // several addends (the shares of a product whose K range was cut) are added in their order;
        // four at a time are asked for before any is added, so that their loads overlap
        for (int a0 = 0; a0 < addends; a0 += 4) {
            float t[4][NV];
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int j = 0; j < NV; ++j) {
                    const int i = threadIdx.x + j * blockDim.x;
                    t[b][j] = (a0 + b < addends && i < d) ? ld(prow + (a0 + b) * addend_stride + i) : 0.f;
                }
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int j = 0; j < NV; ++j) v[j] += t[b][j];
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) ss += v[j] * v[j];
    if (!rows && prow) {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int i = threadIdx.x + j * blockDim.x;
            if (i < d) hrow[i] = v[j];
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
    TO* orow = out + static_cast<size_t>(r) * d;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        if (i < d) st(orow + i, (v[j] * inv) * wv[j]);
    }
}

// The same for rows whose width is a multiple of four: a thread holds G groups of four consecutive
// elements, so that every access is 16 bytes of float32 or 8 bytes of bfloat16 a lane and neighbouring
// lanes touch neighbouring groups (a third of the instructions, and the memory system sees whole lines).
template <typename TP, typename TO, int G>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ h, const TP* __restrict__ pending, int addends, size_t addend_stride,
                                       const float* __restrict__ w, TO* __restrict__ out,
                                       const int32_t* __restrict__ rows, int d, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
    float* hrow = h + src * d;
    const TP* prow = pending ? pending + src * d : nullptr;
    const int groups = d / 4;
    float v[G][4], wv[G][4];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int at = (threadIdx.x + g * blockDim.x) * 4;
        if (at < d) {
            VecIO<float, 4>::load(hrow + at, v[g]);
            VecIO<float, 4>::load(w + at, wv[g]);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[g][e] = wv[g][e] = 0.f;
        }
    }
    if (prow) {
        // the addends in their order, four asked for before any is added
        for (int a0 = 0; a0 < addends; a0 += 4) {
            float t[4][G][4];
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    const int at = (threadIdx.x + g * blockDim.x) * 4;
                    if (a0 + b < addends && at < d) {
                        VecIO<TP, 4>::load(prow + (a0 + b) * addend_stride + at, t[b][g]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) t[b][g][e] = 0.f;
                    }
                }
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int g = 0; g < G; ++g)
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[g][e] += t[b][g][e];
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) ss += v[g][e] * v[g][e];
    if (!rows && prow) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int at = (threadIdx.x + g * blockDim.x) * 4;
            if (at < d) store_packed<float, 4>(hrow + at, v[g]);
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
    TO* orow = out + static_cast<size_t>(r) * d;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int at = (threadIdx.x + g * blockDim.x) * 4;
        if (at < d) {
            float y[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = (v[g][e] * inv) * wv[g][e];
            store_packed<TO, 4>(orow + at, y);
        }
    }
}

// Rows of any width: two passes over memory.
template <typename TP, typename TO>
__global__ void add_rmsnorm_wide_kernel(float* __restrict__ h, const TP* __restrict__ pending, int addends, size_t addend_stride,
                                        const float* __restrict__ w, TO* __restrict__ out,
                                        const int32_t* __restrict__ rows, int d, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
    float* hrow = h + src * d;
    const TP* prow = pending ? pending + src * d : nullptr;
    float ss = 0.f;
    auto sum_at = [&](int i) {
        float v = hrow[i];
        if (prow)
            for (int a = 0; a < addends; ++a) v += ld(prow + a * addend_stride + i);
        return v;
    };
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        const float v = sum_at(i);
        if (!rows && prow) hrow[i] = v;
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
    TO* orow = out + static_cast<size_t>(r) * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        const float v = (rows && prow) ? sum_at(i) : hrow[i];
        st(orow + i, (v * inv) * w[i]);
    }
}

// ---------------------------------------------------------------- rotation table
// cos/sin[pos, p] of the float32 product pos * inv_freq[p]
// (src/op/kernels/cuda/rope_kernel.cu:129-131 of the reference; the frequencies come from the host).
__global__ void rope_table_kernel(const float* __restrict__ inv_freq, float* __restrict__ cos_t,
                                  float* __restrict__ sin_t, int max_pos, int half) {
    size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= static_cast<size_t>(max_pos) * half) return;
    int pos = static_cast<int>(idx / half);
    int p = static_cast<int>(idx % half);
    float angle = static_cast<float>(pos) * inv_freq[p];
    cos_t[idx] = cosf(angle);
    sin_t[idx] = sinf(angle);
}

// ---------------------------------------------------------------- rotation + key/value write
// qkv is [T, (H + 2*KVH) * hd]: q heads, then k heads, then v heads.  Queries are rotated in
// place; rotated keys and plain values go to the pools at slot_mapping[t] (= page*page_size + slot;
// negative: this layer does not write).  Pairs are (j, j + rot/2) inside the first `rot` dims of a
// head, which is the pairing of the checkpoint's row order (the reference permutes rows at export,
// tools/export_llama3.py:571-583, and rotates neighbours, src/op/kernels/cuda/rope_kernel.cu:32-84).
template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, const int32_t* __restrict__ positions,
                                     const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                     const int32_t* __restrict__ slot_mapping, T* __restrict__ kpool,
                                     T* __restrict__ vpool, int H, int KVH, int hd, int rot, int page_size) {
    const int t = blockIdx.x;
    const int half = rot / 2;
    const int row_width = (H + 2 * KVH) * hd;
    T* row = qkv + static_cast<size_t>(t) * row_width;
    const int pos = positions[t];
    const float* c = cos_t ? cos_t + static_cast<size_t>(pos) * half : nullptr;
    const float* s = sin_t ? sin_t + static_cast<size_t>(pos) * half : nullptr;
    const int slot = slot_mapping ? slot_mapping[t] : -1;
    const int page = slot >= 0 ? slot / page_size : 0;
    const int off = slot >= 0 ? slot % page_size : 0;

    // q and k heads: rotate pairs; dims beyond `rot` pass through.
    const int per_head = hd - half;  // `half` pairs + (hd - rot) pass-through dims
    for (int item = threadIdx.x; item < (H + KVH) * per_head; item += blockDim.x) {
        const int head = item / per_head;
        const int j = item % per_head;
        T* hp = row + static_cast<size_t>(head) * hd;
        const bool is_k = head >= H;
        T* dst = nullptr;
        if (is_k && slot >= 0)
            dst = kpool + ((static_cast<size_t>(page) * KVH + (head - H)) * page_size + off) * hd;
        if (j < half) {
            float x0 = ld(hp + j), x1 = ld(hp + j + half);
            float cs = c[j], sn = s[j];
            float y0 = x0 * cs - x1 * sn;
            float y1 = x0 * sn + x1 * cs;
            if (!is_k) {
                st(hp + j, y0);
                st(hp + j + half, y1);
            } else if (dst) {
                st(dst + j, y0);
                st(dst + j + half, y1);
            }
        } else {
            const int dim = rot + (j - half);
            if (is_k && dst) dst[dim] = hp[dim];
        }
    }
    if (slot >= 0) {
        for (int item = threadIdx.x; item < KVH * hd; item += blockDim.x) {
            const int g = item / hd, dim = item % hd;
            vpool[((static_cast<size_t>(page) * KVH + g) * page_size + off) * hd + dim] =
                row[static_cast<size_t>(H + KVH + g) * hd + dim];
        }
    }
}

// ---------------------------------------------------------------- SwiGLU
// out[t, i] = silu(gu[t, i]) * gu[t, I + i]   (src/op/kernels/cuda/swiglu_kernel.cu:31-39 of the
// reference, with expf instead of the fast intrinsic).
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t n) {
    size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    size_t t = idx / I;
    int i = static_cast<int>(idx % I);
    float g = ld(gu + t * 2 * I + i);
    float u = ld(gu + t * 2 * I + I + i);
    st(out + idx, g / (1.0f + expf(-g)) * u);
}

// The same in accesses of 16 bytes, for head sizes and rotated halves that are multiples of 16 bytes
// of elements: an item is one such piece of a pair of halves, of a key's unrotated dims, or of a value.
template <typename T>
__global__ void rope_kv_write_vec_kernel(T* __restrict__ qkv, const int32_t* __restrict__ positions,
                                         const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                         const int32_t* __restrict__ slot_mapping, T* __restrict__ kpool,
                                         T* __restrict__ vpool, int H, int KVH, int hd, int rot, int page_size) {
    constexpr int V = 16 / sizeof(T);
    typedef uint32_t u32x4_hw __attribute__((ext_vector_type(4)));
    const int t = blockIdx.x;
    const int half = rot / 2;
    T* row = qkv + static_cast<size_t>(t) * (H + 2 * KVH) * hd;
    const int pos = positions[t];
    const float* c = cos_t + static_cast<size_t>(pos) * half;
    const float* s = sin_t + static_cast<size_t>(pos) * half;
    const int slot = slot_mapping ? slot_mapping[t] : -1;
    const int page = slot >= 0 ? slot / page_size : 0;
    const int off = slot >= 0 ? slot % page_size : 0;
    const int rot_vecs = half / V, pass_vecs = (hd - rot) / V, head_vecs = hd / V;
    const int n_rot = (H + KVH) * rot_vecs;
    const int n_pass = slot >= 0 ? KVH * pass_vecs : 0;
    const int n_val = slot >= 0 ? KVH * head_vecs : 0;
    for (int item = threadIdx.x; item < n_rot + n_pass + n_val; item += blockDim.x) {
        if (item < n_rot) {
            const int head = item / rot_vecs, j = (item % rot_vecs) * V;
            T* hp = row + static_cast<size_t>(head) * hd;
            const bool is_k = head >= H;
            if (is_k && slot < 0) continue;
            T* dst = is_k ? kpool + ((static_cast<size_t>(page) * KVH + (head - H)) * page_size + off) * hd : hp;
            float x0[V], x1[V], cs[V], sn[V], y0[V], y1[V];
            VecIO<T, V>::load(hp + j, x0);
            VecIO<T, V>::load(hp + j + half, x1);
            VecIO<float, V>::load(c + j, cs);
            VecIO<float, V>::load(s + j, sn);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                y0[e] = x0[e] * cs[e] - x1[e] * sn[e];
                y1[e] = x0[e] * sn[e] + x1[e] * cs[e];
            }
            if constexpr (sizeof(T) == 4) {
                store_packed<T, 4>(dst + j, y0);
                store_packed<T, 4>(dst + j + half, y1);
            } else {
                store_packed<T, 8>(dst + j, y0);
                store_packed<T, 8>(dst + j + half, y1);
            }
        } else if (item < n_rot + n_pass) {
            const int k = item - n_rot, g = k / pass_vecs, dim = rot + (k % pass_vecs) * V;
            T* dst = kpool + ((static_cast<size_t>(page) * KVH + g) * page_size + off) * hd;
            *reinterpret_cast<u32x4_hw*>(dst + dim) = *reinterpret_cast<const u32x4_hw*>(row + static_cast<size_t>(H + g) * hd + dim);
        } else {
            const int k = item - n_rot - n_pass, g = k / head_vecs, dim = (k % head_vecs) * V;
            T* dst = vpool + ((static_cast<size_t>(page) * KVH + g) * page_size + off) * hd;
            *reinterpret_cast<u32x4_hw*>(dst + dim) =
                *reinterpret_cast<const u32x4_hw*>(row + static_cast<size_t>(H + KVH + g) * hd + dim);
        }
    }
}

// The same, 16 bytes of gate and of up per thread (rows whose width is a multiple of V elements).
// The bfloat16 instantiation takes the exponential with the hardware's exp2: its error is far
// below the rounding of the stored result.
template <typename T, int V>
__global__ void swiglu_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t n_vec) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= n_vec) return;
    const int per_row = I / V;
    const size_t t = idx / per_row;
    const int i = static_cast<int>(idx % per_row) * V;
    float g[V], u[V], y[V];
    VecIO<T, V>::load(gu + t * 2 * I + i, g);
    VecIO<T, V>::load(gu + t * 2 * I + I + i, u);
#pragma unroll
    for (int e = 0; e < V; ++e) {
        const float ex = sizeof(T) == 2 ? __expf(-g[e]) : expf(-g[e]);
        y[e] = g[e] / (1.0f + ex) * u[e];
    }
    VecIO<T, V>::store(out + t * I + i, y);
}

// ---------------------------------------------------------------- random weights
// Element `start + i` of the normal stream of `key`: a counter-based generator (splitmix64 over
// key + (index + 1) * gamma, Box-Muller over two 24-bit fractions).  Every operation is an IEEE
// float32 operation rounded on its own (contraction into fused multiply-adds is switched off in
// these routines; division and square root are the correctly rounded ones), and logarithm and
// cosine are fixed polynomials, so that the host's numpy twin of this routine
// (nanoinfer_amd/weights/random_init.py) gives the same bits.
__device__ __forceinline__ float rn_poly6(float x2, float c0, float c1, float c2, float c3, float c4, float c5) {
#pragma clang fp contract(off)
    float acc = c5;
    acc = acc * x2; acc = acc + c4;
    acc = acc * x2; acc = acc + c3;
    acc = acc * x2; acc = acc + c2;
    acc = acc * x2; acc = acc + c1;
    acc = acc * x2; acc = acc + c0;
    return acc;
}

__device__ __forceinline__ float counter_normal(uint64_t key, uint64_t index, float mean, float std) {
#pragma clang fp contract(off)
    uint64_t z = key + (index + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    const int k1 = static_cast<int>(z >> 40) + 1;          // 1 .. 2^24
    const int k2 = static_cast<int>(z & 0xFFFFFFull);      // 0 .. 2^24 - 1
    // -2 ln(k1 / 2^24): k1 = m * 2^e, m brought into [sqrt(1/2), sqrt(2)); ln m = 2 atanh((m-1)/(m+1))
    int e;
    float m = frexpf(static_cast<float>(k1), &e);          // m in [0.5, 1), exact
    if (m < 0.7071067811865476f) { m = m * 2.0f; e -= 1; }
    const float ef = static_cast<float>(e - 24);
    const float num = m - 1.0f, den = m + 1.0f;
    const float s = num / den;                             // correctly rounded (the compiler's default for HIP)
    const float s2 = s * s;
    const float ln_m = s * rn_poly6(s2, 2.0f / 1, 2.0f / 3, 2.0f / 5, 2.0f / 7, 2.0f / 9, 2.0f / 11);
    const float e_ln2 = ef * 0.6931471805599453f;
    const float ln_u = e_ln2 + ln_m;
    const float radius = sqrtf(-2.0f * ln_u);              // correctly rounded as well
    // cos(2 pi k2 / 2^24): quarter turns q, the rest f in [0, 1) folded to [0, 1/2], x = pi/2 f
    const int q = k2 >> 22;
    const float f = static_cast<float>(k2 & 0x3FFFFF) * (1.0f / 4194304.0f);
    const bool fold = f > 0.5f;
    const float x = (fold ? 1.0f - f : f) * 1.5707963267948966f;
    const float x2 = x * x;
    const float sin_x = x * rn_poly6(x2, 1.0f, -1.0f / 6, 1.0f / 120, -1.0f / 5040, 1.0f / 362880, -1.0f / 39916800);
    const float cos_x = rn_poly6(x2, 1.0f, -0.5f, 1.0f / 24, -1.0f / 720, 1.0f / 40320, -1.0f / 3628800);
    const float sin_f = fold ? cos_x : sin_x;
    const float cos_f = fold ? sin_x : cos_x;
    const float c = q == 0 ? cos_f : q == 1 ? -sin_f : q == 2 ? -cos_f : sin_f;
    const float n = radius * c;
    const float scaled = std * n;
    return scaled + mean;
}

template <typename T>
__global__ void random_normal_kernel(T* __restrict__ out, size_t count, uint64_t key, uint64_t start, float mean, float std) {
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride)
        st(out + i, counter_normal(key, start + i, mean, std));
}

// ================================================================ entry points
// dtype codes: 0 = float32, 1 = bfloat16

static inline bool aligned_to(size_t bytes, const void* a, const void* b = nullptr, const void* c = nullptr,
                              const void* d = nullptr) {
    return (reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c) |
            reinterpret_cast<uintptr_t>(d)) % bytes == 0;
}

static inline unsigned blocks_for(size_t n, unsigned per) { return static_cast<unsigned>((n + per - 1) / per); }

NI_EXPORT int ni_embedding(const void* ids, const void* table, void* out, int T, int d, int vocab,
                           int table_dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (table_dtype == 0)
        embedding_kernel<float><<<T, 256, 0, stream>>>((const int32_t*)ids, (const float*)table, (float*)out, d, vocab);
    else
        embedding_kernel<bf16_t><<<T, 256, 0, stream>>>((const int32_t*)ids, (const bf16_t*)table, (float*)out, d, vocab);
    return NI_LAUNCH_RESULT();
}

template <typename TP, typename TO>
static void launch_add_rmsnorm(float* h, const TP* pending, int addends, size_t addend_stride, const float* w, TO* out,
                               const int32_t* rows, int n_rows, int d, float eps, hipStream_t stream) {
    constexpr int NV = 8;
    if (d <= NV * 1024) {
        const int threads = d <= NV * 64 ? 64 : d <= NV * 128 ? 128 : d <= NV * 256 ? 256 : d <= NV * 512 ? 512 : 1024;
        if (d % 4 == 0 && aligned_to(16, h, w) && aligned_to(4 * sizeof(TP), pending) && aligned_to(4 * sizeof(TO), out) &&
            (addends <= 1 || addend_stride % 4 == 0)) {
            add_rmsnorm_vec_kernel<TP, TO, NV / 4><<<n_rows, threads, 0, stream>>>(h, pending, addends, addend_stride, w, out,
                                                                                  rows, d, eps);
            return;
        }
        add_rmsnorm_kernel<TP, TO, NV><<<n_rows, threads, 0, stream>>>(h, pending, addends, addend_stride, w, out, rows, d, eps);
    } else {
        add_rmsnorm_wide_kernel<TP, TO><<<n_rows, 1024, 0, stream>>>(h, pending, addends, addend_stride, w, out, rows, d, eps);
    }
}

// pending: null, or [T, d] of the output type, or (addends >= 1 with float_addends) float32 [addends, T, d], whose
// slices are added in their order.
NI_EXPORT int ni_add_rmsnorm(void* h, const void* pending, int addends, int float_addends, size_t addend_stride,
                             const void* w, void* out, const void* rows, int n_rows, int d, float eps, int dtype,
                             hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (pending && (addends < 1 || (addends > 1 && !float_addends))) return -1;
    if (dtype == 0)
        launch_add_rmsnorm<float, float>((float*)h, (const float*)pending, addends, addend_stride, (const float*)w,
                                         (float*)out, (const int32_t*)rows, n_rows, d, eps, stream);
    else if (float_addends)
        launch_add_rmsnorm<float, bf16_t>((float*)h, (const float*)pending, addends, addend_stride, (const float*)w,
                                          (bf16_t*)out, (const int32_t*)rows, n_rows, d, eps, stream);
    else
        launch_add_rmsnorm<bf16_t, bf16_t>((float*)h, (const bf16_t*)pending, addends, addend_stride, (const float*)w,
                                           (bf16_t*)out, (const int32_t*)rows, n_rows, d, eps, stream);
    return NI_LAUNCH_RESULT();
}

NI_EXPORT int ni_rope_table(const void* inv_freq, void* cos_t, void* sin_t, int max_pos, int half,
                            hipStream_t stream) {
    size_t n = static_cast<size_t>(max_pos) * half;
    if (n == 0) return 0;
    rope_table_kernel<<<blocks_for(n, 256), 256, 0, stream>>>((const float*)inv_freq, (float*)cos_t, (float*)sin_t,
                                                              max_pos, half);
    return NI_LAUNCH_RESULT();
}

NI_EXPORT int ni_rope_kv_write(void* qkv, const void* positions, const void* cos_t, const void* sin_t,
                               const void* slot_mapping, void* kpool, void* vpool, int T, int H, int KVH, int hd,
                               int rot, int page_size, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    const int vec = dtype == 0 ? 4 : 8;           // elements of a 16-byte access
    if (rot > 0 && hd % vec == 0 && (rot / 2) % vec == 0 && aligned_to(16, qkv, cos_t, sin_t) && aligned_to(16, kpool, vpool)) {
        if (dtype == 0)
            rope_kv_write_vec_kernel<float><<<T, 256, 0, stream>>>((float*)qkv, (const int32_t*)positions, (const float*)cos_t,
                                                                   (const float*)sin_t, (const int32_t*)slot_mapping,
                                                                   (float*)kpool, (float*)vpool, H, KVH, hd, rot, page_size);
        else
            rope_kv_write_vec_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)qkv, (const int32_t*)positions,
                                                                    (const float*)cos_t, (const float*)sin_t,
                                                                    (const int32_t*)slot_mapping, (bf16_t*)kpool,
                                                                    (bf16_t*)vpool, H, KVH, hd, rot, page_size);
        return NI_LAUNCH_RESULT();
    }
    if (dtype == 0)
        rope_kv_write_kernel<float><<<T, 256, 0, stream>>>((float*)qkv, (const int32_t*)positions, (const float*)cos_t,
                                                           (const float*)sin_t, (const int32_t*)slot_mapping,
                                                           (float*)kpool, (float*)vpool, H, KVH, hd, rot, page_size);
    else
        rope_kv_write_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)qkv, (const int32_t*)positions,
                                                            (const float*)cos_t, (const float*)sin_t,
                                                            (const int32_t*)slot_mapping, (bf16_t*)kpool,
                                                            (bf16_t*)vpool, H, KVH, hd, rot, page_size);
    return NI_LAUNCH_RESULT();
}

NI_EXPORT int ni_swiglu(const void* gu, void* out, int T, int I, int dtype, hipStream_t stream) {
    size_t n = static_cast<size_t>(T) * I;
    if (n == 0) return 0;
    if (dtype == 0) {
        if (I % 4 == 0)
            swiglu_vec_kernel<float, 4><<<blocks_for(n / 4, 256), 256, 0, stream>>>((const float*)gu, (float*)out, I, n / 4);
        else
            swiglu_kernel<float><<<blocks_for(n, 256), 256, 0, stream>>>((const float*)gu, (float*)out, I, n);
    } else {
        if (I % 8 == 0)
            swiglu_vec_kernel<bf16_t, 8><<<blocks_for(n / 8, 256), 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, n / 8);
        else
            swiglu_kernel<bf16_t><<<blocks_for(n, 256), 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, n);
    }
    return NI_LAUNCH_RESULT();
}

// out[i] = mean + std * normal(key, start + i), i < count, in the output's type (see counter_normal).
NI_EXPORT int ni_random_normal(void* out, size_t count, uint64_t key, uint64_t start, float mean, float std, int dtype,
                               hipStream_t stream) {
    if (count == 0) return 0;
    const unsigned blocks = static_cast<unsigned>(std::min<size_t>((count + 255) / 256, 65536));
    if (dtype == 0)
        random_normal_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, count, key, start, mean, std);
    else
        random_normal_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, count, key, start, mean, std);
    return NI_LAUNCH_RESULT();
}
