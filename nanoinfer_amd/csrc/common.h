// Shared device helpers for the gfx950 kernels: element types, conversions and
// reductions over 64-lane wavefronts.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define WAVE 64

// bfloat16 is carried as its 16 raw bits; conversions are explicit so that rounding
// (to nearest, ties to even) is the same in every kernel.
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
    return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);  // NaN stays NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

// Two floats to two bfloat16 in one word (first argument in the low half) by the hardware's
// conversion, which rounds to nearest even like the routine above.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef __bf16 bf16x2_hw __attribute__((ext_vector_type(2)));
    typedef float floatx2_hw __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2_hw{lo, hi}, bf16x2_hw));
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static __device__ __forceinline__ float load(const float* p) { return *p; }
    static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Elem<bf16_t> {
    static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_bits_to_f32(p->bits); }
    static __device__ __forceinline__ void store(bf16_t* p, float v) { p->bits = f32_to_bf16_bits(v); }
};

template <typename T> __device__ __forceinline__ float ld(const T* p) { return Elem<T>::load(p); }
template <typename T> __device__ __forceinline__ void st(T* p, float v) { Elem<T>::store(p, v); }

// Load N consecutive elements as floats. The widest access that N and the element size
// allow is used; the caller guarantees that p is aligned to that access.
template <typename T, int N> struct VecIO;

template <int N> struct VecIO<float, N> {
    static __device__ __forceinline__ void load(const float* p, float* out) {
        if constexpr (N % 4 == 0) {
#pragma unroll
            for (int i = 0; i < N / 4; ++i) {
                float4 v = reinterpret_cast<const float4*>(p)[i];
                out[4 * i] = v.x; out[4 * i + 1] = v.y; out[4 * i + 2] = v.z; out[4 * i + 3] = v.w;
            }
        } else if constexpr (N % 2 == 0) {
#pragma unroll
            for (int i = 0; i < N / 2; ++i) {
                float2 v = reinterpret_cast<const float2*>(p)[i];
                out[2 * i] = v.x; out[2 * i + 1] = v.y;
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) out[i] = p[i];
        }
    }
    static __device__ __forceinline__ void store(float* p, const float* in) {
        if constexpr (N % 4 == 0) {
#pragma unroll
            for (int i = 0; i < N / 4; ++i)
                reinterpret_cast<float4*>(p)[i] = make_float4(in[4 * i], in[4 * i + 1], in[4 * i + 2], in[4 * i + 3]);
        } else if constexpr (N % 2 == 0) {
#pragma unroll
            for (int i = 0; i < N / 2; ++i) reinterpret_cast<float2*>(p)[i] = make_float2(in[2 * i], in[2 * i + 1]);
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) p[i] = in[i];
        }
    }
};

template <int N> struct VecIO<bf16_t, N> {
    static __device__ __forceinline__ void load(const bf16_t* p, float* out) {
        if constexpr (N % 8 == 0) {
#pragma unroll
            for (int i = 0; i < N / 8; ++i) {
                uint4 v = reinterpret_cast<const uint4*>(p)[i];
                uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    out[8 * i + 2 * j] = __uint_as_float(w[j] << 16);
                    out[8 * i + 2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
                }
            }
        } else if constexpr (N % 4 == 0) {
#pragma unroll
            for (int i = 0; i < N / 4; ++i) {
                uint2 v = reinterpret_cast<const uint2*>(p)[i];
                out[4 * i] = __uint_as_float(v.x << 16);
                out[4 * i + 1] = __uint_as_float(v.x & 0xffff0000u);
                out[4 * i + 2] = __uint_as_float(v.y << 16);
                out[4 * i + 3] = __uint_as_float(v.y & 0xffff0000u);
            }
        } else if constexpr (N % 2 == 0) {
#pragma unroll
            for (int i = 0; i < N / 2; ++i) {
                uint32_t v = reinterpret_cast<const uint32_t*>(p)[i];
                out[2 * i] = __uint_as_float(v << 16);
                out[2 * i + 1] = __uint_as_float(v & 0xffff0000u);
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) out[i] = bf16_bits_to_f32(p[i].bits);
        }
    }
    static __device__ __forceinline__ void store(bf16_t* p, const float* in) {
        if constexpr (N % 2 == 0) {
#pragma unroll
            for (int i = 0; i < N / 2; ++i) {
                uint32_t lo = f32_to_bf16_bits(in[2 * i]);
                uint32_t hi = f32_to_bf16_bits(in[2 * i + 1]);
                reinterpret_cast<uint32_t*>(p)[i] = lo | (hi << 16);
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) p[i].bits = f32_to_bf16_bits(in[i]);
        }
    }
};

// N consecutive elements (4 floats, or 4 or 8 bfloat16) stored from floats in one access of 8 or 16
// bytes; p is aligned to that access.  Rounding to bfloat16 is the hardware's, to nearest even.
template <typename T, int N> __device__ __forceinline__ void store_packed(T* p, const float* in) {
    typedef uint32_t u32x4_hw __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x2_hw __attribute__((ext_vector_type(2)));
    typedef float floatx4_hw __attribute__((ext_vector_type(4)));
    if constexpr (sizeof(T) == 4) {
        static_assert(N == 4, "four floats are 16 bytes");
        *reinterpret_cast<floatx4_hw*>(p) = floatx4_hw{in[0], in[1], in[2], in[3]};
    } else if constexpr (N == 8) {
        *reinterpret_cast<u32x4_hw*>(p) = u32x4_hw{pack_bf16x2(in[0], in[1]), pack_bf16x2(in[2], in[3]),
                                                   pack_bf16x2(in[4], in[5]), pack_bf16x2(in[6], in[7])};
    } else {
        static_assert(N == 4, "four or eight bfloat16");
        *reinterpret_cast<u32x2_hw*>(p) = u32x2_hw{pack_bf16x2(in[0], in[1]), pack_bf16x2(in[2], in[3])};
    }
}

// N consecutive elements kept as loaded (no conversion yet), so that rows waiting in registers
// for their turn cost as few registers as they cost bytes.
template <typename T, int N> struct RawRow {
    static constexpr int BYTES = N * sizeof(T);
    static constexpr int WORDS = (BYTES + 3) / 4;
    uint32_t w[WORDS];
    __device__ __forceinline__ void load(const T* p) {
        if constexpr (BYTES % 16 == 0) {
#pragma unroll
            for (int i = 0; i < BYTES / 16; ++i) {
                const uint4 v = reinterpret_cast<const uint4*>(p)[i];
                w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
            }
        } else if constexpr (BYTES % 8 == 0) {
#pragma unroll
            for (int i = 0; i < BYTES / 8; ++i) {
                const uint2 v = reinterpret_cast<const uint2*>(p)[i];
                w[2 * i] = v.x; w[2 * i + 1] = v.y;
            }
        } else if constexpr (BYTES % 4 == 0) {
#pragma unroll
            for (int i = 0; i < BYTES / 4; ++i) w[i] = reinterpret_cast<const uint32_t*>(p)[i];
        } else {      // an odd number of 16-bit elements
            const uint16_t* q = reinterpret_cast<const uint16_t*>(p);
#pragma unroll
            for (int i = 0; i < WORDS; ++i) {
                const uint32_t lo = q[2 * i];
                const uint32_t hi = (2 * i + 1 < N) ? q[2 * i + 1] : 0u;
                w[i] = lo | (hi << 16);
            }
        }
    }
    __device__ __forceinline__ float get(int i) const {
        if constexpr (sizeof(T) == 4) return __uint_as_float(w[i]);
        else return __uint_as_float((i & 1) ? (w[i / 2] & 0xffff0000u) : (w[i / 2] << 16));
    }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
    return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats of LDS and may be used again after the call returns.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const int nwaves = (blockDim.x + WAVE - 1) / WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int i = 0; i < nwaves; ++i) total += scratch[i];
    return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    v = wave_max(v);
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const int nwaves = (blockDim.x + WAVE - 1) / WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = scratch[0];
    for (int i = 1; i < nwaves; ++i) total = fmaxf(total, scratch[i]);
    return total;
}

#define NI_EXPORT extern "C" __attribute__((visibility("default")))

// Every entry point returns 0 or a hipError_t of the launch.
#define NI_LAUNCH_RESULT() static_cast<int>(hipGetLastError())
