// Skinny matrix products for decoding on gfx950: y[M, N] = x[M, K] . W[N, K]^T with M <= 64,
// where the time is the time to stream W from HBM once.
//
// One workgroup of 8 wavefronts owns NT tiles of 16 output columns.  Its wavefronts split K:
// wavefront w takes the 128-byte pieces w, w+8, ... of every row.  A piece is loaded straight
// from global memory in MFMA operand layout (lane l: row l%16 of the tile, 32 bytes at offset
// (l/16)*32 of the piece) and multiplied against the matching piece of x with
// v_mfma_f32_16x16x32_bf16 (two per piece) or v_mfma_f32_16x16x4_f32 (eight per piece): W is the
// A operand (rows = output columns n), x^T the B operand (columns = batch rows m), so each
// loaded byte of W is used for up to 16 rows of x per instruction, and M up to 64 costs four
// instructions per piece.  The MFMA's k index is only a label, so the same lane-to-k mapping on
// both operands is all that is required.  Partial sums meet in LDS.
//
// W comes either as stored, [N, K] row-major, or re-tiled once at load into the order this kernel
// reads it: [tile of 16 rows][128-byte piece][lane][32 bytes], zero-padded to whole tiles and
// pieces.  A wavefront's load is then 2 KB of consecutive memory instead of sixteen 128-byte
// runs 2*K bytes apart, which is worth about a third on the [2048, 8192] matrix.
//
// Epilogues: store (compute type or float32), or SwiGLU over paired tiles (tile 2j from the gate
// rows, tile 2j+1 from the up rows of a stacked [2I, K] matrix): out[m, n] = silu(g) * u; or
// rotation + cache write for a stacked [q; k; v] matrix: a workgroup owns the two tiles of one
// head that hold the partners (j, j + hd/2) of a rotation, turns them by the angle of the row's
// position, and stores query heads to a buffer, key and value heads straight into their pages.
// float32 inputs are multiplied in true float32 (no reduced-precision MFMA).
#include <type_traits>

#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

#define GV_WAVES 8
#define GV_THREADS (GV_WAVES * WAVE)

template <typename T> struct Piece;   // 32 bytes of one row, and the MFMAs that consume it
template <> struct Piece<bf16_t> {
    static constexpr int ELEMS = 16;          // per lane
    uint4 lo, hi;
    __device__ __forceinline__ void load(const bf16_t* p) {
        lo = reinterpret_cast<const uint4*>(p)[0];
        hi = reinterpret_cast<const uint4*>(p)[1];
    }
    __device__ __forceinline__ void zero() { lo = make_uint4(0, 0, 0, 0); hi = lo; }
    static __device__ __forceinline__ floatx4_t mma(const Piece& a, const Piece& b, floatx4_t c) {
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a.lo), __builtin_bit_cast(bf16x8_t, b.lo), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a.hi), __builtin_bit_cast(bf16x8_t, b.hi), c, 0, 0, 0);
        return c;
    }
};
template <> struct Piece<float> {
    static constexpr int ELEMS = 8;
    float v[8];
    __device__ __forceinline__ void load(const float* p) {
        float4 a = reinterpret_cast<const float4*>(p)[0], b = reinterpret_cast<const float4*>(p)[1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = 0.f;
    }
    static __device__ __forceinline__ floatx4_t mma(const Piece& a, const Piece& b, floatx4_t c) {
#pragma unroll
        for (int i = 0; i < 8; ++i) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[i], b.v[i], c, 0, 0, 0);
        return c;
    }
};

enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_ROPE = 2 };

// What the rotation epilogue needs beside the product.
struct RopeArgs {
    const int32_t* positions;      // [M]
    const float* cos_t;            // [max_pos, hd/2]
    const float* sin_t;
    const int32_t* slot_mapping;   // [M] page * page_size + slot, or null: keys and values are not stored
    void* kpool;                   // [pages, KVH, page_size, hd]
    void* vpool;
    int H, KVH, hd, page_size;
};

template <typename T, typename TOUT, int MB, int NT, int EPI, bool TILED>
__global__ __launch_bounds__(GV_THREADS) void skinny_gemm_kernel(const T* __restrict__ x, const T* __restrict__ W,
                                                                 TOUT* __restrict__ y, int M, int N, int K, int I,
                                                                 RopeArgs rope) {
    constexpr int EL = Piece<T>::ELEMS;
    constexpr int CH = 4 * EL;                       // k elements in a 128-byte piece of a row
    const int tid = threadIdx.x;
    const int wave = tid / WAVE, lane = tid % WAVE;
    const int r = lane % 16, kg = lane / 16;
    const int wg = blockIdx.x;

    // weight row that this lane reads in each tile; tiles may hang over the edge of the matrix, then
    // the row index is clamped (never read past W) and the result is not stored
    const int n_limit = (EPI == EPI_SWIGLU) ? I : N;
    const T* wrow[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int col0 = (EPI == EPI_SWIGLU) ? (wg * (NT / 2) + nt / 2) * 16 : (wg * NT + nt) * 16;
        if (EPI == EPI_ROPE) {      // workgroup = (head, pair of tiles): dims [16 p, 16 p + 16) and the same + hd/2
            const int per_head = rope.hd / 32;
            col0 = (wg / per_head) * rope.hd + (wg % per_head) * 16 + nt * (rope.hd / 2);
        }
        const int shift = (EPI == EPI_SWIGLU && (nt % 2)) ? I : 0;      // odd tiles of a pair come from the up rows
        if (TILED)      // first byte of this lane in piece 0 of the tile; the buffer is padded, nothing to clamp
            wrow[nt] = W + static_cast<size_t>((col0 + shift) / 16) * ((K + CH - 1) / CH) * (WAVE * EL) + lane * EL;
        else
            wrow[nt] = W + static_cast<size_t>(min(col0 + r, n_limit - 1) + shift) * K;
    }
    const T* xrow[MB];
    bool xok[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = mb * 16 + r;
        xok[mb] = m < M;
        xrow[mb] = x + static_cast<size_t>(min(m, M - 1)) * K;
    }

    floatx4_t acc[NT][MB];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[nt][mb] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // PT pieces per trip, all their loads issued before the first multiply, to keep enough bytes in
    // flight; the wavefront covers pieces [first + wave * per_wave, ...) of its K range in order.
    constexpr int PT = (NT * MB <= 2) ? 4 : 2;
    const int pieces = (K + CH - 1) / CH;
    for (int c = wave; c < pieces; c += PT * GV_WAVES) {
        Piece<T> xb[PT][MB], wa[PT][NT];
#pragma unroll
        for (int u = 0; u < PT; ++u) {
            const int piece = c + u * GV_WAVES;
            const int k = piece * CH + kg * EL;
            const bool kok = k < K;                  // K is a multiple of EL: a lane's 32 bytes are all in or all out
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if (TILED) {
                    if (piece < pieces) wa[u][nt].load(wrow[nt] + static_cast<size_t>(piece) * (WAVE * EL)); else wa[u][nt].zero();
                } else {
                    if (kok) wa[u][nt].load(wrow[nt] + k); else wa[u][nt].zero();
                }
            }
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                if (kok && xok[mb]) xb[u][mb].load(xrow[mb] + k); else xb[u][mb].zero();
            }
        }
#pragma unroll
        for (int u = 0; u < PT; ++u)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) acc[nt][mb] = Piece<T>::mma(wa[u][nt], xb[u][mb], acc[nt][mb]);
    }

    // partial sums of the wavefronts meet in LDS: red[wave][tile][lane * 4 + i]
    __shared__ float red[GV_WAVES][NT * MB][WAVE * 4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave][nt * MB + mb][lane * 4 + i] = acc[nt][mb][i];
    __syncthreads();

    // D[n_local][m_local] of a tile sits at lane = (n_local / 4) * 16 + m_local, register n_local % 4
    if constexpr (EPI == EPI_ROPE) {
        const int per_head = rope.hd / 32;
        const int head = wg / per_head;                 // among H query, KVH key, KVH value heads
        const int j0 = (wg % per_head) * 16;            // first of this workgroup's 16 pairs
        const int half = rope.hd / 2;
        for (int item = tid; item < MB * 16 * 16; item += GV_THREADS) {
            const int n_local = item % 16;
            const int m = item / 16;
            if (m >= M) continue;
            const int mb = m / 16, m_local = m % 16;
            const int src = ((n_local / 4) * 16 + m_local) * 4 + (n_local % 4);
            float x0 = 0.f, x1 = 0.f;
#pragma unroll
            for (int w = 0; w < GV_WAVES; ++w) {
                x0 += red[w][0 * MB + mb][src];
                x1 += red[w][1 * MB + mb][src];
            }
            const int j = j0 + n_local;
            if (head < rope.H + rope.KVH) {             // queries and keys turn, values do not
                const int pos = rope.positions[m];
                const float c = rope.cos_t[static_cast<size_t>(pos) * half + j];
                const float sn = rope.sin_t[static_cast<size_t>(pos) * half + j];
                const float y0 = x0 * c - x1 * sn;
                const float y1 = x0 * sn + x1 * c;
                x0 = y0; x1 = y1;
            }
            if (head < rope.H) {
                TOUT* dst = y + static_cast<size_t>(m) * rope.H * rope.hd + static_cast<size_t>(head) * rope.hd;
                st(dst + j, x0);
                st(dst + j + half, x1);
            } else if (rope.slot_mapping) {
                const int slot = rope.slot_mapping[m];
                if (slot >= 0) {
                    const bool is_k = head < rope.H + rope.KVH;
                    const int g = is_k ? head - rope.H : head - rope.H - rope.KVH;
                    TOUT* pool = static_cast<TOUT*>(is_k ? rope.kpool : rope.vpool);
                    TOUT* dst = pool + ((static_cast<size_t>(slot / rope.page_size) * rope.KVH + g) * rope.page_size +
                                        slot % rope.page_size) * rope.hd;
                    st(dst + j, x0);
                    st(dst + j + half, x1);
                }
            }
        }
        return;
    }
    constexpr int NOUT = (EPI == EPI_SWIGLU) ? NT / 2 : NT;      // output tiles of the workgroup
    const int out_n0 = wg * NOUT * 16;
    const int out_width = (EPI == EPI_SWIGLU) ? I : N;
    for (int item = tid; item < MB * 16 * NOUT * 16; item += GV_THREADS) {
        const int n_in = item % (NOUT * 16);
        const int m = item / (NOUT * 16);
        const int ot = n_in / 16, n_local = n_in % 16;
        const int mb = m / 16, m_local = m % 16;
        const int n = out_n0 + n_in;
        if (m >= M || n >= out_width) continue;
        const int src = ((n_local / 4) * 16 + m_local) * 4 + (n_local % 4);
        float v;
        if (EPI == EPI_SWIGLU) {
            float g = 0.f, u = 0.f;
#pragma unroll
            for (int w = 0; w < GV_WAVES; ++w) {
                g += red[w][(2 * ot) * MB + mb][src];
                u += red[w][(2 * ot + 1) * MB + mb][src];
            }
            v = g / (1.0f + expf(-g)) * u;
        } else {
            v = 0.f;
#pragma unroll
            for (int w = 0; w < GV_WAVES; ++w) v += red[w][ot * MB + mb][src];
        }
        st(y + static_cast<size_t>(m) * out_width + n, v);
    }
}

template <typename T, typename TOUT, int MB, int EPI>
static int launch_nt(const void* x, const void* W, void* y, int M, int N, int K, int I, int NT, bool tiled,
                     hipStream_t stream, RopeArgs rope = RopeArgs{}) {
    const int out_width = (EPI == EPI_SWIGLU) ? I : N;
    const int tiles = (out_width + 15) / 16;
    auto run = [&](auto nt_tag) {
        constexpr int NTc = decltype(nt_tag)::value;
        constexpr int NOUT = (EPI == EPI_SWIGLU) ? NTc / 2 : NTc;
        const int grid = (tiles + NOUT - 1) / NOUT;
        if (tiled)
            skinny_gemm_kernel<T, TOUT, MB, NTc, EPI, true><<<grid, GV_THREADS, 0, stream>>>((const T*)x, (const T*)W, (TOUT*)y, M, N, K, I, rope);
        else
            skinny_gemm_kernel<T, TOUT, MB, NTc, EPI, false><<<grid, GV_THREADS, 0, stream>>>((const T*)x, (const T*)W, (TOUT*)y, M, N, K, I, rope);
    };
    // NT * MB fragments of partial sums share 64 KB of LDS: at most 8
    if constexpr (MB <= 2 && EPI != EPI_ROPE) {
        if (NT >= 4) { run(std::integral_constant<int, 4>{}); return NI_LAUNCH_RESULT(); }
    }
    if constexpr (EPI == EPI_SWIGLU || EPI == EPI_ROPE) {
        run(std::integral_constant<int, 2>{});
    } else {
        if (NT >= 2) run(std::integral_constant<int, 2>{});
        else run(std::integral_constant<int, 1>{});
    }
    return NI_LAUNCH_RESULT();
}

template <typename T, typename TOUT, int EPI>
static int launch_mb(const void* x, const void* W, void* y, int M, int N, int K, int I, int NT, bool tiled,
                     hipStream_t stream, RopeArgs rope = RopeArgs{}) {
    if (M <= 16) return launch_nt<T, TOUT, 1, EPI>(x, W, y, M, N, K, I, NT, tiled, stream, rope);
    if (M <= 32) return launch_nt<T, TOUT, 2, EPI>(x, W, y, M, N, K, I, NT, tiled, stream, rope);
    return launch_nt<T, TOUT, 4, EPI>(x, W, y, M, N, K, I, NT, tiled, stream, rope);
}

// epilogue: 0 store in the input type, 1 store float32, 2 SwiGLU (W is [2I, K], y is [M, I]).
// K must be a multiple of 16 bytes' worth of elements x 2 (bf16: 16, f32: 8); M <= 64.
// tiled: W is in the re-tiled order described at the top (swiglu then needs N/2 to be a multiple of 16).
NI_EXPORT int ni_skinny_gemm(const void* x, const void* W, void* y, int M, int N, int K, int epilogue, int tiles_per_group,
                             int tiled, int dtype, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64) return -1;
    const int el = dtype == 0 ? 8 : 16;
    if (K % el != 0) return -2;
    const int I = N / 2;
    if (epilogue == 2 && (N % 2)) return -3;
    if (epilogue == 2 && tiled && (I % 16)) return -4;
    if (dtype == 0) {
        if (epilogue == 2) return launch_mb<float, float, EPI_SWIGLU>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream);
        return launch_mb<float, float, EPI_STORE>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream);
    }
    if (epilogue == 2) return launch_mb<bf16_t, bf16_t, EPI_SWIGLU>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream);
    if (epilogue == 1) return launch_mb<bf16_t, float, EPI_STORE>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream);
    return launch_mb<bf16_t, bf16_t, EPI_STORE>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream);
}

// Product with the stacked [q; k; v] matrix ((H + 2 KVH) * hd rows), rotation of query and key
// heads by the rows' positions, queries to q_out [M, H * hd], keys and values into the pools at
// slot_mapping (null: not stored).  hd must be a multiple of 32 and fully rotated.
NI_EXPORT int ni_skinny_qkv_rope(const void* x, const void* W, void* q_out, const void* positions, const void* cos_t,
                                 const void* sin_t, const void* slot_mapping, void* kpool, void* vpool, int M, int K,
                                 int H, int KVH, int hd, int page_size, int tiled, int dtype, hipStream_t stream) {
    if (M <= 0) return 0;
    if (M > 64) return -1;
    if (K % (dtype == 0 ? 8 : 16) != 0) return -2;
    if (hd % 32 != 0 || H <= 0 || KVH <= 0 || page_size < 1) return -3;
    RopeArgs rope{(const int32_t*)positions, (const float*)cos_t, (const float*)sin_t, (const int32_t*)slot_mapping,
                  kpool, vpool, H, KVH, hd, page_size};
    const int N = (H + 2 * KVH) * hd;
    // launch_nt sizes the grid from the output width: one workgroup per two tiles
    if (dtype == 0) return launch_mb<float, float, EPI_ROPE>(x, W, q_out, M, N, K, 0, 2, tiled != 0, stream, rope);
    return launch_mb<bf16_t, bf16_t, EPI_ROPE>(x, W, q_out, M, N, K, 0, 2, tiled != 0, stream, rope);
}
