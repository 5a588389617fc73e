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
// W comes either as stored, [N, K] row-major, or re-tiled once at load into the order the kernels
// read it: [tile of 16 rows][128-byte piece][lane][32 bytes], zero-padded to whole tiles and
// pieces.  A wavefront's load is then 2 KB of consecutive memory instead of sixteen 128-byte
// runs 2*K bytes apart, which is worth about a third on the [2048, 8192] matrix.  Three kernels:
// the first, described above, takes W as stored (any number of rows up to 64); the other two
// take it re-tiled, one for the decode step proper (at most 16 rows), one for 17 to 64 rows.
//
// Epilogues: store (compute type or float32), or SwiGLU over paired tiles (tile 2j from the gate
// rows, tile 2j+1 from the up rows of a stacked [2I, K] matrix): out[m, n] = silu(g) * u; or
// rotation + cache write for a stacked [q; k; v] matrix: a workgroup owns the two tiles of one
// head that hold the partners (j, j + hd/2) of a rotation, turns them by the angle of the row's
// position, and stores query heads to a buffer, key and value heads straight into their pages.
// or addition into the float32 residual stream (h[m, n] += the product, in place: a workgroup
// reads and writes only its own columns).
//
// The kernel of the decode step proper (at most 16 rows, re-tiled weights) keeps two
// trips in registers (one multiplied while the other's loads are under way), and can take, instead
// of x, the float32 residual stream h [M, K] with the weights and eps of an RMSNorm: every
// workgroup then normalises the rows itself (sums of squares over the wavefronts' K slices, met in
// LDS) while its first pieces of W are already on their way, and keeps the normalised operand in
// registers (K up to XP * 8 pieces).  With that prologue and the residual epilogue a block of a
// decoder needs no kernel of its own for the residual sum or the norm.  Both also take float32
// addends that h has not received yet (the shares of a product whose K range was cut to fill the
// chip): the prologue normalises h plus the addends, the next residual epilogue brings them into
// h with its own product, so the cut costs no kernel either.  The kernel for 17 to 64 rows brings
// x through LDS (see there).
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
    __device__ __forceinline__ void from_floats(const float (&f)[16]) {
        lo = make_uint4(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7]));
        hi = make_uint4(pack_bf16x2(f[8], f[9]), pack_bf16x2(f[10], f[11]), pack_bf16x2(f[12], f[13]), pack_bf16x2(f[14], f[15]));
    }
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
    __device__ __forceinline__ void from_floats(const float (&f)[8]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = f[i];
    }
    static __device__ __forceinline__ floatx4_t mma(const Piece& a, const Piece& b, floatx4_t c) {
#pragma unroll
        for (int i = 0; i < 8; ++i) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[i], b.v[i], c, 0, 0, 0);
        return c;
    }
};

enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_ROPE = 2, EPI_RESIDUAL = 3 };

// The normalising prologue's inputs.
struct NormArgs {
    const float* h;        // [M, K] residual stream
    const float* weight;   // [K]
    float eps;
    // for the merging prologue instead: partial results of an attention whose keys were cut into runs
    const float* part_o = nullptr;     // [M, heads, runs, hd]
    const float* part_ml = nullptr;    // [M, heads, runs, 2]: maximum (base e) and sum of each run
    int runs = 0, heads = 0, hd = 0;
    // Addends that the residual stream has not received yet (the shares of a product whose K range was cut):
    // float32 [n_pend, M, width of h].  The normalising prologue takes its rows as (h + pend[0]) + pend[1];
    // the residual epilogue stores ((h + pend[0]) + pend[1]) + product.  The kernel that normalises does not
    // write h, so between the two nothing has to be ordered.
    const float* pend = nullptr;
    int n_pend = 0;
};
#define PROLOGUE_ADDENDS_MAX 2        // addends the normalising prologue holds in registers beside its rows of h
#define PRO_NORM 0      // the prologue computes RMSNorm(h)
#define PRO_MERGE 1     // the prologue merges the key runs of an attention
#define MERGE_RUNS_MAX 16         // key runs the merging prologue takes for one row
#define MERGE_RUNS_OF(SR) ((SR) == 1 ? MERGE_RUNS_MAX : 32 / (SR))      // and for up to SR rows: 8 for 4, 4 for 8
#define MERGE_FACTORS_MAX 4096     // floats of LDS for the runs' weights: M * heads * (runs + 1) must fit

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

// A norm done in two halves by the products on either side of it.  RMSNorm(h) . W^T = ((h * w) . W^T) / rms(h) row by
// row, so the product that completes the residual stream (residual epilogue, `xn` set) also stores
// xn[m, n] = h[m, n] * w[n] in the compute type and the sum of h[m, n]^2 over its own columns, ss_out[m * parts + wg]
// (parts = its workgroups; past sixteen rows ss_out[m * parts + tile], parts = the tiles of all workgroups: there a
// tile's sums are one wavefront's, and need not meet another's); and the product behind the norm (`ss_in` set) takes
// xn for its x and multiplies its sums by 1 / sqrt(sum over the parts / width + eps) in its epilogue.  No kernel normalises and none reads h for it.
// The sums of squares are float32 of the float32 stream, added in a fixed order.
#define DEFER_PARTS_MAX 256       // sums of squares that the product behind the norm adds up for a row
struct DeferArgs {
    void* xn = nullptr;            // [M, N] compute type: the stream times the next norm's weight
    const float* w = nullptr;      // [N] that weight
    float* ss_out = nullptr;       // [M, parts]
    const float* ss_in = nullptr;  // [M, parts] of the product before
    int parts = 0;
    float eps = 0.f;
    int width = 0;                 // elements of a row of the stream
};

// The taking side: wavefront w adds up the rows w, w + WV, ... (lane l the parts l, l + 64, ...), asked for before the
// first trip of W and settled behind it, and leaves each row's factor in LDS for the epilogue.
template <int WV, int MAXROWS>
struct DeferTake {
    static constexpr int RPW = (MAXROWS + WV - 1) / WV;
    static constexpr int LPR = DEFER_PARTS_MAX / WAVE;
    float v[RPW][LPR];
    __device__ __forceinline__ void ask(const DeferArgs& d, int M, int wave, int lane) {
        if (d.ss_in == nullptr) return;
#pragma unroll
        for (int i = 0; i < RPW; ++i) {
            const int m = wave + i * WV;
#pragma unroll
            for (int j = 0; j < LPR; ++j) {
                const int part = lane + j * WAVE;
                v[i][j] = (m < M && part < d.parts) ? d.ss_in[static_cast<size_t>(m) * d.parts + part] : 0.f;
            }
        }
    }
    __device__ __forceinline__ void settle(const DeferArgs& d, int M, int wave, int lane, float* factors) {
        if (d.ss_in == nullptr) return;
#pragma unroll
        for (int i = 0; i < RPW; ++i) {
            const int m = wave + i * WV;
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < LPR; ++j) s += v[i][j];
#pragma unroll
            for (int off = WAVE / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, WAVE);
            if (lane == 0 && m < M) factors[m] = 1.0f / sqrtf(s / static_cast<float>(d.width) + d.eps);
        }
    }
};

// What an epilogue reads from memory, asked for while W is still streaming instead of at the end, where every
// load is a round trip that nothing hides (the rotation's are two in a row: the position, then its angle).
// For the first item of a thread (item == threadIdx.x), which with at most 16 rows and few tiles is its only one.
// Four consecutive elements from floats in one access (p aligned to it), each rounded as st() rounds it.
__device__ __forceinline__ void store_exact4(float* p, const float (&v)[4]) {
    *reinterpret_cast<floatx4_t*>(p) = floatx4_t{v[0], v[1], v[2], v[3]};
}
__device__ __forceinline__ void store_exact4(bf16_t* p, const float (&v)[4]) {
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    *reinterpret_cast<u32x2_t*>(p) =
        u32x2_t{static_cast<uint32_t>(f32_to_bf16_bits(v[0])) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16),
                static_cast<uint32_t>(f32_to_bf16_bits(v[2])) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16)};
}

struct EpiEarly {
    bool have = false;       // the values below are those of item threadIdx.x
    int pos = 0, slot = -1;  // rotation: the row's position and cache slot
    float a = 0.f, b = 0.f;  // rotation: cos and sin; residual: the stream's value and its first addend
    float c = 0.f;           // residual: the second addend
    float d = 1.f;           // residual: the next norm's weight at the thread's column, where the epilogue leaves h * w behind
};

// The first half for the rotation epilogue (position and slot of the thread's row), the whole for the residual one.
template <int EPI, int NT, int HALVES>
__device__ __forceinline__ void epi_early_first(EpiEarly& e, const void* y, int M, int N, const RopeArgs& rope,
                                                const float* pend, int n_pend, const float* next_w = nullptr) {
    const int item = threadIdx.x;
    const int wg = blockIdx.x / HALVES, wg_half = blockIdx.x % HALVES;
    if constexpr (EPI == EPI_ROPE) {
        const int n_local = item % 16, m = item / 16;
        if (item >= 16 * 16 || m >= M || (HALVES == 2 && (n_local >> 3) != wg_half)) return;
        e.have = true;
        e.pos = rope.positions[m];
        if (rope.slot_mapping) e.slot = rope.slot_mapping[m];
    } else if constexpr (EPI == EPI_RESIDUAL) {
        const int n_in = item % (NT * 16), m = item / (NT * 16);
        const int n = wg * NT * 16 + n_in;
        if (item >= 16 * NT * 16 || m >= M || n >= N || (HALVES == 2 && ((n_in % 16) >> 3) != wg_half)) return;
        e.have = true;
        const float* dst = static_cast<const float*>(y) + static_cast<size_t>(m) * N + n;
        e.a = *dst;
        if (next_w != nullptr) e.d = next_w[n];
        if (n_pend > 0) {
            const float* p = pend + static_cast<size_t>(m) * N + n;
            e.b = p[0];
            e.c = n_pend > 1 ? p[static_cast<size_t>(M) * N] : 0.f;
        }
    }
}
// The second half for the rotation epilogue, once the position has arrived: cos and sin of the thread's pair.
template <int EPI, int HALVES>
__device__ __forceinline__ void epi_early_second(EpiEarly& e, const RopeArgs& rope) {
    if constexpr (EPI == EPI_ROPE) {
        if (!e.have) return;
        const int wg = blockIdx.x / HALVES;
        const int per_head = rope.hd / 32;
        if (wg / per_head >= rope.H + rope.KVH) return;       // values do not turn
        const int j = (wg % per_head) * 16 + static_cast<int>(threadIdx.x) % 16;
        const size_t at = static_cast<size_t>(e.pos) * (rope.hd / 2) + j;
        e.a = rope.cos_t[at];
        e.b = rope.sin_t[at];
    }
}

// What follows the main loop of both kernels: the wavefronts' partial sums meet in LDS and the
// epilogue stores them.
// HALVES == 2: two workgroups share the tiles that one would own; the first stores the first eight
// columns of every tile, the second the others (each has multiplied only its own rows of W).
template <typename T, typename TOUT, int MB, int NT, int EPI, int WV = GV_WAVES, bool EXT = false, int HALVES = 1>
__device__ __forceinline__ void skinny_finish(const floatx4_t (&acc)[NT][MB], TOUT* __restrict__ y, int M, int N, int I,
                                              const RopeArgs& rope, float* ext = nullptr, const float* pend = nullptr,
                                              int n_pend = 0, const EpiEarly* early = nullptr,
                                              const DeferArgs& defer = DeferArgs{}, const float* factors = nullptr) {
    const int tid = threadIdx.x;
    const int wave = tid / WAVE, lane = tid % WAVE;
    const int wg = blockIdx.x / HALVES;
    const int wg_half = blockIdx.x % HALVES;      // which eight columns of every tile are this workgroup's
    // partial sums of the wavefronts meet in LDS: red[wave][tile][lane * 4 + i]; in memory of the
    // function's own, or (EXT) in memory the kernel has no other use for any more
    typedef float (*Red)[NT * MB][WAVE * 4];
    Red red;
    if constexpr (EXT) {
        red = reinterpret_cast<Red>(ext);
    } else {
        __shared__ float red_own[WV][NT * MB][WAVE * 4];
        red = red_own;
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave][nt * MB + mb][lane * 4 + i] = acc[nt][mb][i];
    __syncthreads();
    // the row's factor where the product stands behind a norm whose division it makes itself (1 otherwise)
    const bool scaled = EPI != EPI_RESIDUAL && factors != nullptr && defer.ss_in != nullptr;
    auto factor_of = [&](int m) { return scaled ? factors[m] : 1.0f; };

    // D[n_local][m_local] of a tile sits at lane = (n_local / 4) * 16 + m_local, register n_local % 4
    constexpr bool DEFERS = EPI == EPI_RESIDUAL;       // (decided at run time: defer.xn)
    if constexpr (MB >= 2 && EPI != EPI_ROPE) {
        // Several blocks of rows: the sums are taken in the layout of the accumulators, a thread adding up the four
        // registers of one lane of one tile over the wavefronts with 16-byte reads of neighbouring lanes (read item by
        // item, sixteen lanes of a wavefront would meet in the same few banks, and with four blocks of rows the
        // workgroup spent longer here than on a quarter of its matrix).  The four values are columns n0 .. n0 + 3 of row m;
        // a gate tile and its up tile are taken by the same thread.  (The rotation epilogue, 32 rows a workgroup, was
        // no faster this way and keeps the items below.)
        static_assert(HALVES == 1, "halved tiles come with one block of rows");
        if constexpr (DEFERS) {
            if (defer.xn != nullptr) {
                // The stream's new values and what the next norm needs of them (see DeferArgs): h * w in the compute
                // type, and of every tile its own sum of squares of each row, so that no wavefront has to meet another:
                // ss_out[m * parts + tile], parts = the tiles of all workgroups.  A row's sixteen columns of a tile are
                // the four values of the four lanes m % 16, + 16, + 32, + 48; every lane of a wavefront goes through the
                // same code (a lane without a row or a column adds zero and stores nothing).
                const int parts = static_cast<int>(gridDim.x) * NT;
                for (int q = tid; q < NT * MB * WAVE; q += WV * WAVE) {
                    const int ot = (q / WAVE) / MB, mb = (q / WAVE) % MB;
                    const int m = mb * 16 + lane % 16;
                    const int n0 = (wg * NT + ot) * 16 + (lane / 16) * 4;
                    floatx4_t a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int w = 0; w < WV; ++w) a += *reinterpret_cast<const floatx4_t*>(&red[w][ot * MB + mb][lane * 4]);
                    float sq = 0.f;
                    if (m < M && n0 < N) {
                        float* hd = reinterpret_cast<float*>(y) + static_cast<size_t>(m) * N + n0;
                        T* xd = static_cast<T*>(defer.xn) + static_cast<size_t>(m) * N + n0;
                        const bool whole = n0 + 3 < N && N % 4 == 0;      // four columns in one aligned access
                        float sum[4], wn[4];
                        if (whole) {
                            const floatx4_t h4 = *reinterpret_cast<const floatx4_t*>(hd);
                            const floatx4_t w4 = *reinterpret_cast<const floatx4_t*>(defer.w + n0);
#pragma unroll
                            for (int i = 0; i < 4; ++i) { sum[i] = h4[i]; wn[i] = w4[i]; }
                        } else {
#pragma unroll
                            for (int i = 0; i < 4; ++i) {
                                sum[i] = n0 + i < N ? hd[i] : 0.f;
                                wn[i] = n0 + i < N ? defer.w[n0 + i] : 0.f;
                            }
                        }
                        for (int p = 0; p < n_pend; ++p) {       // what the stream has not received yet, in its order
                            const float* ad = pend + static_cast<size_t>(p) * M * N + static_cast<size_t>(m) * N + n0;
#pragma unroll
                            for (int i = 0; i < 4; ++i) if (n0 + i < N) sum[i] += ad[i];
                        }
                        float xv[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            sum[i] += a[i];
                            xv[i] = sum[i] * wn[i];
                            if (n0 + i < N) sq += sum[i] * sum[i];
                        }
                        if (whole) {
                            *reinterpret_cast<floatx4_t*>(hd) = floatx4_t{sum[0], sum[1], sum[2], sum[3]};
                            store_exact4(xd, xv);
                        } else {
#pragma unroll
                            for (int i = 0; i < 4; ++i) if (n0 + i < N) { hd[i] = sum[i]; st(xd + i, xv[i]); }
                        }
                    }
                    sq += __shfl_xor(sq, 16, WAVE);
                    sq += __shfl_xor(sq, 32, WAVE);
                    // (a tile that lies past the matrix's last column still writes its part: zero)
                    if (lane < 16 && m < M) defer.ss_out[static_cast<size_t>(m) * parts + wg * NT + ot] = sq;
                }
                return;
            }
        }
        if (!(DEFERS && defer.xn != nullptr)) {
            constexpr bool PAIRS = EPI == EPI_SWIGLU;
            constexpr int OUT_T = PAIRS ? NT / 2 : NT;
            const int out_n0 = wg * OUT_T * 16;
            const int out_width = PAIRS ? I : N;
            for (int q = tid; q < OUT_T * MB * WAVE; q += WV * WAVE) {
                const int ot = (q / WAVE) / MB, mb = (q / WAVE) % MB;
                const int m = mb * 16 + lane % 16;
                const int n0 = out_n0 + ot * 16 + (lane / 16) * 4;      // first of the lane's four columns
                const int ta = (PAIRS ? 2 * ot : ot) * MB + mb;
                floatx4_t a = {0.f, 0.f, 0.f, 0.f}, b = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int w = 0; w < WV; ++w) {
                    a += *reinterpret_cast<const floatx4_t*>(&red[w][ta][lane * 4]);
                    if constexpr (PAIRS) b += *reinterpret_cast<const floatx4_t*>(&red[w][ta + MB][lane * 4]);
                }
                if (m >= M || n0 >= out_width) continue;
                if (scaled) {
                    const float f = factor_of(m);
#pragma unroll
                    for (int i = 0; i < 4; ++i) { a[i] *= f; b[i] *= f; }
                }
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if constexpr (PAIRS) v[i] = a[i] / (1.0f + expf(-a[i])) * b[i];
                    else v[i] = a[i];
                }
                TOUT* dst = y + static_cast<size_t>(m) * out_width + n0;
                const bool whole = n0 + 3 < out_width && out_width % 4 == 0;      // four columns in one aligned access
                if constexpr (EPI == EPI_RESIDUAL) {      // float32 residual stream, this workgroup's own columns
                    float* hd = reinterpret_cast<float*>(dst);
                    float sum[4];
                    if (whole) {
                        const floatx4_t h4 = *reinterpret_cast<const floatx4_t*>(hd);
#pragma unroll
                        for (int i = 0; i < 4; ++i) sum[i] = h4[i];
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) sum[i] = n0 + i < out_width ? hd[i] : 0.f;
                    }
                    // what the stream has not received yet, in its order, then the product
                    for (int p = 0; p < n_pend; ++p) {
                        const float* ad = pend + static_cast<size_t>(p) * M * N + static_cast<size_t>(m) * N + n0;
#pragma unroll
                        for (int i = 0; i < 4; ++i) if (n0 + i < out_width) sum[i] += ad[i];
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) sum[i] += v[i];
                    if (whole) {
                        *reinterpret_cast<floatx4_t*>(hd) = floatx4_t{sum[0], sum[1], sum[2], sum[3]};
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) if (n0 + i < out_width) hd[i] = sum[i];
                    }
                } else if (whole) {
                    store_exact4(dst, v);
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) if (n0 + i < out_width) st(dst + i, v[i]);
                }
            }
            return;
        }
    }
    if constexpr (EPI == EPI_ROPE) {
        const int per_head = rope.hd / 32;
        const int head = wg / per_head;                 // among H query, KVH key, KVH value heads
        const int j0 = (wg % per_head) * 16;            // first of this workgroup's 16 pairs
        const int half = rope.hd / 2;
        for (int item = tid; item < MB * 16 * 16; item += WV * WAVE) {
            const int n_local = item % 16;
            const int m = item / 16;
            if (m >= M || (HALVES == 2 && (n_local >> 3) != wg_half)) continue;
            const int mb = m / 16, m_local = m % 16;
            const int src = ((n_local / 4) * 16 + m_local) * 4 + (n_local % 4);
            float x0 = 0.f, x1 = 0.f;
#pragma unroll
            for (int w = 0; w < WV; ++w) {
                x0 += red[w][0 * MB + mb][src];
                x1 += red[w][1 * MB + mb][src];
            }
            if (scaled) { const float f = factor_of(m); x0 *= f; x1 *= f; }
            const int j = j0 + n_local;
            const bool ready = early != nullptr && early->have && item == tid;      // asked for while W was streaming
            if (head < rope.H + rope.KVH) {             // queries and keys turn, values do not
                float c, sn;
                if (ready) {
                    c = early->a; sn = early->b;
                } else {
                    const int pos = rope.positions[m];
                    c = rope.cos_t[static_cast<size_t>(pos) * half + j];
                    sn = rope.sin_t[static_cast<size_t>(pos) * half + j];
                }
                {
                    // two products and their difference or sum, each rounded on its own: left to itself the compiler
                    // fuses one product of each line into the addition in some instances of this function and the other
                    // in others, and the same rows then turn out a last bit apart from kernel to kernel
#pragma clang fp contract(off)
                    const float y0 = x0 * c - x1 * sn;
                    const float y1 = x0 * sn + x1 * c;
                    x0 = y0; x1 = y1;
                }
            }
            if (head < rope.H) {
                TOUT* dst = y + static_cast<size_t>(m) * rope.H * rope.hd + static_cast<size_t>(head) * rope.hd;
                st(dst + j, x0);
                st(dst + j + half, x1);
            } else if (rope.slot_mapping) {
                const int slot = ready ? early->slot : rope.slot_mapping[m];
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
    if constexpr (EPI == EPI_RESIDUAL) {
        if (defer.xn != nullptr) {
            // The stream's new values, and with them what the next norm needs of them: h * w in the compute type, and
            // the sum of squares of each row over this workgroup's columns.  The items of a row are ROWW neighbouring
            // lanes of one wavefront, which add their squares by shuffles: every lane of a wavefront that has items
            // goes through the same code (lanes without a row or a column add zero and store nothing).
            constexpr int ROWW = NT * 16;
            static_assert(ROWW <= WAVE && WAVE % ROWW == 0, "the items of a row lie within a wavefront");
            static_assert(HALVES == 1 || NT == 1, "halved tiles come one to a workgroup");
            const int parts = gridDim.x;          // with HALVES == 2 every half of a tile is a part of its own
            for (int base = 0; base < MB * 16 * ROWW; base += WV * WAVE) {
                const int item = base + tid;
                if (item - lane >= MB * 16 * ROWW) break;           // the whole wavefront is past the items
                const int n_in = item % ROWW, m = item / ROWW;
                const int ot = n_in / 16, n_local = n_in % 16;
                const int mb = m / 16, m_local = m % 16;
                const int n = out_n0 + n_in;
                const bool live = m < M && n < N && (HALVES == 1 || (n_local >> 3) == wg_half);
                float sq = 0.f;
                if (live) {
                    const int src = ((n_local / 4) * 16 + m_local) * 4 + (n_local % 4);
                    float v = 0.f;
#pragma unroll
                    for (int w = 0; w < WV; ++w) v += red[w][ot * MB + mb][src];
                    float* dst = reinterpret_cast<float*>(y) + static_cast<size_t>(m) * N + n;
                    const bool ready = early != nullptr && early->have && item == tid;
                    float sum = ready ? early->a : *dst;
                    const float wn = ready ? early->d : defer.w[n];
                    if (n_pend > 0) {
                        const float* p = pend + static_cast<size_t>(m) * N + n;
                        const size_t stride = static_cast<size_t>(M) * N;
                        float p0, p1;
                        if (ready) {
                            p0 = early->b; p1 = early->c;
                        } else {
                            p0 = p[0]; p1 = n_pend > 1 ? p[stride] : 0.f;
                        }
                        sum = (sum + p0) + p1;
                        for (int a = 2; a < n_pend; ++a) sum += p[a * stride];
                    }
                    const float hv = sum + v;
                    *dst = hv;
                    st(static_cast<T*>(defer.xn) + static_cast<size_t>(m) * N + n, hv * wn);
                    sq = hv * hv;
                }
#pragma unroll
                for (int off = ROWW / 2; off > 0; off >>= 1) sq += __shfl_xor(sq, off, WAVE);
                // (a half tile that lies past the matrix's last column still writes its part: zero)
                if (n_in == (HALVES == 2 ? wg_half * 8 : 0) && m < M)
                    defer.ss_out[static_cast<size_t>(m) * parts + blockIdx.x] = sq;
            }
            return;
        }
    }
    for (int item = tid; item < MB * 16 * NOUT * 16; item += WV * WAVE) {
        const int n_in = item % (NOUT * 16);
        const int m = item / (NOUT * 16);
        const int ot = n_in / 16, n_local = n_in % 16;
        const int mb = m / 16, m_local = m % 16;
        const int n = out_n0 + n_in;
        if (m >= M || n >= out_width || (HALVES == 2 && (n_local >> 3) != wg_half)) continue;
        const int src = ((n_local / 4) * 16 + m_local) * 4 + (n_local % 4);
        float v;
        if (EPI == EPI_SWIGLU) {
            float g = 0.f, u = 0.f;
#pragma unroll
            for (int w = 0; w < WV; ++w) {
                g += red[w][(2 * ot) * MB + mb][src];
                u += red[w][(2 * ot + 1) * MB + mb][src];
            }
            if (scaled) { const float f = factor_of(m); g *= f; u *= f; }
            v = g / (1.0f + expf(-g)) * u;
        } else {
            v = 0.f;
#pragma unroll
            for (int w = 0; w < WV; ++w) v += red[w][ot * MB + mb][src];
            if (scaled) v *= factor_of(m);
        }
        TOUT* dst = y + static_cast<size_t>(m) * out_width + n;
        if constexpr (EPI == EPI_RESIDUAL) {      // float32 residual stream, this workgroup's own columns
            const bool ready = early != nullptr && early->have && item == tid;      // asked for while W was streaming
            float sum = ready ? early->a : *dst;
            if (n_pend > 0) {       // what the stream has not received yet, in its order, then the product
                const float* p = pend + static_cast<size_t>(m) * N + n;
                const size_t stride = static_cast<size_t>(M) * N;
                float p0, p1;
                if (ready) {
                    p0 = early->b; p1 = early->c;
                } else {
                    p0 = p[0]; p1 = n_pend > 1 ? p[stride] : 0.f;      // asked for together
                }
                sum = (sum + p0) + p1;
                for (int a = 2; a < n_pend; ++a) sum += p[a * stride];
            }
            *dst = sum + v;
        } else {
            st(dst, v);
        }
    }
}

template <typename T, typename TOUT, int MB, int NT, int EPI>
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
                if (kok) wa[u][nt].load(wrow[nt] + k); else wa[u][nt].zero();
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

    skinny_finish<T, TOUT, MB, NT, EPI>(acc, y, M, N, I, rope);
}

// The decode step's kernel: at most 16 rows, W re-tiled (and zero-padded to whole pieces, so a lane
// past the end of a row multiplies by zero whatever it read of x).  XP == 0: x is given.
// XP > 0: x = RMSNorm(h) with the wavefront's XP pieces of the normalised row kept in registers.
// WV wavefronts split K: 8, or 16 for a matrix of few tiles and long rows, whose workgroups are too
// few to fill the chip and have to keep more loads in flight each.
// SR > 0 (with XP > 0): the prologue is staged through LDS for up to SR rows.  A vector load costs
// the texture path the same time whatever it fetches, and the operand layout spreads a row over
// few lanes: read in that layout, h and the norm's weights take twice the load instructions of W
// itself.  Staged, the workgroup reads every element once with full loads, normalises, rounds, and
// leaves the rows in LDS, from where the lanes pick their operands.
// HALVES == 2: a matrix of few tiles is streamed by twice the workgroups, each taking eight of a
// tile's sixteen rows (the lanes of the other eight load the same rows again, which costs no
// memory traffic, and their columns of the product are not stored).  A compute unit alone draws
// about 37 GB/s from memory, so a launch of fewer workgroups than compute units cannot stream at
// the chip's rate.
// PEND (staged normalising prologue only): h comes with addends it has not received yet, which the prologue
// adds to its rows.  A kernel of its own, because the addends wait in registers beside the rows of h while the
// first pieces of W are asked for: for eight rows that is 172 registers instead of 120, one workgroup a compute
// unit instead of two, which the products without addends should not pay.
template <typename T, typename TOUT, int NT, int EPI, int XP, int WV, int SR, int HALVES = 1, int PRO = PRO_NORM, bool PEND = false>
__global__ __launch_bounds__(WV * WAVE) void skinny_decode_kernel(const T* __restrict__ x, const T* __restrict__ W,
                                                                   TOUT* __restrict__ y, int M, int N, int K, int I,
                                                                   RopeArgs rope, NormArgs norm, int splits, DeferArgs defer) {
    constexpr int EL = Piece<T>::ELEMS;
    constexpr int CH = 4 * EL;
    __shared__ float factors[16];      // of the rows, where the product makes the division of the norm before it
    // The rows that a staged prologue leaves in LDS are dead once every wavefront has picked its operands
    // from them; where they are large enough, the partial sums of the end take their memory (float32 rows
    // of 2,048 elements for eight rows are 66 KB: with the sums beside them one workgroup would fill a
    // compute unit's LDS, sharing the memory two fit).
    constexpr int STAGED_ROW = XP * WV * CH + 16 / static_cast<int>(sizeof(T));
    constexpr int STAGED_BYTES = (XP > 0 && SR > 0) ? SR * STAGED_ROW * static_cast<int>(sizeof(T)) : 0;
    constexpr int SUMS_BYTES = WV * NT * WAVE * 4 * static_cast<int>(sizeof(float));
    constexpr bool SHARE_LDS = STAGED_BYTES >= SUMS_BYTES;
    __shared__ __attribute__((aligned(16))) unsigned char staged_rows[STAGED_BYTES > 0 ? STAGED_BYTES : 16];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;      // the same in every lane: say so
    const int r = lane % 16, kg = lane / 16;
    const int wg = blockIdx.x / HALVES;
    // the lane of the re-tiled matrix that this lane reads: its own, or with HALVES == 2 the one of this
    // workgroup's half that has the same row modulo eight
    const int wlane = HALVES == 1 ? lane : kg * 16 + ((r & 7) | (static_cast<int>(blockIdx.x % HALVES) << 3));
    const int pieces = (K + CH - 1) / CH;
    // with splits > 1 (no prologue) workgroup (x, y) multiplies the y-th share of the pieces and stores its sums in the y-th [M, N] of y
    const int share = (pieces + splits - 1) / splits;
    const int p_begin = min(pieces, static_cast<int>(blockIdx.y) * share), p_end = min(pieces, p_begin + share);
    y += static_cast<size_t>(blockIdx.y) * M * N;
    EpiEarly early;         // what the epilogue will read, asked for before W (not behind the merging prologue's many
                            // loads, where it gained nothing: the o product of one row 6.6 -> 7.3 us)
    if constexpr (PRO == PRO_NORM) epi_early_first<EPI, NT, HALVES>(early, y, M, N, rope, norm.pend, norm.n_pend, defer.w);

    const T* wrow[NT];      // first byte of this lane in piece 0 of each tile
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int col0 = (EPI == EPI_SWIGLU) ? (wg * (NT / 2) + nt / 2) * 16 : (wg * NT + nt) * 16;
        if (EPI == EPI_ROPE) {
            const int per_head = rope.hd / 32;
            col0 = (wg / per_head) * rope.hd + (wg % per_head) * 16 + nt * (rope.hd / 2);
        }
        const int shift = (EPI == EPI_SWIGLU && (nt % 2)) ? I : 0;
        const int limit = (N + 15) / 16 - 1;         // a workgroup's last tiles may lie past the matrix: read the last one, store nothing
        wrow[nt] = W + static_cast<size_t>(min((col0 + shift) / 16, limit)) * pieces * (WAVE * EL) + wlane * EL;
    }

    floatx4_t acc[NT][1];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt][0] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // PT pieces per trip; trip t of a wavefront covers pieces wave + (t * PT + u) * 8.  Two trips are
    // in registers at a time, in two fixed sets (A and B): one is multiplied while the other's loads
    // are under way.
    // sixteen wavefronts have half the registers each; and the stacked gate/up matrix, whose tiles make two workgroups
    // or more for every compute unit, streams faster with the smaller set of registers, which lets a unit hold more of
    // them (measured at [16384, 2048]: 15.9 -> 15.3 us at eight rows with the normalising prologue, 15.2 -> 13.7 without)
    constexpr int PT = (NT <= 2 && WV <= 8 && EPI != EPI_SWIGLU) ? 4 : 2;
    constexpr int STRIDE = PT * WV;
    auto load_w = [&](int c, Piece<T> (&wa)[PT][NT]) {
#pragma unroll
        for (int u = 0; u < PT; ++u) {
            const int piece = min(c + u * WV, p_end - 1);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) wa[u][nt].load(wrow[nt] + static_cast<size_t>(piece) * (WAVE * EL));
        }
    };
    auto multiply = [&](int c, const Piece<T> (&wa)[PT][NT], const Piece<T> (&xb)[PT][1]) {
#pragma unroll
        for (int u = 0; u < PT; ++u) {
            if (c + u * WV < p_end) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc[nt][0] = Piece<T>::mma(wa[u][nt], xb[u][0], acc[nt][0]);
            }
        }
    };

    Piece<T> wa_a[PT][NT], wa_b[PT][NT];
    const int row = min(r, M - 1);       // columns of rows that do not exist are computed from the last row and not stored
    if constexpr (XP > 0) {
        // Normalising prologue: this lane's elements of its row of h for every piece of the wavefront
        // and the norm's weights at the same places are asked for first, the first trip of W right
        // behind them.  Loads come back in the order they were issued, so the small ones (cache hits)
        // arrive while W is still on its way from HBM, and the sum of squares, its meeting over lanes
        // and wavefronts in LDS and the rounding of (h * weight) * inv to the operand type all happen
        // under the shadow of W.  Lanes whose row does not exist load and compute nothing.
        constexpr int TRIPS = XP / PT;
        static_assert(XP % PT == 0, "whole trips");
        Piece<T> xn[TRIPS][PT][1];
        if constexpr (SR > 0) {
            constexpr int THREADS = WV * WAVE;
            constexpr int KMAX = XP * WV * CH;                 // elements of a row that the compiled size covers
            constexpr int QPT = (KMAX / 4 + THREADS - 1) / THREADS;      // groups of four columns per thread
            constexpr int XROW = KMAX + 16 / sizeof(T);        // 16 bytes of padding: rows start on different banks
            static_assert(XROW == STAGED_ROW, "the staged rows are sized at the top of the kernel");
            T (*xs)[XROW] = reinterpret_cast<T (*)[XROW]>(staged_rows);
            if constexpr (PRO == PRO_MERGE) {
                // x is the output of an attention whose keys were cut into runs: row m, head h is
                // sum_s o[m,h,s,:] * w_s / sum_s l[m,h,s] * w_s with w_s = exp(max[m,h,s] - max over s), as the
                // merge kernel computes it.  The (maximum, sum) pairs are asked for first and the first trip
                // of W right behind them; the weights of the runs meet in LDS, then every thread merges four
                // columns of every row.
                __shared__ float fs[MERGE_FACTORS_MAX];
                constexpr bool FAST = sizeof(T) == 2;
                constexpr int RC = MERGE_RUNS_OF(SR);      // runs whose pieces a thread can hold for all SR rows
                static_assert(QPT == 1, "a thread merges one group of four columns");
                const int runs = norm.runs, stride = runs + 1;
                const int items = M * norm.heads;
                constexpr int IPT = (SR * 128 + THREADS - 1) / THREADS;       // (row, head) items a thread may own
                // everything the prologue reads is asked for before W, so that it is there while W is on its way
                float2 ml[IPT][RC];
#pragma unroll
                for (int i = 0; i < IPT; ++i) {
                    const int item = tid + i * THREADS;
#pragma unroll
                    for (int sp = 0; sp < RC; ++sp)
                        ml[i][sp] = (item < items && sp < runs)
                                        ? *reinterpret_cast<const float2*>(norm.part_ml + (static_cast<size_t>(item) * runs + sp) * 2)
                                        : make_float2(-1.0e30f, 0.f);
                }
                const int k = 4 * tid;
                const int head = min(k, K - 4) / norm.hd, dim = min(k, K - 4) % norm.hd;
                float4 v[SR][RC];
#pragma unroll
                for (int m = 0; m < SR; ++m)
#pragma unroll
                    for (int sp = 0; sp < RC; ++sp) {
                        const size_t at = (static_cast<size_t>(m * norm.heads + head) * runs + sp) * norm.hd + dim;
                        v[m][sp] = (k < K && m < M && sp < runs) ? *reinterpret_cast<const float4*>(norm.part_o + at)
                                                                 : make_float4(0.f, 0.f, 0.f, 0.f);
                    }
                __builtin_amdgcn_sched_barrier(0);
                load_w(wave, wa_a);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < IPT; ++i) {
                    const int item = tid + i * THREADS;
                    float run_max = -1.0e30f;
#pragma unroll
                    for (int sp = 0; sp < RC; ++sp) run_max = fmaxf(run_max, ml[i][sp].x);
                    float total = 0.f;
#pragma unroll
                    for (int sp = 0; sp < RC; ++sp) {
                        const float f = FAST ? __expf(ml[i][sp].x - run_max) : expf(ml[i][sp].x - run_max);
                        total += ml[i][sp].y * f;             // runs that do not exist have sum 0
                        if (item < items && sp < runs) fs[item * stride + sp] = f;
                    }
                    if (item < items) fs[item * stride + runs] = total;
                }
                __syncthreads();
                if (k < K) {
#pragma unroll
                    for (int m = 0; m < SR; ++m) {
                        if (m < M) {
                            const float* w = fs + (m * norm.heads + head) * stride;
                            float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                            for (int sp = 0; sp < RC; ++sp) {
                                const float f = sp < runs ? w[sp] : 0.f;
                                o[0] += v[m][sp].x * f; o[1] += v[m][sp].y * f; o[2] += v[m][sp].z * f; o[3] += v[m][sp].w * f;
                            }
                            const float total = w[runs];
                            const float f4[4] = {o[0] / total, o[1] / total, o[2] / total, o[3] / total};
                            VecIO<T, 4>::store(&xs[m][k], f4);
                        }
                    }
                }
            } else {
            __shared__ float ssum[WV][SR];
            __shared__ float sinv[SR];
            float4 hv[SR][QPT], wv[QPT];
#pragma unroll
            for (int q = 0; q < QPT; ++q) {
                const int k = 4 * (tid + q * THREADS);
                const bool in = k < K;
                wv[q] = in ? *reinterpret_cast<const float4*>(norm.weight + k) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int m = 0; m < SR; ++m)
                    hv[m][q] = (m < M && in) ? *reinterpret_cast<const float4*>(norm.h + static_cast<size_t>(m) * K + k)
                                             : make_float4(0.f, 0.f, 0.f, 0.f);
            }
            if constexpr (PEND) {
                // addends that h has not received yet: asked for with the rows, added in their order
                float4 pv[PROLOGUE_ADDENDS_MAX][SR][QPT];
#pragma unroll
                for (int a = 0; a < PROLOGUE_ADDENDS_MAX; ++a)
#pragma unroll
                    for (int q = 0; q < QPT; ++q) {
                        const int k = 4 * (tid + q * THREADS);
#pragma unroll
                        for (int m = 0; m < SR; ++m)
                            pv[a][m][q] = (a < norm.n_pend && m < M && k < K)
                                              ? *reinterpret_cast<const float4*>(norm.pend + (static_cast<size_t>(a) * M + m) * K + k)
                                              : make_float4(0.f, 0.f, 0.f, 0.f);
                    }
                __builtin_amdgcn_sched_barrier(0);
                load_w(wave, wa_a);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int a = 0; a < PROLOGUE_ADDENDS_MAX; ++a)
#pragma unroll
                    for (int m = 0; m < SR; ++m)
#pragma unroll
                        for (int q = 0; q < QPT; ++q) {
                            hv[m][q].x += pv[a][m][q].x; hv[m][q].y += pv[a][m][q].y;
                            hv[m][q].z += pv[a][m][q].z; hv[m][q].w += pv[a][m][q].w;
                        }
            } else {
                // loads come back in the order they went out: the few of the prologue first, W right behind
                __builtin_amdgcn_sched_barrier(0);
                load_w(wave, wa_a);
                __builtin_amdgcn_sched_barrier(0);
            }
            // all SR rows go through the same straight code (rows that do not exist are zeros): the
            // reductions of the rows then overlap instead of waiting for one another behind branches
            float ss[SR];
#pragma unroll
            for (int m = 0; m < SR; ++m) {
                ss[m] = 0.f;
#pragma unroll
                for (int q = 0; q < QPT; ++q)
                    ss[m] += hv[m][q].x * hv[m][q].x + hv[m][q].y * hv[m][q].y + hv[m][q].z * hv[m][q].z + hv[m][q].w * hv[m][q].w;
            }
#pragma unroll
            for (int off = WAVE / 2; off > 0; off >>= 1)
#pragma unroll
                for (int m = 0; m < SR; ++m) ss[m] += __shfl_xor(ss[m], off, WAVE);
            if (lane < SR) {
                float mine = ss[0];
#pragma unroll
                for (int m = 1; m < SR; ++m) mine = lane == m ? ss[m] : mine;
                ssum[wave][lane] = mine;
            }
            __syncthreads();
            if (tid < SR) {
                float total = 0.f;
#pragma unroll
                for (int w = 0; w < WV; ++w) total += ssum[w][tid];
                sinv[tid] = 1.0f / sqrtf(total / static_cast<float>(K) + norm.eps);
            }
            __syncthreads();
#pragma unroll
            for (int q = 0; q < QPT; ++q) {
                const int k = 4 * (tid + q * THREADS);
                if (k < K) {
#pragma unroll
                    for (int m = 0; m < SR; ++m) {
                        const float inv = sinv[m];
                        const float f[4] = {(hv[m][q].x * inv) * wv[q].x, (hv[m][q].y * inv) * wv[q].y,
                                            (hv[m][q].z * inv) * wv[q].z, (hv[m][q].w * inv) * wv[q].w};
                        VecIO<T, 4>::store(&xs[m][k], f);
                    }
                }
            }
            }
            __syncthreads();
#pragma unroll
            for (int p = 0; p < XP; ++p)
                xn[p / PT][p % PT][0].load(&xs[row][min((wave + p * WV) * CH + kg * EL, K - EL)]);
        } else {
            const float* hrow = norm.h + static_cast<size_t>(row) * K;
            const bool live = r < M;
            constexpr bool KEEP = XP * EL <= 64;        // the row's elements wait in registers, or are read a second time
            float4 hraw[XP][EL / 4], wraw[KEEP ? XP : 1][EL / 4];
            if (live) {
#pragma unroll
                for (int p = 0; p < XP; ++p) {
                    const int kc = min((wave + p * WV) * CH + kg * EL, K - EL);
#pragma unroll
                    for (int e = 0; e < EL / 4; ++e) {
                        hraw[p][e] = *reinterpret_cast<const float4*>(hrow + kc + 4 * e);
                        if constexpr (KEEP) wraw[p][e] = *reinterpret_cast<const float4*>(norm.weight + kc + 4 * e);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            load_w(wave, wa_a);
            __builtin_amdgcn_sched_barrier(0);
            float ss = 0.f;
            if (live) {
#pragma unroll
                for (int p = 0; p < XP; ++p) {
                    const int k = (wave + p * WV) * CH + kg * EL;
                    float part = 0.f;
#pragma unroll
                    for (int e = 0; e < EL / 4; ++e) {
                        const float4 v = hraw[p][e];
                        part += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
                    }
                    ss += k < K ? part : 0.f;
                }
            }
            ss += __shfl_xor(ss, 16, WAVE);
            ss += __shfl_xor(ss, 32, WAVE);
            __shared__ float ssum[WV][16];
            if (kg == 0) ssum[wave][r] = ss;
            __syncthreads();
            float total = 0.f;
#pragma unroll
            for (int w = 0; w < WV; ++w) total += ssum[w][r];
            const float inv = 1.0f / sqrtf(total / static_cast<float>(K) + norm.eps);
#pragma unroll
            for (int p = 0; p < XP; ++p) {
                float f[EL];
                const int kc = min((wave + p * WV) * CH + kg * EL, K - EL);
#pragma unroll
                for (int e = 0; e < EL / 4; ++e) {
                    float4 v = make_float4(0.f, 0.f, 0.f, 0.f), wv = v;
                    if constexpr (KEEP) {
                        if (live) { v = hraw[p][e]; wv = wraw[p][e]; }
                    } else if (live) {
                        v = *reinterpret_cast<const float4*>(hrow + kc + 4 * e);
                        wv = *reinterpret_cast<const float4*>(norm.weight + kc + 4 * e);
                    }
                    f[4 * e] = (v.x * inv) * wv.x; f[4 * e + 1] = (v.y * inv) * wv.y;
                    f[4 * e + 2] = (v.z * inv) * wv.z; f[4 * e + 3] = (v.w * inv) * wv.w;
                }
                xn[p / PT][p % PT][0].from_floats(f);
            }
        }
        epi_early_second<EPI, HALVES>(early, rope);      // behind the first trip of W; the position has arrived long ago
#pragma unroll
        for (int t = 0; t < TRIPS; t += 2) {
            const int c = wave + t * STRIDE;
            if (t + 1 < TRIPS && c + STRIDE < pieces) load_w(c + STRIDE, wa_b);
            multiply(c, wa_a, xn[t]);
            if (t + 2 < TRIPS && c + 2 * STRIDE < pieces) load_w(c + 2 * STRIDE, wa_a);
            if (t + 1 < TRIPS) multiply(c + STRIDE, wa_b, xn[t + 1 < TRIPS ? t + 1 : t]);
        }
    } else {
        DeferTake<WV, 16> take;
        if constexpr (EPI != EPI_RESIDUAL) take.ask(defer, M, wave, lane);      // a few cache hits, ahead of W
        load_w(p_begin + wave, wa_a);
        const T* xrow = x + static_cast<size_t>(row) * K;
        auto load_x = [&](int c, Piece<T> (&xb)[PT][1]) {
#pragma unroll
            for (int u = 0; u < PT; ++u) xb[u][0].load(xrow + min((c + u * WV) * CH + kg * EL, K - EL));
        };
        Piece<T> xb_a[PT][1], xb_b[PT][1];
        load_x(p_begin + wave, xb_a);
        epi_early_second<EPI, HALVES>(early, rope);      // behind the first trip of W and x (waits for the position only)
        if constexpr (EPI != EPI_RESIDUAL) take.settle(defer, M, wave, lane, factors);
        for (int c = p_begin + wave; c < p_end; c += 2 * STRIDE) {
            if (c + STRIDE < p_end) { load_w(c + STRIDE, wa_b); load_x(c + STRIDE, xb_b); }
            multiply(c, wa_a, xb_a);
            if (c + 2 * STRIDE < p_end) { load_w(c + 2 * STRIDE, wa_a); load_x(c + 2 * STRIDE, xb_a); }
            multiply(c + STRIDE, wa_b, xb_b);
        }
    }
    if constexpr (SHARE_LDS) {
        __syncthreads();                   // every wavefront has taken its operands from the staged rows
        skinny_finish<T, TOUT, 1, NT, EPI, WV, true, HALVES>(acc, y, M, N, I, rope, reinterpret_cast<float*>(staged_rows),
                                                             norm.pend, norm.n_pend, &early, defer, factors);
    } else {
        skinny_finish<T, TOUT, 1, NT, EPI, WV, false, HALVES>(acc, y, M, N, I, rope, nullptr, norm.pend, norm.n_pend, &early,
                                                              defer, factors);
    }
}

// 17 to 64 rows with re-tiled W.  The operand layout spreads a row of x over few lanes, so loaded
// in that layout four blocks of rows cost the texture path twice the instructions of W itself (a
// vector load takes it the same time whatever it fetches).  Here a wavefront brings the rows of x
// that belong to its piece of K into LDS with full 16-byte loads of neighbouring lanes (eight
// lanes a row), a slab of its own that needs no workgroup barrier, and picks the operands of all
// its row blocks from there.  Two trips are in registers at a time, in two fixed sets, as in the
// decode kernel.  The slabs' memory takes the partial sums at the end.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));    // 16 bytes that only pass through registers
#define SLAB_ROW 144      // bytes: a 128-byte piece of a row and 16 of padding, so that the rows of a read fall on different banks

template <typename T, typename TOUT, int MB, int NT, int EPI>
__global__ __launch_bounds__(GV_THREADS) void skinny_rows_kernel(const T* __restrict__ x, const T* __restrict__ W,
                                                                 TOUT* __restrict__ y, int M, int N, int K, int I,
                                                                 RopeArgs rope, int splits, DeferArgs defer) {
    constexpr int EL = Piece<T>::ELEMS;
    constexpr int CH = 4 * EL;
    constexpr int WV = GV_WAVES;
    constexpr int ROWS = MB * 16;
    __shared__ float factors[ROWS];    // of the rows, where the product makes the division of the norm before it
    constexpr int XL = ROWS / 8;                       // 16-byte loads of a lane for one piece of all rows
    constexpr int SLAB = ROWS * SLAB_ROW;
    constexpr int RED = NT * MB * WAVE * 4 * static_cast<int>(sizeof(float));
    __shared__ __attribute__((aligned(16))) unsigned char lds[WV * (SLAB > RED ? SLAB : RED)];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;      // the same in every lane: say so
    const int r = lane % 16, kg = lane / 16;
    const int wg = blockIdx.x;
    const int pieces = (K + CH - 1) / CH;
    // with splits > 1 workgroup (x, y) multiplies the y-th share of the pieces and stores its sums in the y-th [M, N] of y
    const int share = (pieces + splits - 1) / splits;
    const int p_begin = min(pieces, static_cast<int>(blockIdx.y) * share), p_end = min(pieces, p_begin + share);
    y += static_cast<size_t>(blockIdx.y) * M * N;
    if constexpr (EPI == EPI_ROPE) {
        // the rows may be dealt out to several workgroups (blockIdx.z), ROWS each: a workgroup then brings
        // only its own rows of x into LDS, which is most of what it loads when the matrix has few tiles
        const int row0 = static_cast<int>(blockIdx.z) * ROWS;
        x += static_cast<size_t>(row0) * K;
        y += static_cast<size_t>(row0) * rope.H * rope.hd;
        rope.positions += row0;
        if (rope.slot_mapping) rope.slot_mapping += row0;
        if (defer.ss_in != nullptr) defer.ss_in += static_cast<size_t>(row0) * defer.parts;
        M = min(M - row0, ROWS);
    }
    unsigned char* slab = lds + wave * SLAB;

    const T* wrow[NT];      // first byte of this lane in piece 0 of each tile
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int col0 = (EPI == EPI_SWIGLU) ? (wg * (NT / 2) + nt / 2) * 16 : (wg * NT + nt) * 16;
        if (EPI == EPI_ROPE) {
            const int per_head = rope.hd / 32;
            col0 = (wg / per_head) * rope.hd + (wg % per_head) * 16 + nt * (rope.hd / 2);
        }
        const int shift = (EPI == EPI_SWIGLU && (nt % 2)) ? I : 0;
        const int limit = (N + 15) / 16 - 1;         // a workgroup's last tiles may lie past the matrix: read the last one, store nothing
        wrow[nt] = W + static_cast<size_t>(min((col0 + shift) / 16, limit)) * pieces * (WAVE * EL) + lane * EL;
    }
    floatx4_t acc[NT][MB];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[nt][mb] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // pieces past the end of a row are read from its last piece and not multiplied: no load is under a branch
    auto load_w = [&](int c, Piece<T> (&wa)[NT]) {
        const int piece = min(c, p_end - 1);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) wa[nt].load(wrow[nt] + static_cast<size_t>(piece) * (WAVE * EL));
    };
    // x: lane l takes 16 bytes number l % 8 of the piece, of rows l / 8, l / 8 + 8, ...  (rows that do
    // not exist read the last row; their columns are not stored).  K is a multiple of 32 bytes'
    // worth of elements, so 16 bytes lie wholly inside a row or wholly past its end (then zeros:
    // W is zero there, but zero times what lies behind x need not be)
    constexpr int PER16 = 16 / static_cast<int>(sizeof(T));
    auto load_x = [&](int c, u32x4_t (&xr)[XL]) {
        const int k = min(c, p_end - 1) * CH + (lane % 8) * PER16;
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int row = min(i * 8 + lane / 8, M - 1);
            const u32x4_t v = *reinterpret_cast<const u32x4_t*>(x + static_cast<size_t>(row) * K + min(k, K - PER16));
            xr[i] = k < K ? v : u32x4_t{0u, 0u, 0u, 0u};
        }
    };
    auto stage = [&](const u32x4_t (&xr)[XL]) {
#pragma unroll
        for (int i = 0; i < XL; ++i)
            *reinterpret_cast<u32x4_t*>(slab + (i * 8 + lane / 8) * SLAB_ROW + (lane % 8) * 16) = xr[i];
    };
    // the lanes of one wavefront run together: ordering its own LDS writes and reads takes no barrier
    auto wave_sync = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    auto multiply = [&](const Piece<T> (&wa)[NT]) {
        Piece<T> xb[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) xb[mb].load(reinterpret_cast<const T*>(slab + (mb * 16 + r) * SLAB_ROW + kg * 32));
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) acc[nt][mb] = Piece<T>::mma(wa[nt], xb[mb], acc[nt][mb]);
    };

    Piece<T> wa_a[NT], wa_b[NT];
    u32x4_t xr_a[XL], xr_b[XL];
    DeferTake<WV, ROWS> take;
    if constexpr (EPI != EPI_RESIDUAL) take.ask(defer, M, wave, lane);      // cache hits, ahead of W
    load_w(p_begin + wave, wa_a);
    load_x(p_begin + wave, xr_a);
    if constexpr (EPI != EPI_RESIDUAL) take.settle(defer, M, wave, lane, factors);
    for (int c = p_begin + wave; c < p_end; c += 2 * WV) {
        stage(xr_a);
        wave_sync();
        load_w(c + WV, wa_b);
        load_x(c + WV, xr_b);
        multiply(wa_a);
        wave_sync();                       // the slab has been read: it may be written again
        if (c + WV < p_end) {
            stage(xr_b);
            wave_sync();
            load_w(c + 2 * WV, wa_a);
            load_x(c + 2 * WV, xr_a);
            multiply(wa_b);
            wave_sync();
        }
    }
    __syncthreads();                       // every wavefront is done with its slab: the partial sums take the memory
    skinny_finish<T, TOUT, MB, NT, EPI, WV, true>(acc, y, M, N, I, rope, reinterpret_cast<float*>(lds), nullptr, 0, nullptr,
                                                  defer, factors);
}

template <typename T, typename TOUT, int MB, int EPI>
static int launch_nt(const void* x, const void* W, void* y, int M, int N, int K, int I, int NT,
                     hipStream_t stream, RopeArgs rope = RopeArgs{}) {
    const int out_width = (EPI == EPI_SWIGLU) ? I : N;
    const int tiles = (out_width + 15) / 16;
    auto run = [&](auto nt_tag) {
        constexpr int NTc = decltype(nt_tag)::value;
        constexpr int NOUT = (EPI == EPI_SWIGLU) ? NTc / 2 : NTc;
        const int grid = (tiles + NOUT - 1) / NOUT;
        skinny_gemm_kernel<T, TOUT, MB, NTc, EPI><<<grid, GV_THREADS, 0, stream>>>((const T*)x, (const T*)W, (TOUT*)y, M, N, K, I, rope);
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

// Workgroups: a launch of no more than this many is doubled by halving the tiles.  A halved workgroup issues the loads of a
// whole tile (the lanes of the other eight rows ask for the same bytes again, and a vector load costs the texture path the
// same time whatever it fetches), so the doubled launch must still be one workgroup a compute unit: 160 pairs of tiles
// as 320 halves put two on a quarter of the units and took 15.2 us where the 160 whole ones take 9 (the 3B shape's
// [5120, 3072] with rotation at eight rows).
#define HALVE_BELOW 128
#define WIDE_BELOW 256        // workgroups: a product of one tile a workgroup and no more workgroups than this takes sixteen wavefronts
#define HALVE_RESIDUAL_FROM 4096      // (the whole product onto the residual stream: from rows of this many elements)

// The decode kernel: NT as launch_nt chooses it.  XP: pieces per wavefront of the normalising prologue, 0 without.
template <typename T, typename TOUT, int EPI, int XP>
static int launch_decode(const void* x, const void* W, void* y, int M, int N, int K, int I, int NT, hipStream_t stream,
                         RopeArgs rope = RopeArgs{}, NormArgs norm = NormArgs{}, int splits = 1, DeferArgs defer = DeferArgs{}) {
    if (splits != 1 && (XP != 0 || EPI != EPI_STORE)) return -8;      // shares are stored, not finished
    if ((defer.xn != nullptr && (EPI != EPI_RESIDUAL || splits != 1)) || (defer.ss_in != nullptr && (XP != 0 || EPI == EPI_RESIDUAL)))
        return -11;     // h * w and the sums of squares come from a whole product onto the stream; they are taken by a product on a given x
    if (norm.n_pend > 0) {
        // addends that the residual stream has not received: for the staged normalising prologue (up to
        // eight rows, at most two tiles a workgroup), or for the residual epilogue
        if (norm.pend == nullptr) return -10;
        if (XP > 0) {
            const bool staged = (XP == 4 || (XP == 8 && std::is_same<T, float>::value)) && M <= 8 && (EPI == EPI_ROPE || NT < 4);
            if (!staged || norm.n_pend > PROLOGUE_ADDENDS_MAX) return -10;
        } else if (EPI != EPI_RESIDUAL) {
            return -10;
        }
    }
    const int out_width = (EPI == EPI_SWIGLU) ? I : N;
    const int tiles = (out_width + 15) / 16;
    bool defer_mismatch = false;       // the caller sized the sums of squares for another number of workgroups
    auto run = [&](auto nt_tag) {
        constexpr int NTc = decltype(nt_tag)::value;
        constexpr int NOUT = (EPI == EPI_SWIGLU) ? NTc / 2 : NTc;
        const int grid = (tiles + NOUT - 1) / NOUT;
        // The stacked [q; k; v] matrix with rotation gives a workgroup two tiles (the partners of a
        // rotation), which leaves a small model few workgroups (96 at the 1B shape): then two
        // workgroups share every pair of tiles.  (For one tile a workgroup, 128 workgroups against
        // 256, the same was measured and gained nothing: not compiled.)
        // A whole product of long rows onto the residual stream (one that leaves the next norm's input behind, and
        // so cannot be cut along K to fill the chip) is doubled the same way.
        constexpr bool CAN_HALVE = EPI == EPI_ROPE || (EPI == EPI_RESIDUAL && NTc == 1 && XP == 0);
        const bool halve = CAN_HALVE && grid <= HALVE_BELOW &&
                           (EPI == EPI_ROPE || (K >= HALVE_RESIDUAL_FROM && splits == 1 && defer.xn != nullptr &&
                                                2 * grid <= DEFER_PARTS_MAX));
        if (defer.xn != nullptr && defer.parts != grid * (halve ? 2 : 1)) { defer_mismatch = true; return; }
        auto launch = [&](auto wv_tag, auto sr_tag, auto halves_tag) {
            constexpr int WVc = decltype(wv_tag)::value, SRc = decltype(sr_tag)::value, Hc = decltype(halves_tag)::value;
            if constexpr (XP > 0 && SRc > 0) {
                if (norm.n_pend > 0) {
                    skinny_decode_kernel<T, TOUT, NTc, EPI, XP, WVc, SRc, Hc, PRO_NORM, true>
                        <<<dim3(grid * Hc, splits), WVc * WAVE, 0, stream>>>((const T*)x, (const T*)W, (TOUT*)y, M, N, K, I,
                                                                              rope, norm, splits, defer);
                    return;
                }
            }
            skinny_decode_kernel<T, TOUT, NTc, EPI, XP, WVc, SRc, Hc><<<dim3(grid * Hc, splits), WVc * WAVE, 0, stream>>>(
                (const T*)x, (const T*)W, (TOUT*)y, M, N, K, I, rope, norm, splits, defer);
        };
        using One = std::integral_constant<int, 1>;
        using Two = std::integral_constant<int, 2>;
        using Waves8 = std::integral_constant<int, GV_WAVES>;
        auto with_halves = [&](auto wv_tag, auto sr_tag) {
            if constexpr (CAN_HALVE) {
                if (halve) { launch(wv_tag, sr_tag, Two{}); return; }
            }
            launch(wv_tag, sr_tag, One{});
        };
        if constexpr (XP == 0 && NTc == 1) {
            // rows of 2,048 elements or more in few workgroups: sixteen wavefronts each
            if (grid <= WIDE_BELOW && K >= 2048) {
                with_halves(std::integral_constant<int, 16>{}, std::integral_constant<int, 0>{});
                return;
            }
        }
        if constexpr ((XP == 4 || (XP == 8 && std::is_same<T, float>::value)) && NTc <= 2) {
            // up to eight rows: the prologue staged through LDS (its rows and the partial sums both fit),
            // compiled for 1, 4 and 8 rows
            if (M == 1) { with_halves(Waves8{}, std::integral_constant<int, 1>{}); return; }
            if (M <= 4) { with_halves(Waves8{}, std::integral_constant<int, 4>{}); return; }
            if (M <= 8) { with_halves(Waves8{}, std::integral_constant<int, 8>{}); return; }
        }
        with_halves(Waves8{}, std::integral_constant<int, 0>{});
    };
    if constexpr (EPI != EPI_ROPE) {
        if (NT >= 4) { run(std::integral_constant<int, 4>{}); return defer_mismatch ? -11 : NI_LAUNCH_RESULT(); }
    }
    if constexpr (EPI == EPI_SWIGLU || EPI == EPI_ROPE) {
        run(std::integral_constant<int, 2>{});
    } else {
        if (NT >= 2) run(std::integral_constant<int, 2>{});
        else run(std::integral_constant<int, 1>{});
    }
    return defer_mismatch ? -11 : NI_LAUNCH_RESULT();
}

// The kernel for 17 to 64 rows: MB blocks of 16 rows, NT as launch_nt chooses it, within the eight
// fragments of partial sums a wavefront may hold.
template <typename T, typename TOUT, int MB, int EPI>
static int launch_rows(const void* x, const void* W, void* y, int M, int N, int K, int I, int NT, hipStream_t stream,
                       RopeArgs rope = RopeArgs{}, int splits = 1, DeferArgs defer = DeferArgs{}) {
    if ((defer.xn != nullptr && (EPI != EPI_RESIDUAL || splits != 1)) || (defer.ss_in != nullptr && EPI == EPI_RESIDUAL)) return -11;
    const int out_width = (EPI == EPI_SWIGLU) ? I : N;
    const int tiles = (out_width + 15) / 16;
    bool defer_mismatch = false;
    auto run = [&](auto nt_tag) {
        constexpr int NTc = decltype(nt_tag)::value;
        constexpr int NOUT = (EPI == EPI_SWIGLU) ? NTc / 2 : NTc;
        const int grid = (tiles + NOUT - 1) / NOUT;
        // (several blocks of rows leave a sum of squares for every tile, not for every workgroup)
        if (defer.xn != nullptr && defer.parts != (MB >= 2 ? grid * NTc : grid)) { defer_mismatch = true; return; }
        skinny_rows_kernel<T, TOUT, MB, NTc, EPI><<<dim3(grid, splits, (M + MB * 16 - 1) / (MB * 16)), GV_THREADS, 0, stream>>>(
            (const T*)x, (const T*)W, (TOUT*)y, M, N, K, I, rope, splits, defer);
    };
    if constexpr (EPI == EPI_SWIGLU) {
        // two pairs of gate and up tiles a workgroup where asked for: half the workgroups, and with them
        // half the loads of x (every workgroup brings all of x into its LDS); bfloat16 only, where the
        // sixteen fragments of partial sums fit the registers beside two trips of W
        if constexpr (sizeof(T) == 2) {
            if (NT >= 4) { run(std::integral_constant<int, 4>{}); return NI_LAUNCH_RESULT(); }
        }
        run(std::integral_constant<int, 2>{});
    } else if constexpr (EPI == EPI_ROPE) {
        run(std::integral_constant<int, 2>{});
    } else {
        if constexpr (MB <= 2) {
            if (NT >= 4) { run(std::integral_constant<int, 4>{}); return NI_LAUNCH_RESULT(); }
        }
        if (NT >= 2) run(std::integral_constant<int, 2>{});
        else run(std::integral_constant<int, 1>{});
    }
    return defer_mismatch ? -11 : NI_LAUNCH_RESULT();
}

// Workgroups of a product onto the residual stream of M rows and N columns, which is how many sums of squares
// a row gets where the product leaves them behind for the next norm (DeferArgs): the launchers above, mirrored.
static int residual_parts(int M, int N, int K, int tiles_per_group) {
    const int tiles = (N + 15) / 16;
    int nt = tiles_per_group >= 4 ? 4 : tiles_per_group >= 2 ? 2 : 1;
    if (M > 32 && nt == 4) nt = 2;       // three and four blocks of sixteen rows hold at most two tiles a workgroup
    const int grid = (tiles + nt - 1) / nt;
    if (M > 16) return grid * nt;        // past sixteen rows every tile leaves its own sums
    return (nt == 1 && grid <= HALVE_BELOW && 2 * grid <= DEFER_PARTS_MAX && K >= HALVE_RESIDUAL_FROM) ? 2 * grid : grid;
}

template <typename T, typename TOUT, int EPI>
static int launch_mb(const void* x, const void* W, void* y, int M, int N, int K, int I, int NT, bool tiled,
                     hipStream_t stream, RopeArgs rope = RopeArgs{}, NormArgs addends = NormArgs{}, DeferArgs defer = DeferArgs{}) {
    if (M <= 16 && tiled) return launch_decode<T, TOUT, EPI, 0>(x, W, y, M, N, K, I, NT, stream, rope, addends, 1, defer);
    if (addends.n_pend > 0) return -10;      // only the kernel of the decode step proper adds them
    if (tiled) {
        // (with the rotation epilogue the rows are dealt out 32 to a workgroup: see skinny_rows_kernel)
        // two, three or four blocks of sixteen rows: what a workgroup brings of x into its LDS grows with them
        // (dealt out only while that is still at most one workgroup a compute unit: the 160 pairs of tiles of the 3B
        // shape as 320 workgroups of 32 rows took 15.0 us at 64 rows, the 192 pairs of the 8B shape as 384 22.3 us)
        const bool dealt = EPI == EPI_ROPE && ((N + 31) / 32) * ((M + 31) / 32) <= 256;
        if constexpr (EPI == EPI_ROPE) {
            // up to 32 rows of a matrix of few pairs of tiles (96 at the 1B shape): 16 rows a workgroup
            if (M <= 32 && ((N + 31) / 32) * ((M + 15) / 16) <= 256)
                return launch_rows<T, TOUT, 1, EPI>(x, W, y, M, N, K, I, NT, stream, rope, 1, defer);
        }
        if (M <= 32 || dealt) return launch_rows<T, TOUT, 2, EPI>(x, W, y, M, N, K, I, NT, stream, rope, 1, defer);
        if (M <= 48) return launch_rows<T, TOUT, 3, EPI>(x, W, y, M, N, K, I, NT, stream, rope, 1, defer);
        return launch_rows<T, TOUT, 4, EPI>(x, W, y, M, N, K, I, NT, stream, rope, 1, defer);
    }
    if (defer.xn != nullptr || defer.ss_in != nullptr) return -11;      // re-tiled matrices only
    if constexpr (EPI == EPI_RESIDUAL) {
        return -7;      // the residual epilogue exists for re-tiled matrices only
    } else {
        if (M <= 16) return launch_nt<T, TOUT, 1, EPI>(x, W, y, M, N, K, I, NT, stream, rope);
        if (M <= 32) return launch_nt<T, TOUT, 2, EPI>(x, W, y, M, N, K, I, NT, stream, rope);
        if (M <= 48) return launch_nt<T, TOUT, 3, EPI>(x, W, y, M, N, K, I, NT, stream, rope);
        return launch_nt<T, TOUT, 4, EPI>(x, W, y, M, N, K, I, NT, stream, rope);
    }
}

// Pieces of 128 bytes that one wavefront holds of a row of K elements, rounded up to what the
// normalising prologue is compiled for, or 0 if the row is too long for it: the normalised row
// has to fit the registers beside two trips of W (bfloat16: K <= 2048, float32: K <= 2048).
template <typename T>
static int prologue_pieces(int K) {
    constexpr int CH = 4 * Piece<T>::ELEMS;
    const int per_wave = ((K + CH - 1) / CH + GV_WAVES - 1) / GV_WAVES;
    if (per_wave <= 4) return 4;
    return (std::is_same<T, float>::value && per_wave <= 8) ? 8 : 0;
}

template <typename T, int EPI>
static int launch_normed(const NormArgs& norm, const void* W, void* y, int M, int N, int K, int I, int NT,
                         hipStream_t stream, RopeArgs rope = RopeArgs{}) {
    const int xp = prologue_pieces<T>(K);
    if (xp == 4) return launch_decode<T, T, EPI, 4>(nullptr, W, y, M, N, K, I, NT, stream, rope, norm);
    if constexpr (std::is_same<T, float>::value) {
        if (xp == 8) return launch_decode<T, T, EPI, 8>(nullptr, W, y, M, N, K, I, NT, stream, rope, norm);
    }
    return -5;
}

// epilogue: 0 store in the input type, 1 store float32, 2 SwiGLU (W is [2I, K], y is [M, I]),
// 3 add into y, the float32 residual stream [M, N] (tiled W).
// K must be a multiple of 16 bytes' worth of elements x 2 (bf16: 16, f32: 8); M <= 64.
// tiled: W is in the re-tiled order described at the top (swiglu then needs N/2 to be a multiple of 16).
// pend, n_pend (epilogue 3, at most 16 rows): float32 [n_pend, M, N] that y has not received yet and that are
// added before the product, y = ((y + pend[0]) + pend[1] ...) + x . W^T; null, 0: none.
//
// A norm in two halves (DeferArgs above; re-tiled W only).  Leaving: epilogue 3 with xn [M, N] of the input type,
// next_w float32 [N] and ss float32 [M, parts], parts = ni_skinny_residual_parts(M, N, K, tiles_per_group): beside adding
// into y the product stores xn = y * next_w and every workgroup's sums of squares of its columns of y.  Taking:
// epilogues 0, 1, 2 with ss float32 [M, parts] of the product before, parts <= 256 and that norm's eps: x is the xn
// that product left, and row m of the sums is multiplied by 1 / sqrt(sum_p ss[m, p] / K + eps) before the epilogue.
// xn and ss null: neither.
NI_EXPORT int ni_skinny_residual_parts(int M, int N, int K, int tiles_per_group) { return residual_parts(M, N, K, tiles_per_group); }

NI_EXPORT int ni_skinny_gemm(const void* x, const void* W, void* y, int M, int N, int K, int epilogue, int tiles_per_group,
                             int tiled, int dtype, const void* pend, int n_pend, void* xn, const void* next_w, void* ss,
                             int parts, float eps, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64) return -1;
    const int el = dtype == 0 ? 8 : 16;
    if (K % el != 0) return -2;
    const int I = N / 2;
    if (epilogue == 2 && (N % 2)) return -3;
    if (epilogue == 2 && tiled && (I % 16)) return -4;
    if (n_pend < 0 || n_pend > 16 || (n_pend > 0 && (epilogue != 3 || !pend))) return -10;
    NormArgs addends{nullptr, nullptr, 0.f};
    addends.pend = (const float*)pend;
    addends.n_pend = n_pend;
    DeferArgs defer;
    if (xn != nullptr || ss != nullptr) {
        if (!tiled || !ss || parts < 1) return -11;
        if (epilogue == 3) {
            if (!xn || !next_w || parts != residual_parts(M, N, K, tiles_per_group)) return -11;
            defer.xn = xn; defer.w = (const float*)next_w; defer.ss_out = (float*)ss;
        } else {
            if (xn != nullptr || parts > DEFER_PARTS_MAX || !(eps > 0.f)) return -11;
            defer.ss_in = (const float*)ss; defer.eps = eps; defer.width = K;
        }
        defer.parts = parts;
    }
    if (dtype == 0) {
        if (epilogue == 3) return launch_mb<float, float, EPI_RESIDUAL>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream, RopeArgs{}, addends, defer);
        if (epilogue == 2) return launch_mb<float, float, EPI_SWIGLU>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream, RopeArgs{}, NormArgs{}, defer);
        return launch_mb<float, float, EPI_STORE>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream, RopeArgs{}, NormArgs{}, defer);
    }
    if (epilogue == 3) return launch_mb<bf16_t, float, EPI_RESIDUAL>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream, RopeArgs{}, addends, defer);
    if (epilogue == 2) return launch_mb<bf16_t, bf16_t, EPI_SWIGLU>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream, RopeArgs{}, NormArgs{}, defer);
    if (epilogue == 1) return launch_mb<bf16_t, float, EPI_STORE>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream, RopeArgs{}, NormArgs{}, defer);
    return launch_mb<bf16_t, bf16_t, EPI_STORE>(x, W, y, M, N, K, I, tiles_per_group, tiled != 0, stream, RopeArgs{}, NormArgs{}, defer);
}

// Up to 64 rows, re-tiled W: the K range cut into `splits` shares of whole 128-byte pieces, the sums of share s
// stored as float32 in y[s] ([splits, M, N]); whoever reads y adds the shares in their order.  A matrix of few
// tiles then fills the chip: 128 tiles in two or four shares are 256 workgroups.  dtype 0: float32, 1: bfloat16.
template <typename T>
static int launch_ksplit(const void* x, const void* W, void* y, int M, int N, int K, int tiles_per_group, int splits,
                         hipStream_t stream) {
    if (M <= 16) return launch_decode<T, float, EPI_STORE, 0>(x, W, y, M, N, K, 0, tiles_per_group, stream, RopeArgs{}, NormArgs{}, splits);
    if (M <= 32) return launch_rows<T, float, 2, EPI_STORE>(x, W, y, M, N, K, 0, tiles_per_group, stream, RopeArgs{}, splits);
    if (M <= 48) return launch_rows<T, float, 3, EPI_STORE>(x, W, y, M, N, K, 0, tiles_per_group, stream, RopeArgs{}, splits);
    return launch_rows<T, float, 4, EPI_STORE>(x, W, y, M, N, K, 0, tiles_per_group, stream, RopeArgs{}, splits);
}

NI_EXPORT int ni_skinny_gemm_ksplit(const void* x, const void* W, void* y, int M, int N, int K, int tiles_per_group, int splits,
                                    int dtype, hipStream_t stream) {
    if (M <= 0 || M > 64 || N <= 0 || K % (dtype == 0 ? 8 : 16) != 0 || splits < 1 || splits > 16) return -1;
    if (dtype == 0) return launch_ksplit<float>(x, W, y, M, N, K, tiles_per_group, splits, stream);
    return launch_ksplit<bf16_t>(x, W, y, M, N, K, tiles_per_group, splits, stream);
}

// Whether the normalising prologue takes M rows of K elements of this type (1) or not (0).  Every
// workgroup reads all M rows of h: past eight rows that is more than the matrix it streams, and the
// norm as a kernel of its own is faster (measured at the 1B shape: 6 % of a decode step at 9 to 16 rows).
#define PROLOGUE_MAX_ROWS 8
NI_EXPORT int ni_skinny_prologue_ok(int M, int K, int dtype) {
    if (M < 1 || M > PROLOGUE_MAX_ROWS || K % (dtype == 0 ? 8 : 16) != 0) return 0;
    return (dtype == 0 ? prologue_pieces<float>(K) : prologue_pieces<bf16_t>(K)) != 0;
}

NI_EXPORT int ni_skinny_prologue_addends() { return PROLOGUE_ADDENDS_MAX; }

// The same product on RMSNorm(h) instead of a given x: h float32 [M <= 8, K], norm_weight float32 [K],
// W re-tiled.  epilogue 0 (store in the compute type) or 2 (SwiGLU).
// pend, n_pend: float32 [n_pend <= 2, M, K] that h has not received yet; the rows are normalised as
// (h + pend[0]) + pend[1] and h itself is left as it is (at most two tiles a workgroup).
NI_EXPORT int ni_skinny_gemm_normed(const void* h, const void* norm_weight, float eps, const void* W, void* y, int M, int N,
                                    int K, int epilogue, int tiles_per_group, int dtype, const void* pend, int n_pend,
                                    hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (!ni_skinny_prologue_ok(M, K, dtype)) return -5;
    if (epilogue != 0 && epilogue != 2) return -6;
    const int I = N / 2;
    if (epilogue == 2 && ((N % 2) || (I % 16))) return -4;
    if (n_pend < 0 || (n_pend > 0 && !pend)) return -10;
    NormArgs norm{(const float*)h, (const float*)norm_weight, eps};
    norm.pend = (const float*)pend;
    norm.n_pend = n_pend;
    if (dtype == 0) {
        if (epilogue == 2) return launch_normed<float, EPI_SWIGLU>(norm, W, y, M, N, K, I, tiles_per_group, stream);
        return launch_normed<float, EPI_STORE>(norm, W, y, M, N, K, I, tiles_per_group, stream);
    }
    if (epilogue == 2) return launch_normed<bf16_t, EPI_SWIGLU>(norm, W, y, M, N, K, I, tiles_per_group, stream);
    return launch_normed<bf16_t, EPI_STORE>(norm, W, y, M, N, K, I, tiles_per_group, stream);
}

// The product on the output of an attention whose keys were cut into runs, merged in the prologue
// instead of by a kernel of its own (same numbers): part_o float32 [M, heads, runs, hd], part_ml
// float32 [M, heads, runs, 2] (maximum in base e, sum).  bfloat16, W re-tiled [N, heads * hd],
// epilogue 0 (store in the compute type) or 3 (add into the float32 residual stream).
NI_EXPORT int ni_skinny_merge_ok(int M, int heads, int hd, int runs, int dtype) {
    if (dtype != 1 || M < 1 || M > PROLOGUE_MAX_ROWS || heads < 1 || heads > 128 || hd < 4 || hd % 4 != 0) return 0;
    const int staged = M == 1 ? 1 : M <= 4 ? 4 : 8;       // the rows the prologue is compiled for
    if (runs < 2 || runs > MERGE_RUNS_OF(staged) || M * heads * (runs + 1) > MERGE_FACTORS_MAX) return 0;
    const long K = static_cast<long>(heads) * hd;
    return K % 16 == 0 && K <= 65536 && prologue_pieces<bf16_t>(static_cast<int>(K)) == 4;
}

template <typename TOUT, int EPI>
static int launch_merged(const NormArgs& merge, const void* W, void* y, int M, int N, int K, hipStream_t stream,
                         DeferArgs defer = DeferArgs{}) {
    const int tiles = (N + 15) / 16;
    if (defer.ss_in != nullptr || (defer.xn != nullptr && EPI != EPI_RESIDUAL)) return -11;
    auto go = [&](auto sr_tag) {
        constexpr int SRc = decltype(sr_tag)::value;
        skinny_decode_kernel<bf16_t, TOUT, 1, EPI, 4, GV_WAVES, SRc, 1, PRO_MERGE><<<tiles, GV_THREADS, 0, stream>>>(
            nullptr, (const bf16_t*)W, (TOUT*)y, M, N, K, 0, RopeArgs{}, merge, 1, defer);
    };
    if (M == 1) go(std::integral_constant<int, 1>{});
    else if (M <= 4) go(std::integral_constant<int, 4>{});
    else go(std::integral_constant<int, 8>{});
    return NI_LAUNCH_RESULT();
}

// pend, n_pend (epilogue 3): as for ni_skinny_gemm.
// xn, next_w, ss (epilogue 3): as for ni_skinny_gemm, with parts = the tiles of N.
NI_EXPORT int ni_skinny_gemm_merged(const void* part_o, const void* part_ml, int runs, int heads, int hd, const void* W,
                                    void* y, int M, int N, int epilogue, int dtype, const void* pend, int n_pend,
                                    void* xn, const void* next_w, void* ss, int parts, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (!part_o || !part_ml || !ni_skinny_merge_ok(M, heads, hd, runs, dtype)) return -5;
    if (epilogue != 0 && epilogue != 3) return -6;
    if (n_pend < 0 || n_pend > 16 || (n_pend > 0 && (epilogue != 3 || !pend))) return -10;
    NormArgs merge{nullptr, nullptr, 0.f};
    merge.pend = (const float*)pend;
    merge.n_pend = n_pend;
    merge.part_o = (const float*)part_o;
    merge.part_ml = (const float*)part_ml;
    merge.runs = runs; merge.heads = heads; merge.hd = hd;
    DeferArgs defer;
    if (xn != nullptr || ss != nullptr) {
        if (epilogue != 3 || !xn || !next_w || !ss || parts != (N + 15) / 16) return -11;
        defer.xn = xn; defer.w = (const float*)next_w; defer.ss_out = (float*)ss; defer.parts = parts;
    }
    if (epilogue == 3) return launch_merged<float, EPI_RESIDUAL>(merge, W, y, M, N, heads * hd, stream, defer);
    return launch_merged<bf16_t, EPI_STORE>(merge, W, y, M, N, heads * hd, stream);
}

// Product with the stacked [q; k; v] matrix ((H + 2 KVH) * hd rows), rotation of query and key
// heads by the rows' positions, queries to q_out [M, H * hd], keys and values into the pools at
// slot_mapping (null: not stored).  hd must be a multiple of 32 and fully rotated.
// With x null the product is taken on RMSNorm(h): h float32 [M <= 8, K], norm_weight [K], W re-tiled; pend, n_pend as
// for ni_skinny_gemm_normed.  With x and ss: x is what the product before left for a norm with this eps, ss [M, parts]
// its sums of squares, and the division is made here (as for ni_skinny_gemm).
NI_EXPORT int ni_skinny_qkv_rope(const void* x, const void* h, const void* norm_weight, float eps, const void* W,
                                 void* q_out, const void* positions, const void* cos_t, const void* sin_t,
                                 const void* slot_mapping, void* kpool, void* vpool, int M, int K, int H, int KVH, int hd,
                                 int page_size, int tiled, int dtype, const void* pend, int n_pend, const void* ss, int parts,
                                 hipStream_t stream) {
    if (M <= 0) return 0;
    if (M > 64) return -1;
    if (K % (dtype == 0 ? 8 : 16) != 0) return -2;
    if (hd % 32 != 0 || H <= 0 || KVH <= 0 || page_size < 1) return -3;
    RopeArgs rope{(const int32_t*)positions, (const float*)cos_t, (const float*)sin_t, (const int32_t*)slot_mapping,
                  kpool, vpool, H, KVH, hd, page_size};
    const int N = (H + 2 * KVH) * hd;
    // the grid is sized from the output width: one workgroup per two tiles
    if (!x) {
        if (ss != nullptr) return -11;
        if (!h || !norm_weight || !tiled || !ni_skinny_prologue_ok(M, K, dtype)) return -5;
        if (n_pend < 0 || (n_pend > 0 && !pend)) return -10;
        NormArgs norm{(const float*)h, (const float*)norm_weight, eps};
        norm.pend = (const float*)pend;
        norm.n_pend = n_pend;
        if (dtype == 0) return launch_normed<float, EPI_ROPE>(norm, W, q_out, M, N, K, 0, 2, stream, rope);
        return launch_normed<bf16_t, EPI_ROPE>(norm, W, q_out, M, N, K, 0, 2, stream, rope);
    }
    if (n_pend != 0) return -10;      // addends go with the normalising prologue only
    DeferArgs defer;
    if (ss != nullptr) {              // x is what the product before left for the norm: the division is made here
        if (!tiled || parts < 1 || parts > DEFER_PARTS_MAX || !(eps > 0.f)) return -11;
        defer.ss_in = (const float*)ss; defer.parts = parts; defer.eps = eps; defer.width = K;
    }
    if (dtype == 0) return launch_mb<float, float, EPI_ROPE>(x, W, q_out, M, N, K, 0, 2, tiled != 0, stream, rope, NormArgs{}, defer);
    return launch_mb<bf16_t, bf16_t, EPI_ROPE>(x, W, q_out, M, N, K, 0, 2, tiled != 0, stream, rope, NormArgs{}, defer);
}
