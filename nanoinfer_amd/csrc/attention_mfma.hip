// Attention of prompt portions over the paged key/value cache on the matrix cores of gfx950.
// bfloat16 only; compiled once per head size (-DHEAD_DIM=n, a multiple of 16 up to 256; the kernel for
// single tokens takes the multiples of 32 among them).
//
// A workgroup of four wavefronts owns one tile of consecutive tokens of one sequence and the
// query heads of one kv head (up to 16 of them at a time).  A "row" is one (token, head) pair; a
// wavefront owns CB blocks of 16 rows (CB = 1 or 2, chosen by the host from the size of the
// step: larger tiles share every staged key among more rows, smaller ones fill the chip when
// the step is short).  All rows of a workgroup read the same keys and values, 32 at a time:
//
//   S^T[key, row]  = K[key, :] . Q[row, :]       v_mfma_f32_16x16x32_bf16, K rows (staged in LDS
//                                                 once for the workgroup) as the A operand, Q as B
//   softmax        float32, online: every lane holds 8 scores of ONE row (its column of S^T),
//                  so the maximum needs two shuffles and the rescaling of the output none
//   O^T[dim, row] += V^T[dim, key] . P^T[key, row]   the scores of a lane are already laid out
//                  as the B operand; V^T comes from a tile of V that the workgroup stages in LDS
//
// Computing the transposes is what makes P need no data movement between the two products: the
// k index of an MFMA is only a label, and a lane's eight scores (keys kg*4+i of both 16-key
// halves) are given the labels kg*8+j on both operands.
//
// Formula as in the token-at-a-time kernel (reference: src/op/kernels/cuda/prefill_attention_kernel.cu:66-141,
// 422-455): the query at position P reads keys max(0, P+1-window)..P, scores are scaled by `scale`,
// softmax subtracts the maximum, divides by the plain sum; probabilities are rounded to bfloat16
// for the second product and summed as rounded, in float32.
#include "common.h"
#include <type_traits>

#include <algorithm>

#ifndef HEAD_DIM
#error "HEAD_DIM must be defined"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size: multiple of 16, at most 256");
// A head size that is an odd multiple of 16 leaves the first product 16 dims after its steps of 32.  A lane
// then holds 4 dims of its key (or of its row of Q) instead of 8, in the first half of its operand; the
// second half is zero in both operands (the k index of a matrix instruction is only a label, so the four
// real dims of every lane meet their partners and the zeros meet zeros).  No lane reads past its row.
// (One instruction of half the depth, v_mfma_f32_16x16x16_bf16, behind the chain of v_mfma_f32_16x16x32_bf16
// into the same accumulator gave wrong scores now and then at head sizes 48 and 80: one kind of matrix
// instruction per chain is kept.)
#define HEAD_HALF (HEAD_DIM % 32 != 0)

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));    // 16 bytes that only pass through registers

#define KSTEP 32
#define MA_WAVES 4
#define NEG_BIG (-1.0e30f)
#define KPAD 8   // elements of padding per staged row of K: the sixteen rows of a 16-byte read fall on different banks
#define VPAD 8   // elements of padding per staged row of V: the eight rows that half a wavefront reads at a time in a
                 // transposing read (32 bytes of each) fall on different banks

// V^T as the A operand of the second product, read from a V tile that lies in LDS as it lies in the
// cache ([key][dim], rows of `row_elems` elements): gfx950's transposing read hands lane (r, kg) the
// four elements V[key0 + 4*kg + i][dim0 + r], i = 0..3, when lane (r, kg) gives the address of
// V[key0 + 4*kg + r/4][dim0 + 4*(r%4)] (within sixteen lanes it transposes the 4 x 16 block that four
// rows of 32 bytes make).  Two reads, for the 16-key halves of a step, give the eight keys of a lane
// in the order of its eight scores.  (Before, V was turned round on its way into LDS, with eight
// 2-byte writes for every 16 bytes loaded: a third of the prompt kernel's LDS time.)
typedef short shortx4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 read_v_operand(const uint16_t* tile, int row_elems, int dim0, int r, int kg) {
    typedef __attribute__((address_space(3))) shortx4_t* lds_ptr;
    const uint16_t* at = tile + (4 * kg + (r >> 2)) * row_elems + dim0 + 4 * (r & 3);
    const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(at));
    const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(at + 16 * row_elems));
    const uint2 a = __builtin_bit_cast(uint2, lo), b = __builtin_bit_cast(uint2, hi);
    return make_uint4(a.x, a.y, b.x, b.y);
}

struct QTile { int32_t seq, row0, ntok, pos0; };   // tokens row0..row0+ntok-1 of the batch, positions pos0..

#define LOG2E 1.4426950408889634f
#define LN2 0.6931471805599453f

// Maximum over the four lanes that hold the scores of one row (lanes r, r+16, r+32, r+48):
// the halves of the wavefront, then the 16-lane rows of each half, are exchanged by the swap
// instructions of gfx950 (plain vector instructions, no trip through LDS).
__device__ __forceinline__ float row_max4(float x) {
    const auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// How far (in powers of two) a row's scores may rise above the reference its weights are taken
// against before the reference is moved and the output rescaled.  Softmax is the same whatever
// the reference is, as long as numerator and denominator share it; weights up to 2^8 keep their
// relative precision in bfloat16 and in the float32 sums.  Without the slack the output would be
// rescaled whenever any of a wavefront's rows meets a new maximum, which is most steps.
#define REF_SLACK 8.0f

// The online softmax of a 32-key step, for a lane that holds eight scores of one row (keys
// key0 + t*16 + i of the two 16-key halves), in three parts.  Reference and sum are kept in the
// base-2 domain (scores are scaled by scale*log2(e) > 0), so an exponential is one v_exp_f32.
// MASKED steps are the ones at the edges of a row's key range [lo, pos]; in the others every key
// counts and no comparison is made.
//
// 1. mask_scores: the scores with the keys outside the row's range set to NEG_BIG; returns the
//    largest of the lane.
template <bool MASKED>
__device__ __forceinline__ float mask_scores(const floatx4_t (&st)[2], int key0, int lo, int pos, bool row_ok,
                                             float (&raw)[8]) {
    float mx = NEG_BIG;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = st[t][i];
            if constexpr (MASKED) {
                const int key = key0 + t * 16 + i;
                v = (row_ok && key <= pos && key >= lo) ? v : NEG_BIG;
            }
            raw[t * 4 + i] = v;
            mx = fmaxf(mx, v);
        }
    return mx;
}
// 2. Whether a lane's scores have risen above the slack over its row's reference; only then (for
//    any lane of the wavefront) move_reference is run: it moves the reference of such rows to
//    their maximum and returns the factor that what was summed so far has to be multiplied with
//    (1 for the other rows).  In most steps no row has risen and nothing crosses the lanes.
__device__ __forceinline__ bool above_reference(float lane_max, float scale2, float m_ref) {
    return fmaf(lane_max, scale2, -REF_SLACK) > m_ref;
}
__device__ __forceinline__ float move_reference(float lane_max, float scale2, float& m_ref) {
    float mx = row_max4(lane_max);
    mx = mx > 0.5f * NEG_BIG ? mx * scale2 : NEG_BIG;       // a row that has no key yet keeps its reference
    const bool move = mx > m_ref + REF_SLACK;
    const float m_new = move ? mx : m_ref;
    const float corr = move ? __builtin_amdgcn_exp2f(m_ref - m_new) : 1.0f;
    m_ref = m_new;
    return corr;
}
// 3. weights: 2^(score - reference), rounded to bfloat16 and laid out as the B operand of the
//    second product.  The sum of a row's weights is taken by the matrix cores as well
//    (row_sum_step): over the rounded weights, the ones the second product uses, so the output is
//    an exact convex combination of values whatever the rounding.
template <bool MASKED>
__device__ __forceinline__ uint4 weights(const float (&raw)[8], float scale2, float m_ref) {
    uint32_t pw[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float p0 = __builtin_amdgcn_exp2f(fmaf(raw[2 * j], scale2, -m_ref));
        float p1 = __builtin_amdgcn_exp2f(fmaf(raw[2 * j + 1], scale2, -m_ref));
        if constexpr (MASKED) {
            p0 = raw[2 * j] > 0.5f * NEG_BIG ? p0 : 0.f;
            p1 = raw[2 * j + 1] > 0.5f * NEG_BIG ? p1 : 0.f;
        }
        pw[j] = pack_bf16x2(p0, p1);
    }
    return make_uint4(pw[0], pw[1], pw[2], pw[3]);
}

// Sum of every row's 32 weights, added to `l` (all four elements of a lane are the sum of its
// row): the second product with a tile of ones in the place of V^T.  The matrix cores have time
// to spare; the vector unit, which would need sixteen instructions for it, has not.
__device__ __forceinline__ floatx4_t row_sum_step(const uint4& pf, floatx4_t l) {
    const uint4 ones = make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);     // eight times bfloat16 1.0
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ones), __builtin_bit_cast(bf16x8_t, pf), l, 0, 0, 0);
}

// (Where the registers allow two wavefronts a SIMD, asking for them also makes the compiler keep the
// accumulators in ordinary vector registers: with a whole register file to itself it parks them in
// the accumulation registers, which the vector unit cannot multiply, and copies them to and fro.)
template <int CB, bool POW2>
__global__ __launch_bounds__(MA_WAVES * WAVE) __attribute__((amdgpu_waves_per_eu(HEAD_DIM * CB <= 128 ? 2 : 1)))
void mfma_attention_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ kpool, const bf16_t* __restrict__ vpool,
    const int32_t* __restrict__ block_table, int table_stride, const QTile* __restrict__ tiles,
    int n_tiles, bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml, int H, int KVH,
    int page_size, int page_shift, int hpt_shift, int window, float scale, int nsplit) {
    constexpr int HD = HEAD_DIM;
    constexpr int MA_THREADS = MA_WAVES * WAVE;
    constexpr int KK = HD / 32;              // k steps of 32 dims of the first product (and 16 dims more where HEAD_HALF)
    constexpr int KKA = KK > 0 ? KK : 1;     // (an array's length)
    constexpr int DT = HD / 16;              // 16-wide tiles of the head dimension in the output
    constexpr int VROW = HD + VPAD;
    constexpr int KROW = HD + KPAD;
    __shared__ __attribute__((aligned(16))) uint16_t ksm[2][KSTEP][KROW];  // K of a step: [key][dim]
    __shared__ __attribute__((aligned(16))) uint16_t vs[2][KSTEP][VROW];   // V of a step, as it lies in the cache: [key][dim]

    // The launch has as many workgroups as the chip holds at once, and the tiles come sorted by the
    // number of keys they have to walk, longest first.  Workgroup w takes tiles w, 2P-1-w, 2P+w, ...
    // (P workgroups in x): to and fro through the sorted list, so that every workgroup gets about
    // the same number of keys and none is left working alone at the end.
    for (int round = 0;; ++round) {
        int tile_at = (round & 1) ? (round + 1) * gridDim.x - 1 - blockIdx.x : round * gridDim.x + blockIdx.x;
        // With one round only nothing pairs long tiles with short ones inside a workgroup.  The chip then holds the
        // whole grid at once, two workgroups a compute unit, and hands them out in the order of their numbers: unit u
        // gets workgroups u and u + half the grid, which is the same x in the lower and the upper half of y.  The
        // upper half walks the list backwards, so that every unit gets a long and a short tile.
        if (n_tiles <= static_cast<int>(gridDim.x) && 2 * blockIdx.y >= gridDim.y && gridDim.y > 1) tile_at = n_tiles - 1 - tile_at;
        if (tile_at >= n_tiles || tile_at < 0) break;                // later rounds lie further on in the list
        const QTile tile = tiles[tile_at];
        const int G = H / KVH;
        const int hpt = 1 << hpt_shift;                      // heads of a tile: a power of two up to 16
        const int chunks = (G + hpt - 1) >> hpt_shift;
        const int g = blockIdx.y / chunks;
        const int chunk = blockIdx.y % chunks;

        const int tid = threadIdx.x;
        const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;      // the same in every lane: say so
        const int r = lane % 16, kg = lane / 16;

        // A wavefront owns CB blocks of 16 rows; a row is one (token, head) pair, heads fastest.  Block c
        // of wavefront w holds the tokens (w*CB + c) * 16/hpt .. of the tile.  What is known of a block
        // as a whole (its first and last position) is the same in every lane and steers the branches.
        const int tok_per_block = 16 >> hpt_shift;
        int pos[CB], row_lo[CB], tt[CB];
        bool row_ok[CB], blk_ok[CB];
        int blk_pmin[CB], blk_pmax[CB], blk_lo_max[CB];
        const int hh = (chunk << hpt_shift) + (r & (hpt - 1));              // head within the group
        const int head = g * G + hh;
#pragma unroll
        for (int c = 0; c < CB; ++c) {
            const int tb0 = (wave * CB + c) * tok_per_block;
            tt[c] = tb0 + (r >> hpt_shift);
            row_ok[c] = tt[c] < tile.ntok && hh < G;
            pos[c] = tile.pos0 + tt[c];
            row_lo[c] = (row_ok[c] && window > 0) ? max(0, pos[c] + 1 - window) : 0;
            blk_ok[c] = tb0 < tile.ntok;
            blk_pmin[c] = tile.pos0 + tb0;
            blk_pmax[c] = tile.pos0 + min(tile.ntok, tb0 + tok_per_block) - 1;
            blk_lo_max[c] = window > 0 ? max(0, blk_pmax[c] + 1 - window) : 0;
        }

        // key range of the workgroup (uniform), walked in steps of 32 from a multiple of 32
        const int kend = tile.pos0 + tile.ntok;
        const int kbeg = (window > 0 ? max(0, tile.pos0 + 1 - window) : 0) / KSTEP * KSTEP;
        const int nsteps_all = (kend - kbeg + KSTEP - 1) / KSTEP;
        // a split (blockIdx.z) takes a contiguous run of steps
        const int per_split = (nsteps_all + nsplit - 1) / nsplit;
        const int s_begin = blockIdx.z * per_split;
        const int nsteps = max(0, min(nsteps_all, s_begin + per_split) - s_begin);
        const int kfirst = kbeg + s_begin * KSTEP;
        const float scale2 = scale * LOG2E;

        const int32_t* table = block_table + static_cast<size_t>(tile.seq) * table_stride;
        auto page_of = [&](int key) { return POW2 ? (key >> page_shift) : key / page_size; };
        auto slot_of = [&](int key) { return POW2 ? (key & (page_size - 1)) : key % page_size; };
        // The block table of the workgroup's keys is copied to LDS, a segment of TBL_MAX pages at a
        // time (one segment, unless the key range is very long): an entry read from global memory
        // inside the loop would have to be waited for before its rows can be asked for, and that
        // wait, being in order, would drain every row load still in flight.
        constexpr int TBL_MAX = 1024;
        __shared__ int32_t tbl[TBL_MAX];
        int key_lo = 0, key_hi = 0, lp0 = 0;              // keys of the current segment, and its first page
        // the first key any row of the tile may read: keys before it (the steps start at a multiple of
        // KSTEP) may lie in pages that a window has passed and given back, and are never loaded
        const int tile_lo = window > 0 ? max(0, tile.pos0 + 1 - window) : 0;
        auto row_address = [&](int key) -> size_t {       // offset of key's row for kv head g, key clamped into the segment
            const int kc = min(max(key, max(key_lo, tile_lo)), key_hi);
            const int page = tbl[page_of(kc) - lp0];
            // the row's number fits 32 bits (the host checks the pool's size); one widening multiply makes the offset
            const uint32_t row = (static_cast<uint32_t>(max(page, 0)) * KVH + g) * page_size + slot_of(kc);
            return static_cast<size_t>(row) * HD;
        };

        // Q as the B operand: lane (row r, group kg) holds dims kk*32 + kg*8 .. +8 (and of the last 16 dims
        // of an odd head size, dims KK*32 + kg*4 .. +4)
        uint4 qf[CB][KKA];
        uint2 qh[CB];
#pragma unroll
        for (int c = 0; c < CB; ++c) {
            const bf16_t* qrow = q + static_cast<size_t>(tile.row0 + (row_ok[c] ? tt[c] : 0)) * q_stride +
                                 static_cast<size_t>(row_ok[c] ? head : 0) * HD;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk)
                qf[c][kk] = row_ok[c] ? *reinterpret_cast<const uint4*>(qrow + kk * 32 + kg * 8) : make_uint4(0, 0, 0, 0);
            qh[c] = make_uint2(0, 0);
            if constexpr (HEAD_HALF) {
                if (row_ok[c]) qh[c] = *reinterpret_cast<const uint2*>(qrow + KK * 32 + kg * 4);
            }
        }

        float m_run[CB];
        floatx4_t o[CB][DT], l_run[CB];
#pragma unroll
        for (int c = 0; c < CB; ++c) {
            m_run[c] = NEG_BIG;
            l_run[c] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) o[c][dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
        }

        // Staging of a step's 32 keys: a thread loads 8 dims (16 bytes) of one key's K row and of its V
        // row, neighbouring threads neighbouring pieces of a row.  Both go to LDS as they are, rows
        // padded against bank conflicts of the reads; the second product's operand is taken from the V
        // tile by transposing reads (read_v_operand).
        constexpr int PIECES = HD / 8;
        constexpr int ITEMS = KSTEP * PIECES;
        constexpr int PER_THREAD = (ITEMS + MA_THREADS - 1) / MA_THREADS;
        // (where the items do not fill the last round of the threads, the spare threads load an item again
        // and do not store it: no load is under a branch)
        auto addresses = [&](int ks, size_t (&at)[PER_THREAD]) {
#pragma unroll
            for (int i = 0; i < PER_THREAD; ++i) {
                const int item = (tid + i * MA_THREADS) % ITEMS;
                at[i] = row_address(ks + item / PIECES) + (item % PIECES) * 8;
            }
        };
        auto load_at = [&](const size_t (&at)[PER_THREAD], u32x4_t (&kdst)[PER_THREAD], u32x4_t (&vdst)[PER_THREAD]) {
#pragma unroll
            for (int i = 0; i < PER_THREAD; ++i) {
                kdst[i] = *reinterpret_cast<const u32x4_t*>(kpool + at[i]);
                vdst[i] = *reinterpret_cast<const u32x4_t*>(vpool + at[i]);
            }
        };
        auto load_kv = [&](int ks, u32x4_t (&kdst)[PER_THREAD], u32x4_t (&vdst)[PER_THREAD]) {
            size_t at[PER_THREAD];
            addresses(ks, at);
            load_at(at, kdst, vdst);
        };
        auto store_kv = [&](int buf, const u32x4_t (&ksrc)[PER_THREAD], const u32x4_t (&vsrc)[PER_THREAD]) {
#pragma unroll
            for (int i = 0; i < PER_THREAD; ++i) {
                const int item = tid + i * MA_THREADS;
                if (item < ITEMS) {
                    const int key = item / PIECES, dim0 = (item % PIECES) * 8;
                    *reinterpret_cast<u32x4_t*>(&ksm[buf][key][dim0]) = ksrc[i];
                    *reinterpret_cast<u32x4_t*>(&vs[buf][key][dim0]) = vsrc[i];
                }
            }
        };

        // Loads run DEPTH steps ahead of the arithmetic: rows wait in registers (a ring of DEPTH slots)
        // while older steps are multiplied, so a step costs its arithmetic, not a memory round trip.
        // K and V of step s+1 are written to LDS during step s.
        constexpr int DEPTH = HD <= 64 ? 4 : HD <= 128 ? 3 : 2;
        u32x4_t kr[DEPTH][PER_THREAD];
        u32x4_t vr[DEPTH][PER_THREAD];
        for (int seg0 = 0; seg0 < nsteps;) {
            key_lo = kfirst + seg0 * KSTEP;
            lp0 = page_of(key_lo);
            const int seg_steps = min(nsteps - seg0, ((lp0 + TBL_MAX) * page_size - key_lo) / KSTEP);
            key_hi = min(key_lo + seg_steps * KSTEP, kend) - 1;
            __syncthreads();                   // nobody still reads the previous segment's table or staged tiles
            for (int i = tid; i <= page_of(key_hi) - lp0; i += MA_THREADS) tbl[i] = table[lp0 + i];
            __syncthreads();
            // rows past the end of the segment are read from its last key and not used: no load is under a branch
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) load_kv(key_lo + d * KSTEP, kr[d], vr[d]);
            store_kv(0, kr[0], vr[0]);
            load_kv(key_lo + DEPTH * KSTEP, kr[0], vr[0]);
            // Step s multiplies the tiles in buffer s % 2 and writes those of step s + 1 (slot (s + 1) % DEPTH
            // of the ring) to the other buffer.  The loop is unrolled DEPTH times so that a slot is a fixed
            // set of registers: rotating the ring by copies would wait for the newest loads.  A slot is
            // asked for its next rows as soon as it has been written to LDS.
            // (A step is compiled twice.  INTERIOR: the step's 32 keys lie inside the key range of every row of
            // every block of this wavefront, known before the loop, so it has no flags to work out, no masks and
            // no branch but the one for a risen row, and the scores stay in the registers the matrix cores left
            // them in.  Most steps of a long key range are of this kind.)
            auto step = [&](auto interior_tag, int s, u32x4_t (&knext)[PER_THREAD], u32x4_t (&vnext)[PER_THREAD]) {
                constexpr bool INTERIOR = decltype(interior_tag)::value;
                const int ks = key_lo + s * KSTEP;
                // where the rows asked for at the end of the step lie: looked up now, so that the table's answer
                // has long come when the loads are issued
                size_t at_next[PER_THREAD];
                addresses(ks + (DEPTH + 1) * KSTEP, at_next);
                if (INTERIOR || s < seg_steps) {
                    // The tiles of this step are in buffer s & 1; nobody still reads the other one.  Only LDS is
                    // ordered here: a full barrier would also wait for every row load in flight for later steps.
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
                    __builtin_amdgcn_s_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
                    // A block takes part in a step unless all its rows lie before the step's keys.  Steps whose 32
                    // keys lie inside the key range of every row of a block need no masking for it.
                    bool act[CB], inner[CB], any_act = INTERIOR, all_inner = true;
#pragma unroll
                    for (int c = 0; c < CB; ++c) {
                        act[c] = INTERIOR || (blk_ok[c] && ks <= blk_pmax[c]);
                        inner[c] = INTERIOR || (act[c] && ks >= blk_lo_max[c] && ks + KSTEP - 1 <= blk_pmin[c]);
                        any_act = any_act || act[c];
                        all_inner = all_inner && inner[c];
                    }
                    if (any_act) {
                        // K as the A operand: lane (key r of a 16-key half, group kg) holds dims kk*32 + kg*8 .. +8
                        const uint16_t (*kb)[KROW] = ksm[s & 1];
                        const uint16_t (*vb)[VROW] = vs[s & 1];
                        uint4 ka[2][KKA];
                        uint2 kh[2];
#pragma unroll
                        for (int t = 0; t < 2; ++t) {
#pragma unroll
                            for (int kk = 0; kk < KK; ++kk)
                                ka[t][kk] = *reinterpret_cast<const uint4*>(&kb[t * 16 + r][kk * 32 + kg * 8]);
                            if constexpr (HEAD_HALF) kh[t] = *reinterpret_cast<const uint2*>(&kb[t * 16 + r][KK * 32 + kg * 4]);
                        }
                        // V^T as the A operand of the second product, asked for now where registers allow: the
                        // answer comes while the first product and the exponentials run
                        constexpr bool EARLY_V = HD * CB <= 128;
                        uint4 vf_early[EARLY_V ? DT : 1];
                        if constexpr (EARLY_V) {
#pragma unroll
                            for (int dt = 0; dt < DT; ++dt) vf_early[dt] = read_v_operand(&vb[0][0], VROW, dt * 16, r, kg);
                        }
                        // S^T of block c for the two 16-key halves; this lane: row r of the block, keys ks + t*16 + kg*4 + i
                        auto scores = [&](int c, floatx4_t (&st)[2]) {
#pragma unroll
                            for (int t = 0; t < 2; ++t) {
                                st[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                                for (int kk = 0; kk < KK; ++kk)
                                    st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ka[t][kk]),
                                                                                    __builtin_bit_cast(bf16x8_t, qf[c][kk]),
                                                                                    st[t], 0, 0, 0);
                                if constexpr (HEAD_HALF) {
                                    const uint4 ka_half = make_uint4(kh[t].x, kh[t].y, 0u, 0u);
                                    const uint4 qf_half = make_uint4(qh[c].x, qh[c].y, 0u, 0u);
                                    st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ka_half),
                                                                                    __builtin_bit_cast(bf16x8_t, qf_half),
                                                                                    st[t], 0, 0, 0);
                                }
                            }
                        };
                        // 1. scores of every block, masked where the step lies at the edge of a block's key range (the
                        //    diagonal of the tile, a window's start).  The common step has no branch between the
                        //    blocks, so that their chains of dependent instructions overlap.
                        float raw[CB][8], lane_max[CB];
                        bool risen = false;
                        if (all_inner) {
                            floatx4_t st[CB][2];
#pragma unroll
                            for (int c = 0; c < CB; ++c) scores(c, st[c]);
#pragma unroll
                            for (int c = 0; c < CB; ++c) {
                                lane_max[c] = mask_scores<false>(st[c], ks + kg * 4, row_lo[c], pos[c], row_ok[c], raw[c]);
                                risen = risen || above_reference(lane_max[c], scale2, m_run[c]);
                            }
                        } else {
#pragma unroll
                            for (int c = 0; c < CB; ++c) {
                                if (act[c]) {
                                    floatx4_t st[2];
                                    scores(c, st);
                                    lane_max[c] = inner[c] ? mask_scores<false>(st, ks + kg * 4, row_lo[c], pos[c], row_ok[c], raw[c])
                                                           : mask_scores<true>(st, ks + kg * 4, row_lo[c], pos[c], row_ok[c], raw[c]);
                                    risen = risen || above_reference(lane_max[c], scale2, m_run[c]);
                                } else {
                                    lane_max[c] = NEG_BIG;
#pragma unroll
                                    for (int i = 0; i < 8; ++i) raw[c][i] = NEG_BIG;
                                }
                            }
                        }
                        // 2. rows whose scores have risen far above their reference: move it, rescale what was summed
                        if (__any(risen)) {
#pragma unroll
                            for (int c = 0; c < CB; ++c) {
                                const float corr = move_reference(lane_max[c], scale2, m_run[c]);
                                l_run[c] *= corr;
#pragma unroll
                                for (int dt = 0; dt < DT; ++dt) o[c][dt] *= corr;
                            }
                        }
                        // 3. weights, their sums, and O^T += V^T . P^T : the A operand of lane (dim r of a 16-dim tile,
                        //    group kg) is V[key_j][dim] for the same eight keys, in the same order, as the lane's scores.
                        //    A block that takes no part has weights of zero.
                        uint4 pf[CB];
#pragma unroll
                        for (int c = 0; c < CB; ++c)
                            pf[c] = all_inner ? weights<false>(raw[c], scale2, m_run[c]) : weights<true>(raw[c], scale2, m_run[c]);
#pragma unroll
                        for (int c = 0; c < CB; ++c) l_run[c] = row_sum_step(pf[c], l_run[c]);
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt) {
                            uint4 vf;
                            if constexpr (EARLY_V) vf = vf_early[dt];
                            else vf = read_v_operand(&vb[0][0], VROW, dt * 16, r, kg);
#pragma unroll
                            for (int c = 0; c < CB; ++c)
                                o[c][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vf),
                                                                                   __builtin_bit_cast(bf16x8_t, pf[c]),
                                                                                   o[c][dt], 0, 0, 0);
                        }
                    }
                    store_kv((s + 1) & 1, knext, vnext);
                }
                load_at(at_next, knext, vnext);
            };
            // the steps [in_lo, in_hi) of the segment, whole turns of the ring, are interior for this wavefront
            int in_lo = seg_steps, in_hi = seg_steps;
            {
                bool every = true;
                int lo_max = 0, p_min = blk_pmin[0];
#pragma unroll
                for (int c = 0; c < CB; ++c) {
                    every = every && blk_ok[c];
                    lo_max = max(lo_max, blk_lo_max[c]);
                    p_min = min(p_min, blk_pmin[c]);
                }
                const int first = lo_max > key_lo ? (lo_max - key_lo + KSTEP - 1) / KSTEP : 0;       // ks >= lo_max
                const int past = p_min - (KSTEP - 1) >= key_lo ? (p_min - (KSTEP - 1) - key_lo) / KSTEP + 1 : 0;   // ks + 31 <= p_min
                const int a = (first + DEPTH - 1) / DEPTH * DEPTH;
                const int b = min(past, seg_steps);
                if (every && b - a >= DEPTH) { in_lo = a; in_hi = a + (b - a) / DEPTH * DEPTH; }
            }
            for (int s0 = 0; s0 < seg_steps; s0 += DEPTH) {
                if (s0 >= in_lo && s0 < in_hi) {
#pragma unroll
                    for (int d = 0; d < DEPTH; ++d)
                        step(std::true_type{}, s0 + d, kr[(d + 1) % DEPTH], vr[(d + 1) % DEPTH]);
                } else {
#pragma unroll
                    for (int d = 0; d < DEPTH; ++d)
                        step(std::false_type{}, s0 + d, kr[(d + 1) % DEPTH], vr[(d + 1) % DEPTH]);
                }
            }
            seg0 += seg_steps;
        }

#pragma unroll
        for (int c = 0; c < CB; ++c) {
            const float l = l_run[c][0];
            if (!row_ok[c]) continue;
            if (nsplit > 1) {
                // partial (maximum, sum, unnormalised output) of this split, merged by a second kernel
                const size_t p = (static_cast<size_t>(tile.row0 + tt[c]) * H + head) * nsplit + blockIdx.z;
                if (kg == 0) { part_ml[p * 2] = m_run[c] * LN2; part_ml[p * 2 + 1] = l; }     // the merge kernel works in base e
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    *reinterpret_cast<float4*>(part_o + p * HD + dt * 16 + kg * 4) =
                        make_float4(o[c][dt][0], o[c][dt][1], o[c][dt][2], o[c][dt][3]);
            } else if (l > 0.f) {
                const float inv = 1.0f / l;
                bf16_t* dst = out + static_cast<size_t>(tile.row0 + tt[c]) * H * HD + static_cast<size_t>(head) * HD;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    float v4[4] = {o[c][dt][0] * inv, o[c][dt][1] * inv, o[c][dt][2] * inv, o[c][dt][3] * inv};
                    VecIO<bf16_t, 4>::store(dst + dt * 16 + kg * 4, v4);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Single tokens (decode steps, short prompt portions): one workgroup per (token, kv head, sixteen
// query heads of its group, split of the key range).  The rows of the products are the query
// heads that share the kv head; the wavefronts of the workgroup take the 32-key steps of the
// range in turn, each with a running (maximum, sum, output) of its own, and meet in LDS at the
// end, so a whole key range needs no second kernel.  Each wavefront stages its own V tile: no
// workgroup barrier inside the loop.
#define DEC_WAVES (HEAD_DIM <= 128 ? 4 : 2)
#if !HEAD_HALF

// (Asked for four wavefronts a SIMD at head size 64, the compiler fits the kernel into 122 registers instead of 148
// without spilling, and a compute unit holds four workgroups instead of three: 11.5 -> 10.8 us at batch 8.)
template <bool POW2>
__global__ __launch_bounds__(DEC_WAVES * WAVE) __attribute__((amdgpu_waves_per_eu(HEAD_DIM <= 64 ? 4 : 2)))
void mfma_decode_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ kpool, const bf16_t* __restrict__ vpool,
    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ positions, bf16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, int H, int KVH, int page_size, int page_shift, int window, float scale, int nsplit) {
    constexpr int HD = HEAD_DIM;
    constexpr int NW = DEC_WAVES;
    constexpr int THREADS = NW * WAVE;
    constexpr int KK = HD / 32;
    constexpr int DT = HD / 16;
    constexpr int VROW = HD + VPAD;
    __shared__ __attribute__((aligned(16))) uint16_t vs[NW][KSTEP][VROW];  // per wavefront: V of its step, [key][dim]
    __shared__ float sm_ml[NW][16][2];
    static_assert(KSTEP * VROW * 2 >= 16 * HD * 4, "a wavefront's V tile is reused for its 16 x HD partial output");

    // Uncut key ranges of many tokens: the chip holds the grid two workgroups a compute unit, u and u + half the grid,
    // which is the same x in the lower and the upper half of y.  The upper half takes the tokens from the far end, so
    // that a caller who brings the tokens in the order of their contexts gets a long and a short one on every unit.
    const int t = (gridDim.z == 1 && gridDim.y > 1 && 2 * blockIdx.y >= gridDim.y) ? gridDim.x - 1 - blockIdx.x : blockIdx.x;
    const int G = H / KVH;
    const int chunks = (G + 15) / 16;
    const int g = blockIdx.y / chunks;
    const int chunk = blockIdx.y % chunks;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;      // the same in every lane: say so
    const int r = lane % 16, kg = lane / 16;
    const int hh = chunk * 16 + r;                   // this lane's row: a query head of the group
    const bool row_ok = hh < G;
    const int head = g * G + hh;

    const int pos = positions[t];
    const int seq = seq_of_token[t];
    const int hi = pos + 1;
    const int lo = window > 0 ? max(0, hi - window) : 0;
    const int kbeg = lo / KSTEP * KSTEP;
    const int nsteps_all = (hi - kbeg + KSTEP - 1) / KSTEP;
    const int per_split = (nsteps_all + nsplit - 1) / nsplit;
    const int s_begin = blockIdx.z * per_split;
    const int nsteps = max(0, min(nsteps_all, s_begin + per_split) - s_begin);
    const int kfirst = kbeg + s_begin * KSTEP;
    const float scale2 = scale * LOG2E;

    const int32_t* table = block_table + static_cast<size_t>(seq) * table_stride;
    auto page_of = [&](int key) { return POW2 ? (key >> page_shift) : key / page_size; };
    auto slot_of = [&](int key) { return POW2 ? (key & (page_size - 1)) : key % page_size; };
    constexpr int TBL_MAX = 1024;
    __shared__ int32_t tbl[TBL_MAX];
    int key_lo = 0, key_hi = 0, lp0 = 0;
    auto row_address = [&](int key) -> size_t {
        // clamped to keys the token may read: those before `lo` may lie in pages already given back
        const int kc = min(max(key, max(key_lo, lo)), key_hi);
        const int page = tbl[page_of(kc) - lp0];
        // the row's number fits 32 bits (the host checks the pool's size); one widening multiply makes the offset
        const uint32_t row = (static_cast<uint32_t>(max(page, 0)) * KVH + g) * page_size + slot_of(kc);
        return static_cast<size_t>(row) * HD;
    };

    uint4 qf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        if (row_ok)
            qf[kk] = *reinterpret_cast<const uint4*>(q + static_cast<size_t>(t) * q_stride + static_cast<size_t>(head) * HD +
                                                     kk * 32 + kg * 8);
        else
            qf[kk] = make_uint4(0, 0, 0, 0);
    }

    float m_run = NEG_BIG;
    floatx4_t l_run = floatx4_t{0.f, 0.f, 0.f, 0.f};
    floatx4_t o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // a lane loads 8 dims of one key (16 bytes) HD/16 times a step, neighbouring lanes neighbouring pieces
    // of a row, and writes them to LDS as they are; the second product takes its operand from there by
    // transposing reads
    constexpr int V_PER_LANE = HD / 16;
    constexpr int PIECES = HD / 8;
    auto load_v = [&](int ks, u32x4_t (&dst)[V_PER_LANE]) {
#pragma unroll
        for (int i = 0; i < V_PER_LANE; ++i) {
            const int item = lane + i * WAVE;
            dst[i] = *reinterpret_cast<const u32x4_t*>(vpool + row_address(ks + item % KSTEP) + (item / KSTEP) * 8);
        }
    };
    auto store_v = [&](const u32x4_t (&src)[V_PER_LANE]) {
#pragma unroll
        for (int i = 0; i < V_PER_LANE; ++i) {
            const int item = lane + i * WAVE;
            *reinterpret_cast<u32x4_t*>(&vs[wave][item % KSTEP][(item / KSTEP) * 8]) = src[i];
        }
    };
    auto load_k = [&](int ks, uint4 (&dst)[2][KK]) {
#pragma unroll
        for (int tile = 0; tile < 2; ++tile) {
            const size_t base = row_address(ks + tile * 16 + r);
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) dst[tile][kk] = *reinterpret_cast<const uint4*>(kpool + base + kk * 32 + kg * 8);
        }
    };
    // the lanes of one wavefront run together: ordering its own LDS writes before its reads takes no barrier
    auto wave_sync = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    constexpr int DEPTH = 2;      // steps whose rows wait in registers ahead of the arithmetic: more (four at head size 64, three at 128) left
                                  // fewer workgroups on a compute unit and were slower at every batch, most of all where the context lengths differ
    uint4 kf[DEPTH][2][KK];
    u32x4_t vr[DEPTH][V_PER_LANE];
    for (int seg0 = 0; seg0 < nsteps;) {
        key_lo = kfirst + seg0 * KSTEP;
        lp0 = page_of(key_lo);
        const int seg_steps = min(nsteps - seg0, ((lp0 + TBL_MAX) * page_size - key_lo) / KSTEP);
        key_hi = min(key_lo + seg_steps * KSTEP, hi) - 1;
        __syncthreads();
        for (int i = tid; i <= page_of(key_hi) - lp0; i += THREADS) tbl[i] = table[lp0 + i];
        __syncthreads();
        // this wavefront's steps of the segment: wave, wave + NW, ...
        const int mine = seg_steps > wave ? (seg_steps - wave + NW - 1) / NW : 0;
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            load_k(key_lo + (wave + d * NW) * KSTEP, kf[d]);
            load_v(key_lo + (wave + d * NW) * KSTEP, vr[d]);
        }
        // Step j lives in slot j % DEPTH of the ring; the loop is unrolled DEPTH times so that a slot
        // is a fixed set of registers (rotating the ring by copies would wait for the newest loads).
        // A slot is asked for its next rows as soon as its step has used it.
        auto step = [&](int j, uint4 (&kslot)[2][KK], u32x4_t (&vslot)[V_PER_LANE]) {
            const int ks = key_lo + (wave + j * NW) * KSTEP;
            if (j < mine) {
                wave_sync();                       // the reads of the previous step are done
                store_v(vslot);
                floatx4_t st[2];
#pragma unroll
                for (int tile = 0; tile < 2; ++tile) {
                    st[tile] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int kk = 0; kk < KK; ++kk)
                        st[tile] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kslot[tile][kk]),
                                                                           __builtin_bit_cast(bf16x8_t, qf[kk]), st[tile], 0, 0, 0);
                }
                const bool inner = ks >= lo && ks + KSTEP - 1 <= pos;
                float raw[8];
                const float lane_max = inner ? mask_scores<false>(st, ks + kg * 4, lo, pos, row_ok, raw)
                                             : mask_scores<true>(st, ks + kg * 4, lo, pos, row_ok, raw);
                if (__any(above_reference(lane_max, scale2, m_run))) {      // some row has risen far above its reference
                    const float corr = move_reference(lane_max, scale2, m_run);
                    l_run *= corr;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) o[dt] *= corr;
                }
                const uint4 pf = inner ? weights<false>(raw, scale2, m_run) : weights<true>(raw, scale2, m_run);
                l_run = row_sum_step(pf, l_run);
                wave_sync();                       // V of this step is in LDS
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const uint4 vf = read_v_operand(&vs[wave][0][0], VROW, dt * 16, r, kg);
                    o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vf),
                                                                    __builtin_bit_cast(bf16x8_t, pf), o[dt], 0, 0, 0);
                }
            }
            load_k(ks + DEPTH * NW * KSTEP, kslot);
            load_v(ks + DEPTH * NW * KSTEP, vslot);
        };
        for (int j0 = 0; j0 < mine; j0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) step(j0 + d, kf[d], vr[d]);
        }
        seg0 += seg_steps;
    }

    // wavefronts meet: every one leaves (maximum, sum) of its rows and its 16 x HD output in LDS
    __syncthreads();                           // every wavefront is done with its V tile
    float* so = reinterpret_cast<float*>(&vs[wave][0][0]);          // [16][HD]
    if (kg == 0) { sm_ml[wave][r][0] = m_run; sm_ml[wave][r][1] = l_run[0]; }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
        *reinterpret_cast<float4*>(so + r * HD + dt * 16 + kg * 4) = make_float4(o[dt][0], o[dt][1], o[dt][2], o[dt][3]);
    __syncthreads();
    const int rows = min(16, G - chunk * 16);
    for (int idx = tid; idx < rows * HD; idx += THREADS) {
        const int row = idx / HD, dim = idx % HD;
        float M = sm_ml[0][row][0];
#pragma unroll
        for (int w = 1; w < NW; ++w) M = fmaxf(M, sm_ml[w][row][0]);
        float Lsum = 0.f, O = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float f = __builtin_amdgcn_exp2f(sm_ml[w][row][0] - M);
            Lsum += sm_ml[w][row][1] * f;
            O += reinterpret_cast<const float*>(&vs[w][0][0])[row * HD + dim] * f;
        }
        const int h = g * G + chunk * 16 + row;
        if (nsplit == 1) {
            st(out + static_cast<size_t>(t) * H * HD + static_cast<size_t>(h) * HD + dim, O / Lsum);
        } else {
            const size_t p = (static_cast<size_t>(t) * H + h) * nsplit + blockIdx.z;
            part_o[p * HD + dim] = O;
            if (dim == 0) { part_ml[p * 2] = M * LN2; part_ml[p * 2 + 1] = Lsum; }     // the merge kernel works in base e
        }
    }
}

#endif   // !HEAD_HALF

NI_EXPORT int ni_mfma_attention_head_dim() { return HEAD_DIM; }

// Blocks of 16 rows that a wavefront can own at this head size.  Registers set the limit: two
// blocks at head size 128, or four at 64, fit only with the accumulators parked in the accumulation
// registers and one wavefront a SIMD, and were slower than one block in every case measured.
#define MA_MAX_BLOCKS (HEAD_DIM <= 64 ? 2 : 1)
NI_EXPORT int ni_mfma_attention_max_blocks() { return MA_MAX_BLOCKS; }

static int heads_per_tile(int group) { return group >= 16 ? 16 : group > 4 ? 8 : group > 2 ? 4 : group > 1 ? 2 : 1; }

// Tokens of one tile for a model with `group` query heads per kv head, when a wavefront owns
// `blocks` blocks of 16 rows (1 or 2, at most ni_mfma_attention_max_blocks()).
NI_EXPORT int ni_mfma_attention_tile_tokens(int group, int blocks) {
    return MA_WAVES * blocks * (16 / heads_per_tile(group));
}

// tiles: QTile [n_tiles] built by the host from the portions of the step with the tile size above
// (for the same `blocks`), sorted by the number of keys a tile walks, longest first (any order
// gives the same result; this one an even spread of the work).  With nsplit > 1 the key range of every tile is cut into nsplit runs;
// partial results go to part_o (float [T, H, nsplit, HEAD_DIM]) and part_ml (float [T, H, nsplit, 2])
// and `out` is left to the merge kernel of the token-at-a-time library (same layout).
NI_EXPORT int ni_mfma_attention(const void* q, int q_stride, const void* kpool, const void* vpool, const void* block_table,
                                int table_stride, const void* tiles, int n_tiles, void* out, void* part_o, void* part_ml,
                                int H, int KVH, int page_size, int window, float scale, int nsplit, int blocks,
                                hipStream_t stream) {
    if (n_tiles <= 0) return 0;
    if (H % KVH != 0 || page_size < 1 || nsplit < 1 || nsplit > 64 || !(scale > 0.f)) return -1;
    if (nsplit > 1 && (!part_o || !part_ml)) return -2;
    if (blocks < 1 || blocks > MA_MAX_BLOCKS) return -3;
    const int G = H / KVH;
    const int hpt = heads_per_tile(G);
    int hpt_shift = 0;
    while ((1 << hpt_shift) < hpt) ++hpt_shift;
    const int chunks = (G + hpt - 1) / hpt;
    // a page size that is a power of two gets shifts and masks, any other divisions
    const bool pow2 = (page_size & (page_size - 1)) == 0;
    int page_shift = 0;
    while (pow2 && (1 << page_shift) < page_size) ++page_shift;
    const int per_tile = KVH * chunks * nsplit;
    // As many workgroups as the chip holds at once (asked of the runtime once per kernel), each walking
    // through its share of the sorted tiles.
#define MA_LAUNCH(CB_)                                                                                              \
    {                                                                                                               \
        auto kernel = pow2 ? mfma_attention_kernel<CB_, true> : mfma_attention_kernel<CB_, false>;                 \
        static int slots[2] = {0, 0}, units[2] = {0, 0};                                                            \
        if (slots[pow2] == 0) {                                                                                     \
            int dev = 0, cus = 0, per_cu = 0;                                                                       \
            if (hipGetDevice(&dev) != hipSuccess ||                                                                 \
                hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||            \
                hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, MA_WAVES * WAVE, 0) != hipSuccess ||  \
                cus < 1 || per_cu < 1)                                                                              \
                return -4;                                                                                          \
            units[pow2] = cus;                                                                                      \
            slots[pow2] = cus * per_cu;                                                                             \
        }                                                                                                           \
        /* with no more tiles than the chip holds workgroups every tile gets one (the kernel pairs them over the */  \
        /* compute units); else two rounds pair long tiles with short ones, or more, as few as fit the chip:      */  \
        /* three rounds leave more workgroups on the chip than four, and their shares differ by less than a tile  */  \
        int rounds = 1;                                                                                             \
        if (n_tiles * per_tile > slots[pow2]) {                                                                     \
            rounds = 2;                                                                                             \
            while ((n_tiles + rounds - 1) / rounds * per_tile > slots[pow2] && rounds < n_tiles) rounds += 1;       \
        }                                                                                                           \
        const int in_x = (n_tiles + rounds - 1) / rounds;                                                           \
        dim3 grid(in_x, KVH * chunks, nsplit);                                                                      \
        kernel<<<grid, MA_WAVES * WAVE, 0, stream>>>(                                                               \
            (const bf16_t*)q, q_stride, (const bf16_t*)kpool, (const bf16_t*)vpool, (const int32_t*)block_table,   \
            table_stride, (const QTile*)tiles, n_tiles, (bf16_t*)out, (float*)part_o, (float*)part_ml, H, KVH,     \
            page_size, page_shift, hpt_shift, window, scale, nsplit);                                               \
    }
    if (blocks == 1) MA_LAUNCH(1)
#if HEAD_DIM <= 64
    else MA_LAUNCH(2)
#endif
#undef MA_LAUNCH
    return NI_LAUNCH_RESULT();
}

// Attention of single tokens on the matrix cores: same arguments and partial-result layout as the
// token-at-a-time kernel (`out` is left to its merge kernel when nsplit > 1).
NI_EXPORT int ni_mfma_token_attention(const void* q, int q_stride, const void* kpool, const void* vpool,
                                      const void* block_table, int table_stride, const void* seq_of_token,
                                      const void* positions, void* out, void* part_o, void* part_ml, int T_tokens,
                                      int H, int KVH, int page_size, int window, float scale, int nsplit,
                                      hipStream_t stream) {
#if HEAD_HALF
    return -5;          // single tokens at this head size are the token-at-a-time kernel's
#else
    if (T_tokens <= 0) return 0;
    if (H % KVH != 0 || page_size < 1 || nsplit < 1 || nsplit > 65535 || !(scale > 0.f)) return -1;
    if (nsplit > 1 && (!part_o || !part_ml)) return -2;
    const int G = H / KVH;
    const int chunks = (G + 15) / 16;
    const bool pow2 = (page_size & (page_size - 1)) == 0;
    int page_shift = 0;
    while (pow2 && (1 << page_shift) < page_size) ++page_shift;
    dim3 grid(T_tokens, KVH * chunks, nsplit);
    auto kernel = pow2 ? mfma_decode_kernel<true> : mfma_decode_kernel<false>;
    kernel<<<grid, DEC_WAVES * WAVE, 0, stream>>>(
        (const bf16_t*)q, q_stride, (const bf16_t*)kpool, (const bf16_t*)vpool, (const int32_t*)block_table, table_stride,
        (const int32_t*)seq_of_token, (const int32_t*)positions, (bf16_t*)out, (float*)part_o, (float*)part_ml, H, KVH,
        page_size, page_shift, window, scale, nsplit);
    return NI_LAUNCH_RESULT();
#endif
}
