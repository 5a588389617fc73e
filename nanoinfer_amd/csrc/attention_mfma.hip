// Attention of prompt portions over the paged key/value cache on the matrix cores of gfx950.
// bfloat16 only; compiled once per head size (-DHEAD_DIM=n, a multiple of 32 up to 256).
//
// A workgroup of four wavefronts owns one tile of consecutive tokens of one sequence and the
// query heads of one kv head (HPT of them at a time).  A wavefront owns 16 "rows": TPT = 16/HPT
// tokens times HPT heads, all reading the same keys and values.  Keys are walked 32 at a time:
//
//   S^T[key, row]  = K[key, :] . Q[row, :]       v_mfma_f32_16x16x32_bf16, K rows straight from
//                                                 global memory as the A operand, Q as B
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

#ifndef HEAD_DIM
#error "HEAD_DIM must be defined"
#endif
static_assert(HEAD_DIM % 32 == 0 && HEAD_DIM >= 32 && HEAD_DIM <= 256, "head size: multiple of 32, at most 256");

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

#define KSTEP 32
#define MA_WAVES 4
#define NEG_BIG (-1.0e30f)
#define VPAD 8   // elements of padding per staged row of V^T: the sixteen rows of a 16-byte read fall on different banks

struct QTile { int32_t seq, row0, ntok, pos0; };   // tokens row0..row0+ntok-1 of the batch, positions pos0..

#define LOG2E 1.4426950408889634f
#define LN2 0.6931471805599453f

// One 32-key step of the online softmax for a lane that holds eight scores of one row (keys
// key0 + t*16 + i of the two 16-key halves).  Maximum and sum are kept in the base-2 domain
// (scores are scaled by scale*log2(e)), so an exponential is one v_exp_f32.  MASKED steps are the
// ones at the edges of a row's key range [lo, pos]; in the others every key counts and no
// comparison is made.  Returns the weights rounded to bfloat16, laid out as the B operand of the
// second product; the sum is taken over the rounded weights, the ones that product uses, so the
// output is an exact convex combination of values whatever the rounding.
template <bool MASKED>
__device__ __forceinline__ uint4 softmax_step(const floatx4_t (&st)[2], float scale2, int key0, int lo, int pos,
                                              bool row_ok, float& m_run, float& l_run, float& corr) {
    float sc[8];
    float mx = NEG_BIG;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = st[t][i] * scale2;
            if constexpr (MASKED) {
                const int key = key0 + t * 16 + i;
                v = (row_ok && key <= pos && key >= lo) ? v : NEG_BIG;
            }
            sc[t * 4 + i] = v;
            mx = fmaxf(mx, v);
        }
    mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
    const float m_new = fmaxf(m_run, mx);
    corr = __builtin_amdgcn_exp2f(m_run - m_new);
    float psum = 0.f;
    uint32_t pw[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float p0 = __builtin_amdgcn_exp2f(sc[2 * j] - m_new), p1 = __builtin_amdgcn_exp2f(sc[2 * j + 1] - m_new);
        if constexpr (MASKED) {
            p0 = sc[2 * j] > 0.5f * NEG_BIG ? p0 : 0.f;
            p1 = sc[2 * j + 1] > 0.5f * NEG_BIG ? p1 : 0.f;
        }
        pw[j] = pack_bf16x2(p0, p1);
        psum += __uint_as_float(pw[j] << 16) + __uint_as_float(pw[j] & 0xffff0000u);
    }
    l_run = l_run * corr + psum;
    m_run = m_new;
    return make_uint4(pw[0], pw[1], pw[2], pw[3]);
}

template <int HPT, bool POW2>
__global__ __launch_bounds__(MA_WAVES * WAVE) void mfma_attention_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ kpool, const bf16_t* __restrict__ vpool,
    const int32_t* __restrict__ block_table, int table_stride, const QTile* __restrict__ tiles,
    bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml, int H, int KVH, int page_size,
    int page_shift, int window, float scale, int nsplit) {
    constexpr int HD = HEAD_DIM;
    constexpr int MA_THREADS = MA_WAVES * WAVE;
    constexpr int TPT = 16 / HPT;            // tokens of a wavefront
    constexpr int KK = HD / 32;              // k steps of the first product
    constexpr int DT = HD / 16;              // 16-wide tiles of the head dimension in the output
    constexpr int VROW = KSTEP + VPAD;
    __shared__ __attribute__((aligned(16))) uint16_t vs[2][HD][VROW];      // V^T of a step: [dim][key, in the lanes' order]

    // the tiles of a portion come in the order of their positions, and a later tile has more keys to
    // walk: the workgroups take them last first, so that the long ones start early and the short ones
    // fill the end of the launch
    const QTile tile = tiles[gridDim.x - 1 - blockIdx.x];
    const int G = H / KVH;
    const int chunks = (G + HPT - 1) / HPT;
    const int g = blockIdx.y / chunks;
    const int chunk = blockIdx.y % chunks;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;      // the same in every lane: say so
    const int r = lane % 16, kg = lane / 16;

    // this lane's row: one (token, head) pair
    const int tt = wave * TPT + r / HPT;                 // token within the tile
    const int hh = chunk * HPT + r % HPT;                // head within the group
    const bool row_ok = tt < tile.ntok && hh < G;
    const int head = g * G + hh;
    const int pos = tile.pos0 + tt;
    const int row_lo = (row_ok && window > 0) ? max(0, pos + 1 - window) : 0;

    // key range of the workgroup (uniform), walked in steps of 32 from a multiple of 32
    const int kend = tile.pos0 + tile.ntok;
    const int kbeg = (window > 0 ? max(0, tile.pos0 + 1 - window) : 0) / KSTEP * KSTEP;
    const int nsteps_all = (kend - kbeg + KSTEP - 1) / KSTEP;
    // a split (blockIdx.z) takes a contiguous run of steps
    const int per_split = (nsteps_all + nsplit - 1) / nsplit;
    const int s_begin = blockIdx.z * per_split;
    const int nsteps = max(0, min(nsteps_all, s_begin + per_split) - s_begin);
    const int kfirst = kbeg + s_begin * KSTEP;
    // last position any row of this wavefront has: steps beyond it are skipped by the wavefront
    const int wave_tok_hi = min(tile.ntok, (wave + 1) * TPT) - 1;
    const bool wave_ok = wave * TPT < tile.ntok;
    const int wave_pmax = tile.pos0 + wave_tok_hi;
    // steps whose 32 keys lie inside the key range of every row of the wavefront need no masking
    const int wave_pmin = tile.pos0 + wave * TPT;
    const int wave_lo_max = window > 0 ? max(0, wave_pmax + 1 - window) : 0;
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
    auto row_address = [&](int key) -> size_t {       // offset of key's row for kv head g, key clamped into the segment
        const int kc = min(max(key, key_lo), key_hi);
        const int page = tbl[page_of(kc) - lp0];
        // the row's number fits 32 bits (the host checks the pool's size); one widening multiply makes the offset
        const uint32_t row = (static_cast<uint32_t>(max(page, 0)) * KVH + g) * page_size + slot_of(kc);
        return static_cast<size_t>(row) * HD;
    };

    // Q as the B operand: lane (row r, group kg) holds dims kk*32 + kg*8 .. +8
    uint4 qf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        if (row_ok)
            qf[kk] = *reinterpret_cast<const uint4*>(q + static_cast<size_t>(tile.row0 + tt) * q_stride +
                                                     static_cast<size_t>(head) * HD + kk * 32 + kg * 8);
        else
            qf[kk] = make_uint4(0, 0, 0, 0);
    }

    float m_run = NEG_BIG, l_run = 0.f;
    floatx4_t o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // Staging of V: a thread loads 8 dims of one key (16 bytes) and writes them to LDS transposed,
    // at the column where the lanes of the second product expect that key: lane group kg reads
    // the eight keys {t*16 + kg*4 + i} as one 16-byte row piece [kg*8 + t*4 + i].  A wavefront
    // covers all 32 keys and two 8-dim chunks, which spreads its 2-byte writes over the banks.
    constexpr int CHUNKS = HD / 8;
    constexpr int V_ITEMS = KSTEP * CHUNKS;
    constexpr int V_PER_THREAD = (V_ITEMS + MA_THREADS - 1) / MA_THREADS;
    auto load_v = [&](int ks, uint4 (&dst)[V_PER_THREAD]) {
#pragma unroll
        for (int i = 0; i < V_PER_THREAD; ++i) {
            const int item = tid + i * MA_THREADS;
            if (item < V_ITEMS)
                dst[i] = *reinterpret_cast<const uint4*>(vpool + row_address(ks + item % KSTEP) + (item / KSTEP) * 8);
        }
    };
    auto store_v = [&](int buf, const uint4 (&src)[V_PER_THREAD]) {
#pragma unroll
        for (int i = 0; i < V_PER_THREAD; ++i) {
            const int item = tid + i * MA_THREADS;
            if (item < V_ITEMS) {
                const int key = item % KSTEP, dim0 = (item / KSTEP) * 8;
                const int col = ((key % 16) / 4) * 8 + (key / 16) * 4 + key % 4;
                const uint32_t w[4] = {src[i].x, src[i].y, src[i].z, src[i].w};
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    vs[buf][dim0 + e][col] = static_cast<uint16_t>(e & 1 ? w[e / 2] >> 16 : w[e / 2] & 0xffffu);
            }
        }
    };
    // K as the A operand: lane (key r of a 16-key half, group kg) holds dims kk*32 + kg*8 .. +8
    auto load_k = [&](int ks, uint4 (&dst)[2][KK]) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const size_t base = row_address(ks + t * 16 + r);
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) dst[t][kk] = *reinterpret_cast<const uint4*>(kpool + base + kk * 32 + kg * 8);
        }
    };

    // Loads run DEPTH - 1 steps ahead of the arithmetic: rows wait in registers (a ring of DEPTH
    // slots) while older steps are multiplied, so a step costs its arithmetic, not a memory round
    // trip.  V of step s+1 is written to LDS during step s.
    constexpr int DEPTH = 4;
    uint4 kf[DEPTH][2][KK];
    uint4 vr[DEPTH][V_PER_THREAD];
    for (int seg0 = 0; seg0 < nsteps;) {
        key_lo = kfirst + seg0 * KSTEP;
        lp0 = page_of(key_lo);
        const int seg_steps = min(nsteps - seg0, ((lp0 + TBL_MAX) * page_size - key_lo) / KSTEP);
        key_hi = min(key_lo + seg_steps * KSTEP, kend) - 1;
        __syncthreads();                   // nobody still reads the previous segment's table or V tiles
        for (int i = tid; i <= page_of(key_hi) - lp0; i += MA_THREADS) tbl[i] = table[lp0 + i];
        __syncthreads();
        // rows past the end of the segment are read from its last key and not used: no load is under a branch
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            load_k(key_lo + d * KSTEP, kf[d]);
            load_v(key_lo + d * KSTEP, vr[d]);
        }
        store_v(0, vr[0]);
        load_v(key_lo + DEPTH * KSTEP, vr[0]);
        // Step s uses K from slot s % DEPTH of the ring and writes V of step s + 1 (slot (s + 1) % DEPTH)
        // to LDS.  The loop is unrolled DEPTH times so that a slot is a fixed set of registers: rotating
        // the ring by copies would wait for the newest loads.  A slot is asked for its next rows as
        // soon as its step has used it.
        auto step = [&](int s, uint4 (&kslot)[2][KK], uint4 (&vnext)[V_PER_THREAD]) {
            const int ks = key_lo + s * KSTEP;
            if (s < seg_steps) {
                // V of this step is in vs[s & 1]; nobody still reads the other buffer.  Only LDS is ordered
                // here: a full barrier would also wait for every row load that is in flight for later steps.
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
                if (wave_ok && ks <= wave_pmax) {
                    // S^T for the two 16-key halves
                    floatx4_t st[2];
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        st[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int kk = 0; kk < KK; ++kk)
                            st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kslot[t][kk]),
                                                                            __builtin_bit_cast(bf16x8_t, qf[kk]), st[t], 0, 0, 0);
                    }
                    // this lane: row r, keys ks + t*16 + kg*4 + i
                    float corr;
                    const bool inner = ks >= wave_lo_max && ks + KSTEP - 1 <= wave_pmin;
                    const uint4 pf = inner ? softmax_step<false>(st, scale2, ks + kg * 4, row_lo, pos, row_ok, m_run, l_run, corr)
                                           : softmax_step<true>(st, scale2, ks + kg * 4, row_lo, pos, row_ok, m_run, l_run, corr);
                    const bool rescale = __any(corr != 1.0f);      // the maximum of some row has moved
                    // O^T += V^T . P^T : the A operand of lane (dim r of a 16-dim tile, group kg) is V[key_j][dim]
                    // for the same eight keys, in the same order, as the lane's scores
                    const uint16_t (*vb)[VROW] = vs[s & 1];
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        const uint4 vf = *reinterpret_cast<const uint4*>(&vb[dt * 16 + r][kg * 8]);
                        if (rescale) o[dt] *= corr;
                        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vf),
                                                                        __builtin_bit_cast(bf16x8_t, pf), o[dt], 0, 0, 0);
                    }
                }
                store_v((s + 1) & 1, vnext);
            }
            load_k(ks + DEPTH * KSTEP, kslot);
            load_v(ks + (DEPTH + 1) * KSTEP, vnext);
        };
        for (int s0 = 0; s0 < seg_steps; s0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) step(s0 + d, kf[d], vr[(d + 1) % DEPTH]);
        }
        seg0 += seg_steps;
    }

    // the sum of a row is spread over the four lanes that share it
    l_run += __shfl_xor(l_run, 16, WAVE);
    l_run += __shfl_xor(l_run, 32, WAVE);
    if (nsplit > 1) {
        // partial (maximum, sum, unnormalised output) of this split, merged by a second kernel
        if (row_ok) {
            const size_t p = (static_cast<size_t>(tile.row0 + tt) * H + head) * nsplit + blockIdx.z;
            if (kg == 0) { part_ml[p * 2] = m_run * LN2; part_ml[p * 2 + 1] = l_run; }     // the merge kernel works in base e
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                *reinterpret_cast<float4*>(part_o + p * HD + dt * 16 + kg * 4) = make_float4(o[dt][0], o[dt][1], o[dt][2], o[dt][3]);
        }
        return;
    }
    if (row_ok && l_run > 0.f) {
        const float inv = 1.0f / l_run;
        bf16_t* dst = out + static_cast<size_t>(tile.row0 + tt) * H * HD + static_cast<size_t>(head) * HD;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            float v4[4] = {o[dt][0] * inv, o[dt][1] * inv, o[dt][2] * inv, o[dt][3] * inv};
            VecIO<bf16_t, 4>::store(dst + dt * 16 + kg * 4, v4);
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

template <bool POW2>
__global__ __launch_bounds__(DEC_WAVES * WAVE) void mfma_decode_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ kpool, const bf16_t* __restrict__ vpool,
    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ positions, bf16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, int H, int KVH, int page_size, int page_shift, int window, float scale, int nsplit) {
    constexpr int HD = HEAD_DIM;
    constexpr int NW = DEC_WAVES;
    constexpr int THREADS = NW * WAVE;
    constexpr int KK = HD / 32;
    constexpr int DT = HD / 16;
    constexpr int VROW = KSTEP + VPAD;
    __shared__ __attribute__((aligned(16))) uint16_t vs[NW][HD][VROW];     // per wavefront: V^T of its step
    __shared__ float sm_ml[NW][16][2];
    static_assert(HD * VROW * 2 >= 16 * HD * 4, "a wavefront's V tile is reused for its 16 x HD partial output");

    const int t = blockIdx.x;
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
        const int kc = min(max(key, key_lo), key_hi);
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

    float m_run = NEG_BIG, l_run = 0.f;
    floatx4_t o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // a lane loads 8 dims of one key (16 bytes) HD/16 times a step and writes them to LDS transposed
    constexpr int V_PER_LANE = HD / 16;
    auto load_v = [&](int ks, uint4 (&dst)[V_PER_LANE]) {
#pragma unroll
        for (int i = 0; i < V_PER_LANE; ++i) {
            const int item = lane + i * WAVE;
            dst[i] = *reinterpret_cast<const uint4*>(vpool + row_address(ks + item % KSTEP) + (item / KSTEP) * 8);
        }
    };
    auto store_v = [&](const uint4 (&src)[V_PER_LANE]) {
#pragma unroll
        for (int i = 0; i < V_PER_LANE; ++i) {
            const int item = lane + i * WAVE;
            const int key = item % KSTEP, dim0 = (item / KSTEP) * 8;
            const int col = ((key % 16) / 4) * 8 + (key / 16) * 4 + key % 4;
            const uint32_t w[4] = {src[i].x, src[i].y, src[i].z, src[i].w};
#pragma unroll
            for (int e = 0; e < 8; ++e)
                vs[wave][dim0 + e][col] = static_cast<uint16_t>(e & 1 ? w[e / 2] >> 16 : w[e / 2] & 0xffffu);
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

    constexpr int DEPTH = HD <= 64 ? 4 : HD <= 128 ? 3 : 2;
    uint4 kf[DEPTH][2][KK];
    uint4 vr[DEPTH][V_PER_LANE];
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
        auto step = [&](int j, uint4 (&kslot)[2][KK], uint4 (&vslot)[V_PER_LANE]) {
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
                float corr;
                const bool inner = ks >= lo && ks + KSTEP - 1 <= pos;
                const uint4 pf = inner ? softmax_step<false>(st, scale2, ks + kg * 4, lo, pos, row_ok, m_run, l_run, corr)
                                       : softmax_step<true>(st, scale2, ks + kg * 4, lo, pos, row_ok, m_run, l_run, corr);
                const bool rescale = __any(corr != 1.0f);      // the maximum of some row has moved
                wave_sync();                       // V^T of this step is in LDS
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const uint4 vf = *reinterpret_cast<const uint4*>(&vs[wave][dt * 16 + r][kg * 8]);
                    if (rescale) o[dt] *= corr;
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

    // the sum of a row is spread over the four lanes that share it
    l_run += __shfl_xor(l_run, 16, WAVE);
    l_run += __shfl_xor(l_run, 32, WAVE);
    // wavefronts meet: every one leaves (maximum, sum) of its rows and its 16 x HD output in LDS
    __syncthreads();                           // every wavefront is done with its V tile
    float* so = reinterpret_cast<float*>(&vs[wave][0][0]);          // [16][HD]
    if (kg == 0) { sm_ml[wave][r][0] = m_run; sm_ml[wave][r][1] = l_run; }
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

NI_EXPORT int ni_mfma_attention_head_dim() { return HEAD_DIM; }

// Tokens of one tile for a model with `group` query heads per kv head.
NI_EXPORT int ni_mfma_attention_tile_tokens(int group) {
    const int hpt = group >= 16 ? 16 : group > 4 ? 8 : group > 2 ? 4 : group > 1 ? 2 : 1;
    return MA_WAVES * (16 / hpt);
}

// tiles: QTile [n_tiles] built by the host from the portions of the step with the tile size above.
// With nsplit > 1 the key range of every tile is cut into nsplit runs; partial results go to part_o
// (float [T, H, nsplit, HEAD_DIM]) and part_ml (float [T, H, nsplit, 2]) and `out` is left to the
// merge kernel of the token-at-a-time library (same layout).
NI_EXPORT int ni_mfma_attention(const void* q, int q_stride, const void* kpool, const void* vpool, const void* block_table,
                                int table_stride, const void* tiles, int n_tiles, void* out, void* part_o, void* part_ml,
                                int H, int KVH, int page_size, int window, float scale, int nsplit, hipStream_t stream) {
    if (n_tiles <= 0) return 0;
    if (H % KVH != 0 || page_size < 1 || nsplit < 1 || nsplit > 64) return -1;
    if (nsplit > 1 && (!part_o || !part_ml)) return -2;
    const int G = H / KVH;
    const int hpt = G >= 16 ? 16 : G > 4 ? 8 : G > 2 ? 4 : G > 1 ? 2 : 1;
    const int chunks = (G + hpt - 1) / hpt;
    // a page size that is a power of two gets shifts and masks, any other divisions
    const bool pow2 = (page_size & (page_size - 1)) == 0;
    int page_shift = 0;
    while (pow2 && (1 << page_shift) < page_size) ++page_shift;
    dim3 grid(n_tiles, KVH * chunks, nsplit);
#define MA_LAUNCH(HPT_)                                                                                             \
    {                                                                                                               \
        auto kernel = pow2 ? mfma_attention_kernel<HPT_, true> : mfma_attention_kernel<HPT_, false>;               \
        kernel<<<grid, MA_WAVES * WAVE, 0, stream>>>(                                                               \
            (const bf16_t*)q, q_stride, (const bf16_t*)kpool, (const bf16_t*)vpool, (const int32_t*)block_table,   \
            table_stride, (const QTile*)tiles, (bf16_t*)out, (float*)part_o, (float*)part_ml, H, KVH, page_size,   \
            page_shift, window, scale, nsplit);                                                                     \
    }
    switch (hpt) {
        case 1: MA_LAUNCH(1); break;
        case 2: MA_LAUNCH(2); break;
        case 4: MA_LAUNCH(4); break;
        case 8: MA_LAUNCH(8); break;
        default: MA_LAUNCH(16); break;
    }
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
    if (T_tokens <= 0) return 0;
    if (H % KVH != 0 || page_size < 1 || nsplit < 1 || nsplit > 65535) return -1;
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
}
