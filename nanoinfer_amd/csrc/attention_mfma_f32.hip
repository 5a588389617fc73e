// Attention over the paged key/value cache on the matrix cores of gfx950, in true float32: both
// products by v_mfma_f32_16x16x4_f32, softmax with the accurate exponential.  Compiled once per
// head size (-DHEAD_DIM=n, a multiple of 16 up to 256).  The float32 twins of the bfloat16 kernels
// of attention_mfma.hip, with the same tiles and the same interfaces: first the kernel for prompt
// portions, described here; at the end of the file the one for single tokens.
//
// A workgroup of four wavefronts owns one tile of consecutive tokens of one sequence and the query
// heads of one kv head (up to 16 at a time).  A "row" is one (token, head) pair; a wavefront owns
// one block of 16 rows.  All rows of a workgroup read the same keys and values, KSTEP at a time,
// staged in LDS once for the workgroup as they lie in the cache (no transposition):
//
//   S^T[key, row]   = K[key, :] . Q[row, :]      K rows as the A operand, Q (scaled) as B.  The k
//                     index of an MFMA is only a label: lane group kg of MFMA j takes dim
//                     kg*HD/4 + j, so a lane reads HD/4 consecutive floats of its key and of its row.
//   softmax           float32, online; a lane holds 4 scores (keys 4*kg + i) of ONE row for each
//                     16-key half, so a row's maximum crosses lanes only when it has to move
//   O^T[dim, row]  += V^T[dim, key] . P^T[key, row]   the weight of key 4*kg + i is register i of
//                     the lane, which is where the B operand of the MFMA for keys {4*kg + i} wants
//                     it; the A operand's row m stands for dim m*HD/16 + db (MFMA db), so a lane
//                     reads HD/16 consecutive floats of V and ends up with HD/4 consecutive dims of
//                     its row's output.
//
// Formula (reference: src/op/kernels/cuda/prefill_attention_kernel.cu:66-141, 422-455, which
// forms the whole score matrix with two library products per chunk): the query at position P
// reads keys max(0, P+1-window)..P, scores are scaled by `scale`, softmax subtracts a reference
// and divides by the plain sum.
#include "common.h"

#ifndef HEAD_DIM
#error "HEAD_DIM must be defined"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size: multiple of 16, at most 256");

typedef float floatx4_t __attribute__((ext_vector_type(4)));

#define MA_WAVES 4
#define NEG_BIG (-1.0e30f)
#define ROW_PAD 4      // floats of padding per staged row: the sixteen rows of a 16-byte read fall on different banks
// How far a row's scores may rise above the reference its weights are taken against before the
// reference is moved and the output rescaled (e^5.545 = 2^8).  Softmax is the same whatever the
// reference, as long as numerator and denominator share it.
#define REF_SLACK 5.545177444479562f

struct QTile { int32_t seq, row0, ntok, pos0; };   // tokens row0..row0+ntok-1 of the batch, positions pos0..

__device__ __forceinline__ float lanes4(float x, bool take_max) {
    // over the four lanes that hold one row (lanes r, r+16, r+32, r+48): maximum or sum
    const auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    const float u = __uint_as_float(a[0]), v = __uint_as_float(a[1]);
    x = take_max ? fmaxf(u, v) : u + v;
    const auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    const float s = __uint_as_float(b[0]), t = __uint_as_float(b[1]);
    return take_max ? fmaxf(s, t) : s + t;
}

template <bool POW2>
__global__ __launch_bounds__(MA_WAVES * WAVE) void mfma_attention_f32_kernel(
    const float* __restrict__ q, int q_stride, const float* __restrict__ kpool, const float* __restrict__ vpool,
    const int32_t* __restrict__ block_table, int table_stride, const QTile* __restrict__ tiles, int n_tiles,
    float* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml, int H, int KVH, int page_size,
    int page_shift, int hpt_shift, int window, float scale, int nsplit) {
    constexpr int HD = HEAD_DIM;
    constexpr int THREADS = MA_WAVES * WAVE;
    constexpr int KSTEP = HD <= 128 ? 32 : 16;     // keys of a step
    constexpr int HALVES = KSTEP / 16;
    constexpr int QK = HD / 4;                     // MFMAs of the first product per 16 keys; floats of Q a lane holds
    constexpr int DB = HD / 16;                    // MFMAs of the second product per 4 keys
    constexpr int ROW = HD + ROW_PAD;
    __shared__ __attribute__((aligned(16))) float ksm[2][KSTEP][ROW];
    __shared__ __attribute__((aligned(16))) float vsm[2][KSTEP][ROW];
    constexpr int TBL_MAX = 1024;
    __shared__ int32_t tbl[TBL_MAX];

    // As many workgroups as the chip holds at once; the tiles come sorted by the keys they walk,
    // longest first, and workgroup w takes tiles w, 2P-1-w, 2P+w, ... (P workgroups in x).
    for (int round = 0;; ++round) {
        int tile_at = (round & 1) ? (round + 1) * gridDim.x - 1 - blockIdx.x : round * gridDim.x + blockIdx.x;
        // one round only: the chip holds the whole grid, and a compute unit gets workgroups of the same x from the lower
        // and the upper half of y; the upper half walks the sorted list backwards, so that long tiles meet short ones there
        if (n_tiles <= static_cast<int>(gridDim.x) && 2 * blockIdx.y >= gridDim.y && gridDim.y > 1) tile_at = n_tiles - 1 - tile_at;
        if (tile_at >= n_tiles || tile_at < 0) break;
        const QTile tile = tiles[tile_at];
        const int G = H / KVH;
        const int hpt = 1 << hpt_shift;
        const int chunks = (G + hpt - 1) >> hpt_shift;
        const int g = blockIdx.y / chunks;
        const int chunk = blockIdx.y % chunks;

        const int tid = threadIdx.x;
        const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
        const int r = lane % 16, kg = lane / 16;

        // the wavefront's block of 16 rows: tokens wave*16/hpt .. of the tile, heads fastest
        const int tok_per_block = 16 >> hpt_shift;
        const int tb0 = wave * tok_per_block;
        const int tt = tb0 + (r >> hpt_shift);
        const int hh = (chunk << hpt_shift) + (r & (hpt - 1));
        const int head = g * G + hh;
        const bool row_ok = tt < tile.ntok && hh < G;
        const int pos = tile.pos0 + tt;
        const int row_lo = (row_ok && window > 0) ? max(0, pos + 1 - window) : 0;
        const bool blk_ok = tb0 < tile.ntok;                                     // uniform in the wavefront
        const int blk_pmin = tile.pos0 + tb0;
        const int blk_pmax = tile.pos0 + min(tile.ntok, tb0 + tok_per_block) - 1;
        const int blk_lo_max = window > 0 ? max(0, blk_pmax + 1 - window) : 0;

        // key range of the workgroup, walked in steps of KSTEP from a multiple of KSTEP; only keys
        // tile_lo..kend-1 are read from the cache (all of them the sequence's own, none given back)
        const int kend = tile.pos0 + tile.ntok;
        const int tile_lo = window > 0 ? max(0, tile.pos0 + 1 - window) : 0;
        const int kbeg = tile_lo / KSTEP * KSTEP;
        const int nsteps_all = (kend - kbeg + KSTEP - 1) / KSTEP;
        const int per_split = (nsteps_all + nsplit - 1) / nsplit;
        const int s_begin = blockIdx.z * per_split;
        const int nsteps = max(0, min(nsteps_all, s_begin + per_split) - s_begin);
        const int kfirst = kbeg + s_begin * KSTEP;

        const int32_t* table = block_table + static_cast<size_t>(tile.seq) * table_stride;
        auto page_of = [&](int key) { return POW2 ? (key >> page_shift) : key / page_size; };
        auto slot_of = [&](int key) { return POW2 ? (key & (page_size - 1)) : key % page_size; };
        int key_lo = 0, key_hi = 0, lp0 = 0;              // keys of the current table segment, and its first page
        auto row_address = [&](int key) -> size_t {       // offset of key's row for kv head g; key clamped to keys that may be read
            const int kc = min(max(key, key_lo), key_hi);
            const int page = tbl[page_of(kc) - lp0];
            return ((static_cast<size_t>(max(page, 0)) * KVH + g) * page_size + slot_of(kc)) * HD;
        };

        // Q, scaled, as the B operand: lane (row r, group kg) holds dims kg*HD/4 .. +HD/4
        float qf[QK];
        if (row_ok) {
            VecIO<float, QK>::load(q + static_cast<size_t>(tile.row0 + tt) * q_stride + static_cast<size_t>(head) * HD + kg * QK, qf);
#pragma unroll
            for (int j = 0; j < QK; ++j) qf[j] *= scale;
        } else {
#pragma unroll
            for (int j = 0; j < QK; ++j) qf[j] = 0.f;
        }

        float m_ref = NEG_BIG, l_lane = 0.f;       // the row's reference; the sum of this lane's own weights
        floatx4_t o[DB];
#pragma unroll
        for (int db = 0; db < DB; ++db) o[db] = floatx4_t{0.f, 0.f, 0.f, 0.f};

        // Staging: a thread loads 16 bytes of one key's K row and of its V row; the lanes of a
        // quarter wavefront or more read one row between them.
        constexpr int PIECES = HD / 4;
        constexpr int ITEMS = KSTEP * PIECES;
        constexpr int PER_THREAD = (ITEMS + THREADS - 1) / THREADS;
        auto load_kv = [&](int ks, float4 (&kdst)[PER_THREAD], float4 (&vdst)[PER_THREAD]) {
#pragma unroll
            for (int i = 0; i < PER_THREAD; ++i) {
                const int item = (tid + i * THREADS) % ITEMS;      // spare threads load an item again and do not store it
                const size_t at = row_address(ks + item / PIECES) + (item % PIECES) * 4;
                kdst[i] = *reinterpret_cast<const float4*>(kpool + at);
                vdst[i] = *reinterpret_cast<const float4*>(vpool + at);
            }
        };
        auto store_kv = [&](int buf, const float4 (&ksrc)[PER_THREAD], const float4 (&vsrc)[PER_THREAD]) {
#pragma unroll
            for (int i = 0; i < PER_THREAD; ++i) {
                const int item = tid + i * THREADS;
                if (item < ITEMS) {
                    *reinterpret_cast<float4*>(&ksm[buf][item / PIECES][(item % PIECES) * 4]) = ksrc[i];
                    *reinterpret_cast<float4*>(&vsm[buf][item / PIECES][(item % PIECES) * 4]) = vsrc[i];
                }
            }
        };

        // Loads run two steps ahead of the arithmetic, in two fixed sets of registers.
        float4 kr[2][PER_THREAD], vr[2][PER_THREAD];
        for (int seg0 = 0; seg0 < nsteps;) {
            const int seg_first = kfirst + seg0 * KSTEP;
            lp0 = page_of(max(seg_first, tile_lo));
            const int seg_steps = min(nsteps - seg0, ((lp0 + TBL_MAX) * page_size - seg_first) / KSTEP);
            key_lo = max(seg_first, tile_lo);
            key_hi = min(seg_first + seg_steps * KSTEP, kend) - 1;
            __syncthreads();                   // nobody still reads the previous segment's table or staged tiles
            for (int i = tid; i <= page_of(key_hi) - lp0; i += THREADS) tbl[i] = table[lp0 + i];
            __syncthreads();
            load_kv(seg_first, kr[0], vr[0]);
            load_kv(seg_first + KSTEP, kr[1], vr[1]);
            store_kv(0, kr[0], vr[0]);
            load_kv(seg_first + 2 * KSTEP, kr[0], vr[0]);

            auto step = [&](int s, float4 (&knext)[PER_THREAD], float4 (&vnext)[PER_THREAD]) {
                if (s >= seg_steps) return;
                const int ks = seg_first + s * KSTEP;
                // the tiles of this step are in buffer s & 1; nobody still reads the other one
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
                const bool act = blk_ok && ks <= blk_pmax;                           // else all rows lie before these keys
                const bool inner = act && ks >= blk_lo_max && ks + KSTEP - 1 <= blk_pmin;   // every key counts for every row
                if (act) {
                    const float (*kb)[ROW] = ksm[s & 1];
                    const float (*vb)[ROW] = vsm[s & 1];
                    // 1. scores: this lane gets row r, keys ks + 16*t + 4*kg + i
                    floatx4_t st[HALVES];
#pragma unroll
                    for (int t = 0; t < HALVES; ++t) {
                        st[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int j4 = 0; j4 < QK / 4; ++j4) {
                            const float4 ka = *reinterpret_cast<const float4*>(&kb[t * 16 + r][kg * QK + j4 * 4]);
                            st[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka.x, qf[j4 * 4 + 0], st[t], 0, 0, 0);
                            st[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka.y, qf[j4 * 4 + 1], st[t], 0, 0, 0);
                            st[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka.z, qf[j4 * 4 + 2], st[t], 0, 0, 0);
                            st[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka.w, qf[j4 * 4 + 3], st[t], 0, 0, 0);
                        }
                    }
                    float sc[HALVES][4];
                    float lane_max = NEG_BIG;
#pragma unroll
                    for (int t = 0; t < HALVES; ++t)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            float v = st[t][i];
                            if (!inner) {
                                const int key = ks + t * 16 + kg * 4 + i;
                                v = (row_ok && key <= pos && key >= row_lo) ? v : NEG_BIG;
                            }
                            sc[t][i] = v;
                            lane_max = fmaxf(lane_max, v);
                        }
                    // 2. a row whose scores have risen far above its reference: move it, rescale what was summed
                    if (__any(lane_max - REF_SLACK > m_ref)) {
                        const float mx = lanes4(lane_max, true);
                        const bool move = mx > 0.5f * NEG_BIG && mx > m_ref + REF_SLACK;
                        const float m_new = move ? mx : m_ref;
                        const float corr = move ? expf(m_ref - m_new) : 1.0f;
                        m_ref = m_new;
                        l_lane *= corr;
#pragma unroll
                        for (int db = 0; db < DB; ++db) o[db] *= corr;
                    }
                    // 3. weights, and O^T += V^T . P^T for the keys {16*t + 4*kg + i} of MFMA (t, i)
#pragma unroll
                    for (int t = 0; t < HALVES; ++t)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            float p = expf(sc[t][i] - m_ref);
                            if (!inner) p = sc[t][i] > 0.5f * NEG_BIG ? p : 0.f;
                            l_lane += p;
                            float va[DB];
                            VecIO<float, DB>::load(&vb[t * 16 + kg * 4 + i][r * DB], va);
#pragma unroll
                            for (int db = 0; db < DB; ++db)
                                o[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(va[db], p, o[db], 0, 0, 0);
                        }
                }
                store_kv((s + 1) & 1, knext, vnext);
                load_kv(ks + 3 * KSTEP, knext, vnext);
            };
            for (int s0 = 0; s0 < seg_steps; s0 += 2) {
                step(s0, kr[1], vr[1]);
                step(s0 + 1, kr[0], vr[0]);
            }
            seg0 += seg_steps;
        }

        const float l = lanes4(l_lane, false);
        if (row_ok) {
            // this lane holds dims kg*HD/4 + i*DB + db of its row in o[db][i]
            float vals[QK];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int db = 0; db < DB; ++db) vals[i * DB + db] = o[db][i];
            if (nsplit > 1) {
                const size_t p = (static_cast<size_t>(tile.row0 + tt) * H + head) * nsplit + blockIdx.z;
                if (kg == 0) { part_ml[p * 2] = m_ref; part_ml[p * 2 + 1] = l; }
                VecIO<float, QK>::store(part_o + p * HD + kg * QK, vals);
            } else if (l > 0.f) {
                const float inv = 1.0f / l;
#pragma unroll
                for (int j = 0; j < QK; ++j) vals[j] *= inv;
                VecIO<float, QK>::store(out + static_cast<size_t>(tile.row0 + tt) * H * HD + static_cast<size_t>(head) * HD + kg * QK, vals);
            }
        }
        __syncthreads();       // the next tile's first stores find nobody reading this one's
    }
}

static int heads_per_tile(int group) { return group >= 16 ? 16 : group > 4 ? 8 : group > 2 ? 4 : group > 1 ? 2 : 1; }

NI_EXPORT int ni_mfma_attention_f32_head_dim() { return HEAD_DIM; }

// Tokens of a tile for `group` query heads per kv head: four blocks of 16 rows.
NI_EXPORT int ni_mfma_attention_f32_tile_tokens(int group) {
    if (group < 1) return 0;
    return MA_WAVES * (16 / heads_per_tile(group));
}

// tiles: int32 [n_tiles, 4] rows of (sequence, first row, tokens, first position), at most
// ni_mfma_attention_f32_tile_tokens tokens each, sorted by the keys they walk (longest first).
// part_o: float [T, H, nsplit, HEAD_DIM], part_ml: float [T, H, nsplit, 2]; unused when nsplit == 1.
NI_EXPORT int ni_mfma_attention_f32(const void* q, int q_stride, const void* kpool, const void* vpool,
                                    const void* block_table, int table_stride, const void* tiles, int n_tiles, void* out,
                                    void* part_o, void* part_ml, int H, int KVH, int page_size, int window, float scale,
                                    int nsplit, hipStream_t stream) {
    if (n_tiles <= 0) return 0;
    if (H < 1 || KVH < 1 || H % KVH != 0 || page_size < 1 || nsplit < 1 || nsplit > 64 || !(scale > 0.f)) return -1;
    if (nsplit > 1 && (!part_o || !part_ml)) return -2;
    if (q_stride % 4 != 0) return -3;
    const int G = H / KVH;
    const int hpt = heads_per_tile(G);
    int hpt_shift = 0;
    while ((1 << hpt_shift) < hpt) ++hpt_shift;
    const int chunks = (G + hpt - 1) / hpt;
    const bool pow2 = (page_size & (page_size - 1)) == 0;
    int page_shift = 0;
    while (pow2 && (1 << page_shift) < page_size) ++page_shift;
    const int per_tile = KVH * chunks * nsplit;
    auto kernel = pow2 ? mfma_attention_f32_kernel<true> : mfma_attention_f32_kernel<false>;
    static int slots[2] = {0, 0}, units[2] = {0, 0};
    if (slots[pow2] == 0) {
        int dev = 0, cus = 0, per_cu = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, MA_WAVES * WAVE, 0) != hipSuccess || cus < 1 ||
            per_cu < 1)
            return -4;
        units[pow2] = cus;
        slots[pow2] = cus * per_cu;
    }
    // with no more tiles than the chip holds workgroups every tile gets one (paired over the compute units, see the
    // kernel); else two rounds pair long tiles with short ones, or more, as few as fit the chip
    int rounds = 1;
    if (n_tiles * per_tile > slots[pow2]) {
        rounds = 2;
        while ((n_tiles + rounds - 1) / rounds * per_tile > slots[pow2] && rounds < n_tiles) rounds += 1;
    }
    const int in_x = (n_tiles + rounds - 1) / rounds;
    dim3 grid(in_x, KVH * chunks, nsplit);
    kernel<<<grid, MA_WAVES * WAVE, 0, stream>>>((const float*)q, q_stride, (const float*)kpool, (const float*)vpool,
                                                 (const int32_t*)block_table, table_stride, (const QTile*)tiles, n_tiles,
                                                 (float*)out, (float*)part_o, (float*)part_ml, H, KVH, page_size, page_shift,
                                                 hpt_shift, window, scale, nsplit);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------------------------------------
// Single tokens (decode steps, short prompt portions) in true float32: one workgroup per (token,
// kv head, sixteen query heads of its group, run of the key range).  The rows of the products are
// the query heads that share the kv head; the wavefronts of the workgroup take the 16-key steps
// of the run in turn, each with a running (reference, sum, output) of its own, and meet in LDS at
// the end.  Both operands that come from the cache are loaded from global memory straight in the
// layout the matrix instructions want, so nothing is staged and no barrier stands in the loop:
//   K as the A operand of S^T = K . Q^T: lane (r, kg) holds dims kg*HD/4 .. +HD/4 of key r, 64
//     bytes in a row at head size 64 (four lanes read one row between them);
//   V^T as the A operand of O^T += V^T . P^T: for the keys {4*kg + i} of MFMA i, lane (r, kg)
//     holds dims r*HD/16 .. +HD/16 of key 4*kg + i (sixteen lanes read one row between them).
// The rows of a step wait in registers, DEC_DEPTH steps ahead of the arithmetic: two, which leaves the registers
// for two workgroups a compute unit up to head size 128 (with three or four steps ahead a decode batch of mixed
// context lengths ran slower: one workgroup a unit cannot pair a long token with a short one).
#define DEC_WAVES 4
#define DEC_KEYS 16
#define DEC_DEPTH 2

template <bool POW2>
__global__ __launch_bounds__(DEC_WAVES * WAVE) void mfma_decode_f32_kernel(
    const float* __restrict__ q, int q_stride, const float* __restrict__ kpool, const float* __restrict__ vpool,
    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ positions, float* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, int H, int KVH, int page_size, int page_shift, int window, float scale, int nsplit) {
    constexpr int HD = HEAD_DIM;
    constexpr int NW = DEC_WAVES;
    constexpr int THREADS = NW * WAVE;
    constexpr int KS = DEC_KEYS;
    constexpr int QK = HD / 4;                     // MFMAs of the first product per step; floats of Q and of a key a lane holds
    constexpr int DB = HD / 16;                    // MFMAs of the second product per 4 keys
    constexpr int DEPTH = DEC_DEPTH;
    __shared__ __attribute__((aligned(16))) float so[NW][16][HD];      // the wavefronts' outputs, met at the end
    __shared__ float sm_ml[NW][16][2];
    constexpr int TBL_MAX = 1024;
    __shared__ int32_t tbl[TBL_MAX];

    // (uncut key ranges of many tokens: a compute unit holds workgroups u and u + half the grid, the same x in the
    // lower and the upper half of y; the upper half takes the tokens from the far end, so that tokens that come in
    // the order of their contexts put a long and a short one on every unit)
    const int t = (gridDim.z == 1 && gridDim.y > 1 && 2 * blockIdx.y >= gridDim.y) ? gridDim.x - 1 - blockIdx.x : blockIdx.x;
    const int G = H / KVH;
    const int chunks = (G + 15) / 16;
    const int g = blockIdx.y / chunks;
    const int chunk = blockIdx.y % chunks;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
    const int r = lane % 16, kg = lane / 16;
    const int hh = chunk * 16 + r;                 // this lane's row: a query head of the group
    const bool row_ok = hh < G;
    const int head = g * G + hh;

    const int pos = positions[t];
    const int seq = seq_of_token[t];
    const int hi = pos + 1;
    const int lo = window > 0 ? max(0, hi - window) : 0;
    const int kbeg = lo / KS * KS;
    const int nsteps_all = (hi - kbeg + KS - 1) / KS;
    const int per_split = (nsteps_all + nsplit - 1) / nsplit;
    const int s_begin = blockIdx.z * per_split;
    const int nsteps = max(0, min(nsteps_all, s_begin + per_split) - s_begin);
    const int kfirst = kbeg + s_begin * KS;

    const int32_t* table = block_table + static_cast<size_t>(seq) * table_stride;
    auto page_of = [&](int key) { return POW2 ? (key >> page_shift) : key / page_size; };
    auto slot_of = [&](int key) { return POW2 ? (key & (page_size - 1)) : key % page_size; };
    int key_lo = 0, key_hi = 0, lp0 = 0;
    auto row_address = [&](int key) -> size_t {
        // clamped to keys the token may read: those before `lo` may lie in pages already given back
        const int kc = min(max(key, max(key_lo, lo)), key_hi);
        const int page = tbl[page_of(kc) - lp0];
        return ((static_cast<size_t>(max(page, 0)) * KVH + g) * page_size + slot_of(kc)) * HD;
    };

    // Q, scaled, as the B operand: lane (row r, group kg) holds dims kg*HD/4 .. +HD/4
    float qf[QK];
    if (row_ok) {
        VecIO<float, QK>::load(q + static_cast<size_t>(t) * q_stride + static_cast<size_t>(head) * HD + kg * QK, qf);
#pragma unroll
        for (int j = 0; j < QK; ++j) qf[j] *= scale;
    } else {
#pragma unroll
        for (int j = 0; j < QK; ++j) qf[j] = 0.f;
    }

    float m_ref = NEG_BIG, l_lane = 0.f;       // the row's reference; the sum of this lane's own weights
    floatx4_t o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) o[db] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    struct StepRows { float k[QK]; float v[4][DB]; };
    auto load_rows = [&](int ks, StepRows& rows) {
        VecIO<float, QK>::load(kpool + row_address(ks + r) + kg * QK, rows.k);
#pragma unroll
        for (int i = 0; i < 4; ++i) VecIO<float, DB>::load(vpool + row_address(ks + 4 * kg + i) + r * DB, rows.v[i]);
    };

    StepRows ring[DEPTH];
    for (int seg0 = 0; seg0 < nsteps;) {
        key_lo = kfirst + seg0 * KS;
        lp0 = page_of(max(key_lo, lo));
        const int seg_steps = min(nsteps - seg0, ((lp0 + TBL_MAX) * page_size - key_lo) / KS);
        key_hi = min(key_lo + seg_steps * KS, hi) - 1;
        __syncthreads();
        for (int i = tid; i <= page_of(key_hi) - lp0; i += THREADS) tbl[i] = table[lp0 + i];
        __syncthreads();
        // this wavefront's steps of the segment: wave, wave + NW, ...
        const int mine = seg_steps > wave ? (seg_steps - wave + NW - 1) / NW : 0;
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) load_rows(key_lo + (wave + d * NW) * KS, ring[d]);
        // Step j lives in slot j % DEPTH of the ring; the loop is unrolled DEPTH times so that a slot is a
        // fixed set of registers, asked for its next rows as soon as its step has used it.
        auto step = [&](int j, StepRows& rows) {
            const int ks = key_lo + (wave + j * NW) * KS;
            if (j < mine) {
                // 1. scores: this lane gets row r, keys ks + 4*kg + i
                floatx4_t st = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j1 = 0; j1 < QK; ++j1) st = __builtin_amdgcn_mfma_f32_16x16x4f32(rows.k[j1], qf[j1], st, 0, 0, 0);
                const bool inner = ks >= lo && ks + KS - 1 <= pos;
                float sc[4];
                float lane_max = NEG_BIG;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float v = st[i];
                    if (!inner) {
                        const int key = ks + 4 * kg + i;
                        v = (key <= pos && key >= lo) ? v : NEG_BIG;
                    }
                    sc[i] = v;
                    lane_max = fmaxf(lane_max, v);
                }
                // 2. a row whose scores have risen far above its reference: move it, rescale what was summed
                if (__any(lane_max - REF_SLACK > m_ref)) {
                    const float mx = lanes4(lane_max, true);
                    const bool move = mx > 0.5f * NEG_BIG && mx > m_ref + REF_SLACK;
                    const float m_new = move ? mx : m_ref;
                    const float corr = move ? expf(m_ref - m_new) : 1.0f;
                    m_ref = m_new;
                    l_lane *= corr;
#pragma unroll
                    for (int db = 0; db < DB; ++db) o[db] *= corr;
                }
                // 3. weights, and O^T += V^T . P^T for the keys {4*kg + i} of MFMA i
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float p = expf(sc[i] - m_ref);
                    if (!inner) p = sc[i] > 0.5f * NEG_BIG ? p : 0.f;
                    l_lane += p;
#pragma unroll
                    for (int db = 0; db < DB; ++db) o[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(rows.v[i][db], p, o[db], 0, 0, 0);
                }
            }
            load_rows(ks + DEPTH * NW * KS, rows);
        };
        for (int j0 = 0; j0 < mine; j0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) step(j0 + d, ring[d]);
        }
        seg0 += seg_steps;
    }

    // wavefronts meet: every one leaves (reference, sum) of its rows and its 16 x HD output in LDS; this lane
    // holds dims (4*kg + i)*DB + db of its row in o[db][i]
    const float l = lanes4(l_lane, false);
    if (kg == 0) { sm_ml[wave][r][0] = m_ref; sm_ml[wave][r][1] = l; }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int db = 0; db < DB; ++db) so[wave][r][(4 * kg + i) * DB + db] = o[db][i];
    __syncthreads();
    const int rows_here = min(16, G - chunk * 16);
    for (int idx = tid; idx < rows_here * HD; idx += THREADS) {
        const int row = idx / HD, dim = idx % HD;
        float M = sm_ml[0][row][0];
#pragma unroll
        for (int w = 1; w < NW; ++w) M = fmaxf(M, sm_ml[w][row][0]);
        float Lsum = 0.f, O = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float f = expf(sm_ml[w][row][0] - M);
            Lsum += sm_ml[w][row][1] * f;
            O += so[w][row][dim] * f;
        }
        const int h = g * G + chunk * 16 + row;
        if (nsplit == 1) {
            out[static_cast<size_t>(t) * H * HD + static_cast<size_t>(h) * HD + dim] = O / Lsum;
        } else {
            const size_t p = (static_cast<size_t>(t) * H + h) * nsplit + blockIdx.z;
            part_o[p * HD + dim] = O;
            if (dim == 0) { part_ml[p * 2] = M; part_ml[p * 2 + 1] = Lsum; }
        }
    }
}

// Attention of single tokens on the matrix cores in float32: same arguments and partial-result layout as the
// token-at-a-time kernel (`out` is left to its merge kernel when nsplit > 1).
NI_EXPORT int ni_mfma_token_attention_f32(const void* q, int q_stride, const void* kpool, const void* vpool,
                                          const void* block_table, int table_stride, const void* seq_of_token,
                                          const void* positions, void* out, void* part_o, void* part_ml, int T_tokens,
                                          int H, int KVH, int page_size, int window, float scale, int nsplit,
                                          hipStream_t stream) {
    if (T_tokens <= 0) return 0;
    if (H < 1 || KVH < 1 || H % KVH != 0 || page_size < 1 || nsplit < 1 || nsplit > 65535 || !(scale > 0.f)) return -1;
    if (nsplit > 1 && (!part_o || !part_ml)) return -2;
    if (q_stride % 4 != 0) return -3;
    const int G = H / KVH;
    const int chunks = (G + 15) / 16;
    const bool pow2 = (page_size & (page_size - 1)) == 0;
    int page_shift = 0;
    while (pow2 && (1 << page_shift) < page_size) ++page_shift;
    dim3 grid(T_tokens, KVH * chunks, nsplit);
    auto kernel = pow2 ? mfma_decode_f32_kernel<true> : mfma_decode_f32_kernel<false>;
    kernel<<<grid, DEC_WAVES * WAVE, 0, stream>>>(
        (const float*)q, q_stride, (const float*)kpool, (const float*)vpool, (const int32_t*)block_table, table_stride,
        (const int32_t*)seq_of_token, (const int32_t*)positions, (float*)out, (float*)part_o, (float*)part_ml, H, KVH,
        page_size, page_shift, window, scale, nsplit);
    return NI_LAUNCH_RESULT();
}
