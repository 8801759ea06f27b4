// Chunked-prefill causal attention over the paged pool on gfx950 matrix cores:
// the one dense contraction of the path (MFMA-bound, not HBM-bound).
//
// Replaces  F.scaled_dot_product_attention(query, full_key, full_value,
//           attn_mask=None, is_causal=True)       opt_prime/opt_prime/kv_cache.py:404-415
// for a chunk of new tokens whose K/V rows are already in the pool.  The mask
// is bottom-right aligned: query i of a chunk with prior context P sees keys
// j <= P + i.  At P == 0 that is the reference's is_causal=True (Lq == Lk), at
// chunk length 1 it is the reference's decode (kv_cache.py:397-403).
//
// Flops per chunk: 4 * Hq * D * (C*P + C(C+1)/2)   (QK^T and PV, causal).
//
// Work split   one workgroup (4 waves) per (64 or 128 query rows, sequence).  A "row" is
//              a (position, query head) pair: with `gpack` = G heads of one KV
//              head packed per position, the rows are consecutive positions x G
//              heads, so every K/V tile staged in LDS serves the whole GQA group.
//              Groups that do not divide 16 use gpack = 1.  Workgroups of one KV head
//              are adjacent in the grid (one XCD's L2 serves them).  With 2 to 16 chunks the
//              workgroups take their (chunk, query tile) items in order of cost, a long item
//              and a short one side by side on a CU; otherwise the longest query tiles of
//              every chunk are launched first.
// K/V tiles    32 or 64 tokens per step, double-buffered in LDS, one barrier per tile.  16-bit
//              pools (bf16, fp16) and two column groups: loaded straight into LDS
//              (global_load_lds_dwordx4, 1 KB = four or eight token rows per wave
//              instruction) one tile ahead, rows unpadded with their 16-byte chunks
//              XOR-swizzled by the row index.
//              Otherwise: coalesced 16-byte loads into registers ahead of their use, written
//              to LDS (one padded row per token; fp8 is widened to the query's type on the way).
// head_dim     128 or 64, one instantiation each.
// Per wave     16 or 32 rows (one or two column groups).  S^T = K Q^T with K rows as
//              the A operand and the wave's query rows as B columns
//              (v_mfma_f32_16x16x32_bf16 / _f16), the score multiplier folded into Q and the
//              running max into the accumulators' starting value; online softmax per column
//              with a lazily moved max: the exponentials are taken against the current
//              max and their sum tells whether it has to move (then, rarely, the row max is
//              found with two lane swaps and the exponentials are redone); O^T += V^T P^T
//              with the V^T operand read out of the row-major V tile by gfx950's transposing
//              LDS read (ds_read_b64_tr_b16), in the token order the QK product was laid out
//              in, so P never leaves its lane.  With two column groups every LDS operand
//              read feeds two MFMAs.
#include "common.h"

#include <atomic>
#include <type_traits>

namespace aicomp {

namespace {

constexpr int BS = 16;
constexpr int ROWS = 64;               // query rows per workgroup and column group (16 per wave)
constexpr float NEG_BIG = -1.0e30f;

struct PrefillParams {
    void* out;
    const void* query;
    const void* k_pool;
    const void* v_pool;
    const int32_t* block_table;
    int64_t block_table_stride;
    const int32_t* context_lens;
    const int32_t* cu_q_lens;
    int hq, hkv, group, gpack, max_blocks;
    int num_blocks;
    int num_cus;                       // CUs of the device (0: keep the grid order)
    float qk_mul;
    const float* k_scale;
    const float* v_scale;
    const int32_t* items;              // (sequence, query tile) pairs; grid.y numbers them (NULL: none)
    int num_seqs;
};

// max over lanes l and l^16 (l^32): gfx950's lane-swap instructions, no LDS round trip.
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of
// its second; with both operands holding x, every lane ends up with its own value in one
// result and its partner's in the other.
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float xor16_max(float x) {
    const u32x2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xor32_max(float x) {
    const u32x2_t r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// register stage of one K and one V tile: NL loads of the workgroup each
template <bool FP8, int NL> struct Stage;
template <int NL> struct Stage<false, NL> { uint4 k[NL], v[NL]; };
template <int NL> struct Stage<true, NL> { uint2 k[NL], v[NL]; };

// R = 16-row column groups per wave (1 or 2).  With R = 2 every K and V operand read from LDS
// (and every V permute) feeds two MFMAs, and the two groups' softmax chains are independent, so
// LDS traffic and permute work per flop halve and the scheduler has two chains to interleave.
// DH = head_dim (128 or 64).  An LDS row is one token: 2*DH bytes plus, in the register-staged
// variants, 16 bytes of padding, so that the sixteen rows of an operand read start in different
// banks (272 B: 4 banks apart; 144 B: 36).
// KT = rows of an LDS tile (KT/16 blocks): 32 with two register stages for R = 1, 64 with one stage
// for R = 2, where the per-step work that does not scale with the tile (barrier, block lookups,
// loop control, the running-max test) is paid half as often.
// DMA = tiles go from the pool straight into LDS (bf16 / fp16 pools, R = 2): no staging registers, no
// LDS writes by the waves.  The two buffers are separate __shared__ arrays and every read address
// is one offset from its array, which is what lets the compiler see that a read of one buffer
// need not wait for the loads in flight into the other; the only wait is the explicit one at the
// barrier that opens a step, for the loads issued one step earlier.
#define GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
// E = the 16-bit element format of queries, output and (unless FP8) the pools.
template <typename E, bool FP8, int R, int DH, bool DMA>
__global__ void __launch_bounds__(256, (R == 1 || DH == 64) ? 3 : 2)
paged_prefill_mfma_kernel(PrefillParams p) {
    static_assert(!DMA || (!FP8 && R == 2), "direct-to-LDS tiles: 16-bit pools, two column groups");
    constexpr int KROW = DMA ? 2 * DH : 2 * DH + 16;          // LDS row stride in bytes
    constexpr int NSL = DH / 32;               // 32-element k-slots of a row (QK^T MFMAs per 16 x 16 tile)
    constexpr int NJ = DH / 16;                // 16-element output tiles (PV MFMAs per 32 tokens)
    constexpr int CPR = DH / 8;                // 8-element chunks per row
    constexpr int RPL = 256 / CPR;             // rows one load of the workgroup covers (16 or 32)
    constexpr int KT = R == 1 ? 32 : 64;
    constexpr int NH = KT / 16;                // 16-row groups of a tile
    constexpr int TILE_BYTES = KT * KROW;
    constexpr int NL = KT / RPL;               // loads per tile and pool
    typedef Stage<FP8, NL> StageT;
    // Grid: x = head group (fastest: the workgroups of one KV head land on one XCD and share its
    // L2 copy of that head's K/V); (y, z) number the (sequence, query tile) items.
    constexpr int TT = KT;                     // tokens per LDS tile
    constexpr int CR = 16;                     // query rows per 16-column group
    constexpr int WROWS = CR * R;              // rows per wave
    const int hgroup = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g4 = lane >> 4;
    const int pos_per_wg = 4 * WROWS / p.gpack;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // [2][K tile | V tile]
    // Direct-to-LDS tiles: four separate arrays, so that the compiler can tell a read of one
    // buffer from the loads in flight into the other.
    __shared__ __attribute__((aligned(16))) unsigned char dma_k0[DMA ? TILE_BYTES : 16];
    __shared__ __attribute__((aligned(16))) unsigned char dma_v0[DMA ? TILE_BYTES : 16];
    __shared__ __attribute__((aligned(16))) unsigned char dma_k1[DMA ? TILE_BYTES : 16];
    __shared__ __attribute__((aligned(16))) unsigned char dma_v1[DMA ? TILE_BYTES : 16];

    // Which item this workgroup takes.  Workgroups are dispatched in grid order, the first
    // num_cus of them one per CU, the next num_cus beside them, the rest as places free up; an
    // item costs as many tile steps as its last row has keys, and chunks with different prior
    // contexts differ several-fold.  For 2 to 16 chunks and up to 256 items every workgroup ranks
    // the items by cost (same inputs, same answer everywhere) and takes the item whose rank is its
    // own place in the dispatch order, odd rounds of num_cus reversed: the two workgroups that share
    // a CU from the start are then a long item and a short one, and later places are handed out
    // longest first.  An item's rank comes in closed form from the other chunks' lengths (its
    // cost c, then per chunk the number of tiles costing >= c and >= c + 1), so the work is per
    // chunk, not per item.  Other grids (a single prompt, many chunks) take their query tile slices in
    // the order of prefill_tile_of_slice: expensive first, or, when the whole grid is resident at
    // once, expensive and cheap tiles paired on a CU.
    int seq = blockIdx.y, qtile = prefill_tile_of_slice(blockIdx.z, gridDim.z, p.num_cus, gridDim.x * gridDim.y);
    const int nseq = gridDim.y, ntile = gridDim.z, items = nseq * ntile;
    bool ranked = false;
    int r_ctx = 0, r_n = 0, r_qb = 0;
    if (p.items != nullptr) {
        // The caller ranked the items itself (it knows the lengths on the host): workgroup row y
        // takes pair y.  A pair that names no sequence is skipped; a tile beyond its chunk exits below.
        seq = p.items[2 * blockIdx.y];
        qtile = p.items[2 * blockIdx.y + 1];
        if (seq < 0 || seq >= p.num_seqs || qtile < 0) return;
    } else if (p.num_cus > 0 && nseq > 1 && nseq <= 16 && items <= 256) {     // workgroup-uniform
        int* scratch = (int*)(DMA ? dma_k0 : lds);                     // the tile buffers are still unused
        if (tid < nseq) {
            const int qb_t = p.cu_q_lens[tid];
            const int n_t = p.cu_q_lens[tid + 1] - qb_t;
            const int ctx_t = min(p.context_lens[tid], p.max_blocks * BS);
            scratch[4 * tid] = ctx_t;
            scratch[4 * tid + 1] = ctx_t - n_t;
            scratch[4 * tid + 3] = qb_t;
            scratch[4 * tid + 2] = (n_t > 0 && ctx_t >= n_t) ? min(ntile, (n_t + pos_per_wg - 1) / pos_per_wg) : 0;   // tiles with work
        }
        __syncthreads();
        // this workgroup's place among the items, and the rank it takes
        const int place = blockIdx.y + nseq * blockIdx.z;
        int want = place;
        const int per_round = p.num_cus / (int)gridDim.x;
        if (per_round > 0 && p.num_cus % (int)gridDim.x == 0) {
            const int round = place / per_round, pos = place % per_round;
            const int cnt = min(per_round, items - round * per_round);
            if (round & 1) want = round * per_round + (cnt - 1 - pos);
        }
        const int shift = __builtin_ctz(pos_per_wg);                    // a power of two
        // tiles of a chunk (context, prior, tiles) that cost at least c steps (c >= 1)
        auto count_ge = [&](int ctx_s, int prior_s, int tiles_s, int c) {
            const int x = (c - 1) * KT;
            if (tiles_s == 0 || ctx_s <= x) return 0;
            return max(0, tiles_s - (x < prior_s ? 0 : (x - prior_s) >> shift));
        };
        if (tid < items) {
            const int s_t = tid / ntile, q_t = tid - s_t * ntile;
            const int ctx_t = scratch[4 * s_t], prior_t = scratch[4 * s_t + 1], tiles_t = scratch[4 * s_t + 2];
            const bool work = q_t < tiles_t;
            const int c = work ? (min(ctx_t, prior_t + (q_t + 1) * pos_per_wg) + KT - 1) / KT : 0;
            int dearer = 0, equal_before = 0, all_work = 0, idle_before = 0;
            for (int s2 = 0; s2 < nseq; ++s2) {
                const int ctx2 = scratch[4 * s2], prior2 = scratch[4 * s2 + 1], tiles2 = scratch[4 * s2 + 2];
                const int ge1 = count_ge(ctx2, prior2, tiles2, c + 1), ge0 = count_ge(ctx2, prior2, tiles2, max(c, 1));
                dearer += ge1;
                if (s2 < s_t) { equal_before += ge0 - ge1; idle_before += ntile - tiles2; }
                if (s2 == s_t) equal_before += q_t - (tiles2 - ge0);    // costs do not fall along a chunk
                all_work += tiles2;
            }
            const int rank = work ? dearer + equal_before : all_work + idle_before + (q_t - tiles_t);
            if (rank == want) { scratch[64] = s_t; scratch[65] = q_t; }
        }
        __syncthreads();
        seq = __builtin_amdgcn_readfirstlane(scratch[64]);
        qtile = __builtin_amdgcn_readfirstlane(scratch[65]);
        // the chosen chunk's numbers are in the scratch already: no second trip to memory for them
        r_ctx = __builtin_amdgcn_readfirstlane(scratch[4 * seq]);
        r_n = r_ctx - __builtin_amdgcn_readfirstlane(scratch[4 * seq + 1]);
        r_qb = __builtin_amdgcn_readfirstlane(scratch[4 * seq + 3]);
        ranked = true;
        __syncthreads();                       // before the first tile is written over the scratch
    }

    const int q_begin = ranked ? r_qb : p.cu_q_lens[seq];
    const int n = ranked ? r_n : p.cu_q_lens[seq + 1] - q_begin;
    const int ctx = ranked ? r_ctx : min(p.context_lens[seq], p.max_blocks * BS);
    const int prior = ctx - n;
    const int q0 = qtile * pos_per_wg;
    if (q0 >= n || n <= 0) return;
    if (prior < 0) {
        // a context shorter than the chunk itself: there is no consistent set of keys, the rows
        // are defined as zero (the vector-ALU kernel gives the same) rather than left unwritten
        for (int i = tid; i < 4 * WROWS * (DH / 8); i += 256) {
            const int row = i / (DH / 8), chunk = i % (DH / 8);
            const int pos = q0 + row / p.gpack, hd = hgroup * p.gpack + row % p.gpack;
            if (pos < n)
                *(uint4*)((uint16_t*)p.out + ((int64_t)(q_begin + pos) * p.hq + hd) * DH + 8 * chunk) = make_uint4(0, 0, 0, 0);
        }
        return;
    }

    // rows of this lane's columns: row = WROWS*w + CR*c + (column, or column / 2) -> (position, head)
    const int kvh = (hgroup * p.gpack) / p.group;          // workgroup-uniform
    int qpos[R], head[R], qabs[R];
    bool row_valid[R];
#pragma unroll
    for (int c = 0; c < R; ++c) {
        const int row = WROWS * w + CR * c + r16;
        qpos[c] = q0 + row / p.gpack;
        head[c] = hgroup * p.gpack + row % p.gpack;
        row_valid[c] = qpos[c] < n;
        qabs[c] = row_valid[c] ? prior + qpos[c] : ctx - 1;    // padded rows: computed, never stored
    }
    // last key any row of this wave / workgroup may see (exclusive)
    // (a wave whose rows all lie beyond the chunk's end has nothing to compute: it only takes part in
    // the tile loads and barriers)
    const int wave_kv_end = q0 + (WROWS * w) / p.gpack >= n ? 0 : min(ctx, prior + q0 + (WROWS * w + WROWS - 1) / p.gpack + 1);
    const int wave_kv_min = prior + q0 + (WROWS * w) / p.gpack;    // smallest qabs in the wave (if valid)
    const int kv_end = min(ctx, prior + q0 + pos_per_wg);
    const int ntiles = (kv_end + TT - 1) / TT;

    // Q as the B operand: column = this lane's row, k-slots = dims 32s + 8*g4 ..
    uint4 qf[R][NSL];
#pragma unroll
    for (int c = 0; c < R; ++c) {
        const uint16_t* qrow = (const uint16_t*)p.query + ((int64_t)(q_begin + min(qpos[c], n - 1)) * p.hq + head[c]) * DH;
#pragma unroll
        for (int s = 0; s < NSL; ++s)                           // k-slot s, k-group g4: elements 32s + 8*g4 ..
            qf[c][s] = *(const uint4*)(qrow + 32 * s + 8 * g4);
    }
    // The score multiplier log2(e) * scale (* k_scale for an fp8 pool) goes into Q once, here, so
    // that the matrix cores deliver the scores already in the exponent's units and the softmax
    // spends no multiply on them (one rounding of q * multiplier to the 16-bit format: a relative
    // 2^-9 per element for bf16, far below the rounding of the probabilities themselves).
    {
        const float cmul = p.qk_mul * (FP8 ? p.k_scale[kvh] : 1.f);
#pragma unroll
        for (int c = 0; c < R; ++c)
#pragma unroll
            for (int s = 0; s < NSL; ++s) {
                uint32_t* w = (uint32_t*)&qf[c][s];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    w[i] = E::pack(E::to_f32((uint16_t)(w[i] & 0xffffu)) * cmul, E::to_f32((uint16_t)(w[i] >> 16)) * cmul);
            }
    }

    // m = reference max of a row in the exponent's units; its negative is what the score
    // accumulators start from (the C operand of the first QK^T MFMA), so a score comes out of the
    // matrix core as s - m, ready for the exponential.  The first tile starts from 0 and always
    // takes the path that adopts the tile's own row maximum.
    float m[R], lsum[R];
    f32x4_t binit[R];
    f32x4_t O[R][NJ];
#pragma unroll
    for (int c = 0; c < R; ++c) {
        m[c] = 0.f; lsum[c] = 0.f; binit[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < NJ; ++j) O[c][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;
    const_i32_ptr table = (const_i32_ptr)(p.block_table + (int64_t)seq * p.block_table_stride);

    // global -> registers: one load of the workgroup covers RPL rows of CPR chunks (one block at
    // D = 128; two blocks at D = 64, waves 0-1 the first, waves 2-3 the second).  The block ids of
    // a tile are consecutive table entries: one scalar load when all of them exist.
    constexpr int NB = KT / 16;                                // table entries per tile
    auto fetch = [&](int t, StageT& st) {
        int ids[NB];
        const int first = NB * t;
        if (first + NB <= p.max_blocks) {
            typedef int idvec_t __attribute__((ext_vector_type(NB), aligned(4)));
            typedef const __attribute__((address_space(4))) idvec_t* const_idvec_ptr;
            const idvec_t v = *(const_idvec_ptr)(table + first);
#pragma unroll
            for (int i = 0; i < NB; ++i) ids[i] = v[i];
        } else {
#pragma unroll
            for (int i = 0; i < NB; ++i) ids[i] = first + i < p.max_blocks ? table[first + i] : 0;
        }
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            int b;
            if constexpr (RPL == 32) b = (w >> 1) ? ids[2 * i + 1] : ids[2 * i];
            else b = ids[i];
            const int blk = max(0, min(b, p.num_blocks - 1));
            // uniform 64-bit base of this head's slice of the block + a constant 32-bit lane offset
            constexpr int ESZ = FP8 ? 1 : 2;
            const int64_t base = ((int64_t)blk * p.hkv + kvh) * (BS * DH * ESZ);
            const int lane_off = (tid & (16 * CPR - 1)) * (8 * ESZ);
            if constexpr (FP8) {
                st.k[i] = *(const uint2*)((const char*)p.k_pool + base + lane_off);
                st.v[i] = *(const uint2*)((const char*)p.v_pool + base + lane_off);
            } else {
                st.k[i] = *(const uint4*)((const char*)p.k_pool + base + lane_off);
                st.v[i] = *(const uint4*)((const char*)p.v_pool + base + lane_off);
            }
        }
    };
    // registers -> LDS buffer `buf`.  On the tile that reaches the end of the context, V rows at
    // or beyond it are zeroed (a masked probability of 0 times a non-finite leftover would still
    // poison the row).
    auto stash_rows = [&](int t, int buf, const StageT& st, auto tail_tag) {
        constexpr bool TAIL = decltype(tail_tag)::value;
        unsigned char* kb = lds + buf * 2 * TILE_BYTES;
        unsigned char* vb = kb + TILE_BYTES;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const int tok_local = RPL * i + tid / CPR;           // LDS row
            const int off = tok_local * KROW + (tid % CPR) * 16;
            uint4 kk, vv;
            if constexpr (FP8) { kk = E::from_fp8(st.k[i]); vv = E::from_fp8(st.v[i]); }
            else { kk = st.k[i]; vv = st.v[i]; }
            if constexpr (TAIL) {
                if (t * KT + tok_local >= ctx) vv = make_uint4(0, 0, 0, 0);
            }
            *(uint4*)(kb + off) = kk;
            *(uint4*)(vb + off) = vv;
        }
    };
    auto stash = [&](int t, int buf, const StageT& st) {
        if ((t + 1) * TT > ctx) stash_rows(t, buf, st, std::true_type{});     // workgroup-uniform
        else stash_rows(t, buf, st, std::false_type{});
    };

    const int prow = 4 * (r16 & 3) + (r16 >> 2);                       // permuted K row
    const int rd_k = prow * KROW + g4 * 16;                            // chunk g4
    const int vrow = 4 * (r16 >> 2) + g4;
    // transposing V read: lane k of a 16-lane group addresses token row 4*(k/4) + g4, elements 4*(k%4) ..
    const int rd_v = (4 * (r16 >> 2) + g4) * KROW + (r16 & 3) * 8;

    // The next tile of a stage is requested as soon as the stage has been written to LDS (two
    // stages of 32 rows: tile t+2; one stage of 64 rows: tile t+1), so a tile's loads have the
    // time of 64 rows of arithmetic to land.
    constexpr int AHEAD = KT == 32 ? 2 : 1;
    // Direct-to-LDS fetch of tile t: wave w brings in block w of the tile (16 token rows) with
    // 1 KB instructions, four rows of 256 bytes or eight of 128 each; lane l of instruction q lands
    // at row RPI*q + l/CPR, chunk slot l%CPR, and the slot holds chunk (l%CPR) ^ swz(row) (the XOR
    // swizzle that lets the operand reads run at the full LDS rate without padding), so the lane
    // reads that chunk from the pool.  One block per wave: one table entry, one base address and
    // one LDS base per pool; the instruction's immediate offset moves the pool and the LDS address
    // together by 1 KB per q.
    static_assert(!DMA || NB == 4, "one block of the tile per wave");
    constexpr int RPI = 1024 / KROW;           // token rows one 1 KB instruction lands (4 or 8)
    constexpr int NQ = 16 / RPI;               // instructions per block and pool (4 or 2)
    // Chunk slot s of LDS row r holds chunk s ^ swz(r), with one swizzle for the K tile and one for
    // the V tile, each fitted to how the LDS serves its operand read.  Measured on this part (a
    // wave of reads per instruction, 16 waves): the 64 banks deliver 256 bytes per clock only when
    // (a) every four consecutive lanes of a 16-byte read (eight of the 8-byte transposing read)
    // address one aligned 64-byte segment, and (b) each half-wave spreads its segments evenly over
    // the four segments of a bank line; a pattern that is merely free of bank collisions among the
    // sixteen lanes of an MFMA row group (row-index XOR, or padded rows) runs at half that rate.
    // K operand: lanes 4i .. 4i+3 read rows i, 4+i, 8+i, 12+i of a 16-row group at one chunk
    // index: the row's position among those four goes into the slot's low bits, i picks the segment.
    // V operand (transposing read): lanes 0-3 / 4-7 of a group read 32 bytes of rows g, 4+g, the
    // next eight lanes of rows 8+g, 12+g: adjacent 32-byte units for the first pair and the second,
    // the other half of the bank line for odd g.  With 128-byte rows (head_dim 64) even and odd
    // rows are the two halves of a bank line by themselves.
    auto swz_k = [](int row) {
        const int a = (row >> 2) & 3, b = row & 3;
        return DH == 128 ? (a | (b << 2)) : (a | ((b >> 1) << 2));
    };
    auto swz_v = [](int row) {
        const int a = (row >> 2) & 3, b = row & 3;
        return DH == 128 ? ((a | ((b & 1) << 2)) << 1) : (a << 1);
    };
    const uint32_t dma_blk_stride = (uint32_t)p.hkv * (BS * DH * 2);              // bytes per block, < 2^32
    const char* dma_kp = (const char*)p.k_pool + (int64_t)kvh * (BS * DH * 2);   // this KV head's slice of block 0
    const char* dma_vp = (const char*)p.v_pool + (int64_t)kvh * (BS * DH * 2);
    const int dma_lrow = lane / CPR, dma_slot = lane % CPR;     // this lane's row and slot within 1 KB
    uint32_t dma_offk[NQ], dma_offv[NQ];       // pool offset of this lane's chunk, less the immediate
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        dma_offk[q] = dma_lrow * KROW + ((dma_slot ^ swz_k(RPI * q + dma_lrow)) << 4);
        dma_offv[q] = dma_lrow * KROW + ((dma_slot ^ swz_v(RPI * q + dma_lrow)) << 4);
    }
    auto fetch_dma = [&](int t, unsigned char* kb, unsigned char* vb) {
        const int first = NB * t;
        const bool tail = (t + 1) * KT > ctx || first + NB > p.max_blocks;     // workgroup-uniform
        if (!tail) {
            const uint32_t blk = min((uint32_t)table[first + w], (uint32_t)(p.num_blocks - 1));
            const uint64_t base = (uint64_t)blk * dma_blk_stride;
            // The offset is an immediate: explicit instances.  The lane offsets are made opaque once
            // per step, so that each address stays a uniform 64-bit base plus a 32-bit lane offset
            // (the load's scalar-base form) instead of a per-lane 64-bit pointer built with VALU adds.
            uint32_t ok[4] = {dma_offk[0], dma_offk[1], dma_offk[NQ > 2 ? 2 : 0], dma_offk[NQ > 2 ? 3 : 1]};
            uint32_t ov[4] = {dma_offv[0], dma_offv[1], dma_offv[NQ > 2 ? 2 : 0], dma_offv[NQ > 2 ? 3 : 1]};
            asm volatile("" : "+v"(ok[0]), "+v"(ok[1]), "+v"(ok[2]), "+v"(ok[3]));
            asm volatile("" : "+v"(ov[0]), "+v"(ov[1]), "+v"(ov[2]), "+v"(ov[3]));
            const char* kaddr = dma_kp + base;
            const char* vaddr = dma_vp + base;
#define AICOMP_DMA_ROWS(addr, o, buf, q)                                                                            \
            if constexpr (q < NQ)                                                                                   \
                __builtin_amdgcn_global_load_lds(GLOBAL_PTR(addr + o[q]), LDS_PTR(buf + 16 * w * KROW), 16, 1024 * q, 0);
            AICOMP_DMA_ROWS(kaddr, ok, kb, 0) AICOMP_DMA_ROWS(kaddr, ok, kb, 1) AICOMP_DMA_ROWS(kaddr, ok, kb, 2) AICOMP_DMA_ROWS(kaddr, ok, kb, 3)
            AICOMP_DMA_ROWS(vaddr, ov, vb, 0) AICOMP_DMA_ROWS(vaddr, ov, vb, 1) AICOMP_DMA_ROWS(vaddr, ov, vb, 2) AICOMP_DMA_ROWS(vaddr, ov, vb, 3)
#undef AICOMP_DMA_ROWS
        } else {
            // rows at or beyond the context take the last valid row instead (finite data for
            // the masked probabilities of 0 to multiply)
            const int last = ctx - 1, last_blk = last >> 4;
            const int bi = min(first + w, last_blk);
            const uint32_t blk = min((uint32_t)table[bi], (uint32_t)(p.num_blocks - 1));
            const uint64_t base = (uint64_t)blk * dma_blk_stride;
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                const int row = RPI * q + dma_lrow;
                const int tok = min(16 * (first + w) + row, last);
                const uint32_t offk = (tok - 16 * bi) * KROW + ((dma_slot ^ swz_k(row)) << 4);
                const uint32_t offv = (tok - 16 * bi) * KROW + ((dma_slot ^ swz_v(row)) << 4);
                __builtin_amdgcn_global_load_lds(GLOBAL_PTR(dma_kp + base + offk), LDS_PTR(kb + (16 * w + RPI * q) * KROW), 16, 0, 0);
                __builtin_amdgcn_global_load_lds(GLOBAL_PTR(dma_vp + base + offv), LDS_PTR(vb + (16 * w + RPI * q) * KROW), 16, 0, 0);
            }
        }
    };
    auto step = [&](int t, StageT& st, unsigned char* kb_, unsigned char* vb_, unsigned char* kn, unsigned char* vn) {
        const int buf = t & 1;
        const unsigned char* kb;
        const unsigned char* vb;
        if constexpr (DMA) {
            // Tile t has landed once every wave has waited for its own direct-to-LDS loads and
            // then met the others.  The wait is explicit: the compiler only waits for such loads
            // before this wave's own aliasing LDS reads, which says nothing about the other waves'
            // loads, and on the loop's back edge it was seen to emit no wait at all.
            __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0)
            __syncthreads();      // also: tile t-1 is no longer read by anyone
            if (t + 1 < ntiles) fetch_dma(t + 1, kn, vn);
            kb = kb_; vb = vb_;
        } else {
            stash(t, buf, st);
            fetch(min(t + AHEAD, ntiles - 1), st);  // unconditional: a static count of loads in flight
            __syncthreads();          // tile t visible; everyone is done with the buffer tile t+1 will use
            kb = lds + buf * 2 * TILE_BYTES;
            vb = kb + TILE_BYTES;
        }
        const int sub_start = t * TT;
        if (sub_start >= wave_kv_end) return;                          // wave-uniform: above the diagonal

        // ---- S^T = K Q^T: each K operand read feeds the R column groups
        f32x4_t sa[NH][R];
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int c = 0; c < R; ++c) sa[h][c] = binit[c];
#pragma unroll
        for (int s = 0; s < NSL; ++s) {
            uint4 a[NH];
#pragma unroll
            for (int h = 0; h < NH; ++h)
                if constexpr (DMA)   // chunk 4s + g4 of row 16h + prow sits at chunk slot (4s + g4) ^ swz_k(prow)
                    a[h] = *(const uint4*)(kb + 16 * h * KROW + prow * KROW + (((4 * s + g4) ^ swz_k(prow)) << 4));
                else
                    a[h] = *(const uint4*)(kb + 16 * h * KROW + rd_k + s * 64);
#pragma unroll
            for (int h = 0; h < NH; ++h)
#pragma unroll
                for (int c = 0; c < R; ++c)
                    sa[h][c] = E::mfma(a[h], qf[c][s], sa[h][c]);
        }
        // Issue order of the block above: the K operand reads run two k-slots ahead of the MFMAs
        // that consume them, so a wave that has the SIMD to itself for a while (its neighbour
        // waiting at the barrier or in its softmax) does not stall on every operand.
        if constexpr (DMA && DH == 128) {        // (head_dim 64 runs three workgroups per CU: no registers to spare)
            __builtin_amdgcn_sched_group_barrier(0x100, NSL > 1 ? 2 * NH : NH, 0);       // DS reads
#pragma unroll
            for (int s = 0; s < NSL; ++s) {
                __builtin_amdgcn_sched_group_barrier(0x008, NH * R, 0);                  // MFMA
                if (s + 2 < NSL) __builtin_amdgcn_sched_group_barrier(0x100, NH, 0);
            }
        }
        // Online softmax: the scores arrive as s - m in the exponent's units (multiplier in Q, -m in
        // the accumulators' starting value), so a probability is one exponential.  The max is moved
        // lazily: the exponentials are first taken against the current max, and as long as a lane's
        // sum of them stays <= 2^8 every P is at most 256, exact enough in the 16-bit format and
        // f32, and neither the max nor the accumulators are touched.  Only tiles that cross the
        // diagonal pay for the mask.
        const bool need_mask = sub_start + TT - 1 > wave_kv_min;       // wave-uniform
        uint4 pf[R][NH / 2];
        float alpha[R];
        bool grew[R];                                                  // wave-uniform
        auto softmax = [&](auto mask_tag) {
            constexpr bool MASK = decltype(mask_tag)::value;
#pragma unroll
            for (int c = 0; c < R; ++c) {
                constexpr int NS = 4 * NH;                                      // scores per lane
                float sc[NS];
                bool dead[NS];
#pragma unroll
                for (int k = 0; k < NS; ++k) sc[k] = sa[k >> 2][c][k & 3];
#pragma unroll
                for (int k = 0; k < NS; ++k) {
                    const int r = 16 * (k >> 2) + 4 * (k & 3) + g4;              // LDS row of this score
                    dead[k] = MASK && sub_start + r > qabs[c];
                    if (MASK && dead[k]) sc[k] = NEG_BIG;
                }
                // Exponentials against the current reference max, rounded to bf16 in pairs; the sum
                // of the rounded pairs (v_dot2c_f32_bf16 against ones: one instruction per two
                // probabilities, and the sum of exactly what the PV product multiplies) doubles as
                // the test that none of them outgrew the max.  The first tile always fails it (the
                // initial max is -1e30); a NaN sum is carried through on either path.
                uint32_t pk[NS / 2];
                float psum = 0.f;
                auto exps = [&]() {
                    psum = 0.f;
#pragma unroll
                    for (int k = 0; k < NS; k += 2) {
                        float p0 = __builtin_amdgcn_exp2f(sc[k]);
                        float p1 = __builtin_amdgcn_exp2f(sc[k + 1]);
                        if (MASK && dead[k]) p0 = 0.f;
                        if (MASK && dead[k + 1]) p1 = 0.f;
                        pk[k >> 1] = E::pack(p0, p1);
                        psum = E::pair_sum(pk[k >> 1], psum);
                    }
                };
                exps();
                // A row's scores sit in four lanes (l, l^16, l^32, l^48), which must share one
                // reference max, so the whole wave takes the slow path together: row max over the
                // lanes, rescale factor, exponentials again (the accumulator rescale is below).
                grew[c] = t == 0 || __any(!(psum <= 256.f));
                if (grew[c]) {
                    float mx_lane = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])),
                                          fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
                    if constexpr (NS == 16)
                        mx_lane = fmaxf(mx_lane, fmaxf(fmaxf(fmaxf(sc[8], sc[9]), fmaxf(sc[10], sc[11])),
                                                       fmaxf(fmaxf(sc[12], sc[13]), fmaxf(sc[14], sc[15]))));
                    float mx = xor16_max(mx_lane);
                    mx = xor32_max(mx);
                    // mx is relative to the current reference; the first tile adopts it whatever its sign
                    const float shift = (t == 0 || mx > 0.f) ? mx : 0.f;
                    alpha[c] = t == 0 ? 0.f : __builtin_amdgcn_exp2f(-shift);
                    m[c] += shift;
                    binit[c] = f32x4_t{-m[c], -m[c], -m[c], -m[c]};
                    lsum[c] *= alpha[c];
#pragma unroll
                    for (int k = 0; k < NS; ++k) sc[k] -= shift;
                    exps();
                }
                lsum[c] += psum;
#pragma unroll
                for (int hp = 0; hp < NH / 2; ++hp) {
                    uint4 pw;
                    pw.x = pk[4 * hp + 0]; pw.y = pk[4 * hp + 1]; pw.z = pk[4 * hp + 2]; pw.w = pk[4 * hp + 3];
                    pf[c][hp] = pw;
                }
            }
        };
        if (need_mask) softmax(std::true_type{}); else softmax(std::false_type{});
#pragma unroll
        for (int c = 0; c < R; ++c) {
            if (grew[c]) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) O[c][j] *= alpha[c];
            }
        }

        // ---- O^T += V^T P^T.  The A operand (element 16j + m for lane column m, eight tokens of
        // k-group g4) comes straight out of the row-major V tile with gfx950's transposing LDS
        // read: within 16 lanes, lane k points at four consecutive elements of one token (token
        // slot k/4, elements 16j + 4*(k%4) ..) and lane m receives element m%4 of the rows given
        // by lanes 4e + m/4, e = 0..3, i.e. element 16j + m of four tokens.  Two reads (k-slots
        // 0..3, 4..7) make one operand, which feeds the R column groups.
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            typedef short v4i16_t __attribute__((ext_vector_type(4)));
            typedef __attribute__((address_space(3))) v4i16_t* lds_v4i16_ptr;
            typedef short v8i16_t __attribute__((ext_vector_type(8)));
#pragma unroll
            for (int hp = 0; hp < NH / 2; ++hp) {
                const int voff = DMA ? 32 * hp * KROW + vrow * KROW + (((2 * j + ((r16 >> 1) & 1)) ^ swz_v(vrow)) << 4) + (r16 & 1) * 8
                                     : 32 * hp * KROW + rd_v + j * 32;
                const v4i16_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(vb + voff));
                const v4i16_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(vb + (voff + 16 * KROW)));
                const v8i16_t av = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                const uint4 a = __builtin_bit_cast(uint4, av);
#pragma unroll
                for (int c = 0; c < R; ++c)
                    O[c][j] = E::mfma(a, pf[c][hp], O[c][j]);
            }
        }
        // same for the V operand reads: two output tiles ahead of their MFMAs
        if constexpr (DMA && DH == 128) {
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * NH, 1);
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                __builtin_amdgcn_sched_group_barrier(0x008, (NH / 2) * R, 1);
                if (j + 2 < NJ) __builtin_amdgcn_sched_group_barrier(0x100, NH, 1);
            }
        }
    };
    // Every step issues its loads, also past the end (clamped to the last tile, never used): with
    // a fixed number of loads in flight the wait before a stage is written to LDS covers that
    // stage's loads only, not the younger ones of the other stage.  With two stages the loop
    // always runs both; a step past the last tile stages it again and skips the arithmetic.
    if constexpr (DMA) {
        StageT st;
        fetch_dma(0, dma_k0, dma_v0);
        for (int t = 0; t < ntiles; t += 2) {
            step(t, st, dma_k0, dma_v0, dma_k1, dma_v1);
            if (t + 1 < ntiles) step(t + 1, st, dma_k1, dma_v1, dma_k0, dma_v0);
        }
    } else if constexpr (KT == 32) {
        StageT st_a, st_b;
        fetch(0, st_a);
        fetch(min(1, ntiles - 1), st_b);
        for (int t = 0; t < ntiles; t += 2) {
            step(t, st_a, nullptr, nullptr, nullptr, nullptr);
            step(t + 1, st_b, nullptr, nullptr, nullptr, nullptr);
        }
    } else {
        StageT st;
        fetch(0, st);
        for (int t = 0; t < ntiles; ++t) step(t, st, nullptr, nullptr, nullptr, nullptr);
    }

    // lane (column r16 of column group c, g4) holds O^T[element 16*j + 4*g4 + i][column] in O[c][j][i]
#pragma unroll
    for (int c = 0; c < R; ++c) {
        float l = lsum[c];
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        if (row_valid[c]) {
            const float inv = (l > 0.f ? 1.f / l : 0.f) * (FP8 ? p.v_scale[kvh] : 1.f);
            uint16_t* o = (uint16_t*)p.out + ((int64_t)(q_begin + qpos[c]) * p.hq + head[c]) * DH + 4 * g4;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                *(uint2*)(o + 16 * j) = make_uint2(E::pack(O[c][j][0] * inv, O[c][j][1] * inv),
                                                   E::pack(O[c][j][2] * inv, O[c][j][3] * inv));
        }
    }
}

template <typename E, bool FP8, int R, int DH, bool DMA = false>
static hipError_t launch_prefill_variant(const PrefillParams& p, dim3 grid, size_t lds_bytes, hipStream_t stream) {
    // Two column groups stage 64-row tiles: 70 KB of dynamic LDS, above the 64 KB a kernel may use
    // without asking.  The limit is a per-device function attribute: set once per device.
    static std::atomic<unsigned long long> done{0};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const bool known = dev < 64 && ((done.load(std::memory_order_acquire) >> dev) & 1ull);
    if (!known) {
        e = hipFuncSetAttribute((const void*)paged_prefill_mfma_kernel<E, FP8, R, DH, DMA>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return e;
        if (dev < 64) done.fetch_or(1ull << dev, std::memory_order_release);
    }
    hipLaunchKernelGGL((paged_prefill_mfma_kernel<E, FP8, R, DH, DMA>), grid, dim3(256), lds_bytes, stream, p);
    return hipSuccess;
}

}  // namespace

bool prefill_mfma_supported(const DecodeArgs& a, int max_q_len) {
    const int group = a.hkv > 0 ? a.hq / a.hkv : 0;
    return a.cu_q_lens != nullptr && max_q_len > 0 && (a.d == 128 || a.d == 64) && a.bs == BS &&
           is_16bit_float(a.q_dtype) &&
           (a.kv_dtype == a.q_dtype || a.kv_dtype == AICOMP_KV_FP8_E4M3) && group >= 1 &&
           // the score multiplier is rounded into Q: fp16 queries keep it within a range where
           // q * multiplier stays a normal fp16 number for ordinary q (bf16 has float's range)
           a.scale > 0.f && (a.q_dtype == AICOMP_KV_BF16 || (a.scale >= 0x1p-12f && a.scale <= 0x1p8f)) && a.num_seqs <= 65535 && ((uintptr_t)a.query % 16 == 0) &&
           ((uintptr_t)a.out % 16 == 0) && ((uintptr_t)a.k_pool % 16 == 0) &&
           ((uintptr_t)a.v_pool % 16 == 0);
}

// positions of one query tile (one workgroup row) for these shapes: what an item list is cut into
int prefill_mfma_tile_positions(int hq, int hkv, int max_q_len) {
    const int group = hq / hkv;
    const int gpack = (16 % group == 0) ? group : 1;
    const int R = (int64_t)max_q_len * gpack >= 2 * ROWS ? 2 : 1;
    return ROWS * R / gpack;
}

int launch_prefill_mfma(const DecodeArgs& a, int max_q_len) {
    PrefillParams p;
    p.out = a.out; p.query = a.query; p.k_pool = a.k_pool; p.v_pool = a.v_pool;
    p.block_table = a.block_table; p.block_table_stride = a.block_table_stride;
    p.context_lens = a.context_lens; p.cu_q_lens = a.cu_q_lens;
    p.hq = a.hq; p.hkv = a.hkv; p.group = a.hq / a.hkv; p.max_blocks = a.max_blocks;
    AICOMP_REQUIRE(a.num_blocks <= INT32_MAX, AICOMP_KV_EINVAL, "paged_prefill_attn: num_blocks too large");
    p.num_blocks = (int)a.num_blocks;
    p.gpack = (16 % p.group == 0) ? p.group : 1;      // heads of one KV head packed per position
    // CU count of the first device used (every GPU of a node is the same part); 0 if unknown, which
    // only turns the cost-ranked item order off
    static std::atomic<int> cached_cus{-1};
    int num_cus = cached_cus.load(std::memory_order_relaxed);
    if (num_cus < 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 0)
            n = 0;
        num_cus = n;
        cached_cus.store(n, std::memory_order_relaxed);
    }
    p.num_cus = num_cus;
    p.qk_mul = a.scale * LOG2E;
    p.k_scale = a.k_scale; p.v_scale = a.v_scale;
    p.items = a.items; p.num_seqs = a.num_seqs;
    // two column groups per wave (128 rows per workgroup) once a chunk has that many rows
    const int R = (int64_t)max_q_len * p.gpack >= 2 * ROWS ? 2 : 1;
    const int pos_per_wg = ROWS * R / p.gpack;
    const int qtiles = (max_q_len + pos_per_wg - 1) / pos_per_wg;
    AICOMP_REQUIRE(qtiles <= 65535, AICOMP_KV_EINVAL, "paged_prefill_attn: grid too large");
    dim3 grid((unsigned)(a.hq / p.gpack), (unsigned)a.num_seqs, (unsigned)qtiles);
    if (a.items != nullptr) grid = dim3((unsigned)(a.hq / p.gpack), (unsigned)a.num_items, 1);
    // double-buffered K and V tiles of 32 (R = 1) or 64 rows of 2*D + 16 bytes
    const size_t lds_bytes = (size_t)4 * (R == 1 ? 32 : 64) * (2 * a.d + 16);
    const bool fp8 = a.kv_dtype == AICOMP_KV_FP8_E4M3;
    hipError_t e;
#define AICOMP_LAUNCH_PREFILL(E)                                                                                      \
    do {                                                                                                              \
        if (a.d == 64) {                                                                                              \
            if (fp8 && R == 2) e = launch_prefill_variant<E, true, 2, 64>(p, grid, lds_bytes, a.stream);              \
            else if (fp8) e = launch_prefill_variant<E, true, 1, 64>(p, grid, lds_bytes, a.stream);                   \
            else if (R == 2) e = launch_prefill_variant<E, false, 2, 64, true>(p, grid, 0, a.stream);  /* static LDS */ \
            else e = launch_prefill_variant<E, false, 1, 64>(p, grid, lds_bytes, a.stream);                           \
        } else {                                                                                                      \
            if (fp8 && R == 2) e = launch_prefill_variant<E, true, 2, 128>(p, grid, lds_bytes, a.stream);             \
            else if (fp8) e = launch_prefill_variant<E, true, 1, 128>(p, grid, lds_bytes, a.stream);                  \
            else if (R == 2) e = launch_prefill_variant<E, false, 2, 128, true>(p, grid, 0, a.stream); /* static LDS */ \
            else e = launch_prefill_variant<E, false, 1, 128>(p, grid, lds_bytes, a.stream);                          \
        }                                                                                                             \
    } while (0)
    if (a.q_dtype == AICOMP_KV_F16) AICOMP_LAUNCH_PREFILL(F16Fmt);
    else AICOMP_LAUNCH_PREFILL(Bf16Fmt);
#undef AICOMP_LAUNCH_PREFILL
    AICOMP_REQUIRE(e == hipSuccess, AICOMP_KV_EHIP, "paged_prefill_attn: %s", hipGetErrorString(e));
    AICOMP_HIP_LAUNCH_CHECK();
    return AICOMP_KV_OK;
}

}  // namespace aicomp
