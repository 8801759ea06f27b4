// Paged decode attention on gfx950 matrix cores: the hot kernel of the path.
//
// Replaces  F.scaled_dot_product_attention(query, full_key, full_value,
//           attn_mask=None, is_causal=False)      opt_prime/opt_prime/kv_cache.py:397-403
// and the two .contiguous() prefix copies that feed it (kv_cache.py:391-392):
// K and V are read once, in place, through the block table.
//
// Shape covered: head_dim 128, block_size 16, bf16 or fp16 queries, pools of the query type or
// fp8-e4m3 (the kernels are written over a 16-bit element format, see common.h), up to 16 query heads per KV head; and head_dim 64 (up to 8 heads per KV
// head) by treating two consecutive tokens, which are contiguous in the pool, as
// one 128-element row: every head takes two B-operand columns, one per token
// parity, with the query in the matching half of the row and zeros in the other,
// and the two columns' partial softmaxes are merged at the end.  Same instruction
// stream per byte as head_dim 128.  Everything else goes to the vector-ALU kernel.
//
// HBM-bound: per sequence 2 * L * Hkv * D * e_kv bytes of K/V are streamed and
// used exactly once; 4 * G flop per byte (bf16), far below the MFMA roof, so
// the design goal is bytes in flight, not flops.
//
// Work split   one workgroup (4 waves) per (partition, KV head, sequence).
//              A wave owns whole 32-token tiles (two 16-token blocks) and its
//              own online-softmax state; no workgroup barrier in the loop.
// Loads        a (block, KV head) tile is 16 rows * 256 B contiguous (bf16):
//              each global_load_dwordx4 of a wave reads 1 KB = 4 whole rows,
//              lane l -> row l/16, 16-byte chunk l%16.  One table lookup per
//              block, wave-uniform (scalar).
// K            staged through a wave-private LDS tile (unpadded 256-byte rows whose
//              16-byte chunks are permuted by a function of the row, so that the
//              operand reads run at the full LDS rate) and read back
//              as the A operand of  S^T = K Q^T  (v_mfma_f32_16x16x32_bf16 / _f16),
//              the G query heads (padded to 16 columns) sharing every K tile.
// V            never touches LDS.  Lane (c = l%16, q = l/16) of load i holds
//              dims 8c..8c+7 of token 4i+q; picking the j-th 16-bit half of
//              loads 0..7 (v_perm_b32) is exactly the A operand of
//              O^T[dim 8c+j][head] += V^T P^T  for the token order the QK
//              product was laid out in (rows of the K tile are permuted on the
//              LDS read to match), so P goes from accumulator to operand
//              without leaving its lane.
// Softmax      log2 domain, running max per head made wave-uniform with two
//              wave shuffles (lanes l, l^16, l^32, l^48 hold the same head).
// Split-K      partitions write (max, sum, unnormalised output) to the
//              workspace; a second, small kernel merges them.
#include "common.h"

#include <atomic>

namespace aicomp {

namespace {

constexpr int D = 128;
constexpr int BS = 16;
constexpr int TILE = 32;               // tokens per wave iteration (two blocks)
constexpr int NWAVES = 4;
constexpr int KROW = 256;              // LDS row stride in bytes: unpadded, 16-byte chunks swizzled (below)
constexpr int KTILE_BYTES = TILE * KROW;   // 8192 per wave
constexpr float NEG_BIG = -1.0e30f;
constexpr int SK_MAX_WAVES = 4096;     // balanced schedule: at most 1024 workgroups of 4 waves

struct MfmaParams {
    void* out;
    const void* query;
    void* k_pool;
    void* v_pool;
    const int32_t* block_table;
    int64_t block_table_stride;
    const int32_t* context_lens;
    int hq, hkv, group, max_blocks;
    int64_t num_blocks;
    float qk_mul;               // scale * log2(e)
    const float* k_scale;
    const float* v_scale;
    int partition_size, num_parts;
    float* ws_acc;
    float* ws_ml;
    // fused append (optional): row b of new_key / new_value is token context_lens[b]-1
    const uint16_t* new_key;
    const uint16_t* new_value;
    int64_t new_token_stride, new_head_stride;     // elements
};

template <bool FP8> struct TileRegs;
template <> struct TileRegs<false> { uint4 r[8]; };
template <> struct TileRegs<true> { uint2 r[8]; };

// Issue the 8 loads of one 32-token tile of one pool.  blk0/blk1 are the two
// physical blocks (wave-uniform); lane l reads row l/16, chunk l%16 of each
// 4-row group.
// K/V rows are read exactly once per call: non-temporal loads keep them from displacing
// everything else in L2 (measured: 114 -> 101 us on the Llama-3-8B decode shape).
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 tile_ld(const uint4* p) {
    u32x4_t v = __builtin_nontemporal_load((const u32x4_t*)p);
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint2 tile_ld(const uint2* p) {
    u32x2_t v = __builtin_nontemporal_load((const u32x2_t*)p);
    return make_uint2(v[0], v[1]);
}
#define TILE_LD(ptr) tile_ld(ptr)
template <bool FP8>
__device__ __forceinline__ void load_tile(TileRegs<FP8>& t, const void* pool, int64_t blk0,
                                          int64_t blk1, int hkv, int kvh, int lane) {
    if constexpr (FP8) {
        const uint2* p0 = (const uint2*)pool + (blk0 * hkv + kvh) * (BS * D / 8) + lane;
        const uint2* p1 = (const uint2*)pool + (blk1 * hkv + kvh) * (BS * D / 8) + lane;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            t.r[i] = TILE_LD(p0 + i * 64);
            t.r[4 + i] = TILE_LD(p1 + i * 64);
        }
    } else {
        const uint4* p0 = (const uint4*)pool + (blk0 * hkv + kvh) * (BS * D / 8) + lane;
        const uint4* p1 = (const uint4*)pool + (blk1 * hkv + kvh) * (BS * D / 8) + lane;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            t.r[i] = TILE_LD(p0 + i * 64);
            t.r[4 + i] = TILE_LD(p1 + i * 64);
        }
    }
}

// head_dim 64: a 32-row tile of 128-element rows is 64 tokens, each row a PAIR of consecutive
// tokens (token 2r in elements 0..63, token 2r+1 in 64..127; contiguous in the pool).  Four
// blocks of 8 such rows.
template <bool FP8>
__device__ __forceinline__ void load_tile_pair(TileRegs<FP8>& t, const void* pool, int64_t blk0, int64_t blk1,
                                               int64_t blk2, int64_t blk3, int hkv, int kvh, int lane) {
    const int64_t blk[4] = {blk0, blk1, blk2, blk3};
    if constexpr (FP8) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint2* p = (const uint2*)pool + (blk[b] * hkv + kvh) * (BS * 64 / 8) + lane;
            t.r[2 * b] = TILE_LD(p);
            t.r[2 * b + 1] = TILE_LD(p + 64);
        }
    } else {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint4* p = (const uint4*)pool + (blk[b] * hkv + kvh) * (BS * 64 / 8) + lane;
            t.r[2 * b] = TILE_LD(p);
            t.r[2 * b + 1] = TILE_LD(p + 64);
        }
    }
}

// load i of a tile as eight elements of the query's 16-bit format E (fp8 pools are widened, exactly)
template <typename E, bool FP8>
__device__ __forceinline__ uint4 tile_elems(const TileRegs<FP8>& t, int i) {
    if constexpr (FP8) return E::from_fp8(t.r[i]);
    else return t.r[i];
}

__device__ __forceinline__ int64_t clamp_block(int b, int64_t num_blocks) {
    return b < 0 ? 0 : (b >= num_blocks ? num_blocks - 1 : (int64_t)b);
}

// Where a lane writes and reads the wave's K tile.  Chunk slot s of tile row r holds the row's
// chunk s ^ swz(r), swz(r) = ((r / 4) % 4) | ((r % 4) * 4): the operand read below then has every
// four consecutive lanes in one aligned 64-byte segment and each half-wave spread evenly over the
// four segments of a 256-byte bank line, which is what the LDS needs to deliver 256 bytes per
// clock (rows padded to 272 bytes are free of bank collisions among the sixteen lanes of an MFMA
// row group, yet run at half that rate: a quarter of the LDS cycles were conflict cycles).
//   write  load i of lane (q = lane / 16, c = lane % 16) is row 4 i + q, chunk c:
//          swz = (i % 4) | (q * 4), so four distinct offsets, picked by i % 4
//   read   sub-tile a, k-step s, lane (r16, g4): row 16 a + 4 (r16 % 4) + r16 / 4, chunk 4 s + g4:
//          swz of that row is r16 itself, so the slot is (4 s + g4) ^ r16
struct KTileOffsets {
    int wr[4];
    int rd[4];
};
__device__ __forceinline__ KTileOffsets k_tile_offsets(int lane) {
    const int r16 = lane & 15, g4 = lane >> 4;
    KTileOffsets o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        o.wr[k] = g4 * KROW + ((r16 ^ (k | (g4 << 2))) << 4);
        o.rd[k] = (4 * (r16 & 3) + (r16 >> 2)) * KROW + (((4 * k + g4) ^ r16) << 4);
    }
    return o;
}

// Per-wave running state of the online softmax and the output accumulators.
struct WaveState {
    float m, lsum;
    f32x4_t O[8];
};

// One 32-token tile: K registers -> LDS -> S^T = K Q^T -> online softmax -> O^T += V^T P^T.
// NEXT: prefetch the wave's next tile (blocks nb0/nb1) into the same registers.
// MASK: the tile crosses `end`; scores beyond it are dropped and their V rows zeroed.
// PAIR: rows are token pairs (head_dim 64): row r of the tile holds tokens tile_start + 2r and
// + 2r + 1, the B-operand columns are (head, parity) pairs, column c scoring token 2r + (c & 1).
template <typename E, bool FP8, bool NEXT, bool MASK, bool PAIR = false>
__device__ __forceinline__ void process_tile(WaveState& st, TileRegs<FP8>& kr, TileRegs<FP8>& vr,
                                             const uint4 (&qf)[4], unsigned char* kt, const KTileOffsets& ko,
                                             const void* k_pool, const void* v_pool,
                                             int64_t nb0, int64_t nb1, int hkv, int kvh_next, int lane,
                                             int g4, int tile_start, int end, float cmul,
                                             int64_t nb2 = 0, int64_t nb3 = 0) {
    // ---- K tile -> LDS, then prefetch the next K tile into the same registers
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        uint4 kk = tile_elems<E, FP8>(kr, i);
        // PAIR: a row's two tokens share every dot product (the query column is zero over the other
        // token's half), so a token beyond the context must not leave non-finite values in the row
        if (PAIR && MASK && tile_start + 2 * (4 * i + g4) + ((lane & 15) >> 3) >= end) kk = make_uint4(0, 0, 0, 0);
        *(uint4*)(kt + ko.wr[i & 3] + i * 4 * KROW) = kk;
    }
    if (NEXT) {
        if constexpr (PAIR) load_tile_pair<FP8>(kr, k_pool, nb0, nb1, nb2, nb3, hkv, kvh_next, lane);
        else load_tile<FP8>(kr, k_pool, nb0, nb1, hkv, kvh_next, lane);
    }

    // ---- S^T = K Q^T for the two 16-token sub-tiles
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        const uint4 a0 = *(const uint4*)(kt + ko.rd[s]);
        const uint4 a1 = *(const uint4*)(kt + ko.rd[s] + 16 * KROW);
        s0 = E::mfma(a0, qf[s], s0);
        s1 = E::mfma(a1, qf[s], s1);
    }
    // lane (head r16, g4) now holds tokens tile_start + 16a + 4i + g4 in s_a[i]
    float sc[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) { sc[i] = s0[i] * cmul; sc[4 + i] = s1[i] * cmul; }
    if (MASK) {
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int r = 16 * (k >> 2) + 4 * (k & 3) + g4;
            const int tok = PAIR ? tile_start + 2 * r + (lane & 1) : tile_start + r;
            if (tok >= end) sc[k] = NEG_BIG;
        }
    }
    float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])),
                     fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(st.m, mx);
    const float alpha = exp2f(st.m - m_new);
    float pr[8], psum = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        pr[k] = exp2f(sc[k] - m_new);
        if (MASK && sc[k] == NEG_BIG) pr[k] = 0.f;
        psum += pr[k];
    }
    st.lsum = st.lsum * alpha + psum;
    st.m = m_new;
    if (__any(alpha != 1.f)) {
#pragma unroll
        for (int j = 0; j < 8; ++j) st.O[j] *= alpha;
    }
    // P^T as the B operand: k-slot 4a + i <-> token 16a + 4i + g4, this lane's own values
    uint4 pw;
    pw.x = E::pack(pr[0], pr[1]); pw.y = E::pack(pr[2], pr[3]);
    pw.z = E::pack(pr[4], pr[5]); pw.w = E::pack(pr[6], pr[7]);

    // ---- V: registers -> A operand of O^T += V^T P^T.  Load i of lane (c, q) is token 4i + q.
    uint4 vv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        vv[i] = tile_elems<E, FP8>(vr, i);
        // PAIR: chunks 8..15 of a row belong to the pair's second token
        const int vtok = PAIR ? tile_start + 2 * (4 * i + g4) + ((lane & 15) >> 3) : tile_start + 4 * i + g4;
        if (MASK && vtok >= end) vv[i] = make_uint4(0, 0, 0, 0);
    }
    uint4 af[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
        const uint32_t* v0 = (const uint32_t*)&vv[0];
        af[j].x = __builtin_amdgcn_perm(v0[4 * 1 + (j >> 1)], v0[4 * 0 + (j >> 1)], sel);
        af[j].y = __builtin_amdgcn_perm(v0[4 * 3 + (j >> 1)], v0[4 * 2 + (j >> 1)], sel);
        af[j].z = __builtin_amdgcn_perm(v0[4 * 5 + (j >> 1)], v0[4 * 4 + (j >> 1)], sel);
        af[j].w = __builtin_amdgcn_perm(v0[4 * 7 + (j >> 1)], v0[4 * 6 + (j >> 1)], sel);
    }
    if (NEXT) {
        if constexpr (PAIR) load_tile_pair<FP8>(vr, v_pool, nb0, nb1, nb2, nb3, hkv, kvh_next, lane);
        else load_tile<FP8>(vr, v_pool, nb0, nb1, hkv, kvh_next, lane);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
        st.O[j] = E::mfma(af[j], pw, st.O[j]);
}

// 8 elements of format E -> 8 e4m3 codes: clamp(x / scale, +-448), round to nearest even
template <typename E>
__device__ __forceinline__ uint2 quant8_fp8(const uint4& x, float scale) {
    const uint32_t w[4] = {x.x, x.y, x.z, x.w};
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = fminf(fmaxf(E::to_f32((uint16_t)(w[i] & 0xffffu)) / scale, -448.f), 448.f);
        f[2 * i + 1] = fminf(fmaxf(E::to_f32((uint16_t)(w[i] >> 16)) / scale, -448.f), 448.f);
    }
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
    return make_uint2((uint32_t)lo, (uint32_t)hi);
}

// Fused append for the grid-scheduled kernel: the tile that holds the sequence's newest token
// (context_lens - 1) takes its K/V row from new_key / new_value instead of what was loaded from
// the pool, and writes it to the pool (the append itself).  No other wave of the launch reads
// that token.  A tile row is one token (16 lanes of 8 elements), or with PAIR half a row (8 lanes).
template <typename E, bool FP8, bool PAIR, typename Params>
__device__ __forceinline__ void inject_new_row_grid(TileRegs<FP8>& kr, TileRegs<FP8>& vr, const Params& p,
                                                    int seq, int kvh, int lane, int tile_start, int len,
                                                    const int64_t (&bb)[4]) {
    constexpr int DQ = PAIR ? 64 : D;
    const int tau = len - 1 - tile_start;              // token within the tile, wave-uniform
    const int blk_i = tau >> 4, tb = tau & 15;         // block of the tile, token within the block
    const int c = PAIR ? (lane & 7) : (lane & 15);     // 8-element chunk of the new row this lane holds
    // register slot and lanes of that token: load i of lane l is row 4i + l/16 (chunk l%16) of the tile
    const int row = PAIR ? (tau >> 1) : tau;
    const bool mine = (lane >> 4) == (row & 3) && (!PAIR || ((lane >> 3) & 1) == (tau & 1));
    const int slot = row >> 2;
    const int64_t src = (int64_t)seq * p.new_token_stride + (int64_t)kvh * p.new_head_stride + 8 * c;
    const uint4 nk = *(const uint4*)(p.new_key + src);
    const uint4 nv = *(const uint4*)(p.new_value + src);
    const int64_t blk = bb[blk_i];
    const int64_t dst = ((blk * p.hkv + kvh) * BS + tb) * (DQ / 8) + c;        // 8-element chunks
    if constexpr (FP8) {
        const uint2 ck = quant8_fp8<E>(nk, p.k_scale[kvh]);
        const uint2 cv = quant8_fp8<E>(nv, p.v_scale[kvh]);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (mine && i == slot) { kr.r[i] = ck; vr.r[i] = cv; }
        if (mine) { ((uint2*)p.k_pool)[dst] = ck; ((uint2*)p.v_pool)[dst] = cv; }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (mine && i == slot) { kr.r[i] = nk; vr.r[i] = nv; }
        if (mine) { ((uint4*)p.k_pool)[dst] = nk; ((uint4*)p.v_pool)[dst] = nv; }
    }
}

template <typename E, bool FP8, bool PAIR>
__global__ void __launch_bounds__(256, 2)
paged_decode_mfma_kernel(MfmaParams p) {
    // KV head fastest: the workgroups launched together read the Hkv slices of the same
    // physical blocks, i.e. one contiguous Hkv*4 KB piece of each pool
    constexpr int DQ = PAIR ? 64 : D;            // head_dim of the tensors
    constexpr int TT = PAIR ? 2 * TILE : TILE;   // tokens per tile
    constexpr int BPT = TT / BS;                 // blocks per tile
    const int kvh = blockIdx.x;
    const int part = blockIdx.y;
    const int seq = blockIdx.z;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15;      // MFMA row / column index of this lane
    const int g4 = lane >> 4;       // MFMA k-group of this lane
    const int G = p.group;
    const int ncol = PAIR ? 2 * G : G;           // B-operand columns in use
    const int start = part * p.partition_size;
    const int blk_base = start / BS;

    // Prologue loads, all issued before anything waits: the context length (scalar), the
    // partition's slice of the block table (one coalesced vector load: lane i holds entry
    // blk_base + i, later picked out with v_readlane, so the loop has no table loads at
    // all) and the query rows.
    const int32_t* table = p.block_table + (int64_t)seq * p.block_table_stride;
    int tab_first = 0;                       // first entry (relative to blk_base) held in `tab`
    int tab = (blk_base + lane < p.max_blocks) ? table[blk_base + lane] : 0;

    // Q as the B operand of S^T = K Q^T: column = head r16, k-slots = dims 32s + 8*g4 ..
    // PAIR: column c is (head c/2, parity c%2); a row of the K tile is [token 2r | token 2r+1], so
    // the column carries the query in elements 0..63 (parity 0) or 64..127 (parity 1), zeros elsewhere.
    uint4 qf[4];
    {
        const int h = PAIR ? (r16 >> 1) : r16;
        const uint16_t* qrow = (const uint16_t*)p.query + ((int64_t)seq * p.hq + kvh * G + min(h, G - 1)) * DQ;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int e0 = 32 * s + 8 * g4;                       // first element of this k-slot in the row
            bool use = r16 < ncol;
            int src = e0;
            if constexpr (PAIR) {
                use = use && ((e0 >= 64) == ((r16 & 1) != 0));
                src = e0 & 63;
            }
            uint4 v = *(const uint4*)(qrow + src);
            if (!use) v = make_uint4(0, 0, 0, 0);
            qf[s] = v;
        }
    }

    const int len = min(p.context_lens[seq], p.max_blocks * BS);   // never read past the table row
    if (start >= len) {
        if (len <= 0 && part == 0) {   // nothing to attend to: the output row is defined as zero
            uint16_t* o = (uint16_t*)p.out + ((int64_t)seq * p.hq + kvh * G) * DQ;
            for (int i = tid; i < G * DQ; i += blockDim.x) o[i] = 0;
        }
        return;
    }
    const int end = min(len, start + p.partition_size);
    const int ntiles = (end - start + TT - 1) / TT;

    __shared__ __attribute__((aligned(16))) unsigned char lds[NWAVES * KTILE_BYTES];
    __shared__ float sm_m[NWAVES][16];
    __shared__ float sm_l[NWAVES][16];
    unsigned char* kt = lds + w * KTILE_BYTES;

    const float cmul = p.qk_mul * (FP8 ? p.k_scale[kvh] : 1.f);

    WaveState st;
    st.m = NEG_BIG; st.lsum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) st.O[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // physical blocks of tile tt (wave-uniform); the held table slice is refilled every 64 blocks
    int64_t bb[4] = {0, 0, 0, 0};
    auto tile_blocks = [&](int tt) {
        const int i0 = BPT * tt;
        if (i0 - tab_first >= 64) {
            tab_first = i0;
            tab = (blk_base + i0 + lane < p.max_blocks) ? table[blk_base + i0 + lane] : 0;
            __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0) here, so the common path never waits on `tab`
        }
#pragma unroll
        for (int j = 0; j < BPT; ++j)
            bb[j] = clamp_block(__builtin_amdgcn_readlane(tab, i0 + j - tab_first), p.num_blocks);
    };

    const KTileOffsets ko = k_tile_offsets(lane);

    if (w < ntiles) {
        TileRegs<FP8> kr, vr;
        tile_blocks(w);
        // Q must have landed before the tile loads are issued: the loop's waits then count
        // only tile loads, so a wave computes on tile t while tile t+1 is still in flight.
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        if constexpr (PAIR) {
            load_tile_pair<FP8>(kr, p.k_pool, bb[0], bb[1], bb[2], bb[3], p.hkv, kvh, lane);
            load_tile_pair<FP8>(vr, p.v_pool, bb[0], bb[1], bb[2], bb[3], p.hkv, kvh, lane);
        } else {
            load_tile<FP8>(kr, p.k_pool, bb[0], bb[1], p.hkv, kvh, lane);
            load_tile<FP8>(vr, p.v_pool, bb[0], bb[1], p.hkv, kvh, lane);
        }
        int tt = w;
        for (; tt + NWAVES < ntiles; tt += NWAVES) {      // steady state: never the partition's last tile
            tile_blocks(tt + NWAVES);
            process_tile<E, FP8, true, false, PAIR>(st, kr, vr, qf, kt, ko, p.k_pool, p.v_pool, bb[0],
                                                 bb[1], p.hkv, kvh, lane, g4, start + tt * TT, end, cmul,
                                                 bb[2], bb[3]);
        }
        const int tile_start = start + tt * TT;
        // the sequence's newest token lives in this tile (bb still holds its blocks: the last lookup
        // above was for this wave's final tile)
        if (p.new_key != nullptr && end == len && tile_start < len && tile_start + TT >= len) {
            // Same rule as the separate one-token append: the row is stored only where the table names a
            // block of the pool and the length fits the table; otherwise the call leaves the pools alone
            // (and attends over what the clamped table entry holds, like the unfused sequence of calls).
            const int raw_blk = __builtin_amdgcn_readlane(tab, BPT * tt + ((len - 1 - tile_start) >> 4) - tab_first);
            if (p.context_lens[seq] == len && raw_blk >= 0 && raw_blk < p.num_blocks)
                inject_new_row_grid<E, FP8, PAIR>(kr, vr, p, seq, kvh, lane, tile_start, len, bb);
        }
        if (tile_start + TT > end)
            process_tile<E, FP8, false, true, PAIR>(st, kr, vr, qf, kt, ko, p.k_pool, p.v_pool, 0, 0,
                                                 p.hkv, kvh, lane, g4, tile_start, end, cmul);
        else
            process_tile<E, FP8, false, false, PAIR>(st, kr, vr, qf, kt, ko, p.k_pool, p.v_pool, 0, 0,
                                                  p.hkv, kvh, lane, g4, tile_start, end, cmul);
    }
    const float m = st.m;
    float lsum = st.lsum;
    f32x4_t (&O)[8] = st.O;

    // ---- wave result: lane (column r16, g4) holds O^T[element 32*g4 + 8*i + j][column] in O[j][i]
    lsum += __shfl_xor(lsum, 16);
    lsum += __shfl_xor(lsum, 32);
    float* osm = (float*)kt;        // this wave's own K tile region, 16 columns * 128 floats = 8192 bytes, the whole tile
    if (r16 < ncol) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float4 a = make_float4(O[0][i], O[1][i], O[2][i], O[3][i]);
            float4 b = make_float4(O[4][i], O[5][i], O[6][i], O[7][i]);
            float* dst = osm + r16 * D + 32 * g4 + 8 * i;
            *(float4*)dst = a;
            *(float4*)(dst + 4) = b;
        }
        if (g4 == 0) { sm_m[w][r16] = m; sm_l[w][r16] = lsum; }
    }
    __syncthreads();

    // merge of the waves (PAIR: and of the two parity columns of a head, whose useful halves are
    // elements 0..63 and 64..127 of their accumulators)
    const float vs = FP8 ? p.v_scale[kvh] : 1.f;
    const bool direct = p.num_parts == 1;     // unsplit call: no merge needed
    constexpr int NPAR = PAIR ? 2 : 1;
    for (int idx = tid; idx < G * DQ; idx += 256) {
        const int h = idx / DQ, dd = idx % DQ;
        float mxw = NEG_BIG;
#pragma unroll
        for (int ww = 0; ww < NWAVES; ++ww)
#pragma unroll
            for (int par = 0; par < NPAR; ++par) mxw = fmaxf(mxw, sm_m[ww][NPAR * h + par]);
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int ww = 0; ww < NWAVES; ++ww) {
#pragma unroll
            for (int par = 0; par < NPAR; ++par) {
                const int c = NPAR * h + par;
                const float f = exp2f(sm_m[ww][c] - mxw);
                num = fmaf(f, ((const float*)(lds + ww * KTILE_BYTES))[c * D + dd + 64 * par], num);
                den = fmaf(f, sm_l[ww][c], den);
            }
        }
        const int head = kvh * G + h;
        if (direct) {
            ((uint16_t*)p.out)[((int64_t)seq * p.hq + head) * DQ + dd] =
                E::from_f32(den > 0.f ? vs * num / den : 0.f);
        } else {
            const int64_t slot = ((int64_t)seq * p.hq + head) * p.num_parts + part;
            p.ws_acc[slot * DQ + dd] = num;
            if (dd == 0) { p.ws_ml[slot * 2] = mxw; p.ws_ml[slot * 2 + 1] = den; }
        }
    }
}


// ---------------------------------------------------------------------------------------
// Balanced schedule.  The grid above gives the hardware dispatcher workgroups of unequal
// size and leaves a tail where few of them are still streaming.  Here the launch is
// exactly one workgroup per CU and every WAVE gets the same number of 32-token tiles.
// Waves are dealt to KV heads first (wave i: head i % Hkv, part i / Hkv of that head); the
// tiles of one head over all sequences form one sequence of N tiles and part j of W owns
// tiles [j*N/W, (j+1)*N/W).  The Hkv waves of one part walk the same tiles of the same
// sequences side by side, i.e. the Hkv adjacent head slices of the same physical blocks at
// about the same time, whatever the sequences' lengths (with KV heads inside the tile order
// instead, waves drift apart on batches of unequal lengths and read isolated 2 - 4 KB slices:
// 221 -> 211 us on the fp8 Llama-3-70B shape, bf16 shapes unchanged).  A wave crossing a
// sequence boundary flushes its partial (max, sum, unnormalised output) and starts the next
// sequence, so all waves start together, stream the same number of bytes and finish together.
// Partials of head h go to slot h * (W + S) + part + sequence - strictly increasing along a
// head's schedule, hence unique - and streamk_reduce_kernel merges the slots of each row.
// No barrier after the prologue.
constexpr int SK_MAX_SEQS = 1024;

struct StreamKParams {
    void* out;
    const void* query;
    void* k_pool;
    void* v_pool;
    const int32_t* block_table;
    int64_t block_table_stride;
    const int32_t* context_lens;
    int num_seqs, hq, hkv, group, max_blocks;
    int64_t num_blocks;
    float qk_mul;
    const float* k_scale;
    const float* v_scale;
    int num_waves;
    int waves_per_head;     // num_waves / hkv
    float* ws_acc;      // [slots][G][D]
    float* ws_ml;       // [slots][G][2]
    int* ws_rows;       // [rows][2]: first and last part (wave of the row's head) holding a partial of the row
    // fused append (optional): row b of new_key / new_value is token context_lens[b]-1
    const uint16_t* new_key;
    const uint16_t* new_value;
    int64_t new_token_stride, new_head_stride;     // elements
};

// Fused append: the row's last tile holds the sequence's newest token, whose K/V are not in
// the pool yet.  The 16 lanes that own that row take it from new_key / new_value instead of
// what they loaded, and write it to the pool (the append itself).  No other wave of this
// launch reads that token, so no cross-wave ordering is needed.
template <typename E, bool FP8>
__device__ __forceinline__ void inject_new_row(TileRegs<FP8>& kr, TileRegs<FP8>& vr,
                                               const StreamKParams& p, int seq, int kvh, int lane,
                                               int tile_start, int len, int64_t b0, int64_t b1) {
    const int tau = len - 1 - tile_start;              // 0..31, wave-uniform
    const int c = lane & 15, q = lane >> 4;
    const int64_t src = (int64_t)seq * p.new_token_stride + (int64_t)kvh * p.new_head_stride + 8 * c;
    const uint4 nk = *(const uint4*)(p.new_key + src);
    const uint4 nv = *(const uint4*)(p.new_value + src);
    const bool mine = (tau & 3) == q;
    const int64_t blk = tau < 16 ? b0 : b1;
    const int64_t dst = ((blk * p.hkv + kvh) * BS + (tau & 15)) * (D / 8) + c;   // 8-element chunks
    if constexpr (FP8) {
        const uint2 ck = quant8_fp8<E>(nk, p.k_scale[kvh]);
        const uint2 cv = quant8_fp8<E>(nv, p.v_scale[kvh]);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (mine && i == (tau >> 2)) { kr.r[i] = ck; vr.r[i] = cv; }
        if (mine) { ((uint2*)p.k_pool)[dst] = ck; ((uint2*)p.v_pool)[dst] = cv; }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (mine && i == (tau >> 2)) { kr.r[i] = nk; vr.r[i] = nv; }
        if (mine) { ((uint4*)p.k_pool)[dst] = nk; ((uint4*)p.v_pool)[dst] = nv; }
    }
}

template <int TT>
__device__ __forceinline__ int sk_tiles(int len, int max_blocks) {
    len = min(max(len, 0), max_blocks * BS);
    return (len + TT - 1) / TT;
}


// PAIR: head_dim 64 as rows of token pairs (see paged_decode_mfma_kernel): a tile is 64 tokens in
// four blocks, every head takes two B-operand columns (one per token parity), and a flush merges
// the two columns of a head inside the wave and writes one partial of 64 floats per head.
template <typename E, bool FP8, bool PAIR>
__global__ void __launch_bounds__(256, 1)     // one workgroup per CU: a wave may use the whole register file
streamk_decode_kernel(StreamKParams p) {
    constexpr int DQ = PAIR ? 64 : D;            // head_dim of the tensors
    constexpr int TT = PAIR ? 2 * TILE : TILE;   // tokens per tile
    constexpr int BPT = TT / BS;                 // blocks per tile
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g4 = lane >> 4;
    const int G = p.group, B = p.num_seqs;
    const int ncol = PAIR ? 2 * G : G;           // B-operand columns in use

    __shared__ __attribute__((aligned(16))) unsigned char lds[NWAVES * KTILE_BYTES];
    __shared__ int prefix[SK_MAX_SEQS + 1];     // prefix[s] = tiles of the sequences before s
    __shared__ int wave_tot[NWAVES];
    unsigned char* kt = lds + w * KTILE_BYTES;

    // ---- prologue: tiles per sequence -> exclusive prefix sums
    if (B <= 64) {
        // every wave scans for itself and reads back only what it wrote: no barrier (the
        // four waves write identical values to the same words)
        const int mine = lane < B ? sk_tiles<TT>(p.context_lens[lane], p.max_blocks) : 0;
        int inc = mine;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(inc, o);
            if (lane >= o) inc += v;
        }
        prefix[lane] = inc - mine;
        if (lane == 63) prefix[64] = inc;
        if (B < 64 && lane == B) prefix[B] = inc - mine;      // == total: lanes >= B add nothing
    } else {
        int loc[4], sum = 0;                                  // 4 sequences per thread
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int sidx = 4 * tid + k;
            loc[k] = sidx < B ? sk_tiles<TT>(p.context_lens[sidx], p.max_blocks) : 0;
            sum += loc[k];
        }
        int inc = sum;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(inc, o);
            if (lane >= o) inc += v;
        }
        if (lane == 63) wave_tot[w] = inc;
        __syncthreads();
        int base = inc - sum;
        for (int ww = 0; ww < w; ++ww) base += wave_tot[ww];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int sidx = 4 * tid + k;
            if (sidx <= B) prefix[sidx] = base;
            base += loc[k];
        }
        if (tid == 255 && B == SK_MAX_SEQS) prefix[SK_MAX_SEQS] = base;
        __syncthreads();
    }
    // Waves are dealt to KV heads first: wave i works on head i % Hkv, and the waves_per_head waves
    // of a head split that head's tiles of all sequences evenly.  The Hkv waves with the same
    // i / Hkv then walk the same tiles of the same sequences side by side, i.e. the Hkv adjacent
    // head slices of the same physical blocks at about the same time.
    const int64_t N = __builtin_amdgcn_readfirstlane(prefix[B]);       // tiles of one head
    const int wave_id = blockIdx.x * NWAVES + w;
    const int kvh_mine = wave_id % p.hkv, part = wave_id / p.hkv;
    const int W = (int)min((int64_t)p.waves_per_head, N);  // with fewer tiles than waves, one tile each
    if (part >= W) return;
    const int64_t g0 = (int64_t)part * N / W;
    const int64_t g1 = (int64_t)(part + 1) * N / W;

    // ---- first row of this wave: largest s with prefix[s] <= g0
    int seq;
    {
        const int x = (int)g0;
        int lo = 0, hi = B;            // invariant: prefix[lo] <= x < prefix[hi]
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (prefix[mid] <= x) lo = mid; else hi = mid;
        }
        seq = __builtin_amdgcn_readfirstlane(lo);
    }
    // everything that steers the loop is wave-uniform: keep it in scalar registers
    int row_tiles = __builtin_amdgcn_readfirstlane(prefix[seq + 1] - prefix[seq]);
    int kvh = __builtin_amdgcn_readfirstlane(kvh_mine);
    int t = __builtin_amdgcn_readfirstlane((int)(g0 - prefix[seq]));

    const KTileOffsets ko = k_tile_offsets(lane);

    // ---- segments.  A segment is the part of one (sequence, KV head) row that falls into this
    // wave's tile range.  The next segment's query rows and table slice are requested while the
    // current one streams, and its first K/V tile is prefetched by the current segment's last
    // tile, so the loads never drain at a row boundary.
    // raw query rows of (sequence, KV head); columns beyond the group are zeroed by q_operand
    // only when the rows are used, so that issuing the loads never waits for them
    auto load_q = [&](int sq, int kh, uint4 (&q)[4]) {
        if constexpr (PAIR) {
            // column c = (head c / 2, parity c % 2): k-slot s covers row elements 32s + 8 g4 .., which are
            // the query's elements (32s + 8 g4) % 64 when the slot lies in the column's own half of the row
            const uint16_t* qrow = (const uint16_t*)p.query + ((int64_t)sq * p.hq + kh * G + min(r16 >> 1, G - 1)) * DQ;
#pragma unroll
            for (int s = 0; s < 4; ++s) q[s] = *(const uint4*)(qrow + ((32 * s + 8 * g4) & 63));
        } else {
            const uint4* qp = (const uint4*)((const uint16_t*)p.query +
                                             ((int64_t)sq * p.hq + kh * G + min(r16, G - 1)) * D + 8 * g4);
#pragma unroll
            for (int s = 0; s < 4; ++s) q[s] = qp[s * 4];
        }
    };
    auto q_operand = [&](const uint4 (&raw)[4], uint4 (&q)[4]) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            bool use = r16 < ncol;
            if constexpr (PAIR) use = use && ((32 * s + 8 * g4 >= 64) == ((r16 & 1) != 0));
            q[s] = use ? raw[s] : make_uint4(0, 0, 0, 0);
        }
    };
    auto load_tab = [&](int sq, int first_block) {
        const int32_t* table = p.block_table + (int64_t)sq * p.block_table_stride;
        return (first_block + lane < p.max_blocks) ? table[first_block + lane] : 0;
    };

    int nt = (int)min((int64_t)(row_tiles - t), g1 - g0);          // tiles of the current segment (>= 1)
    uint4 qf[4];
    uint4 qraw[4];
    load_q(seq, kvh, qraw);
    int tab = load_tab(seq, BPT * t);
    TileRegs<FP8> kr, vr;
    // the blocks of a tile out of a table slice held one entry per lane
    auto slice_blocks = [&](int slice, int first, int64_t (&bb)[4]) {
#pragma unroll
        for (int j = 0; j < BPT; ++j) bb[j] = clamp_block(__builtin_amdgcn_readlane(slice, first + j), p.num_blocks);
    };
    auto load_kv = [&](const int64_t (&bb)[4], int kh) {
        if constexpr (PAIR) {
            load_tile_pair<FP8>(kr, p.k_pool, bb[0], bb[1], bb[2], bb[3], p.hkv, kh, lane);
            load_tile_pair<FP8>(vr, p.v_pool, bb[0], bb[1], bb[2], bb[3], p.hkv, kh, lane);
        } else {
            load_tile<FP8>(kr, p.k_pool, bb[0], bb[1], p.hkv, kh, lane);
            load_tile<FP8>(vr, p.v_pool, bb[0], bb[1], p.hkv, kh, lane);
        }
    };
    {
        __builtin_amdgcn_s_waitcnt(0x0F70);                        // Q and table have landed
        q_operand(qraw, qf);
        int64_t bb[4] = {0, 0, 0, 0};
        slice_blocks(tab, 0, bb);
        load_kv(bb, kvh);
    }

    for (int64_t g = g0; g < g1 && seq < B;) {
        const int len = min(p.context_lens[seq], p.max_blocks * BS);
        const int blk_base = BPT * t;
        const int32_t* table = p.block_table + (int64_t)seq * p.block_table_stride;
        int tab_first = 0;
        const float cmul = p.qk_mul * (FP8 ? p.k_scale[kvh] : 1.f);
        auto tile_blocks = [&](int k, int64_t (&bb)[4]) {              // k-th tile of the segment
            const int i0 = BPT * k;
            if (i0 - tab_first >= 64) {
                tab_first = i0;
                tab = (blk_base + i0 + lane < p.max_blocks) ? table[blk_base + i0 + lane] : 0;
                __builtin_amdgcn_s_waitcnt(0x0F70);
            }
            slice_blocks(tab, i0 - tab_first, bb);
        };

        // the segment after this one (same wave, same KV head): the next sequence with tokens
        int nseq = seq, nkvh = kvh, nrow_tiles = row_tiles;
        const bool more = g + nt < g1;
        if (more) {
            do { ++nseq; } while (nseq < B && __builtin_amdgcn_readfirstlane(prefix[nseq + 1] - prefix[nseq]) == 0);
            nrow_tiles = nseq < B ? __builtin_amdgcn_readfirstlane(prefix[nseq + 1] - prefix[nseq]) : 0;
        }
        const bool has_next = more && nseq < B;
        int tabn = 0;
        uint4 qn[4];
        if (has_next) {
            load_q(nseq, nkvh, qraw);
            tabn = load_tab(nseq, 0);
        }

        WaveState st;
        st.m = NEG_BIG; st.lsum = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) st.O[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

        int64_t bb[4] = {0, 0, 0, 0};
        int k = 0;
        for (; k + 1 < nt; ++k) {
            tile_blocks(k + 1, bb);
            process_tile<E, FP8, true, false, PAIR>(st, kr, vr, qf, kt, ko, p.k_pool, p.v_pool, bb[0], bb[1],
                                                    p.hkv, kvh, lane, g4, (t + k) * TT, len, cmul, bb[2], bb[3]);
        }
        const int tile_start = (t + k) * TT;
        if (p.new_key != nullptr && t + k == row_tiles - 1) {       // the row's newest token lives here
            tile_blocks(k, bb);
            // Same rule as the separate one-token append: the row is stored only where the table names a
            // block of the pool and the length fits the table; otherwise the call leaves the pools alone
            // (and attends over what the clamped table entry holds, like the unfused sequence of calls).
            const int raw_blk = __builtin_amdgcn_readlane(tab, BPT * k + ((len - 1 - tile_start) >> 4) - tab_first);
            if (p.context_lens[seq] == len && raw_blk >= 0 && raw_blk < p.num_blocks) {
                if constexpr (PAIR) inject_new_row_grid<E, FP8, true>(kr, vr, p, seq, kvh, lane, tile_start, len, bb);
                else inject_new_row<E, FP8>(kr, vr, p, seq, kvh, lane, tile_start, len, bb[0], bb[1]);
            }
        }
        // The segment's last tile always runs the masked body (a full tile simply masks nothing):
        // one prefetching call site, so the prefetched registers need no merging afterwards.
        int tab_ready = 0;
        if (has_next) {
            // prefetch the first tile of the next segment
            __builtin_amdgcn_s_waitcnt(0x0F70);      // next Q rows and table slice (and this tile) have landed
            q_operand(qraw, qn);
            tab_ready = tabn;
            slice_blocks(tab_ready, 0, bb);
            process_tile<E, FP8, true, true, PAIR>(st, kr, vr, qf, kt, ko, p.k_pool, p.v_pool, bb[0], bb[1],
                                                   p.hkv, nkvh, lane, g4, tile_start, len, cmul, bb[2], bb[3]);
        } else {
            process_tile<E, FP8, false, true, PAIR>(st, kr, vr, qf, kt, ko, p.k_pool, p.v_pool, 0, 0,
                                                    p.hkv, kvh, lane, g4, tile_start, len, cmul);
        }

        // ---- flush: lane (head r16, g4) holds O^T[dim 32*g4 + 8*i + j][head] in O[j][i]
        float lsum = st.lsum;
        lsum += __shfl_xor(lsum, 16);
        lsum += __shfl_xor(lsum, 32);
        const int64_t slot = (int64_t)kvh * (p.waves_per_head + B) + part + seq;
        if constexpr (PAIR) {
            // Column (head, parity) holds its own token's half of the pair rows: parity 0 elements 0..63 of
            // its accumulator (lanes g4 = 0, 1), parity 1 elements 64..127 (lanes g4 = 2, 3).  The two are
            // partial softmaxes over the even and the odd tokens of the same segment: merged here, inside the
            // wave, so that a flush writes ONE partial of 64 floats per head.  Lane (column 2h, g4 = a) takes
            // the matching values of lane (column 2h + 1, g4 = a + 2), 33 lanes up.
            const float m1 = __shfl_xor(st.m, 1), l1 = __shfl_xor(lsum, 1);
            const float mm = fmaxf(st.m, m1);
            const float f0 = exp2f(st.m - mm), f1 = exp2f(m1 - mm);
            float mine[8][4];
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) mine[j][i] = fmaf(f1, __shfl(st.O[j][i], lane + 33), f0 * st.O[j][i]);
            if (r16 < ncol && (r16 & 1) == 0 && g4 < 2) {
                float* dst = p.ws_acc + (slot * G + (r16 >> 1)) * DQ + 32 * g4;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    *(float4*)(dst + 8 * i) = make_float4(mine[0][i], mine[1][i], mine[2][i], mine[3][i]);
                    *(float4*)(dst + 8 * i + 4) = make_float4(mine[4][i], mine[5][i], mine[6][i], mine[7][i]);
                }
                if (g4 == 0) *(float2*)(p.ws_ml + (slot * G + (r16 >> 1)) * 2) = make_float2(mm, f0 * lsum + f1 * l1);
            }
        } else if (r16 < ncol) {
            float* dst = p.ws_acc + (slot * G + r16) * DQ + 32 * g4;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                *(float4*)(dst + 8 * i) = make_float4(st.O[0][i], st.O[1][i], st.O[2][i], st.O[3][i]);
                *(float4*)(dst + 8 * i + 4) = make_float4(st.O[4][i], st.O[5][i], st.O[6][i], st.O[7][i]);
            }
            if (g4 == 0) *(float2*)(p.ws_ml + (slot * G + r16) * 2) = make_float2(st.m, lsum);
        }
        // the waves holding a row's first and last tile tell the merge kernel where its partials are
        if (lane == 0) {
            int* rm = p.ws_rows + 2 * ((int64_t)seq * p.hkv + kvh);
            if (t == 0) rm[0] = part;
            if (t + nt == row_tiles) rm[1] = part;
        }

        // ---- next segment
        g += nt;
        if (!has_next) break;
        seq = nseq; kvh = nkvh; row_tiles = nrow_tiles; t = 0;
        nt = (int)min((int64_t)row_tiles, g1 - g);
        tab = tab_ready;
#pragma unroll
        for (int s = 0; s < 4; ++s) qf[s] = qn[s];
    }
}

// Merge of the balanced schedule's partials: one workgroup per (KV head, sequence), S waves per
// head of the group.  The row's partials sit in consecutive slots of its head's region,
// head_slots * head + first + sequence .. + last + sequence (first / last part recorded by the
// main kernel); their weights 2^(m_i - M) are computed once (one lane
// per partial) and parked in LDS, then each lane accumulates its output dims (two at head_dim
// 128, one at head_dim 64) with independent loads.  With S = 1 (few partials per row, the usual
// batch) reductions are shuffles and there is no barrier; with S > 1 (a handful of very long rows,
// hundreds of partials each) the waves of a head take alternate groups of eight partials and add
// up through LDS.
constexpr int RED_WGT = 256;       // weights parked in LDS per wave; rows with more partials recompute the rest
template <typename E, int DQ>
__global__ void __launch_bounds__(1024)
streamk_reduce_kernel(uint16_t* __restrict__ out, const float* __restrict__ ws_acc,
                      const float* __restrict__ ws_ml, const int* __restrict__ ws_rows,
                      const int32_t* __restrict__ context_lens, int hq, int hkv, int group,
                      const float* __restrict__ v_scale, int head_slots) {
    constexpr int NV = DQ / 64;                            // output dims per lane
    const int kvh = blockIdx.x, seq = blockIdx.y, wv = threadIdx.x >> 6;
    const int S = (int)(blockDim.x >> 6) / group;          // waves per head
    const int h = wv / S, sub = wv % S;
    const int lane = threadIdx.x & 63;
    __shared__ float wgt_all[16][RED_WGT];
    __shared__ float part[16][DQ];
    float* wgt = wgt_all[wv];
    const int64_t row = (int64_t)seq * hkv + kvh;
    uint16_t* o = out + ((int64_t)seq * hq + kvh * group + h) * DQ;
    // the length and the row's record are requested together (the record of an empty row was never
    // written and is not used)
    const int ctx = context_lens[seq];
    const int first = ws_rows[2 * row], last = ws_rows[2 * row + 1];
    if (ctx <= 0) {                          // no tiles, no partials: the output row is zero (whole workgroup)
        if (sub == 0) {
#pragma unroll
            for (int e = 0; e < NV; ++e) o[lane + 64 * e] = 0;
        }
        return;
    }
    const int np = last - first + 1;
    const int64_t slot0 = (int64_t)kvh * head_slots + first + seq;       // the row's partials: slots slot0 .. slot0 + np - 1
    const float* ml = ws_ml + (slot0 * group + h) * 2;                  // partial i at ml[i * group * 2]
    const float* acc = ws_acc + (slot0 * group + h) * DQ + lane;        // partial i at acc[i * group * DQ]
    const int64_t stride = (int64_t)group * DQ;
    if (S == 1 && np <= 8) {
        // The usual batch: a handful of partials per row.  Their (max, sum) pairs and this lane's
        // output dims of each are requested in one go, so the kernel is two memory latencies
        // deep (record, then partials) instead of four.
        float2 mlv[8];
        float a[8][NV];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = min(u, np - 1);
            mlv[u] = *(const float2*)(ml + (int64_t)i * group * 2);
#pragma unroll
            for (int e = 0; e < NV; ++e) a[u][e] = acc[i * stride + 64 * e];
        }
        float mx = NEG_BIG;
#pragma unroll
        for (int u = 0; u < 8; ++u) mx = fmaxf(mx, mlv[u].x);           // repeats of the last partial change nothing
        float den = 0.f, num[NV] = {};
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float f = u < np ? exp2f(mlv[u].x - mx) : 0.f;
            den = fmaf(f, mlv[u].y, den);
#pragma unroll
            for (int e = 0; e < NV; ++e) num[e] = fmaf(f, a[u][e], num[e]);
        }
        const float inv = den > 0.f ? (v_scale ? v_scale[kvh] : 1.f) / den : 0.f;
#pragma unroll
        for (int e = 0; e < NV; ++e) o[lane + 64 * e] = E::from_f32(num[e] * inv);
        return;
    }
    // every wave of a head computes the row's max, denominator and weights for itself (np / 64 loads per lane)
    float mx = NEG_BIG;
    for (int i = lane; i < np; i += 64) mx = fmaxf(mx, ml[(int64_t)i * group * 2]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    float den = 0.f;
    for (int i = lane; i < np; i += 64) {
        const float2 v = *(const float2*)(ml + (int64_t)i * group * 2);
        const float f = exp2f(v.x - mx);
        if (i < RED_WGT) wgt[i] = f;
        den = fmaf(f, v.y, den);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) den += __shfl_xor(den, off);
    // eight partials in flight per step: the loop is pure load latency
    float num[NV] = {};
    for (int i0 = 8 * sub; i0 < np; i0 += 8 * S) {
        float a[8][NV];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = min(i0 + u, np - 1);
#pragma unroll
            for (int e = 0; e < NV; ++e) a[u][e] = acc[i * stride + 64 * e];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i0 + u;
            const float f = i >= np ? 0.f : (i < RED_WGT ? wgt[i] : exp2f(ml[(int64_t)i * group * 2] - mx));
#pragma unroll
            for (int e = 0; e < NV; ++e) num[e] = fmaf(f, a[u][e], num[e]);
        }
    }
    if (S > 1) {                             // workgroup-uniform
#pragma unroll
        for (int e = 0; e < NV; ++e) part[wv][lane + 64 * e] = num[e];
        __syncthreads();
        if (sub != 0) return;
        for (int k = 1; k < S; ++k)
#pragma unroll
            for (int e = 0; e < NV; ++e) num[e] += part[wv + k][lane + 64 * e];
    }
    const float inv = den > 0.f ? (v_scale ? v_scale[kvh] : 1.f) / den : 0.f;
#pragma unroll
    for (int e = 0; e < NV; ++e) o[lane + 64 * e] = E::from_f32(num[e] * inv);
}

}  // namespace

// head_dim 128, or head_dim 64 handled as rows of token pairs (two B-operand columns per head,
// hence groups up to 8 and partitions of whole 64-token tiles)
bool decode_mfma_supported(const DecodeArgs& a) {
    const int group = a.hkv > 0 ? a.hq / a.hkv : 0;
    const bool shape = (a.d == D && group <= 16 && a.partition_size % TILE == 0) ||
                       (a.d == 64 && group <= 8 && a.partition_size % (2 * TILE) == 0);
    return a.cu_q_lens == nullptr && shape && a.bs == BS && is_16bit_float(a.q_dtype) &&
           (a.kv_dtype == a.q_dtype || a.kv_dtype == AICOMP_KV_FP8_E4M3) && group >= 1 &&
           a.scale > 0.f && a.rows <= 65535 &&
           a.num_parts <= 65535 && ((uintptr_t)a.query % 16 == 0) && ((uintptr_t)a.k_pool % 16 == 0) &&
           ((uintptr_t)a.v_pool % 16 == 0);
}

bool decode_streamk_supported(const DecodeArgs& a) {
    // every KV head needs at least one wave of the 4 x CUs the schedule launches
    return decode_mfma_supported(a) && a.rows <= SK_MAX_SEQS && a.hkv <= 256;
}

// per slot one partial per head: G x (head_dim + 2) floats
size_t decode_streamk_workspace_bytes(int64_t rows, int hq, int hkv, int d) {
    const int64_t slots = SK_MAX_WAVES + rows * hkv;
    const int ncol = hq / hkv;
    return (size_t)slots * ncol * (size_t)(d + 2) * sizeof(float) + (size_t)rows * hkv * 2 * sizeof(int);
}

int launch_decode_streamk(const DecodeArgs& a, void* workspace) {
    // CU count of the first device used (every GPU of a node is the same part); an atomic so that
    // callers on several threads may race here harmlessly
    static std::atomic<int> cached_cus{0};
    int num_cus = cached_cus.load(std::memory_order_relaxed);
    if (num_cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            set_error("paged_decode_attn: cannot query the CU count");
            return AICOMP_KV_EHIP;
        }
        num_cus = n;
        cached_cus.store(n, std::memory_order_relaxed);
    }
    // one workgroup per CU measured fastest (4 waves of 16 KB in flight each already cover the
    // HBM latency; a second workgroup per CU only adds partials and start-up work)
    const int wgs = min(num_cus, SK_MAX_WAVES / NWAVES);
    const int group = a.hq / a.hkv;
    const int64_t slots = SK_MAX_WAVES + a.rows * a.hkv;
    StreamKParams p;
    p.out = a.out; p.query = a.query; p.k_pool = (void*)a.k_pool; p.v_pool = (void*)a.v_pool;
    p.block_table = a.block_table; p.block_table_stride = a.block_table_stride;
    p.context_lens = a.context_lens;
    p.num_seqs = (int)a.rows; p.hq = a.hq; p.hkv = a.hkv; p.group = group; p.max_blocks = a.max_blocks;
    p.num_blocks = a.num_blocks;
    p.qk_mul = a.scale * LOG2E;
    p.k_scale = a.k_scale; p.v_scale = a.v_scale;
    p.num_waves = wgs * NWAVES;
    p.waves_per_head = p.num_waves / a.hkv;
    const bool pair = a.d == 64;
    const int ncol = group;
    p.ws_acc = (float*)workspace;
    p.ws_ml = p.ws_acc + slots * ncol * a.d;
    p.ws_rows = (int*)(p.ws_ml + slots * ncol * 2);
    p.new_key = (const uint16_t*)a.new_key; p.new_value = (const uint16_t*)a.new_value;
    p.new_token_stride = a.new_token_stride; p.new_head_stride = a.new_head_stride;
    const bool fp8 = a.kv_dtype == AICOMP_KV_FP8_E4M3, f16 = a.q_dtype == AICOMP_KV_F16;
#define AICOMP_LAUNCH_SK(E, PAIR)                                                                                  \
    do {                                                                                                           \
        if (fp8) hipLaunchKernelGGL((streamk_decode_kernel<E, true, PAIR>), dim3(wgs), dim3(256), 0, a.stream, p);  \
        else hipLaunchKernelGGL((streamk_decode_kernel<E, false, PAIR>), dim3(wgs), dim3(256), 0, a.stream, p);    \
    } while (0)
    if (pair) { if (f16) AICOMP_LAUNCH_SK(F16Fmt, true); else AICOMP_LAUNCH_SK(Bf16Fmt, true); }
    else { if (f16) AICOMP_LAUNCH_SK(F16Fmt, false); else AICOMP_LAUNCH_SK(Bf16Fmt, false); }
#undef AICOMP_LAUNCH_SK
    AICOMP_HIP_LAUNCH_CHECK();
    // waves per head in the merge: one, unless rows are few and long (many partials per row)
    const int64_t per_row = (int64_t)p.waves_per_head / a.rows + 2;
    const int sub = per_row > 8 ? 16 / group : 1;
#define AICOMP_LAUNCH_RED(E, DQ)                                                                                  \
    hipLaunchKernelGGL((streamk_reduce_kernel<E, DQ>), dim3(a.hkv, (unsigned)a.rows), dim3(64 * group * sub), 0,  \
                       a.stream, (uint16_t*)a.out, p.ws_acc, p.ws_ml, p.ws_rows, a.context_lens, a.hq, a.hkv,     \
                       group, a.v_scale, p.waves_per_head + (int)a.rows)
    if (pair) { if (f16) AICOMP_LAUNCH_RED(F16Fmt, 64); else AICOMP_LAUNCH_RED(Bf16Fmt, 64); }
    else { if (f16) AICOMP_LAUNCH_RED(F16Fmt, 128); else AICOMP_LAUNCH_RED(Bf16Fmt, 128); }
#undef AICOMP_LAUNCH_RED
    AICOMP_HIP_LAUNCH_CHECK();
    return AICOMP_KV_OK;
}

int launch_decode_mfma(const DecodeArgs& a) {
    MfmaParams p;
    p.out = a.out; p.query = a.query; p.k_pool = (void*)a.k_pool; p.v_pool = (void*)a.v_pool;
    p.block_table = a.block_table; p.block_table_stride = a.block_table_stride;
    p.context_lens = a.context_lens;
    p.hq = a.hq; p.hkv = a.hkv; p.group = a.hq / a.hkv; p.max_blocks = a.max_blocks;
    p.num_blocks = a.num_blocks;
    p.qk_mul = a.scale * LOG2E;
    p.k_scale = a.k_scale; p.v_scale = a.v_scale;
    p.partition_size = a.partition_size; p.num_parts = a.num_parts;
    p.ws_acc = a.ws.acc; p.ws_ml = a.ws.ml;
    p.new_key = (const uint16_t*)a.new_key; p.new_value = (const uint16_t*)a.new_value;
    p.new_token_stride = a.new_token_stride; p.new_head_stride = a.new_head_stride;
    dim3 grid((unsigned)a.hkv, (unsigned)a.num_parts, (unsigned)a.rows);
    const bool fp8 = a.kv_dtype == AICOMP_KV_FP8_E4M3;
#define AICOMP_LAUNCH_GRID(E)                                                                                       \
    do {                                                                                                            \
        if (a.d == 64) {                                                                                            \
            if (fp8) hipLaunchKernelGGL((paged_decode_mfma_kernel<E, true, true>), grid, dim3(256), 0, a.stream, p); \
            else hipLaunchKernelGGL((paged_decode_mfma_kernel<E, false, true>), grid, dim3(256), 0, a.stream, p);   \
        } else {                                                                                                    \
            if (fp8) hipLaunchKernelGGL((paged_decode_mfma_kernel<E, true, false>), grid, dim3(256), 0, a.stream, p); \
            else hipLaunchKernelGGL((paged_decode_mfma_kernel<E, false, false>), grid, dim3(256), 0, a.stream, p);  \
        }                                                                                                           \
    } while (0)
    if (a.q_dtype == AICOMP_KV_F16) AICOMP_LAUNCH_GRID(F16Fmt);
    else AICOMP_LAUNCH_GRID(Bf16Fmt);
#undef AICOMP_LAUNCH_GRID
    AICOMP_HIP_LAUNCH_CHECK();
    if (a.num_parts > 1) return launch_split_reduce(a);
    return AICOMP_KV_OK;
}

}  // namespace aicomp
