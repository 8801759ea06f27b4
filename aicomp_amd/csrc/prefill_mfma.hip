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
// Work split   one workgroup (4 waves) per (64 query rows, sequence).  A "row" is
//              a (position, query head) pair: with `gpack` = G heads of one KV
//              head packed per position, the 64 rows are 64/G consecutive
//              positions x G heads, so every K/V tile staged in LDS serves the
//              whole GQA group.  Groups that do not divide 16 use gpack = 1.
// K/V tiles    64 tokens (4 blocks) per step, fetched by the whole workgroup with
//              coalesced 16-byte loads into registers one tile ahead, written to
//              a double-buffered LDS tile (row stride 272 B): one barrier per tile.
// Per wave     16 rows.  S^T = K Q^T with K rows as the A operand and the wave's
//              16 query rows as B columns (v_mfma_f32_16x16x32_bf16); online
//              softmax per column, lane-local except the row max (two wave
//              shuffles); O^T += V^T P^T with V read from LDS as 16-byte row chunks
//              and the j-th halves picked with v_perm_b32, the same register
//              layout as the decode kernel, so P never leaves its lane.
#include "common.h"

namespace aicomp {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int D = 128;
constexpr int BS = 16;
constexpr int KT = 64;                 // tokens per LDS tile
constexpr int ROWS = 64;               // query rows per workgroup (16 per wave)
constexpr int KROW = 272;              // LDS row stride in bytes (256 + 16 pad)
constexpr int TILE_BYTES = KT * KROW;  // 17408
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
    int64_t num_blocks;
    float qk_mul;
    const float* k_scale;
    const float* v_scale;
};

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    bf16x2_t p = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, p);
}

__device__ __forceinline__ uint4 fp8x8_to_bf16x8(uint2 r) {
    // gfx950 converts two e4m3 codes straight to two packed bf16 (exact: 3 mantissa bits);
    // the scale operand is 1.0
    uint4 o;
    o.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(r.x, 1.0f, false));
    o.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(r.x, 1.0f, true));
    o.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(r.y, 1.0f, false));
    o.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(r.y, 1.0f, true));
    return o;
}

template <bool FP8> struct Stage;
template <> struct Stage<false> { uint4 k[4], v[4]; };
template <> struct Stage<true> { uint2 k[4], v[4]; };

template <bool FP8>
__global__ void __launch_bounds__(256, 2)
paged_prefill_mfma_kernel(PrefillParams p) {
    const int seq = blockIdx.z;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g4 = lane >> 4;

    const int q_begin = p.cu_q_lens[seq];
    const int n = p.cu_q_lens[seq + 1] - q_begin;
    const int ctx = min(p.context_lens[seq], p.max_blocks * BS);
    const int prior = ctx - n;
    const int pos_per_wg = ROWS / p.gpack;
    const int q0 = blockIdx.x * pos_per_wg;
    if (q0 >= n || n <= 0 || prior < 0) return;

    // rows of this lane's column: row = 16w + r16 -> (position, head)
    const int row = 16 * w + r16;
    const int qpos = q0 + row / p.gpack;
    const int head = blockIdx.y * p.gpack + row % p.gpack;
    const int kvh = (blockIdx.y * p.gpack) / p.group;          // workgroup-uniform
    const bool row_valid = qpos < n;
    const int qabs = row_valid ? prior + qpos : ctx - 1;        // padded rows: computed, never stored
    // last key any row of this wave / workgroup may see (exclusive)
    const int wave_kv_end = min(ctx, prior + q0 + (16 * w + 15) / p.gpack + 1);
    const int wave_kv_min = prior + q0 + (16 * w) / p.gpack;    // smallest qabs in the wave (if valid)
    const int kv_end = min(ctx, prior + q0 + pos_per_wg);
    const int ntiles = (kv_end + KT - 1) / KT;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // [2][K tile | V tile]

    // Q as the B operand: column = this lane's row, k-slots = dims 32s + 8*g4 ..
    bf16x8_t qf[4];
    {
        const uint4* qp = (const uint4*)((const bf16_t*)p.query +
                                         ((int64_t)(q_begin + min(qpos, n - 1)) * p.hq + head) * D + 8 * g4);
#pragma unroll
        for (int s = 0; s < 4; ++s) qf[s] = __builtin_bit_cast(bf16x8_t, qp[s * 4]);
    }
    const float cmul = p.qk_mul * (FP8 ? p.k_scale[kvh] : 1.f);

    float m = NEG_BIG, lsum = 0.f;
    f32x4_t O[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) O[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;
    const_i32_ptr table = (const_i32_ptr)(p.block_table + (int64_t)seq * p.block_table_stride);

    // global -> registers: load i of the tile is block 4t + i (16 tokens x 16 chunks = 256 lanes)
    Stage<FP8> st;
    auto fetch = [&](int t) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int bi = 4 * t + i;
            int b = bi < p.max_blocks ? table[bi] : 0;
            const int64_t blk = b < 0 ? 0 : (b >= p.num_blocks ? p.num_blocks - 1 : (int64_t)b);
            const int64_t off = (blk * p.hkv + kvh) * (BS * D / 8) + tid;
            if constexpr (FP8) {
                st.k[i] = ((const uint2*)p.k_pool)[off];
                st.v[i] = ((const uint2*)p.v_pool)[off];
            } else {
                st.k[i] = ((const uint4*)p.k_pool)[off];
                st.v[i] = ((const uint4*)p.v_pool)[off];
            }
        }
    };
    // registers -> LDS buffer `buf`; V rows at or beyond the context are zeroed (a masked
    // probability of 0 times a non-finite leftover would still poison the row)
    auto stash = [&](int t, int buf) {
        unsigned char* kb = lds + buf * 2 * TILE_BYTES;
        unsigned char* vb = kb + TILE_BYTES;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int tok_local = 16 * i + (tid >> 4);
            const int off = tok_local * KROW + (tid & 15) * 16;
            uint4 kk, vv;
            if constexpr (FP8) { kk = fp8x8_to_bf16x8(st.k[i]); vv = fp8x8_to_bf16x8(st.v[i]); }
            else { kk = st.k[i]; vv = st.v[i]; }
            if (t * KT + tok_local >= ctx) vv = make_uint4(0, 0, 0, 0);
            *(uint4*)(kb + off) = kk;
            *(uint4*)(vb + off) = vv;
        }
    };

    const int rd_k = (4 * (r16 & 3) + (r16 >> 2)) * KROW + g4 * 16;   // permuted K row, chunk g4
    const int rd_v = g4 * KROW + r16 * 16;                            // V row 4i + g4, chunk r16

    fetch(0);
    for (int t = 0; t < ntiles; ++t) {
        const int buf = t & 1;
        stash(t, buf);
        if (t + 1 < ntiles) fetch(t + 1);
        __syncthreads();          // tile t visible; everyone is done with the buffer tile t+1 will use

        const unsigned char* kb = lds + buf * 2 * TILE_BYTES;
        const unsigned char* vb = kb + TILE_BYTES;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            const int sub_start = t * KT + sub * 32;
            if (sub_start >= wave_kv_end) continue;                    // wave-uniform: above the diagonal
            f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const uint4 a0 = *(const uint4*)(kb + sub * 32 * KROW + rd_k + s * 64);
                const uint4 a1 = *(const uint4*)(kb + (sub * 32 + 16) * KROW + rd_k + s * 64);
                s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a0), qf[s], s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a1), qf[s], s1, 0, 0, 0);
            }
            float sc[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) { sc[i] = s0[i] * cmul; sc[4 + i] = s1[i] * cmul; }
            const bool need_mask = sub_start + 31 > wave_kv_min;       // wave-uniform
            if (need_mask) {
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int tok = sub_start + 16 * (k >> 2) + 4 * (k & 3) + g4;
                    if (tok > qabs) sc[k] = NEG_BIG;
                }
            }
            float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])),
                             fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
            mx = fmaxf(mx, __shfl_xor(mx, 16));
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m, mx);
            const float alpha = exp2f(m - m_new);
            float pr[8], psum = 0.f;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                pr[k] = exp2f(sc[k] - m_new);
                if (need_mask && sc[k] == NEG_BIG) pr[k] = 0.f;
                psum += pr[k];
            }
            lsum = lsum * alpha + psum;
            m = m_new;
            if (__any(alpha != 1.f)) {
#pragma unroll
                for (int j = 0; j < 8; ++j) O[j] *= alpha;
            }
            uint4 pw;
            pw.x = pack_bf16(pr[0], pr[1]); pw.y = pack_bf16(pr[2], pr[3]);
            pw.z = pack_bf16(pr[4], pr[5]); pw.w = pack_bf16(pr[6], pr[7]);
            const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, pw);

            uint4 vv[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                vv[i] = *(const uint4*)(vb + (sub * 32 + 4 * i) * KROW + rd_v);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
                const uint32_t* v0 = (const uint32_t*)&vv[0];
                uint4 a;
                a.x = __builtin_amdgcn_perm(v0[4 * 1 + (j >> 1)], v0[4 * 0 + (j >> 1)], sel);
                a.y = __builtin_amdgcn_perm(v0[4 * 3 + (j >> 1)], v0[4 * 2 + (j >> 1)], sel);
                a.z = __builtin_amdgcn_perm(v0[4 * 5 + (j >> 1)], v0[4 * 4 + (j >> 1)], sel);
                a.w = __builtin_amdgcn_perm(v0[4 * 7 + (j >> 1)], v0[4 * 6 + (j >> 1)], sel);
                O[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), pf, O[j], 0, 0, 0);
            }
        }
    }

    // lane (row r16 of the wave, g4) holds O^T[dim 32*g4 + 8*i + j][row] in O[j][i]
    lsum += __shfl_xor(lsum, 16);
    lsum += __shfl_xor(lsum, 32);
    if (row_valid) {
        const float inv = (lsum > 0.f ? 1.f / lsum : 0.f) * (FP8 ? p.v_scale[kvh] : 1.f);
        bf16_t* o = (bf16_t*)p.out + ((int64_t)(q_begin + qpos) * p.hq + head) * D + 32 * g4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint4 pk;
            pk.x = pack_bf16(O[0][i] * inv, O[1][i] * inv);
            pk.y = pack_bf16(O[2][i] * inv, O[3][i] * inv);
            pk.z = pack_bf16(O[4][i] * inv, O[5][i] * inv);
            pk.w = pack_bf16(O[6][i] * inv, O[7][i] * inv);
            *(uint4*)(o + 8 * i) = pk;
        }
    }
}

}  // namespace

bool prefill_mfma_supported(const DecodeArgs& a, int max_q_len) {
    const int group = a.hkv > 0 ? a.hq / a.hkv : 0;
    return a.cu_q_lens != nullptr && max_q_len > 0 && a.d == D && a.bs == BS &&
           a.q_dtype == AICOMP_KV_BF16 &&
           (a.kv_dtype == AICOMP_KV_BF16 || a.kv_dtype == AICOMP_KV_FP8_E4M3) && group >= 1 &&
           a.scale > 0.f && a.num_seqs <= 65535 && ((uintptr_t)a.query % 16 == 0) &&
           ((uintptr_t)a.out % 16 == 0) && ((uintptr_t)a.k_pool % 16 == 0) &&
           ((uintptr_t)a.v_pool % 16 == 0);
}

int launch_prefill_mfma(const DecodeArgs& a, int max_q_len) {
    PrefillParams p;
    p.out = a.out; p.query = a.query; p.k_pool = a.k_pool; p.v_pool = a.v_pool;
    p.block_table = a.block_table; p.block_table_stride = a.block_table_stride;
    p.context_lens = a.context_lens; p.cu_q_lens = a.cu_q_lens;
    p.hq = a.hq; p.hkv = a.hkv; p.group = a.hq / a.hkv; p.max_blocks = a.max_blocks;
    p.num_blocks = a.num_blocks;
    p.gpack = (16 % p.group == 0) ? p.group : 1;      // heads of one KV head packed per position
    p.qk_mul = a.scale * LOG2E;
    p.k_scale = a.k_scale; p.v_scale = a.v_scale;
    const int pos_per_wg = ROWS / p.gpack;
    const int qtiles = (max_q_len + pos_per_wg - 1) / pos_per_wg;
    AICOMP_REQUIRE(qtiles <= 65535 * 32768 && a.hq / p.gpack <= 65535, AICOMP_KV_EINVAL,
                   "paged_prefill_attn: grid too large");
    dim3 grid((unsigned)qtiles, (unsigned)(a.hq / p.gpack), (unsigned)a.num_seqs);
    const size_t lds_bytes = 4 * TILE_BYTES;   // double-buffered K and V tiles
    if (a.kv_dtype == AICOMP_KV_FP8_E4M3) {
        static bool once_fp8 = false;
        if (!once_fp8) {
            hipFuncSetAttribute((const void*)paged_prefill_mfma_kernel<true>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
            once_fp8 = true;
        }
        hipLaunchKernelGGL(paged_prefill_mfma_kernel<true>, grid, dim3(256), lds_bytes, a.stream, p);
    } else {
        static bool once = false;
        if (!once) {
            hipFuncSetAttribute((const void*)paged_prefill_mfma_kernel<false>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
            once = true;
        }
        hipLaunchKernelGGL(paged_prefill_mfma_kernel<false>, grid, dim3(256), lds_bytes, a.stream, p);
    }
    AICOMP_HIP_LAUNCH_CHECK();
    return AICOMP_KV_OK;
}

}  // namespace aicomp
