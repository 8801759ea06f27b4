// Chunked-prefill causal attention for float32 models on gfx950's float32 matrix instruction.
//
// Replaces  F.scaled_dot_product_attention(query, full_key, full_value, attn_mask=None,
//           is_causal=True)                       opt_prime/opt_prime/kv_cache.py:404-415
// when the engine runs in float32 (examples/single_gpu_inference_llama.py:98-110, --dtype
// float32): queries, pools and output are float32, and every product and sum stays float32
// (v_mfma_f32_16x16x4_f32: D[16x16] += A[16x4] B[4x16], 2048 flop in 32 cycles per SIMD, the
// same 157 TFLOP/s roof as the vector ALUs but with a sixteenth of the instructions, so the
// softmax and the operand traffic hide under it).  Same mask rule as the 16-bit kernel: query i
// of a chunk with prior context P sees keys j <= P + i.
//
// Work split   one workgroup (4 waves) per (128 query rows, sequence); a row is a (position,
//              head) pair, the G heads of one KV head packed per position when G divides 16, so a
//              K/V tile staged in LDS serves the whole group.  A wave owns two 16-row column groups.
// K/V tiles    32 tokens, global -> registers (one tile ahead) -> LDS rows of head_dim floats + 16
//              bytes (the operand reads below are then free of bank conflicts), double-buffered,
//              one barrier per tile.
// S^T = K Q^T  A = K rows from LDS, B = the wave's query rows (registers, pre-multiplied by
//              scale * log2 e).  The k index of MFMA m in lane group g is 16 (m / 4) + 4 g + m % 4:
//              one 16-byte LDS read supplies the A operands of four MFMAs, for both column groups.
// softmax      online, base 2, per lane one query; the row max crosses the four lanes of a row
//              with two shuffles; the accumulators are rescaled only when a max moved.
// O^T += V^T P^T  A = V^T: lane (dim r, g) reads V[token 4 g + m][16 j + r], one 4-byte LDS read per
//              MFMA and column-group pair; B = P^T is exactly what the lane already holds.
#include "common.h"

#include <atomic>

namespace aicomp {

namespace {

constexpr int BS = 16;
constexpr int KT = 32;                  // tokens per LDS tile
constexpr int R = 2;                    // 16-row column groups per wave
constexpr int WG_ROWS = 4 * 16 * R;     // query rows per workgroup
constexpr float NEG_BIG = -1.0e30f;

struct PrefillF32Params {
    float* out;
    const float* query;
    const float* k_pool;
    const float* v_pool;
    const int32_t* block_table;
    int64_t block_table_stride;
    const int32_t* context_lens;
    const int32_t* cu_q_lens;
    int hq, hkv, group, gpack, max_blocks;
    int num_blocks;
    int num_cus;                        // CUs of the device (0: expensive tiles first)
    float qk_mul;
    const int32_t* items;               // (sequence, query tile) pairs; grid.y numbers them (NULL: none)
    int num_seqs;
};

template <int DH>
__global__ void __launch_bounds__(256, 2)
paged_prefill_mfma_f32_kernel(PrefillF32Params p) {
    constexpr int KROW = DH * 4 + 16;           // LDS row stride in bytes
    constexpr int KROWF = KROW / 4;             // ... in floats
    constexpr int TILE_F = KT * KROWF;          // floats per K (or V) tile
    constexpr int NQ = DH / 16;                 // 16-element chunks of a row (QK: 4 MFMAs each; PV: output tiles)
    constexpr int CPR = DH / 4;                 // float4 chunks per row
    constexpr int RPL = 256 / CPR;              // rows one load of the workgroup covers (8 or 16)
    constexpr int NL = KT / RPL;                // loads per tile and pool (4 or 2)
    const int hgroup = blockIdx.x;
    int seq = blockIdx.y;
    int qtile = prefill_tile_of_slice(blockIdx.z, gridDim.z, p.num_cus, gridDim.x * gridDim.y);
    if (p.items != nullptr) {           // the caller's own order: workgroup row y takes pair y
        seq = p.items[2 * blockIdx.y];
        qtile = p.items[2 * blockIdx.y + 1];
        if (seq < 0 || seq >= p.num_seqs || qtile < 0) return;
    }
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g4 = lane >> 4;
    const int pos_per_wg = WG_ROWS / p.gpack;

    extern __shared__ __attribute__((aligned(16))) float lds[];     // [2][K tile | V tile]

    const int q_begin = p.cu_q_lens[seq];
    const int n = p.cu_q_lens[seq + 1] - q_begin;
    const int ctx = min(p.context_lens[seq], p.max_blocks * BS);
    const int prior = ctx - n;
    const int q0 = qtile * pos_per_wg;
    if (q0 >= n || n <= 0) return;
    if (prior < 0) {
        // a context shorter than the chunk itself: the rows are defined as zero, as in the other kernels
        for (int i = tid; i < WG_ROWS * CPR; i += 256) {
            const int row = i / CPR, chunk = i % CPR;
            const int pos = q0 + row / p.gpack, hd = hgroup * p.gpack + row % p.gpack;
            if (pos < n)
                *(float4*)(p.out + ((int64_t)(q_begin + pos) * p.hq + hd) * DH + 4 * chunk) = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        return;
    }

    const int kvh = (hgroup * p.gpack) / p.group;
    int qpos[R], head[R], qabs[R];
    bool row_valid[R];
#pragma unroll
    for (int c = 0; c < R; ++c) {
        const int row = 16 * R * w + 16 * c + r16;
        qpos[c] = q0 + row / p.gpack;
        head[c] = hgroup * p.gpack + row % p.gpack;
        row_valid[c] = qpos[c] < n;
        qabs[c] = row_valid[c] ? prior + qpos[c] : ctx - 1;     // padded rows: computed, never stored
    }
    // (a wave whose rows all lie beyond the chunk's end has nothing to compute: it only takes part in
    // the tile loads and barriers)
    const int wave_kv_end = q0 + (16 * R * w) / p.gpack >= n ? 0 : min(ctx, prior + q0 + (16 * R * w + 16 * R - 1) / p.gpack + 1);
    const int wave_kv_min = prior + q0 + (16 * R * w) / p.gpack;
    const int kv_end = min(ctx, prior + q0 + pos_per_wg);
    const int ntiles = (kv_end + KT - 1) / KT;

    // Q as the B operand: MFMA 4 q + e of chunk q takes element 16 q + 4 g4 + e of this lane's row
    float4 qf[R][NQ];
#pragma unroll
    for (int c = 0; c < R; ++c) {
        const float* qrow = p.query + ((int64_t)(q_begin + min(qpos[c], n - 1)) * p.hq + head[c]) * DH + 4 * g4;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            float4 v = *(const float4*)(qrow + 16 * q);
            v.x *= p.qk_mul; v.y *= p.qk_mul; v.z *= p.qk_mul; v.w *= p.qk_mul;
            qf[c][q] = v;
        }
    }

    float m[R], lsum[R];
    f32x4_t O[R][NQ];
#pragma unroll
    for (int c = 0; c < R; ++c) {
        m[c] = NEG_BIG; lsum[c] = 0.f;
#pragma unroll
        for (int j = 0; j < NQ; ++j) O[c][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    const int32_t* table = p.block_table + (int64_t)seq * p.block_table_stride;
    const int last_blk = (ctx - 1) >> 4;

    // global -> registers: load i of the workgroup covers rows RPL * i .. of the tile, this thread
    // one 16-byte chunk of one row.  Rows at or beyond the context read the last valid block
    // (their K scores are masked and their V rows zeroed when the tile is written to LDS).
    float4 sk[NL], sv[NL];
    auto fetch = [&](int t) {
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const int row = RPL * i + tid / CPR;
            const int tok = t * KT + row;
            const int bi = min(tok >> 4, last_blk);
            const int blk = max(0, min(table[bi], p.num_blocks - 1));
            const int64_t off = (((int64_t)blk * p.hkv + kvh) * BS + (tok & 15)) * DH + 4 * (tid % CPR);
            sk[i] = *(const float4*)(p.k_pool + off);
            sv[i] = *(const float4*)(p.v_pool + off);
        }
    };
    auto stash = [&](int t, int buf) {
        float* kb = lds + buf * 2 * TILE_F;
        float* vb = kb + TILE_F;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const int row = RPL * i + tid / CPR;
            float4 vv = sv[i];
            if (t * KT + row >= ctx) vv = make_float4(0.f, 0.f, 0.f, 0.f);
            *(float4*)(kb + row * KROWF + 4 * (tid % CPR)) = sk[i];
            *(float4*)(vb + row * KROWF + 4 * (tid % CPR)) = vv;
        }
    };

    fetch(0);
    for (int t = 0; t < ntiles; ++t) {
        const int buf = t & 1;
        stash(t, buf);
        if (t + 1 < ntiles) fetch(t + 1);
        __syncthreads();          // tile t visible; everyone is done with the buffer tile t + 1 will use
        const int tile_start = t * KT;
        if (tile_start >= wave_kv_end) continue;                       // wave-uniform: above the diagonal
        const float* kb = lds + buf * 2 * TILE_F;
        const float* vb = kb + TILE_F;

        // ---- S^T = K Q^T for the two 16-token blocks of the tile
        f32x4_t sa[2][R];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int c = 0; c < R; ++c) sa[h][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            float4 a[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) a[h] = *(const float4*)(kb + (16 * h + r16) * KROWF + 16 * q + 4 * g4);
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int c = 0; c < R; ++c) {
                    sa[h][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[h].x, qf[c][q].x, sa[h][c], 0, 0, 0);
                    sa[h][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[h].y, qf[c][q].y, sa[h][c], 0, 0, 0);
                    sa[h][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[h].z, qf[c][q].z, sa[h][c], 0, 0, 0);
                    sa[h][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[h].w, qf[c][q].w, sa[h][c], 0, 0, 0);
                }
        }

        // ---- online softmax: lane (query r16, g4) holds tokens tile_start + 16 h + 4 g4 + i
        const bool need_mask = tile_start + KT - 1 > wave_kv_min;      // wave-uniform
        float pr[R][8];
#pragma unroll
        for (int c = 0; c < R; ++c) {
            float sc[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) sc[k] = sa[k >> 2][c][k & 3];
            if (need_mask) {
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (tile_start + 16 * (k >> 2) + 4 * g4 + (k & 3) > qabs[c]) sc[k] = NEG_BIG;
            }
            float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
            mx = fmaxf(mx, __shfl_xor(mx, 16));
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m[c], mx);
            const float alpha = exp2f(m[c] - m_new);
            float psum = 0.f;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                float e = exp2f(sc[k] - m_new);
                if (need_mask && sc[k] == NEG_BIG) e = 0.f;
                pr[c][k] = e;
                psum += e;
            }
            lsum[c] = lsum[c] * alpha + psum;
            m[c] = m_new;
            if (__any(alpha != 1.f)) {
#pragma unroll
                for (int j = 0; j < NQ; ++j) O[c][j] *= alpha;
            }
        }

        // ---- O^T += V^T P^T: A = V[token 16 h + 4 g4 + e][16 j + r16], B = this lane's own P values
#pragma unroll
        for (int j = 0; j < NQ; ++j) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float a[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) a[e] = vb[(16 * h + 4 * g4 + e) * KROWF + 16 * j + r16];
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int c = 0; c < R; ++c)
                        O[c][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], pr[c][4 * h + e], O[c][j], 0, 0, 0);
            }
        }
    }

    // lane (query r16 of column group c, g4) holds O^T[element 16 j + 4 g4 + i][query] in O[c][j][i]
#pragma unroll
    for (int c = 0; c < R; ++c) {
        float l = lsum[c];
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        if (row_valid[c]) {
            const float inv = l > 0.f ? 1.f / l : 0.f;
            float* o = p.out + ((int64_t)(q_begin + qpos[c]) * p.hq + head[c]) * DH + 4 * g4;
#pragma unroll
            for (int j = 0; j < NQ; ++j)
                *(float4*)(o + 16 * j) = make_float4(O[c][j][0] * inv, O[c][j][1] * inv, O[c][j][2] * inv, O[c][j][3] * inv);
        }
    }
}

template <int DH>
hipError_t launch_f32_variant(const PrefillF32Params& p, dim3 grid, hipStream_t stream) {
    constexpr size_t lds_bytes = (size_t)4 * KT * (DH * 4 + 16);       // two buffers of a K and a V tile
    if (lds_bytes > 64 * 1024) {
        // above the 64 KB a kernel may use without asking: a per-device function attribute, set once
        static std::atomic<unsigned long long> done{0};
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        if (!(dev < 64 && ((done.load(std::memory_order_acquire) >> dev) & 1ull))) {
            e = hipFuncSetAttribute((const void*)paged_prefill_mfma_f32_kernel<DH>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
            if (e != hipSuccess) return e;
            if (dev < 64) done.fetch_or(1ull << dev, std::memory_order_release);
        }
    }
    hipLaunchKernelGGL((paged_prefill_mfma_f32_kernel<DH>), grid, dim3(256), lds_bytes, stream, p);
    return hipSuccess;
}

}  // namespace

bool prefill_mfma_f32_supported(const DecodeArgs& a, int max_q_len) {
    return a.cu_q_lens != nullptr && max_q_len > 0 && a.q_dtype == AICOMP_KV_F32 && a.kv_dtype == AICOMP_KV_F32 &&
           (a.d == 128 || a.d == 64) && a.bs == BS && a.hkv > 0 && a.hq % a.hkv == 0 && a.scale > 0.f &&
           a.num_seqs <= 65535 && a.num_blocks <= INT32_MAX && ((uintptr_t)a.query % 16 == 0) &&
           ((uintptr_t)a.out % 16 == 0) && ((uintptr_t)a.k_pool % 16 == 0) && ((uintptr_t)a.v_pool % 16 == 0);
}

int prefill_mfma_f32_tile_positions(int hq, int hkv) {
    const int group = hq / hkv;
    return WG_ROWS / ((16 % group == 0) ? group : 1);
}

int launch_prefill_mfma_f32(const DecodeArgs& a, int max_q_len) {
    PrefillF32Params p;
    p.out = (float*)a.out; p.query = (const float*)a.query;
    p.k_pool = (const float*)a.k_pool; p.v_pool = (const float*)a.v_pool;
    p.block_table = a.block_table; p.block_table_stride = a.block_table_stride;
    p.context_lens = a.context_lens; p.cu_q_lens = a.cu_q_lens;
    p.hq = a.hq; p.hkv = a.hkv; p.group = a.hq / a.hkv; p.max_blocks = a.max_blocks;
    p.num_blocks = (int)a.num_blocks;
    p.gpack = (16 % p.group == 0) ? p.group : 1;
    p.qk_mul = a.scale * LOG2E;
    // CU count of the first device used (every GPU of a node is the same part); 0 if unknown
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
    p.items = a.items; p.num_seqs = a.num_seqs;
    const int pos_per_wg = WG_ROWS / p.gpack;
    const int qtiles = (max_q_len + pos_per_wg - 1) / pos_per_wg;
    AICOMP_REQUIRE(qtiles <= 65535, AICOMP_KV_EINVAL, "paged_prefill_attn: grid too large");
    dim3 grid((unsigned)(a.hq / p.gpack), (unsigned)a.num_seqs, (unsigned)qtiles);
    if (a.items != nullptr) grid = dim3((unsigned)(a.hq / p.gpack), (unsigned)a.num_items, 1);
    const hipError_t e = a.d == 64 ? launch_f32_variant<64>(p, grid, a.stream) : launch_f32_variant<128>(p, grid, a.stream);
    AICOMP_REQUIRE(e == hipSuccess, AICOMP_KV_EHIP, "paged_prefill_attn: %s", hipGetErrorString(e));
    AICOMP_HIP_LAUNCH_CHECK();
    return AICOMP_KV_OK;
}

}  // namespace aicomp
