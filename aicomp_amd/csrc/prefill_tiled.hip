// Chunked-prefill causal attention for the shapes the matrix-core kernel does not take
// (float32 models, head_dim 256, block sizes other than 16): a tiled vector-ALU kernel.
//
// Replaces  F.scaled_dot_product_attention(query, full_key, full_value,
//           attn_mask=None, is_causal=True)       opt_prime/opt_prime/kv_cache.py:404-415
// with the same mask as the matrix-core kernel: query i of a chunk with prior context P
// sees keys j <= P + i.
//
// One workgroup (256 lanes) owns 32 query rows, a row being (position, head): PP positions x
// HP heads of ONE KV head (HP = the GQA group when it is 1, 2, 4 or 8, else 1), and walks the
// keys in tiles of 32 tokens.  A K/V tile is read from the pool once per workgroup (16-byte
// coalesced loads through the block table, the next tile's loads in flight while the current
// one is used), widened to float32 and staged in LDS, so HBM traffic is linear in the context:
// K/V are read once per 32 rows, not once per row.  All arithmetic is float32 (the float32 path
// of the reference must hold 1e-5).
//
// Lane (ty = lane/16, tx = lane%16 within the workgroup's 16 x 16 grid) computes the scores of
// rows 2ty, 2ty+1 against keys 2tx, 2tx+1 (float4 reads over the head dimension: 16 FMAs per
// four LDS reads), takes the row maxima with shuffles over its 16 neighbours, writes the
// probabilities to an LDS tile, and accumulates its D/16 output columns of the two rows.
#include "common.h"

#include <atomic>

namespace aicomp {

namespace {

constexpr int BM = 32;                 // query rows per workgroup
constexpr int BN = 32;                 // keys per tile
constexpr float NEG_BIG = -1.0e30f;

struct TiledParams {
    void* out;
    const void* query;
    const void* k_pool;
    const void* v_pool;
    const int32_t* block_table;
    int64_t block_table_stride;
    const int32_t* context_lens;
    const int32_t* cu_q_lens;
    int hq, hkv, group, hp, bs, max_blocks;
    int64_t num_blocks;
    float qk_mul;                      // scale * log2(e)
    const float* k_scale;
    const float* v_scale;
};

// 8 or 16 raw bytes of pool type KV_T -> N floats
template <typename KV_T> struct Chunk;
template <> struct Chunk<float> {
    static constexpr int N = 4;
    typedef uint4 Raw;
    __device__ __forceinline__ static void unpack(const Raw& r, float* f) { Vec16<float>::unpack(r, f); }
};
template <> struct Chunk<bf16_t> {
    static constexpr int N = 8;
    typedef uint4 Raw;
    __device__ __forceinline__ static void unpack(const Raw& r, float* f) { Vec16<bf16_t>::unpack(r, f); }
};
template <> struct Chunk<f16_t> {
    static constexpr int N = 8;
    typedef uint4 Raw;
    __device__ __forceinline__ static void unpack(const Raw& r, float* f) { Vec16<f16_t>::unpack(r, f); }
};
template <> struct Chunk<fp8_t> {
    static constexpr int N = 8;
    typedef uint2 Raw;
    __device__ __forceinline__ static void unpack(const Raw& r, float* f) {
        const uint32_t w[2] = {r.x, r.y};
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            auto lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], false);
            auto hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], true);
            f[4 * i] = lo[0]; f[4 * i + 1] = lo[1];
            f[4 * i + 2] = hi[0]; f[4 * i + 3] = hi[1];
        }
    }
};

template <typename KV_T, typename Q_T, int D>
__global__ void __launch_bounds__(256)
paged_prefill_tiled_kernel(TiledParams p) {
    constexpr int N = Chunk<KV_T>::N;
    typedef typename Chunk<KV_T>::Raw Raw;
    constexpr int CPR = D / N;                         // chunks per K/V row
    constexpr int NLD = BN * CPR / 256;                // chunks per lane, tile and pool
    static_assert(BN * CPR % 256 == 0 && NLD >= 1, "tile must split evenly over the workgroup");
    constexpr int KSTR = D + 4;                        // K row stride in floats: keys 2tx land 8 banks apart
    constexpr int PSTR = BN + 1;
    constexpr int DC = D / 16;                         // output columns per lane

    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* sq = smem;                                  // [BM][D]     query rows, scaled
    float* sk = sq + BM * D;                           // [BN][KSTR]
    float* sv = sk + BN * KSTR;                        // [BN][D]
    float* sp = sv + BN * D;                           // [BM][PSTR]  probabilities of the tile

    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int seq = blockIdx.z;
    const int hp = p.hp, pp = BM / hp;                 // heads and positions per workgroup
    const int head0 = blockIdx.y * hp;                 // first query head; all hp heads share one KV head
    const int kvh = head0 / p.group;
    const int q_begin = p.cu_q_lens[seq];
    const int n = p.cu_q_lens[seq + 1] - q_begin;
    const int q0 = blockIdx.x * pp;
    if (n <= 0 || q0 >= n) return;
    const int ctx = min(p.context_lens[seq], p.max_blocks * p.bs);
    const int prior = ctx - n;
    Q_T* out = (Q_T*)p.out;
    if (prior < 0) {                                   // inconsistent lengths: rows defined as zero
        for (int i = tid; i < BM * D; i += 256) {
            const int r = i / D, pos = q0 + r / hp;
            if (pos < n) store_elem<Q_T>(out + ((int64_t)(q_begin + pos) * p.hq + head0 + r % hp) * D + i % D, 0.f);
        }
        return;
    }
    // ---- query rows -> LDS, multiplied by scale * log2(e) (* k_scale for an fp8 pool)
    {
        const float mul = p.qk_mul * (p.k_scale ? p.k_scale[kvh] : 1.f);
        const Q_T* q = (const Q_T*)p.query;
        for (int i = tid; i < BM * D; i += 256) {
            const int r = i / D, pos = min(q0 + r / hp, n - 1);
            sq[i] = load_elem<Q_T>(q + ((int64_t)(q_begin + pos) * p.hq + head0 + r % hp) * D + i % D) * mul;
        }
    }
    // keys this workgroup needs: up to the last position's own token
    const int kv_end = min(ctx, prior + min(q0 + pp, n));
    const int ntiles = (kv_end + BN - 1) / BN;
    const int32_t* table = p.block_table + (int64_t)seq * p.block_table_stride;
    const KV_T* kp = (const KV_T*)p.k_pool;
    const KV_T* vp = (const KV_T*)p.v_pool;

    Raw kreg[NLD], vreg[NLD];
    auto fetch = [&](int t) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int c = tid + 256 * i;               // chunk of the tile
            const int tok = min(t * BN + c / CPR, ctx - 1);          // clamped: always loadable
            int64_t blk = table[tok / p.bs];
            blk = blk < 0 ? 0 : (blk >= p.num_blocks ? p.num_blocks - 1 : blk);
            const int64_t base = ((blk * p.hkv + kvh) * p.bs + tok % p.bs) * D + (c % CPR) * N;
            kreg[i] = *(const Raw*)(kp + base);
            vreg[i] = *(const Raw*)(vp + base);
        }
    };
    auto stash = [&](int t) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int c = tid + 256 * i;
            const int row = c / CPR, col = (c % CPR) * N;
            float kf[N], vf[N];
            Chunk<KV_T>::unpack(kreg[i], kf);
            Chunk<KV_T>::unpack(vreg[i], vf);
            const bool live = t * BN + row < ctx;      // beyond the context: zeros, never non-finite leftovers
#pragma unroll
            for (int e = 0; e < N; e += 4) {
                *(float4*)(sk + row * KSTR + col + e) = live ? make_float4(kf[e], kf[e + 1], kf[e + 2], kf[e + 3])
                                                             : make_float4(0.f, 0.f, 0.f, 0.f);
                *(float4*)(sv + row * D + col + e) = live ? make_float4(vf[e], vf[e + 1], vf[e + 2], vf[e + 3])
                                                          : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    };

    // this lane's two rows
    int qabs[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int pos = q0 + (2 * ty + r) / hp;
        qabs[r] = pos < n ? prior + pos : -1;          // rows past the chunk see no key
    }
    float m[2] = {NEG_BIG, NEG_BIG}, l[2] = {0.f, 0.f};
    float o[2][DC];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int c = 0; c < DC; ++c) o[r][c] = 0.f;

    fetch(0);
    for (int t = 0; t < ntiles; ++t) {
        __syncthreads();                               // everyone is done with the previous tile (and sq is written)
        stash(t);
        if (t + 1 < ntiles) fetch(t + 1);
        __syncthreads();
        // ---- scores of rows 2ty, 2ty+1 against keys 2tx, 2tx+1
        float s[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
        const float* q0p = sq + (2 * ty) * D;
        const float* k0p = sk + (2 * tx) * KSTR;
#pragma unroll 8
        for (int d = 0; d < D; d += 4) {
            const float4 qa = *(const float4*)(q0p + d), qb = *(const float4*)(q0p + D + d);
            const float4 ka = *(const float4*)(k0p + d), kb = *(const float4*)(k0p + KSTR + d);
            s[0][0] = fmaf(qa.x, ka.x, fmaf(qa.y, ka.y, fmaf(qa.z, ka.z, fmaf(qa.w, ka.w, s[0][0]))));
            s[0][1] = fmaf(qa.x, kb.x, fmaf(qa.y, kb.y, fmaf(qa.z, kb.z, fmaf(qa.w, kb.w, s[0][1]))));
            s[1][0] = fmaf(qb.x, ka.x, fmaf(qb.y, ka.y, fmaf(qb.z, ka.z, fmaf(qb.w, ka.w, s[1][0]))));
            s[1][1] = fmaf(qb.x, kb.x, fmaf(qb.y, kb.y, fmaf(qb.z, kb.z, fmaf(qb.w, kb.w, s[1][1]))));
        }
        // ---- online softmax per row (log2 domain); the 16 lanes of a row sit side by side
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int key0 = t * BN + 2 * tx;
            const bool live0 = key0 <= qabs[r], live1 = key0 + 1 <= qabs[r];
            float mx = fmaxf(live0 ? s[r][0] : NEG_BIG, live1 ? s[r][1] : NEG_BIG);
#pragma unroll
            for (int off = 1; off < 16; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
            const float m_new = fmaxf(m[r], mx);
            const float alpha = exp2f(m[r] - m_new);
            const float p0 = live0 ? exp2f(s[r][0] - m_new) : 0.f;
            const float p1 = live1 ? exp2f(s[r][1] - m_new) : 0.f;
            float ps = p0 + p1;
#pragma unroll
            for (int off = 1; off < 16; off <<= 1) ps += __shfl_xor(ps, off);
            l[r] = l[r] * alpha + ps;
            m[r] = m_new;
#pragma unroll
            for (int c = 0; c < DC; ++c) o[r][c] *= alpha;
            sp[(2 * ty + r) * PSTR + 2 * tx] = p0;
            sp[(2 * ty + r) * PSTR + 2 * tx + 1] = p1;
        }
        // the probabilities of a row are written and read by the same 16 lanes of one wave, and a
        // wave's LDS operations complete in program order: no workgroup barrier
        __builtin_amdgcn_wave_barrier();
        // ---- O += P V over this lane's DC columns
        const float* pr = sp + (2 * ty) * PSTR;
        const float* vcol = sv + tx * DC;
#pragma unroll 4
        for (int j = 0; j < BN; ++j) {
            const float pa = pr[j], pb = pr[PSTR + j];
#pragma unroll
            for (int c = 0; c < DC; c += 4) {
                const float4 vv = *(const float4*)(vcol + j * D + c);
                o[0][c] = fmaf(pa, vv.x, o[0][c]); o[0][c + 1] = fmaf(pa, vv.y, o[0][c + 1]);
                o[0][c + 2] = fmaf(pa, vv.z, o[0][c + 2]); o[0][c + 3] = fmaf(pa, vv.w, o[0][c + 3]);
                o[1][c] = fmaf(pb, vv.x, o[1][c]); o[1][c + 1] = fmaf(pb, vv.y, o[1][c + 1]);
                o[1][c + 2] = fmaf(pb, vv.z, o[1][c + 2]); o[1][c + 3] = fmaf(pb, vv.w, o[1][c + 3]);
            }
        }
    }
    const float vs = p.v_scale ? p.v_scale[kvh] : 1.f;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int row = 2 * ty + r, pos = q0 + row / hp;
        if (pos >= n) continue;
        const float inv = l[r] > 0.f ? vs / l[r] : 0.f;
        Q_T* dst = out + ((int64_t)(q_begin + pos) * p.hq + head0 + row % hp) * D + tx * DC;
#pragma unroll
        for (int c = 0; c < DC; ++c) store_elem<Q_T>(dst + c, o[r][c] * inv);
    }
}

template <typename KV_T, typename Q_T, int D>
hipError_t launch_variant(const TiledParams& p, dim3 grid, hipStream_t stream) {
    const size_t lds = sizeof(float) * (BM * D + BN * (D + 4) + BN * D + BM * (BN + 1));
    if (lds > 64 * 1024) {
        // above the 64 KB a kernel may use without asking: a per-device function attribute, set once
        static std::atomic<unsigned long long> done{0};
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        if (!(dev < 64 && ((done.load(std::memory_order_acquire) >> dev) & 1ull))) {
            e = hipFuncSetAttribute((const void*)paged_prefill_tiled_kernel<KV_T, Q_T, D>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            if (dev < 64) done.fetch_or(1ull << dev, std::memory_order_release);
        }
    }
    hipLaunchKernelGGL((paged_prefill_tiled_kernel<KV_T, Q_T, D>), grid, dim3(256), lds, stream, p);
    return hipSuccess;
}

template <typename KV_T, typename Q_T>
hipError_t launch_d(const TiledParams& p, int d, dim3 grid, hipStream_t stream) {
    switch (d) {
        case 64: return launch_variant<KV_T, Q_T, 64>(p, grid, stream);
        case 128: return launch_variant<KV_T, Q_T, 128>(p, grid, stream);
        default: return launch_variant<KV_T, Q_T, 256>(p, grid, stream);
    }
}

}  // namespace

bool prefill_tiled_supported(const DecodeArgs& a, int max_q_len) {
    const bool types = (a.q_dtype == AICOMP_KV_F32 && a.kv_dtype == AICOMP_KV_F32) ||
                       (is_16bit_float(a.q_dtype) && (a.kv_dtype == a.q_dtype || a.kv_dtype == AICOMP_KV_FP8_E4M3));
    const int e = dtype_size(a.kv_dtype);
    return a.cu_q_lens != nullptr && max_q_len > 0 && types && (a.d == 64 || a.d == 128 || a.d == 256) &&
           a.hkv > 0 && a.hq % a.hkv == 0 && a.num_seqs <= 65535 && a.hq <= 65535 &&
           ((uintptr_t)a.k_pool % 16 == 0) && ((uintptr_t)a.v_pool % 16 == 0) && (a.d * e) % 16 == 0;
}

int launch_prefill_tiled(const DecodeArgs& a, int max_q_len) {
    TiledParams p;
    p.out = a.out; p.query = a.query; p.k_pool = a.k_pool; p.v_pool = a.v_pool;
    p.block_table = a.block_table; p.block_table_stride = a.block_table_stride;
    p.context_lens = a.context_lens; p.cu_q_lens = a.cu_q_lens;
    p.hq = a.hq; p.hkv = a.hkv; p.group = a.hq / a.hkv; p.bs = a.bs; p.max_blocks = a.max_blocks;
    p.num_blocks = a.num_blocks;
    p.hp = (p.group == 2 || p.group == 4 || p.group == 8) ? p.group : 1;
    p.qk_mul = a.scale * LOG2E;
    p.k_scale = a.k_scale; p.v_scale = a.v_scale;
    const int pp = BM / p.hp;
    const int64_t qtiles = ((int64_t)max_q_len + pp - 1) / pp;
    AICOMP_REQUIRE(qtiles < (1ll << 31), AICOMP_KV_EINVAL, "paged_prefill_attn: grid too large");
    dim3 grid((unsigned)qtiles, (unsigned)(a.hq / p.hp), (unsigned)a.num_seqs);
    hipError_t e;
    if (a.q_dtype == AICOMP_KV_F32) e = launch_d<float, float>(p, a.d, grid, a.stream);
    else if (a.q_dtype == AICOMP_KV_BF16 && a.kv_dtype == AICOMP_KV_BF16) e = launch_d<bf16_t, bf16_t>(p, a.d, grid, a.stream);
    else if (a.q_dtype == AICOMP_KV_BF16) e = launch_d<fp8_t, bf16_t>(p, a.d, grid, a.stream);
    else if (a.kv_dtype == AICOMP_KV_F16) e = launch_d<f16_t, f16_t>(p, a.d, grid, a.stream);
    else e = launch_d<fp8_t, f16_t>(p, a.d, grid, a.stream);
    AICOMP_REQUIRE(e == hipSuccess, AICOMP_KV_EHIP, "paged_prefill_attn: %s", hipGetErrorString(e));
    AICOMP_HIP_LAUNCH_CHECK();
    return AICOMP_KV_OK;
}

}  // namespace aicomp
