// Generic paged attention kernel (vector ALU): any supported storage type,
// head_dim 64/128/256, any GQA group, any block size.  It is the path for
// shapes the MFMA kernels do not cover (fp32 pools, head_dim != 128, block
// sizes other than 16) and the split-K reduce shared by every decode kernel.
//
// Replaces  F.scaled_dot_product_attention(query, full_key, full_value,
//           attn_mask=None, is_causal=False)       opt_prime/opt_prime/kv_cache.py:397-403
// (and, with cu_q_lens, the is_causal=True prefill of kv_cache.py:404-415, one
// query row at a time) reading K/V through the block table instead of from the
// .contiguous() prefix copy of kv_cache.py:391-392.
//
// Work split: one workgroup (4 waves) per (query row, KV head, partition).
// A K/V row of D elements is read by LPR consecutive lanes with one 16-byte
// (8-byte for fp8) load each, so a wave reads 64/LPR whole rows per load:
// full-line, coalesced requests.  Every lane group keeps its own online-softmax
// state (running max, sum, accumulator) for the tokens it visits; the groups
// are merged with wave shuffles, the waves through LDS.  All G query heads of
// the KV head share each loaded K/V chunk.
#include "common.h"

namespace aicomp {

// K/V rows are read once per call: non-temporal loads (streaming, no reuse in L2)
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 stream_ld16(const void* p) {
    u32x4_t v = __builtin_nontemporal_load((const u32x4_t*)p);
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint2 stream_ld8(const void* p) {
    u32x2_t v = __builtin_nontemporal_load((const u32x2_t*)p);
    return make_uint2(v[0], v[1]);
}

template <typename KV_T> struct KvLoad;
template <> struct KvLoad<float> {
    static constexpr int N = 4;
    typedef uint4 Raw;
    __device__ __forceinline__ static Raw raw(const float* p) { return stream_ld16(p); }
    __device__ __forceinline__ static void unpack(const Raw& r, float* f) { Vec16<float>::unpack(r, f); }
};
template <> struct KvLoad<bf16_t> {
    static constexpr int N = 8;
    typedef uint4 Raw;
    __device__ __forceinline__ static Raw raw(const bf16_t* p) { return stream_ld16(p); }
    __device__ __forceinline__ static void unpack(const Raw& r, float* f) { Vec16<bf16_t>::unpack(r, f); }
};
template <> struct KvLoad<f16_t> {
    static constexpr int N = 8;
    typedef uint4 Raw;
    __device__ __forceinline__ static Raw raw(const f16_t* p) { return stream_ld16(p); }
    __device__ __forceinline__ static void unpack(const Raw& r, float* f) { Vec16<f16_t>::unpack(r, f); }
};
template <> struct KvLoad<fp8_t> {
    static constexpr int N = 8;
    typedef uint2 Raw;
    __device__ __forceinline__ static Raw raw(const fp8_t* p) { return stream_ld8(p); }
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

struct GenericParams {
    void* out;
    const void* query;
    const void* k_pool;
    const void* v_pool;
    const int32_t* block_table;
    int64_t block_table_stride;
    const int32_t* context_lens;
    const int32_t* cu_q_lens;
    int num_seqs;
    int hq, hkv, group, bs;
    int64_t num_blocks;
    float qk_mul;               // scale * log2(e)
    const float* k_scale;
    const float* v_scale;
    int partition_size, num_parts;
    float* ws_acc;
    float* ws_ml;
};

// sequence and attended length of a query row
__device__ __forceinline__ void row_info(int64_t row, const int32_t* cu, const int32_t* ctx,
                                         int num_seqs, int& seq, int& len) {
    if (cu == nullptr) {
        seq = (int)row;
        len = ctx[row];
    } else {
        int lo = 0, hi = num_seqs;       // largest s with cu[s] <= row
        while (hi - lo > 1) {
            int mid = (lo + hi) >> 1;
            if (cu[mid] <= row) lo = mid; else hi = mid;
        }
        seq = lo;
        int n = cu[lo + 1] - cu[lo];
        int i = (int)(row - cu[lo]);
        len = ctx[lo] < n ? 0 : ctx[lo] - n + i + 1;       // bottom-right aligned causal mask; a context
                                                            // shorter than its chunk: zero rows
    }
    if (len < 0) len = 0;
}

constexpr float NEG_BIG = -1.0e30f;

template <typename KV_T, typename Q_T, int D, int GMAX>
__global__ void __launch_bounds__(256)
paged_attn_generic_kernel(GenericParams p) {
    constexpr int N = KvLoad<KV_T>::N;
    constexpr int LPR = D / N;            // lanes per K/V row
    constexpr int TPW = WAVE / LPR;       // rows per wave per load
    constexpr int NW = 4;
    static_assert(LPR >= 1 && LPR <= 64 && (LPR & (LPR - 1)) == 0, "row must split over 2^k lanes");

    const int64_t row = blockIdx.x;
    const int groups_per_kv = (p.group + GMAX - 1) / GMAX;
    const int kvh = blockIdx.y / groups_per_kv;
    const int g0 = (blockIdx.y % groups_per_kv) * GMAX;      // first head of the group handled here
    const int gn = min(GMAX, p.group - g0);
    const int part = blockIdx.z;

    int seq, len;
    row_info(row, p.cu_q_lens, p.context_lens, p.num_seqs, seq, len);
    const int start = part * p.partition_size;
    const int end = min(len, start + p.partition_size);
    const int tid = threadIdx.x;
    const int head0 = kvh * p.group + g0;

    if (start >= end) {
        // nothing here; an unsplit call still owes the caller a defined output
        if (p.num_parts == 1) {
            Q_T* o = (Q_T*)p.out + (row * p.hq + head0) * D;
            for (int i = tid; i < gn * D; i += blockDim.x) store_elem<Q_T>(o + i, 0.f);
        }
        return;
    }

    const int w = tid / WAVE, lane = tid % WAVE;
    const int sub = lane / LPR, lr = lane % LPR;

    float q[GMAX][N];
    {
        const float mul = p.qk_mul * (p.k_scale ? p.k_scale[kvh] : 1.f);
        const Q_T* qp = (const Q_T*)p.query + (row * p.hq + head0) * D + lr * N;
#pragma unroll
        for (int g = 0; g < GMAX; ++g)
#pragma unroll
            for (int e = 0; e < N; ++e)
                q[g][e] = (g < gn) ? load_elem<Q_T>(qp + g * D + e) * mul : 0.f;
    }

    float m[GMAX], l[GMAX], acc[GMAX][N];
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
        m[g] = NEG_BIG; l[g] = 0.f;
#pragma unroll
        for (int e = 0; e < N; ++e) acc[g][e] = 0.f;
    }

    const int32_t* table = p.block_table + (int64_t)seq * p.block_table_stride;
    const KV_T* kp = (const KV_T*)p.k_pool;
    const KV_T* vp = (const KV_T*)p.v_pool;
    // Two tokens per lane group and step, and the next step's four K/V chunks are requested before
    // the current ones are used: eight 16-byte loads in flight per lane.  One running-max update
    // (one rescale of the accumulators) serves both tokens.
    constexpr int STEP = 2 * NW * TPW;                 // tokens per workgroup step
    const int steps = (end - start + STEP - 1) / STEP;
    typedef typename KvLoad<KV_T>::Raw Raw;
    auto fetch = [&](int it, Raw (&kraw)[2], Raw (&vraw)[2]) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int tok = min(start + it * STEP + u * NW * TPW + w * TPW + sub, end - 1);   // clamped: always loadable
            int64_t blk = table[tok / p.bs];
            blk = blk < 0 ? 0 : (blk >= p.num_blocks ? p.num_blocks - 1 : blk);  // never leave the pool
            const int64_t base = ((blk * p.hkv + kvh) * p.bs + tok % p.bs) * D + lr * N;
            kraw[u] = KvLoad<KV_T>::raw(kp + base);
            vraw[u] = KvLoad<KV_T>::raw(vp + base);
        }
    };
    Raw kcur[2], vcur[2], knext[2], vnext[2];
    fetch(0, kcur, vcur);
    for (int it = 0; it < steps; ++it) {
        if (it + 1 < steps) fetch(it + 1, knext, vnext);
        const int tok0 = start + it * STEP + w * TPW + sub;
        const bool valid0 = tok0 < end, valid1 = tok0 + NW * TPW < end;
        float k0[N], v0[N], k1[N], v1[N];
        KvLoad<KV_T>::unpack(kcur[0], k0);
        KvLoad<KV_T>::unpack(kcur[1], k1);
        KvLoad<KV_T>::unpack(vcur[0], v0);
        KvLoad<KV_T>::unpack(vcur[1], v1);
        if (!valid0) {
#pragma unroll
            for (int e = 0; e < N; ++e) v0[e] = 0.f;           // a clamped reload may hold anything
        }
        if (!valid1) {
#pragma unroll
            for (int e = 0; e < N; ++e) v1[e] = 0.f;
        }
#pragma unroll
        for (int g = 0; g < GMAX; ++g) {
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int e = 0; e < N; ++e) { s0 = fmaf(q[g][e], k0[e], s0); s1 = fmaf(q[g][e], k1[e], s1); }
#pragma unroll
            for (int o = 1; o < LPR; o <<= 1) { s0 += __shfl_xor(s0, o); s1 += __shfl_xor(s1, o); }
            float m_new = m[g];
            if (valid0) m_new = fmaxf(m_new, s0);
            if (valid1) m_new = fmaxf(m_new, s1);
            const float alpha = __builtin_amdgcn_exp2f(m[g] - m_new);
            const float p0 = valid0 ? __builtin_amdgcn_exp2f(s0 - m_new) : 0.f;
            const float p1 = valid1 ? __builtin_amdgcn_exp2f(s1 - m_new) : 0.f;
            m[g] = m_new;
            l[g] = l[g] * alpha + p0 + p1;
#pragma unroll
            for (int e = 0; e < N; ++e) acc[g][e] = fmaf(p1, v1[e], fmaf(p0, v0[e], acc[g][e] * alpha));
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) { kcur[u] = knext[u]; vcur[u] = vnext[u]; }
    }

    // merge the TPW lane groups of the wave
#pragma unroll
    for (int o = LPR; o < WAVE; o <<= 1) {
#pragma unroll
        for (int g = 0; g < GMAX; ++g) {
            const float mo = __shfl_xor(m[g], o);
            const float lo = __shfl_xor(l[g], o);
            const float mn = fmaxf(m[g], mo);
            const float a = exp2f(m[g] - mn), b = exp2f(mo - mn);
            l[g] = l[g] * a + lo * b;
#pragma unroll
            for (int e = 0; e < N; ++e) {
                const float ao = __shfl_xor(acc[g][e], o);
                acc[g][e] = acc[g][e] * a + ao * b;
            }
            m[g] = mn;
        }
    }

    // merge the waves through LDS
    __shared__ float sm_m[NW][GMAX];
    __shared__ float sm_l[NW][GMAX];
    __shared__ float sm_acc[NW][GMAX][D];
    if (sub == 0) {
#pragma unroll
        for (int g = 0; g < GMAX; ++g) {
            if (lr == 0) { sm_m[w][g] = m[g]; sm_l[w][g] = l[g]; }
#pragma unroll
            for (int e = 0; e < N; ++e) sm_acc[w][g][lr * N + e] = acc[g][e];
        }
    }
    __syncthreads();

    const float vs = p.v_scale ? p.v_scale[kvh] : 1.f;
    for (int i = tid; i < gn * D; i += blockDim.x) {
        const int g = i / D, dd = i % D;
        float mx = sm_m[0][g];
#pragma unroll
        for (int ww = 1; ww < NW; ++ww) mx = fmaxf(mx, sm_m[ww][g]);
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int ww = 0; ww < NW; ++ww) {
            const float f = exp2f(sm_m[ww][g] - mx);
            num = fmaf(f, sm_acc[ww][g][dd], num);
            den = fmaf(f, sm_l[ww][g], den);
        }
        const int head = head0 + g;
        if (p.num_parts == 1) {
            store_elem<Q_T>((Q_T*)p.out + (row * p.hq + head) * D + dd, den > 0.f ? vs * num / den : 0.f);
        } else {
            const int64_t slot = (row * p.hq + head) * p.num_parts + part;
            p.ws_acc[slot * D + dd] = num;
            if (dd == 0) { p.ws_ml[slot * 2] = mx; p.ws_ml[slot * 2 + 1] = den; }
        }
    }
}

// Split-K merge: out = sum_p 2^(m_p - M) acc_p / sum_p 2^(m_p - M) l_p, M = max_p m_p.
// One workgroup per (row, head); only the partitions that hold tokens are read.  The
// weights 2^(m_p - M) / sum are computed once (one lane per partition, wave reduction) and
// parked in LDS; the accumulation loop then issues independent loads.
template <typename Q_T>
__global__ void __launch_bounds__(128)
split_reduce_kernel(Q_T* __restrict__ out, const float* __restrict__ ws_acc,
                    const float* __restrict__ ws_ml, const int32_t* __restrict__ context_lens,
                    const int32_t* __restrict__ cu_q_lens, int num_seqs, int hq, int group, int d,
                    int partition_size, int num_parts, const float* __restrict__ v_scale) {
    const int64_t row = blockIdx.x;
    const int head = blockIdx.y;
    int seq, len;
    row_info(row, cu_q_lens, context_lens, num_seqs, seq, len);
    const int np = min(num_parts, (len + partition_size - 1) / partition_size);
    const int64_t slot0 = (row * hq + head) * num_parts;
    __shared__ float wgt[1024];
    __shared__ float red[2][2];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    // pass 1: max over partitions
    float mx = NEG_BIG;
    for (int pi = tid; pi < np; pi += blockDim.x) mx = fmaxf(mx, ws_ml[(slot0 + pi) * 2]);
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if (lane == 0) red[0][wv] = mx;
    __syncthreads();
    mx = fmaxf(red[0][0], red[0][1]);
    // pass 2: weights and their sum (np <= 1024 partitions are cached in LDS)
    float den = 0.f;
    for (int pi = tid; pi < np; pi += blockDim.x) {
        const float f = exp2f(ws_ml[(slot0 + pi) * 2] - mx);
        if (pi < 1024) wgt[pi] = f;
        den = fmaf(f, ws_ml[(slot0 + pi) * 2 + 1], den);
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) den += __shfl_xor(den, o);
    if (lane == 0) red[1][wv] = den;
    __syncthreads();
    den = red[1][0] + red[1][1];
    const float vs = v_scale ? v_scale[head / group] : 1.f;
    const float inv = den > 0.f ? vs / den : 0.f;
    for (int dd = tid; dd < d; dd += blockDim.x) {
        float num = 0.f;
        const float* a = ws_acc + slot0 * d + dd;
        int pi = 0;
        for (; pi + 4 <= np && pi + 4 <= 1024; pi += 4) {
            const float a0 = a[(int64_t)pi * d], a1 = a[(int64_t)(pi + 1) * d];
            const float a2 = a[(int64_t)(pi + 2) * d], a3 = a[(int64_t)(pi + 3) * d];
            num = fmaf(wgt[pi], a0, num); num = fmaf(wgt[pi + 1], a1, num);
            num = fmaf(wgt[pi + 2], a2, num); num = fmaf(wgt[pi + 3], a3, num);
        }
        for (; pi < np; ++pi) {
            const float f = pi < 1024 ? wgt[pi] : exp2f(ws_ml[(slot0 + pi) * 2] - mx);
            num = fmaf(f, a[(int64_t)pi * d], num);
        }
        store_elem<Q_T>(out + (row * hq + head) * d + dd, num * inv);
    }
}

int launch_split_reduce(const DecodeArgs& a) {
    dim3 grid((unsigned)a.rows, (unsigned)a.hq);
    const int threads = 128;
    const int group = a.hq / a.hkv;
    if (a.q_dtype == AICOMP_KV_F32)
        hipLaunchKernelGGL(split_reduce_kernel<float>, grid, dim3(threads), 0, a.stream,
                           (float*)a.out, a.ws.acc, a.ws.ml, a.context_lens, a.cu_q_lens,
                           a.num_seqs, a.hq, group, a.d, a.partition_size, a.num_parts, a.v_scale);
    else if (a.q_dtype == AICOMP_KV_F16)
        hipLaunchKernelGGL(split_reduce_kernel<f16_t>, grid, dim3(threads), 0, a.stream,
                           (f16_t*)a.out, a.ws.acc, a.ws.ml, a.context_lens, a.cu_q_lens,
                           a.num_seqs, a.hq, group, a.d, a.partition_size, a.num_parts, a.v_scale);
    else
        hipLaunchKernelGGL(split_reduce_kernel<bf16_t>, grid, dim3(threads), 0, a.stream,
                           (bf16_t*)a.out, a.ws.acc, a.ws.ml, a.context_lens, a.cu_q_lens,
                           a.num_seqs, a.hq, group, a.d, a.partition_size, a.num_parts, a.v_scale);
    AICOMP_HIP_LAUNCH_CHECK();
    return AICOMP_KV_OK;
}

template <typename KV_T, typename Q_T, int D>
static int launch_generic_d(const DecodeArgs& a, const GenericParams& p) {
    const int group = a.hq / a.hkv;
    if (group <= 4) {
        dim3 grid((unsigned)a.rows, (unsigned)a.hkv, (unsigned)a.num_parts);
        hipLaunchKernelGGL((paged_attn_generic_kernel<KV_T, Q_T, D, 4>), grid, dim3(256), 0,
                           a.stream, p);
    } else {
        const int gpk = (group + 7) / 8;
        dim3 grid((unsigned)a.rows, (unsigned)(a.hkv * gpk), (unsigned)a.num_parts);
        hipLaunchKernelGGL((paged_attn_generic_kernel<KV_T, Q_T, D, 8>), grid, dim3(256), 0,
                           a.stream, p);
    }
    AICOMP_HIP_LAUNCH_CHECK();
    return AICOMP_KV_OK;
}

template <typename KV_T, typename Q_T>
static int launch_generic_t(const DecodeArgs& a, const GenericParams& p) {
    switch (a.d) {
        case 64: return launch_generic_d<KV_T, Q_T, 64>(a, p);
        case 128: return launch_generic_d<KV_T, Q_T, 128>(a, p);
        case 256: return launch_generic_d<KV_T, Q_T, 256>(a, p);
        default:
            set_error("paged attention: head_dim %d not supported (64, 128, 256)", a.d);
            return AICOMP_KV_EUNSUPPORTED;
    }
}

int launch_decode_generic(const DecodeArgs& a) {
    if (a.rows == 0) return AICOMP_KV_OK;
    AICOMP_REQUIRE(a.rows < (1ll << 31) && a.num_parts <= 65535 && a.hkv * ((a.hq / a.hkv + 7) / 8) <= 65535, AICOMP_KV_EINVAL,
                   "paged attention: grid too large");
    GenericParams p;
    p.out = a.out; p.query = a.query; p.k_pool = a.k_pool; p.v_pool = a.v_pool;
    p.block_table = a.block_table; p.block_table_stride = a.block_table_stride;
    p.context_lens = a.context_lens; p.cu_q_lens = a.cu_q_lens; p.num_seqs = a.num_seqs;
    p.hq = a.hq; p.hkv = a.hkv; p.group = a.hq / a.hkv; p.bs = a.bs; p.num_blocks = a.num_blocks;
    p.qk_mul = a.scale * LOG2E;
    p.k_scale = a.k_scale; p.v_scale = a.v_scale;
    p.partition_size = a.partition_size; p.num_parts = a.num_parts;
    p.ws_acc = a.ws.acc; p.ws_ml = a.ws.ml;
    int rc;
    if (a.kv_dtype == AICOMP_KV_F32 && a.q_dtype == AICOMP_KV_F32)
        rc = launch_generic_t<float, float>(a, p);
    else if (a.kv_dtype == AICOMP_KV_BF16 && a.q_dtype == AICOMP_KV_BF16)
        rc = launch_generic_t<bf16_t, bf16_t>(a, p);
    else if (a.kv_dtype == AICOMP_KV_FP8_E4M3 && a.q_dtype == AICOMP_KV_BF16)
        rc = launch_generic_t<fp8_t, bf16_t>(a, p);
    else if (a.kv_dtype == AICOMP_KV_F16 && a.q_dtype == AICOMP_KV_F16)
        rc = launch_generic_t<f16_t, f16_t>(a, p);
    else if (a.kv_dtype == AICOMP_KV_FP8_E4M3 && a.q_dtype == AICOMP_KV_F16)
        rc = launch_generic_t<fp8_t, f16_t>(a, p);
    else {
        set_error("paged attention: unsupported type pair (query %d, pool %d); supported: "
                  "f32/f32, bf16/bf16, f16/f16, bf16/fp8, f16/fp8", a.q_dtype, a.kv_dtype);
        return AICOMP_KV_EUNSUPPORTED;
    }
    if (rc != AICOMP_KV_OK) return rc;
    if (a.num_parts > 1) return launch_split_reduce(a);
    return AICOMP_KV_OK;
}

}  // namespace aicomp
