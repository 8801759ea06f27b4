// Rotary position embedding fused with the KV-cache append.
//
// What the caller of the attention operator does before it, in three separate passes
// over Q and K plus a G-fold expansion of K and V:
//   q_embed = (q * cos) + (rotate_half(q) * sin)          compiler_fx/modeling_llama.py:200-231
//   k_embed = (k * cos) + (rotate_half(k) * sin)          (call site :582)
//   key_states = repeat_kv(key_states, G)                 compiler_fx/modeling_llama.py:268-277, :589-590
// followed by the operator's own append                   opt_prime/opt_prime/kv_cache.py:387-388
// becomes one launch: Q is rotated into `q_out`, K is rotated and written straight
// into its pool slot, V is copied into its slot; KV heads are stored once.
//
// Arithmetic follows the reference's eager evaluation step by step, so the result is
// bit-identical to it: each product is rounded to the tensor type (bf16 or fp32), then
// the sum is rounded again; no fused multiply-add.  cos/sin come from a table in the
// tensor's type, indexed by position (or by row when `positions` is null), all D columns
// read as given (the reference's table repeats its first half; nothing here relies on it).
// With an fp8 pool the rotated K and the V row are quantised like the plain append does.
//
// HBM-bound and small.  One lane owns 8 columns j .. j+7 of the low half and the matching
// 8 of the high half of one (token, head) row: both halves of a rotation pair are in
// the same lane, every access is a 16-byte (bf16) or 2 x 16-byte (fp32) vector.
#include "common.h"

namespace aicomp {

namespace {

struct RopeParams {
    const void* q_in; void* q_out;
    int64_t q_ts, q_hs, qo_ts, qo_hs;          // element strides (token, head)
    const void* key; const void* value;
    int64_t kv_ts, kv_hs;
    const void* cos_tab; const void* sin_tab;
    int64_t tab_stride, tab_rows;
    const int64_t* positions;                  // null: row t of the table belongs to token t
    void* k_pool; void* v_pool;
    const int64_t* slot_mapping;
    const float* k_scale; const float* v_scale;
    int64_t total;                             // T * (Hq + 2 Hkv) * D/16 lanes
    int hq, hkv, d, bs;
    int64_t num_slots;
};

template <typename T> struct Row8;
template <> struct Row8<bf16_t> {
    __device__ __forceinline__ static void load(const bf16_t* p, float* f) {
        Vec16<bf16_t>::unpack(*(const uint4*)p, f);
    }
    // gfx950 converts in hardware (v_cvt_pk_bf16_f32, round to nearest even)
    __device__ __forceinline__ static uint32_t pack2(float a, float b) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        const bf16x2 v = {(__bf16)a, (__bf16)b};
        return __builtin_bit_cast(uint32_t, v);
    }
    __device__ __forceinline__ static void store(bf16_t* p, const float* f) {
        *(uint4*)p = make_uint4(pack2(f[0], f[1]), pack2(f[2], f[3]), pack2(f[4], f[5]), pack2(f[6], f[7]));
    }
    // value as the tensor type holds it
    __device__ __forceinline__ static float round(float v) { return (float)(__bf16)v; }
};
template <> struct Row8<f16_t> {
    __device__ __forceinline__ static void load(const f16_t* p, float* f) {
        Vec16<f16_t>::unpack(*(const uint4*)p, f);
    }
    __device__ __forceinline__ static void store(f16_t* p, const float* f) {
        *(uint4*)p = make_uint4(F16Fmt::pack(f[0], f[1]), F16Fmt::pack(f[2], f[3]), F16Fmt::pack(f[4], f[5]),
                                F16Fmt::pack(f[6], f[7]));
    }
    __device__ __forceinline__ static float round(float v) { return (float)(_Float16)v; }
};
template <> struct Row8<float> {
    __device__ __forceinline__ static void load(const float* p, float* f) {
        const float4 a = ((const float4*)p)[0], b = ((const float4*)p)[1];
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    }
    __device__ __forceinline__ static void store(float* p, const float* f) {
        ((float4*)p)[0] = make_float4(f[0], f[1], f[2], f[3]);
        ((float4*)p)[1] = make_float4(f[4], f[5], f[6], f[7]);
    }
    __device__ __forceinline__ static float round(float v) { return v; }
};

// 8 floats -> 8 e4m3 codes: e4m3_rne(clamp(x / scale, +-448)), the plain append's rule
__device__ __forceinline__ uint2 quant8(const float* f, float scale) {
    float q[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = fminf(fmaxf(f[j] / scale, -448.f), 448.f);
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], hi, true);
    return make_uint2((uint32_t)lo, (uint32_t)hi);
}

// out = round(round(x * c) + round(r * s)), products and sum as separate roundings
template <typename T>
__device__ __forceinline__ float rot1(float x, float r, float c, float s) {
#pragma clang fp contract(off)
    const float p1 = Row8<T>::round(x * c);
    const float p2 = Row8<T>::round(r * s);
    return Row8<T>::round(p1 + p2);
}

template <typename T, bool FP8POOL>
__global__ void __launch_bounds__(256)
rope_kv_append_kernel(RopeParams p) {
    // 32-bit index arithmetic throughout (the launcher bounds the lane count and the slot range)
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= (uint32_t)p.total) return;
    const uint32_t chunks = (uint32_t)p.d / 16u;
    const uint32_t slots_per_tok = (uint32_t)(p.hq + 2 * p.hkv);
    const uint32_t lanes_per_tok = slots_per_tok * chunks;
    const uint32_t t = i / lanes_per_tok;
    const uint32_t rem = i - t * lanes_per_tok;
    const int hs = (int)(rem / chunks);
    const int c = (int)(rem - (uint32_t)hs * chunks);
    const int half = p.d / 2;
    const int lo_col = 8 * c, hi_col = half + 8 * c;

    const bool is_q = hs < p.hq;
    const bool is_k = !is_q && hs < p.hq + p.hkv;
    const int h = is_q ? hs : (is_k ? hs - p.hq : hs - p.hq - p.hkv);

    const int64_t pos = p.positions ? p.positions[t] : (int64_t)t;
    if (pos < 0 || pos >= p.tab_rows) return;                 // no table row: the token is left alone
    uint32_t blk = 0, off = 0;
    if (!is_q) {
        const int64_t slot = p.slot_mapping[t];
        if (slot < 0 || slot >= p.num_slots) return;          // padding row: nothing to store
        blk = (uint32_t)slot / (uint32_t)p.bs;
        off = (uint32_t)slot - blk * (uint32_t)p.bs;
    }
    const int64_t row = ((int64_t)blk * p.hkv + h) * p.bs + off;              // pool row of D elements

    const T* src = is_q ? (const T*)p.q_in + (int64_t)t * p.q_ts + h * p.q_hs
                        : (const T*)(is_k ? p.key : p.value) + (int64_t)t * p.kv_ts + h * p.kv_hs;
    if constexpr (!FP8POOL) {
        if (!is_q && !is_k) {                                 // V into a pool of its own type: raw bytes
            T* dst = (T*)p.v_pool + row * p.d;
            constexpr int V16 = 8 * sizeof(T) / 16;           // 16-byte vectors per 8 elements
#pragma unroll
            for (int k = 0; k < V16; ++k) {
                ((uint4*)(dst + lo_col))[k] = ((const uint4*)(src + lo_col))[k];
                ((uint4*)(dst + hi_col))[k] = ((const uint4*)(src + hi_col))[k];
            }
            return;
        }
    }
    float lo[8], hi[8];
    Row8<T>::load(src + lo_col, lo);
    Row8<T>::load(src + hi_col, hi);

    if (is_q || is_k) {
        const T* cr = (const T*)p.cos_tab + pos * p.tab_stride;
        const T* sr = (const T*)p.sin_tab + pos * p.tab_stride;
        float cl[8], ch[8], sl[8], sh[8], ol[8], oh[8];
        Row8<T>::load(cr + lo_col, cl);
        Row8<T>::load(cr + hi_col, ch);
        Row8<T>::load(sr + lo_col, sl);
        Row8<T>::load(sr + hi_col, sh);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            ol[j] = rot1<T>(lo[j], -hi[j], cl[j], sl[j]);     // rotate_half: (-x2, x1)
            oh[j] = rot1<T>(hi[j], lo[j], ch[j], sh[j]);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) { lo[j] = ol[j]; hi[j] = oh[j]; }
    }

    if (is_q) {
        T* dst = (T*)p.q_out + (int64_t)t * p.qo_ts + h * p.qo_hs;
        Row8<T>::store(dst + lo_col, lo);
        Row8<T>::store(dst + hi_col, hi);
        return;
    }
    if constexpr (FP8POOL) {
        const float sc = (is_k ? p.k_scale : p.v_scale)[h];
        uint8_t* dst = (uint8_t*)(is_k ? p.k_pool : p.v_pool) + row * p.d;
        *(uint2*)(dst + lo_col) = quant8(lo, sc);
        *(uint2*)(dst + hi_col) = quant8(hi, sc);
    } else {
        T* dst = (T*)(is_k ? p.k_pool : p.v_pool) + row * p.d;
        Row8<T>::store(dst + lo_col, lo);
        Row8<T>::store(dst + hi_col, hi);
    }
}

}  // namespace

int launch_rope_kv_append(const void* q_in, void* q_out, int64_t q_ts, int64_t q_hs, int64_t qo_ts,
                          int64_t qo_hs, const void* key, const void* value, int64_t kv_ts,
                          int64_t kv_hs, const void* cos_tab, const void* sin_tab, int64_t tab_stride,
                          int64_t tab_rows, const int64_t* positions, void* k_pool, void* v_pool,
                          const int64_t* slot_mapping, int64_t num_tokens, int hq, int hkv, int d, int bs,
                          int64_t num_blocks, int in_dtype, int pool_dtype, const float* k_scale,
                          const float* v_scale, hipStream_t stream) {
    RopeParams p;
    p.q_in = q_in; p.q_out = q_out; p.q_ts = q_ts; p.q_hs = q_hs; p.qo_ts = qo_ts; p.qo_hs = qo_hs;
    p.key = key; p.value = value; p.kv_ts = kv_ts; p.kv_hs = kv_hs;
    p.cos_tab = cos_tab; p.sin_tab = sin_tab; p.tab_stride = tab_stride; p.tab_rows = tab_rows;
    p.positions = positions; p.k_pool = k_pool; p.v_pool = v_pool; p.slot_mapping = slot_mapping;
    p.k_scale = k_scale; p.v_scale = v_scale;
    p.hq = hq; p.hkv = hkv; p.d = d; p.bs = bs;
    p.num_slots = num_blocks * bs;
    p.total = num_tokens * (hq + 2 * hkv) * (d / 16);
    AICOMP_REQUIRE(p.total < (int64_t)1 << 31 && p.num_slots < (int64_t)1 << 31, AICOMP_KV_EINVAL,
                   "rope_kv_append: %lld tokens / %lld slots exceed one launch's 32-bit index range",
                   (long long)num_tokens, (long long)p.num_slots);
    const int64_t blocks = (p.total + 255) / 256;
    const bool fp8 = pool_dtype == AICOMP_KV_FP8_E4M3;
    dim3 grid((unsigned)blocks), block(256);
    if (in_dtype == AICOMP_KV_BF16) {
        if (fp8) hipLaunchKernelGGL((rope_kv_append_kernel<bf16_t, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((rope_kv_append_kernel<bf16_t, false>), grid, block, 0, stream, p);
    } else if (in_dtype == AICOMP_KV_F16) {
        if (fp8) hipLaunchKernelGGL((rope_kv_append_kernel<f16_t, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((rope_kv_append_kernel<f16_t, false>), grid, block, 0, stream, p);
    } else {
        if (fp8) hipLaunchKernelGGL((rope_kv_append_kernel<float, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((rope_kv_append_kernel<float, false>), grid, block, 0, stream, p);
    }
    AICOMP_HIP_LAUNCH_CHECK();
    return AICOMP_KV_OK;
}

}  // namespace aicomp
