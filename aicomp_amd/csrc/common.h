// Shared device/host helpers for the paged KV-cache attention kernels (gfx950).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/aicomp_kv.h"

namespace aicomp {

// ---------------------------------------------------------------- errors ---
void set_error(const char* fmt, ...);

#define AICOMP_REQUIRE(cond, code, ...)                 \
    do {                                                \
        if (!(cond)) {                                  \
            ::aicomp::set_error(__VA_ARGS__);           \
            return (code);                              \
        }                                               \
    } while (0)

#define AICOMP_HIP_LAUNCH_CHECK()                                              \
    do {                                                                       \
        hipError_t e__ = hipGetLastError();                                    \
        if (e__ != hipSuccess) {                                               \
            ::aicomp::set_error("HIP launch failed: %s", hipGetErrorString(e__)); \
            return AICOMP_KV_EHIP;                                             \
        }                                                                      \
    } while (0)

inline int dtype_size(int dt) {
    switch (dt) {
        case AICOMP_KV_F32: return 4;
        case AICOMP_KV_BF16: return 2;
        case AICOMP_KV_F16: return 2;
        case AICOMP_KV_FP8_E4M3: return 1;
        default: return 0;
    }
}

// --------------------------------------------------------- element types ---
struct bf16_t { uint16_t bits; };
struct f16_t { uint16_t bits; };
struct fp8_t { uint8_t bits; };

inline bool is_16bit_float(int dt) { return dt == AICOMP_KV_BF16 || dt == AICOMP_KV_F16; }

constexpr int WAVE = 64;
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
    return __uint_as_float(((uint32_t)b) << 16);
}

// round-to-nearest-even, NaN kept quiet (same rule as torch's bfloat16 cast)
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// IEEE binary16 <-> float (hardware conversions, round to nearest even; what torch's cast does)
__device__ __forceinline__ float f16_to_f32(uint16_t b) {
    return (float)__builtin_bit_cast(_Float16, b);
}
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
    return __builtin_bit_cast(uint16_t, (_Float16)f);
}

// OCP e4m3 code -> float: gfx950's hardware conversion (byte 0 of the word)
__device__ __forceinline__ float fp8_to_f32(uint8_t c) {
    return __builtin_amdgcn_cvt_f32_fp8((int)c, 0);
}

// 16 raw bytes -> floats, by storage type
template <typename T> struct Vec16;

template <> struct Vec16<float> {
    static constexpr int N = 4;
    __device__ __forceinline__ static void unpack(const uint4& r, float* f) {
        f[0] = __uint_as_float(r.x); f[1] = __uint_as_float(r.y);
        f[2] = __uint_as_float(r.z); f[3] = __uint_as_float(r.w);
    }
};
template <> struct Vec16<bf16_t> {
    static constexpr int N = 8;
    __device__ __forceinline__ static void unpack(const uint4& r, float* f) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
};
template <> struct Vec16<f16_t> {
    static constexpr int N = 8;
    __device__ __forceinline__ static void unpack(const uint4& r, float* f) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = f16_to_f32((uint16_t)(w[i] & 0xffffu));
            f[2 * i + 1] = f16_to_f32((uint16_t)(w[i] >> 16));
        }
    }
};
template <> struct Vec16<fp8_t> {
    static constexpr int N = 16;
    __device__ __forceinline__ static void unpack(const uint4& r, float* f) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            auto lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], false);
            auto hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], true);
            f[4 * i] = lo[0]; f[4 * i + 1] = lo[1];
            f[4 * i + 2] = hi[0]; f[4 * i + 3] = hi[1];
        }
    }
};

template <typename T> __device__ __forceinline__ float load_elem(const T* p);
template <> __device__ __forceinline__ float load_elem<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_elem<bf16_t>(const bf16_t* p) { return bf16_to_f32(p->bits); }
template <> __device__ __forceinline__ float load_elem<f16_t>(const f16_t* p) { return f16_to_f32(p->bits); }

template <typename T> __device__ __forceinline__ void store_elem(T* p, float v);
template <> __device__ __forceinline__ void store_elem<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_elem<bf16_t>(bf16_t* p, float v) { p->bits = f32_to_bf16(v); }
template <> __device__ __forceinline__ void store_elem<f16_t>(f16_t* p, float v) { p->bits = f32_to_f16(v); }

// ------------------------------------- 16-bit formats of the matrix-core kernels ---
// The decode and prefill kernels are written once over a 16-bit element format: operands travel
// as raw 128-bit words, and everything that depends on the format (the MFMA instruction, the
// float <-> element conversions, fp8 widening, the pair sum) goes through one of these.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

struct Bf16Fmt {
    typedef bf16_t elem;
    static constexpr int DT = AICOMP_KV_BF16;
    // D[16x16] += A[16x32] * B[32x16]: v_mfma_f32_16x16x32_bf16
    __device__ __forceinline__ static f32x4_t mfma(const uint4& a, const uint4& b, const f32x4_t& c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                       __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    // two floats -> two packed elements, round to nearest even (v_cvt_pk_bf16_f32)
    __device__ __forceinline__ static uint32_t pack(float lo, float hi) {
        const bf16x2_t p = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, p);
    }
    __device__ __forceinline__ static float to_f32(uint16_t b) { return bf16_to_f32(b); }
    __device__ __forceinline__ static uint16_t from_f32(float f) { return f32_to_bf16(f); }
    // 8 e4m3 codes -> 8 elements, exact (3 mantissa bits); the scale operand is 1.0
    __device__ __forceinline__ static uint4 from_fp8(const uint2& r) {
        uint4 o;
        o.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(r.x, 1.0f, false));
        o.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(r.x, 1.0f, true));
        o.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(r.y, 1.0f, false));
        o.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(r.y, 1.0f, true));
        return o;
    }
    // acc + lo + hi of a packed pair (v_dot2c_f32_bf16 against a pair of ones)
    __device__ __forceinline__ static float pair_sum(uint32_t pp, float acc) {
        const bf16x2_t one = {(__bf16)1.0f, (__bf16)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pp), one, acc, false);
    }
    static constexpr uint32_t SIGN_PAIR = 0x80008000u;
};

struct F16Fmt {
    typedef f16_t elem;
    static constexpr int DT = AICOMP_KV_F16;
    __device__ __forceinline__ static f32x4_t mfma(const uint4& a, const uint4& b, const f32x4_t& c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                      __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    __device__ __forceinline__ static uint32_t pack(float lo, float hi) {       // v_cvt_pk_f16_f32
        const f16x2_t p = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, p);
    }
    __device__ __forceinline__ static float to_f32(uint16_t b) { return f16_to_f32(b); }
    __device__ __forceinline__ static uint16_t from_f32(float f) { return f32_to_f16(f); }
    __device__ __forceinline__ static uint4 from_fp8(const uint2& r) {
        uint4 o;
        o.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(r.x, 1.0f, false));
        o.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(r.x, 1.0f, true));
        o.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(r.y, 1.0f, false));
        o.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(r.y, 1.0f, true));
        return o;
    }
    __device__ __forceinline__ static float pair_sum(uint32_t pp, float acc) {  // v_dot2c_f32_f16
        const f16x2_t one = {(_Float16)1.0f, (_Float16)1.0f};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, pp), one, acc, false);
    }
    static constexpr uint32_t SIGN_PAIR = 0x80008000u;
};

// --------------------------------------- order of query tiles in a prefill grid ---
// A prefill grid is (head group, sequence, query tile slice), dispatched x fastest: the first
// num_cus workgroups land one per CU, the next num_cus beside them, the rest as places free up.
// A query tile of a causal chunk costs as many steps as it has keys, so tile index = cost order.
// A grid of at most two workgroups per CU is resident all at once, so which two share a CU decides
// when the kernel ends: its slices are handed out in rounds of num_cus workgroups, the first from
// the expensive end downwards and the second from the cheap end upwards, so that the two
// workgroups of a CU are the p-th most expensive and the p-th cheapest tile (a fresh 2048-token
// prompt is 512 workgroups: expensive first, CU 0 gets tiles 63 and 31 and CU 255 tiles 32 and 0;
// this way every CU gets 63 steps: 482 -> 382 us for such a float32 prompt).  Larger grids are
// dispatched as places free up, and there expensive first is the better order (an 8192-token
// prompt: 470 us against 498 us zig-zag).  Returns the tile of slice z (a bijection of 0 .. Z-1
// for any Z).
__device__ __forceinline__ int prefill_tile_of_slice(int z, int Z, int num_cus, int wgs_per_slice) {
    if (num_cus <= 0 || wgs_per_slice <= 0 || num_cus % wgs_per_slice != 0 || Z * wgs_per_slice > 2 * num_cus)
        return Z - 1 - z;
    const int per_round = num_cus / wgs_per_slice;
    const int k = z / per_round, pos = z - k * per_round;
    return (k & 1) ? (k >> 1) * per_round + pos : Z - 1 - (k >> 1) * per_round - pos;
}

// ------------------------------------------------- split-K workspace view ---
// part_acc [rows][Hq][P][D] float : sum_j 2^(s_j - m) v_j   (not normalised)
// part_ml  [rows][Hq][P][2] float : m (log2 domain), l = sum_j 2^(s_j - m)
// Every slot a merge reads has been written by the same call: no initialisation needed.
struct SplitWorkspace {
    float* acc;
    float* ml;
};

inline size_t split_workspace_bytes(int64_t rows, int hq, int hkv, int d, int parts) {
    (void)hkv;
    return (size_t)rows * hq * parts * (size_t)(d + 2) * sizeof(float);
}
inline SplitWorkspace split_workspace_view(void* ws, int64_t rows, int hq, int hkv, int d, int parts) {
    (void)hkv;
    SplitWorkspace v;
    v.acc = (float*)ws;
    v.ml = v.acc + (size_t)rows * hq * parts * d;
    return v;
}

// ------------------------------------------------------- kernel launchers ---
struct DecodeArgs {
    void* out;
    const void* query;
    const void* k_pool;
    const void* v_pool;
    const int32_t* block_table;
    int64_t block_table_stride;
    const int32_t* context_lens;
    const int32_t* cu_q_lens;   // NULL: one query row per sequence (decode)
    int num_seqs;
    int64_t rows;               // query rows (== num_seqs for decode)
    int hq, hkv, d, bs, max_blocks;
    int64_t num_blocks;
    float scale;
    int q_dtype, kv_dtype;
    const float* k_scale;
    const float* v_scale;
    int partition_size;         // tokens, multiple of bs
    int num_parts;              // ceil(max_blocks*bs / partition_size)
    SplitWorkspace ws;
    hipStream_t stream;
    // fused append of one new token per sequence (decode only; NULL = none)
    const void* new_key;
    const void* new_value;
    int64_t new_token_stride, new_head_stride;
    // prefill only (NULL = none): (sequence, query tile) pairs, one workgroup row each, in the order
    // the workgroups are to take them
    const int32_t* items;
    int num_items;
};

int launch_decode_generic(const DecodeArgs& a);
bool decode_mfma_supported(const DecodeArgs& a);
int launch_decode_mfma(const DecodeArgs& a);
bool decode_streamk_supported(const DecodeArgs& a);
size_t decode_streamk_workspace_bytes(int64_t rows, int hq, int hkv, int d);
int launch_decode_streamk(const DecodeArgs& a, void* workspace);
int launch_kv_append_last(const void* key, const void* value, int64_t token_stride, int64_t head_stride,
                          void* k_pool, void* v_pool, const int32_t* block_table,
                          int64_t block_table_stride, const int32_t* context_lens, int batch, int hkv,
                          int d, int bs, int max_blocks, int64_t num_blocks, int in_dtype,
                          int pool_dtype, const float* k_scale, const float* v_scale,
                          hipStream_t stream);
int launch_split_reduce(const DecodeArgs& a);
int launch_sample(int64_t* out, const void* logits, int64_t row_stride, float* probs_out,
                  const float* uniforms, int batch, int vocab, float temperature, int top_k, float top_p,
                  int greedy, int dtype, hipStream_t stream);
int launch_rope_kv_append(const void* q_in, void* q_out, int64_t q_ts, int64_t q_hs, int64_t qo_ts,
                          int64_t qo_hs, const void* key, const void* value, int64_t kv_ts,
                          int64_t kv_hs, const void* cos_tab, const void* sin_tab, int64_t tab_stride,
                          int64_t tab_rows, const int64_t* positions, void* k_pool, void* v_pool,
                          const int64_t* slot_mapping, int64_t num_tokens, int hq, int hkv, int d, int bs,
                          int64_t num_blocks, int in_dtype, int pool_dtype, const float* k_scale,
                          const float* v_scale, hipStream_t stream);

}  // namespace aicomp
