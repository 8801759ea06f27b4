// KV-cache append: scatter new K/V rows into the paged pools by slot_mapping.
//
// Replaces the reference's slice assignment
//   key_cache[:, :, position:end_position, :] = new_k     opt_prime/opt_prime/kv_cache.py:159-160
//   self.cache_k[:, :, self.cache_pos:end_pos, :] = key   opt_prime/opt_prime/kv_cache.py:387-388
// Pure byte copy when the storage types agree (bit-exact); with an fp8 pool the
// row is quantised on the way in.
//
// HBM-bound, tiny: per token it reads 2*Hkv*D*e_in and writes 2*Hkv*D*e_pool
// bytes.  One lane moves 16 bytes; a (token, head) row of D*e bytes is written
// by consecutive lanes, so every store is a full 128-bit, fully coalesced
// access to one contiguous pool row.
#include "common.h"

namespace aicomp {

// raw copy, 16 bytes per lane.  chunks_per_row = D*e/16.
__global__ void __launch_bounds__(256)
kv_append_copy16(const uint4* __restrict__ key, const uint4* __restrict__ value,
                 int64_t token_stride16, int64_t head_stride16,   // in 16-byte units
                 uint4* __restrict__ k_pool, uint4* __restrict__ v_pool,
                 const int64_t* __restrict__ slot_mapping,
                 int64_t total, int hkv, int chunks_per_row, int bs, int64_t num_slots) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    int c = (int)(i % chunks_per_row);
    int64_t r = i / chunks_per_row;
    int h = (int)(r % hkv);
    int64_t t = r / hkv;
    int64_t slot = slot_mapping[t];
    if (slot < 0 || slot >= num_slots) return;   // padding row, or out of the pool: skipped
    int64_t blk = slot / bs;
    int off = (int)(slot % bs);
    int64_t src = t * token_stride16 + h * head_stride16 + c;
    int64_t dst = ((blk * hkv + h) * bs + off) * chunks_per_row + c;
    k_pool[dst] = key[src];
    v_pool[dst] = value[src];
}

// raw copy, element by element (rows that are not 16-byte aligned)
template <typename T>
__global__ void __launch_bounds__(256)
kv_append_copy_elem(const T* __restrict__ key, const T* __restrict__ value,
                    int64_t token_stride, int64_t head_stride,
                    T* __restrict__ k_pool, T* __restrict__ v_pool,
                    const int64_t* __restrict__ slot_mapping,
                    int64_t total, int hkv, int d, int bs, int64_t num_slots) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    int c = (int)(i % d);
    int64_t r = i / d;
    int h = (int)(r % hkv);
    int64_t t = r / hkv;
    int64_t slot = slot_mapping[t];
    if (slot < 0 || slot >= num_slots) return;
    int64_t blk = slot / bs;
    int off = (int)(slot % bs);
    int64_t src = t * token_stride + h * head_stride + c;
    int64_t dst = ((blk * hkv + h) * bs + off) * d + c;
    k_pool[dst] = key[src];
    v_pool[dst] = value[src];
}

// quantising append: code = e4m3_rne(clamp(x / scale[h], +-448)); 4 elements per lane
template <typename IN_T>
__global__ void __launch_bounds__(256)
kv_append_quant_fp8(const IN_T* __restrict__ key, const IN_T* __restrict__ value,
                    int64_t token_stride, int64_t head_stride,
                    uint32_t* __restrict__ k_pool, uint32_t* __restrict__ v_pool,
                    const int64_t* __restrict__ slot_mapping,
                    const float* __restrict__ k_scale, const float* __restrict__ v_scale,
                    int64_t total, int hkv, int d4, int bs, int64_t num_slots) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    int c = (int)(i % d4);
    int64_t r = i / d4;
    int h = (int)(r % hkv);
    int64_t t = r / hkv;
    int64_t slot = slot_mapping[t];
    if (slot < 0 || slot >= num_slots) return;
    int64_t blk = slot / bs;
    int off = (int)(slot % bs);
    int64_t src = t * token_stride + h * head_stride + 4 * c;
    int64_t dst = ((blk * hkv + h) * bs + off) * d4 + c;
    const float ks = k_scale[h], vs = v_scale[h];
    float kf[4], vf[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        kf[j] = fminf(fmaxf(load_elem<IN_T>(key + src + j) / ks, -448.f), 448.f);
        vf[j] = fminf(fmaxf(load_elem<IN_T>(value + src + j) / vs, -448.f), 448.f);
    }
    int kw = 0, vw = 0;
    kw = __builtin_amdgcn_cvt_pk_fp8_f32(kf[0], kf[1], kw, false);
    kw = __builtin_amdgcn_cvt_pk_fp8_f32(kf[2], kf[3], kw, true);
    vw = __builtin_amdgcn_cvt_pk_fp8_f32(vf[0], vf[1], vw, false);
    vw = __builtin_amdgcn_cvt_pk_fp8_f32(vf[2], vf[3], vw, true);
    k_pool[dst] = (uint32_t)kw;
    v_pool[dst] = (uint32_t)vw;
}

// Append of ONE token per sequence at position context_lens[b] - 1, slot taken from the
// block table on the device (no slot_mapping).  Used by the fused append+decode entry point
// for the shapes whose decode kernel does not do the append itself.
template <typename T>
__global__ void __launch_bounds__(256)
kv_append_last_copy(const T* __restrict__ key, const T* __restrict__ value, int64_t token_stride,
                    int64_t head_stride, T* __restrict__ k_pool, T* __restrict__ v_pool,
                    const int32_t* __restrict__ block_table, int64_t table_stride,
                    const int32_t* __restrict__ context_lens, int64_t total, int hkv, int d, int bs,
                    int max_blocks, int64_t num_blocks) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int c = (int)(i % d);
    const int64_t r = i / d;
    const int h = (int)(r % hkv);
    const int64_t b = r / hkv;
    const int pos = context_lens[b] - 1;
    if (pos < 0 || pos / bs >= max_blocks) return;
    const int64_t blk = block_table[b * table_stride + pos / bs];
    if (blk < 0 || blk >= num_blocks) return;
    const int64_t dst = ((blk * hkv + h) * bs + pos % bs) * d + c;
    const int64_t src = b * token_stride + h * head_stride + c;
    k_pool[dst] = key[src];
    v_pool[dst] = value[src];
}

template <typename IN_T>
__global__ void __launch_bounds__(256)
kv_append_last_quant(const IN_T* __restrict__ key, const IN_T* __restrict__ value, int64_t token_stride,
                     int64_t head_stride, uint32_t* __restrict__ k_pool, uint32_t* __restrict__ v_pool,
                     const int32_t* __restrict__ block_table, int64_t table_stride,
                     const int32_t* __restrict__ context_lens, const float* __restrict__ k_scale,
                     const float* __restrict__ v_scale, int64_t total, int hkv, int d4, int bs,
                     int max_blocks, int64_t num_blocks) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int c = (int)(i % d4);
    const int64_t r = i / d4;
    const int h = (int)(r % hkv);
    const int64_t b = r / hkv;
    const int pos = context_lens[b] - 1;
    if (pos < 0 || pos / bs >= max_blocks) return;
    const int64_t blk = block_table[b * table_stride + pos / bs];
    if (blk < 0 || blk >= num_blocks) return;
    const int64_t dst = ((blk * hkv + h) * bs + pos % bs) * d4 + c;
    const int64_t src = b * token_stride + h * head_stride + 4 * c;
    const float ks = k_scale[h], vs = v_scale[h];
    float kf[4], vf[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        kf[j] = fminf(fmaxf(load_elem<IN_T>(key + src + j) / ks, -448.f), 448.f);
        vf[j] = fminf(fmaxf(load_elem<IN_T>(value + src + j) / vs, -448.f), 448.f);
    }
    int kw = 0, vw = 0;
    kw = __builtin_amdgcn_cvt_pk_fp8_f32(kf[0], kf[1], kw, false);
    kw = __builtin_amdgcn_cvt_pk_fp8_f32(kf[2], kf[3], kw, true);
    vw = __builtin_amdgcn_cvt_pk_fp8_f32(vf[0], vf[1], vw, false);
    vw = __builtin_amdgcn_cvt_pk_fp8_f32(vf[2], vf[3], vw, true);
    k_pool[dst] = (uint32_t)kw;
    v_pool[dst] = (uint32_t)vw;
}

int launch_kv_append_last(const void* key, const void* value, int64_t token_stride, int64_t head_stride,
                          void* k_pool, void* v_pool, const int32_t* block_table,
                          int64_t block_table_stride, const int32_t* context_lens, int batch, int hkv,
                          int d, int bs, int max_blocks, int64_t num_blocks, int in_dtype,
                          int pool_dtype, const float* k_scale, const float* v_scale,
                          hipStream_t stream) {
    if (batch == 0) return AICOMP_KV_OK;
    const int threads = 256;
    if (in_dtype == pool_dtype) {
        const int64_t total = (int64_t)batch * hkv * d;
        const unsigned blocks = (unsigned)((total + threads - 1) / threads);
#define LAUNCH_LAST(TY)                                                                          \
    hipLaunchKernelGGL(kv_append_last_copy<TY>, dim3(blocks), dim3(threads), 0, stream,          \
                       (const TY*)key, (const TY*)value, token_stride, head_stride, (TY*)k_pool, \
                       (TY*)v_pool, block_table, block_table_stride, context_lens, total, hkv, d, \
                       bs, max_blocks, num_blocks)
        const int e = dtype_size(in_dtype);
        if (e == 4) LAUNCH_LAST(uint32_t);
        else if (e == 2) LAUNCH_LAST(uint16_t);
        else LAUNCH_LAST(uint8_t);
#undef LAUNCH_LAST
    } else {
        AICOMP_REQUIRE(pool_dtype == AICOMP_KV_FP8_E4M3 &&
                           (is_16bit_float(in_dtype) || in_dtype == AICOMP_KV_F32) && d % 4 == 0,
                       AICOMP_KV_EUNSUPPORTED, "append: only f32/bf16/f16 -> fp8 conversion is supported");
        AICOMP_REQUIRE(k_scale && v_scale, AICOMP_KV_EINVAL, "append: an fp8 pool needs k_scale and v_scale");
        const int64_t total = (int64_t)batch * hkv * (d / 4);
        const unsigned blocks = (unsigned)((total + threads - 1) / threads);
        if (in_dtype == AICOMP_KV_BF16)
            hipLaunchKernelGGL(kv_append_last_quant<bf16_t>, dim3(blocks), dim3(threads), 0, stream,
                               (const bf16_t*)key, (const bf16_t*)value, token_stride, head_stride,
                               (uint32_t*)k_pool, (uint32_t*)v_pool, block_table, block_table_stride,
                               context_lens, k_scale, v_scale, total, hkv, d / 4, bs, max_blocks, num_blocks);
        else if (in_dtype == AICOMP_KV_F16)
            hipLaunchKernelGGL(kv_append_last_quant<f16_t>, dim3(blocks), dim3(threads), 0, stream,
                               (const f16_t*)key, (const f16_t*)value, token_stride, head_stride,
                               (uint32_t*)k_pool, (uint32_t*)v_pool, block_table, block_table_stride,
                               context_lens, k_scale, v_scale, total, hkv, d / 4, bs, max_blocks, num_blocks);
        else
            hipLaunchKernelGGL(kv_append_last_quant<float>, dim3(blocks), dim3(threads), 0, stream,
                               (const float*)key, (const float*)value, token_stride, head_stride,
                               (uint32_t*)k_pool, (uint32_t*)v_pool, block_table, block_table_stride,
                               context_lens, k_scale, v_scale, total, hkv, d / 4, bs, max_blocks, num_blocks);
    }
    AICOMP_HIP_LAUNCH_CHECK();
    return AICOMP_KV_OK;
}

int launch_kv_append(const void* key, const void* value, int64_t token_stride, int64_t head_stride,
                     void* k_pool, void* v_pool, const int64_t* slot_mapping,
                     int64_t T, int hkv, int d, int bs, int64_t num_blocks,
                     int in_dtype, int pool_dtype, const float* k_scale, const float* v_scale,
                     hipStream_t stream) {
    if (T == 0) return AICOMP_KV_OK;
    const int64_t num_slots = num_blocks * bs;
    const int threads = 256;
    if (in_dtype == pool_dtype) {
        const int e = dtype_size(in_dtype);
        const bool aligned =
            (d * e) % 16 == 0 && (token_stride * e) % 16 == 0 && (head_stride * e) % 16 == 0 &&
            ((uintptr_t)key % 16 == 0) && ((uintptr_t)value % 16 == 0) &&
            ((uintptr_t)k_pool % 16 == 0) && ((uintptr_t)v_pool % 16 == 0);
        if (aligned) {
            const int cpr = d * e / 16;
            const int64_t total = T * hkv * cpr;
            const int64_t blocks = (total + threads - 1) / threads;
            AICOMP_REQUIRE(blocks < (1ll << 31), AICOMP_KV_EINVAL, "kv_append: too many rows");
            hipLaunchKernelGGL(kv_append_copy16, dim3((unsigned)blocks), dim3(threads), 0, stream,
                               (const uint4*)key, (const uint4*)value, token_stride * e / 16,
                               head_stride * e / 16, (uint4*)k_pool, (uint4*)v_pool, slot_mapping,
                               total, hkv, cpr, bs, num_slots);
        } else {
            const int64_t total = T * hkv * d;
            const int64_t blocks = (total + threads - 1) / threads;
            AICOMP_REQUIRE(blocks < (1ll << 31), AICOMP_KV_EINVAL, "kv_append: too many rows");
#define LAUNCH_ELEM(TY)                                                                       \
    hipLaunchKernelGGL(kv_append_copy_elem<TY>, dim3((unsigned)blocks), dim3(threads), 0,     \
                       stream, (const TY*)key, (const TY*)value, token_stride, head_stride,   \
                       (TY*)k_pool, (TY*)v_pool, slot_mapping, total, hkv, d, bs, num_slots)
            if (e == 4) LAUNCH_ELEM(uint32_t);
            else if (e == 2) LAUNCH_ELEM(uint16_t);
            else LAUNCH_ELEM(uint8_t);
#undef LAUNCH_ELEM
        }
    } else {
        AICOMP_REQUIRE(pool_dtype == AICOMP_KV_FP8_E4M3 &&
                           (is_16bit_float(in_dtype) || in_dtype == AICOMP_KV_F32),
                       AICOMP_KV_EUNSUPPORTED,
                       "kv_append: only f32/bf16/f16 -> fp8 conversion is supported (in %d, pool %d)",
                       in_dtype, pool_dtype);
        AICOMP_REQUIRE(k_scale && v_scale, AICOMP_KV_EINVAL,
                       "kv_append: an fp8 pool needs k_scale and v_scale");
        AICOMP_REQUIRE(d % 4 == 0, AICOMP_KV_EUNSUPPORTED, "kv_append: fp8 needs head_dim %% 4 == 0");
        const int64_t total = T * hkv * (d / 4);
        const int64_t blocks = (total + threads - 1) / threads;
        AICOMP_REQUIRE(blocks < (1ll << 31), AICOMP_KV_EINVAL, "kv_append: too many rows");
        if (in_dtype == AICOMP_KV_BF16)
            hipLaunchKernelGGL(kv_append_quant_fp8<bf16_t>, dim3((unsigned)blocks), dim3(threads), 0,
                               stream, (const bf16_t*)key, (const bf16_t*)value, token_stride,
                               head_stride, (uint32_t*)k_pool, (uint32_t*)v_pool, slot_mapping,
                               k_scale, v_scale, total, hkv, d / 4, bs, num_slots);
        else if (in_dtype == AICOMP_KV_F16)
            hipLaunchKernelGGL(kv_append_quant_fp8<f16_t>, dim3((unsigned)blocks), dim3(threads), 0,
                               stream, (const f16_t*)key, (const f16_t*)value, token_stride,
                               head_stride, (uint32_t*)k_pool, (uint32_t*)v_pool, slot_mapping,
                               k_scale, v_scale, total, hkv, d / 4, bs, num_slots);
        else
            hipLaunchKernelGGL(kv_append_quant_fp8<float>, dim3((unsigned)blocks), dim3(threads), 0,
                               stream, (const float*)key, (const float*)value, token_stride,
                               head_stride, (uint32_t*)k_pool, (uint32_t*)v_pool, slot_mapping,
                               k_scale, v_scale, total, hkv, d / 4, bs, num_slots);
    }
    AICOMP_HIP_LAUNCH_CHECK();
    return AICOMP_KV_OK;
}

}  // namespace aicomp
