// extern "C" entry points: argument validation and kernel dispatch.
// The declarations, with the reference interfaces they replace, are in
// include/aicomp_kv.h.
#include "common.h"

#include <stdlib.h>
#include <string.h>

#include <atomic>

// Split-K scratch of aicomp_paged_decode_attn_append_static: device memory that belongs to the
// loaded library, one copy per GPU, held until the process ends.  In host code this name is only
// a handle for hipGetSymbolAddress: the address a kernel may use is what that call returns.
static __device__ __align__(256) unsigned char scratch[AICOMP_KV_STATIC_SCRATCH_BYTES];

namespace aicomp {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int launch_kv_append(const void* key, const void* value, int64_t token_stride, int64_t head_stride,
                     void* k_pool, void* v_pool, const int64_t* slot_mapping, int64_t T, int hkv,
                     int d, int bs, int64_t num_blocks, int in_dtype, int pool_dtype,
                     const float* k_scale, const float* v_scale, hipStream_t stream);

bool prefill_mfma_supported(const DecodeArgs& a, int max_q_len);
int launch_prefill_mfma(const DecodeArgs& a, int max_q_len);
int prefill_mfma_tile_positions(int hq, int hkv, int max_q_len);
int prefill_mfma_f32_tile_positions(int hq, int hkv);
bool prefill_mfma_f32_supported(const DecodeArgs& a, int max_q_len);
int launch_prefill_mfma_f32(const DecodeArgs& a, int max_q_len);
bool prefill_tiled_supported(const DecodeArgs& a, int max_q_len);
int launch_prefill_tiled(const DecodeArgs& a, int max_q_len);

static int check_common(int hq, int hkv, int d, int bs, int max_blocks, int64_t num_blocks,
                        int q_dtype, int kv_dtype, const float* k_scale, const float* v_scale,
                        const char* who) {
    AICOMP_REQUIRE(hq > 0 && hkv > 0 && hq % hkv == 0, AICOMP_KV_EINVAL,
                   "%s: %d query heads are not a multiple of %d KV heads", who, hq, hkv);
    AICOMP_REQUIRE(d > 0 && bs > 0 && max_blocks >= 0 && num_blocks > 0, AICOMP_KV_EINVAL,
                   "%s: bad sizes (head_dim %d, block_size %d, max_blocks %d, num_blocks %lld)",
                   who, d, bs, max_blocks, (long long)num_blocks);
    AICOMP_REQUIRE(dtype_size(q_dtype) && dtype_size(kv_dtype), AICOMP_KV_EINVAL,
                   "%s: unknown element type (query %d, pool %d)", who, q_dtype, kv_dtype);
    if (kv_dtype == AICOMP_KV_FP8_E4M3)
        AICOMP_REQUIRE(k_scale && v_scale, AICOMP_KV_EINVAL,
                       "%s: an fp8 pool needs k_scale and v_scale", who);
    return AICOMP_KV_OK;
}

// shapes the balanced schedule and the matrix-core grid schedule both take
static bool streamk_shape(int batch, int hq, int hkv, int d, int bs, int q_dtype, int kv_dtype) {
    return ((d == 128 && hq / hkv <= 16) || (d == 64 && hq / hkv <= 8)) && bs == 16 && is_16bit_float(q_dtype) &&
           (kv_dtype == q_dtype || kv_dtype == AICOMP_KV_FP8_E4M3) && batch <= 1024;
}

// A decode call over few, short rows is a chain of launch and memory latencies, not a stream: the
// balanced schedule (set up for 256 CUs of work, always followed by its merge kernel) then loses to
// one workgroup per (row, KV head, partition) on the grid schedule, without any merge kernel when
// no row can be longer than 640 tokens (measured on 1 to 16 rows of 512 and 2048 tokens: 5.4-8.5
// against 9-13 us, 8-15 against 11-17 us).  "Small" is rows x (table width x block size) at or
// below a process-wide threshold: 32768 by default, or the value of the environment variable
// AICOMP_KV_SMALL_DECODE_TOKENS when the library first needs it (read once, never again), or what
// aicomp_kv_set_small_decode_tokens() stored last (0 keeps every automatic call of a supported
// shape on the balanced schedule).  The sizing helpers and the decode calls read the same word.
static std::atomic<long long>& small_decode_tokens() {
    static std::atomic<long long> limit{[] {
        const char* e = getenv("AICOMP_KV_SMALL_DECODE_TOKENS");
        return e ? atoll(e) : 32768LL;
    }()};
    return limit;
}

static bool small_call(int64_t rows, int bs, int max_blocks) {
    return rows * (int64_t)max_blocks * bs <= small_decode_tokens().load(std::memory_order_relaxed);
}

static int auto_partition(int64_t rows, int hkv, int bs, int max_blocks, bool matrix_shape) {
    // Longer partitions amortise a workgroup's start-up and merge; shorter ones give the
    // 256 CUs enough workgroups when there are few (sequence, KV head) rows.
    const int64_t max_ctx = (int64_t)max_blocks * bs;
    int ps;
    if (matrix_shape && small_call(rows, bs, max_blocks)) {
        // matrix-core grid schedule: whole rows (a whole number of its 64-token tiles), or 256 tokens
        ps = max_ctx <= 640 ? (int)((max_ctx + 63) / 64 * 64) : 256;
    } else {
        ps = 64;       // vector-ALU kernel on few short rows: spread the call wide
        for (int cand : {1024, 512, 256, 128}) {
            if (rows * hkv * ((max_ctx + cand - 1) / cand) >= 1024) { ps = cand; break; }
        }
    }
    ps = (ps + bs - 1) / bs * bs;
    return ps;
}

}  // namespace aicomp

using namespace aicomp;

extern "C" {

int aicomp_kv_version(void) { return 200; }

const char* aicomp_kv_last_error(void) { return g_err; }

long long aicomp_kv_set_small_decode_tokens(long long tokens) {
    std::atomic<long long>& limit = small_decode_tokens();
    return tokens < 0 ? limit.load(std::memory_order_relaxed) : limit.exchange(tokens, std::memory_order_relaxed);
}

int aicomp_kv_append(const void* key, const void* value, int64_t kv_token_stride,
                     int64_t kv_head_stride, void* k_pool, void* v_pool,
                     const int64_t* slot_mapping, int64_t num_tokens, int num_kv_heads,
                     int head_dim, int block_size, int64_t num_blocks, int in_dtype,
                     int pool_dtype, const float* k_scale, const float* v_scale, void* stream) {
    AICOMP_REQUIRE(num_tokens >= 0, AICOMP_KV_EINVAL, "kv_append: negative token count");
    if (num_tokens == 0) return AICOMP_KV_OK;
    AICOMP_REQUIRE(key && value && k_pool && v_pool && slot_mapping, AICOMP_KV_EINVAL,
                   "kv_append: null pointer");
    AICOMP_REQUIRE(num_kv_heads > 0 && head_dim > 0 && block_size > 0 && num_blocks > 0,
                   AICOMP_KV_EINVAL, "kv_append: bad sizes (Hkv %d, D %d, BS %d, blocks %lld)",
                   num_kv_heads, head_dim, block_size, (long long)num_blocks);
    AICOMP_REQUIRE(dtype_size(in_dtype) && dtype_size(pool_dtype), AICOMP_KV_EINVAL,
                   "kv_append: unknown element type (in %d, pool %d)", in_dtype, pool_dtype);
    AICOMP_REQUIRE(kv_head_stride >= head_dim && kv_token_stride >= 0, AICOMP_KV_EINVAL,
                   "kv_append: strides (%lld, %lld) overlap rows of %d elements",
                   (long long)kv_token_stride, (long long)kv_head_stride, head_dim);
    return launch_kv_append(key, value, kv_token_stride, kv_head_stride, k_pool, v_pool,
                            slot_mapping, num_tokens, num_kv_heads, head_dim, block_size,
                            num_blocks, in_dtype, pool_dtype, k_scale, v_scale,
                            (hipStream_t)stream);
}

int aicomp_rope_kv_append(const void* q_in, void* q_out, int64_t q_token_stride,
                          int64_t q_head_stride, int64_t qo_token_stride, int64_t qo_head_stride,
                          const void* key, const void* value, int64_t kv_token_stride,
                          int64_t kv_head_stride, const void* cos, const void* sin,
                          int64_t table_stride, int64_t table_rows, const int64_t* positions,
                          void* k_pool, void* v_pool, const int64_t* slot_mapping,
                          int64_t num_tokens, int num_q_heads, int num_kv_heads, int head_dim,
                          int block_size, int64_t num_blocks, int in_dtype, int pool_dtype,
                          const float* k_scale, const float* v_scale, void* stream) {
    AICOMP_REQUIRE(num_tokens >= 0, AICOMP_KV_EINVAL, "rope_kv_append: negative token count");
    if (num_tokens == 0) return AICOMP_KV_OK;
    AICOMP_REQUIRE(q_in && q_out && key && value && cos && sin && k_pool && v_pool && slot_mapping,
                   AICOMP_KV_EINVAL, "rope_kv_append: null pointer");
    AICOMP_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && head_dim > 0 && block_size > 0 &&
                   num_blocks > 0 && table_rows > 0, AICOMP_KV_EINVAL,
                   "rope_kv_append: bad sizes (Hq %d, Hkv %d, D %d, BS %d, blocks %lld, table rows %lld)",
                   num_q_heads, num_kv_heads, head_dim, block_size, (long long)num_blocks,
                   (long long)table_rows);
    AICOMP_REQUIRE(in_dtype == AICOMP_KV_F32 || is_16bit_float(in_dtype), AICOMP_KV_EUNSUPPORTED,
                   "rope_kv_append: inputs must be float32, bfloat16 or float16 (got %d)", in_dtype);
    AICOMP_REQUIRE(pool_dtype == in_dtype || pool_dtype == AICOMP_KV_FP8_E4M3, AICOMP_KV_EUNSUPPORTED,
                   "rope_kv_append: pool type %d must be the input type %d or fp8-e4m3", pool_dtype,
                   in_dtype);
    AICOMP_REQUIRE(pool_dtype != AICOMP_KV_FP8_E4M3 || (k_scale && v_scale), AICOMP_KV_EINVAL,
                   "rope_kv_append: an fp8 pool needs k_scale and v_scale");
    AICOMP_REQUIRE(head_dim % 16 == 0, AICOMP_KV_EUNSUPPORTED,
                   "rope_kv_append: head_dim %d is not a multiple of 16", head_dim);
    const int64_t v = 16 / dtype_size(in_dtype);       // elements per 16 bytes
    AICOMP_REQUIRE(q_head_stride >= head_dim && qo_head_stride >= head_dim &&
                   kv_head_stride >= head_dim && table_stride >= head_dim && q_token_stride >= 0 &&
                   qo_token_stride >= 0 && kv_token_stride >= 0, AICOMP_KV_EINVAL,
                   "rope_kv_append: strides overlap rows of %d elements", head_dim);
    AICOMP_REQUIRE(q_token_stride % v == 0 && q_head_stride % v == 0 && qo_token_stride % v == 0 &&
                   qo_head_stride % v == 0 && kv_token_stride % v == 0 && kv_head_stride % v == 0 &&
                   table_stride % v == 0, AICOMP_KV_EUNSUPPORTED,
                   "rope_kv_append: strides must be multiples of %lld elements (16 bytes)", (long long)v);
    AICOMP_REQUIRE(((uintptr_t)q_in | (uintptr_t)q_out | (uintptr_t)key | (uintptr_t)value |
                    (uintptr_t)cos | (uintptr_t)sin | (uintptr_t)k_pool | (uintptr_t)v_pool) % 16 == 0,
                   AICOMP_KV_EUNSUPPORTED, "rope_kv_append: pointers must be 16-byte aligned");
    return launch_rope_kv_append(q_in, q_out, q_token_stride, q_head_stride, qo_token_stride,
                                 qo_head_stride, key, value, kv_token_stride, kv_head_stride, cos, sin,
                                 table_stride, table_rows, positions, k_pool, v_pool, slot_mapping,
                                 num_tokens, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks,
                                 in_dtype, pool_dtype, k_scale, v_scale, (hipStream_t)stream);
}

int aicomp_sample_tokens(int64_t* out, const void* logits, int64_t row_stride, float* probs_out,
                         const float* uniforms, int batch, int vocab, float temperature, int top_k,
                         float top_p, int greedy, int logits_dtype, void* stream) {
    AICOMP_REQUIRE(batch >= 0, AICOMP_KV_EINVAL, "sample_tokens: negative batch");
    if (batch == 0) return AICOMP_KV_OK;
    AICOMP_REQUIRE(out && logits, AICOMP_KV_EINVAL, "sample_tokens: null pointer");
    AICOMP_REQUIRE(vocab > 0 && row_stride >= vocab, AICOMP_KV_EINVAL,
                   "sample_tokens: bad sizes (vocab %d, row stride %lld)", vocab, (long long)row_stride);
    AICOMP_REQUIRE(logits_dtype == AICOMP_KV_F32 || is_16bit_float(logits_dtype), AICOMP_KV_EUNSUPPORTED,
                   "sample_tokens: logits must be float32, bfloat16 or float16 (got %d)", logits_dtype);
    if (!greedy) {
        AICOMP_REQUIRE(uniforms, AICOMP_KV_EINVAL, "sample_tokens: sampling needs uniforms");
        AICOMP_REQUIRE(temperature > 0.f, AICOMP_KV_EINVAL,
                       "sample_tokens: temperature must be positive (got %g)", (double)temperature);
        AICOMP_REQUIRE(top_p == top_p, AICOMP_KV_EINVAL, "sample_tokens: top_p is NaN");
    }
    return launch_sample(out, logits, row_stride, probs_out, uniforms, batch, vocab, temperature, top_k,
                         top_p, greedy ? 1 : 0, logits_dtype, (hipStream_t)stream);
}

int aicomp_paged_decode_partition_size(int batch, int num_q_heads, int num_kv_heads, int head_dim,
                                       int block_size, int max_blocks_per_seq, int q_dtype,
                                       int kv_dtype) {
    if (batch <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 || block_size <= 0 || max_blocks_per_seq <= 0) return 0;
    return auto_partition(batch, num_kv_heads, block_size, max_blocks_per_seq,
                          streamk_shape(batch, num_q_heads, num_kv_heads, head_dim, block_size, q_dtype, kv_dtype));
}

static int resolve_parts(int64_t rows, int hkv, int bs, int max_blocks, bool matrix_shape, int& partition_size) {
    if (partition_size <= 0) partition_size = auto_partition(rows, hkv, bs, max_blocks, matrix_shape);
    const int64_t max_ctx = (int64_t)max_blocks * bs;
    int64_t parts = (max_ctx + partition_size - 1) / partition_size;
    return (int)(parts < 1 ? 1 : parts);
}

size_t aicomp_paged_decode_workspace_bytes(int batch, int num_q_heads, int num_kv_heads,
                                           int head_dim, int block_size, int max_blocks_per_seq,
                                           int q_dtype, int kv_dtype, int partition_size) {
    if (batch <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || block_size <= 0 ||
        max_blocks_per_seq <= 0 || num_q_heads % num_kv_heads)
        return 0;
    const bool automatic = partition_size <= 0;
    const bool matrix_shape = streamk_shape(batch, num_q_heads, num_kv_heads, head_dim, block_size, q_dtype, kv_dtype);
    const int parts = resolve_parts(batch, num_kv_heads, block_size, max_blocks_per_seq, matrix_shape, partition_size);
    size_t need = parts <= 1 ? 0 : split_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim, parts);
    if (automatic && matrix_shape && !small_call(batch, block_size, max_blocks_per_seq)) {
        const size_t sk = decode_streamk_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim);
        if (sk > need) need = sk;
    }
    return need;
}

static int decode_impl(void* out, const void* query, const void* new_key, const void* new_value,
                       int64_t kv_token_stride, int64_t kv_head_stride, void* k_pool, void* v_pool,
                       const int32_t* block_table, int64_t block_table_stride,
                       const int32_t* context_lens, int batch, int num_q_heads, int num_kv_heads,
                       int head_dim, int block_size, int max_blocks_per_seq, int64_t num_blocks,
                       float scale, int q_dtype, int kv_dtype, const float* k_scale,
                       const float* v_scale, int partition_size, void* workspace,
                       size_t workspace_bytes, void* stream, const char* who) {
    AICOMP_REQUIRE(batch >= 0, AICOMP_KV_EINVAL, "%s: negative batch", who);
    if (batch == 0) return AICOMP_KV_OK;
    AICOMP_REQUIRE(out && query && k_pool && v_pool && block_table && context_lens,
                   AICOMP_KV_EINVAL, "%s: null pointer", who);
    int rc = check_common(num_q_heads, num_kv_heads, head_dim, block_size, max_blocks_per_seq,
                          num_blocks, q_dtype, kv_dtype, k_scale, v_scale, who);
    if (rc) return rc;
    AICOMP_REQUIRE(max_blocks_per_seq > 0 && block_table_stride >= max_blocks_per_seq,
                   AICOMP_KV_EINVAL, "%s: block table stride %lld < width %d", who,
                   (long long)block_table_stride, max_blocks_per_seq);
    AICOMP_REQUIRE(partition_size >= 0 && partition_size % block_size == 0, AICOMP_KV_EINVAL,
                   "%s: partition_size %d is not a multiple of block_size %d", who, partition_size,
                   block_size);
    const bool fused = new_key != nullptr;
    if (fused)
        AICOMP_REQUIRE(new_value && kv_head_stride >= head_dim && kv_token_stride >= 0, AICOMP_KV_EINVAL,
                       "%s: bad new_key / new_value arguments", who);
    DecodeArgs a;
    memset(&a, 0, sizeof(a));
    a.out = out; a.query = query; a.k_pool = k_pool; a.v_pool = v_pool;
    a.block_table = block_table; a.block_table_stride = block_table_stride;
    a.context_lens = context_lens; a.cu_q_lens = nullptr;
    a.num_seqs = batch; a.rows = batch;
    a.hq = num_q_heads; a.hkv = num_kv_heads; a.d = head_dim; a.bs = block_size;
    a.max_blocks = max_blocks_per_seq; a.num_blocks = num_blocks;
    a.scale = scale; a.q_dtype = q_dtype; a.kv_dtype = kv_dtype;
    a.k_scale = kv_dtype == AICOMP_KV_FP8_E4M3 ? k_scale : nullptr;
    a.v_scale = kv_dtype == AICOMP_KV_FP8_E4M3 ? v_scale : nullptr;
    a.partition_size = partition_size;
    const bool matrix_shape = streamk_shape(batch, num_q_heads, num_kv_heads, head_dim, block_size, q_dtype, kv_dtype);
    a.num_parts = resolve_parts(batch, num_kv_heads, block_size, max_blocks_per_seq, matrix_shape, a.partition_size);
    a.stream = (hipStream_t)stream;
    // the matrix-core kernels append the new rows themselves when they can read them 16 bytes at a time
    const bool injectable = fused && is_16bit_float(q_dtype) && kv_token_stride % 8 == 0 &&
                            kv_head_stride % 8 == 0 && (uintptr_t)new_key % 16 == 0 &&
                            (uintptr_t)new_value % 16 == 0;
    if (partition_size == 0 && decode_streamk_supported(a) && !small_call(batch, block_size, max_blocks_per_seq)) {
        // balanced schedule: equal tile counts per wave, merged by a second kernel
        const size_t need = decode_streamk_workspace_bytes(a.rows, a.hq, a.hkv, a.d);
        AICOMP_REQUIRE(workspace && workspace_bytes >= need, AICOMP_KV_EWORKSPACE,
                       "%s: workspace of %zu bytes needed, %zu given", who, need,
                       workspace ? workspace_bytes : (size_t)0);
        AICOMP_REQUIRE((uintptr_t)workspace % 16 == 0, AICOMP_KV_EINVAL,
                       "%s: workspace must be 16-byte aligned", who);
        const bool in_kernel = injectable;
        if (fused && !in_kernel) {
            rc = launch_kv_append_last(new_key, new_value, kv_token_stride, kv_head_stride, k_pool, v_pool,
                                       block_table, block_table_stride, context_lens, batch,
                                       num_kv_heads, head_dim, block_size, max_blocks_per_seq,
                                       num_blocks, q_dtype, kv_dtype, k_scale, v_scale, a.stream);
            if (rc) return rc;
        }
        if (in_kernel) {
            a.new_key = new_key; a.new_value = new_value;
            a.new_token_stride = kv_token_stride; a.new_head_stride = kv_head_stride;
        }
        return launch_decode_streamk(a, workspace);
    }
    const bool mfma = decode_mfma_supported(a);
    const bool in_kernel = injectable && mfma;
    if (in_kernel) {
        a.new_key = new_key; a.new_value = new_value;
        a.new_token_stride = kv_token_stride; a.new_head_stride = kv_head_stride;
    } else if (fused) {
        rc = launch_kv_append_last(new_key, new_value, kv_token_stride, kv_head_stride, k_pool, v_pool,
                                   block_table, block_table_stride, context_lens, batch, num_kv_heads,
                                   head_dim, block_size, max_blocks_per_seq, num_blocks, q_dtype,
                                   kv_dtype, k_scale, v_scale, a.stream);
        if (rc) return rc;
    }
    if (a.num_parts > 1) {
        const size_t need = split_workspace_bytes(a.rows, a.hq, a.hkv, a.d, a.num_parts);
        AICOMP_REQUIRE(workspace && workspace_bytes >= need, AICOMP_KV_EWORKSPACE,
                       "%s: workspace of %zu bytes needed, %zu given", who, need,
                       workspace ? workspace_bytes : (size_t)0);
        AICOMP_REQUIRE((uintptr_t)workspace % 16 == 0, AICOMP_KV_EINVAL,
                       "%s: workspace must be 16-byte aligned", who);
        a.ws = split_workspace_view(workspace, a.rows, a.hq, a.hkv, a.d, a.num_parts);
    }
    if (mfma) return launch_decode_mfma(a);
    return launch_decode_generic(a);
}

int aicomp_paged_decode_attn(void* out, const void* query, const void* k_pool, const void* v_pool,
                             const int32_t* block_table, int64_t block_table_stride,
                             const int32_t* context_lens, int batch, int num_q_heads,
                             int num_kv_heads, int head_dim, int block_size,
                             int max_blocks_per_seq, int64_t num_blocks, float scale, int q_dtype,
                             int kv_dtype, const float* k_scale, const float* v_scale,
                             int partition_size, void* workspace, size_t workspace_bytes,
                             void* stream) {
    return decode_impl(out, query, nullptr, nullptr, 0, 0, (void*)k_pool, (void*)v_pool, block_table,
                       block_table_stride, context_lens, batch, num_q_heads, num_kv_heads, head_dim,
                       block_size, max_blocks_per_seq, num_blocks, scale, q_dtype, kv_dtype, k_scale,
                       v_scale, partition_size, workspace, workspace_bytes, stream,
                       "paged_decode_attn");
}

int aicomp_paged_decode_attn_append(void* out, const void* query, const void* new_key,
                                    const void* new_value, int64_t kv_token_stride,
                                    int64_t kv_head_stride, void* k_pool, void* v_pool,
                                    const int32_t* block_table, int64_t block_table_stride,
                                    const int32_t* context_lens, int batch, int num_q_heads,
                                    int num_kv_heads, int head_dim, int block_size,
                                    int max_blocks_per_seq, int64_t num_blocks, float scale,
                                    int q_dtype, int kv_dtype, const float* k_scale,
                                    const float* v_scale, int partition_size, void* workspace,
                                    size_t workspace_bytes, void* stream) {
    AICOMP_REQUIRE(batch <= 0 || (new_key && new_value), AICOMP_KV_EINVAL,
                   "paged_decode_attn_append: null new_key / new_value");
    return decode_impl(out, query, new_key, new_value, kv_token_stride, kv_head_stride, k_pool, v_pool,
                       block_table, block_table_stride, context_lens, batch, num_q_heads, num_kv_heads,
                       head_dim, block_size, max_blocks_per_seq, num_blocks, scale, q_dtype, kv_dtype,
                       k_scale, v_scale, partition_size, workspace, workspace_bytes, stream,
                       "paged_decode_attn_append");
}

// Device address of `scratch` on the current device, looked up once per device.
static int static_scratch(void** ptr, const char* who) {
    constexpr int MAX_DEVICES = 64;
    static std::atomic<void*> per_device[MAX_DEVICES];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        set_error("%s: cannot identify the current device (%d)", who, dev);
        return AICOMP_KV_EHIP;
    }
    void* p = per_device[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr) {
            set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev,
                      hipGetErrorString(e));
            return AICOMP_KV_EHIP;
        }
        per_device[dev].store(p, std::memory_order_release);     // racing threads store the same address
    }
    *ptr = p;
    return AICOMP_KV_OK;
}

int aicomp_paged_decode_attn_append_static(void* out, const void* query, const void* new_key,
                                           const void* new_value, int64_t kv_token_stride,
                                           int64_t kv_head_stride, void* k_pool, void* v_pool,
                                           const int32_t* block_table, int64_t block_table_stride,
                                           const int32_t* context_lens, int batch, int num_q_heads,
                                           int num_kv_heads, int head_dim, int block_size,
                                           int max_blocks_per_seq, int64_t num_blocks, float scale,
                                           int q_dtype, int kv_dtype, const float* k_scale,
                                           const float* v_scale, int partition_size, void* stream) {
    const char* who = "paged_decode_attn_append_static";
    AICOMP_REQUIRE(batch <= 0 || (new_key && new_value), AICOMP_KV_EINVAL, "%s: null new_key / new_value", who);
    const size_t need = aicomp_paged_decode_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim,
                                                            block_size, max_blocks_per_seq, q_dtype,
                                                            kv_dtype, partition_size);
    AICOMP_REQUIRE(need <= (size_t)AICOMP_KV_STATIC_SCRATCH_BYTES, AICOMP_KV_EWORKSPACE,
                   "%s: this shape needs %zu bytes of split-K scratch, the built-in scratch holds %zu; "
                   "use aicomp_paged_decode_attn_append with a workspace of the caller's", who, need,
                   (size_t)AICOMP_KV_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    if (need > 0) {
        const int rc = static_scratch(&ws, who);
        if (rc) return rc;
    }
    return decode_impl(out, query, new_key, new_value, kv_token_stride, kv_head_stride, k_pool, v_pool,
                       block_table, block_table_stride, context_lens, batch, num_q_heads, num_kv_heads,
                       head_dim, block_size, max_blocks_per_seq, num_blocks, scale, q_dtype, kv_dtype,
                       k_scale, v_scale, partition_size, ws, need, stream, who);
}

static int prefill_impl(void* out, const void* query, const void* k_pool, const void* v_pool,
                        const int32_t* block_table, int64_t block_table_stride,
                        const int32_t* context_lens, const int32_t* cu_q_lens, int num_seqs,
                        int64_t total_q, int max_q_len, int num_q_heads, int num_kv_heads,
                        int head_dim, int block_size, int max_blocks_per_seq,
                        int64_t num_blocks, float scale, int q_dtype, int kv_dtype,
                        const float* k_scale, const float* v_scale, const int32_t* items, int num_items,
                        void* stream) {
    AICOMP_REQUIRE(num_seqs >= 0 && total_q >= 0, AICOMP_KV_EINVAL,
                   "paged_prefill_attn: negative sizes");
    if (num_seqs == 0 || total_q == 0) return AICOMP_KV_OK;
    AICOMP_REQUIRE(out && query && k_pool && v_pool && block_table && context_lens && cu_q_lens,
                   AICOMP_KV_EINVAL, "paged_prefill_attn: null pointer");
    int rc = check_common(num_q_heads, num_kv_heads, head_dim, block_size, max_blocks_per_seq,
                          num_blocks, q_dtype, kv_dtype, k_scale, v_scale, "paged_prefill_attn");
    if (rc) return rc;
    AICOMP_REQUIRE(max_q_len > 0 && max_q_len <= total_q, AICOMP_KV_EINVAL,
                   "paged_prefill_attn: max_q_len %d out of range (total %lld)", max_q_len,
                   (long long)total_q);
    AICOMP_REQUIRE(max_blocks_per_seq > 0 && block_table_stride >= max_blocks_per_seq,
                   AICOMP_KV_EINVAL, "paged_prefill_attn: block table stride %lld < width %d",
                   (long long)block_table_stride, max_blocks_per_seq);
    AICOMP_REQUIRE(items == nullptr || num_items > 0, AICOMP_KV_EINVAL,
                   "paged_prefill_attn: an item list needs at least one item");
    DecodeArgs a;
    memset(&a, 0, sizeof(a));
    a.out = out; a.query = query; a.k_pool = k_pool; a.v_pool = v_pool;
    a.block_table = block_table; a.block_table_stride = block_table_stride;
    a.context_lens = context_lens; a.cu_q_lens = cu_q_lens;
    a.num_seqs = num_seqs; a.rows = total_q;
    a.hq = num_q_heads; a.hkv = num_kv_heads; a.d = head_dim; a.bs = block_size;
    a.max_blocks = max_blocks_per_seq; a.num_blocks = num_blocks;
    a.scale = scale; a.q_dtype = q_dtype; a.kv_dtype = kv_dtype;
    a.k_scale = kv_dtype == AICOMP_KV_FP8_E4M3 ? k_scale : nullptr;
    a.v_scale = kv_dtype == AICOMP_KV_FP8_E4M3 ? v_scale : nullptr;
    a.stream = (hipStream_t)stream;
    // an item list is taken by the two matrix-instruction kernels (and only while its length fits a
    // grid dimension); the other kernels walk the whole grid, which covers the same tiles
    if (items != nullptr && num_items <= 65535) { a.items = items; a.num_items = num_items; }
    if (prefill_mfma_supported(a, max_q_len)) return launch_prefill_mfma(a, max_q_len);
    // float32 models at head_dim 64 / 128: the float32 matrix instruction
    if (prefill_mfma_f32_supported(a, max_q_len)) return launch_prefill_mfma_f32(a, max_q_len);
    // head_dim 256, other block sizes: the tiled vector-ALU kernel (K/V staged in LDS once per 32
    // query rows)
    if (prefill_tiled_supported(a, max_q_len)) return launch_prefill_tiled(a, max_q_len);
    // what is left (pools that cannot be read 16 bytes at a time): every query row as its own
    // unsplit attention problem over its causal prefix
    a.partition_size = (int)(((int64_t)max_blocks_per_seq * block_size + block_size - 1) /
                             block_size * block_size);
    a.num_parts = 1;
    return launch_decode_generic(a);
}

int aicomp_paged_prefill_attn(void* out, const void* query, const void* k_pool, const void* v_pool,
                              const int32_t* block_table, int64_t block_table_stride,
                              const int32_t* context_lens, const int32_t* cu_q_lens, int num_seqs,
                              int64_t total_q, int max_q_len, int num_q_heads, int num_kv_heads,
                              int head_dim, int block_size, int max_blocks_per_seq,
                              int64_t num_blocks, float scale, int q_dtype, int kv_dtype,
                              const float* k_scale, const float* v_scale, void* stream) {
    return prefill_impl(out, query, k_pool, v_pool, block_table, block_table_stride, context_lens, cu_q_lens,
                        num_seqs, total_q, max_q_len, num_q_heads, num_kv_heads, head_dim, block_size,
                        max_blocks_per_seq, num_blocks, scale, q_dtype, kv_dtype, k_scale, v_scale, nullptr, 0,
                        stream);
}

int aicomp_paged_prefill_attn_items(void* out, const void* query, const void* k_pool, const void* v_pool,
                                    const int32_t* block_table, int64_t block_table_stride,
                                    const int32_t* context_lens, const int32_t* cu_q_lens, int num_seqs,
                                    int64_t total_q, int max_q_len, int num_q_heads, int num_kv_heads,
                                    int head_dim, int block_size, int max_blocks_per_seq,
                                    int64_t num_blocks, float scale, int q_dtype, int kv_dtype,
                                    const float* k_scale, const float* v_scale, const int32_t* items,
                                    int num_items, void* stream) {
    AICOMP_REQUIRE(num_items >= 0 && (items != nullptr || num_items == 0), AICOMP_KV_EINVAL,
                   "paged_prefill_attn_items: %d items without a list", num_items);
    return prefill_impl(out, query, k_pool, v_pool, block_table, block_table_stride, context_lens, cu_q_lens,
                        num_seqs, total_q, max_q_len, num_q_heads, num_kv_heads, head_dim, block_size,
                        max_blocks_per_seq, num_blocks, scale, q_dtype, kv_dtype, k_scale, v_scale,
                        num_items > 0 ? items : nullptr, num_items, stream);
}

int aicomp_paged_prefill_tile_positions(int num_q_heads, int num_kv_heads, int head_dim, int block_size,
                                        int q_dtype, int kv_dtype, int max_q_len) {
    if (num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads || max_q_len <= 0 || block_size != 16 ||
        (head_dim != 64 && head_dim != 128))
        return 0;
    if (is_16bit_float(q_dtype) && (kv_dtype == q_dtype || kv_dtype == AICOMP_KV_FP8_E4M3))
        return prefill_mfma_tile_positions(num_q_heads, num_kv_heads, max_q_len);
    if (q_dtype == AICOMP_KV_F32 && kv_dtype == AICOMP_KV_F32)
        return prefill_mfma_f32_tile_positions(num_q_heads, num_kv_heads);
    return 0;
}

}  // extern "C"
