// PyTorch operator registration over the C ABI of libaicomp_kv.so:
//
//   torch.ops.mi355_kv.kv_append / paged_decode_attn / paged_decode_attn_append /
//   paged_prefill_attn / decode_step
//
// The library itself has no torch types in its interface (include/aicomp_kv.h); this file is
// the thin host layer a PyTorch caller goes through instead of ctypes: tensors are checked the
// way TORCH_CHECK does (RuntimeError on dtype / shape / contiguity / device mismatch), raw
// device pointers and the CURRENT HIP stream go to the C entry points, nothing synchronises.
// All ops are in place on `out` and the pools; the only allocations are decode_step's output
// tensor and, for decode calls that were not handed a workspace, a scratch buffer per stream that
// is kept and grown as needed.
//
// decode_step is the reference operator's decode call in one dispatch: the tensors exactly as
// CachedScaledDotProductAttention.forward receives them (opt_prime/opt_prime/kv_cache.py:340-349,
// query [B, Hq, 1, D], key / value [B, H, 1, D] with H = Hkv or Hkv * group as HF's repeat_kv
// leaves them) -> append at `position` + attention over position + 1 tokens
// (kv_cache.py:372-403) -> [B, Hq, 1, D].
#include <ATen/ATen.h>
#include <ATen/hip/HIPContext.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <utility>

#include "../../include/aicomp_kv.h"

namespace {

int dtype_code(const at::Tensor& t, const char* what) {
    switch (t.scalar_type()) {
        case at::kFloat: return AICOMP_KV_F32;
        case at::kBFloat16: return AICOMP_KV_BF16;
        case at::kHalf: return AICOMP_KV_F16;
        case at::kFloat8_e4m3fn: return AICOMP_KV_FP8_E4M3;
        default: TORCH_CHECK(false, what, ": unsupported dtype ", t.scalar_type(),
                             " (float32, bfloat16, float16, float8_e4m3fn)");
    }
    return -1;
}

void check_rc(int rc) {
    TORCH_CHECK(rc == AICOMP_KV_OK, "aicomp_kv error ", rc, ": ", aicomp_kv_last_error());
}

void* stream_of(const at::Tensor& t) {
    return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

struct Pools {
    int64_t nb;
    int hkv, bs, d;
};

Pools check_pools(const at::Tensor& k_pool, const at::Tensor& v_pool) {
    TORCH_CHECK(k_pool.is_cuda(), "tensors must live on a ROCm device (there is no CPU path)");
    TORCH_CHECK(k_pool.dim() == 4 && v_pool.sizes() == k_pool.sizes(),
                "pools must both be [num_blocks, Hkv, BS, D]; got ", k_pool.sizes(), " and ", v_pool.sizes());
    TORCH_CHECK(k_pool.scalar_type() == v_pool.scalar_type(), "k_pool and v_pool dtypes differ");
    TORCH_CHECK(k_pool.is_contiguous() && v_pool.is_contiguous(), "pools must be contiguous");
    TORCH_CHECK(v_pool.device() == k_pool.device(), "v_pool is on ", v_pool.device(), ", expected ", k_pool.device());
    return {k_pool.size(0), (int)k_pool.size(1), (int)k_pool.size(2), (int)k_pool.size(3)};
}

// k_scale / v_scale pointers of an fp8 pool (checked), nullptr otherwise
void scales(const at::Tensor& pool, const c10::optional<at::Tensor>& ks, const c10::optional<at::Tensor>& vs,
            int hkv, const float*& kp, const float*& vp) {
    kp = vp = nullptr;
    if (pool.scalar_type() != at::kFloat8_e4m3fn) return;
    TORCH_CHECK(ks.has_value() && vs.has_value(), "an fp8 pool needs k_scale and v_scale");
    for (const at::Tensor* s : {&*ks, &*vs})
        TORCH_CHECK(s->scalar_type() == at::kFloat && s->is_contiguous() && s->numel() == hkv &&
                    s->device() == pool.device(),
                    "k_scale / v_scale must be contiguous float32 tensors of ", hkv, " elements on ", pool.device());
    kp = ks->data_ptr<float>();
    vp = vs->data_ptr<float>();
}

void check_table(const at::Tensor& block_table, const at::Tensor& context_lens, int64_t rows, const at::Tensor& ref) {
    TORCH_CHECK(block_table.scalar_type() == at::kInt && block_table.dim() == 2 && block_table.size(0) == rows &&
                block_table.stride(1) == 1 && block_table.device() == ref.device(),
                "block_table must be int32 [", rows, ", max_blocks] on ", ref.device(), ", rows contiguous");
    TORCH_CHECK(context_lens.scalar_type() == at::kInt && context_lens.numel() == rows && context_lens.is_contiguous() &&
                context_lens.device() == ref.device(),
                "context_lens must be contiguous int32 [", rows, "] on ", ref.device());
}

void kv_append(const at::Tensor& key, const at::Tensor& value, at::Tensor& k_pool, at::Tensor& v_pool,
               const at::Tensor& slot_mapping, const c10::optional<at::Tensor>& k_scale,
               const c10::optional<at::Tensor>& v_scale) {
    const Pools p = check_pools(k_pool, v_pool);
    const c10::DeviceGuard guard(k_pool.device());          // launches go to the tensors' device, whatever is current
    TORCH_CHECK(key.dim() == 3 && key.sizes() == value.sizes() && key.scalar_type() == value.scalar_type(),
                "key/value must both be [T, Hkv, D]; got ", key.sizes(), " and ", value.sizes());
    TORCH_CHECK(key.size(1) == p.hkv && key.size(2) == p.d, "key is ", key.sizes(), " but the pool holds [", p.hkv,
                ", ", p.d, "] rows");
    TORCH_CHECK(slot_mapping.scalar_type() == at::kLong && slot_mapping.dim() == 1 &&
                slot_mapping.numel() == key.size(0) && slot_mapping.is_contiguous(),
                "slot_mapping must be a contiguous int64 vector with one entry per row");
    TORCH_CHECK(value.device() == key.device() && k_pool.device() == key.device() && slot_mapping.device() == key.device(),
                "key, value, pools and slot_mapping must be on one device");
    const float *ks = nullptr, *vs = nullptr;
    if (key.scalar_type() != k_pool.scalar_type()) scales(k_pool, k_scale, v_scale, p.hkv, ks, vs);
    at::Tensor k = key, v = value;
    if (k.stride(2) != 1 || k.strides() != v.strides()) { k = k.contiguous(); v = v.contiguous(); }
    check_rc(aicomp_kv_append(k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1), k_pool.data_ptr(),
                              v_pool.data_ptr(), slot_mapping.data_ptr<int64_t>(), k.size(0), p.hkv, p.d, p.bs, p.nb,
                              dtype_code(k, "key"), dtype_code(k_pool, "pool"), ks, vs, stream_of(k)));
}

// Scratch the ops keep for callers that pass none: one growing buffer per (device, stream), like
// the Python wrappers'.  A decode call's scratch needs no initialisation and holds nothing between
// calls, and calls on one stream run one after the other, so reuse is safe.  The map is never
// destroyed (tensors freed at process exit, after the allocator, would fault).
at::Tensor& cached_scratch(const at::Tensor& ref, size_t bytes) {
    static std::mutex mu;
    static auto* table = new std::map<std::pair<int, void*>, at::Tensor>();
    std::lock_guard<std::mutex> lock(mu);
    at::Tensor& t = (*table)[{(int)ref.device().index(), stream_of(ref)}];
    if (!t.defined() || (size_t)t.numel() < bytes) t = at::empty({(int64_t)bytes}, ref.options().dtype(at::kByte));
    return t;
}

// scratch of a decode call: the caller's, or the ops' own buffer of the size the library asks for
void* decode_workspace(const c10::optional<at::Tensor>& workspace, at::Tensor& own, const at::Tensor& ref,
                       int B, int hq, const Pools& p, int max_blocks, int qd, int kd, int partition_size,
                       size_t& bytes) {
    if (workspace.has_value()) {
        TORCH_CHECK(workspace->device() == ref.device() && workspace->is_contiguous(), "workspace must be a contiguous tensor on ", ref.device());
        bytes = (size_t)workspace->numel() * workspace->element_size();
        return workspace->data_ptr();
    }
    bytes = aicomp_paged_decode_workspace_bytes(B, hq, p.hkv, p.d, p.bs, max_blocks, qd, kd, partition_size);
    if (bytes == 0) return nullptr;
    own = cached_scratch(ref, bytes);
    bytes = (size_t)own.numel();
    return own.data_ptr();
}

void decode_impl(at::Tensor& out, const at::Tensor& query, const at::Tensor* new_key, const at::Tensor* new_value,
                 const at::Tensor& k_pool, const at::Tensor& v_pool, const at::Tensor& block_table,
                 const at::Tensor& context_lens, double scale, const c10::optional<at::Tensor>& k_scale,
                 const c10::optional<at::Tensor>& v_scale, int64_t partition_size,
                 const c10::optional<at::Tensor>& workspace) {
    const Pools p = check_pools(k_pool, v_pool);
    const c10::DeviceGuard guard(k_pool.device());
    TORCH_CHECK(query.dim() == 3 && out.sizes() == query.sizes() && out.scalar_type() == query.scalar_type(),
                "out/query must both be [B, Hq, D]; got ", out.sizes(), " and ", query.sizes());
    const int B = (int)query.size(0), hq = (int)query.size(1);
    TORCH_CHECK(query.size(2) == p.d, "query head_dim ", query.size(2), " != pool head_dim ", p.d);
    TORCH_CHECK(query.is_contiguous() && out.is_contiguous(), "query and out must be contiguous");
    TORCH_CHECK(out.device() == query.device() && k_pool.device() == query.device(), "out, query and pools must be on one device");
    check_table(block_table, context_lens, B, query);
    const float *ks, *vs;
    scales(k_pool, k_scale, v_scale, p.hkv, ks, vs);
    const int qd = dtype_code(query, "query"), kd = dtype_code(k_pool, "pool");
    at::Tensor own;
    size_t ws_bytes = 0;
    void* ws = decode_workspace(workspace, own, query, B, hq, p, (int)block_table.size(1), qd, kd, (int)partition_size, ws_bytes);
    if (new_key == nullptr) {
        check_rc(aicomp_paged_decode_attn(out.data_ptr(), query.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(),
                                          block_table.data_ptr<int32_t>(), block_table.stride(0),
                                          context_lens.data_ptr<int32_t>(), B, hq, p.hkv, p.d, p.bs,
                                          (int)block_table.size(1), p.nb, (float)scale, qd, kd, ks, vs,
                                          (int)partition_size, ws, ws_bytes, stream_of(query)));
        return;
    }
    at::Tensor nk = *new_key, nv = *new_value;
    TORCH_CHECK(nk.dim() == 3 && nk.size(0) == B && nk.size(1) == p.hkv && nk.size(2) == p.d && nv.sizes() == nk.sizes() &&
                nk.scalar_type() == query.scalar_type() && nv.scalar_type() == query.scalar_type() &&
                nk.device() == query.device() && nv.device() == query.device(),
                "new_key/new_value must both be [", B, ", ", p.hkv, ", ", p.d, "] of the query dtype on ", query.device());
    if (nk.stride(2) != 1 || nk.strides() != nv.strides()) { nk = nk.contiguous(); nv = nv.contiguous(); }
    check_rc(aicomp_paged_decode_attn_append(out.data_ptr(), query.data_ptr(), nk.data_ptr(), nv.data_ptr(), nk.stride(0),
                                             nk.stride(1), k_pool.data_ptr(), v_pool.data_ptr(),
                                             block_table.data_ptr<int32_t>(), block_table.stride(0),
                                             context_lens.data_ptr<int32_t>(), B, hq, p.hkv, p.d, p.bs,
                                             (int)block_table.size(1), p.nb, (float)scale, qd, kd, ks, vs,
                                             (int)partition_size, ws, ws_bytes, stream_of(query)));
}

void paged_decode_attn(at::Tensor& out, const at::Tensor& query, const at::Tensor& k_pool, const at::Tensor& v_pool,
                       const at::Tensor& block_table, const at::Tensor& context_lens, double scale,
                       const c10::optional<at::Tensor>& k_scale, const c10::optional<at::Tensor>& v_scale,
                       int64_t partition_size, const c10::optional<at::Tensor>& workspace) {
    decode_impl(out, query, nullptr, nullptr, k_pool, v_pool, block_table, context_lens, scale, k_scale, v_scale,
                partition_size, workspace);
}

void paged_decode_attn_append(at::Tensor& out, const at::Tensor& query, const at::Tensor& new_key,
                              const at::Tensor& new_value, at::Tensor& k_pool, at::Tensor& v_pool,
                              const at::Tensor& block_table, const at::Tensor& context_lens, double scale,
                              const c10::optional<at::Tensor>& k_scale, const c10::optional<at::Tensor>& v_scale,
                              int64_t partition_size, const c10::optional<at::Tensor>& workspace) {
    decode_impl(out, query, &new_key, &new_value, k_pool, v_pool, block_table, context_lens, scale, k_scale, v_scale,
                partition_size, workspace);
}

void paged_prefill_attn(at::Tensor& out, const at::Tensor& query, const at::Tensor& k_pool, const at::Tensor& v_pool,
                        const at::Tensor& block_table, const at::Tensor& context_lens, const at::Tensor& cu_q_lens,
                        double scale, int64_t max_q_len, const c10::optional<at::Tensor>& k_scale,
                        const c10::optional<at::Tensor>& v_scale, const c10::optional<at::Tensor>& items) {
    const Pools p = check_pools(k_pool, v_pool);
    const c10::DeviceGuard guard(k_pool.device());
    TORCH_CHECK(query.dim() == 3 && out.sizes() == query.sizes() && out.scalar_type() == query.scalar_type(),
                "out/query must both be [T, Hq, D]; got ", out.sizes(), " and ", query.sizes());
    TORCH_CHECK(query.size(2) == p.d, "query head_dim ", query.size(2), " != pool head_dim ", p.d);
    TORCH_CHECK(query.is_contiguous() && out.is_contiguous(), "query and out must be contiguous");
    TORCH_CHECK(out.device() == query.device() && k_pool.device() == query.device(), "out, query and pools must be on one device");
    const int64_t S = context_lens.numel();
    check_table(block_table, context_lens, S, query);
    TORCH_CHECK(cu_q_lens.scalar_type() == at::kInt && cu_q_lens.numel() == S + 1 && cu_q_lens.is_contiguous() &&
                cu_q_lens.device() == query.device(), "cu_q_lens must be contiguous int32 [S+1] on ", query.device());
    TORCH_CHECK(max_q_len > 0 || query.size(0) == 0, "max_q_len must be the host-side bound on the chunk lengths");
    const float *ks, *vs;
    scales(k_pool, k_scale, v_scale, p.hkv, ks, vs);
    const int32_t* item_ptr = nullptr;
    int num_items = 0;
    if (items.has_value() && items->numel() > 0) {
        TORCH_CHECK(items->scalar_type() == at::kInt && items->dim() == 2 && items->size(1) == 2 && items->is_contiguous() &&
                    items->device() == query.device(),
                    "items must be a contiguous int32 [n, 2] tensor of (sequence, query tile) pairs on ", query.device());
        item_ptr = items->data_ptr<int32_t>();
        num_items = (int)items->size(0);
    }
    check_rc(aicomp_paged_prefill_attn_items(out.data_ptr(), query.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(),
                                             block_table.data_ptr<int32_t>(), block_table.stride(0),
                                             context_lens.data_ptr<int32_t>(), cu_q_lens.data_ptr<int32_t>(), (int)S,
                                             query.size(0), (int)max_q_len, (int)query.size(1), p.hkv, p.d, p.bs,
                                             (int)block_table.size(1), p.nb, (float)scale, dtype_code(query, "query"),
                                             dtype_code(k_pool, "pool"), ks, vs, item_ptr, num_items, stream_of(query)));
}

at::Tensor decode_step(const at::Tensor& query_in, const at::Tensor& key, const at::Tensor& value, at::Tensor& k_pool,
                       at::Tensor& v_pool, const at::Tensor& block_table, const at::Tensor& ctx_rows, int64_t position,
                       int64_t group, double scale, const c10::optional<at::Tensor>& workspace) {
    const Pools p = check_pools(k_pool, v_pool);
    const c10::DeviceGuard guard(k_pool.device());
    TORCH_CHECK(query_in.dim() == 4 && query_in.size(2) == 1 && query_in.size(3) == p.d &&
                query_in.device() == k_pool.device(),
                "query must be a [B, Hq, 1, ", p.d, "] tensor on ", k_pool.device(), "; got ", query_in.sizes());
    const at::Tensor query = query_in.is_contiguous() ? query_in : query_in.contiguous();
    const int B = (int)query.size(0), hq = (int)query.size(1);
    TORCH_CHECK(hq % p.hkv == 0, hq, " query heads over ", p.hkv, " KV heads");
    const int64_t H = key.dim() == 4 ? key.size(1) : -1;
    const int64_t hstep = (group > 1 && H == (int64_t)p.hkv * group) ? group : 1;
    TORCH_CHECK(key.dim() == 4 && key.size(0) == B && H == p.hkv * hstep && key.size(2) == 1 && key.size(3) == p.d &&
                value.sizes() == key.sizes() && key.scalar_type() == query.scalar_type() &&
                value.scalar_type() == query.scalar_type() && key.device() == query.device() &&
                value.device() == query.device(),
                "key/value must both be [", B, ", ", p.hkv, " or ", p.hkv, "*group, 1, ", p.d, "] of the query dtype on ",
                query.device(), "; got ", key.sizes(), " and ", value.sizes());
    TORCH_CHECK(block_table.scalar_type() == at::kInt && block_table.dim() == 2 && block_table.size(0) == B &&
                block_table.stride(1) == 1 && block_table.device() == query.device(),
                "block_table must be int32 [", B, ", max_blocks] on ", query.device(), ", rows contiguous");
    // row `position + 1` of ctx_rows is the step's context-length vector (every sequence of the
    // batch shares one write position, kv_cache.py:69,290)
    TORCH_CHECK(ctx_rows.scalar_type() == at::kInt && ctx_rows.dim() == 2 && ctx_rows.size(1) == B &&
                ctx_rows.stride(1) == 1 && ctx_rows.device() == query.device() && position >= 0 &&
                position + 1 < ctx_rows.size(0),
                "ctx_rows must be int32 [positions + 1, ", B, "] on ", query.device(), " and hold row ", position + 1);
    at::Tensor k = key, v = value;
    if (k.stride(3) != 1 || k.strides() != v.strides()) { k = k.contiguous(); v = v.contiguous(); }
    const int qd = dtype_code(query, "query"), kd = dtype_code(k_pool, "pool");
    TORCH_CHECK(kd == qd, "decode_step stores the rows as they are: pools of the query dtype only");
    // Every sequence attends to position + 1 tokens, so only that many table columns are in use:
    // telling the library so lets it size the split for the context as it is now instead of for
    // the longest one the table could hold (a short context then runs as whole rows: one launch,
    // no scratch, no merge kernel).
    const int width = (int)std::min<int64_t>(block_table.size(1), (position + p.bs) / p.bs);
    at::Tensor own;
    size_t ws_bytes = 0;
    void* ws = decode_workspace(workspace, own, query, B, hq, p, width, qd, kd, 0, ws_bytes);
    at::Tensor out = at::empty_like(query);
    check_rc(aicomp_paged_decode_attn_append(out.data_ptr(), query.data_ptr(), k.data_ptr(), v.data_ptr(), k.stride(0),
                                             k.stride(1) * hstep, k_pool.data_ptr(), v_pool.data_ptr(),
                                             block_table.data_ptr<int32_t>(), block_table.stride(0),
                                             ctx_rows.data_ptr<int32_t>() + (position + 1) * ctx_rows.stride(0), B, hq,
                                             p.hkv, p.d, p.bs, width, p.nb, (float)scale, qd, kd,
                                             nullptr, nullptr, 0, ws, ws_bytes, stream_of(query)));
    return out;
}

}  // namespace

TORCH_LIBRARY(mi355_kv, m) {
    m.def("kv_append(Tensor key, Tensor value, Tensor(a!) k_pool, Tensor(b!) v_pool, Tensor slot_mapping, "
          "Tensor? k_scale=None, Tensor? v_scale=None) -> ()");
    m.def("paged_decode_attn(Tensor(a!) out, Tensor query, Tensor k_pool, Tensor v_pool, Tensor block_table, "
          "Tensor context_lens, float scale, Tensor? k_scale=None, Tensor? v_scale=None, int partition_size=0, "
          "Tensor? workspace=None) -> ()");
    m.def("paged_decode_attn_append(Tensor(a!) out, Tensor query, Tensor new_key, Tensor new_value, Tensor(b!) k_pool, "
          "Tensor(c!) v_pool, Tensor block_table, Tensor context_lens, float scale, Tensor? k_scale=None, "
          "Tensor? v_scale=None, int partition_size=0, Tensor? workspace=None) -> ()");
    m.def("paged_prefill_attn(Tensor(a!) out, Tensor query, Tensor k_pool, Tensor v_pool, Tensor block_table, "
          "Tensor context_lens, Tensor cu_q_lens, float scale, int max_q_len, Tensor? k_scale=None, "
          "Tensor? v_scale=None, Tensor? items=None) -> ()");
    m.def("decode_step(Tensor query, Tensor key, Tensor value, Tensor(a!) k_pool, Tensor(b!) v_pool, Tensor block_table, "
          "Tensor ctx_rows, int position, int group, float scale, Tensor? workspace=None) -> Tensor");
}

TORCH_LIBRARY_IMPL(mi355_kv, CUDA, m) {       // the dispatch key of ROCm devices
    m.impl("kv_append", &kv_append);
    m.impl("paged_decode_attn", &paged_decode_attn);
    m.impl("paged_decode_attn_append", &paged_decode_attn_append);
    m.impl("paged_prefill_attn", &paged_prefill_attn);
    m.impl("decode_step", &decode_step);
}
