// CPython entry for the drop-in operator's decode call at small batch: the leanest host route
// from CachedScaledDotProductAttention.forward (opt_prime/opt_prime/kv_cache.py:340-403) into
// aicomp_paged_decode_attn_append.  The reference's own engine decodes at batch 1
// (inference.py:1036-1044), where the GPU needs 5 to 8 us per call and every microsecond of host
// time is step time.  torch.ops.mi355_kv.decode_step (torch_ops.cpp) spends about three of its eight
// microseconds in the dispatcher and in re-checking tensors that never change between steps; here
// a layer's pools, table and context-length rows are checked once and kept in a capsule, and a
// step is one METH_FASTCALL function: three tensors unpacked, the output allocated, one C call.
//
//   layer = _aicomp_fast.layer(k_pool, v_pool, block_table, ctx_rows)
//   out   = _aicomp_fast.decode_step(layer, query, key, value, position, group, scale)
//
// Same checks, same errors (RuntimeError), same results as the registered operator.
#include <Python.h>

#include <ATen/ATen.h>
#include <ATen/hip/EmptyTensor.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/csrc/autograd/python_variable.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <utility>

#include "../../include/aicomp_kv.h"

namespace {

struct Layer {
    at::Tensor k_pool, v_pool, block_table, ctx_rows;     // kept alive; the pointers below are theirs
    void* kp;
    void* vp;
    const int32_t* table;
    const int32_t* ctx;
    int64_t table_stride, ctx_stride, ctx_count, nb;
    int B, hkv, bs, d, width, dt;
    at::ScalarType st;
    c10::Device dev{c10::DeviceType::CPU};
};

int dtype_code(at::ScalarType t) {
    switch (t) {
        case at::kFloat: return AICOMP_KV_F32;
        case at::kBFloat16: return AICOMP_KV_BF16;
        case at::kHalf: return AICOMP_KV_F16;
        default: return -1;
    }
}

void layer_free(PyObject* cap) { delete (Layer*)PyCapsule_GetPointer(cap, "aicomp_amd.layer"); }

// scratch of calls that need a merge: one growing buffer per (device, stream), never destroyed
// (tensors freed at interpreter exit, after the allocator, would fault)
at::Tensor& cached_scratch(const c10::Device& dev, void* stream, size_t bytes) {
    static std::mutex mu;
    static auto* table = new std::map<std::pair<int, void*>, at::Tensor>();
    std::lock_guard<std::mutex> lock(mu);
    at::Tensor& t = (*table)[{(int)dev.index(), stream}];
    if (!t.defined() || (size_t)t.numel() < bytes)
        t = at::empty({(int64_t)bytes}, at::TensorOptions().dtype(at::kByte).device(dev));
    return t;
}

#define FAIL(...)                                             \
    do {                                                      \
        PyErr_Format(PyExc_RuntimeError, __VA_ARGS__);        \
        return nullptr;                                       \
    } while (0)

PyObject* layer_new(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
    try {
        if (nargs != 4) FAIL("layer(k_pool, v_pool, block_table, ctx_rows)");
        for (int i = 0; i < 4; ++i)
            if (!THPVariable_Check(args[i])) FAIL("layer: argument %d is not a tensor", i);
        auto L = std::make_unique<Layer>();
        L->k_pool = THPVariable_Unpack(args[0]);
        L->v_pool = THPVariable_Unpack(args[1]);
        L->block_table = THPVariable_Unpack(args[2]);
        L->ctx_rows = THPVariable_Unpack(args[3]);
        const at::Tensor &k = L->k_pool, &v = L->v_pool, &bt = L->block_table, &cr = L->ctx_rows;
        if (!k.is_cuda()) FAIL("tensors must live on a ROCm device (there is no CPU path)");
        if (k.dim() != 4 || v.sizes() != k.sizes() || k.scalar_type() != v.scalar_type() || !k.is_contiguous() ||
            !v.is_contiguous() || v.device() != k.device())
            FAIL("pools must both be contiguous [num_blocks, Hkv, BS, D] tensors of one dtype on one device");
        L->dt = dtype_code(k.scalar_type());
        if (L->dt < 0) FAIL("decode_step stores the rows as they are: float32, bfloat16 or float16 pools");
        L->B = (int)bt.size(0);
        if (bt.scalar_type() != at::kInt || bt.dim() != 2 || bt.stride(1) != 1 || bt.device() != k.device())
            FAIL("block_table must be int32 [B, max_blocks] on the pools' device, rows contiguous");
        if (cr.scalar_type() != at::kInt || cr.dim() != 2 || cr.size(1) != L->B || cr.stride(1) != 1 ||
            cr.device() != k.device())
            FAIL("ctx_rows must be int32 [positions + 1, B] on the pools' device");
        L->kp = k.data_ptr(); L->vp = v.data_ptr();
        L->table = bt.data_ptr<int32_t>(); L->table_stride = bt.stride(0); L->width = (int)bt.size(1);
        L->ctx = cr.data_ptr<int32_t>(); L->ctx_stride = cr.stride(0); L->ctx_count = cr.size(0);
        L->nb = k.size(0); L->hkv = (int)k.size(1); L->bs = (int)k.size(2); L->d = (int)k.size(3);
        L->st = k.scalar_type(); L->dev = k.device();
        return PyCapsule_New(L.release(), "aicomp_amd.layer", layer_free);
    } catch (const std::exception& e) {
        FAIL("%s", e.what());
    }
}

PyObject* decode_step(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
    try {
        if (nargs != 7) FAIL("decode_step(layer, query, key, value, position, group, scale)");
        const Layer* L = (const Layer*)PyCapsule_GetPointer(args[0], "aicomp_amd.layer");
        if (L == nullptr) return nullptr;
        if (!THPVariable_Check(args[1]) || !THPVariable_Check(args[2]) || !THPVariable_Check(args[3]))
            FAIL("decode_step: query, key and value must be tensors");
        const at::Tensor& q_in = THPVariable_Unpack(args[1]);
        const at::Tensor& key = THPVariable_Unpack(args[2]);
        const at::Tensor& value = THPVariable_Unpack(args[3]);
        const int64_t position = PyLong_AsLongLong(args[4]);
        const int64_t group = PyLong_AsLongLong(args[5]);
        const double scale = PyFloat_AsDouble(args[6]);
        if (PyErr_Occurred()) return nullptr;
        if (q_in.dim() != 4 || q_in.size(0) != L->B || q_in.size(2) != 1 || q_in.size(3) != L->d ||
            q_in.scalar_type() != L->st || q_in.device() != L->dev)
            FAIL("query must be a [%d, Hq, 1, %d] tensor of the pools' dtype on their device", L->B, L->d);
        const int hq = (int)q_in.size(1);
        if (hq % L->hkv) FAIL("%d query heads over %d KV heads", hq, L->hkv);
        const int64_t H = key.dim() == 4 ? key.size(1) : -1;
        const int64_t hstep = (group > 1 && H == (int64_t)L->hkv * group) ? group : 1;
        if (key.dim() != 4 || key.size(0) != L->B || H != L->hkv * hstep || key.size(2) != 1 || key.size(3) != L->d ||
            value.sizes() != key.sizes() || key.scalar_type() != L->st || value.scalar_type() != L->st ||
            key.device() != L->dev || value.device() != L->dev)
            FAIL("key/value must both be [%d, %d or %d*group, 1, %d] of the query dtype on its device", L->B, L->hkv,
                 L->hkv, L->d);
        if (position < 0 || position + 1 >= L->ctx_count) FAIL("ctx_rows does not hold row %lld", (long long)(position + 1));
        const c10::DeviceGuard guard(L->dev);              // launches go to the layer's device, whatever is current
        const at::Tensor query = q_in.is_contiguous() ? q_in : q_in.contiguous();
        at::Tensor k = key, v = value;
        if (k.stride(3) != 1 || k.strides() != v.strides()) { k = k.contiguous(); v = v.contiguous(); }
        // only the table columns that hold position + 1 tokens are in use: the library sizes the
        // split for the context as it is now (a short context: one launch, no scratch, no merge)
        const int width = (int)std::min<int64_t>(L->width, (position + L->bs) / L->bs);
        void* stream = (void*)c10::hip::getCurrentHIPStream(L->dev.index()).stream();
        size_t ws_bytes = aicomp_paged_decode_workspace_bytes(L->B, hq, L->hkv, L->d, L->bs, width, L->dt, L->dt, 0);
        void* ws = nullptr;
        if (ws_bytes) {
            at::Tensor& t = cached_scratch(L->dev, stream, ws_bytes);
            ws = t.data_ptr();
            ws_bytes = (size_t)t.numel();
        }
        // (the allocator's own entry: at::empty goes through the dispatcher for the same result)
        at::Tensor out(at::detail::empty_cuda(query.sizes(), L->st, L->dev, c10::MemoryFormat::Contiguous));
        const int rc = aicomp_paged_decode_attn_append(
            out.data_ptr(), query.data_ptr(), k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1) * hstep, L->kp, L->vp,
            L->table, L->table_stride, L->ctx + (position + 1) * L->ctx_stride, L->B, hq, L->hkv, L->d, L->bs, width,
            L->nb, (float)scale, L->dt, L->dt, nullptr, nullptr, 0, ws, ws_bytes, stream);
        if (rc != AICOMP_KV_OK) FAIL("aicomp_kv error %d: %s", rc, aicomp_kv_last_error());
        return THPVariable_Wrap(std::move(out));
    } catch (const std::exception& e) {
        FAIL("%s", e.what());
    }
}

PyMethodDef methods[] = {
    {"layer", (PyCFunction)(void (*)(void))layer_new, METH_FASTCALL,
     "layer(k_pool, v_pool, block_table, ctx_rows) -> handle: a layer's static tensors, checked once"},
    {"decode_step", (PyCFunction)(void (*)(void))decode_step, METH_FASTCALL,
     "decode_step(layer, query, key, value, position, group, scale) -> out [B, Hq, 1, D]"},
    {nullptr, nullptr, 0, nullptr}};

PyModuleDef module = {PyModuleDef_HEAD_INIT, "_aicomp_fast", "decode step of the paged KV-cache operator, lean host route",
                      -1, methods, nullptr, nullptr, nullptr, nullptr};

}  // namespace

PyMODINIT_FUNC PyInit__aicomp_fast(void) { return PyModule_Create(&module); }
