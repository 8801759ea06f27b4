"""torch.ops.mi355_kv.*: the C ABI registered as PyTorch operators.  Every op is compared bit for
bit with the ctypes route (aicomp_amd.ops) on the same inputs: both end in the same C entry point,
so any difference is a binding mistake (argument order, strides, stream, dtype codes)."""
import math

import pytest
import torch

from aicomp_amd import _lib, ops, workloads
from aicomp_amd import kv_cache as akv

pytestmark = pytest.mark.gpu


def bits(t):
    return t.view(torch.uint8) if t.dtype == torch.float8_e4m3fn else t.view(torch.int16) if t.element_size() == 2 else t


def small(name, **kw):
    s = workloads.SHAPES[name]
    return workloads.Shape(**{**s.__dict__, **kw})


@pytest.mark.parametrize("name", ["llama3_8b_decode", "llama3_70b_decode_fp8", "llama32_1b_decode", "decode_fp32_small"])
def test_registered_ops_equal_the_ctypes_route(device, name):
    t = _lib.torch_ops()
    w = workloads.make_workload("x", device=device, seed=3, shape=small(name, batch=5, ctx_lo=30, ctx_hi=700))
    k1, v1, k2, v2 = w.k_pool.clone(), w.v_pool.clone(), w.k_pool.clone(), w.v_pool.clone()
    # append
    ops.kv_append(w.new_key, w.new_value, k1, v1, w.slot_mapping, w.k_scale, w.v_scale)
    t.kv_append(w.new_key, w.new_value, k2, v2, w.slot_mapping, w.k_scale, w.v_scale)
    assert torch.equal(bits(k1), bits(k2)) and torch.equal(bits(v1), bits(v2))
    # decode, automatic and explicit split, library-allocated and caller's scratch
    for ps in (0, 128):
        a = torch.full_like(w.query, float("nan"))
        b = torch.full_like(w.query, float("nan"))
        ops.paged_decode_attn(a, w.query, k1, v1, w.block_table, w.context_lens, w.scale, w.k_scale, w.v_scale,
                              partition_size=ps)
        t.paged_decode_attn(b, w.query, k2, v2, w.block_table, w.context_lens, w.scale, w.k_scale, w.v_scale, ps)
        assert torch.equal(bits(a), bits(b)) and torch.isfinite(b.float()).all()
        need = ops.decode_workspace_bytes(5, w.shape.num_q_heads, w.shape.num_kv_heads, w.shape.head_dim, 16,
                                          w.block_table.shape[1], w.query.dtype, k2.dtype, ps)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
        c = torch.full_like(w.query, float("nan"))
        t.paged_decode_attn(c, w.query, k2, v2, w.block_table, w.context_lens, w.scale, w.k_scale, w.v_scale, ps, ws)
        assert torch.equal(bits(a), bits(c))
    # fused append + decode on fresh pools
    k3, v3 = w.k_pool.clone(), w.v_pool.clone()
    d = torch.full_like(w.query, float("nan"))
    t.paged_decode_attn_append(d, w.query, w.new_key, w.new_value, k3, v3, w.block_table, w.context_lens, w.scale,
                               w.k_scale, w.v_scale)
    assert torch.equal(bits(k3), bits(k1)) and torch.equal(bits(v3), bits(v1))
    e = torch.full_like(w.query, float("nan"))
    ops.paged_decode_attn(e, w.query, w.k_pool.clone(), w.v_pool.clone(), w.block_table, w.context_lens, w.scale,
                          w.k_scale, w.v_scale, new_key=w.new_key, new_value=w.new_value)
    assert torch.equal(bits(d), bits(e))


@pytest.mark.parametrize("kv", [None, torch.float8_e4m3fn])
def test_registered_prefill_equals_the_ctypes_route(device, kv):
    import test_gpu_prefill as tp
    t = _lib.torch_ops()
    c = tp.build_case(device, priors=[0, 37, 300], news=[130, 20, 64], hq=8, hkv=2, d=128, kv_dtype=kv, seed=4)
    a = tp.run(c, max_q_len=130)
    b = torch.full_like(c["q"], float("nan"))
    t.paged_prefill_attn(b, c["q"], c["k_pool"], c["v_pool"], c["table"], c["ctx"], c["cu"], c["scale"], 130,
                         c["ks"], c["vs"])
    torch.cuda.synchronize()
    assert torch.equal(bits(a), bits(b))


@pytest.mark.parametrize("B,hq,g,d,expanded", [(1, 32, 4, 64, True), (3, 32, 4, 128, True), (2, 8, 2, 128, False)])
def test_decode_step_op_equals_the_prepared_ctypes_call(device, B, hq, g, d, expanded):
    """The adapter's decode step through the registered op and through ops.PreparedDecode.step4d:
    same output bits, same pools, on the operator's own 4-D tensors (K/V expanded by repeat_kv or not)."""
    t = _lib.torch_ops()
    hkv = hq // g
    layer_a = akv._PagedLayer(B, hkv, d, 256, torch.bfloat16, device)
    layer_b = akv._PagedLayer(B, hkv, d, 256, torch.bfloat16, device)
    gen = torch.Generator().manual_seed(B * 100 + d)
    mk = lambda n, h: torch.randn(B, h, n, d, generator=gen).to(torch.bfloat16).to(device)
    k0, v0 = mk(40, hkv), mk(40, hkv)
    for layer in (layer_a, layer_b):
        layer.append(k0, v0, 0, 1)
    for pos in range(40, 45):
        q, k, v = mk(1, hq), mk(1, hkv), mk(1, hkv)
        if expanded:
            k, v = k.repeat_interleave(g, 1), v.repeat_interleave(g, 1)
        got = t.decode_step(q, k, v, layer_a.k_pool, layer_a.v_pool, layer_a.block_table, layer_a.ctx_rows, pos, g,
                            1 / math.sqrt(d), None)
        call = ops.PreparedDecode(layer_b.k_pool, layer_b.v_pool, layer_b.block_table, layer_b.context_lens, hq,
                                  torch.bfloat16, 1 / math.sqrt(d))
        want = call.step4d(torch.empty_like(q), q, k, v, g, layer_b.ctx_rows[pos + 1], width=pos // 16 + 1)
        assert got.shape == (B, hq, 1, d) and torch.equal(bits(got), bits(want))
        assert torch.equal(bits(layer_a.k_pool), bits(layer_b.k_pool)) and torch.equal(bits(layer_a.v_pool), bits(layer_b.v_pool))


def test_registered_ops_reject_bad_arguments_with_runtime_errors(device):
    t = _lib.torch_ops()
    w = workloads.make_workload("x", device=device, shape=small("llama3_8b_decode", batch=2, ctx_lo=20, ctx_hi=60))
    out = torch.empty_like(w.query)
    with pytest.raises(RuntimeError, match="contiguous"):
        t.paged_decode_attn(out, w.query.transpose(0, 1).contiguous().transpose(0, 1), w.k_pool, w.v_pool,
                            w.block_table, w.context_lens, w.scale)
    with pytest.raises(RuntimeError, match="int32"):
        t.paged_decode_attn(out, w.query, w.k_pool, w.v_pool, w.block_table.long(), w.context_lens, w.scale)
    with pytest.raises(RuntimeError, match="head_dim"):
        t.paged_decode_attn(out[..., :64].contiguous(), w.query[..., :64].contiguous(), w.k_pool, w.v_pool,
                            w.block_table, w.context_lens, w.scale)
    with pytest.raises(RuntimeError):                    # CPU tensors: there is no CPU kernel to dispatch to
        t.paged_decode_attn(out.cpu(), w.query.cpu(), w.k_pool.cpu(), w.v_pool.cpu(), w.block_table.cpu(),
                            w.context_lens.cpu(), w.scale)
    with pytest.raises(RuntimeError, match="slot_mapping"):
        t.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping.int())
    with pytest.raises(RuntimeError, match="hold row"):
        layer = akv._PagedLayer(2, 8, 128, 64, torch.bfloat16, device)
        q = torch.zeros(2, 32, 1, 128, dtype=torch.bfloat16, device=device)
        k = torch.zeros(2, 8, 1, 128, dtype=torch.bfloat16, device=device)
        t.decode_step(q, k, k, layer.k_pool, layer.v_pool, layer.block_table, layer.ctx_rows, 64, 4, 0.1, None)


@pytest.mark.parametrize("B,hq,g,d,dtype", [(1, 32, 4, 64, torch.bfloat16), (3, 16, 4, 128, torch.float16), (2, 8, 2, 64, torch.float32)])
def test_lean_decode_call_equals_the_registered_op(device, B, hq, g, d, dtype):
    """aicomp_amd._aicomp_fast.decode_step (a layer's static tensors behind a handle, one CPython
    call per step) against torch.ops.mi355_kv.decode_step: same output bits, same pools, across a
    block boundary and the point where the call starts to need a merge (640 tokens)."""
    from aicomp_amd import _aicomp_fast as fast
    t = _lib.torch_ops()
    hkv = hq // g
    a = akv._PagedLayer(B, hkv, d, 1024, dtype, device)
    b = akv._PagedLayer(B, hkv, d, 1024, dtype, device)
    gen = torch.Generator().manual_seed(B + d)
    mk = lambda n, h: torch.randn(B, h, n, d, generator=gen).to(dtype).to(device)
    k0, v0 = mk(636, hkv), mk(636, hkv)
    a.append(k0, v0, 0, 1)
    b.append(k0, v0, 0, 1)
    handle = fast.layer(a.k_pool, a.v_pool, a.block_table, a.ctx_rows)
    for pos in range(636, 644):
        q, k, v = mk(1, hq), mk(1, hkv).repeat_interleave(g, 1), mk(1, hkv).repeat_interleave(g, 1)
        got = fast.decode_step(handle, q, k, v, pos, g, 1 / math.sqrt(d))
        want = t.decode_step(q, k, v, b.k_pool, b.v_pool, b.block_table, b.ctx_rows, pos, g, 1 / math.sqrt(d), None)
        assert got.shape == want.shape and got.dtype == dtype and torch.equal(bits(got), bits(want)), pos
    assert torch.equal(bits(a.k_pool), bits(b.k_pool)) and torch.equal(bits(a.v_pool), bits(b.v_pool))
    # a transposed (non-contiguous) query and strided K/V views are taken as they are or copied, as in the op
    q = mk(1, hq).transpose(1, 3).contiguous().transpose(1, 3)
    k = mk(1, hkv)
    got = fast.decode_step(handle, q, k, k, 644, g, 0.1)
    want = t.decode_step(q, k, k, b.k_pool, b.v_pool, b.block_table, b.ctx_rows, 644, g, 0.1, None)
    assert torch.equal(bits(got), bits(want))
    for bad in (lambda: fast.decode_step(handle, q[:, :, :, :8], k, k, 645, g, 0.1),               # head_dim
                lambda: fast.decode_step(handle, q, mk(1, hkv + 1), mk(1, hkv + 1), 645, g, 0.1),  # K/V heads
                lambda: fast.decode_step(handle, q.float() if dtype != torch.float32 else q.half(), k, k, 645, g, 0.1),
                lambda: fast.decode_step(handle, q, k, k, 5000, g, 0.1),                            # beyond ctx_rows
                lambda: fast.decode_step(handle, q.cpu(), k, k, 645, g, 0.1),
                lambda: fast.layer(a.k_pool.cpu(), a.v_pool.cpu(), a.block_table.cpu(), a.ctx_rows.cpu())):
        with pytest.raises(RuntimeError):
            bad()
