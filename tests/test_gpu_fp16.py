"""float16 through every entry point of the path.

The reference's inference drivers offer ``--dtype float16``
(opt_prime/examples/single_gpu_inference_llama.py:98-110) and its operator is dtype-generic
(opt_prime/opt_prime/kv_cache.py:372-415), so the drop-in must take half-precision tensors too.
Same oracle as bf16 (float64 textbook attention on the fp16 values); the tolerance is the
benchmark's bf16 bound tightened to what 10 mantissa bits give: max-abs 2e-3 or rel 1e-2.
Copies, rotations and quantisation are bit-exact.
"""
import math

import numpy as np
import pytest
import torch

from aicomp_amd import kv_cache as akv
from aicomp_amd import ops, workloads
from oracle import contiguous_ref as cref
from oracle import paged_kv_oracle as orc
from oracle import rope_oracle as R
from oracle import sample_oracle as S
from helpers import NAME, assert_close_attn, raw, to_f64
import test_gpu_prefill as tp
import test_gpu_rope as tr
import test_gpu_sample as ts

pytestmark = pytest.mark.gpu
F16 = torch.float16
F16_ATOL, F16_RTOL = 2e-3, 1e-2


def _shape(name, **kw):
    s = workloads.SHAPES[name]
    base = dict(q_dtype=F16, kv_dtype=F16)
    if s.kv_dtype == torch.float8_e4m3fn:
        base["kv_dtype"] = s.kv_dtype
    return workloads.Shape(**{**s.__dict__, **base, **kw})


def _oracle_decode(w, ctx=None):
    ks = None if w.k_scale is None else w.k_scale.cpu().numpy()
    vs = None if w.v_scale is None else w.v_scale.cpu().numpy()
    return orc.paged_decode_attn(raw(w.query), raw(w.k_pool), raw(w.v_pool), w.block_table.cpu().numpy(),
                                 w.ctx_list if ctx is None else ctx, w.scale, NAME[w.query.dtype],
                                 NAME[w.k_pool.dtype], ks, vs)


@pytest.mark.parametrize("name,batch,partition", [
    ("llama3_8b_decode", 5, 0),            # balanced schedule, head_dim 128
    ("llama3_8b_decode", 5, 512),          # grid schedule, split
    ("llama32_1b_decode", 5, 0),           # head_dim 64: rows of token pairs
    ("llama3_70b_decode_fp8", 3, 0),       # fp16 queries over an fp8 pool, group 8
    ("long_context_skewed", 3, 0),
])
def test_fp16_decode_vs_oracle_and_fused_append(device, name, batch, partition):
    w = workloads.make_workload("x", device=device, seed=4, shape=_shape(name, batch=batch))
    assert w.query.dtype == F16
    k2, v2 = w.k_pool.clone(), w.v_pool.clone()
    ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping, w.k_scale, w.v_scale)
    out = torch.full_like(w.query, float("nan"))
    ops.paged_decode_attn(out, w.query, w.k_pool, w.v_pool, w.block_table, w.context_lens, w.scale,
                          w.k_scale, w.v_scale, partition_size=partition)
    torch.cuda.synchronize()
    assert_close_attn(to_f64(out), _oracle_decode(w), F16_ATOL, F16_RTOL, f"fp16 decode {name} ps {partition}")
    # one fused call on the untouched pools: same pools, same output bits
    fused = torch.full_like(w.query, float("nan"))
    ops.paged_decode_attn(fused, w.query, k2, v2, w.block_table, w.context_lens, w.scale, w.k_scale, w.v_scale,
                          partition_size=partition, new_key=w.new_key, new_value=w.new_value)
    torch.cuda.synchronize()
    assert torch.equal(k2.view(torch.uint8), w.k_pool.view(torch.uint8))
    assert torch.equal(v2.view(torch.uint8), w.v_pool.view(torch.uint8))
    assert torch.equal(fused.view(torch.int16), out.view(torch.int16))


def test_fp16_decode_vector_kernel_shapes(device):
    """Shapes the matrix-core kernels do not cover (head_dim 256; block size 32) run the vector-ALU
    kernel, which takes fp16 as well."""
    for d, bs in ((256, 16), (128, 32)):
        sh = workloads.Shape("t", 4, 8, 2, d, block_size=bs, q_dtype=F16, kv_dtype=F16, kv_std=0.5,
                             ctx_lo=30, ctx_hi=400)
        w = workloads.make_workload("t", device=device, seed=6, shape=sh)
        ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping)
        for ps in (0, 4 * bs):
            out = torch.full_like(w.query, float("nan"))
            ops.paged_decode_attn(out, w.query, w.k_pool, w.v_pool, w.block_table, w.context_lens, w.scale,
                                  partition_size=ps)
            torch.cuda.synchronize()
            assert_close_attn(to_f64(out), _oracle_decode(w), F16_ATOL, F16_RTOL, f"fp16 generic D {d} BS {bs}")


def test_fp16_append_raw_and_quantised(device):
    """Raw copy of fp16 rows is bit-exact; fp16 -> e4m3 quantisation equals torch's cast for every
    finite fp16 value (scale 1) and the oracle's rule under per-head scales."""
    hkv, d = 2, 128
    codes = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(F16)
    finite = codes[torch.isfinite(codes.float())]
    T = finite.numel() // (hkv * d)
    rows = finite[: T * hkv * d].view(T, hkv, d).to(device)
    nb = (T + 15) // 16
    slots = torch.randperm(nb * 16, generator=torch.Generator().manual_seed(0))[:T].to(device)
    kp = torch.zeros(nb, hkv, 16, d, dtype=F16, device=device)
    vp = torch.zeros_like(kp)
    ops.kv_append(rows, rows.flip(0), kp, vp, slots)
    want_k, want_v = raw(kp) * 0, raw(vp) * 0
    orc.kv_append_fast(raw(rows), raw(rows.flip(0)), want_k, want_v, slots.cpu().numpy())
    assert np.array_equal(raw(kp), want_k) and np.array_equal(raw(vp), want_v)
    one = torch.ones(hkv, device=device)
    k8 = torch.zeros(nb, hkv, 16, d, dtype=torch.float8_e4m3fn, device=device)
    v8 = torch.zeros_like(k8)
    ops.kv_append(rows, rows, k8, v8, slots, one, one)
    want = rows.float().clamp(-448, 448).to(torch.float8_e4m3fn)
    got = k8.view(torch.uint8).permute(0, 2, 1, 3).reshape(nb * 16, hkv, d)[slots]
    assert torch.equal(got, want.view(torch.uint8))
    scales = torch.tensor([0.013, 2.7], device=device)
    ops.kv_append(rows, rows, k8, v8, slots, scales, scales)
    ko, vo = raw(k8) * 0, raw(v8) * 0
    sub = slice(0, 64)                                   # the oracle's quantising append loops in Python
    orc.kv_append(raw(rows[sub]), raw(rows[sub]), ko, vo, slots[sub].cpu().numpy(), scales.cpu().numpy(),
                  scales.cpu().numpy(), pool_dtype="fp8", in_dtype="f16")
    sl = slots[sub].cpu()
    assert np.array_equal(raw(k8)[sl // 16, :, sl % 16], ko[sl // 16, :, sl % 16])


@pytest.mark.parametrize("d", [128, 64])
def test_fp16_prefill_vs_oracle(device, d):
    """Ragged chunks (register-staged tiles), chunks of >= 128 rows (tiles straight into LDS, with
    NaN / Inf beyond every context), and fp8 pools under fp16 queries."""
    c = tp.build_case(device, priors=[0, 5, 37, 200, 0, 63], news=[70, 1, 33, 17, 1, 130], hq=8, hkv=2, d=d,
                      dtype=F16)
    assert_close_attn(to_f64(tp.run(c, max_q_len=130)), tp.oracle(c), F16_ATOL, F16_RTOL, f"fp16 ragged D {d}")
    for ctx in (64, 129, 300):
        c = tp.build_case(device, priors=[0, ctx - 40], news=[ctx, 40], hq=8, hkv=2, d=d, dtype=F16, seed=ctx)
        assert_close_attn(to_f64(tp.run(c, max_q_len=ctx)), tp.oracle(c), F16_ATOL, F16_RTOL, f"fp16 ctx {ctx} D {d}")
    c = tp.build_case(device, priors=[0, 300, 77], news=[200, 130, 40], hq=8, hkv=2, d=d, dtype=F16,
                      kv_dtype=torch.float8_e4m3fn)
    assert_close_attn(to_f64(tp.run(c, max_q_len=200)), tp.oracle(c), F16_ATOL, F16_RTOL, f"fp16 over fp8 D {d}")


def test_fp16_prefill_reduces_to_torch_causal_sdpa(device):
    """prior == 0 is the reference's call (kv_cache.py:412-415): compare with torch's own
    is_causal=True attention on the same fp16 values, computed in float64 on the CPU."""
    c = tp.build_case(device, priors=[0], news=[160], hq=8, hkv=2, d=128, dtype=F16, poison=False)
    got = tp.run(c, max_q_len=160).double().cpu()
    L = 160
    t = torch.arange(L)
    k = c["k_pool"].cpu()[c["table"].cpu()[0, t // 16].long(), :, t % 16].double()       # [L, Hkv, D]
    v = c["v_pool"].cpu()[c["table"].cpu()[0, t // 16].long(), :, t % 16].double()
    q = c["q"].double().cpu().transpose(0, 1)[None]                                        # [1, Hq, L, D]
    ke = k.transpose(0, 1).repeat_interleave(4, 0)[None]
    ve = v.transpose(0, 1).repeat_interleave(4, 0)[None]
    want = torch.nn.functional.scaled_dot_product_attention(q, ke, ve, is_causal=True)[0].transpose(0, 1)
    assert_close_attn(got.numpy(), want.numpy(), F16_ATOL, F16_RTOL, "fp16 prefill vs torch SDPA")


@pytest.mark.parametrize("hq,hkv,d,fp8", [(8, 2, 128, False), (4, 4, 64, False), (8, 2, 128, True)])
def test_fp16_rope_append_bit_exact(device, hq, hkv, d, fp8):
    c = tr.make_case(device, 41, hq, hkv, d, F16)
    if fp8:
        kp = torch.zeros(c["nb"], hkv, 16, d, dtype=torch.float8_e4m3fn, device=device)
        vp = torch.zeros_like(kp)
        ks = torch.full((hkv,), 0.02, device=device)
        vs = torch.full((hkv,), 0.01, device=device)
        want_q, want_k, want_v = tr.run_oracle(c, kp, vp, F16, ks=ks, vs=vs, pool_dtype="fp8")
        out = ops.rope_kv_append(c["q"], c["k"], c["v"], c["cos"], c["sin"], c["pos"], kp, vp, c["slots"], ks, vs)
    else:
        kp, vp = tr.sentinel_pools(c, hkv, d, F16, device)
        want_q, want_k, want_v = tr.run_oracle(c, kp, vp, F16)
        out = ops.rope_kv_append(c["q"], c["k"], c["v"], c["cos"], c["sin"], c["pos"], kp, vp, c["slots"])
    torch.cuda.synchronize()
    assert np.array_equal(raw(out), want_q)
    assert np.array_equal(raw(kp), want_k) and np.array_equal(raw(vp), want_v)


def test_fp16_rope_matches_torch_eager_expression(device):
    """The reference's expression (modeling_llama.py:200-231) evaluated by torch's own fp16 kernels."""
    T, hq, hkv, d = 300, 8, 2, 128
    c = tr.make_case(device, T, hq, hkv, d, F16, table_rows=1024, seed=2)
    kp, vp = tr.sentinel_pools(c, hkv, d, F16, device)
    cos, sin = c["cos"][c["pos"]][:, None, :], c["sin"][c["pos"]][:, None, :]
    half = lambda x: torch.cat((-x[..., d // 2:], x[..., :d // 2]), dim=-1)
    q_ref = (c["q"] * cos) + (half(c["q"]) * sin)
    k_ref = (c["k"] * cos) + (half(c["k"]) * sin)
    kp_ref, vp_ref = kp.clone(), vp.clone()
    ops.kv_append(k_ref, c["v"], kp_ref, vp_ref, c["slots"])
    out = ops.rope_kv_append(c["q"].clone(), c["k"], c["v"], c["cos"], c["sin"], c["pos"], kp, vp, c["slots"])
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), q_ref.view(torch.int16))
    assert torch.equal(kp.view(torch.int16), kp_ref.view(torch.int16))
    assert torch.equal(vp.view(torch.int16), vp_ref.view(torch.int16))


def test_fp16_adapter_session(device):
    """The drop-in operator on a float16 model (``--dtype float16`` of the reference's examples):
    prefill, decode steps across a block boundary, clear, again; both head sizes."""
    for hq, g, d in ((32, 4, 128), (32, 4, 64)):
        B = 2
        new = akv.CachedScaledDotProductAttention(0, max_seq_len=256, dtype=F16)
        ref = cref.ContiguousCachedAttention(0, 256)
        new.enable(); ref.enable()
        torch.manual_seed(0)
        hkv = hq // g
        for n in [77, 1, 1, 1, 1]:
            q = torch.randn(B, hq, n, d).to(F16)
            k = (torch.randn(B, hkv, n, d) * 0.5).to(F16)
            v = (torch.randn(B, hkv, n, d) * 0.5).to(F16)
            ke, ve = k.repeat_interleave(g, 1), v.repeat_interleave(g, 1)
            want = ref(q.float(), ke.float(), ve.float(), attn_mask=None, is_causal=True)
            got = new(q.to(device), ke.to(device), ve.to(device), attn_mask=None, is_causal=True)
            assert got.dtype == F16 and got.shape == want.shape
            assert_close_attn(to_f64(got), want.double().numpy(), F16_ATOL, F16_RTOL, f"fp16 adapter n={n} D {d}")
            assert new.cache_pos == ref.pos
        assert new.cache_k.dtype == F16
        new.disable()


def test_fp16_sampler(device):
    """fp16 logits: the temperature division is rounded to fp16 like the eager division, then the
    reference's statements in float64 (the oracle); values down in fp16's subnormal range included."""
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((6, 5003)) * 3).astype(np.float32)
    for temperature, top_k, top_p in ((0.7, 20, 0.95), (1.3, 0, 0.9), (1.0, 50, 1.0), (2.0, 1000, 0.5)):
        ts.check_rows(device, x, temperature, top_k, top_p, dtype=F16)
    tiny = (rng.standard_normal((4, 3000)) * 3e-5).astype(np.float32)       # quotients round in the subnormal range
    for temperature, top_k, top_p in ((1.7, 40, 1.0), (0.9, 500, 0.9)):
        ts.check_rows(device, tiny, temperature, top_k, top_p, dtype=F16)
    xt = torch.from_numpy(x).to(F16)
    greedy = ops.sample_tokens(xt.to(device), do_sample=False)
    assert greedy.cpu().tolist() == [S.greedy(r) for r in xt.float().numpy()]
