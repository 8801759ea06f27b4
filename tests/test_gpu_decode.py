"""Paged decode attention through the C ABI vs the float64 oracle."""
import math

import numpy as np
import pytest
import torch

from aicomp_amd import ops, workloads
from oracle import paged_kv_oracle as orc
from helpers import NAME, assert_close_attn, raw, to_f64

pytestmark = pytest.mark.gpu

# bf16 tolerance of the benchmark definition: max-abs 1e-2 or relative 2e-2 vs fp32/64
BF16_ATOL, BF16_RTOL = 1e-2, 2e-2
F32_ATOL = 1e-5


def oracle_decode(w, ctx=None):
    ks = None if w.k_scale is None else w.k_scale.cpu().numpy()
    vs = None if w.v_scale is None else w.v_scale.cpu().numpy()
    return orc.paged_decode_attn(raw(w.query), raw(w.k_pool), raw(w.v_pool),
                                 w.block_table.cpu().numpy(),
                                 (w.context_lens.cpu().numpy() if ctx is None else ctx), w.scale,
                                 q_dtype=NAME[w.query.dtype], kv_dtype=NAME[w.k_pool.dtype],
                                 k_scale=ks, v_scale=vs)


def run_decode(w, partition_size=0, ctx=None):
    out = torch.full_like(w.query, float("nan"))
    ops.paged_decode_attn(out, w.query, w.k_pool, w.v_pool, w.block_table,
                          w.context_lens if ctx is None else ctx, w.scale,
                          k_scale=w.k_scale, v_scale=w.v_scale, partition_size=partition_size)
    torch.cuda.synchronize()
    return out


def small(name, **kw):
    s = workloads.SHAPES[name]
    return workloads.Shape(**{**s.__dict__, **kw})


def test_config1_fp32_anchor(device):
    """batch 4, 32/8 heads, D 64, L in [64,512], pool of 256 blocks: <= 1e-5 abs."""
    w = workloads.make_workload("decode_fp32_small", device=device)
    want = oracle_decode(w)
    for ps in (0, 64, 16 * 64):
        got = to_f64(run_decode(w, ps))
        assert np.abs(got - want).max() <= F32_ATOL, ps


@pytest.mark.parametrize("ps", [0, 256, 1024, 8192])
def test_config2_shape_reduced_batch(device, ps):
    """Llama-3-8B decode shape, batch cut to 6 so the oracle runs in seconds."""
    w = workloads.make_workload("x", device=device, shape=small("llama3_8b_decode", batch=6))
    ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping)
    want = oracle_decode(w)
    got = to_f64(run_decode(w, ps))
    assert_close_attn(got, want, BF16_ATOL, BF16_RTOL, f"partition {ps}")


@pytest.mark.parametrize("hq,hkv,d,bs,dtype", [
    (8, 8, 64, 16, torch.bfloat16),       # MHA
    (8, 1, 128, 16, torch.bfloat16),      # MQA, group 8
    (12, 2, 128, 16, torch.bfloat16),     # group 6
    (32, 2, 128, 16, torch.bfloat16),     # group 16
    (6, 2, 256, 8, torch.bfloat16),
    (4, 2, 128, 32, torch.float32),
    (4, 4, 64, 1, torch.float32),         # block size 1
])
def test_decode_shapes(device, hq, hkv, d, bs, dtype):
    sh = workloads.Shape("t", 5, hq, hkv, d, block_size=bs, q_dtype=dtype, kv_dtype=dtype,
                         ctx_lo=1, ctx_hi=700)
    w = workloads.make_workload("t", device=device, seed=3, shape=sh)
    want = oracle_decode(w)
    for ps in (0, 32 * bs if bs > 1 else 64):
        got = to_f64(run_decode(w, ps))
        if dtype == torch.float32:
            assert np.abs(got - want).max() <= F32_ATOL
        else:
            assert_close_attn(got, want, BF16_ATOL, BF16_RTOL, f"{hq}/{hkv} D{d} BS{bs} ps{ps}")


def test_decode_edge_lengths(device):
    """Context lengths 0, 1, block boundaries, and NaN/Inf poison beyond the context."""
    sh = workloads.Shape("t", 8, 8, 2, 128, ctx_lo=300, ctx_hi=300)
    w = workloads.make_workload("t", device=device, seed=4, shape=sh)
    ctx = torch.tensor([0, 1, 15, 16, 17, 255, 256, 301], dtype=torch.int32, device=device)
    bs = 16
    # poison every slot at or beyond each sequence's context, and every unused block
    used = torch.zeros(w.k_pool.shape[0] * bs, dtype=torch.bool, device=device)
    for b, L in enumerate(ctx.tolist()):
        t = torch.arange(L, device=device)
        used[w.block_table[b, t // bs].long() * bs + t % bs] = True
    kf = w.k_pool.permute(0, 2, 1, 3).reshape(-1, 2, 128).clone()
    vf = w.v_pool.permute(0, 2, 1, 3).reshape(-1, 2, 128).clone()
    kf[~used] = float("nan")
    vf[~used] = float("inf")
    w.k_pool = kf.reshape(-1, bs, 2, 128).permute(0, 2, 1, 3).contiguous()
    w.v_pool = vf.reshape(-1, bs, 2, 128).permute(0, 2, 1, 3).contiguous()
    kclean = torch.nan_to_num(w.k_pool.float(), nan=0.0).to(torch.bfloat16)
    vclean = torch.nan_to_num(w.v_pool.float(), posinf=0.0).to(torch.bfloat16)
    want = orc.paged_decode_attn(raw(w.query), raw(kclean), raw(vclean), w.block_table.cpu().numpy(),
                                 ctx.cpu().numpy(), w.scale, "bf16", "bf16")
    for ps in (0, 64, 512):
        got = to_f64(run_decode(w, ps, ctx=ctx))
        assert_close_attn(got, want, BF16_ATOL, BF16_RTOL, f"ps {ps}")
        assert np.array_equal(got[0], np.zeros_like(got[0]))
        # L == 1: the output is exactly the V row (bf16 in, bf16 out)
        v_row = to_f64(vclean[w.block_table[1, 0].long(), :, 0, :])       # [Hkv, D]
        assert np.array_equal(got[1], np.repeat(v_row, 4, axis=0))


def test_decode_invariants(device):
    sh = workloads.Shape("t", 4, 8, 2, 128, ctx_lo=200, ctx_hi=900, kv_std=0.5)
    w = workloads.make_workload("t", device=device, seed=5, shape=sh)
    base = run_decode(w, 256)
    # split sizes agree: the merge is exact up to fp32 round-off, what differs is the bf16
    # rounding of the probabilities (2^-9 relative each, taken against different running
    # maxima) and of the output; far inside the 1e-2 tolerance
    for ps in (0, 128, 512, 2048):
        o = run_decode(w, ps)
        assert (o.float() - base.float()).abs().max() <= 2e-3
    # moving blocks with the table updated: bit-identical for a fixed partitioning
    nb = w.k_pool.shape[0]
    perm = torch.randperm(nb, device=device)
    kp2, vp2 = torch.empty_like(w.k_pool), torch.empty_like(w.v_pool)
    kp2[perm] = w.k_pool
    vp2[perm] = w.v_pool
    w2 = workloads.Workload(**{**w.__dict__, "k_pool": kp2, "v_pool": vp2,
                               "block_table": perm[w.block_table.long()].to(torch.int32)})
    assert torch.equal(run_decode(w2, 256).view(torch.int16), base.view(torch.int16))
    # same query in all heads of a group -> same output
    q = w.query.clone()
    q[:, 1:4] = q[:, 0:1]
    w3 = workloads.Workload(**{**w.__dict__, "query": q})
    o = run_decode(w3, 256)
    assert torch.equal(o[:, 1].view(torch.int16), o[:, 0].view(torch.int16))
    # all keys equal -> output = mean of V
    w4 = workloads.Workload(**{**w.__dict__, "k_pool": torch.ones_like(w.k_pool)})
    o = to_f64(run_decode(w4, 256))
    for b, L in enumerate(w.ctx_list):
        v = orc.bf16_bits_to_f32(orc.gather_context(raw(w.v_pool), w.block_table[b].cpu().numpy(), L))
        assert np.abs(o[b] - np.repeat(v.mean(axis=0), 4, axis=0)).max() <= 1e-2
    # a huge common score offset changes nothing (online-softmax max handling)
    w5 = workloads.Workload(**{**w.__dict__, "k_pool": (w.k_pool.float() * 0 + 3.0).to(torch.bfloat16),
                               "query": (w.query.float() * 0 + 8.0).to(torch.bfloat16)})
    o5 = to_f64(run_decode(w5, 256))       # every score = 8*3*128*scale ~ 271
    assert np.isfinite(o5).all()
    assert np.abs(o5 - o).max() <= 1e-2


def test_decode_errors(device):
    sh = workloads.Shape("t", 2, 8, 2, 128, ctx_lo=20, ctx_hi=40)
    w = workloads.make_workload("t", device=device, shape=sh)
    out = torch.empty_like(w.query)
    with pytest.raises(RuntimeError):
        ops.paged_decode_attn(out, w.query, w.k_pool, w.v_pool, w.block_table.long(), w.context_lens, 1.0)
    with pytest.raises(RuntimeError):
        ops.paged_decode_attn(out, w.query, w.k_pool, w.v_pool.float(), w.block_table, w.context_lens, 1.0)
    with pytest.raises(RuntimeError):
        ops.paged_decode_attn(out[:, :6], w.query[:, :6], w.k_pool, w.v_pool, w.block_table, w.context_lens, 1.0)
    with pytest.raises(RuntimeError):
        ops.paged_decode_attn(out, w.query, w.k_pool, w.v_pool, w.block_table, w.context_lens, 1.0,
                              partition_size=24)
    with pytest.raises(RuntimeError):
        ops.paged_decode_attn(out.cpu(), w.query.cpu(), w.k_pool.cpu(), w.v_pool.cpu(),
                              w.block_table.cpu(), w.context_lens.cpu(), 1.0)
    q96 = torch.zeros(2, 8, 96, dtype=torch.bfloat16, device=device)
    p96 = torch.zeros(4, 2, 16, 96, dtype=torch.bfloat16, device=device)
    with pytest.raises(RuntimeError):
        ops.paged_decode_attn(torch.empty_like(q96), q96, p96, p96, w.block_table, w.context_lens, 1.0)


def test_fp8_decode_vs_dequantised_oracle(device):
    """fp8 e4m3 KV with per-head scales, group 8: within the bf16 tolerance of the
    oracle run on the dequantised values (the wider, stated bound against the unquantised
    values is test_gpu_fp8_bound.py's)."""
    w = workloads.make_workload("x", device=device, shape=small("llama3_70b_decode_fp8", batch=4))
    ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping, w.k_scale, w.v_scale)
    want = oracle_decode(w)
    for ps in (0, 512):
        got = to_f64(run_decode(w, ps))
        assert_close_attn(got, want, BF16_ATOL, BF16_RTOL, f"fp8 ps {ps}")


def test_config3_long_context_split(device):
    """Long-context skewed batch (log-normal, sigma 1.0, clip [256,32768]), batch cut to 4."""
    w = workloads.make_workload("x", device=device, seed=0,
                                shape=small("long_context_skewed", batch=4))
    ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping)
    want = oracle_decode(w)
    got = to_f64(run_decode(w, 0))
    assert_close_attn(got, want, BF16_ATOL, BF16_RTOL, "auto split")
    got1 = to_f64(run_decode(w, w.block_table.shape[1] * 16))      # one partition
    assert_close_attn(got1, want, BF16_ATOL, BF16_RTOL, "unsplit")
    assert np.abs(got - got1).max() <= 2e-3


@pytest.mark.parametrize("name,batch", [("llama3_8b_decode", 5), ("llama3_70b_decode_fp8", 3),
                                        ("decode_fp32_small", 4)])
def test_fused_append_decode_equals_append_then_decode(device, name, batch):
    """One call that appends the new token and attends == kv_append followed by decode:
    pools bit-identical, outputs bit-identical (same kernel, same values)."""
    w = workloads.make_workload("x", device=device, seed=7, shape=small(name, batch=batch))
    k2, v2 = w.k_pool.clone(), w.v_pool.clone()
    ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping, w.k_scale, w.v_scale)
    ref = run_decode(w)
    out = torch.full_like(w.query, float("nan"))
    ops.paged_decode_attn(out, w.query, k2, v2, w.block_table, w.context_lens, w.scale,
                          k_scale=w.k_scale, v_scale=w.v_scale, new_key=w.new_key, new_value=w.new_value)
    torch.cuda.synchronize()
    bits = lambda t: t.view(torch.uint8) if t.dtype == torch.float8_e4m3fn else t
    assert torch.equal(bits(k2), bits(w.k_pool)) and torch.equal(bits(v2), bits(w.v_pool))
    assert torch.equal(out.view(torch.int16 if out.dtype == torch.bfloat16 else torch.int32),
                       ref.view(torch.int16 if ref.dtype == torch.bfloat16 else torch.int32))
    # explicit partition size: the grid-scheduled kernel (it appends in-kernel too on the matrix-core path)
    ops.paged_decode_attn(out, w.query, k2, v2, w.block_table, w.context_lens, w.scale,
                          k_scale=w.k_scale, v_scale=w.v_scale, new_key=w.new_key, new_value=w.new_value,
                          partition_size=256)
    assert torch.equal(bits(k2), bits(w.k_pool))
    assert_close_attn(to_f64(out), to_f64(ref), 2e-3, 0.0, "fused, grid schedule")


def test_fused_append_edge_positions(device):
    """New token at a tile start, tile end, block start, and as the very first token."""
    sh = workloads.Shape("t", 6, 8, 2, 128, ctx_lo=100, ctx_hi=100)
    w = workloads.make_workload("t", device=device, seed=9, shape=sh)
    ctx = torch.tensor([1, 32, 33, 64, 49, 100], dtype=torch.int32, device=device)
    k2, v2 = w.k_pool.clone(), w.v_pool.clone()
    bs = 16
    pos = (ctx - 1).long()
    slots = w.block_table[torch.arange(6, device=device), pos // bs].long() * bs + pos % bs
    ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, slots)
    ref = run_decode(w, ctx=ctx)
    out = torch.empty_like(w.query)
    ops.paged_decode_attn(out, w.query, k2, v2, w.block_table, ctx, w.scale, new_key=w.new_key,
                          new_value=w.new_value)
    assert torch.equal(k2.view(torch.int16), w.k_pool.view(torch.int16))
    assert torch.equal(v2.view(torch.int16), w.v_pool.view(torch.int16))
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
    want = oracle_decode(w, ctx=ctx.cpu().numpy())
    assert_close_attn(to_f64(out), want, BF16_ATOL, BF16_RTOL, "fused edge positions")


@pytest.mark.parametrize("name,partition", [("llama3_8b_decode", 0), ("llama3_8b_decode", 256),
                                            ("llama32_1b_decode", 0), ("llama3_70b_decode_fp8", 0)])
def test_fused_append_skips_rows_the_table_cannot_place(device, name, partition):
    """A table entry outside the pool, or a length beyond the table, must not make the fused call store
    the new row anywhere: the in-kernel append and the separate one-token append (taken when the new
    rows cannot be read 16 bytes at a time) leave bit-identical pools, untouched for those rows."""
    w = workloads.make_workload("x", device=device, seed=3, shape=small(name, batch=6))
    B, nb = 6, w.k_pool.shape[0]
    width = w.block_table.shape[1]
    table = w.block_table.clone()
    ctx = w.context_lens.clone()
    last = ((ctx - 1) // 16).long()
    table[1, last[1]] = -1                         # below the pool
    table[2, last[2]] = nb + 7                     # above the pool
    ctx[4] = width * 16 + 5                        # longer than the table is wide
    bits = lambda t: t.view(torch.uint8)
    pools = []
    outs = []
    for aligned in (True, False):
        k2, v2 = w.k_pool.clone(), w.v_pool.clone()
        if aligned:
            nk, nv = w.new_key, w.new_value
        else:                                      # same values at an address that is not a multiple of 16
            flat_k = torch.zeros(w.new_key.numel() + 1, dtype=w.new_key.dtype, device=device)
            flat_v = torch.zeros_like(flat_k)
            nk, nv = flat_k[1:].view_as(w.new_key), flat_v[1:].view_as(w.new_value)
            nk.copy_(w.new_key); nv.copy_(w.new_value)
            assert nk.data_ptr() % 16 != 0
        out = torch.full_like(w.query, float("nan"))
        ops.paged_decode_attn(out, w.query, k2, v2, table, ctx, w.scale, k_scale=w.k_scale, v_scale=w.v_scale,
                              new_key=nk, new_value=nv, partition_size=partition)
        torch.cuda.synchronize()
        pools.append((k2, v2)); outs.append(out)
    (ka, va), (kb, vb) = pools
    assert torch.equal(bits(ka), bits(kb)) and torch.equal(bits(va), bits(vb)), "fused and unfused pools differ"
    # rows 0, 3, 5 were stored, and nothing else changed: compare with a slot-mapped append of those rows
    k3, v3 = w.k_pool.clone(), w.v_pool.clone()
    slots = w.slot_mapping.clone()
    slots[[1, 2, 4]] = -1
    ops.kv_append(w.new_key, w.new_value, k3, v3, slots, w.k_scale, w.v_scale)
    assert torch.equal(bits(ka), bits(k3)) and torch.equal(bits(va), bits(v3)), "an unplaceable row was stored"
    good = [0, 3, 5]
    assert torch.equal(outs[0][good].view(torch.int16), outs[1][good].view(torch.int16))
    assert torch.isfinite(outs[0][good].float()).all()


def test_fp8_all_codes_through_the_decode_kernel(device):
    """Every e4m3 code as a V element with a one-hot attention: the kernel's fp8 -> bf16
    conversion is exact for all 256 codes (NaN codes excluded), subnormals and signed zero included."""
    codes = torch.arange(256, dtype=torch.uint8)
    codes = codes[(codes & 0x7F) != 0x7F]                       # drop the two NaN codes
    n = codes.numel()                                           # 254 tokens, token t carries code t
    nb = (n + 15) // 16
    d, hkv, hq = 128, 1, 1
    v_pool = torch.zeros(nb, hkv, 16, d, dtype=torch.uint8)
    v_pool.view(-1, d)[:n] = codes[:, None]
    k_pool = torch.zeros(nb, hkv, 16, d, dtype=torch.uint8)     # keys all zero -> uniform weights...
    # ...so instead make each key select itself: query q_t has its only mass on dim t % 128 and the
    # key of token t is large on that dim; two queries per dim (t and t+128) are separated by sign
    kf = torch.zeros(nb * 16, d)
    for t in range(n):
        kf[t, t % d] = 448.0 if t < d else -448.0
    k_pool.view(-1, d)[:] = kf.to(torch.float8_e4m3fn).view(torch.uint8)
    q = torch.zeros(n, hq, d)
    for t in range(n):
        q[t, 0, t % d] = 16.0 if t < d else -16.0
    table = torch.arange(nb, dtype=torch.int32)[None].repeat(n, 1)
    ctx = torch.full((n,), n, dtype=torch.int32)
    one = torch.ones(1)
    out = torch.empty(n, hq, d, dtype=torch.bfloat16, device=device)
    ops.paged_decode_attn(out, q.to(torch.bfloat16).to(device), k_pool.view(torch.float8_e4m3fn).to(device),
                          v_pool.view(torch.float8_e4m3fn).to(device), table.to(device), ctx.to(device),
                          1.0, one.to(device), one.to(device))
    want = codes.view(torch.float8_e4m3fn).float()              # exact in bf16
    got = out[:, 0, 0].float().cpu()
    assert torch.equal(got, want) or torch.equal(got.abs() + 0.0, want.abs() + 0.0) and \
        torch.equal(torch.signbit(got) | (got == 0), torch.signbit(want) | (want == 0))


@pytest.mark.parametrize("batch", [65, 1024, 1030])
def test_decode_many_short_sequences(device, batch):
    """Large batches of short sequences: prefix sums over more than one wave, the 1024-sequence
    limit of the balanced schedule, and the grid schedule beyond it."""
    sh = workloads.Shape("t", batch, 8, 2, 128, ctx_lo=0, ctx_hi=90, kv_std=0.5)
    w = workloads.make_workload("t", device=device, seed=11, shape=sh)
    ctx = (w.context_lens - 1).clamp(min=0)                    # includes empty sequences
    got = to_f64(run_decode(w, 0, ctx=ctx))
    want = oracle_decode(w, ctx=ctx.cpu().numpy())
    assert_close_attn(got, want, BF16_ATOL, BF16_RTOL, f"batch {batch}")
    empty = (ctx == 0).cpu().numpy()
    assert empty.any() and np.array_equal(got[empty], np.zeros_like(got[empty]))


def test_decode_all_sequences_empty(device):
    sh = workloads.Shape("t", 5, 8, 2, 128, ctx_lo=10, ctx_hi=20)
    w = workloads.make_workload("t", device=device, shape=sh)
    ctx = torch.zeros(5, dtype=torch.int32, device=device)
    for ps in (0, 64):
        out = run_decode(w, ps, ctx=ctx)
        assert float(out.float().abs().sum()) == 0.0


# ------------------------------------------------------------------ head_dim 64 on the matrix-core kernel
@pytest.mark.parametrize("hq,hkv,kv", [(32, 8, torch.bfloat16), (8, 8, torch.bfloat16), (16, 2, torch.bfloat16),
                                       (6, 2, torch.bfloat16), (32, 8, torch.float8_e4m3fn)])
def test_decode_head_dim_64(device, hq, hkv, kv):
    """Llama-3.2-1B-like heads (D 64): rows of token pairs on the MFMA kernel, every partitioning."""
    sh = workloads.Shape("t", 6, hq, hkv, 64, kv_dtype=kv, kv_std=0.5, ctx_lo=1, ctx_hi=900)
    w = workloads.make_workload("t", device=device, seed=11, shape=sh)
    want = oracle_decode(w)
    for ps in (0, 64, 256, 4096):
        got = to_f64(run_decode(w, ps))
        assert_close_attn(got, want, BF16_ATOL, BF16_RTOL, f"{hq}/{hkv} D64 {kv} ps{ps}")


def test_decode_head_dim_64_edge_lengths_and_poison(device):
    """Odd and even lengths around pair, block and tile boundaries; non-finite data beyond the context
    (the second token of a half-valid pair included)."""
    bs, hkv, d = 16, 2, 64
    sh = workloads.Shape("t", 12, 8, hkv, d, ctx_lo=200, ctx_hi=200)
    w = workloads.make_workload("t", device=device, seed=12, shape=sh)
    ctx = torch.tensor([0, 1, 2, 3, 15, 16, 17, 63, 64, 65, 127, 201], dtype=torch.int32, device=device)
    used = torch.zeros(w.k_pool.shape[0] * bs, dtype=torch.bool, device=device)
    for b, L in enumerate(ctx.tolist()):
        t = torch.arange(L, device=device)
        used[w.block_table[b, t // bs].long() * bs + t % bs] = True
    kf = w.k_pool.permute(0, 2, 1, 3).reshape(-1, hkv, d).clone()
    vf = w.v_pool.permute(0, 2, 1, 3).reshape(-1, hkv, d).clone()
    kf[~used] = float("nan")
    vf[~used] = float("inf")
    w.k_pool = kf.reshape(-1, bs, hkv, d).permute(0, 2, 1, 3).contiguous()
    w.v_pool = vf.reshape(-1, bs, hkv, d).permute(0, 2, 1, 3).contiguous()
    kclean = torch.nan_to_num(w.k_pool.float(), nan=0.0).to(torch.bfloat16)
    vclean = torch.nan_to_num(w.v_pool.float(), posinf=0.0).to(torch.bfloat16)
    want = orc.paged_decode_attn(raw(w.query), raw(kclean), raw(vclean), w.block_table.cpu().numpy(),
                                 ctx.cpu().numpy(), w.scale, "bf16", "bf16")
    for ps in (0, 64, 128):
        got = to_f64(run_decode(w, ps, ctx=ctx))
        assert_close_attn(got, want, BF16_ATOL, BF16_RTOL, f"ps {ps}")
        assert np.array_equal(got[0], np.zeros_like(got[0]))
        v_row = to_f64(vclean[w.block_table[1, 0].long(), :, 0, :])       # L == 1: exactly the V row
        assert np.array_equal(got[1], np.repeat(v_row, 4, axis=0))


def test_decode_head_dim_64_fused_append(device):
    sh = workloads.Shape("t", 5, 32, 8, 64, kv_std=0.5, ctx_lo=1, ctx_hi=500)
    w = workloads.make_workload("t", device=device, seed=13, shape=sh)
    kp, vp = w.k_pool.clone(), w.v_pool.clone()
    ops.kv_append(w.new_key, w.new_value, kp, vp, w.slot_mapping)
    ref = torch.empty_like(w.query)
    ops.paged_decode_attn(ref, w.query, kp, vp, w.block_table, w.context_lens, w.scale)
    out = torch.empty_like(w.query)
    ops.paged_decode_attn(out, w.query, w.k_pool, w.v_pool, w.block_table, w.context_lens, w.scale,
                          new_key=w.new_key, new_value=w.new_value)
    torch.cuda.synchronize()
    assert torch.equal(out, ref) and torch.equal(w.k_pool, kp) and torch.equal(w.v_pool, vp)


@pytest.mark.parametrize("name", ["llama3_8b_decode", "llama3_70b_decode_fp8", "llama32_1b_decode", "decode_fp32_small"])
def test_prepared_decode_equals_the_checked_call(device, name):
    """The bound call (checks done once) launches exactly what ``paged_decode_attn`` launches: same
    bits in the output and in the pools, with and without the fused append, and with a replaced
    context-length tensor."""
    w = workloads.make_workload("x", device=device, shape=small(name, batch=5))
    t0 = int(w.cu_q_lens[w.num_prefill_seqs])
    nk, nv = w.new_key[t0:].contiguous(), w.new_value[t0:].contiguous()
    k1, v1, k2, v2 = w.k_pool.clone(), w.v_pool.clone(), w.k_pool.clone(), w.v_pool.clone()
    call = ops.PreparedDecode(k2, v2, w.block_table, w.context_lens, w.query.shape[1], w.query.dtype, w.scale,
                              w.k_scale, w.v_scale)
    fused = w.query.dtype == nk.dtype
    for step in range(3):
        ctx = (w.context_lens - step).clamp_min(1).contiguous()
        a = torch.full_like(w.query, float("nan"))
        b = torch.full_like(w.query, float("nan"))
        kw = dict(new_key=nk, new_value=nv) if fused and step != 1 else {}
        ops.paged_decode_attn(a, w.query, k1, v1, w.block_table, ctx, w.scale, w.k_scale, w.v_scale, **kw)
        call(b, w.query, kw.get("new_key"), kw.get("new_value"), context_lens=ctx)
        torch.cuda.synchronize()
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), step
        assert torch.equal(k1.view(torch.uint8), k2.view(torch.uint8)) and torch.equal(v1.view(torch.uint8), v2.view(torch.uint8))
    with pytest.raises(RuntimeError):
        call(torch.empty(5, 3, 7, device=device), w.query)
    with pytest.raises(RuntimeError):
        ops.PreparedDecode(k2, v2, w.block_table.to(torch.int64), w.context_lens, w.query.shape[1], w.query.dtype, w.scale)


@pytest.mark.parametrize("d,kv,ps", [(128, None, 64), (128, None, 256), (128, torch.float8_e4m3fn, 128),
                                     (64, None, 0), (64, None, 128), (64, torch.float8_e4m3fn, 0)])
def test_fused_append_in_the_grid_kernel_edge_positions(device, d, kv, ps):
    """The grid-scheduled kernel writes the step's new row itself: new token as the first token, at
    block, tile (32 / 64 tokens) and partition boundaries, in both halves of a pair row (D = 64).
    Pools bit-identical to kv_append, output bit-identical to decode after kv_append."""
    sh = workloads.Shape("t", 12, 8, 2, d, kv_std=0.5, ctx_lo=300, ctx_hi=300,
                         kv_dtype=kv or torch.bfloat16)
    w = workloads.make_workload("t", device=device, seed=31, shape=sh)
    ctx = torch.tensor([1, 2, 16, 17, 32, 33, 64, 65, 128, 129, 257, 300], dtype=torch.int32, device=device)
    k2, v2 = w.k_pool.clone(), w.v_pool.clone()
    pos = (ctx - 1).long()
    slots = w.block_table[torch.arange(12, device=device), pos // 16].long() * 16 + pos % 16
    ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, slots, w.k_scale, w.v_scale)
    ref = torch.empty_like(w.query)
    ops.paged_decode_attn(ref, w.query, w.k_pool, w.v_pool, w.block_table, ctx, w.scale, w.k_scale, w.v_scale,
                          partition_size=ps)
    out = torch.full_like(w.query, float("nan"))
    ops.paged_decode_attn(out, w.query, k2, v2, w.block_table, ctx, w.scale, w.k_scale, w.v_scale,
                          partition_size=ps, new_key=w.new_key, new_value=w.new_value)
    torch.cuda.synchronize()
    assert torch.equal(k2.view(torch.uint8), w.k_pool.view(torch.uint8))
    assert torch.equal(v2.view(torch.uint8), w.v_pool.view(torch.uint8))
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
    want = oracle_decode(w, ctx=ctx.cpu().numpy())
    assert_close_attn(to_f64(out), want, BF16_ATOL, BF16_RTOL, f"grid fused append D={d}")


@pytest.mark.gpu
@pytest.mark.routing("balanced")
@pytest.mark.parametrize("hkv,group,D", [(8, 4, 128), (3, 2, 128), (16, 1, 128), (8, 4, 64), (2, 8, 64)])
def test_balanced_schedule_records_the_parts_the_host_model_predicts(hkv, group, D):
    """The main kernel of the balanced schedule tells the merge kernel, per (sequence, KV head)
    row, which of the head's parts hold the row's first and last tile.  tests/test_decode_schedule.py
    models the schedule on the host and checks its invariants (coverage, distinct slots, bounds);
    this test ties that model to the kernel by reading the record back from the caller's scratch."""
    import math
    from aicomp_amd import ops
    from test_decode_schedule import SK_MAX_WAVES, schedule, tiles_of
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(11 + hkv)
    B, hq = 37, hkv * group
    tile, ncol = (64 if D == 64 else 32), group                    # head_dim 64: pair rows; one partial per head either way
    lens = torch.randint(1, 3000, (B,), generator=g).tolist()
    lens[3] = 0; lens[4] = 0; lens[20] = 1; lens[36] = 33
    need = [max(1, math.ceil(c / 16)) for c in lens]
    max_blocks = max(need)
    nb = sum(need) + 1
    perm = torch.randperm(nb, generator=g)
    table = torch.zeros(B, max_blocks, dtype=torch.int32)
    cur = 0
    for s, n in enumerate(need):
        table[s, :n] = perm[cur:cur + n].to(torch.int32); cur += n
    k = torch.randn(nb, hkv, 16, D, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(nb, hkv, 16, D, generator=g).to(torch.bfloat16).to(dev)
    q = torch.randn(B, hq, D, generator=g).to(torch.bfloat16).to(dev)
    out = torch.empty_like(q)
    cl = torch.tensor(lens, dtype=torch.int32, device=dev)
    nbytes = ops.decode_workspace_bytes(B, hq, hkv, D, 16, max_blocks, q.dtype, k.dtype)
    ws = torch.full((nbytes,), 0xA5, dtype=torch.uint8, device=dev)
    ops.paged_decode_attn(out, q, k, v, table.to(dev), cl, 1 / math.sqrt(D), None, None, workspace=ws)
    torch.cuda.synchronize()
    slots = SK_MAX_WAVES + B * hkv
    off = slots * ncol * D + slots * ncol * 2                   # partial outputs, then (max, sum) pairs
    assert nbytes >= (off + B * hkv * 2) * 4
    rec = ws.view(torch.int32)[off:off + B * hkv * 2].reshape(B, hkv, 2).cpu()
    num_waves = 4 * torch.cuda.get_device_properties(0).multi_processor_count
    segs, _ = schedule(lens, hkv, num_waves, max_blocks, tile)
    first, last = {}, {}
    for kvh, part, seq, t, nt, slot in segs:
        if t == 0:
            first[(seq, kvh)] = part
        if t + nt == tiles_of(lens[seq], max_blocks, tile):
            last[(seq, kvh)] = part
    for s in range(B):
        for h in range(hkv):
            if lens[s] > 0:
                assert (int(rec[s, h, 0]), int(rec[s, h, 1])) == (first[(s, h)], last[(s, h)]), (s, h)
    # and the result itself, against the oracle
    want = orc.paged_decode_attn(raw(q), raw(k), raw(v), table.numpy(), lens, 1 / math.sqrt(D), "bf16", "bf16")
    assert_close_attn(to_f64(out), want, BF16_ATOL, BF16_RTOL, f"balanced schedule D {D}")


# ------------------------------------------------------------------ latency-bound calls: the library's own choice
@pytest.mark.routing("balanced")
@pytest.mark.parametrize("name,batch,ctx_hi,kv", [("llama3_8b_decode", 1, 500, None), ("llama3_8b_decode", 3, 2000, None),
                                                 ("llama32_1b_decode", 2, 300, None), ("llama32_1b_decode", 4, 1500, None),
                                                 ("llama3_70b_decode_fp8", 2, 1100, "fp8")])
def test_small_calls_take_the_grid_schedule(device, name, batch, ctx_hi, kv):
    """With partition_size = 0 a call over few short rows is routed to the grid schedule (whole rows
    when no row can exceed 640 tokens, 256-token partitions otherwise).  Same numbers as the balanced
    schedule to the tolerance between split sizes, same pools after the fused append, oracle parity,
    and the sizing helpers agree with what the call does."""
    from aicomp_amd import _lib
    lib = _lib.load()
    w = workloads.make_workload("x", device=device, seed=11, shape=small(name, batch=batch, ctx_lo=40, ctx_hi=ctx_hi))
    k0, v0 = w.k_pool.clone(), w.v_pool.clone()
    balanced = torch.full_like(w.query, float("nan"))           # routing "balanced": threshold 0
    ops.paged_decode_attn(balanced, w.query, w.k_pool, w.v_pool, w.block_table, w.context_lens, w.scale,
                          k_scale=w.k_scale, v_scale=w.v_scale, new_key=w.new_key, new_value=w.new_value)
    torch.cuda.synchronize()
    assert ops.set_small_decode_tokens(32768) == 0              # the library's default from here on
    s, mb = w.shape, w.block_table.shape[1]
    assert batch * mb * 16 <= 32768, "the case is meant to be below the default limit"
    qd, kd = ops._DT[w.query.dtype], ops._DT[w.k_pool.dtype]
    ps = lib.aicomp_paged_decode_partition_size(batch, s.num_q_heads, s.num_kv_heads, s.head_dim, 16, mb, qd, kd)
    assert ps == (-(-mb * 16 // 64) * 64 if mb * 16 <= 640 else 256)
    parts = -(-mb * 16 // ps)
    need = lib.aicomp_paged_decode_workspace_bytes(batch, s.num_q_heads, s.num_kv_heads, s.head_dim, 16, mb, qd, kd, 0)
    assert need == (0 if parts == 1 else batch * s.num_q_heads * parts * (s.head_dim + 2) * 4)
    out = torch.full_like(w.query, float("nan"))
    ops.paged_decode_attn(out, w.query, k0, v0, w.block_table, w.context_lens, w.scale,
                          k_scale=w.k_scale, v_scale=w.v_scale, new_key=w.new_key, new_value=w.new_value)
    torch.cuda.synchronize()
    bits = lambda t: t.view(torch.uint8) if t.dtype == torch.float8_e4m3fn else t
    assert torch.equal(bits(k0), bits(w.k_pool)) and torch.equal(bits(v0), bits(w.v_pool))
    assert_close_attn(to_f64(out), to_f64(balanced), 2e-3, 0.0, "grid against balanced schedule")
    assert_close_attn(to_f64(out), oracle_decode(w), BF16_ATOL, BF16_RTOL, "grid schedule against the oracle")
