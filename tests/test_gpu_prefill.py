"""Chunked-prefill causal attention through the C ABI vs the float64 oracle."""
import math

import numpy as np
import pytest
import torch

from aicomp_amd import ops, workloads
from oracle import paged_kv_oracle as orc
from helpers import NAME, assert_close_attn, raw, to_f64

pytestmark = pytest.mark.gpu
BF16_ATOL, BF16_RTOL = 1e-2, 2e-2


def build_case(device, priors, news, hq, hkv, d, bs=16, dtype=torch.bfloat16, kv_dtype=None, seed=0,
               poison=True):
    """Random pool + table for sequences with the given prior and chunk lengths."""
    kv_dtype = kv_dtype or dtype
    g = torch.Generator().manual_seed(seed)
    ctx = [p + n for p, n in zip(priors, news)]
    need = [max(1, math.ceil(c / bs)) for c in ctx]
    nb = sum(need) + 7
    perm = torch.randperm(nb, generator=g)
    table = torch.zeros(len(ctx), max(need), dtype=torch.int32)
    cur = 0
    for s, k in enumerate(need):
        table[s, :k] = perm[cur:cur + k].to(torch.int32)
        cur += k
    T = sum(news)
    q = torch.randn(T, hq, d, generator=g).to(dtype)
    kf = (torch.randn(nb, hkv, bs, d, generator=g) * 0.5)
    vf = (torch.randn(nb, hkv, bs, d, generator=g) * 0.5)
    ks = vs = None
    if kv_dtype == torch.float8_e4m3fn:
        ks = (kf.abs().amax(dim=(0, 2, 3)) / 448).float()
        vs = (vf.abs().amax(dim=(0, 2, 3)) / 448).float()
        k_pool = (kf / ks[None, :, None, None]).to(kv_dtype)
        v_pool = (vf / vs[None, :, None, None]).to(kv_dtype)
    else:
        k_pool, v_pool = kf.to(kv_dtype), vf.to(kv_dtype)
        if poison and (kv_dtype != torch.float32 or poison == "all"):
            # every slot at or beyond a sequence's context is non-finite
            used = torch.zeros(nb * bs, dtype=torch.bool)
            for s, c in enumerate(ctx):
                t = torch.arange(c)
                used[table[s, t // bs].long() * bs + t % bs] = True
            kflat = k_pool.permute(0, 2, 1, 3).reshape(nb * bs, hkv, d).clone()
            vflat = v_pool.permute(0, 2, 1, 3).reshape(nb * bs, hkv, d).clone()
            kflat[~used] = float("nan")
            vflat[~used] = float("inf")
            k_pool = kflat.reshape(nb, bs, hkv, d).permute(0, 2, 1, 3).contiguous()
            v_pool = vflat.reshape(nb, bs, hkv, d).permute(0, 2, 1, 3).contiguous()
    cu = torch.tensor([0] + list(np.cumsum(news)), dtype=torch.int32)
    dev = lambda t: None if t is None else t.to(device)
    return dict(q=dev(q), k_pool=dev(k_pool), v_pool=dev(v_pool), table=dev(table),
                ctx=dev(torch.tensor(ctx, dtype=torch.int32)), cu=dev(cu), ks=dev(ks), vs=dev(vs),
                scale=1 / math.sqrt(d), news=news, ctx_list=ctx)


def oracle(c):
    kp = torch.nan_to_num(c["k_pool"].float().cpu(), nan=0.0, posinf=0.0).to(c["k_pool"].dtype)
    vp = torch.nan_to_num(c["v_pool"].float().cpu(), nan=0.0, posinf=0.0).to(c["v_pool"].dtype)
    return orc.paged_prefill_attn(raw(c["q"]), raw(kp), raw(vp), c["table"].cpu().numpy(), c["ctx_list"],
                                  c["cu"].cpu().numpy(), c["scale"], NAME[c["q"].dtype],
                                  NAME[c["k_pool"].dtype],
                                  None if c["ks"] is None else c["ks"].cpu().numpy(),
                                  None if c["vs"] is None else c["vs"].cpu().numpy())


def run(c, max_q_len=None):
    out = torch.full_like(c["q"], float("nan"))
    ops.paged_prefill_attn(out, c["q"], c["k_pool"], c["v_pool"], c["table"], c["ctx"], c["cu"],
                           c["scale"], max_q_len=max_q_len, k_scale=c["ks"], v_scale=c["vs"])
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("hq,hkv", [(8, 2), (4, 4), (16, 2), (6, 2), (16, 1)])
def test_prefill_small_ragged(device, hq, hkv):
    """Ragged chunks: prior 0, prior inside a block, chunk of 1, chunk crossing tiles."""
    c = build_case(device, priors=[0, 5, 37, 200, 0, 63], news=[70, 1, 33, 17, 1, 130], hq=hq, hkv=hkv, d=128)
    got = to_f64(run(c, max_q_len=130))
    assert_close_attn(got, oracle(c), BF16_ATOL, BF16_RTOL, f"{hq}/{hkv}")


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("ctx", [33, 63, 64, 65, 80, 127, 128, 129, 191, 193, 256, 300])
def test_prefill_tiles_loaded_straight_into_lds(device, ctx, d):
    """bf16 pools, >= 128 rows per chunk: the kernels whose 64-token tiles go from the pool
    straight into LDS.  Context lengths around the tile and block boundaries, as a fresh prompt and
    as a second chunk; every slot beyond a context is NaN (K) / Inf (V), and the table is exactly
    as wide as the longest sequence needs (a tile's block ids then run past its end)."""
    n2 = min(ctx, 40)
    c = build_case(device, priors=[0, ctx - n2], news=[ctx, n2], hq=8, hkv=2, d=d, seed=ctx)
    got = to_f64(run(c, max_q_len=ctx))
    assert_close_attn(got, oracle(c), BF16_ATOL, BF16_RTOL, f"ctx {ctx} D {d}")


@pytest.mark.parametrize("d", [128, 64])
def test_prefill_items_taken_in_cost_order(device, d):
    """2 to 16 chunks: workgroups take (chunk, query tile) items by rank of cost, not by grid
    position.  Chunks of very different prior context and length, one of them empty, equal costs
    across chunks, more tiles in the grid than most chunks have: every row must still be computed
    exactly once (the output starts as NaN)."""
    priors = [1900, 0, 300, 300, 77, 1024, 0, 512, 5]
    news = [512, 512, 40, 40, 0, 130, 1, 200, 333]
    c = build_case(device, priors=priors, news=news, hq=8, hkv=2, d=d, seed=5)
    got = run(c, max_q_len=512)
    assert torch.isfinite(got.float()).all()
    assert_close_attn(to_f64(got), oracle(c), BF16_ATOL, BF16_RTOL, f"cost order D {d}")
    # sixteen chunks, and seventeen (which keeps the grid order)
    for nseq in (16, 17):
        pr = [(i * 211) % 700 for i in range(nseq)]
        nw = [32 + (i * 37) % 150 for i in range(nseq)]
        c = build_case(device, priors=pr, news=nw, hq=8, hkv=2, d=d, seed=nseq)
        assert_close_attn(to_f64(run(c, max_q_len=max(nw))), oracle(c), BF16_ATOL, BF16_RTOL, f"{nseq} chunks D {d}")


def test_prefill_reductions(device):
    c = build_case(device, priors=[0, 300], news=[96, 1], hq=8, hkv=2, d=128, poison=False)
    got = run(c)
    # prior 0: torch's is_causal=True on the gathered K/V, the reference's prefill call
    L = 96
    blocks = c["table"][0, : L // 16].long()
    k = c["k_pool"][blocks].permute(1, 0, 2, 3).reshape(2, L, 128).float().cpu()
    v = c["v_pool"][blocks].permute(1, 0, 2, 3).reshape(2, L, 128).float().cpu()
    q = c["q"][:L].float().cpu().permute(1, 0, 2)[None]
    want = torch.nn.functional.scaled_dot_product_attention(
        q, k.repeat_interleave(4, 0)[None], v.repeat_interleave(4, 0)[None], is_causal=True)
    assert_close_attn(to_f64(got[:L]), want[0].permute(1, 0, 2).double().numpy(), BF16_ATOL, BF16_RTOL, "causal")
    # chunk of one token: the decode kernel on the same sequence
    out_d = torch.empty(1, 8, 128, dtype=torch.bfloat16, device=device)
    ops.paged_decode_attn(out_d, c["q"][L:L + 1], c["k_pool"], c["v_pool"], c["table"][1:2].contiguous(),
                          c["ctx"][1:2].contiguous(), c["scale"])
    assert (out_d[0].float() - got[L].float()).abs().max() <= 2e-3


def test_prefill_fp32_and_other_shapes_use_the_generic_kernel(device):
    c = build_case(device, priors=[0, 9], news=[20, 7], hq=4, hkv=2, d=64, bs=8, dtype=torch.float32)
    got = to_f64(run(c))
    assert np.abs(got - oracle(c)).max() <= 1e-5


@pytest.mark.parametrize("hq,hkv,d,bs", [(8, 2, 128, 16), (4, 4, 64, 16), (6, 2, 128, 16), (16, 2, 64, 32),
                                         (4, 1, 256, 16), (32, 8, 64, 16), (16, 1, 128, 16), (16, 2, 128, 16)])
def test_prefill_fp32_kernels(device, hq, hkv, d, bs):
    """float32 models (the reference's ``--dtype float32``) take the float32 matrix-instruction kernel
    (head_dim 64 / 128, block 16) or the tiled vector kernel (the rest): a fresh 512-token prompt, a
    continuation across tile and block boundaries, ragged and one-token chunks, groups of 1, 3 (one
    head per workgroup), 4, 8 and 16; <= 1e-5 against the float64 oracle."""
    c = build_case(device, priors=[0, 300, 5, 0, 63, 31], news=[512, 130, 33, 1, 1, 70], hq=hq, hkv=hkv, d=d, bs=bs,
                   dtype=torch.float32, seed=d + bs)
    got = run(c, max_q_len=512)
    assert torch.isfinite(got).all()
    assert np.abs(to_f64(got) - oracle(c)).max() <= 1e-5


@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (8, 8, 64), (3, 1, 128)])
def test_prefill_fp32_matrix_kernel_ignores_everything_beyond_the_context(device, hq, hkv, d):
    """float32 pools with NaN in every K slot and Inf in every V slot at or beyond a sequence's
    context (tile tails, table padding): none of it may reach the output.  Priors and lengths put
    the context end at every position of a 32-token tile's two blocks."""
    c = build_case(device, priors=[0, 17, 31, 100, 3], news=[33, 16, 1, 61, 160], hq=hq, hkv=hkv, d=d,
                   dtype=torch.float32, seed=7 + d, poison="all")
    got = run(c, max_q_len=160)
    assert torch.isfinite(got).all()
    assert np.abs(to_f64(got) - oracle(c)).max() <= 1e-5


@pytest.mark.parametrize("n,dtype", [(1024, torch.bfloat16), (1500, torch.bfloat16), (2048, torch.bfloat16),
                                     (1500, torch.float32), (700, torch.float16)])
def test_single_prompt_whose_grid_is_resident_at_once(device, n, dtype):
    """A fresh prompt of at most two workgroups per CU takes its query tiles in paired order (an
    expensive and a cheap tile per CU): one round, two full rounds, and a second round that is only
    partly filled.  Every row must still be computed exactly once (the output starts as NaN) and
    match the float64 oracle."""
    c = build_case(device, priors=[0], news=[n], hq=32, hkv=8, d=128, dtype=dtype, seed=n, poison=False)
    got = run(c)
    assert torch.isfinite(got.float()).all()
    want = orc.paged_prefill_attn(raw(c["q"]), raw(c["k_pool"]), raw(c["v_pool"]), c["table"].cpu().numpy(), [n], [0, n],
                                  c["scale"], NAME[dtype], NAME[dtype], gather=orc.gather_context_fast)
    if dtype == torch.float32:
        assert np.abs(to_f64(got) - want).max() <= 1e-5
    else:
        assert_close_attn(to_f64(got), want, BF16_ATOL, BF16_RTOL, f"{n}-token prompt, {dtype}")


def test_prefill_fp32_long_prompt_all_rows(device):
    """A fresh 2048-token float32 prompt at the Llama-3 head shape (the bench's float32 shape): every
    row within 1e-5 of the float64 oracle, and equal to torch's own is_causal=True float32 SDPA on
    the gathered K/V to float32 round-off."""
    n = 2048
    c = build_case(device, priors=[0], news=[n], hq=32, hkv=8, d=128, dtype=torch.float32, seed=9)
    got = run(c)
    want = orc.paged_prefill_attn(raw(c["q"]), raw(c["k_pool"]), raw(c["v_pool"]), c["table"].cpu().numpy(), [n], [0, n],
                                  c["scale"], "f32", "f32", gather=orc.gather_context_fast)
    assert np.abs(to_f64(got) - want).max() <= 1e-5
    blocks = c["table"][0, : n // 16].long()
    k = c["k_pool"][blocks].permute(1, 0, 2, 3).reshape(8, n, 128)
    v = c["v_pool"][blocks].permute(1, 0, 2, 3).reshape(8, n, 128)
    ref = torch.nn.functional.scaled_dot_product_attention(
        c["q"].permute(1, 0, 2)[None], k.repeat_interleave(4, 0)[None], v.repeat_interleave(4, 0)[None], is_causal=True)
    assert (ref[0].permute(1, 0, 2) - got).abs().max().item() <= 2e-5


@pytest.mark.parametrize("dtype,kv_dtype,d,bs", [(torch.bfloat16, None, 256, 16), (torch.bfloat16, None, 128, 32),
                                                 (torch.float16, None, 256, 16),
                                                 (torch.bfloat16, torch.float8_e4m3fn, 256, 16),
                                                 (torch.float16, torch.float8_e4m3fn, 128, 8)])
def test_prefill_16bit_shapes_outside_the_matrix_core_kernel(device, dtype, kv_dtype, d, bs):
    """head_dim 256 and block sizes other than 16 with 16-bit queries: the tiled kernel widens the pool
    rows to float32 in LDS; NaN / Inf beyond every context must not reach the output."""
    c = build_case(device, priors=[0, 200, 37], news=[300, 64, 17], hq=8, hkv=2, d=d, bs=bs, dtype=dtype,
                   kv_dtype=kv_dtype, seed=3)
    got = run(c, max_q_len=300)
    assert torch.isfinite(got.float()).all()
    assert_close_attn(to_f64(got), oracle(c), BF16_ATOL, BF16_RTOL, f"tiled {dtype} D {d} BS {bs}")


def test_prefill_fp8_kv(device):
    c = build_case(device, priors=[0, 100], news=[64, 40], hq=16, hkv=2, d=128, kv_dtype=torch.float8_e4m3fn)
    got = to_f64(run(c))
    assert_close_attn(got, oracle(c), BF16_ATOL, BF16_RTOL, "fp8 prefill")


def test_config4_chunked_prefill_reduced(device):
    """4 chunks of 512 new tokens, prior uniform in [0,2048], 32/8 heads: the named shape with the
    decode tail cut to 2 sequences; append of all new rows first (bit-exact), then prefill."""
    s = workloads.SHAPES["chunked_prefill_mixed"]
    w = workloads.make_workload("x", device=device, shape=workloads.Shape(**{**s.__dict__, "batch": 2}))
    ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping)
    sm, bs = w.slot_mapping, 16
    assert torch.equal(w.k_pool[sm // bs, :, sm % bs, :].view(torch.int16), w.new_key.view(torch.int16))
    npre = w.num_prefill_seqs
    T = int(w.cu_q_lens[npre])
    out = torch.empty(T, 32, 128, dtype=torch.bfloat16, device=device)
    ops.paged_prefill_attn(out, w.query[:T].contiguous(), w.k_pool, w.v_pool,
                           w.block_table[:npre].contiguous(), w.context_lens[:npre].contiguous(),
                           w.cu_q_lens[:npre + 1].contiguous(), w.scale, max_q_len=512)
    torch.cuda.synchronize()
    # every row of every chunk against the float64 oracle
    want = orc.paged_prefill_attn(raw(w.query[:T]), raw(w.k_pool), raw(w.v_pool), w.block_table.cpu().numpy()[:npre],
                                  w.ctx_list[:npre], w.cu_q_lens.cpu().numpy()[:npre + 1], w.scale, "bf16", "bf16",
                                  gather=orc.gather_context_fast)
    assert_close_attn(to_f64(out), want, BF16_ATOL, BF16_RTOL, "all rows of the four chunks")


# ------------------------------------------------------------------ head_dim 64 on the matrix-core kernel
@pytest.mark.parametrize("hq,hkv,kv", [(8, 2, None), (4, 4, None), (32, 8, None), (6, 2, None), (16, 1, None),
                                       (16, 2, torch.float8_e4m3fn)])
def test_prefill_head_dim_64(device, hq, hkv, kv):
    """Llama-3.2-1B-like heads: ragged chunks with odd priors and lengths (both token parities on the
    diagonal), non-finite poison beyond every context."""
    c = build_case(device, priors=[0, 5, 37, 200, 0, 63, 1], news=[70, 1, 33, 17, 1, 130, 2], hq=hq, hkv=hkv, d=64,
                   kv_dtype=kv, seed=21)
    got = to_f64(run(c, max_q_len=130))
    assert_close_attn(got, oracle(c), BF16_ATOL, BF16_RTOL, f"D64 {hq}/{hkv}")


def test_prefill_head_dim_64_long_chunks(device):
    # two column groups per wave (chunks of >= 64 rows), several 64-token tiles, a chunk of 512
    c = build_case(device, priors=[0, 333], news=[512, 200], hq=8, hkv=2, d=64, seed=22)
    got = to_f64(run(c))
    assert_close_attn(got, oracle(c), BF16_ATOL, BF16_RTOL, "D64 long")
    # prior 0: torch's is_causal=True on the gathered K/V
    L = 512
    blocks = c["table"][0, : L // 16].long()
    k = c["k_pool"][blocks].permute(1, 0, 2, 3).reshape(2, L, 64).float().cpu()
    v = c["v_pool"][blocks].permute(1, 0, 2, 3).reshape(2, L, 64).float().cpu()
    q = c["q"][:L].float().cpu().permute(1, 0, 2)[None]
    want = torch.nn.functional.scaled_dot_product_attention(
        q, k.repeat_interleave(4, 0)[None], v.repeat_interleave(4, 0)[None], is_causal=True)
    assert_close_attn(got[:L], want[0].permute(1, 0, 2).double().numpy(), BF16_ATOL, BF16_RTOL, "causal D64")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_prefill_context_shorter_than_chunk_gives_zero_rows(device, dtype):
    """A sequence whose context length is smaller than its chunk (an inconsistent plan) must not
    leave its output rows unwritten: both kernels define them as zero, the other chunks are unaffected."""
    c = build_case(device, priors=[10, 0, 33], news=[130, 140, 20], hq=8, hkv=2, d=128, dtype=dtype, poison=False)
    want = oracle(c)
    ctx = c["ctx"].clone()
    ctx[1] = 100                                   # 140 new rows, but only 100 tokens of context
    c2 = dict(c, ctx=ctx)
    got = run(c2, max_q_len=140)
    lo, hi = int(c["cu"][1]), int(c["cu"][2])
    assert float(got[lo:hi].float().abs().max()) == 0.0
    keep = np.r_[0:lo, hi:got.shape[0]]
    tol = (BF16_ATOL, BF16_RTOL) if dtype == torch.bfloat16 else (1e-5, 0.0)
    assert_close_attn(to_f64(got)[keep], want[keep], tol[0], tol[1], "chunks beside the inconsistent one")


def test_long_prompt_all_rows_and_scaling_in_v(device):
    """One fresh prompt of 4096 tokens at the Llama-3-8B head shape (the size class of the long-prompt
    bench shapes): every row against the float64 oracle, and the size-independent property that
    doubling V doubles the output bit for bit (the probabilities do not depend on V, and a factor of
    two is exact in bf16)."""
    n = 4096
    c = build_case(device, priors=[0], news=[n], hq=32, hkv=8, d=128, seed=31, poison=True)
    got = run(c)
    assert torch.isfinite(got.float()).all()
    c2 = dict(c, v_pool=(c["v_pool"].float() * 2).to(torch.bfloat16))
    got2 = run(c2)
    assert torch.equal((got.float() * 2).to(torch.bfloat16).view(torch.int16), got2.view(torch.int16))
    kp = torch.nan_to_num(c["k_pool"].float().cpu(), nan=0.0, posinf=0.0).to(torch.bfloat16)
    vp = torch.nan_to_num(c["v_pool"].float().cpu(), nan=0.0, posinf=0.0).to(torch.bfloat16)
    want = orc.paged_prefill_attn(raw(c["q"]), raw(kp), raw(vp), c["table"].cpu().numpy(), [n], [0, n], c["scale"],
                                  "bf16", "bf16", gather=orc.gather_context_fast)
    assert_close_attn(to_f64(got), want, BF16_ATOL, BF16_RTOL, "4096-token prompt, all rows")


# ------------------------------------------------------------------ caller-ranked item lists
@pytest.mark.parametrize("dtype,kv,d,hq,hkv", [(torch.bfloat16, None, 128, 32, 8), (torch.bfloat16, None, 64, 8, 2),
                                               (torch.bfloat16, torch.float8_e4m3fn, 128, 16, 2),
                                               (torch.float16, None, 128, 6, 2), (torch.float32, None, 128, 8, 2),
                                               (torch.float32, None, 64, 4, 4), (torch.bfloat16, None, 256, 4, 1)])
def test_prefill_with_a_caller_ranked_item_list_equals_grid_order(device, dtype, kv, d, hq, hkv):
    """aicomp_paged_prefill_attn_items: the same launch with its (sequence, query tile) pairs in the
    order a planner ranks them.  Bit for bit the result of the plain call, on ragged chunk batches
    (lengths 1 to 300, priors 0 to 700, an empty chunk), for every kernel that takes a list, with
    chunk bounds that select one and two column groups per wave; pairs that name no sequence or no
    tile are skipped; a kernel that takes no list (head_dim 256) ignores it."""
    priors = [0, 700, 33, 5, 0, 310, 64, 1, 200, 17]
    for news in ([300, 1, 40, 130, 0, 64, 17, 2, 96, 33], [20, 1, 16, 7, 0, 3, 17, 2, 9, 12]):
        c = build_case(device, priors, news, hq, hkv, d, dtype=dtype, kv_dtype=kv, seed=len(news) + d)
        plain = run(c, max_q_len=max(news))
        tile = ops.prefill_tile_positions(hq, hkv, d, 16, dtype, c["k_pool"].dtype, max(news))
        assert (tile == 0) == (d == 256)
        items = ops.prefill_items(c["ctx_list"], news, tile or 32, num_head_groups=hq // (hq // hkv), num_cus=256)
        junk = np.array([[-1, 0], [len(news), 0], [0, 1000], [3, -2]], dtype=np.int32)
        items = np.concatenate([junk[:2], items, junk[2:]])
        out = torch.full_like(c["q"], float("nan"))
        ops.paged_prefill_attn(out, c["q"], c["k_pool"], c["v_pool"], c["table"], c["ctx"], c["cu"], c["scale"],
                               max_q_len=max(news), k_scale=c["ks"], v_scale=c["vs"],
                               items=torch.from_numpy(items).to(device))
        torch.cuda.synchronize()
        bits = lambda t: t.view(torch.int16) if t.element_size() == 2 else t
        assert torch.equal(bits(out), bits(plain)), (dtype, kv, d, news[0])
    # the registered operator takes the same list
    t = __import__("aicomp_amd")._lib.torch_ops()
    out2 = torch.full_like(c["q"], float("nan"))
    t.paged_prefill_attn(out2, c["q"], c["k_pool"], c["v_pool"], c["table"], c["ctx"], c["cu"], c["scale"], max(news),
                         c["ks"], c["vs"], torch.from_numpy(items).to(device))
    torch.cuda.synchronize()
    assert torch.equal(bits(out2), bits(plain))


def test_item_list_longer_than_a_grid_dimension_is_ignored(device):
    """More than 65535 pairs do not fit the launch grid's second dimension: the call then walks the
    whole grid as the plain call does (the header says so), whatever the list holds."""
    c = build_case(device, [5, 40], [70, 33], 8, 2, 128, seed=9)
    plain = run(c, max_q_len=70)
    items = torch.full((70000, 2), -7, dtype=torch.int32, device=device)
    out = torch.full_like(c["q"], float("nan"))
    ops.paged_prefill_attn(out, c["q"], c["k_pool"], c["v_pool"], c["table"], c["ctx"], c["cu"], c["scale"],
                           max_q_len=70, items=items)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), plain.view(torch.int16))
