"""Seeded synthetic workloads for the paged KV-cache attention path.

The five shapes are the ones the benchmark definition names (decode parity
anchor in fp32, Llama-3-8B decode, long-context skewed batch, chunked prefill
mixed with decode, Llama-3-70B per-GPU decode with fp8 KV).  Lengths and block
tables come from a CPU ``torch.Generator`` so they are identical on every
machine; tensor payloads are drawn on the target device from a seeded
generator of that device.

Pool layout everywhere: ``[num_blocks, Hkv, block_size, D]``; token t of
sequence b lives at slot ``block_table[b, t // BS] * BS + t % BS``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import torch

FP8_MAX = 448.0


@dataclass
class Shape:
    name: str
    batch: int
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    block_size: int = 16
    q_dtype: torch.dtype = torch.bfloat16
    kv_dtype: torch.dtype = torch.bfloat16
    kv_std: float = 1.0
    pool_blocks: Optional[int] = None      # fixed pool size, else total + 10 %
    ctx: str = "uniform"                   # "uniform" | "lognormal"
    ctx_lo: int = 0
    ctx_hi: int = 0
    ctx_median: int = 0
    ctx_sigma: float = 1.0
    prefill_chunks: int = 0
    chunk_len: int = 0
    prior_lo: int = 0
    prior_hi: int = 0


SHAPES: Dict[str, Shape] = {
    # batch 4, fp32, 32/8 heads, D 64, L in [64,512], pool of 256 blocks
    "decode_fp32_small": Shape("decode_fp32_small", 4, 32, 8, 64, q_dtype=torch.float32,
                               kv_dtype=torch.float32, kv_std=1.0, pool_blocks=256,
                               ctx_lo=64, ctx_hi=512),
    # Llama-3-8B decode: batch 64, bf16, 32/8 heads, D 128, L in [512,4096]
    "llama3_8b_decode": Shape("llama3_8b_decode", 64, 32, 8, 128, kv_std=0.5,
                              ctx_lo=512, ctx_hi=4096),
    # Llama-3.2-1B decode (the model of the reference's examples): head_dim 64, same batch and contexts
    "llama32_1b_decode": Shape("llama32_1b_decode", 64, 32, 8, 64, kv_std=0.5,
                               ctx_lo=512, ctx_hi=4096),
    # long-context skewed batch: batch 16, log-normal median 4096, sigma 1.0
    "long_context_skewed": Shape("long_context_skewed", 16, 32, 8, 128, kv_std=0.5,
                                 ctx="lognormal", ctx_lo=256, ctx_hi=32768,
                                 ctx_median=4096, ctx_sigma=1.0),
    # 4 prefill chunks of 512 (prior in [0,2048]) + 60 decode sequences
    "chunked_prefill_mixed": Shape("chunked_prefill_mixed", 60, 32, 8, 128, kv_std=0.5,
                                   ctx_lo=512, ctx_hi=4096, prefill_chunks=4,
                                   chunk_len=512, prior_lo=0, prior_hi=2048),
    # Llama-3-70B per-GPU decode, fp8 e4m3 KV: batch 128, 64/8 heads, L in [1024,8192]
    "llama3_70b_decode_fp8": Shape("llama3_70b_decode_fp8", 128, 64, 8, 128,
                                   kv_dtype=torch.float8_e4m3fn, kv_std=1.0,
                                   ctx_lo=1024, ctx_hi=8192),
}


@dataclass
class Workload:
    shape: Shape
    scale: float
    # one step = append `new_key/new_value` at `slot_mapping`, then attend
    query: torch.Tensor                 # [T, Hq, D]
    new_key: torch.Tensor               # [T, Hkv, D]  (q dtype; quantised on append for fp8)
    new_value: torch.Tensor
    k_pool: torch.Tensor                # [num_blocks, Hkv, BS, D]
    v_pool: torch.Tensor
    block_table: torch.Tensor           # [S, max_blocks] int32
    context_lens: torch.Tensor          # [S] int32, AFTER the append
    slot_mapping: torch.Tensor          # [T] int64
    cu_q_lens: torch.Tensor             # [S+1] int32 new tokens per sequence (prefix sums)
    num_prefill_seqs: int = 0           # the first sequences are prefill chunks
    k_scale: Optional[torch.Tensor] = None   # [Hkv] fp32 (fp8 pools only)
    v_scale: Optional[torch.Tensor] = None
    ctx_list: List[int] = field(default_factory=list)
    new_list: List[int] = field(default_factory=list)

    @property
    def num_seqs(self) -> int:
        return len(self.ctx_list)

    def decode_kv_bytes(self) -> int:
        """Algorithmic bytes of the decode part: K and V rows of every context
        token, query and output rows, the block-table entries and lengths."""
        s = self.shape
        e_kv = self.k_pool.element_size()
        e_q = self.query.element_size()
        total = 0
        for L, n in zip(self.ctx_list, self.new_list):
            if n != 1:
                continue
            total += 2 * L * s.num_kv_heads * s.head_dim * e_kv
            total += 2 * s.num_q_heads * s.head_dim * e_q
            total += math.ceil(L / s.block_size) * 4 + 4
            if self.k_scale is not None:
                total += 2 * s.num_kv_heads * 4
        return total

    def append_bytes(self) -> int:
        s = self.shape
        T = int(self.slot_mapping.numel())
        return T * (2 * s.num_kv_heads * s.head_dim * self.new_key.element_size()
                    + 2 * s.num_kv_heads * s.head_dim * self.k_pool.element_size() + 8)

    def prefill_flops(self) -> int:
        s = self.shape
        fl = 0
        for L, n in zip(self.ctx_list, self.new_list):
            if n <= 1:
                continue
            prior = L - n
            fl += 4 * s.num_q_heads * s.head_dim * (n * prior + n * (n + 1) // 2)
        return fl


def _context_lengths(shape: Shape, g: torch.Generator) -> List[int]:
    if shape.ctx == "uniform":
        return torch.randint(shape.ctx_lo, shape.ctx_hi + 1, (shape.batch,), generator=g).tolist()
    z = torch.randn(shape.batch, generator=g, dtype=torch.float64)
    L = torch.exp(math.log(shape.ctx_median) + shape.ctx_sigma * z).round()
    return L.clamp(shape.ctx_lo, shape.ctx_hi).long().tolist()


def _fp8_source_chunks(pool_shape, dev: torch.device, seed: int):
    """The N(0,1) data an fp8 pool is quantised from, a few thousand blocks at a time:
    yields (first block, blocks, K chunk, V chunk) in float32, the same values on every pass."""
    pool_blocks, hkv, bs, d = pool_shape
    step = max(1, (1 << 24) // (hkv * bs * d))
    sg = torch.Generator(device=dev).manual_seed(seed + 2)
    for i in range(0, pool_blocks, step):
        m = min(step, pool_blocks - i)
        kk = torch.randn(m, hkv, bs, d, generator=sg, device=dev)
        vv = torch.randn(m, hkv, bs, d, generator=sg, device=dev)
        yield i, m, kk, vv


def unquantised_context(w: "Workload", seqs: Sequence[int], seed: int = 0):
    """For an fp8 workload built by ``make_workload(..., seed=seed)``: the float32 K and V rows,
    before quantisation, of the given sequences' contexts, the step's new token included
    (``[(K [L, Hkv, D], V [L, Hkv, D]), ...]`` on the workload's device).  What the fp8 path's
    error against the unquantised model is measured from."""
    if w.k_pool.dtype != torch.float8_e4m3fn:
        raise ValueError("unquantised_context is for fp8 workloads")
    dev, bs = w.k_pool.device, w.shape.block_size
    tables = w.block_table.cpu()
    want = []
    for s in seqs:
        L = w.ctx_list[s]
        t = torch.arange(L)
        want.append((tables[s, t // bs].long(), t % bs))
    outs = [(torch.empty(w.ctx_list[s], w.k_pool.shape[1], w.k_pool.shape[3], device=dev),
             torch.empty(w.ctx_list[s], w.k_pool.shape[1], w.k_pool.shape[3], device=dev)) for s in seqs]
    for i, m, kk, vv in _fp8_source_chunks(tuple(w.k_pool.shape), dev, seed):
        for (blk, off), (ko, vo) in zip(want, outs):
            hit = ((blk >= i) & (blk < i + m)).nonzero().flatten()
            if hit.numel():
                b, o = (blk[hit] - i).to(dev), off[hit].to(dev)
                ko[hit.to(dev)] = kk[b, :, o, :]
                vo[hit.to(dev)] = vv[b, :, o, :]
    cu = w.cu_q_lens.cpu().tolist()
    for s, (ko, vo) in zip(seqs, outs):               # the step's own rows come from new_key / new_value
        n = w.new_list[s]
        ko[w.ctx_list[s] - n:] = w.new_key[cu[s]:cu[s] + n].float()
        vo[w.ctx_list[s] - n:] = w.new_value[cu[s]:cu[s] + n].float()
    return outs


def make_workload(name: str, device="cpu", seed: int = 0, shape: Optional[Shape] = None) -> Workload:
    """Build one step of the named workload.

    ``ctx`` drawn from the shape is the PRIOR length of each decode sequence;
    the step appends one token, so the attended context is prior + 1.  Prefill
    chunks (if any) come first in sequence order: prior P_k, then ``chunk_len``
    new tokens.
    """
    shape = shape or SHAPES[name]
    g = torch.Generator().manual_seed(seed)
    bs = shape.block_size
    priors: List[int] = []
    news: List[int] = []
    if shape.prefill_chunks:
        pri = torch.randint(shape.prior_lo, shape.prior_hi + 1, (shape.prefill_chunks,), generator=g)
        priors += pri.tolist()
        news += [shape.chunk_len] * shape.prefill_chunks
    dec = _context_lengths(shape, g)
    priors += dec
    news += [1] * len(dec)
    ctx = [p + n for p, n in zip(priors, news)]
    need = [math.ceil(c / bs) for c in ctx]
    total_blocks = sum(need)
    pool_blocks = shape.pool_blocks or math.ceil(1.1 * total_blocks)
    if total_blocks > pool_blocks:
        raise ValueError(f"pool of {pool_blocks} blocks cannot hold {total_blocks}")
    perm = torch.randperm(pool_blocks, generator=g)
    max_blocks = max(need)
    table = torch.zeros(len(ctx), max_blocks, dtype=torch.int32)
    cur = 0
    for s, nblk in enumerate(need):
        table[s, :nblk] = perm[cur:cur + nblk].to(torch.int32)
        cur += nblk
    slots: List[int] = []
    for s, (p, n) in enumerate(zip(priors, news)):
        for t in range(p, p + n):
            slots.append(int(table[s, t // bs]) * bs + t % bs)
    cu = [0]
    for n in news:
        cu.append(cu[-1] + n)
    T = cu[-1]

    dev = torch.device(device)
    dg = torch.Generator(device=dev).manual_seed(seed + 1)
    hq, hkv, d = shape.num_q_heads, shape.num_kv_heads, shape.head_dim

    def randn(*size, std=1.0, dtype=torch.float32):
        # drawn in fp32 chunks so the fp32 staging copy stays small
        out = torch.empty(*size, dtype=dtype, device=dev)
        flat = out.view(-1)
        step = 1 << 26
        for i in range(0, flat.numel(), step):
            m = min(step, flat.numel() - i)
            flat[i:i + m] = (torch.randn(m, generator=dg, device=dev) * std).to(dtype)
        return out

    query = randn(T, hq, d, dtype=shape.q_dtype)
    new_key = randn(T, hkv, d, std=shape.kv_std, dtype=shape.q_dtype)
    new_value = randn(T, hkv, d, std=shape.kv_std, dtype=shape.q_dtype)
    k_scale = v_scale = None
    pool_shape = (pool_blocks, hkv, bs, d)
    if shape.kv_dtype == torch.float8_e4m3fn:
        # per-KV-head scale from the absmax of N(0,1) data; payload quantised
        # block by block to keep the fp32 staging small
        k_pool = torch.empty(pool_shape, dtype=shape.kv_dtype, device=dev)
        v_pool = torch.empty(pool_shape, dtype=shape.kv_dtype, device=dev)
        amax_k = torch.zeros(hkv, device=dev)
        amax_v = torch.zeros(hkv, device=dev)
        for i, m, kk, vv in _fp8_source_chunks(pool_shape, dev, seed):
            amax_k = torch.maximum(amax_k, kk.abs().amax(dim=(0, 2, 3)))
            amax_v = torch.maximum(amax_v, vv.abs().amax(dim=(0, 2, 3)))
        amax_k = torch.maximum(amax_k, new_key.float().abs().amax(dim=(0, 2)))
        amax_v = torch.maximum(amax_v, new_value.float().abs().amax(dim=(0, 2)))
        k_scale = (amax_k / FP8_MAX).float()
        v_scale = (amax_v / FP8_MAX).float()
        for i, m, kk, vv in _fp8_source_chunks(pool_shape, dev, seed):
            k_pool[i:i + m] = (kk / k_scale[None, :, None, None]).clamp(-FP8_MAX, FP8_MAX).to(shape.kv_dtype)
            v_pool[i:i + m] = (vv / v_scale[None, :, None, None]).clamp(-FP8_MAX, FP8_MAX).to(shape.kv_dtype)
    else:
        k_pool = randn(*pool_shape, std=shape.kv_std, dtype=shape.kv_dtype)
        v_pool = randn(*pool_shape, std=shape.kv_std, dtype=shape.kv_dtype)

    return Workload(
        shape=shape, scale=1.0 / math.sqrt(d), query=query, new_key=new_key, new_value=new_value,
        k_pool=k_pool, v_pool=v_pool, block_table=table.to(dev),
        context_lens=torch.tensor(ctx, dtype=torch.int32, device=dev),
        slot_mapping=torch.tensor(slots, dtype=torch.int64, device=dev),
        cu_q_lens=torch.tensor(cu, dtype=torch.int32, device=dev),
        num_prefill_seqs=shape.prefill_chunks, k_scale=k_scale, v_scale=v_scale,
        ctx_list=ctx, new_list=news)
