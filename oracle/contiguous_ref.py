"""CPU restatement of the reference operator on its own (contiguous) layout.

TEST INFRASTRUCTURE ONLY - the product package never imports this file.  It
is (1) the checker for the drop-in adapter's state machine and results and
(2) the ``cpu_baseline`` ("port") leg of the bench: the reference's CPU path,
restated in this repository's own torch code and timed on the host cores.

What is restated (reference lines in ``opt_prime/opt_prime/kv_cache.py``):

* storage ``[B, H, max_seq_len, D]`` zero-filled, one tensor each for K and V
  (``:96-108`` manager, ``:372-381`` lazy internal allocation);
* append = slice assignment at ``pos:pos+n`` (``:159-160``, ``:387-388``);
  the manager raises ``ValueError`` for an unknown layer (``:132-136``) and on
  overflow (``:152-156``), and moves its own ``_seq_len`` only for its first
  local layer (``:163-164``);
* attend = ``.contiguous()`` copy of the prefix (``:367-368``, ``:391-392``)
  followed by ``F.scaled_dot_product_attention`` with no mask when the write
  position on entry was > 0 (``:397-403``) and ``is_causal=True`` when it was 0
  (``:404-415``); the caller's ``attn_mask`` is dropped, other kwargs pass
  through;
* disabled -> plain SDPA pass-through (``:350-354``).
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch
import torch.nn.functional as F


class ContiguousStore:
    """The manager's storage and position rules (kv_cache.py:39-217)."""

    def __init__(self, num_layers, max_batch_size, max_seq_len, num_heads, head_dim,
                 dtype=torch.bfloat16, device="cpu", layer_start=0, layer_end=None):
        self.max_batch_size = max_batch_size
        self.max_seq_len = max_seq_len
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.dtype = dtype
        self.device = torch.device(device)
        self.layer_start = layer_start
        self.layer_end = num_layers if layer_end is None else layer_end
        self.seq_len = 0
        self.batch = 0
        self.k: Dict[int, torch.Tensor] = {}
        self.v: Dict[int, torch.Tensor] = {}

    def allocate(self, batch_size: int, seq_len: Optional[int] = None) -> None:
        seq_len = self.max_seq_len if seq_len is None else seq_len
        if batch_size > self.max_batch_size:
            raise ValueError("batch size over the maximum")
        if seq_len > self.max_seq_len:
            raise ValueError("seq_len over the maximum")
        self.batch = batch_size
        self.seq_len = 0
        shape = (batch_size, self.num_heads, self.max_seq_len, self.head_dim)
        for layer in range(self.layer_start, self.layer_end):
            self.k[layer] = torch.zeros(shape, dtype=self.dtype, device=self.device)
            self.v[layer] = torch.zeros(shape, dtype=self.dtype, device=self.device)

    def update(self, layer, new_k, new_v, position=None) -> Tuple[torch.Tensor, torch.Tensor]:
        if layer not in self.k:
            raise ValueError("layer not held by this store")
        pos = self.seq_len if position is None else position
        if new_k.dim() == 3:
            new_k, new_v = new_k[None], new_v[None]
        end = pos + new_k.size(2)
        if end > self.max_seq_len:
            raise ValueError("cache overflow")
        self.k[layer][:, :, pos:end, :] = new_k
        self.v[layer][:, :, pos:end, :] = new_v
        if layer == self.layer_start:
            self.seq_len = max(self.seq_len, end)
        return self.k[layer][:, :, :end, :], self.v[layer][:, :, :end, :]

    def clear(self) -> None:
        self.seq_len = 0
        for layer in self.k:
            self.k[layer].zero_()
            self.v[layer].zero_()


class ContiguousCachedAttention:
    """The operator's append-then-attend rule (kv_cache.py:340-415)."""

    def __init__(self, layer_idx: int, max_seq_len: int = 2048):
        self.layer_idx = layer_idx
        self.max_seq_len = max_seq_len
        self.pos = 0
        self.enabled = False
        self.k: Optional[torch.Tensor] = None
        self.v: Optional[torch.Tensor] = None
        self.store: Optional[ContiguousStore] = None

    def enable(self):
        self.enabled, self.pos = True, 0

    def disable(self):
        self.enabled, self.pos, self.k, self.v = False, 0, None, None

    def clear(self):
        self.pos = 0
        if self.store is None and self.k is not None:
            self.k.zero_()
            self.v.zero_()

    def __call__(self, query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, **kw):
        if not self.enabled:
            return F.scaled_dot_product_attention(
                query, key, value, attn_mask=attn_mask, dropout_p=dropout_p,
                is_causal=is_causal, **kw)
        n = key.size(2)
        entry_pos = self.pos
        if self.store is not None:
            fk, fv = self.store.update(self.layer_idx, key, value, position=entry_pos)
        else:
            if self.k is None:
                b, h, _, d = key.shape
                self.k = torch.zeros(b, h, self.max_seq_len, d, dtype=key.dtype, device=key.device)
                self.v = torch.zeros(b, h, self.max_seq_len, d, dtype=value.dtype, device=value.device)
            self.k[:, :, entry_pos:entry_pos + n, :] = key
            self.v[:, :, entry_pos:entry_pos + n, :] = value
            fk = self.k[:, :, :entry_pos + n, :]
            fv = self.v[:, :, :entry_pos + n, :]
        self.pos = entry_pos + n
        fk, fv = fk.contiguous(), fv.contiguous()
        return F.scaled_dot_product_attention(
            query, fk, fv, attn_mask=None, dropout_p=dropout_p,
            is_causal=(entry_pos == 0), **kw)


def reference_cpu_decode(query, k_pool, v_pool, block_table, context_lens, scale,
                         k_scale=None, v_scale=None, compute_dtype=None):
    """The reference's decode step on paged inputs, the way its CPU path runs it.

    Per sequence: gather its blocks to a contiguous ``[1, Hkv, L, D]``, expand
    to the query heads (``repeat_kv``, modeling_llama.py:268-277), make it
    contiguous (kv_cache.py:391-392) and call SDPA without a mask
    (kv_cache.py:400-403).  Sequences have different lengths, so the batch
    dimension is walked (the reference's shared ``cache_pos`` cannot express a
    ragged batch).  query [B, Hq, D]; pools [num_blocks, Hkv, BS, D]; returns
    [B, Hq, D] in the compute dtype.
    """
    B, hq, d = query.shape
    nb, hkv, bs, _ = k_pool.shape
    g = hq // hkv
    cd = compute_dtype or query.dtype
    out = torch.empty(B, hq, d, dtype=cd)
    for b in range(B):
        L = int(context_lens[b])
        nblk = (L + bs - 1) // bs
        blocks = block_table[b, :nblk].long()
        k = k_pool[blocks].permute(1, 0, 2, 3).reshape(hkv, nblk * bs, d)[:, :L]
        v = v_pool[blocks].permute(1, 0, 2, 3).reshape(hkv, nblk * bs, d)[:, :L]
        k, v = k.to(cd), v.to(cd)
        if k_scale is not None:
            k = (k.float() * k_scale.float()[:, None, None]).to(cd)
            v = (v.float() * v_scale.float()[:, None, None]).to(cd)
        k = k[:, None].expand(hkv, g, L, d).reshape(1, hq, L, d).contiguous()
        v = v[:, None].expand(hkv, g, L, d).reshape(1, hq, L, d).contiguous()
        q = query[b].to(cd).reshape(1, hq, 1, d)
        out[b] = F.scaled_dot_product_attention(q, k, v, attn_mask=None, is_causal=False,
                                                scale=scale)[0, :, 0]
    return out


def reference_cpu_prefill(query, k_pool, v_pool, block_table, context_len, scale, compute_dtype=None):
    """The reference's prefill call for ONE chunk on paged inputs, the way its CPU path runs it:
    gather the sequence's blocks to a contiguous ``[1, Hkv, L, D]``, ``repeat_kv`` to the query
    heads (modeling_llama.py:268-277), ``.contiguous()`` (kv_cache.py:391-392) and SDPA
    (kv_cache.py:404-415).  A chunk that starts the sequence is ``is_causal=True`` as in the
    reference; a chunk over a prior context gets the causal-within-the-chunk mask this build
    defines for that case (the reference never issues such a call).  query ``[n, Hq, D]`` (the
    chunk's tokens, in order), context_len = prior + n; returns ``[n, Hq, D]``."""
    n, hq, d = query.shape
    nb, hkv, bs, _ = k_pool.shape
    g = hq // hkv
    cd = compute_dtype or query.dtype
    L = int(context_len)
    prior = L - n
    nblk = (L + bs - 1) // bs
    blocks = block_table[:nblk].long()
    k = k_pool[blocks].permute(1, 0, 2, 3).reshape(hkv, nblk * bs, d)[:, :L].to(cd)
    v = v_pool[blocks].permute(1, 0, 2, 3).reshape(hkv, nblk * bs, d)[:, :L].to(cd)
    k = k[:, None].expand(hkv, g, L, d).reshape(1, hq, L, d).contiguous()
    v = v[:, None].expand(hkv, g, L, d).reshape(1, hq, L, d).contiguous()
    q = query.to(cd).permute(1, 0, 2).reshape(1, hq, n, d)
    if prior == 0:
        out = F.scaled_dot_product_attention(q, k, v, attn_mask=None, is_causal=True, scale=scale)
    else:
        mask = torch.arange(L)[None, :] <= (prior + torch.arange(n))[:, None]
        out = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, is_causal=False, scale=scale)
    return out[0].permute(1, 0, 2)
