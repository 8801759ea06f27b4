"""Drop-in KV-cache operator for opt_prime's inference runtime, backed by the paged HIP path.

Mirrors ``opt_prime/opt_prime/kv_cache.py``:

* ``CachedScaledDotProductAttention``  (reference ``kv_cache.py:257-424``) - same
  constructor ``(layer_idx, max_seq_len=2048, dtype=torch.bfloat16)``, same
  ``forward(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False,
  **kwargs)``, same ``enable / disable / clear / set_kv_manager /
  clear_kv_manager`` and the attributes the engine reads (``_enabled``,
  ``layer_idx``, ``cache_pos``; ``inference.py:946-955, 1100-1111, 1146-1148``).
* ``KVCacheManager``  (reference ``kv_cache.py:19-254``) - same constructor and
  ``allocate / update / get / get_seq_len / set_seq_len / clear / free /
  is_allocated / batch_size / get_memory_usage``, same ``ValueError``s.

Swapping the class the engine instantiates at ``inference.py:888`` (or
assigning ``opt_prime.kv_cache.CachedScaledDotProductAttention`` before the
engine is built) is the whole integration.

What differs underneath: the reference keeps ``[B, H, max_seq_len, D]`` tensors
with H already expanded to the query heads by ``repeat_kv``, copies the whole
prefix with ``.contiguous()`` every call and hands it to torch SDPA
(``kv_cache.py:387-403``).  Here K/V live once per KV head in a block pool
``[num_blocks, Hkv, 16, D]``; the new rows are scattered in by slot
(``ops.kv_append``) and attention reads the pool in place through a block table
(``ops.paged_decode_attn`` / ``ops.paged_prefill_attn``).  All sequences of a
batch share one write position, as in the reference (``kv_cache.py:69,290``), so
``context_lens`` is uniform and the tables are static.

One deliberate extension: for a call with ``cache_pos > 0`` and more than one new
token (a second prompt chunk) the reference applies no mask at all
(``kv_cache.py:363,397-403``; it never issues such a call).  This operator
masks causally inside the chunk (query i sees keys ``<= cache_pos + i``), which
equals the reference for ``cache_pos == 0`` and for single-token decode.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F
import torch.nn.modules.module as _nn_module

from . import _lib, ops

BLOCK_SIZE = 16

# Host routes of a decode step into the HIP library, leanest first.  All three end in the same C
# entry point (aicomp_paged_decode_attn_append); they differ in host time per call, which at
# batch 1 is step time: "fast", a CPython function over a per-layer handle (csrc/fast_call.cpp);
# "torch_op", the registered operator torch.ops.mi355_kv.decode_step (csrc/torch_ops.cpp);
# "ctypes", which remains for device-side positions and for installations where the two host
# libraries were not built.
try:
    from . import _aicomp_fast as _FAST
except ImportError:
    _FAST = None
try:
    _TORCH_DECODE = _lib.torch_ops().decode_step.default
except _lib.LibraryMissing:
    _TORCH_DECODE = None
_PLAIN_KWARGS = frozenset(("attn_mask", "dropout_p", "is_causal"))      # keywords that leave a decode call as it is
_route = "fast" if _FAST is not None else ("torch_op" if _TORCH_DECODE is not None else "ctypes")


def _detect_group(key: torch.Tensor) -> int:
    """Largest G such that the heads of ``key [B, H, n, D]`` come in runs of G
    identical copies - what HF ``repeat_kv`` produces
    (``compiler_fx/modeling_llama.py:268-277``).  One device synchronisation."""
    B, H, n, D = key.shape
    for g in sorted((d for d in range(2, H + 1) if H % d == 0), reverse=True):
        v = key.reshape(B, H // g, g, n, D)
        if bool((v == v[:, :, :1]).all()):
            return g
    return 1


_CTX_ROWS: Dict[tuple, torch.Tensor] = {}


def _ctx_rows(rows: int, batch: int, device: torch.device) -> torch.Tensor:
    """``[rows, batch]`` int32 with row L filled with L; one tensor per geometry, shared by the layers."""
    key = (device.type, device.index, rows, batch)
    t = _CTX_ROWS.get(key)
    if t is None:
        t = torch.arange(rows, dtype=torch.int32, device=device)[:, None].expand(-1, batch).contiguous()
        _CTX_ROWS[key] = t
    return t


class _PagedLayer:
    """K and V block pools of one layer plus the static tables of a fixed batch."""

    def __init__(self, batch: int, kv_heads: int, head_dim: int, max_seq_len: int,
                 dtype: torch.dtype, device: torch.device, block_size: int = BLOCK_SIZE):
        self.batch, self.kv_heads, self.head_dim = batch, kv_heads, head_dim
        self.default_scale = 1.0 / math.sqrt(head_dim)
        self.dtype = dtype
        self.max_seq_len, self.block_size = max_seq_len, block_size
        self.blocks_per_seq = max(1, math.ceil(max_seq_len / block_size))
        nb = batch * self.blocks_per_seq
        shape = (nb, kv_heads, block_size, head_dim)
        self.k_pool = torch.zeros(shape, dtype=dtype, device=device)
        self.v_pool = torch.zeros(shape, dtype=dtype, device=device)
        # sequence b owns blocks b*blocks_per_seq .. ; slot of (b, t) is closed-form
        self.block_table = torch.arange(nb, dtype=torch.int32, device=device).view(batch, self.blocks_per_seq)
        t = torch.arange(self.blocks_per_seq * block_size, dtype=torch.int64, device=device)
        base = torch.arange(batch, dtype=torch.int64, device=device) * (self.blocks_per_seq * block_size)
        self.slot_table = base[:, None] + t[None, :]                       # [B, padded max_seq]
        self.context_lens = torch.zeros(batch, dtype=torch.int32, device=device)
        # row L of this table is the context-length vector of a step that sees L tokens: all
        # sequences share one position, so a decode step takes a view instead of launching a fill
        self.ctx_rows = _ctx_rows(self.blocks_per_seq * block_size + 1, batch, torch.device(device))
        # the same vector kept on the device and advanced by a kernel, for decode steps that are
        # replayed from a HIP graph (a replay runs no host code, so it cannot pick another row)
        self.live_ctx = torch.zeros(batch, dtype=torch.int32, device=device)
        self._ctx_base, self._ctx_pitch = self.ctx_rows.data_ptr(), self.ctx_rows.stride(0) * 4
        # the static tensors, checked once, behind a handle for the lean decode call (pools of the
        # operator's own element types; the handle keeps the tensors alive)
        self._fast = None
        if _FAST is not None and self.k_pool.is_cuda and dtype in (torch.float32, torch.bfloat16, torch.float16):
            self._fast = _FAST.layer(self.k_pool, self.v_pool, self.block_table, self.ctx_rows)
        self._decode: Dict[tuple, ops.PreparedDecode] = {}
        self.cu_q_lens = torch.zeros(batch + 1, dtype=torch.int32, device=device)
        self._cu_n = -1

    def nbytes(self) -> int:
        return 2 * self.k_pool.numel() * self.k_pool.element_size()

    def append(self, key: torch.Tensor, value: torch.Tensor, pos: int, group: int) -> None:
        """key/value ``[B, H, n, D]`` (H = Hkv, or Hkv*group expanded) written at pos..pos+n."""
        B, H, n, D = key.shape
        if H == self.kv_heads * group and group > 1:
            key, value = key[:, ::group], value[:, ::group]
        if n == 1:
            rows_k, rows_v = key[:, :, 0, :], value[:, :, 0, :]            # strided views, no copy
        else:
            rows_k = key.permute(0, 2, 1, 3).reshape(B * n, self.kv_heads, D)
            rows_v = value.permute(0, 2, 1, 3).reshape(B * n, self.kv_heads, D)
        slots = self.slot_table[:, pos:pos + n].reshape(-1).contiguous()
        ops.kv_append(rows_k, rows_v, self.k_pool, self.v_pool, slots)

    def decode_step(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, pos: int,
                    group: int, scale: float, live: bool = False) -> torch.Tensor:
        """One decode step, append and attention in a single call: query ``[B, Hq, 1, D]``,
        key/value ``[B, H, 1, D]`` written at position pos.  With ``live`` the position is the
        device-side counter ``live_ctx`` (advanced here by a one-element-per-sequence kernel), so
        the step can be captured into a HIP graph and replayed."""
        if not live and _route != "ctypes":
            # checks, output allocation, current stream and the fused append + decode call all in C++
            if _route == "fast" and self._fast is not None:
                return _FAST.decode_step(self._fast, query, key, value, pos, group, scale)
            if _TORCH_DECODE is not None:
                return _TORCH_DECODE(query, key, value, self.k_pool, self.v_pool, self.block_table, self.ctx_rows,
                                     pos, group, scale, None)
        Hq = query.shape[1]
        call = self._decode.get((Hq, query.dtype, scale))
        if call is None:
            call = ops.PreparedDecode(self.k_pool, self.v_pool, self.block_table, self.context_lens, Hq,
                                      query.dtype, scale)
            self._decode[(Hq, query.dtype, scale)] = call
        if not query.is_contiguous():
            query = query.contiguous()
        if live:
            # the counter moves only once the call's arguments have passed their checks (a rejected
            # call must leave it where it was); add_ is a fill-type kernel, safe inside a captured graph
            ctx, ready, width = self.live_ctx.data_ptr(), self._bump_live, None
        else:
            # row pos + 1 of the context-length table, by address (a view tensor costs microseconds);
            # only the table columns that hold those pos + 1 tokens are in use
            ctx, ready, width = self._ctx_base + (pos + 1) * self._ctx_pitch, None, pos // self.block_size + 1
        # [B, Hq, 1, D] has the memory layout of [B, Hq, D]: the call takes the tensors as they are
        return call.step4d(torch.empty_like(query), query, key, value, group, ctx, ready, width)

    def _bump_live(self) -> None:
        self.live_ctx.add_(1)

    def attend(self, query: torch.Tensor, pos: int, scale: float) -> torch.Tensor:
        """query ``[B, Hq, n, D]`` at positions pos..pos+n (rows already appended)."""
        B, Hq, n, D = query.shape
        ctx = self.ctx_rows[pos + n]              # every sequence sees pos + n tokens: a row view, no fill launch
        if n == 1:
            q = query[:, :, 0, :].contiguous()
            out = torch.empty_like(q)
            ops.paged_decode_attn(out, q, self.k_pool, self.v_pool, self.block_table, ctx, scale)
            return out.view(B, Hq, 1, D)
        if self._cu_n != n:
            self.cu_q_lens.copy_(torch.arange(B + 1, dtype=torch.int32, device=query.device) * n)
            self._cu_n = n
        # token-major rows; for batch 1 the reshape is a strided view, hence the explicit copy
        q = query.permute(0, 2, 1, 3).reshape(B * n, Hq, D).contiguous()
        out = torch.empty_like(q)
        ops.paged_prefill_attn(out, q, self.k_pool, self.v_pool, self.block_table,
                               ctx, self.cu_q_lens, scale, max_q_len=n)
        return out.view(B, n, Hq, D).permute(0, 2, 1, 3)

    def gather(self, end: int, heads: int, which: str = "kv") -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        """Dense ``[B, heads, end, D]`` copies (heads = Hkv or the expanded count) of K, V or both."""
        B, bps, bs = self.batch, self.blocks_per_seq, self.block_size

        def dense(pool):
            x = pool.view(B, bps, self.kv_heads, bs, self.head_dim).permute(0, 2, 1, 3, 4)
            x = x.reshape(B, self.kv_heads, bps * bs, self.head_dim)[:, :, :end]
            if heads != self.kv_heads:
                x = x.repeat_interleave(heads // self.kv_heads, dim=1)
            return x.contiguous()

        return (dense(self.k_pool) if "k" in which else None, dense(self.v_pool) if "v" in which else None)


class PagedKVView:
    """What ``KVCacheManager.update/get`` hand back in place of the reference's
    ``cache[:, :, :end, :]`` views (``kv_cache.py:166-170, 172-195``): the prefix
    ``[B, heads, end, D]`` of one layer's K or V.  It stays paged until a caller touches the
    data; then it gathers a dense tensor of the pool's current contents (like the reference's
    view, it shows rows written after it was made) and behaves as that tensor: ``shape``,
    ``dtype``, ``device``, ``dim()`` and ``size()`` cost nothing; indexing, ``torch.*``
    functions and every other tensor method (``.float()``, ``.transpose(...)``, ...) run on
    the gathered copy.  It is read-only: the pools are written by ``update`` alone."""

    def __init__(self, layer: _PagedLayer, which: str, end: int, heads: int):
        self._layer, self._which, self.end, self.heads = layer, which, end, heads

    @property
    def shape(self):
        return torch.Size((self._layer.batch, self.heads, self.end, self._layer.head_dim))

    def size(self, dim: Optional[int] = None):
        return self.shape if dim is None else self.shape[dim]

    def dim(self) -> int:
        return 4

    ndim = property(dim)

    def numel(self) -> int:
        return self.shape.numel()

    @property
    def dtype(self) -> torch.dtype:
        return self._layer.k_pool.dtype

    @property
    def device(self) -> torch.device:
        return self._layer.k_pool.device

    @property
    def is_cuda(self) -> bool:
        return self._layer.k_pool.is_cuda

    def to_dense(self) -> torch.Tensor:
        k, v = self._layer.gather(self.end, self.heads, self._which)
        return k if self._which == "k" else v

    contiguous = to_dense

    def __len__(self) -> int:
        return self._layer.batch

    def __getitem__(self, index):
        return self.to_dense()[index]

    def __setitem__(self, index, value):
        raise TypeError("a PagedKVView is read-only: rows enter the pools through KVCacheManager.update")

    def __getattr__(self, name):
        # anything else a tensor offers, on the gathered copy (only reached for names not defined above)
        if name.startswith("_"):
            raise AttributeError(name)
        return getattr(self.to_dense(), name)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        dense = lambda x: x.to_dense() if isinstance(x, PagedKVView) else x
        args = tuple(type(a)(dense(x) for x in a) if isinstance(a, (list, tuple)) else dense(a) for a in args)
        kwargs = {k: dense(v) for k, v in (kwargs or {}).items()}
        return func(*args, **kwargs)

    def __repr__(self) -> str:
        return f"PagedKVView({self._which}, shape={tuple(self.shape)}, dtype={self.dtype}, device={self.device})"


class KVCacheManager:
    """Paged stand-in for the reference's ``KVCacheManager`` (``kv_cache.py:19-254``).

    ``num_heads`` is what the reference passes: the number of heads K/V arrive
    with at the operator, i.e. query heads after ``repeat_kv``
    (``examples/single_gpu_inference_llama.py:172-176``).  ``num_kv_heads`` (extra,
    optional) tells the store how many of them are distinct; K/V are kept once per
    KV head.  Without it every arriving head is stored.
    """

    def __init__(self, num_layers: int, max_batch_size: int, max_seq_len: int, num_heads: int,
                 head_dim: int, dtype: torch.dtype = torch.bfloat16, device: torch.device = None,
                 layer_start: int = 0, layer_end: int = None, num_kv_heads: Optional[int] = None):
        self.num_layers = num_layers
        self.max_batch_size = max_batch_size
        self.max_seq_len = max_seq_len
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads or num_heads
        if num_heads % self.num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {self.num_kv_heads} KV heads")
        self.group = num_heads // self.num_kv_heads
        self.head_dim = head_dim
        self.dtype = dtype
        self.device = device or torch.device("cuda")
        self.layer_start = layer_start
        self.layer_end = layer_end if layer_end is not None else num_layers
        self.num_local_layers = self.layer_end - self.layer_start
        self._cache: Dict[int, _PagedLayer] = {}
        self._seq_len = 0
        self._batch_size = 0
        self._allocated = False

    def allocate(self, batch_size: int, seq_len: Optional[int] = None) -> None:
        if seq_len is None:
            seq_len = self.max_seq_len
        if batch_size > self.max_batch_size:
            raise ValueError(f"Requested batch size {batch_size} exceeds max {self.max_batch_size}")
        if seq_len > self.max_seq_len:
            raise ValueError(f"Requested seq_len {seq_len} exceeds max {self.max_seq_len}")
        self._batch_size = batch_size
        self._seq_len = 0
        for layer_idx in range(self.layer_start, self.layer_end):
            self._cache[layer_idx] = _PagedLayer(batch_size, self.num_kv_heads, self.head_dim,
                                                 self.max_seq_len, self.dtype, self.device)
        self._allocated = True

    def _layer(self, layer_idx: int) -> _PagedLayer:
        if layer_idx not in self._cache:
            raise ValueError(f"Layer {layer_idx} not in this stage's cache "
                             f"(range: {self.layer_start}-{self.layer_end})")
        return self._cache[layer_idx]

    def _place(self, layer_idx: int, new_k: torch.Tensor, new_v: torch.Tensor, position: Optional[int]):
        """The checks and shape rules of ``update`` (``kv_cache.py:132-156``): unknown layer and
        overflow raise ``ValueError``, 3-D input is batch 1, batch 1 broadcasts over the batch."""
        layer = self._layer(layer_idx)
        if position is None:
            position = self._seq_len
        if new_k.dim() == 3:
            new_k, new_v = new_k.unsqueeze(0), new_v.unsqueeze(0)
        if new_k.size(0) == 1 and layer.batch > 1:          # slice assignment broadcasts batch 1
            new_k = new_k.expand(layer.batch, -1, -1, -1)
            new_v = new_v.expand(layer.batch, -1, -1, -1)
        end_position = position + new_k.size(2)
        if end_position > self.max_seq_len:
            raise ValueError(f"Cache overflow: position {position} + new_seq_len {new_k.size(2)} "
                             f"> max_seq_len {self.max_seq_len}")
        return layer, new_k, new_v, position, end_position

    def _advance(self, layer_idx: int, end_position: int) -> None:
        # only the stage's first layer moves the shared length (kv_cache.py:163-164)
        if layer_idx == self.layer_start:
            self._seq_len = max(self._seq_len, end_position)

    def append(self, layer_idx: int, new_k: torch.Tensor, new_v: torch.Tensor,
               position: Optional[int] = None) -> Tuple[_PagedLayer, int, int]:
        """The storage half of ``update``: returns (layer store, start, end)."""
        layer, new_k, new_v, position, end_position = self._place(layer_idx, new_k, new_v, position)
        layer.append(new_k, new_v, position, self.group)
        self._advance(layer_idx, end_position)
        return layer, position, end_position

    def decode_step(self, layer_idx: int, query: torch.Tensor, new_k: torch.Tensor, new_v: torch.Tensor,
                    position: Optional[int], scale: float) -> Optional[torch.Tensor]:
        """``update`` of one new token per sequence and the attention over the result in ONE library
        call (the fused append + decode entry point), with ``update``'s checks and length rule.
        Returns ``None`` when the step is not of that form (more than one token, or rows that need a
        type conversion): the caller then appends and attends separately."""
        if new_k.size(-2) != 1:
            return None
        layer, new_k, new_v, position, end_position = self._place(layer_idx, new_k, new_v, position)
        if new_k.dtype != layer.k_pool.dtype or query.size(0) != layer.batch:
            return None
        out = layer.decode_step(query, new_k, new_v, position, self.group, scale)
        self._advance(layer_idx, end_position)
        return out

    def update(self, layer_idx: int, new_k: torch.Tensor, new_v: torch.Tensor,
               position: Optional[int] = None) -> Tuple[PagedKVView, PagedKVView]:
        layer, _, end = self.append(layer_idx, new_k, new_v, position)
        return PagedKVView(layer, "k", end, self.num_heads), PagedKVView(layer, "v", end, self.num_heads)

    def get(self, layer_idx: int) -> Optional[Tuple[PagedKVView, PagedKVView]]:
        if layer_idx not in self._cache or self._seq_len == 0:
            return None
        layer = self._cache[layer_idx]
        return (PagedKVView(layer, "k", self._seq_len, self.num_heads),
                PagedKVView(layer, "v", self._seq_len, self.num_heads))

    def get_seq_len(self) -> int:
        return self._seq_len

    def set_seq_len(self, seq_len: int) -> None:
        self._seq_len = seq_len

    def clear(self) -> None:
        """New generation.  The reference also zero-fills its tensors
        (``kv_cache.py:204-210``); nothing beyond the write position is ever read
        here, so the pools are left as they are."""
        self._seq_len = 0

    def free(self) -> None:
        self._cache.clear()
        self._allocated = False
        self._seq_len = 0
        self._batch_size = 0

    @property
    def is_allocated(self) -> bool:
        return self._allocated

    @property
    def batch_size(self) -> int:
        return self._batch_size

    def get_memory_usage(self) -> int:
        """Bytes held by the pools (the reference's figure is G times larger: it
        stores every query head and the full ``max_seq_len``, ``kv_cache.py:229-245``)."""
        if not self._allocated:
            return 0
        return sum(layer.nbytes() for layer in self._cache.values())

    def __repr__(self) -> str:
        return (f"KVCacheManager(layers={self.layer_start}-{self.layer_end}, "
                f"batch_size={self._batch_size}, seq_len={self._seq_len}/{self.max_seq_len}, "
                f"allocated={self._allocated}, paged, kv_heads={self.num_kv_heads})")


class CachedScaledDotProductAttention(nn.Module):
    """``scaled_dot_product_attention`` with a KV cache, on the paged HIP kernels.

    Args:
        layer_idx, max_seq_len, dtype: as in the reference (``kv_cache.py:276-285``).
        num_kv_groups: query heads per KV head of the K/V the caller passes in
            (HF Llama passes them already expanded).  ``None`` detects it on the first
            cached call by comparing adjacent heads (one synchronisation); ``1`` stores
            every head.
    """

    def __init__(self, layer_idx: int, max_seq_len: int = 2048, dtype: torch.dtype = torch.bfloat16,
                 num_kv_groups: Optional[int] = None):
        super().__init__()
        self.layer_idx = layer_idx
        self.max_seq_len = max_seq_len
        self.dtype = dtype
        self.num_kv_groups = num_kv_groups
        self._store: Optional[_PagedLayer] = None
        self.cache_pos: int = 0
        self._enabled: bool = False
        self._device_positions: bool = False
        self.kv_manager: Optional[KVCacheManager] = None

    # the reference exposes its tensors under these names; here they are the block pools
    @property
    def cache_k(self) -> Optional[torch.Tensor]:
        return None if self._store is None else self._store.k_pool

    @property
    def cache_v(self) -> Optional[torch.Tensor]:
        return None if self._store is None else self._store.v_pool

    def enable(self) -> None:
        self._enabled = True
        self.cache_pos = 0

    def set_kv_manager(self, kv_manager: KVCacheManager) -> None:
        if not isinstance(kv_manager, KVCacheManager):
            raise TypeError("kv_manager must be an aicomp_amd.kv_cache.KVCacheManager "
                            "(the paged store); a contiguous manager cannot back this operator")
        self.kv_manager = kv_manager

    def clear_kv_manager(self) -> None:
        self.kv_manager = None

    def disable(self) -> None:
        self._enabled = False
        self._device_positions = False
        self.cache_pos = 0
        self._store = None

    def use_device_positions(self, on: bool = True) -> None:
        """Keep the decode position on the device (no counterpart in the reference, whose cache
        position is a Python integer, ``kv_cache.py:372-388``): for callers that capture a decode
        step into a HIP graph.  A replay runs no Python, so it can neither advance ``cache_pos``
        nor choose another context-length vector; with this switch a decode step first advances a
        per-layer device counter and attends with it.  Call it after the prompt has been ingested
        (it starts the counter at the current ``cache_pos``), capture and replay decode steps,
        then ``advance(n)`` by the number of replays before the next eager call.  Internal mode
        only.  A replay past ``max_seq_len`` stores nothing (the kernel's bounds rule) and
        attends to the full cache."""
        if on:
            if self.kv_manager is not None:
                raise RuntimeError("device positions need the operator's own cache (no kv_manager)")
            if self._store is None:
                raise RuntimeError("device positions start from an ingested prompt: run the prefill first")
            self._store.live_ctx.fill_(self.cache_pos)
        elif self._device_positions:
            self._resync_position()
        self._device_positions = on

    def _resync_position(self) -> None:
        """Leaving device positions: the device counter is the truth (replays advanced it without
        running Python), so the host position is read back from it - one device-to-host copy,
        outside any capture.  A caller that forgot ``advance(n)`` therefore cannot end up writing
        over live tokens."""
        if self._store is not None and not torch.cuda.is_current_stream_capturing():
            self.cache_pos = min(int(self._store.live_ctx[0].item()), self.max_seq_len)

    def advance(self, steps: int) -> None:
        """Account on the host for decode steps that were replayed from a graph."""
        if steps < 0 or self.cache_pos + steps > self.max_seq_len:
            raise RuntimeError(f"advance({steps}) from position {self.cache_pos} leaves the cache "
                               f"(max_seq_len {self.max_seq_len})")
        self.cache_pos += steps

    def clear(self) -> None:
        """Reset the write position; the allocation is kept (``kv_cache.py:324-338``)."""
        self.cache_pos = 0
        self._device_positions = False          # the next use_device_positions() starts the counter afresh

    def __call__(self, *args, **kwargs):
        # One call per layer and token at batch 1 is bound by the host: nn.Module's hook dispatch
        # costs a microsecond per call and is only taken when some hook is actually registered.
        if (self._forward_hooks or self._forward_pre_hooks or self._backward_hooks or self._backward_pre_hooks
                or _nn_module._global_forward_hooks or _nn_module._global_forward_pre_hooks
                or _nn_module._global_backward_hooks or _nn_module._global_backward_pre_hooks):
            return super().__call__(*args, **kwargs)
        if len(args) == 3 and (not kwargs or (kwargs.keys() <= _PLAIN_KWARGS and not kwargs.get("dropout_p"))):
            # the model's own call on a decode step, attn(query, key, value, attn_mask=..., dropout_p=0.0,
            # is_causal=...) as compiler_fx/modeling_llama.py:607-614 issues it (the mask and the causal
            # flag of a one-token call change nothing, kv_cache.py:397-403): same route as in forward()
            # below, one Python frame less
            store = self._store
            if (store is not None and store._fast is not None and _route == "fast" and self._enabled
                    and self.kv_manager is None and not self._device_positions):
                query, key, value = args
                pos = self.cache_pos
                if query.dim() == 4 and query.shape[2] == 1 and key.dtype == store.dtype and pos < self.max_seq_len:
                    out = _FAST.decode_step(store._fast, query, key, value, pos, self._group, store.default_scale)
                    self.__dict__["cache_pos"] = pos + 1      # (nn.Module.__setattr__ costs 0.5 us; a plain int needs none of it)
                    return out
        return self.forward(*args, **kwargs)

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                attn_mask: Optional[torch.Tensor] = None, dropout_p: float = 0.0,
                is_causal: bool = False, **kwargs) -> torch.Tensor:
        # decode step on the operator's own cache, the call a generation loop makes once per layer
        # and token: straight to the lean C++ entry (checks, output, stream and launch in one call)
        store = self._store
        if (store is not None and store._fast is not None and _route == "fast" and self._enabled
                and self.kv_manager is None and not self._device_positions and dropout_p == 0.0
                and query.dim() == 4 and query.shape[2] == 1 and key.dtype == store.dtype):
            pos = self.cache_pos
            if pos < self.max_seq_len:
                out = _FAST.decode_step(store._fast, query, key, value, pos, self._group,
                                        store.default_scale if not kwargs or kwargs.get("scale") is None
                                        else float(kwargs["scale"]))
                self.__dict__["cache_pos"] = pos + 1
                return out
        if not self._enabled:
            return F.scaled_dot_product_attention(query, key, value, attn_mask=attn_mask,
                                                  dropout_p=dropout_p, is_causal=is_causal, **kwargs)
        if dropout_p != 0.0:
            raise ValueError("cached attention is an inference path: dropout_p must be 0")
        B, Hq, n, D = query.shape
        scale = kwargs.get("scale")
        scale = 1.0 / math.sqrt(D) if scale is None else float(scale)
        pos = self.cache_pos

        if self.kv_manager is not None:
            # external mode (kv_cache.py:356-368): storage belongs to the manager; the explicit
            # position keeps several layers of one forward pass on the same write position
            if n == 1:                            # decode step: one fused call, as in internal mode
                out = self.kv_manager.decode_step(self.layer_idx, query, key, value, pos, scale)
                if out is not None:
                    self.__dict__["cache_pos"] = pos + 1
                    return out
            store, _, _ = self.kv_manager.append(self.layer_idx, key, value, position=pos)
        else:
            if self._store is None:
                Hk = key.shape[1]
                if Hk != Hq:
                    group = 1                    # unexpanded K/V (enable_gqa callers): stored as is
                else:
                    group = self.num_kv_groups or _detect_group(key)
                if Hk % group:
                    raise RuntimeError(f"{Hk} K/V heads are not a multiple of num_kv_groups={group}")
                self._group = group
                self._store = _PagedLayer(B, Hk // group, D, self.max_seq_len, key.dtype, key.device)
            store = self._store
            if self._device_positions and n != 1:
                # a prompt chunk while decode positions live on the device: take the position from
                # the device counter first, then go on with host positions
                self._resync_position()
                self._device_positions = False
                pos = self.cache_pos
            if pos + n > self.max_seq_len:
                raise RuntimeError(f"cache overflow: position {pos} + {n} new tokens > max_seq_len "
                                   f"{self.max_seq_len}")
            if n == 1 and key.dtype == store.k_pool.dtype:
                # decode step: append fused into the attention call.  A call that is only being
                # recorded into a graph executes nothing: the host position stays (see advance()).
                out = store.decode_step(query, key, value, pos, self._group, scale, live=self._device_positions)
                if not (self._device_positions and torch.cuda.is_current_stream_capturing()):
                    self.__dict__["cache_pos"] = pos + 1      # only after the call was accepted
                return out
            store.append(key, value, pos, self._group)
        self.cache_pos = pos + n
        # the caller's attn_mask is dropped, as in the reference (kv_cache.py:400-415): decode sees
        # the whole prefix, a chunk is causal
        return store.attend(query, pos, scale)

    def __repr__(self) -> str:
        mode = "external" if self.kv_manager is not None else "internal"
        return (f"CachedScaledDotProductAttention(layer={self.layer_idx}, "
                f"cache_pos={self.cache_pos}/{self.max_seq_len}, enabled={self._enabled}, "
                f"mode={mode}, paged)")
