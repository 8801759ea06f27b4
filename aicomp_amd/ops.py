"""Tensor-level wrappers of the C ABI: the three native ops of the path.

``kv_append``, ``paged_decode_attn`` and ``paged_prefill_attn`` take torch
tensors on a ROCm device, check them the way a ``TORCH_CHECK`` would
(``RuntimeError`` on dtype / shape / contiguity / device mismatch), and pass
raw device pointers plus the current HIP stream to libaicomp_kv.so.  torch is
used for device memory and streams only.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from . import _lib

_DT = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16,
       torch.float8_e4m3fn: _lib.FP8_E4M3}


def _dt(t: torch.Tensor, what: str) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise RuntimeError(f"{what}: unsupported dtype {t.dtype} (float32, bfloat16, float16, float8_e4m3fn)")


def _req(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _dev(t: torch.Tensor, ref: torch.Tensor, what: str) -> None:
    _req(t.device == ref.device, f"{what} is on {t.device}, expected {ref.device}")


# torch's raw-stream getter (what its own compiled-kernel launchers call) costs a fraction of a
# microsecond; building a torch.cuda.Stream object per call costs about four
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _current_stream(device: torch.device) -> int:
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


def _stream(t: torch.Tensor) -> int:
    _req(t.is_cuda, "tensors must live on a ROCm device (there is no CPU path)")
    return _current_stream(t.device)


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check_pools(k_pool: torch.Tensor, v_pool: torch.Tensor) -> Tuple[int, int, int, int]:
    _req(k_pool.dim() == 4 and v_pool.shape == k_pool.shape,
         f"pools must both be [num_blocks, Hkv, BS, D]; got {tuple(k_pool.shape)} and {tuple(v_pool.shape)}")
    _req(k_pool.dtype == v_pool.dtype, "k_pool and v_pool dtypes differ")
    _req(k_pool.is_contiguous() and v_pool.is_contiguous(), "pools must be contiguous")
    _dev(v_pool, k_pool, "v_pool")
    return tuple(k_pool.shape)  # type: ignore[return-value]


def _check_scales(k_scale, v_scale, pool: torch.Tensor, hkv: int):
    if pool.dtype == torch.float8_e4m3fn:
        _req(k_scale is not None and v_scale is not None, "an fp8 pool needs k_scale and v_scale")
        for s, n in ((k_scale, "k_scale"), (v_scale, "v_scale")):
            _req(s.dtype == torch.float32 and s.is_contiguous() and s.numel() == hkv,
                 f"{n} must be a contiguous float32 tensor of {hkv} elements")
            _dev(s, pool, n)
        return k_scale, v_scale
    return None, None


def kv_append(key: torch.Tensor, value: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
              slot_mapping: torch.Tensor, k_scale: Optional[torch.Tensor] = None,
              v_scale: Optional[torch.Tensor] = None) -> None:
    """Scatter ``key/value [T, Hkv, D]`` into the pools at ``slot_mapping [T]`` (int64).

    In place on the pools, on the current stream.  Same dtype in and out is a
    raw copy; a float8_e4m3fn pool quantises with the per-KV-head scales.
    """
    lib = _lib.load()
    nb, hkv, bs, d = _check_pools(k_pool, v_pool)
    _req(key.dim() == 3 and key.shape == value.shape and key.dtype == value.dtype,
         f"key/value must both be [T, Hkv, D]; got {tuple(key.shape)} and {tuple(value.shape)}")
    _req(key.shape[1] == hkv and key.shape[2] == d,
         f"key is [T, {key.shape[1]}, {key.shape[2]}] but the pool holds [{hkv}, {d}] rows")
    _req(slot_mapping.dtype == torch.int64 and slot_mapping.dim() == 1
         and slot_mapping.numel() == key.shape[0] and slot_mapping.is_contiguous(),
         "slot_mapping must be a contiguous int64 vector with one entry per row")
    for t, n in ((value, "value"), (k_pool, "k_pool"), (slot_mapping, "slot_mapping")):
        _dev(t, key, n)
    ks, vs = (None, None) if key.dtype == k_pool.dtype else _check_scales(k_scale, v_scale, k_pool, hkv)
    if key.stride(2) != 1 or key.stride() != value.stride():
        key, value = key.contiguous(), value.contiguous()
    rc = lib.aicomp_kv_append(key.data_ptr(), value.data_ptr(), key.stride(0), key.stride(1),
                              k_pool.data_ptr(), v_pool.data_ptr(), slot_mapping.data_ptr(),
                              key.shape[0], hkv, d, bs, nb, _dt(key, "key"), _dt(k_pool, "pool"),
                              _ptr(ks), _ptr(vs), _stream(key))
    _lib.check(rc, lib)


# split-K scratch, one growing buffer per (device, stream)
_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}


def _workspace(device: torch.device, nbytes: int, stream: Optional[int] = None) -> Optional[torch.Tensor]:
    if nbytes == 0:
        return None
    key = (device.index or 0, _current_stream(device) if stream is None else stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


# bumped whenever the routing threshold changes: sizes cached under an older value are asked for again
_route_epoch = 0


def set_small_decode_tokens(tokens: int) -> int:
    """Set the library's routing threshold between the two decode schedules (tokens = rows x table
    width x block size up to which an automatic call takes the grid schedule; 0: always balanced)
    and return the previous value; a negative value only queries.  Process-wide."""
    global _route_epoch
    prev = int(_lib.load().aicomp_kv_set_small_decode_tokens(int(tokens)))
    if tokens >= 0 and tokens != prev:
        _route_epoch += 1
    return prev


def decode_partition_size(batch: int, hq: int, hkv: int, d: int, bs: int, max_blocks: int,
                          q_dtype: torch.dtype, kv_dtype: torch.dtype) -> int:
    lib = _lib.load()
    return lib.aicomp_paged_decode_partition_size(batch, hq, hkv, d, bs, max_blocks,
                                                  _DT[q_dtype], _DT[kv_dtype])


def decode_workspace_bytes(batch: int, hq: int, hkv: int, d: int, bs: int, max_blocks: int,
                           q_dtype: torch.dtype, kv_dtype: torch.dtype, partition_size: int = 0) -> int:
    """Scratch bytes ``paged_decode_attn`` needs for these shapes.  A caller that must not allocate
    inside the call (a step recorded into a HIP graph) allocates this once and passes it as
    ``workspace``; the buffer needs no initialisation."""
    lib = _lib.load()
    return lib.aicomp_paged_decode_workspace_bytes(batch, hq, hkv, d, bs, max_blocks, _DT[q_dtype],
                                                   _DT[kv_dtype], partition_size)


def paged_decode_attn(out: torch.Tensor, query: torch.Tensor, k_pool: torch.Tensor,
                      v_pool: torch.Tensor, block_table: torch.Tensor,
                      context_lens: torch.Tensor, scale: float,
                      k_scale: Optional[torch.Tensor] = None,
                      v_scale: Optional[torch.Tensor] = None, partition_size: int = 0,
                      workspace: Optional[torch.Tensor] = None,
                      new_key: Optional[torch.Tensor] = None,
                      new_value: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[b, h] = softmax(q[b, h] . K_b^T * scale) V_b`` over the paged context.

    ``out``/``query`` ``[B, Hq, D]``; ``block_table [B, max_blocks]`` int32;
    ``context_lens [B]`` int32.  In place on ``out``, on the current stream.

    With ``new_key`` / ``new_value`` ``[B, Hkv, D]`` the call first appends row b as token
    ``context_lens[b] - 1`` of sequence b (the pools are written) - one decode step of the
    reference operator in one call.
    """
    lib = _lib.load()
    _req(query.is_cuda, "tensors must live on a ROCm device (there is no CPU path)")
    nb, hkv, bs, d = _check_pools(k_pool, v_pool)
    _req(query.dim() == 3 and out.shape == query.shape and out.dtype == query.dtype,
         f"out/query must both be [B, Hq, D]; got {tuple(out.shape)} and {tuple(query.shape)}")
    B, hq, dq = query.shape
    _req(dq == d, f"query head_dim {dq} != pool head_dim {d}")
    _req(query.is_contiguous() and out.is_contiguous(), "query and out must be contiguous")
    _req(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] == B
         and block_table.stride(1) == 1, "block_table must be int32 [B, max_blocks], rows contiguous")
    _req(context_lens.dtype == torch.int32 and context_lens.numel() == B
         and context_lens.is_contiguous(), "context_lens must be contiguous int32 [B]")
    for t, n in ((out, "out"), (k_pool, "k_pool"), (block_table, "block_table"),
                 (context_lens, "context_lens")):
        _dev(t, query, n)
    ks, vs = _check_scales(k_scale, v_scale, k_pool, hkv)
    qd, kd = _dt(query, "query"), _dt(k_pool, "pool")
    need = lib.aicomp_paged_decode_workspace_bytes(B, hq, hkv, d, bs, block_table.shape[1], qd, kd,
                                                   partition_size)
    if workspace is None:
        workspace = _workspace(query.device, need)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    if new_key is not None:
        _req(new_value is not None and new_key.shape == (B, hkv, d) and new_value.shape == (B, hkv, d)
             and new_key.dtype == query.dtype and new_value.dtype == query.dtype,
             f"new_key/new_value must both be [{B}, {hkv}, {d}] of the query dtype")
        _dev(new_key, query, "new_key")
        _dev(new_value, query, "new_value")
        if new_key.stride(2) != 1 or new_key.stride() != new_value.stride():
            new_key, new_value = new_key.contiguous(), new_value.contiguous()
        rc = lib.aicomp_paged_decode_attn_append(
            out.data_ptr(), query.data_ptr(), new_key.data_ptr(), new_value.data_ptr(),
            new_key.stride(0), new_key.stride(1), k_pool.data_ptr(), v_pool.data_ptr(),
            block_table.data_ptr(), block_table.stride(0), context_lens.data_ptr(), B, hq, hkv, d, bs,
            block_table.shape[1], nb, float(scale), qd, kd, _ptr(ks), _ptr(vs), partition_size,
            _ptr(workspace), ws_bytes, _stream(query))
        _lib.check(rc, lib)
        return out
    rc = lib.aicomp_paged_decode_attn(out.data_ptr(), query.data_ptr(), k_pool.data_ptr(),
                                      v_pool.data_ptr(), block_table.data_ptr(),
                                      block_table.stride(0), context_lens.data_ptr(), B, hq, hkv, d,
                                      bs, block_table.shape[1], nb, float(scale), qd, kd,
                                      _ptr(ks), _ptr(vs), partition_size, _ptr(workspace),
                                      ws_bytes, _stream(query))
    _lib.check(rc, lib)
    return out


class PreparedDecode:
    """``paged_decode_attn`` bound to fixed pools, block table, scales and head geometry.

    The shape / dtype / device / contiguity checks of everything that does not change from step
    to step run once, here; a call checks only the per-step tensors.  For callers that own their
    pools and tables (one decode call per layer and token at small batch is bound by the host, not
    by the GPU).  ``context_lens`` may be replaced per call by another contiguous int32 ``[B]``
    tensor on the same device.
    """

    def __init__(self, k_pool: torch.Tensor, v_pool: torch.Tensor, block_table: torch.Tensor,
                 context_lens: torch.Tensor, num_q_heads: int, q_dtype: torch.dtype, scale: float,
                 k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None,
                 partition_size: int = 0) -> None:
        self.lib = _lib.load()
        _req(k_pool.is_cuda, "tensors must live on a ROCm device (there is no CPU path)")
        nb, hkv, bs, d = _check_pools(k_pool, v_pool)
        B = block_table.shape[0]
        _req(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
             "block_table must be int32 [B, max_blocks], rows contiguous")
        _req(context_lens.dtype == torch.int32 and context_lens.numel() == B and context_lens.is_contiguous(),
             "context_lens must be contiguous int32 [B]")
        _req(num_q_heads > 0 and num_q_heads % hkv == 0, f"{num_q_heads} query heads over {hkv} KV heads")
        _dev(block_table, k_pool, "block_table")
        _dev(context_lens, k_pool, "context_lens")
        ks, vs = _check_scales(k_scale, v_scale, k_pool, hkv)
        try:
            qd = _DT[q_dtype]
        except KeyError:
            raise RuntimeError(f"query: unsupported dtype {q_dtype}")
        self.device, self.q_dtype = k_pool.device, q_dtype
        self.q_shape = (B, num_q_heads, d)
        self.kv_shape = (B, hkv, d)
        self.context_lens = context_lens
        self._need_args = (B, num_q_heads, hkv, d, bs, block_table.shape[1], qd, _dt(k_pool, "pool"), partition_size)
        self._need, self._epoch = self.lib.aicomp_paged_decode_workspace_bytes(*self._need_args), _route_epoch
        # keep the tensors alive; everything below is what the C entry points take
        self._keep = (k_pool, v_pool, block_table, ks, vs)
        self._head = (k_pool.data_ptr(), v_pool.data_ptr(), block_table.data_ptr(), block_table.stride(0))
        self._tail = (B, num_q_heads, hkv, d, bs, block_table.shape[1], nb, float(scale), qd,
                      _dt(k_pool, "pool"), _ptr(ks), _ptr(vs), partition_size)

    @property
    def need(self) -> int:
        """Scratch bytes of a call, for the routing threshold in force now."""
        if self._epoch != _route_epoch:
            self._need, self._epoch = self.lib.aicomp_paged_decode_workspace_bytes(*self._need_args), _route_epoch
        return self._need

    def __call__(self, out: torch.Tensor, query: torch.Tensor, new_key: Optional[torch.Tensor] = None,
                 new_value: Optional[torch.Tensor] = None,
                 context_lens: Optional[torch.Tensor] = None) -> torch.Tensor:
        _req(query.shape == self.q_shape and out.shape == self.q_shape and query.dtype == self.q_dtype
             and out.dtype == self.q_dtype and query.device == self.device and out.device == self.device
             and query.is_contiguous() and out.is_contiguous(),
             f"out/query must be contiguous {self.q_shape} {self.q_dtype} tensors on {self.device}")
        ctx = self.context_lens if context_lens is None else context_lens
        stream = _current_stream(self.device)
        ws = _workspace(self.device, self.need, stream)
        ws_ptr, ws_bytes = (None, 0) if ws is None else (ws.data_ptr(), ws.numel())
        if new_key is None:
            rc = self.lib.aicomp_paged_decode_attn(out.data_ptr(), query.data_ptr(), *self._head, ctx.data_ptr(),
                                                   *self._tail, ws_ptr, ws_bytes, stream)
        else:
            _req(new_value is not None and new_key.shape == self.kv_shape and new_value.shape == self.kv_shape
                 and new_key.dtype == self.q_dtype and new_value.dtype == self.q_dtype
                 and new_key.device == self.device and new_value.device == self.device,
                 f"new_key/new_value must both be {self.kv_shape} of the query dtype on {self.device}")
            if new_key.stride(2) != 1 or new_key.stride() != new_value.stride():
                new_key, new_value = new_key.contiguous(), new_value.contiguous()
            rc = self.lib.aicomp_paged_decode_attn_append(
                out.data_ptr(), query.data_ptr(), new_key.data_ptr(), new_value.data_ptr(),
                new_key.stride(0), new_key.stride(1), *self._head, ctx.data_ptr(), *self._tail,
                ws_ptr, ws_bytes, stream)
        _lib.check(rc, self.lib)
        return out

    def step4d(self, out: torch.Tensor, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
               group: int, context_lens, ready=None, width: Optional[int] = None) -> torch.Tensor:
        """The fused append + decode call on the operator's own tensors: ``query`` / ``out``
        ``[B, Hq, 1, D]`` contiguous, ``key`` / ``value`` ``[B, H, 1, D]`` with H = Hkv or
        Hkv * group (heads repeated ``group`` times, as HF's ``repeat_kv`` leaves them: every
        group-th head is read).  No view tensors are made: the strides go to the library as they
        are.  ``context_lens`` is an int32 ``[B]`` tensor on the device, or its device address.
        ``ready``, if given, is called once the arguments have passed every check, right before
        the launch (for work that must not happen for a rejected call).  ``width`` (at most the
        table's width) tells the library how many table columns are in use, so that it sizes the
        split for the contexts as they are now."""
        B, Hq, D = self.q_shape
        hkv = self.kv_shape[1]
        H = key.shape[1]
        hstep = group if (group > 1 and H == hkv * group) else 1
        _req(query.shape == (B, Hq, 1, D) and out.shape == (B, Hq, 1, D) and query.dtype == self.q_dtype
             and out.dtype == self.q_dtype and query.device == self.device and out.device == self.device
             and query.is_contiguous() and out.is_contiguous(),
             f"out/query must be contiguous {(B, Hq, 1, D)} {self.q_dtype} tensors on {self.device}")
        _req(key.shape == (B, hkv * hstep, 1, D) and value.shape == key.shape and key.dtype == self.q_dtype
             and value.dtype == self.q_dtype and key.device == self.device and value.device == self.device,
             f"key/value must both be [{B}, {hkv} or {hkv}*group, 1, {D}] of the query dtype on {self.device}")
        if key.stride(3) != 1 or key.stride() != value.stride():
            key, value = key.contiguous(), value.contiguous()
        stream = _current_stream(self.device)
        ws = _workspace(self.device, self.need, stream)
        ws_ptr, ws_bytes = (None, 0) if ws is None else (ws.data_ptr(), ws.numel())
        if ready is not None:
            ready()
        tail = self._tail
        if width is not None and 0 < width < tail[5]:
            tail = tail[:5] + (width,) + tail[6:]
        rc = self.lib.aicomp_paged_decode_attn_append(
            out.data_ptr(), query.data_ptr(), key.data_ptr(), value.data_ptr(),
            key.stride(0), key.stride(1) * hstep, *self._head,
            context_lens if isinstance(context_lens, int) else context_lens.data_ptr(), *tail,
            ws_ptr, ws_bytes, stream)
        _lib.check(rc, self.lib)
        return out


def prefill_tile_positions(num_q_heads: int, num_kv_heads: int, head_dim: int, block_size: int,
                           q_dtype: torch.dtype, kv_dtype: torch.dtype, max_q_len: int) -> int:
    """Positions per query tile (one workgroup row) of the kernel a prefill call with these shapes
    runs on; 0 when that kernel takes no item list."""
    return _lib.load().aicomp_paged_prefill_tile_positions(num_q_heads, num_kv_heads, head_dim, block_size,
                                                           _DT[q_dtype], _DT[kv_dtype], int(max_q_len))


def prefill_items(context_lens, new_lens, tile_positions: int, num_head_groups: int = 1,
                  num_cus: int = 0):
    """The order in which a prefill launch should take its (sequence, query tile) pairs, from the
    lengths a step planner holds on the host: an ``int32 [n, 2]`` numpy array for
    ``paged_prefill_attn(items=...)``, every tile that has rows exactly once.

    A tile costs as many steps as its last row has keys (prior context + positions up to the
    tile's end), and chunks of different priors and lengths differ several-fold, so the list is
    sorted by that, most expensive first: places that free up go to the longest tiles left.
    When the whole launch is resident at once (at most two workgroups per CU;
    ``num_head_groups`` workgroups per item) the second round is handed out from the cheap end
    instead, so that the two workgroups sharing a CU are an expensive and a cheap tile.
    """
    import numpy as np
    ctx = np.asarray(context_lens, dtype=np.int64)
    new = np.asarray(new_lens, dtype=np.int64)
    if tile_positions <= 0 or ctx.shape != new.shape:
        raise ValueError("prefill_items: tile_positions must be positive and the two length vectors alike")
    # (a chunk longer than its context, an inconsistent plan, keeps its tiles: the kernel defines its rows as zero)
    tiles = np.where(new > 0, -(-new // tile_positions), 0)
    seq = np.repeat(np.arange(ctx.size), tiles)
    first = np.cumsum(tiles) - tiles
    q = np.arange(seq.size) - np.repeat(first, tiles)
    keys = np.minimum(ctx[seq], ctx[seq] - new[seq] + (q + 1) * tile_positions)
    order = np.argsort(-keys, kind="stable")
    n = order.size
    per_round = num_cus // num_head_groups if num_cus > 0 and num_head_groups > 0 and num_cus % num_head_groups == 0 else 0
    if per_round and per_round < n <= 2 * per_round:
        # the first pass over the CUs takes the per_round most expensive tiles in falling order, the second the rest in rising order
        order = np.concatenate([order[:per_round], order[per_round:][::-1]])
    return np.stack([seq[order], q[order]], axis=1).astype(np.int32)


def step_items(context_lens, new_lens, num_prefill_seqs: int, tile_positions: int,
               num_head_groups: int = 1, num_cus: int = 0):
    """Item order for ONE prefill launch over a whole mixed step: the first ``num_prefill_seqs``
    sequences are prompt chunks, the others one-token decode rows (chunks of one token, which the
    kernel handles), ``int32 [n, 2]`` for ``paged_prefill_attn(items=...)``.

    A chunk tile is bound by the matrix cores, a decode row by the latency of its loads; two
    workgroups share a CU, and the launch is shortest when they are one of each kind.  When the
    decode rows are the longer items the list therefore opens with one CU-round of decode rows
    (longest first), then one of chunk tiles, which land beside them, and hands the rest out
    alternately, each kind longest first.  When the chunk tiles are the longer items the order is
    simply falling cost: the short rows then fill the launch's tail.  Measured on 32 / 8 heads,
    head_dim 128: 4 chunks of 512 with 60 rows of 512 to 4096 tokens 138 us against 144 us in
    falling order and 174 us chunks first; with rows of 128 to 1024 tokens falling order wins,
    78 against 93 us.
    """
    import numpy as np
    ctx = np.asarray(context_lens, dtype=np.int64)
    new = np.asarray(new_lens, dtype=np.int64)
    base = prefill_items(ctx, new, tile_positions, num_head_groups, 0)          # falling cost
    pre, dec = base[base[:, 0] < num_prefill_seqs], base[base[:, 0] >= num_prefill_seqs]
    per_round = num_cus // num_head_groups if num_cus > 0 and num_head_groups > 0 else 0
    if not len(pre) or not len(dec) or per_round <= 0:
        return base
    cost = lambda it: np.minimum(ctx[it[:, 0]], ctx[it[:, 0]] - new[it[:, 0]] + (it[:, 1] + 1) * tile_positions)
    if cost(dec).mean() < cost(pre).mean():
        return base
    a, b = dec[per_round:], pre[per_round:]
    k = min(len(a), len(b))
    rest = np.empty((2 * k, 2), dtype=base.dtype)
    rest[0::2], rest[1::2] = a[:k], b[:k]
    return np.concatenate([dec[:per_round], pre[:per_round], rest, a[k:], b[k:]]).astype(np.int32)


def paged_prefill_attn(out: torch.Tensor, query: torch.Tensor, k_pool: torch.Tensor,
                       v_pool: torch.Tensor, block_table: torch.Tensor,
                       context_lens: torch.Tensor, cu_q_lens: torch.Tensor, scale: float,
                       max_q_len: Optional[int] = None,
                       k_scale: Optional[torch.Tensor] = None,
                       v_scale: Optional[torch.Tensor] = None,
                       items: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of concatenated chunks ``query [T, Hq, D]`` over the pool.

    Chunk s owns rows ``cu_q_lens[s]:cu_q_lens[s+1]``; its context of
    ``context_lens[s]`` tokens (chunk included) must already be in the pool.
    ``max_q_len`` is the host-side bound on the chunk lengths; when omitted it
    is read back from ``cu_q_lens`` (a device synchronisation).  ``items`` (``int32 [n, 2]`` on
    the device, see ``prefill_items``) gives the order of the (sequence, query tile) pairs.
    """
    lib = _lib.load()
    nb, hkv, bs, d = _check_pools(k_pool, v_pool)
    _req(query.dim() == 3 and out.shape == query.shape and out.dtype == query.dtype,
         f"out/query must both be [T, Hq, D]; got {tuple(out.shape)} and {tuple(query.shape)}")
    T, hq, dq = query.shape
    _req(dq == d, f"query head_dim {dq} != pool head_dim {d}")
    _req(query.is_contiguous() and out.is_contiguous(), "query and out must be contiguous")
    S = context_lens.numel()
    _req(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] == S
         and block_table.stride(1) == 1, "block_table must be int32 [S, max_blocks], rows contiguous")
    _req(context_lens.dtype == torch.int32 and context_lens.is_contiguous(),
         "context_lens must be contiguous int32 [S]")
    _req(cu_q_lens.dtype == torch.int32 and cu_q_lens.numel() == S + 1 and cu_q_lens.is_contiguous(),
         "cu_q_lens must be contiguous int32 [S+1]")
    for t, n in ((out, "out"), (k_pool, "k_pool"), (block_table, "block_table"),
                 (context_lens, "context_lens"), (cu_q_lens, "cu_q_lens")):
        _dev(t, query, n)
    ks, vs = _check_scales(k_scale, v_scale, k_pool, hkv)
    if max_q_len is None:
        cu = cu_q_lens.cpu()
        max_q_len = int((cu[1:] - cu[:-1]).max()) if S else 0
    if items is not None and items.numel():
        _req(items.dtype == torch.int32 and items.dim() == 2 and items.shape[1] == 2 and items.is_contiguous(),
             "items must be a contiguous int32 [n, 2] tensor of (sequence, query tile) pairs")
        _dev(items, query, "items")
        rc = lib.aicomp_paged_prefill_attn_items(out.data_ptr(), query.data_ptr(), k_pool.data_ptr(),
                                                 v_pool.data_ptr(), block_table.data_ptr(),
                                                 block_table.stride(0), context_lens.data_ptr(),
                                                 cu_q_lens.data_ptr(), S, T, int(max_q_len), hq, hkv, d, bs,
                                                 block_table.shape[1], nb, float(scale),
                                                 _dt(query, "query"), _dt(k_pool, "pool"), _ptr(ks), _ptr(vs),
                                                 items.data_ptr(), items.shape[0], _stream(query))
        _lib.check(rc, lib)
        return out
    rc = lib.aicomp_paged_prefill_attn(out.data_ptr(), query.data_ptr(), k_pool.data_ptr(),
                                       v_pool.data_ptr(), block_table.data_ptr(),
                                       block_table.stride(0), context_lens.data_ptr(),
                                       cu_q_lens.data_ptr(), S, T, int(max_q_len), hq, hkv, d, bs,
                                       block_table.shape[1], nb, float(scale),
                                       _dt(query, "query"), _dt(k_pool, "pool"), _ptr(ks), _ptr(vs),
                                       _stream(query))
    _lib.check(rc, lib)
    return out


def rotary_tables(inv_freq: torch.Tensor, num_positions: int, dtype: torch.dtype,
                  attention_scaling: float = 1.0, device=None):
    """cos / sin tables ``[num_positions, D]`` the way the reference's rotary module builds them
    per call (compiler_fx/modeling_llama.py:150-168): ``freqs = position * inv_freq`` in
    float32, ``emb = cat(freqs, freqs)``, ``cos(emb) * attention_scaling`` cast to the
    tensor type.  Built once; ``rope_kv_append`` indexes them by position.
    """
    device = inv_freq.device if device is None else device
    inv = inv_freq.to(device=device, dtype=torch.float32)
    pos = torch.arange(num_positions, device=device, dtype=torch.float32)
    freqs = (inv[:, None] @ pos[None, :]).transpose(0, 1)          # the reference's matmul form
    emb = torch.cat((freqs, freqs), dim=-1)
    cos = (emb.cos() * attention_scaling).to(dtype).contiguous()
    sin = (emb.sin() * attention_scaling).to(dtype).contiguous()
    return cos, sin


def rope_kv_append(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, cos: torch.Tensor,
                   sin: torch.Tensor, positions: Optional[torch.Tensor], k_pool: torch.Tensor,
                   v_pool: torch.Tensor, slot_mapping: torch.Tensor,
                   k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None,
                   query_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotate ``query [T, Hq, D]`` and ``key [T, Hkv, D]`` by their positions and append the rotated
    key and ``value`` to the pools, in one launch.

    ``cos`` / ``sin`` are ``[P, D]`` tables of the query dtype; ``positions [T]`` int64 selects the
    row of each token (``None``: row t, i.e. per-token cos/sin as the reference passes them).
    Returns the rotated query (``query_out``, by default ``query`` itself, in place).  The three
    inputs may be views into one fused QKV projection output (last dimension contiguous).
    """
    lib = _lib.load()
    _req(query.is_cuda, "tensors must live on a ROCm device (there is no CPU path)")
    nb, hkv, bs, d = _check_pools(k_pool, v_pool)
    out = query if query_out is None else query_out
    _req(query.dim() == 3 and key.dim() == 3 and value.shape == key.shape and out.shape == query.shape,
         "query/query_out must be [T, Hq, D], key/value [T, Hkv, D]")
    T, hq, dq = query.shape
    _req(key.shape == (T, hkv, d) and dq == d,
         f"key/value {tuple(key.shape)} and query {tuple(query.shape)} do not match pools {tuple(k_pool.shape)}")
    _req(key.dtype == query.dtype and value.dtype == query.dtype and out.dtype == query.dtype,
         "query, key, value and query_out must share one dtype")
    _req(query.dtype in (torch.float32, torch.bfloat16, torch.float16), f"unsupported input dtype {query.dtype}")
    for t, n in ((query, "query"), (out, "query_out"), (key, "key"), (value, "value")):
        _req(t.stride(2) == 1, f"{n}: last dimension must be contiguous")
    _req(key.stride() == value.stride(), "key and value must have equal strides")
    _req(cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] == d and cos.dtype == query.dtype
         and sin.dtype == query.dtype and cos.stride(1) == 1 and cos.stride() == sin.stride(),
         f"cos/sin must be [P, {d}] tables of {query.dtype} with equal strides")
    if positions is not None:
        _req(positions.dtype == torch.int64 and positions.numel() == T and positions.is_contiguous(),
             "positions must be contiguous int64 [T]")
        _dev(positions, query, "positions")
    else:
        _req(cos.shape[0] >= T, "without positions the tables need one row per token")
    _req(slot_mapping.dtype == torch.int64 and slot_mapping.numel() == T and slot_mapping.is_contiguous(),
         "slot_mapping must be contiguous int64 [T]")
    for t, n in ((key, "key"), (value, "value"), (out, "query_out"), (cos, "cos"), (sin, "sin"),
                 (k_pool, "k_pool"), (slot_mapping, "slot_mapping")):
        _dev(t, query, n)
    _req(k_pool.dtype in (query.dtype, torch.float8_e4m3fn),
         f"pool dtype {k_pool.dtype} must be {query.dtype} or float8_e4m3fn")
    ks, vs = _check_scales(k_scale, v_scale, k_pool, hkv)
    if T == 0:
        return out
    rc = lib.aicomp_rope_kv_append(
        query.data_ptr(), out.data_ptr(), query.stride(0), query.stride(1), out.stride(0), out.stride(1),
        key.data_ptr(), value.data_ptr(), key.stride(0), key.stride(1), cos.data_ptr(), sin.data_ptr(),
        cos.stride(0), cos.shape[0], _ptr(positions), k_pool.data_ptr(), v_pool.data_ptr(),
        slot_mapping.data_ptr(), T, hq, hkv, d, bs, nb, _dt(query, "query"), _dt(k_pool, "pool"),
        _ptr(ks), _ptr(vs), _stream(query))
    _lib.check(rc, lib)
    return out


def sample_tokens(logits: torch.Tensor, temperature: float = 1.0, top_k: int = 0, top_p: float = 1.0,
                  do_sample: bool = True, uniforms: Optional[torch.Tensor] = None,
                  generator: Optional[torch.Generator] = None, return_probs: bool = False):
    """Next token of every row of ``logits [B, V]`` (float32 or bfloat16), as ``_sample_token`` of the
    reference picks it (opt_prime/opt_prime/inference.py:786-843): greedy argmax when ``do_sample``
    is false, otherwise temperature, top-k, top-p and one draw per row.  ``logits`` is not modified.

    ``uniforms [B]`` (float32 in [0, 1)) makes the draw reproducible; by default they come from
    ``torch.rand`` with ``generator``.  Returns ``tokens [B]`` int64, or ``(tokens, probs [B, V])``.
    """
    lib = _lib.load()
    _req(logits.is_cuda, "tensors must live on a ROCm device (there is no CPU path)")
    _req(logits.dim() == 2 and logits.stride(1) == 1, "logits must be [B, V] with contiguous rows")
    _req(logits.dtype in (torch.float32, torch.bfloat16, torch.float16), f"unsupported logits dtype {logits.dtype}")
    B, V = logits.shape
    out = torch.empty(B, dtype=torch.int64, device=logits.device)
    probs = torch.empty(B, V, dtype=torch.float32, device=logits.device) if return_probs else None
    if do_sample:
        if uniforms is None:
            uniforms = torch.rand(B, dtype=torch.float32, device=logits.device, generator=generator)
        _req(uniforms.dtype == torch.float32 and uniforms.numel() == B and uniforms.is_contiguous(),
             "uniforms must be contiguous float32 [B]")
        _dev(uniforms, logits, "uniforms")
    if B:
        rc = lib.aicomp_sample_tokens(out.data_ptr(), logits.data_ptr(), logits.stride(0), _ptr(probs),
                                      _ptr(uniforms) if do_sample else None, B, V, float(temperature),
                                      int(top_k), float(top_p), 0 if do_sample else 1, _dt(logits, "logits"),
                                      _stream(logits))
        _lib.check(rc, lib)
    return (out, probs) if return_probs else out
