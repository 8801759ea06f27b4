"""Host side of the paged pool: block allocator and per-step planner.

The reference keeps one scalar write position shared by every sequence of a
batch (``cache_pos`` in opt_prime/opt_prime/kv_cache.py:290, ``_seq_len`` in
kv_cache.py:69) and resets it between requests (opt_prime/opt_prime/
inference.py:946-955, 1100-1111).  A paged pool needs more: which physical
blocks each sequence owns, and, for every step, the four index tensors the
kernels read (``block_table``, ``context_lens``, ``slot_mapping``,
``cu_q_lens``).  This module produces them.

``BlockAllocator``  LIFO free list over the pool's block ids with an owner
                    check on free (a double free would alias two sequences).
``StepPlanner``     sequences with independent lengths: admit, chunked prompt
                    ingestion under a per-step token budget, one token per
                    running sequence per decode step, preemption of the
                    youngest sequence when the pool runs dry, release on
                    finish.  ``schedule()`` returns a ``StepPlan`` whose
                    tensors are already on the device: the whole plan is
                    packed into one pinned staging buffer and moved with a
                    single asynchronous copy.

Row order inside a plan: sequences that ingest more than one token (prompt
chunks) first, then the one-token sequences; ``paged_attention_step`` below
runs the append, the chunked-prefill kernel on the first group and the decode
kernel on the second, or, for a mixed step with a moderate decode part, one
launch of the chunked-prefill kernel over both (``StepPlan.step_items``).

Token t of a sequence lives in slot ``block_table[t // BS] * BS + t % BS``.
"""
from __future__ import annotations

import os
from collections import deque
from dataclasses import dataclass
from typing import Deque, Dict, Iterable, List, Optional

import numpy as np
import torch


class OutOfBlocks(ValueError):
    """The pool has fewer free blocks than the request needs (the reference's cache
    overflow is a ``ValueError`` too: opt_prime/opt_prime/kv_cache.py:152-156)."""


class PlanError(ValueError):
    """A step plan that would make the kernels read or write outside what it owns."""


def check_plan(plan: "StepPlan", num_blocks: int, block_size: int) -> None:
    """Host-side self-check of a plan, from its host arrays, before anything is launched on it.

    The kernels do not fault on a bad plan: an append row whose slot is outside the pool is
    skipped and a block id outside the pool is clamped into it, so a planner bug would show up as
    silently wrong attention.  This makes it loud: every slot inside the pool and used once, every
    table entry a sequence needs inside the pool and owned by that sequence alone, lengths within
    the table, chunk rows consistent with the lengths, slots and positions consistent with the table.
    Raises ``PlanError``.
    """
    bt, cl, cu = plan.host_block_table, plan.host_context_lens, plan.host_cu_q_lens
    slot, pos = plan.host_slot_mapping, plan.host_positions
    S = len(plan.seq_ids)
    T = int(plan.total_new_tokens)
    if bt.shape[0] != S or cl.shape[0] != S or cu.shape[0] != S + 1 or slot.shape[0] != T or pos.shape[0] != T:
        raise PlanError(f"plan arrays do not match {S} sequences / {T} new tokens")
    if cu[0] != 0 or cu[-1] != T or (np.diff(cu) < 0).any():
        raise PlanError(f"cu_q_lens is not a prefix sum ending at {T}: {cu.tolist()}")
    new = np.diff(cu)
    if (new != plan.new_lens).any():
        raise PlanError("cu_q_lens and new_lens disagree")
    if (cl < new).any() or (cl <= 0).any():
        bad = int(np.flatnonzero((cl < new) | (cl <= 0))[0])
        raise PlanError(f"sequence row {bad}: context length {int(cl[bad])} < its {int(new[bad])} new tokens")
    if (cl > bt.shape[1] * block_size).any():
        bad = int(np.flatnonzero(cl > bt.shape[1] * block_size)[0])
        raise PlanError(f"sequence row {bad}: context length {int(cl[bad])} exceeds the table width "
                        f"{bt.shape[1]} x {block_size}")
    if T and ((slot < 0).any() or (slot >= num_blocks * block_size).any()):
        bad = int(np.flatnonzero((slot < 0) | (slot >= num_blocks * block_size))[0])
        raise PlanError(f"new token {bad}: slot {int(slot[bad])} is outside the pool of "
                        f"{num_blocks} x {block_size} slots")
    if T and np.unique(slot).size != T:
        raise PlanError("two new tokens share a slot")
    need = -(-cl.astype(np.int64) // block_size)
    owned = []
    for r in range(S):
        ids = bt[r, :need[r]]
        if ((ids < 0) | (ids >= num_blocks)).any():
            bad = int(ids[(ids < 0) | (ids >= num_blocks)][0])
            raise PlanError(f"sequence row {r}: block id {bad} is outside the pool of {num_blocks} blocks")
        owned.append(ids)
        p = pos[cu[r]:cu[r + 1]]
        if (p != np.arange(cl[r] - new[r], cl[r])).any():
            raise PlanError(f"sequence row {r}: positions are not {int(cl[r] - new[r])}..{int(cl[r]) - 1}")
        if (slot[cu[r]:cu[r + 1]] != ids[p // block_size].astype(np.int64) * block_size + p % block_size).any():
            raise PlanError(f"sequence row {r}: slots do not follow from its block table")
    if owned:
        allb = np.concatenate(owned)
        if np.unique(allb).size != allb.size:
            raise PlanError("two sequences of the plan share a block")


class BlockAllocator:
    """Free list over block ids ``0 .. num_blocks-1``.

    LIFO, so a block released by a finished sequence is the next one handed out (its
    lines are the most likely to still be in a cache).  ``allocate`` is all-or-nothing.
    """

    def __init__(self, num_blocks: int, block_size: int = 16) -> None:
        if num_blocks <= 0 or block_size <= 0:
            raise ValueError(f"num_blocks and block_size must be positive, got {num_blocks}, {block_size}")
        self.num_blocks = int(num_blocks)
        self.block_size = int(block_size)
        # stack of free ids; block 0 is handed out first
        self._free = np.arange(self.num_blocks - 1, -1, -1, dtype=np.int32)
        self._top = self.num_blocks
        self._owned = np.zeros(self.num_blocks, dtype=bool)

    @property
    def num_free(self) -> int:
        return self._top

    @property
    def num_used(self) -> int:
        return self.num_blocks - self._top

    def can_allocate(self, n: int) -> bool:
        return 0 <= n <= self._top

    def allocate(self, n: int) -> np.ndarray:
        if n < 0:
            raise ValueError(f"cannot allocate {n} blocks")
        if n > self._top:
            raise OutOfBlocks(f"need {n} blocks, {self._top} of {self.num_blocks} free")
        out = self._free[self._top - n:self._top][::-1].copy()
        self._top -= n
        self._owned[out] = True
        return out

    def free(self, blocks: Iterable[int]) -> None:
        b = np.asarray(list(blocks) if not isinstance(blocks, np.ndarray) else blocks, dtype=np.int64)
        if b.size == 0:
            return
        if b.min() < 0 or b.max() >= self.num_blocks:
            raise ValueError("block id out of range")
        if np.unique(b).size != b.size or not self._owned[b].all():
            raise ValueError("freeing a block that is not allocated (double free)")
        self._owned[b] = False
        self._free[self._top:self._top + b.size] = b[::-1].astype(np.int32)
        self._top += b.size

    def blocks_for(self, num_tokens: int) -> int:
        return -(-int(num_tokens) // self.block_size)


def pool_blocks_for_budget(budget_bytes: int, num_layers: int, num_kv_heads: int, head_dim: int,
                           dtype: torch.dtype, block_size: int = 16) -> int:
    """Blocks per layer that fit ``budget_bytes`` of HBM (K and V pools of every layer)."""
    per_block = 2 * num_layers * num_kv_heads * block_size * head_dim * torch.empty((), dtype=dtype).element_size()
    return int(budget_bytes // per_block)


@dataclass
class StepPlan:
    """Index tensors of one step, in the row order of the kernels.

    ``seq_ids[i]`` ingests ``new_lens[i]`` tokens at positions
    ``context_lens[i] - new_lens[i] .. context_lens[i] - 1``.
    """
    seq_ids: List[object]
    num_prefill_seqs: int
    new_lens: np.ndarray                  # [S] int32 (host)
    max_q_len: int                        # longest chunk among the first num_prefill_seqs rows
    total_new_tokens: int
    block_table: torch.Tensor             # [S, max_blocks_per_seq] int32
    context_lens: torch.Tensor            # [S] int32, after this step's append
    cu_q_lens: torch.Tensor               # [S+1] int32
    slot_mapping: torch.Tensor            # [T] int64
    positions: torch.Tensor               # [T] int64 position of each new token in its sequence
    preempted: List[object]               # sequences sent back to the waiting queue by this call
    # host copies of the same arrays (what the tests and the oracle read)
    host_block_table: np.ndarray = None
    host_context_lens: np.ndarray = None
    host_cu_q_lens: np.ndarray = None
    host_slot_mapping: np.ndarray = None
    host_positions: np.ndarray = None
    # order of the prompt chunks' query tiles per (tile size, head groups): one list serves every layer of the step
    _prefill_items: dict = None

    def prefill_items(self, query: torch.Tensor, k_pool: torch.Tensor) -> Optional[torch.Tensor]:
        """The (sequence, query tile) pairs of this step's prompt chunks, most expensive first, as the
        device tensor ``ops.paged_prefill_attn(items=...)`` takes; ``None`` when the step has fewer
        than two chunks (the kernel's own order is as good) or the kernel at hand takes no list.
        Built once per step from the host copies of the lengths and reused by every layer."""
        from . import ops
        npre = self.num_prefill_seqs
        if npre < 2:
            return None
        hq, hkv, d, bs = query.shape[1], k_pool.shape[1], k_pool.shape[3], k_pool.shape[2]
        tile = ops.prefill_tile_positions(hq, hkv, d, bs, query.dtype, k_pool.dtype, self.max_q_len)
        if tile <= 0:
            return None
        group = hq // hkv
        hgroups = hq // (group if 16 % group == 0 else 1)
        key = (tile, hgroups, query.device)
        if self._prefill_items is None:
            self._prefill_items = {}
        if key not in self._prefill_items:
            cus = torch.cuda.get_device_properties(query.device).multi_processor_count if query.is_cuda else 0
            items = ops.prefill_items(self.host_context_lens[:npre], self.new_lens[:npre], tile, hgroups, cus)
            self._prefill_items[key] = torch.from_numpy(items).to(query.device, non_blocking=True)
        return self._prefill_items[key]

    # Longest decode row and largest decode batch for which a mixed step goes through one launch
    # (measured on MI355X, 32 / 8 and 64 / 8 heads, head_dim 64 and 128, 1 to 16 chunks of 128 to
    # 2048 tokens with 16 to 250 rows: within these bounds the one launch takes 0.95 to 1.65 times
    # less than chunks and rows through their own kernels, 1.06 on 4 x 512 + 60 rows of up to 4096
    # tokens; a row of 8192 and more tokens, walked by a single workgroup row, makes it up to
    # twice as slow, and beyond ~128 rows the decode kernel's faster streaming wins)
    ONE_LAUNCH_MAX_CONTEXT = 4608
    ONE_LAUNCH_MAX_ROWS = 128

    def step_items(self, query: torch.Tensor, k_pool: torch.Tensor) -> Optional[torch.Tensor]:
        """Item list over ALL sequences of a mixed step (chunks and one-token rows) for one launch
        of the chunked-prefill kernel, or ``None`` when the step should go through the prefill
        and decode kernels separately: no chunk or no decode row in it, pools of another type
        than the 16-bit queries, a kernel that takes no list, a chunk bound too short for the
        two-column-group kernel, or a decode part outside the bounds above.  Cached per step."""
        from . import ops
        npre, ndec = self.num_prefill_seqs, self.num_decode_seqs
        if not npre or not ndec or ndec > self.ONE_LAUNCH_MAX_ROWS:
            return None
        if query.dtype not in (torch.bfloat16, torch.float16) or k_pool.dtype != query.dtype:
            return None
        if int(self.host_context_lens[npre:].max()) > self.ONE_LAUNCH_MAX_CONTEXT:
            return None
        hq, hkv, d, bs = query.shape[1], k_pool.shape[1], k_pool.shape[3], k_pool.shape[2]
        tile = ops.prefill_tile_positions(hq, hkv, d, bs, query.dtype, k_pool.dtype, self.max_q_len)
        group = hq // hkv
        gpack = group if 16 % group == 0 else 1
        if tile * gpack != 128:                   # (0: no list; 64: the one-column-group kernel)
            return None
        hgroups = hq // gpack
        key = ("step", tile, hgroups, query.device)
        if self._prefill_items is None:
            self._prefill_items = {}
        if key not in self._prefill_items:
            cus = torch.cuda.get_device_properties(query.device).multi_processor_count if query.is_cuda else 0
            items = ops.step_items(self.host_context_lens, self.new_lens, npre, tile, hgroups, cus)
            self._prefill_items[key] = torch.from_numpy(items).to(query.device, non_blocking=True)
        return self._prefill_items[key]

    @property
    def num_seqs(self) -> int:
        return len(self.seq_ids)

    @property
    def num_decode_seqs(self) -> int:
        return len(self.seq_ids) - self.num_prefill_seqs

    @property
    def num_prefill_tokens(self) -> int:
        return int(self.host_cu_q_lens[self.num_prefill_seqs])


class _Staging:
    """Ring of pinned host buffers, each paired with a device buffer and an event."""

    def __init__(self, nbytes: int, device: torch.device, depth: int = 4) -> None:
        self.device = device
        self.cuda = device.type == "cuda"
        self.nbytes = nbytes
        self.host = [torch.empty(nbytes, dtype=torch.uint8, pin_memory=self.cuda) for _ in range(depth)]
        self.dev = [torch.empty(nbytes, dtype=torch.uint8, device=device) for _ in range(depth)] if self.cuda else self.host
        # typed views of the device buffers, made once: a plan's tensors are then one slice each
        self.dev32 = [d[:nbytes // 8 * 8].view(torch.int32) for d in self.dev]
        self.dev64 = [d[:nbytes // 8 * 8].view(torch.int64) for d in self.dev]
        self.done = [torch.cuda.Event() if self.cuda else None for _ in range(depth)]
        self.used = [False] * depth
        self.i = 0

    def next(self):
        i = self.i
        self.i = (i + 1) % len(self.host)
        if self.cuda and self.used[i]:
            self.done[i].synchronize()          # the copy that last read this host buffer
        return i

    def upload(self, i: int, nbytes: int) -> int:
        if self.cuda:
            self.dev[i][:nbytes].copy_(self.host[i][:nbytes], non_blocking=True)
            self.done[i].record()
            self.used[i] = True
        return i


class StepPlanner:
    """Continuous batching over one paged pool.

    ``add_request`` queues a sequence; ``schedule`` decides what runs this step and
    returns the index tensors; ``finish`` releases a sequence's blocks.  Policy
    (first come, first served):

    1. every running sequence past its prompt gets one token (oldest first, within the
       step's token budget ``max_num_batched_tokens``);
    2. running sequences still inside their prompt, then waiting ones in arrival
       order, get a chunk of at most ``prefill_chunk`` tokens while the budget and
       the pool allow;
    3. if a running sequence needs a block and none is free, the youngest running
       sequence is preempted: its blocks are released and it re-enters the head of
       the waiting queue, to be recomputed from its prompt plus what it generated.

    Per-sequence state lives in arrays indexed by a row number (block-table row, cached
    length, block count), so a pure decode step is planned with a handful of vectorised
    numpy operations whatever the batch size.

    A plan's device tensors stay valid for ``staging_depth - 1`` further ``schedule``
    calls (they are views of a ring of staging buffers).
    """

    def __init__(self, num_blocks: int, block_size: int = 16, max_seqs: int = 256,
                 max_seq_len: int = 8192, max_num_batched_tokens: int = 4096,
                 prefill_chunk: int = 512, device="cuda", staging_depth: int = 4,
                 check_plans: Optional[bool] = None) -> None:
        # debug flag: run check_plan on every plan before its host-to-device copy (also switched on
        # by the environment variable AICOMP_CHECK_PLANS=1); off by default, it costs host time
        self.check_plans = (os.environ.get("AICOMP_CHECK_PLANS", "0") not in ("", "0")) if check_plans is None \
            else bool(check_plans)
        if max_seqs <= 0 or max_seq_len <= 0 or max_num_batched_tokens <= 0 or prefill_chunk <= 0:
            raise ValueError("max_seqs, max_seq_len, max_num_batched_tokens and prefill_chunk must be positive")
        self.alloc = BlockAllocator(num_blocks, block_size)
        self.block_size = block_size
        self.max_seqs = max_seqs
        self.max_seq_len = max_seq_len
        self.max_blocks_per_seq = -(-max_seq_len // block_size)
        self.max_num_batched_tokens = max_num_batched_tokens
        self.prefill_chunk = prefill_chunk
        self.device = torch.device(device)
        self.num_preemptions = 0
        self._arrivals = 0
        # waiting queue: (seq_id, tokens to ingest, original prompt length, max_new_tokens, arrival)
        self.waiting: Deque[tuple] = deque()
        self._waiting_ids = set()
        # running sequences, by row
        MB = self.max_blocks_per_seq
        self._row_of: Dict[object, int] = {}
        self._id_of: List[object] = [None] * max_seqs
        self._free_rows = list(range(max_seqs - 1, -1, -1))
        self._tab = np.zeros((max_seqs, MB), dtype=np.int32)
        self._nblk = np.zeros(max_seqs, dtype=np.int32)
        self._len = np.zeros(max_seqs, dtype=np.int32)        # tokens whose K/V rows are (being) written
        self._prompt = np.zeros(max_seqs, dtype=np.int32)     # tokens to ingest before decoding
        self._orig = np.zeros(max_seqs, dtype=np.int32)       # the request's own prompt length
        self._maxnew = np.zeros(max_seqs, dtype=np.int64)     # -1: unbounded
        self._arr = np.zeros(max_seqs, dtype=np.int64)
        self._live = np.zeros(max_seqs, dtype=bool)
        # packed layout (bytes): slot_mapping int64 [T] | positions int64 [T] | block_table int32 [S*MB] |
        # context_lens [S] | cu_q_lens [S+1]
        cap = 16 * max_num_batched_tokens + 4 * (max_seqs * MB + 2 * max_seqs + 1) + 64
        self._staging = _Staging(cap, self.device, staging_depth)

    # ------------------------------------------------------------------ requests
    def add_request(self, seq_id, prompt_len: int, max_new_tokens: Optional[int] = None) -> None:
        if prompt_len <= 0:
            raise ValueError(f"prompt_len must be positive, got {prompt_len}")
        if max_new_tokens is not None and max_new_tokens < 0:
            raise ValueError(f"max_new_tokens must be non-negative, got {max_new_tokens}")
        total = prompt_len + (max_new_tokens or 0)
        if total > self.max_seq_len:
            raise ValueError(f"sequence of {total} tokens exceeds max_seq_len {self.max_seq_len}")
        if self.alloc.blocks_for(total) > self.alloc.num_blocks:
            raise ValueError(f"sequence of {total} tokens can never fit a pool of {self.alloc.num_blocks} blocks")
        if seq_id in self._row_of or seq_id in self._waiting_ids:
            raise ValueError(f"sequence id {seq_id!r} is already known")
        self.waiting.append((seq_id, int(prompt_len), int(prompt_len),
                             -1 if max_new_tokens is None else int(max_new_tokens), self._arrivals))
        self._waiting_ids.add(seq_id)
        self._arrivals += 1

    def finish(self, seq_id) -> None:
        """Release a sequence (running or still waiting)."""
        r = self._row_of.pop(seq_id, None)
        if r is None:
            if seq_id not in self._waiting_ids:
                raise ValueError(f"unknown sequence id {seq_id!r}")
            self._waiting_ids.discard(seq_id)
            self.waiting = deque(w for w in self.waiting if w[0] != seq_id)
            return
        self._release_row(r)

    def _release_row(self, r: int) -> None:
        self.alloc.free(self._tab[r, :self._nblk[r]])
        self._nblk[r] = 0
        self._len[r] = 0
        self._live[r] = False
        self._id_of[r] = None
        self._free_rows.append(r)

    def context_len(self, seq_id) -> int:
        return int(self._len[self._row_of[seq_id]])

    def blocks_of(self, seq_id) -> List[int]:
        r = self._row_of[seq_id]
        return self._tab[r, :self._nblk[r]].tolist()

    def num_generated(self, seq_id) -> int:
        """Tokens sampled so far for a running sequence (the first one comes out of the step that
        ingests the end of its prompt)."""
        r = self._row_of[seq_id]
        return max(0, int(self._len[r]) - int(self._orig[r]) + 1)

    def completed(self) -> List[object]:
        """Running sequences that have produced their ``max_new_tokens``; the caller finishes them."""
        rows = np.flatnonzero(self._live & (self._maxnew >= 0) & (self._len >= self._prompt) &
                              (self._len - self._orig + 1 >= self._maxnew))
        return [self._id_of[r] for r in rows]

    @property
    def num_running(self) -> int:
        return len(self._row_of)

    def has_work(self) -> bool:
        return bool(self.waiting) or bool(self._row_of)

    # ------------------------------------------------------------------ scheduling
    def _preempt_youngest(self, protect: np.ndarray) -> Optional[object]:
        """Evict the most recently arrived running sequence outside ``protect`` (a row mask)."""
        cand = np.flatnonzero(self._live & ~protect)
        if cand.size == 0:
            return None
        r = int(cand[np.argmax(self._arr[cand])])
        sid = self._id_of[r]
        # recompute later: everything cached so far must be ingested again
        redo = int(self._len[r]) if self._len[r] >= self._prompt[r] else int(self._prompt[r])
        self.waiting.appendleft((sid, redo, int(self._orig[r]), int(self._maxnew[r]), int(self._arr[r])))
        self._waiting_ids.add(sid)
        del self._row_of[sid]
        self._release_row(r)
        self.num_preemptions += 1
        return sid

    def _grow_row(self, r: int, n_new: int) -> bool:
        need = self.alloc.blocks_for(int(self._len[r]) + n_new) - int(self._nblk[r])
        if need > 0:
            if not self.alloc.can_allocate(need):
                return False
            self._tab[r, self._nblk[r]:self._nblk[r] + need] = self.alloc.allocate(need)
            self._nblk[r] += need
        return True

    def schedule(self, decode: Optional[Iterable[object]] = None) -> Optional[StepPlan]:
        """Plan one step.  ``decode`` restricts which running sequences may take their one
        token this step (default: all of them); a driver that ingests a whole batch of prompts
        before its first decode step passes ``()`` until the last prompt is in."""
        budget = self.max_num_batched_tokens
        BS = self.block_size
        preempted: List[object] = []
        protect = np.zeros(self.max_seqs, dtype=bool)

        # 1. one token for every running sequence past its prompt, oldest first (vectorised)
        dec = np.flatnonzero(self._live & (self._len >= self._prompt) &
                             ((self._maxnew < 0) | (self._len - self._orig + 1 < self._maxnew)))
        if decode is not None:
            allowed = np.zeros(self.max_seqs, dtype=bool)
            rows = [self._row_of[sid] for sid in decode if sid in self._row_of]
            allowed[rows] = True
            dec = dec[allowed[dec]]
        if dec.size:
            dec = dec[np.argsort(self._arr[dec], kind="stable")][:budget]
            if int(self._len[dec].max()) + 1 > self.max_seq_len:
                bad = self._id_of[int(dec[np.argmax(self._len[dec])])]
                raise ValueError(f"sequence {bad!r} would exceed max_seq_len {self.max_seq_len}")
            while True:
                need = self._nblk[dec] * BS == self._len[dec]           # the new token opens a block
                n_need = int(need.sum())
                if self.alloc.can_allocate(n_need):
                    break
                # evict from the young end; a decode row itself may go
                protect[:] = False
                protect[dec[:1]] = True
                sid = self._preempt_youngest(protect)
                if sid is None:
                    raise OutOfBlocks("the oldest sequence needs a block and nothing can be preempted")
                preempted.append(sid)
                dec = dec[self._live[dec]]
            if n_need:
                rows = dec[need]
                self._tab[rows, self._nblk[rows]] = self.alloc.allocate(n_need)
                self._nblk[rows] += 1
            budget -= dec.size
        protect[:] = False
        protect[dec] = True

        # 2. prompt chunks: running sequences still inside their prompt (oldest first), then the queue
        chunks: List[tuple] = []            # (row, n)
        pre = np.flatnonzero(self._live & (self._len < self._prompt))
        for r in pre[np.argsort(self._arr[pre], kind="stable")]:
            r = int(r)
            if not self._live[r]:
                continue
            n = min(self.prefill_chunk, int(self._prompt[r] - self._len[r]), budget)
            if n <= 0:
                continue
            protect[r] = True
            ok = self._grow_row(r, n)
            while not ok:
                sid = self._preempt_youngest(protect)
                if sid is None:
                    break
                preempted.append(sid)
                ok = self._grow_row(r, n)
            if not ok:
                protect[r] = False
                continue
            chunks.append((r, n))
            budget -= n
        while self.waiting and budget > 0 and self._free_rows:
            sid, todo, orig, maxnew, arrival = self.waiting[0]
            n = min(self.prefill_chunk, todo, budget)
            if not self.alloc.can_allocate(self.alloc.blocks_for(n)):
                break
            self.waiting.popleft()
            self._waiting_ids.discard(sid)
            r = self._free_rows.pop()
            self._row_of[sid] = r
            self._id_of[r] = sid
            self._live[r] = True
            self._len[r] = 0
            self._nblk[r] = 0
            self._prompt[r], self._orig[r], self._maxnew[r], self._arr[r] = todo, orig, maxnew, arrival
            self._grow_row(r, n)
            chunks.append((r, n))
            budget -= n

        # a sequence preempted after it was given a chunk or a token is gone from this step
        chunks = [(r, n) for r, n in chunks if self._live[r]]
        dec = dec[self._live[dec]] if dec.size else dec
        if not chunks and dec.size == 0:
            return None
        # rows: multi-token sequences first (prefill kernel), one-token sequences after (decode kernel);
        # a last prompt chunk that happens to be one token long is a decode row like any other
        multi = [(r, n) for r, n in chunks if n > 1]
        ones = np.asarray([r for r, n in chunks if n == 1], dtype=np.int64)
        rows = np.concatenate([np.asarray([r for r, _ in multi], dtype=np.int64), dec.astype(np.int64), ones])
        lens = np.concatenate([np.asarray([n for _, n in multi], dtype=np.int32),
                               np.ones(dec.size + ones.size, dtype=np.int32)])
        return self._pack(rows, lens, len(multi), preempted)

    def _pack(self, rows: np.ndarray, new_lens: np.ndarray, npre: int, preempted: List[object]) -> StepPlan:
        S, MB, BS = int(rows.size), self.max_blocks_per_seq, self.block_size
        T = int(new_lens.sum())
        i = self._staging.next()
        raw = self._staging.host[i].numpy()
        off_pos = 8 * T
        off_bt = 16 * T
        off_cl = off_bt + 4 * S * MB
        off_cu = off_cl + 4 * S
        end = off_cu + 4 * (S + 1)
        slot = raw[:off_pos].view(np.int64)
        posn = raw[off_pos:off_bt].view(np.int64)
        bt = raw[off_bt:off_cl].view(np.int32).reshape(S, MB)
        cl = raw[off_cl:off_cu].view(np.int32)
        cu = raw[off_cu:end].view(np.int32)
        np.take(self._tab, rows, axis=0, out=bt)
        cu[0] = 0
        np.cumsum(new_lens, out=cu[1:])
        start = self._len[rows]
        for k in range(npre):                                   # prompt chunks: a few per step
            pos = np.arange(start[k], start[k] + new_lens[k])
            slot[cu[k]:cu[k + 1]] = bt[k, pos // BS].astype(np.int64) * BS + pos % BS
            posn[cu[k]:cu[k + 1]] = pos
        if S > npre:                                            # one-token rows, all at once
            p1 = start[npre:].astype(np.int64)
            slot[cu[npre]:] = bt[np.arange(npre, S), p1 // BS].astype(np.int64) * BS + p1 % BS
            posn[cu[npre]:] = p1
        np.add(start, new_lens, out=cl)
        if self.check_plans:
            probe = StepPlan(seq_ids=[self._id_of[int(r)] for r in rows], num_prefill_seqs=npre, new_lens=new_lens,
                             max_q_len=0, total_new_tokens=T, block_table=None, context_lens=None, cu_q_lens=None,
                             slot_mapping=None, positions=None, preempted=preempted, host_block_table=bt,
                             host_context_lens=cl, host_cu_q_lens=cu, host_slot_mapping=slot, host_positions=posn)
            check_plan(probe, self.alloc.num_blocks, BS)       # raises before anything reaches the device
        self._len[rows] = cl
        self._staging.upload(i, end)
        d32, d64 = self._staging.dev32[i], self._staging.dev64[i]      # (every offset is a multiple of its element size)
        ids = self._id_of
        return StepPlan(
            seq_ids=[ids[r] for r in rows.tolist()], num_prefill_seqs=npre, new_lens=new_lens,
            max_q_len=int(new_lens[:npre].max()) if npre else 0, total_new_tokens=T,
            block_table=d32[off_bt // 4:off_cl // 4].view(S, MB),
            context_lens=d32[off_cl // 4:off_cu // 4],
            cu_q_lens=d32[off_cu // 4:end // 4],
            slot_mapping=d64[:T],
            positions=d64[T:2 * T],
            preempted=preempted,
            host_block_table=bt.copy(), host_context_lens=cl.copy(), host_cu_q_lens=cu.copy(),
            host_slot_mapping=slot.copy(), host_positions=posn.copy(),
        )


def paged_attention_step(plan: StepPlan, out: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                         value: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, scale: float,
                         k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One layer's attention for a planned step: append every new K/V row, then attend.

    ``query`` / ``out`` are ``[T, Hq, D]``, ``key`` / ``value`` ``[T, Hkv, D]`` in the plan's
    row order (``cu_q_lens``).  The prompt chunks go through the chunked-prefill kernel;
    the one-token rows go through the decode kernel with their append fused into it, or, in a
    mixed step whose decode part is small enough (``StepPlan.step_items``), through the same
    launch as the chunks.
    Replaces, per sequence, the append + ``.contiguous()`` + SDPA of
    opt_prime/opt_prime/kv_cache.py:385-415.
    """
    from . import ops
    npre, S = plan.num_prefill_seqs, plan.num_seqs
    t_pre = plan.num_prefill_tokens
    items = plan.step_items(query, k_pool)
    if items is not None:
        # mixed step, decode part within the measured bounds: every new row appended, then one
        # launch over all sequences (a decode row is a chunk of one token)
        ops.kv_append(key, value, k_pool, v_pool, plan.slot_mapping, k_scale, v_scale)
        return ops.paged_prefill_attn(out, query, k_pool, v_pool, plan.block_table, plan.context_lens,
                                      plan.cu_q_lens, scale, max_q_len=plan.max_q_len, k_scale=k_scale,
                                      v_scale=v_scale, items=items)
    if npre:
        ops.kv_append(key[:t_pre], value[:t_pre], k_pool, v_pool, plan.slot_mapping[:t_pre], k_scale, v_scale)
        ops.paged_prefill_attn(out[:t_pre], query[:t_pre], k_pool, v_pool, plan.block_table[:npre],
                               plan.context_lens[:npre], plan.cu_q_lens[:npre + 1], scale,
                               max_q_len=plan.max_q_len, k_scale=k_scale, v_scale=v_scale,
                               items=plan.prefill_items(query, k_pool))
    if S > npre:
        ops.paged_decode_attn(out[t_pre:], query[t_pre:], k_pool, v_pool, plan.block_table[npre:],
                              plan.context_lens[npre:], scale, k_scale, v_scale,
                              new_key=key[t_pre:], new_value=value[t_pre:])
    return out
