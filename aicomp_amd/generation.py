"""Generation driver over the paged path: the caller of the attention operator.

Mirrors ``ScheduleGeneration`` of the reference
(opt_prime/opt_prime/schedule_infer.py:341-449): ``prefill`` runs the prompt and
returns the logits of the last position, ``decode_step`` runs one token per
sequence, ``clear_cache`` resets.  Differences, all on purpose:

* every sequence has its own length and position (the reference shares one scalar
  position, ``schedule_infer.py:425-430``), so prompts of different lengths and
  continuous batching work;
* the next-step input may be ``[B]`` or ``[B, 1]``: it is flattened to one token per
  sequence.  The reference's loop builds it with ``next_token.unsqueeze(0)``
  (opt_prime/opt_prime/inference.py:1041-1043), i.e. ``[1, B]``, which only has the
  right shape for batch 1;
* the model is called token-major: ``model(input_ids [T], positions [T]) ->
  logits [T, V]``, its attention layers calling ``PagedAttentionBackend.attend``.

``PagedAttentionBackend`` owns one K and one V pool per layer and runs, per layer and
step, the rotary embedding fused with the append followed by the chunked-prefill
kernel on the prompt-chunk rows and the decode kernel on the one-token rows.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional, Sequence

import torch

from . import ops
from .block_manager import StepPlan, StepPlanner


class PagedAttentionBackend:
    """Per-layer paged K/V pools plus the per-step attention call of a decoder layer.

    ``inv_freq`` (the rotary module's buffer, compiler_fx/modeling_llama.py:130-132) switches
    the rotary embedding on: ``attend`` then takes Q/K as projected and rotates them itself.
    Without it Q/K must arrive rotated.
    """

    def __init__(self, num_layers: int, num_blocks: int, num_kv_heads: int, head_dim: int,
                 dtype: torch.dtype = torch.bfloat16, device="cuda", kv_dtype: Optional[torch.dtype] = None,
                 inv_freq: Optional[torch.Tensor] = None, max_positions: int = 8192,
                 attention_scaling: float = 1.0, scale: Optional[float] = None, block_size: int = 16) -> None:
        self.device = torch.device(device)
        self.dtype = dtype
        kv_dtype = kv_dtype or dtype
        shape = (num_blocks, num_kv_heads, block_size, head_dim)
        self.k_pools = [torch.zeros(shape, dtype=kv_dtype, device=self.device) for _ in range(num_layers)]
        self.v_pools = [torch.zeros(shape, dtype=kv_dtype, device=self.device) for _ in range(num_layers)]
        self.k_scales: List[Optional[torch.Tensor]] = [None] * num_layers
        self.v_scales: List[Optional[torch.Tensor]] = [None] * num_layers
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else scale
        self.cos = self.sin = None
        if inv_freq is not None:
            self.cos, self.sin = ops.rotary_tables(inv_freq, max_positions, dtype, attention_scaling, self.device)
        self.plan: Optional[StepPlan] = None

    def set_scales(self, layer_idx: int, k_scale: torch.Tensor, v_scale: torch.Tensor) -> None:
        """Per-KV-head dequantisation scales of an fp8 pool."""
        self.k_scales[layer_idx] = k_scale.to(self.device, torch.float32).contiguous()
        self.v_scales[layer_idx] = v_scale.to(self.device, torch.float32).contiguous()

    def begin_step(self, plan: StepPlan) -> None:
        self.plan = plan

    def attend(self, layer_idx: int, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
        """``query [T, Hq, D]``, ``key`` / ``value [T, Hkv, D]`` in the plan's row order -> ``[T, Hq, D]``."""
        plan = self.plan
        if plan is None:
            raise RuntimeError("PagedAttentionBackend.attend called outside a step (begin_step first)")
        kp, vp = self.k_pools[layer_idx], self.v_pools[layer_idx]
        ks, vs = self.k_scales[layer_idx], self.v_scales[layer_idx]
        out = torch.empty(query.shape, dtype=query.dtype, device=query.device)
        if self.cos is None:
            from .block_manager import paged_attention_step
            return paged_attention_step(plan, out, query.contiguous(), key, value, kp, vp, self.scale, ks, vs)
        q = torch.empty(query.shape, dtype=query.dtype, device=query.device)
        ops.rope_kv_append(query, key, value, self.cos, self.sin, plan.positions, kp, vp, plan.slot_mapping,
                           ks, vs, query_out=q)
        npre, S, t_pre = plan.num_prefill_seqs, plan.num_seqs, plan.num_prefill_tokens
        items = plan.step_items(q, kp)
        if items is not None:                      # mixed step: chunks and decode rows in one launch
            return ops.paged_prefill_attn(out, q, kp, vp, plan.block_table, plan.context_lens, plan.cu_q_lens,
                                          self.scale, max_q_len=plan.max_q_len, k_scale=ks, v_scale=vs, items=items)
        if npre:
            ops.paged_prefill_attn(out[:t_pre], q[:t_pre], kp, vp, plan.block_table[:npre], plan.context_lens[:npre],
                                   plan.cu_q_lens[:npre + 1], self.scale, max_q_len=plan.max_q_len,
                                   k_scale=ks, v_scale=vs, items=plan.prefill_items(q, kp))
        if S > npre:
            ops.paged_decode_attn(out[t_pre:], q[t_pre:], kp, vp, plan.block_table[npre:], plan.context_lens[npre:],
                                  self.scale, ks, vs)
        return out


class ScheduleGeneration:
    """``prefill`` / ``decode_step`` / ``clear_cache`` over a token-major model and a planner."""

    def __init__(self, model: Callable[[torch.Tensor, torch.Tensor], torch.Tensor],
                 backend: PagedAttentionBackend, planner: StepPlanner) -> None:
        # a token whose position has no row in the rotary tables would be left unrotated and
        # unstored by the fused rotary + append launch: refuse the combination up front
        cos = getattr(backend, "cos", None)
        if cos is not None and planner.max_seq_len > cos.shape[0]:
            raise ValueError(f"the planner admits sequences of {planner.max_seq_len} tokens but the backend's "
                             f"rotary tables hold {cos.shape[0]} positions (max_positions)")
        self.model = model
        self.backend = backend
        self.planner = planner
        self._batch: List[object] = []
        self._offset: Dict[object, int] = {}

    # one planner step: returns {seq_id: logits row of its last new token}
    @torch.no_grad()
    def _step(self, tokens_of: Dict[object, torch.Tensor], decode=None) -> Dict[object, torch.Tensor]:
        plan = self.planner.schedule(decode)
        if plan is None:
            return {}
        if plan.preempted:
            raise RuntimeError(f"pool too small for this batch: sequences {plan.preempted} were preempted")
        cu = plan.host_cu_q_lens
        pieces = []
        for r, sid in enumerate(plan.seq_ids):
            n = int(plan.new_lens[r])
            start = int(plan.host_positions[cu[r]]) - self._offset.get(sid, 0)
            pieces.append(tokens_of[sid][start:start + n])
        ids = torch.cat(pieces).to(self.backend.device)
        self.backend.begin_step(plan)
        logits = self.model(ids, plan.positions)
        last = torch.as_tensor(cu[1:] - 1, dtype=torch.int64, device=logits.device)
        rows = logits.index_select(0, last)
        return {sid: rows[r] for r, sid in enumerate(plan.seq_ids)}

    @torch.no_grad()
    def prefill(self, input_ids: torch.Tensor, position_ids: Optional[torch.Tensor] = None,
                prompt_lens: Optional[Sequence[int]] = None) -> torch.Tensor:
        """Ingest the prompts ``input_ids [B, S]`` (right-padded when ``prompt_lens`` gives shorter
        lengths) and return the logits after each prompt's last token, ``[B, V]``
        (schedule_infer.py:363-407).  ``position_ids`` is accepted for signature compatibility;
        positions always run from 0 per sequence."""
        if input_ids.dim() == 1:
            input_ids = input_ids[None, :]
        B, S = input_ids.shape
        lens = [S] * B if prompt_lens is None else [int(n) for n in prompt_lens]
        self.clear_cache()
        self._offset = {}
        toks = {}
        for b in range(B):
            self.planner.add_request(b, lens[b])
            toks[b] = input_ids[b, :lens[b]]
        self._batch = list(range(B))
        final: Dict[object, torch.Tensor] = {}
        while len(final) < B:
            got = self._step(toks, decode=())      # nobody decodes until every prompt is in
            if not got:
                raise RuntimeError("planner made no progress during prefill")
            for sid, row in got.items():
                if self.planner.context_len(sid) == lens[sid]:
                    final[sid] = row
        return torch.stack([final[b] for b in range(B)])

    @torch.no_grad()
    def decode_step(self, input_token: torch.Tensor, position=None) -> torch.Tensor:
        """One token per sequence: ``input_token`` ``[B]``, ``[B, 1]`` (or the reference's ``[1, B]``),
        returns logits ``[B, V]`` (schedule_infer.py:409-449).  ``position`` is checked against each
        sequence's own length when given (an int, or one value per sequence)."""
        tok = input_token.reshape(-1)
        B = len(self._batch)
        if tok.numel() != B:
            raise ValueError(f"decode_step needs one token per sequence: got {tok.numel()} for batch {B}")
        if position is not None:
            want = [int(position)] * B if not hasattr(position, "__len__") else [int(p) for p in position]
            have = [self.planner.context_len(b) for b in self._batch]
            if want != have:
                raise ValueError(f"position {want} does not match the cached lengths {have}")
        toks = {}
        for i, b in enumerate(self._batch):
            self._offset[b] = self.planner.context_len(b)
            toks[b] = tok[i:i + 1]
        got = self._step(toks)
        if len(got) != B:
            raise RuntimeError("not every sequence could be scheduled in this decode step")
        return torch.stack([got[b] for b in self._batch])

    def clear_cache(self) -> None:
        """Release every sequence of the current batch (schedule_infer.py:451-454)."""
        for b in self._batch:
            try:
                self.planner.finish(b)
            except ValueError:
                pass
        self._batch = []
