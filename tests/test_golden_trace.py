"""The oracle's restatement of the reference operator against the trace recorded from the
reference's own kv_cache.py (CPU, no GPU needed)."""
import torch

from oracle import contiguous_ref as cref
from trace_replay import load_trace, replay


def test_oracle_restatement_matches_reference_trace():
    meta, z = load_trace()

    def attach(op, mgr):
        op.store = mgr

    replay(meta, z,
           make_op=lambda layer, max_seq: cref.ContiguousCachedAttention(layer, max_seq),
           make_mgr=lambda **kw: cref.ContiguousStore(**kw),
           device="cpu", atol=1e-6, attach=attach)


def test_trace_covers_the_state_machine():
    meta, _ = load_trace()
    ops = [s["op"] for s in meta["sessions"][0]["steps"]]
    assert ops == ["forward_disabled", "enable", "forward", "forward", "forward", "forward", "clear",
                   "forward", "forward", "disable"]
    pos = [s["cache_pos"] for s in meta["sessions"][0]["steps"]]
    assert pos == [0, 0, 5, 6, 7, 8, 0, 3, 4, 0]
    assert dict(meta["sessions"][1]["errors"]) == {
        "allocate_overbatch": "ValueError", "allocate_overlen": "ValueError",
        "update_unknown_layer": "ValueError", "update_overflow": "ValueError"}
