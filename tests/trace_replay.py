"""Replay of tests/golden/reference_trace.npz (recorded from the reference's kv_cache.py by
tests/golden/make_reference_trace.py) against any implementation of the two classes."""
import json
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def load_trace():
    z = np.load(os.path.join(HERE, "golden", "reference_trace.npz"), allow_pickle=False)
    meta = json.loads(str(z["meta"]))
    return meta, z


def replay(meta, z, make_op, make_mgr, device, atol, attach, dtype=torch.float32):
    """make_op(layer_idx, max_seq_len) -> operator; make_mgr(**kw) -> manager;
    attach(op, mgr) attaches.  Asserts outputs and bookkeeping after every step."""
    B, HQ, G, D = meta["B"], meta["HQ"], meta["G"], meta["D"]
    HKV = HQ // G

    def T(key):
        return torch.from_numpy(z[key]).to(device=device, dtype=dtype)

    def expand(x):
        n = x.size(2)
        return x[:, :, None].expand(B, HKV, G, n, D).reshape(B, HQ, n, D)

    def check_out(got, key, what):
        want = torch.from_numpy(z[key]).double()
        err = (got.detach().double().cpu() - want).abs().max().item()
        assert err <= atol, f"{what}: max abs err {err:.3e} > {atol}"

    def pos_of(op):
        return op.cache_pos if hasattr(op, "cache_pos") else op.pos

    def enabled_of(op):
        return op._enabled if hasattr(op, "_enabled") else op.enabled

    # ---- session 1: internal cache
    ses = meta["sessions"][0]
    op = make_op(0, meta["max_seq_len"])
    for i, st in enumerate(ses["steps"]):
        what = f"internal step {i} ({st['op']})"
        if st["op"] in ("forward", "forward_disabled"):
            q, k, v = T(st["q"]), T(st["k"]), T(st["v"])
            n = st["n"]
            out = op(q, expand(k), expand(v), attn_mask=torch.zeros(n, n, device=device, dtype=dtype),
                     dropout_p=0.0, is_causal=False, **st["kwargs"])
            assert tuple(out.shape) == (B, HQ, n, D), what
            check_out(out, st["out"], what)
        elif st["op"] == "enable":
            op.enable()
        elif st["op"] == "clear":
            op.clear()
        elif st["op"] == "disable":
            op.disable()
        assert pos_of(op) == st["cache_pos"], what
        assert enabled_of(op) == st["enabled"], what

    # ---- session 2: external manager shared by two layers
    ses = meta["sessions"][1]
    mgr = make_mgr(num_layers=ses["num_layers"], max_batch_size=B, max_seq_len=meta["max_seq_len"],
                   num_heads=HQ, head_dim=D, dtype=dtype, device=torch.device(device),
                   layer_start=ses["layer_start"], layer_end=ses["layer_end"])
    zeros = lambda n: torch.zeros(B, HQ, n, D, device=device, dtype=dtype)
    probes = {
        "allocate_overbatch": lambda: mgr.allocate(B + 1),
        "allocate_overlen": lambda: mgr.allocate(B, meta["max_seq_len"] + 1),
        "update_unknown_layer": lambda: mgr.update(0, zeros(1), zeros(1)),
        "update_overflow": lambda: mgr.update(1, zeros(meta["max_seq_len"] + 1), zeros(meta["max_seq_len"] + 1)),
    }

    def probe(name, expected):
        try:
            probes[name]()
            got = None
        except Exception as e:           # noqa: BLE001 - the kind of error is what is compared
            got = type(e).__name__
        assert got == expected, f"{name}: raised {got}, the reference raises {expected}"

    errs = dict(ses["errors"])
    probe("allocate_overbatch", errs["allocate_overbatch"])
    probe("allocate_overlen", errs["allocate_overlen"])
    ops_ = {}
    for i, st in enumerate(ses["steps"]):
        what = f"external step {i} ({st['op']})"
        if st["op"] == "allocate":
            mgr.allocate(B)
            seq_len = mgr.get_seq_len() if hasattr(mgr, "get_seq_len") else mgr.seq_len
            assert seq_len == st["seq_len"], what
            if hasattr(mgr, "is_allocated"):
                assert mgr.is_allocated == st["is_allocated"] and mgr.batch_size == st["batch_size"], what
                assert (mgr.get(1) is None) == st["get_layer1_is_none"], what
                assert (mgr.get(0) is None) == st["get_layer0_is_none"], what
            probe("update_unknown_layer", errs["update_unknown_layer"])
            probe("update_overflow", errs["update_overflow"])
            for layer in (1, 2):
                ops_[layer] = make_op(layer, meta["max_seq_len"])
                attach(ops_[layer], mgr)
                ops_[layer].enable()
        elif st["op"] == "forward":
            o = ops_[st["layer"]]
            q, k, v = T(st["q"]), T(st["k"]), T(st["v"])
            out = o(q, expand(k), expand(v), attn_mask=None, dropout_p=0.0, is_causal=True)
            check_out(out, st["out"], what)
            assert pos_of(o) == st["cache_pos"], what
            seq_len = mgr.get_seq_len() if hasattr(mgr, "get_seq_len") else mgr.seq_len
            assert seq_len == st["mgr_seq_len"], what
        elif st["op"] == "get" and hasattr(mgr, "get"):
            kk, vv = mgr.get(st["layer"])
            assert list(kk.shape) == st["k_shape"], what
            check_out(kk.contiguous(), st["k"], what + " K")
            check_out(vv.contiguous(), st["v"], what + " V")
        elif st["op"] == "set_seq_len" and hasattr(mgr, "set_seq_len"):
            mgr.set_seq_len(st["value"])
            assert mgr.get_seq_len() == st["mgr_seq_len"], what
            assert list(mgr.get(1)[0].shape) == st["get_shape"], what
        elif st["op"] == "clear_all":
            for o in ops_.values():
                o.clear()
            mgr.clear()
            assert [pos_of(ops_[1]), pos_of(ops_[2])] == st["cache_pos"], what
            if hasattr(mgr, "get"):
                assert (mgr.get(1) is None) == st["get_is_none"], what
        elif st["op"] == "free" and hasattr(mgr, "free"):
            for o in ops_.values():
                o.disable()
            mgr.free()
            assert mgr.is_allocated == st["is_allocated"] and mgr.batch_size == st["batch_size"], what
            assert mgr.get_memory_usage() == st["memory"] and mgr.get_seq_len() == st["mgr_seq_len"], what
