"""Write tests/golden/reference_trace.npz from the reference's own kv_cache.py.

Run ONCE, in the build container only (the reference tree does not travel):
    python tests/golden/make_reference_trace.py /root/reference
It loads opt_prime/opt_prime/kv_cache.py by file path (that file imports only
torch), drives CachedScaledDotProductAttention and KVCacheManager on CPU with
tiny seeded fp32 tensors, and records inputs, outputs and the position
bookkeeping after every call.  The fixture pins what no formula pins: the
state machine (cache_pos / _seq_len across enable, prefill, decode, clear,
disable, manager attach) and the error conditions.
"""
import importlib.util
import json
import os
import sys

import torch


def load(ref_root):
    path = os.path.join(ref_root, "opt_prime", "opt_prime", "kv_cache.py")
    spec = importlib.util.spec_from_file_location("_ref_kv_cache", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


ARRAYS = {}


def t2l(t):
    """Park the tensor in the npz payload, return its key."""
    key = f"a{len(ARRAYS)}"
    ARRAYS[key] = t.detach().to(torch.float32).contiguous().numpy()
    return key


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    ref = load(ref_root)
    g = torch.Generator().manual_seed(1234)
    B, HQ, G, D, MAXSEQ = 2, 4, 2, 64, 16
    HKV = HQ // G

    def qkv(n):
        q = torch.randn(B, HQ, n, D, generator=g)
        k = torch.randn(B, HKV, n, D, generator=g)
        v = torch.randn(B, HKV, n, D, generator=g)
        return q, k, v

    def expand(x):          # HF repeat_kv order: KV head h -> query heads h*G .. h*G+G-1
        return x[:, :, None].expand(B, HKV, G, x.size(2), D).reshape(B, HQ, x.size(2), D)

    trace = {"B": B, "HQ": HQ, "G": G, "D": D, "max_seq_len": MAXSEQ, "sessions": []}

    # ---- session 1: internal cache: disabled pass-through, enable, prefill 5, decode x3, clear, prefill 3, decode, disable
    m = ref.CachedScaledDotProductAttention(layer_idx=0, max_seq_len=MAXSEQ, dtype=torch.float32)
    steps = []

    def call(mod, n, op="forward", **kw):
        q, k, v = qkv(n)
        out = mod(q, expand(k), expand(v), attn_mask=torch.zeros(n, n), dropout_p=0.0, is_causal=False, **kw)
        steps.append({"op": op, "n": n, "q": t2l(q), "k": t2l(k), "v": t2l(v), "out": t2l(out),
                      "cache_pos": mod.cache_pos, "enabled": mod._enabled, "kwargs": kw})

    call(m, 3, op="forward_disabled")
    m.enable(); steps.append({"op": "enable", "cache_pos": m.cache_pos, "enabled": m._enabled})
    call(m, 5)
    call(m, 1); call(m, 1); call(m, 1, scale=0.5)
    m.clear(); steps.append({"op": "clear", "cache_pos": m.cache_pos, "enabled": m._enabled})
    call(m, 3); call(m, 1)
    m.disable(); steps.append({"op": "disable", "cache_pos": m.cache_pos, "enabled": m._enabled,
                               "cache_is_none": m.cache_k is None})
    trace["sessions"].append({"mode": "internal", "steps": steps})

    # ---- session 2: external KVCacheManager, two layers sharing one manager
    steps = []
    mgr = ref.KVCacheManager(num_layers=4, max_batch_size=B, max_seq_len=MAXSEQ, num_heads=HQ, head_dim=D,
                             dtype=torch.float32, device=torch.device("cpu"), layer_start=1, layer_end=3)
    errors = []
    for what, fn in (("allocate_overbatch", lambda: mgr.allocate(B + 1)),
                     ("allocate_overlen", lambda: mgr.allocate(B, MAXSEQ + 1))):
        try:
            fn(); errors.append([what, None])
        except Exception as e:
            errors.append([what, type(e).__name__])
    mgr.allocate(B)
    steps.append({"op": "allocate", "seq_len": mgr.get_seq_len(), "is_allocated": mgr.is_allocated,
                  "batch_size": mgr.batch_size, "memory": mgr.get_memory_usage(),
                  "get_layer1_is_none": mgr.get(1) is None, "get_layer0_is_none": mgr.get(0) is None})
    for what, fn in (("update_unknown_layer", lambda: mgr.update(0, torch.zeros(B, HQ, 1, D), torch.zeros(B, HQ, 1, D))),
                     ("update_overflow", lambda: mgr.update(1, torch.zeros(B, HQ, MAXSEQ + 1, D), torch.zeros(B, HQ, MAXSEQ + 1, D)))):
        try:
            fn(); errors.append([what, None])
        except Exception as e:
            errors.append([what, type(e).__name__])
    mods = [ref.CachedScaledDotProductAttention(layer_idx=i, max_seq_len=MAXSEQ, dtype=torch.float32) for i in (1, 2)]
    for mm in mods:
        mm.set_kv_manager(mgr); mm.enable()

    def call2(n):
        for mm in mods:
            q, k, v = qkv(n)
            out = mm(q, expand(k), expand(v), attn_mask=None, dropout_p=0.0, is_causal=True)
            steps.append({"op": "forward", "layer": mm.layer_idx, "n": n, "q": t2l(q), "k": t2l(k), "v": t2l(v),
                          "out": t2l(out), "cache_pos": mm.cache_pos, "mgr_seq_len": mgr.get_seq_len()})

    call2(4); call2(1); call2(1)
    kv = mgr.get(2)
    steps.append({"op": "get", "layer": 2, "k_shape": list(kv[0].shape), "k": t2l(kv[0]), "v": t2l(kv[1])})
    mgr.set_seq_len(3); steps.append({"op": "set_seq_len", "value": 3, "mgr_seq_len": mgr.get_seq_len(),
                                      "get_shape": list(mgr.get(1)[0].shape)})
    for mm in mods:
        mm.clear()
    mgr.clear()
    steps.append({"op": "clear_all", "cache_pos": [mm.cache_pos for mm in mods], "mgr_seq_len": mgr.get_seq_len(),
                  "get_is_none": mgr.get(1) is None})
    call2(2); call2(1)
    for mm in mods:
        mm.disable()
    mgr.free()
    steps.append({"op": "free", "is_allocated": mgr.is_allocated, "batch_size": mgr.batch_size,
                  "memory": mgr.get_memory_usage(), "mgr_seq_len": mgr.get_seq_len()})
    trace["sessions"].append({"mode": "external", "layer_start": 1, "layer_end": 3, "num_layers": 4,
                              "errors": errors, "steps": steps})

    import numpy as np
    out_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_trace.npz")
    np.savez_compressed(out_path, meta=np.array(json.dumps(trace)), **ARRAYS)
    print("wrote", out_path, os.path.getsize(out_path), "bytes,", len(ARRAYS), "arrays")


if __name__ == "__main__":
    main()
