"""The decode step under HIP graph capture: the library allocates nothing and clears nothing,
so a captured step replays with new inputs written into the same buffers.

Every replay is checked against the same call made eagerly on a twin pool, with ordinary eager
work and synchronisations between the replays.
"""
import math

import pytest
import torch

from aicomp_amd import ops

pytestmark = pytest.mark.gpu


def _state(device, seed, B=8, hq=8, hkv=2, d=128, max_ctx=300, steps=4, kv_dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    ctx = torch.randint(1, max_ctx, (B,), generator=g)
    width = math.ceil((max_ctx + steps) / 16)
    nb = B * width + 3
    perm = torch.randperm(nb, generator=g)[: B * width].reshape(B, width).to(torch.int32)
    k = (torch.randn(nb, hkv, 16, d, generator=g) * 0.5).to(torch.bfloat16)
    v = (torch.randn(nb, hkv, 16, d, generator=g) * 0.5).to(torch.bfloat16)
    ks = vs = None
    if kv_dtype == torch.float8_e4m3fn:
        ks = torch.full((hkv,), 2.0 / 448, dtype=torch.float32, device=device)
        vs = torch.full((hkv,), 2.0 / 448, dtype=torch.float32, device=device)
        k, v = (k.float() * 224).to(kv_dtype), (v.float() * 224).to(kv_dtype)
    feed = [(torch.randn(B, hq, d, generator=g).to(torch.bfloat16).to(device),
             (torch.randn(B, hkv, d, generator=g) * 0.5).to(torch.bfloat16).to(device),
             (torch.randn(B, hkv, d, generator=g) * 0.5).to(torch.bfloat16).to(device)) for _ in range(steps)]
    return dict(table=perm.to(device), ctx=ctx.to(torch.int32).to(device), k=k.to(device), v=v.to(device),
                ks=ks, vs=vs, feed=feed, B=B, hq=hq, hkv=hkv, d=d, scale=1 / math.sqrt(d))


@pytest.mark.parametrize("kv_dtype", [torch.bfloat16, torch.float8_e4m3fn])
def test_fused_decode_step_replays_under_a_graph(device, kv_dtype):
    s = _state(device, seed=5, kv_dtype=kv_dtype)
    B, hq, hkv, d = s["B"], s["hq"], s["hkv"], s["d"]
    # graph side: static buffers
    k_g, v_g = s["k"].clone(), s["v"].clone()
    q_s = torch.zeros(B, hq, d, dtype=torch.bfloat16, device=device)
    nk_s = torch.zeros(B, hkv, d, dtype=torch.bfloat16, device=device)
    nv_s = torch.zeros_like(nk_s)
    ctx_s = s["ctx"].clone() + 1                       # context including the step's new token
    out_s = torch.zeros_like(q_s)
    need = ops.decode_workspace_bytes(B, hq, hkv, d, 16, s["table"].shape[1], torch.bfloat16, kv_dtype)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=device)

    def step_graph():
        ops.paged_decode_attn(out_s, q_s, k_g, v_g, s["table"], ctx_s, s["scale"], s["ks"], s["vs"],
                              new_key=nk_s, new_value=nv_s, workspace=ws)

    # eager twin
    k_e, v_e = s["k"].clone(), s["v"].clone()
    ctx_e = s["ctx"].clone() + 1

    def step_eager(q, nk, nv):
        out = torch.empty_like(q)
        ops.paged_decode_attn(out, q, k_e, v_e, s["table"], ctx_e, s["scale"], s["ks"], s["vs"],
                              new_key=nk, new_value=nv)
        return out

    # warm-up outside capture (one-time function attributes), on scratch copies of the state
    q0, nk0, nv0 = s["feed"][0]
    q_s.copy_(q0); nk_s.copy_(nk0); nv_s.copy_(nv0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step_graph()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    k_g.copy_(s["k"]); v_g.copy_(s["v"])              # undo the warm-up's append

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step_graph()
    k_g.copy_(s["k"]); v_g.copy_(s["v"])              # capture does not run the kernels, but be explicit

    for i, (q, nk, nv) in enumerate(s["feed"]):
        q_s.copy_(q); nk_s.copy_(nk); nv_s.copy_(nv)
        graph.replay()
        want = step_eager(q, nk, nv)
        torch.cuda.synchronize()
        assert torch.equal(out_s.view(torch.int16), want.view(torch.int16)), f"replay {i}: output differs"
        assert torch.equal(k_g.view(torch.uint8), k_e.view(torch.uint8)), f"replay {i}: K pool differs"
        assert torch.equal(v_g.view(torch.uint8), v_e.view(torch.uint8)), f"replay {i}: V pool differs"
        # eager work between replays: the sequences grow by the token just appended
        ctx_s += 1
        ctx_e += 1
        _ = (out_s.float() @ out_s.float().transpose(1, 2)).sum().item()


@pytest.mark.parametrize("B,d,prompt", [(2, 64, 37), (4, 128, 600)])
def test_adapter_decode_step_replays_from_a_graph(device, decode_routing, B, d, prompt):
    """Two layers of the drop-in operator with device-side positions: one decode step (both layers)
    is captured once and replayed with new inputs; every replay equals the same step made eagerly by
    a twin pair of operators, bit for bit, and the host positions agree after ``advance``.  Runs under
    both routings (with the library's own choice these sizes take the grid schedule) and with eager
    work between the replays."""
    from aicomp_amd import kv_cache as akv
    # A replayed step cannot know its position on the host, so it sizes the split for the whole
    # table; the eager twin sizes it for the context as it is.  On the balanced schedule the tiles
    # are dealt the same way either way (bit-identical results); under the library's own routing
    # the two may take different splits, which agree to the tolerance between split sizes.
    def same(a, b, what=""):
        if decode_routing == "balanced":
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), what
        else:
            assert (a.float() - b.float()).abs().max().item() <= 2e-3, what
    hq, g = 8, 4
    hkv = hq // g
    gen = torch.Generator().manual_seed(3)
    mk = lambda n, h: torch.randn(B, h, n, d, generator=gen).to(torch.bfloat16).to(device)
    expand = lambda t: t.repeat_interleave(g, 1)
    graph_ops = [akv.CachedScaledDotProductAttention(i, 1024, num_kv_groups=g) for i in range(2)]
    eager_ops = [akv.CachedScaledDotProductAttention(i, 1024, num_kv_groups=g) for i in range(2)]
    for op in graph_ops + eager_ops:
        op.enable()
    for i in range(2):                                   # prompt, eagerly, same data for the twins
        q, k, v = mk(prompt, hq), expand(mk(prompt, hkv)), expand(mk(prompt, hkv))
        a = graph_ops[i](q, k, v, is_causal=True)
        b = eager_ops[i](q, k, v, is_causal=True)
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    for op in graph_ops:
        op.use_device_positions()
    q_s = [torch.zeros(B, hq, 1, d, dtype=torch.bfloat16, device=device) for _ in range(2)]
    k_s = [torch.zeros(B, hq, 1, d, dtype=torch.bfloat16, device=device) for _ in range(2)]
    v_s = [torch.zeros(B, hq, 1, d, dtype=torch.bfloat16, device=device) for _ in range(2)]
    out_s = [None, None]

    def step():
        for i in range(2):
            out_s[i] = graph_ops[i](q_s[i], k_s[i], v_s[i])

    # one eager step on the capture stream first (allocates the per-stream scratch), then the capture
    steps = 5
    feed = [[(mk(1, hq), expand(mk(1, hkv)), expand(mk(1, hkv))) for _ in range(2)] for _ in range(steps)]
    want = []
    for t in range(steps):
        want.append([eager_ops[i](*feed[t][i]).clone() for i in range(2)])
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        for i in range(2):
            q_s[i].copy_(feed[0][i][0]); k_s[i].copy_(feed[0][i][1]); v_s[i].copy_(feed[0][i][2])
        step()                                           # eager: this IS step 0
        got0 = [o.clone() for o in out_s]
        side.synchronize()
        pos_before = [op.cache_pos for op in graph_ops]
        with torch.cuda.graph(graph, stream=side):
            step()
        assert [op.cache_pos for op in graph_ops] == pos_before, "a recorded call is not a step"
    torch.cuda.synchronize()
    for i in range(2):
        same(got0[i], want[0][i])
    filler = torch.empty(1 << 24, dtype=torch.uint8, device=device)
    for t in range(1, steps):
        for i in range(2):
            q_s[i].copy_(feed[t][i][0]); k_s[i].copy_(feed[t][i][1]); v_s[i].copy_(feed[t][i][2])
        filler.fill_(t)                                  # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i in range(2):
            same(out_s[i], want[t][i], f"replay {t}, layer {i}")
    for op in graph_ops:
        op.advance(steps - 1)
    assert [op.cache_pos for op in graph_ops] == [op.cache_pos for op in eager_ops] == [prompt + steps] * 2
    # the caches hold the same rows, and an eager step after the replays continues from there
    for i in range(2):
        assert torch.equal(graph_ops[i].cache_k.view(torch.int16), eager_ops[i].cache_k.view(torch.int16))
        q, k, v = mk(1, hq), expand(mk(1, hkv)), expand(mk(1, hkv))
        same(graph_ops[i](q, k, v), eager_ops[i](q, k, v))
