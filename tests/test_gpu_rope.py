"""Fused rotary embedding + KV append through the C ABI vs the oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from aicomp_amd import ops
from oracle import rope_oracle as R
from helpers import NAME, raw

pytestmark = pytest.mark.gpu


def make_case(device, T, hq, hkv, d, dtype, nb=None, seed=0, table_rows=512, fused_qkv=False):
    g = torch.Generator().manual_seed(seed)
    nb = nb or (T + 15) // 16 + 3
    if fused_qkv:      # one projection output [T, (Hq + 2 Hkv) * D]; q, k, v are column slices of it
        qkv = torch.randn(T, (hq + 2 * hkv) * d, generator=g).to(dtype).to(device)
        q = qkv[:, :hq * d].view(T, hq, d)
        k = qkv[:, hq * d:(hq + hkv) * d].view(T, hkv, d)
        v = qkv[:, (hq + hkv) * d:].view(T, hkv, d)
    else:
        q = torch.randn(T, hq, d, generator=g).to(dtype).to(device)
        k = (torch.randn(T, hkv, d, generator=g) * 2).to(dtype).to(device)
        v = torch.randn(T, hkv, d, generator=g).to(dtype).to(device)
    inv = torch.from_numpy(R.default_inv_freq(d, 500000.0))
    cos, sin = ops.rotary_tables(inv, table_rows, dtype, device=device)
    pos = torch.randint(0, table_rows, (T,), generator=g, dtype=torch.int64).to(device)
    slots = torch.randperm(nb * 16, generator=g)[:T].to(torch.int64).to(device)
    return dict(q=q, k=k, v=v, cos=cos, sin=sin, pos=pos, slots=slots, nb=nb)


def sentinel_pools(c, hkv, d, dtype, device):
    kp = torch.full((c["nb"], hkv, 16, d), -7.0, dtype=torch.float32, device=device).to(dtype)
    return kp, kp.clone()


def run_oracle(c, kp, vp, dtype, positions="given", ks=None, vs=None, pool_dtype=None):
    name = NAME[dtype]
    kpo, vpo = raw(kp).copy(), raw(vp).copy()
    pos = None if positions is None else c["pos"].cpu().numpy()
    q_out = R.rope_kv_append(raw(c["q"]), raw(c["k"]), raw(c["v"]), raw(c["cos"]), raw(c["sin"]), pos, kpo, vpo,
                             c["slots"].cpu().numpy(), name,
                             None if ks is None else ks.cpu().numpy(), None if vs is None else vs.cpu().numpy(),
                             pool_dtype=pool_dtype)
    return q_out, kpo, vpo


@pytest.mark.parametrize("dtype,hq,hkv,d", [(torch.bfloat16, 8, 2, 128), (torch.float32, 4, 4, 64),
                                            (torch.bfloat16, 3, 1, 256), (torch.float32, 2, 1, 16)])
def test_rope_append_bit_exact(device, dtype, hq, hkv, d):
    c = make_case(device, 37, hq, hkv, d, dtype)
    kp, vp = sentinel_pools(c, hkv, d, dtype, device)
    want_q, want_k, want_v = run_oracle(c, kp, vp, dtype)
    q_in = c["q"].clone()
    out = ops.rope_kv_append(c["q"], c["k"], c["v"], c["cos"], c["sin"], c["pos"], kp, vp, c["slots"])
    torch.cuda.synchronize()
    assert out.data_ptr() == c["q"].data_ptr()                     # in place by default
    assert np.array_equal(raw(out), want_q)
    assert np.array_equal(raw(kp), want_k) and np.array_equal(raw(vp), want_v)   # untouched slots included
    # out of place gives the same bits and leaves the input alone
    kp2, vp2 = sentinel_pools(c, hkv, d, dtype, device)
    q2 = q_in.clone()
    dst = torch.empty_like(q2)
    ops.rope_kv_append(q2, c["k"], c["v"], c["cos"], c["sin"], c["pos"], kp2, vp2, c["slots"], query_out=dst)
    torch.cuda.synchronize()
    assert torch.equal(q2, q_in) and np.array_equal(raw(dst), want_q) and torch.equal(kp2, kp)


def test_rope_append_matches_eager_reference_expression(device):
    """The same expression the reference evaluates (modeling_llama.py:200-231), run by torch's own
    GPU kernels in bf16, followed by repeat_kv-free append: bit-identical at a prefill-sized T."""
    T, hq, hkv, d = 2108, 32, 8, 128
    c = make_case(device, T, hq, hkv, d, torch.bfloat16, table_rows=4096, seed=1)
    kp, vp = sentinel_pools(c, hkv, d, torch.bfloat16, device)
    cos, sin = c["cos"][c["pos"]][:, None, :], c["sin"][c["pos"]][:, None, :]
    half = lambda x: torch.cat((-x[..., d // 2:], x[..., :d // 2]), dim=-1)
    q_ref = (c["q"] * cos) + (half(c["q"]) * sin)
    k_ref = (c["k"] * cos) + (half(c["k"]) * sin)
    kp_ref, vp_ref = kp.clone(), vp.clone()
    ops.kv_append(k_ref, c["v"], kp_ref, vp_ref, c["slots"])
    out = ops.rope_kv_append(c["q"], c["k"], c["v"], c["cos"], c["sin"], c["pos"], kp, vp, c["slots"])
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), q_ref.view(torch.int16))
    assert torch.equal(kp.view(torch.int16), kp_ref.view(torch.int16))
    assert torch.equal(vp.view(torch.int16), vp_ref.view(torch.int16))


def test_rope_append_fused_qkv_views_and_row_tables(device):
    # inputs are column slices of one [T, (Hq+2Hkv)*D] buffer; cos/sin given per token (positions None)
    T, hq, hkv, d = 64, 32, 8, 128
    c = make_case(device, T, hq, hkv, d, torch.bfloat16, fused_qkv=True, table_rows=T)
    assert not c["q"].is_contiguous()
    kp, vp = sentinel_pools(c, hkv, d, torch.bfloat16, device)
    want_q, want_k, want_v = run_oracle(c, kp, vp, torch.bfloat16, positions=None)
    dst = torch.empty(T, hq, d, dtype=torch.bfloat16, device=device)
    ops.rope_kv_append(c["q"], c["k"], c["v"], c["cos"], c["sin"], None, kp, vp, c["slots"], query_out=dst)
    torch.cuda.synchronize()
    assert np.array_equal(raw(dst), want_q) and np.array_equal(raw(kp), want_k) and np.array_equal(raw(vp), want_v)


def test_rope_append_padding_and_missing_positions(device):
    T, hq, hkv, d = 23, 4, 2, 64
    c = make_case(device, T, hq, hkv, d, torch.bfloat16, table_rows=100)
    c["slots"][4] = -1                       # padding row: Q rotated, K/V not stored
    c["slots"][9] = c["nb"] * 16             # beyond the pool: treated the same
    c["pos"][7] = 100                        # no table row: token left alone
    c["pos"][8] = -3
    kp, vp = sentinel_pools(c, hkv, d, torch.bfloat16, device)
    oc = dict(c)
    oc["slots"] = c["slots"].clone()
    oc["slots"][9] = -1
    want_q, want_k, want_v = run_oracle(oc, kp, vp, torch.bfloat16)
    out = ops.rope_kv_append(c["q"], c["k"], c["v"], c["cos"], c["sin"], c["pos"], kp, vp, c["slots"])
    torch.cuda.synchronize()
    assert np.array_equal(raw(out), want_q) and np.array_equal(raw(kp), want_k) and np.array_equal(raw(vp), want_v)


def test_rope_append_fp8_pool_equals_rotate_then_quantising_append(device):
    T, hq, hkv, d = 50, 16, 2, 128
    c = make_case(device, T, hq, hkv, d, torch.bfloat16)
    ks = torch.tensor([9.0 / 448, 7.5 / 448], dtype=torch.float32, device=device)
    vs = torch.tensor([4.0 / 448, 5.0 / 448], dtype=torch.float32, device=device)
    kp = torch.zeros(c["nb"], hkv, 16, d, dtype=torch.uint8, device=device).view(torch.float8_e4m3fn)
    vp = kp.clone()
    want_q, want_k, want_v = run_oracle(c, kp, vp, torch.bfloat16, ks=ks, vs=vs, pool_dtype="fp8")
    out = ops.rope_kv_append(c["q"], c["k"], c["v"], c["cos"], c["sin"], c["pos"], kp, vp, c["slots"], ks, vs)
    torch.cuda.synchronize()
    assert np.array_equal(raw(out), want_q) and np.array_equal(raw(kp), want_k) and np.array_equal(raw(vp), want_v)


def test_rope_append_rejects_bad_arguments(device):
    c = make_case(device, 8, 4, 2, 64, torch.bfloat16)
    kp, vp = sentinel_pools(c, 2, 64, torch.bfloat16, device)
    with pytest.raises(RuntimeError):
        ops.rope_kv_append(c["q"], c["k"], c["v"], c["cos"].float(), c["sin"].float(), c["pos"], kp, vp, c["slots"])
    with pytest.raises(RuntimeError):
        ops.rope_kv_append(c["q"], c["k"], c["v"], c["cos"], c["sin"], c["pos"].int(), kp, vp, c["slots"])
    with pytest.raises(RuntimeError):
        ops.rope_kv_append(c["q"], c["k"], c["v"], c["cos"][:4], c["sin"][:4], None, kp, vp, c["slots"])
    with pytest.raises(RuntimeError):
        ops.rope_kv_append(c["q"], c["k"][:, :1], c["v"][:, :1], c["cos"], c["sin"], c["pos"], kp, vp, c["slots"])
    with pytest.raises(RuntimeError):
        ops.rope_kv_append(c["q"].cpu(), c["k"], c["v"], c["cos"], c["sin"], c["pos"], kp, vp, c["slots"])
    # head_dim not a multiple of 16 is refused by the library
    q = torch.zeros(2, 1, 24, dtype=torch.bfloat16, device=device)
    p24 = torch.zeros(2, 1, 16, 24, dtype=torch.bfloat16, device=device)
    t24 = torch.zeros(4, 24, dtype=torch.bfloat16, device=device)
    with pytest.raises(RuntimeError):
        ops.rope_kv_append(q, q.clone(), q.clone(), t24, t24, None, p24, p24.clone(),
                           torch.arange(2, device=device))


def test_rope_then_attention_scores_depend_on_distance_only(device):
    """Property at full pipeline level: rotate with positions p and p + 1000, append, decode; the outputs
    agree to bf16 accuracy because rotary scores depend on relative position only."""
    import math
    B, hq, hkv, d, L = 4, 8, 2, 128, 200
    g = torch.Generator().manual_seed(5)
    inv = torch.from_numpy(R.default_inv_freq(d))
    cos, sin = ops.rotary_tables(inv, 2048, torch.bfloat16, device=device)
    k_all = (torch.randn(B * L, hkv, d, generator=g) * 0.5).to(torch.bfloat16).to(device)
    v_all = (torch.randn(B * L, hkv, d, generator=g) * 0.5).to(torch.bfloat16).to(device)
    q_all = torch.randn(B * L, hq, d, generator=g).to(torch.bfloat16).to(device)
    nb = B * ((L + 15) // 16)
    table = torch.arange(nb, dtype=torch.int32, device=device).view(B, -1)
    tok = torch.arange(L, device=device)
    slots = (table[:, tok // 16].long() * 16 + tok % 16).reshape(-1)
    outs = []
    for shift in (0, 1000):
        kp = torch.zeros(nb, hkv, 16, d, dtype=torch.bfloat16, device=device)
        vp = torch.zeros_like(kp)
        pos = (tok + shift).repeat(B)
        qr = torch.empty_like(q_all)
        ops.rope_kv_append(q_all, k_all, v_all, cos, sin, pos, kp, vp, slots, query_out=qr)
        q_last = qr.view(B, L, hq, d)[:, -1].contiguous()
        out = torch.empty_like(q_last)
        ops.paged_decode_attn(out, q_last, kp, vp, table, torch.full((B,), L, dtype=torch.int32, device=device),
                              1 / math.sqrt(d))
        outs.append(out.float())
    torch.cuda.synchronize()
    assert (outs[0] - outs[1]).abs().max().item() < 3e-2
    assert outs[0].abs().max().item() > 0.05
