"""Pin the CPU oracle: number formats against torch's casts, the attention
formula against brute force, closed forms and torch's CPU SDPA (an independent
library routine), the paged layout against the contiguous one.  No GPU."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import contiguous_ref as cref
from oracle import paged_kv_oracle as orc
from helpers import raw


# ----------------------------------------------------------------- formats --

def test_bf16_decode_all_codes_match_torch():
    codes = np.arange(65536, dtype=np.uint16)
    want = torch.from_numpy(codes.view(np.int16)).view(torch.bfloat16).float().numpy()
    got = orc.bf16_bits_to_f32(codes)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_bf16_encode_rne_matches_torch():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(200000, generator=g) * 10
    # exact ties and boundaries
    ties = torch.tensor([1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, -1.0 - 2 ** -8, 3.3895314e38, 0.0, -0.0,
                         float("inf"), -float("inf"), 1e-40])
    x = torch.cat([x, ties])
    want = raw(x.to(torch.bfloat16))
    got = orc.f32_to_bf16_bits(x.numpy())
    assert np.array_equal(got, want)


def test_f16_decode_all_codes_match_torch():
    codes = np.arange(65536, dtype=np.uint16)
    want = torch.from_numpy(codes.view(np.int16)).view(torch.float16).float().numpy()
    got = orc.f16_bits_to_f32(codes)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.array_equal(np.isnan(got), np.isnan(want))


def test_f16_encode_rne_matches_torch():
    g = torch.Generator().manual_seed(2)
    x = torch.cat([torch.randn(200000, generator=g) * 10, torch.randn(50000, generator=g) * 1e-6,
                   torch.randn(20000, generator=g) * 3e4])
    # ties (even and odd neighbours), the overflow threshold, the subnormal range, signed zeros
    ties = torch.tensor([1.0 + 2 ** -11, 1.0 + 3 * 2 ** -11, -1.0 - 2 ** -11, 65504.0, 65519.99, 65520.0, 7e4,
                         2 ** -24, 2 ** -25, 1.5 * 2 ** -25, 3 * 2 ** -25, 6.0e-5, 6.1e-5, 0.0, -0.0,
                         float("inf"), -float("inf"), 1e-10])
    x = torch.cat([x, ties])
    want = raw(x.to(torch.float16))
    got = orc.f32_to_f16_bits(x.numpy())
    assert np.array_equal(got, want)
    # and back: every finite code survives a round trip
    codes = np.arange(65536, dtype=np.uint16)
    finite = ((codes >> 10) & 0x1F) != 31
    assert np.array_equal(orc.f32_to_f16_bits(orc.f16_bits_to_f32(codes[finite])), codes[finite])


def test_e4m3_table_matches_torch_all_codes():
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fn).float().numpy()
    got = orc.e4m3_code_table()
    nan = np.isnan(want)
    assert np.array_equal(nan, np.isnan(got))
    assert np.array_equal(got[~nan], want[~nan])
    assert got[126] == 448.0 and nan.sum() == 2


def test_e4m3_encode_matches_torch():
    g = torch.Generator().manual_seed(2)
    x = torch.cat([torch.randn(100000, generator=g) * 100, torch.randn(100000, generator=g),
                   torch.randn(50000, generator=g) * 0.01])
    t = orc.e4m3_code_table()[:127]
    mids = torch.tensor((t[:-1] + t[1:]) / 2)        # exact ties between neighbours
    x = torch.cat([x, mids, -mids, torch.tensor(t), torch.tensor([500.0, -1e9, 448.0, 464.0])])
    xc = x.clamp(-448, 448)
    want = raw(xc.to(torch.float8_e4m3fn))
    got = orc.f32_to_e4m3_bits(x.numpy())
    assert np.array_equal(got, want)


# ------------------------------------------------------------------ append --

def _rand_table(rng, lens, bs, pool_blocks):
    need = [math.ceil(L / bs) for L in lens]
    perm = rng.permutation(pool_blocks)
    table = np.zeros((len(lens), max(need)), dtype=np.int32)
    cur = 0
    for s, n in enumerate(need):
        table[s, :n] = perm[cur:cur + n]
        cur += n
    return table


def test_append_gather_round_trip_and_sentinels():
    rng = np.random.default_rng(0)
    hkv, d, bs, nb = 3, 8, 4, 40
    lens = [1, 4, 5, 17, 0, 9]
    table = _rand_table(rng, [max(L, 1) for L in lens], bs, nb)
    k_pool = np.full((nb, hkv, bs, d), 0xBEEF, dtype=np.uint16)
    v_pool = np.full((nb, hkv, bs, d), 0xDEAD, dtype=np.uint16)
    hist_k, hist_v, slots = [], [], []
    for s, L in enumerate(lens):
        for t in range(L):
            slots.append(orc.slot_of(table[s], t, bs))
    T = len(slots)
    key = rng.integers(0, 65536, size=(T, hkv, d), dtype=np.uint16)
    val = rng.integers(0, 65536, size=(T, hkv, d), dtype=np.uint16)
    # a padding row (slot -1) in the middle must be skipped
    slots2 = slots[:3] + [-1] + slots[3:]
    key2 = np.concatenate([key[:3], key[:1], key[3:]])
    val2 = np.concatenate([val[:3], val[:1], val[3:]])
    orc.kv_append(key2, val2, k_pool, v_pool, slots2)
    kp2 = np.full_like(k_pool, 0xBEEF)
    vp2 = np.full_like(v_pool, 0xDEAD)
    orc.kv_append_fast(key2, val2, kp2, vp2, slots2)
    assert np.array_equal(k_pool, kp2) and np.array_equal(v_pool, vp2)
    cur = 0
    for s, L in enumerate(lens):
        assert np.array_equal(orc.gather_context(k_pool, table[s], L), key[cur:cur + L])
        assert np.array_equal(orc.gather_context(v_pool, table[s], L), val[cur:cur + L])
        # the vectorised gather the full-size tests use is the token loop, element for element
        assert np.array_equal(orc.gather_context_fast(k_pool, table[s], L), key[cur:cur + L])
        assert orc.gather_context_fast(v_pool, table[s], L).shape == (L, hkv, d)
        cur += L
    touched = np.zeros(nb * bs, dtype=bool)
    touched[slots] = True
    flat_k = k_pool.transpose(0, 2, 1, 3).reshape(nb * bs, hkv, d)
    assert (flat_k[~touched] == 0xBEEF).all()
    assert len(set(slots)) == len(slots)


def test_vectorised_gather_equals_the_token_loop_in_the_attention_oracle():
    """paged_decode_attn / paged_prefill_attn give identical float64 results with either gather,
    on ragged lengths that end inside a block, at a block edge and on an empty row."""
    rng = np.random.default_rng(7)
    hq, hkv, d, bs, nb = 4, 2, 8, 4, 64
    lens = [1, 4, 5, 17, 0, 33]
    table = _rand_table(rng, [max(L, 1) for L in lens], bs, nb)
    kp = rng.standard_normal((nb, hkv, bs, d)).astype(np.float32)
    vp = rng.standard_normal((nb, hkv, bs, d)).astype(np.float32)
    q = rng.standard_normal((len(lens), hq, d)).astype(np.float32)
    a = orc.paged_decode_attn(q, kp, vp, table, lens, 0.3)
    b = orc.paged_decode_attn(q, kp, vp, table, lens, 0.3, gather=orc.gather_context_fast)
    assert np.array_equal(a, b)
    news = [1, 2, 5, 9, 0, 20]
    cu = np.concatenate([[0], np.cumsum(news)])
    qq = rng.standard_normal((cu[-1], hq, d)).astype(np.float32)
    a = orc.paged_prefill_attn(qq, kp, vp, table, lens, cu, 0.3)
    b = orc.paged_prefill_attn(qq, kp, vp, table, lens, cu, 0.3, gather=orc.gather_context_fast)
    assert np.array_equal(a, b)


def test_append_equals_reference_slice_assign():
    """Paged append + gather == the contiguous cache[:, :, pos:end] = new of the
    reference layout, for prefill then three decode steps."""
    torch.manual_seed(0)
    B, H, D, bs, max_seq = 2, 3, 8, 4, 32
    store = cref.ContiguousStore(1, B, max_seq, H, D, dtype=torch.float32)
    store.allocate(B)
    nb = B * max_seq // bs
    rng = np.random.default_rng(1)
    table = _rand_table(rng, [max_seq] * B, bs, nb)
    k_pool = np.zeros((nb, H, bs, D), dtype=np.float32)
    v_pool = np.zeros_like(k_pool)
    pos = 0
    for n in (5, 1, 1, 1):
        nk, nv = torch.randn(B, H, n, D), torch.randn(B, H, n, D)
        fk, fv = store.update(0, nk, nv, position=pos)
        slots = [orc.slot_of(table[b], pos + i, bs) for b in range(B) for i in range(n)]
        rows_k = nk.permute(0, 2, 1, 3).reshape(B * n, H, D).numpy()
        rows_v = nv.permute(0, 2, 1, 3).reshape(B * n, H, D).numpy()
        orc.kv_append(rows_k, rows_v, k_pool, v_pool, slots)
        pos += n
        for b in range(B):
            got = orc.gather_context(k_pool, table[b], pos)            # [L, H, D]
            assert np.array_equal(got, fk[b].permute(1, 0, 2).numpy())
            got = orc.gather_context(v_pool, table[b], pos)
            assert np.array_equal(got, fv[b].permute(1, 0, 2).numpy())
    assert store.seq_len == 8


# --------------------------------------------------------------- attention --

def _rand_qkv(rng, n, L, hq, hkv, d):
    return (rng.standard_normal((n, hq, d)), rng.standard_normal((L, hkv, d)),
            rng.standard_normal((L, hkv, d)))


@pytest.mark.parametrize("prior", [None, 0, 3])
def test_attention_matches_bruteforce(prior):
    rng = np.random.default_rng(3)
    n = 1 if prior is None else 4
    L = 9 if prior is None else prior + n
    q, k, v = _rand_qkv(rng, n, L, 4, 2, 5)
    a = orc.attend_contiguous(q, k, v, 0.37, prior)
    b = orc.attend_bruteforce(q, k, v, 0.37, prior)
    assert np.allclose(a, b, rtol=1e-12, atol=1e-13)


def test_attention_matches_torch_sdpa_decode_and_causal():
    rng = np.random.default_rng(4)
    hq, hkv, d, L = 8, 2, 16, 37
    g = hq // hkv
    q, k, v = _rand_qkv(rng, L, L, hq, hkv, d)
    tq = torch.from_numpy(q).permute(1, 0, 2)[None]                      # [1,Hq,L,D]
    tk = torch.from_numpy(k).permute(1, 0, 2).repeat_interleave(g, 0)[None]
    tv = torch.from_numpy(v).permute(1, 0, 2).repeat_interleave(g, 0)[None]
    scale = 1 / math.sqrt(d)
    want = F.scaled_dot_product_attention(tq, tk, tv, is_causal=True)[0].permute(1, 0, 2).numpy()
    got = orc.attend_contiguous(q, k, v, scale, prior=0)
    assert np.allclose(got, want, rtol=1e-10, atol=1e-12)
    want = F.scaled_dot_product_attention(tq[:, :, -1:], tk, tv)[0].permute(1, 0, 2).numpy()
    got = orc.attend_contiguous(q[-1:], k, v, scale, prior=None)
    assert np.allclose(got, want, rtol=1e-10, atol=1e-12)
    # a one-token chunk with prior L-1 is the decode
    got2 = orc.attend_contiguous(q[-1:], k, v, scale, prior=L - 1)
    assert np.array_equal(got, got2)


def test_attention_closed_forms():
    rng = np.random.default_rng(5)
    hq, hkv, d = 4, 2, 8
    q, k, v = _rand_qkv(rng, 1, 11, hq, hkv, d)
    # L == 1: the output is the V row of the head's KV head
    o = orc.attend_contiguous(q, k[:1], v[:1], 0.3)
    assert np.allclose(o[0], v[0][orc.repeat_kv_index(hq, hkv)], rtol=0, atol=1e-15)
    # all keys equal: uniform weights, output = mean of V
    keq = np.repeat(k[:1], 11, axis=0)
    o = orc.attend_contiguous(q, keq, v, 0.3)
    assert np.allclose(o[0], v.mean(axis=0)[orc.repeat_kv_index(hq, hkv)], atol=1e-14)
    # shift invariance: K + c*q_dir changes every score of a row by the same amount only if
    # the shift is along a key-independent direction: add the same vector to every key
    shift = rng.standard_normal((1, hkv, d)) * 50
    o1 = orc.attend_contiguous(q, k, v, 0.3)
    o2 = orc.attend_contiguous(q, k + shift, v, 0.3)
    assert np.allclose(o1, o2, atol=1e-9)
    # heads of one GQA group with the same query give the same output
    q2 = q.copy()
    q2[:, 1] = q2[:, 0]
    o = orc.attend_contiguous(q2, k, v, 0.3)
    assert np.array_equal(o[:, 0], o[:, 1])
    # a one-hot-dominant score picks one V row
    kk = np.zeros((5, hkv, d)); kk[3] = q[0, ::2] * 100
    o = orc.attend_contiguous(q, kk, v[:5], 1.0)
    assert np.allclose(o[0, 0], v[3, 0], atol=1e-12)


def test_paged_decode_ignores_tail_and_block_order():
    rng = np.random.default_rng(6)
    hq, hkv, d, bs, nb = 4, 2, 8, 4, 24
    lens = [5, 13, 1, 0]
    table = _rand_table(rng, [max(L, 1) for L in lens], bs, nb)
    k_pool = rng.standard_normal((nb, hkv, bs, d)).astype(np.float32)
    v_pool = rng.standard_normal((nb, hkv, bs, d)).astype(np.float32)
    q = rng.standard_normal((len(lens), hq, d)).astype(np.float32)
    base = orc.paged_decode_attn(q, k_pool, v_pool, table, lens, 0.35)
    assert np.array_equal(base[3], np.zeros((hq, d)))
    # poison every slot beyond the context in the last block, and all unused blocks
    kp, vp = k_pool.copy(), v_pool.copy()
    used = set()
    for s, L in enumerate(lens):
        for t in range(L):
            used.add(orc.slot_of(table[s], t, bs))
    for slot in range(nb * bs):
        if slot not in used:
            kp[slot // bs, :, slot % bs] = np.nan
            vp[slot // bs, :, slot % bs] = np.inf
    assert np.array_equal(orc.paged_decode_attn(q, kp, vp, table, lens, 0.35), base)
    # move every block elsewhere, update the table: same result bit for bit
    perm = rng.permutation(nb)
    kp2, vp2 = np.empty_like(k_pool), np.empty_like(v_pool)
    kp2[perm] = k_pool
    vp2[perm] = v_pool
    assert np.array_equal(orc.paged_decode_attn(q, kp2, vp2, perm[table].astype(np.int32), lens, 0.35), base)
    # against the contiguous formula on the gathered history
    for s, L in enumerate(lens[:3]):
        k = orc.gather_context(k_pool, table[s], L).astype(np.float64)
        v = orc.gather_context(v_pool, table[s], L).astype(np.float64)
        want = orc.attend_bruteforce(q[s][None].astype(np.float64), k, v, 0.35)[0]
        assert np.allclose(base[s], want, rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("psize", [1, 3, 4, 16])
def test_splitk_merge_equals_unsplit(psize):
    rng = np.random.default_rng(7)
    hq, hkv, d, L = 4, 2, 8, 13
    q, k, v = _rand_qkv(rng, 1, L, hq, hkv, d)
    k[4] += 20 * np.repeat(q[0, ::2], 1, axis=0)          # one dominant key: max handling matters
    full = orc.attend_contiguous(q, k, v, 0.5)[0]
    parts = [orc.partition_partial(q[0], k[i:i + psize], v[i:i + psize], 0.5)
             for i in range(0, L, psize)]
    parts.append(orc.partition_partial(q[0], k[:0], v[:0], 0.5))  # an empty partition
    ms, ls, os_ = zip(*parts)
    assert np.allclose(orc.splitk_merge(ms, ls, os_), full, rtol=1e-12, atol=1e-13)


def test_paged_prefill_reductions():
    rng = np.random.default_rng(8)
    hq, hkv, d, bs, nb = 4, 2, 8, 4, 32
    priors, news = [0, 6, 9], [7, 5, 1]
    ctx = [p + n for p, n in zip(priors, news)]
    table = _rand_table(rng, ctx, bs, nb)
    k_pool = rng.standard_normal((nb, hkv, bs, d)).astype(np.float32)
    v_pool = rng.standard_normal((nb, hkv, bs, d)).astype(np.float32)
    cu = np.concatenate([[0], np.cumsum(news)])
    q = rng.standard_normal((cu[-1], hq, d)).astype(np.float32)
    out = orc.paged_prefill_attn(q, k_pool, v_pool, table, ctx, cu, 0.4)
    # prior == 0: torch SDPA is_causal=True on the gathered K/V (kv_cache.py:412-415)
    k = torch.from_numpy(orc.gather_context(k_pool, table[0], 7)).double().permute(1, 0, 2)
    v = torch.from_numpy(orc.gather_context(v_pool, table[0], 7)).double().permute(1, 0, 2)
    tq = torch.from_numpy(q[:7]).double().permute(1, 0, 2)[None]
    want = F.scaled_dot_product_attention(tq, k.repeat_interleave(2, 0)[None],
                                          v.repeat_interleave(2, 0)[None], is_causal=True, scale=0.4)
    assert np.allclose(out[:7], want[0].permute(1, 0, 2).numpy(), rtol=1e-10, atol=1e-12)
    # chunk of one token == decode
    dec = orc.paged_decode_attn(q[12:13], k_pool, v_pool, table[2:3], [10], 0.4)
    assert np.array_equal(out[12], dec[0])
    # prior > 0: row i is a decode over prior + i + 1 tokens
    for i in range(5):
        dec = orc.paged_decode_attn(q[7 + i:8 + i], k_pool, v_pool, table[1:2], [6 + i + 1], 0.4)
        assert np.allclose(out[7 + i], dec[0], rtol=1e-13, atol=1e-14)


def test_fp8_scales_and_dequant_oracle():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((50, 3, 16)).astype(np.float32)
    s = orc.absmax_scales(x)
    assert s.shape == (3,) and np.allclose(s * 448, np.abs(x).max(axis=(0, 2)))
    codes = orc.f32_to_e4m3_bits(x / s[None, :, None])
    deq = orc.e4m3_bits_to_f32(codes) * s[None, :, None]
    assert np.abs(deq - x).max() <= 0.0625 * np.abs(x).max() + 1e-6   # half an ulp at 3 mantissa bits


# --------------------------------------------- reference operator restated --

def test_contiguous_operator_equals_paged_oracle():
    """On a paged state that is the image of a contiguous cache, the paged oracle
    reproduces the reference operator (append -> contiguous -> SDPA)."""
    torch.manual_seed(3)
    B, hq, hkv, D, bs, max_seq = 2, 4, 2, 8, 4, 32
    g = hq // hkv
    op = cref.ContiguousCachedAttention(0, max_seq)
    op.enable()
    nb = B * max_seq // bs
    rng = np.random.default_rng(2)
    table = _rand_table(rng, [max_seq] * B, bs, nb)
    k_pool = np.zeros((nb, hkv, bs, D), dtype=np.float32)
    v_pool = np.zeros_like(k_pool)
    pos = 0
    for n in (6, 1, 1):
        q = torch.randn(B, hq, n, D)
        k = torch.randn(B, hkv, n, D)
        v = torch.randn(B, hkv, n, D)
        want = op(q, k.repeat_interleave(g, 1), v.repeat_interleave(g, 1),
                  attn_mask=torch.ones(n, n), is_causal=False)       # mask must be ignored
        slots = [orc.slot_of(table[b], pos + i, bs) for b in range(B) for i in range(n)]
        orc.kv_append(k.permute(0, 2, 1, 3).reshape(B * n, hkv, D).numpy(),
                      v.permute(0, 2, 1, 3).reshape(B * n, hkv, D).numpy(), k_pool, v_pool, slots)
        qrows = q.permute(0, 2, 1, 3).reshape(B * n, hq, D).numpy()
        ctx = [pos + n] * B
        cu = np.arange(B + 1) * n
        got = orc.paged_prefill_attn(qrows, k_pool, v_pool, table, ctx, cu, 1 / math.sqrt(D))
        got = got.reshape(B, n, hq, D).transpose(0, 2, 1, 3)
        assert np.allclose(got, want.double().numpy(), rtol=1e-5, atol=1e-6)
        pos += n
    assert op.pos == 8


def test_contiguous_store_errors():
    st = cref.ContiguousStore(4, 2, 8, 2, 4, dtype=torch.float32, layer_start=1, layer_end=3)
    with pytest.raises(ValueError):
        st.allocate(3)
    with pytest.raises(ValueError):
        st.allocate(2, seq_len=9)
    st.allocate(2)
    with pytest.raises(ValueError):
        st.update(0, torch.zeros(2, 2, 1, 4), torch.zeros(2, 2, 1, 4))
    with pytest.raises(ValueError):
        st.update(1, torch.zeros(2, 2, 9, 4), torch.zeros(2, 2, 9, 4))
    st.update(2, torch.ones(2, 2, 3, 4), torch.ones(2, 2, 3, 4), position=0)
    assert st.seq_len == 0                      # only the first local layer moves the length
    st.update(1, torch.ones(2, 2, 3, 4), torch.ones(2, 2, 3, 4), position=0)
    assert st.seq_len == 3
    k3, _ = st.update(1, torch.ones(2, 3, 4), torch.ones(2, 3, 4))   # 3-D input: batch 1 broadcast
    assert k3.shape == (2, 2, 6, 4)


@pytest.mark.parametrize("prior,n", [(0, 1), (0, 37), (13, 9), (64, 40)])
def test_cpu_prefill_restatement_equals_the_paged_oracle(prior, n):
    """The bench's CPU baseline for chunked prefill (gather -> repeat_kv -> contiguous -> SDPA) gives
    what the float64 paged oracle gives, for a chunk that starts a sequence (is_causal, as in the
    reference) and for one over a prior context (this build's causal-within-the-chunk rule)."""
    torch.manual_seed(prior + n)
    hq, hkv, d, bs = 6, 2, 16, 16
    L = prior + n
    nblk = -(-L // bs)
    kp, vp = torch.randn(nblk + 3, hkv, bs, d), torch.randn(nblk + 3, hkv, bs, d)
    tab = torch.randperm(nblk + 3)[:nblk].to(torch.int32)
    q = torch.randn(n, hq, d)
    got = cref.reference_cpu_prefill(q, kp, vp, tab, L, 1 / d ** 0.5).double().numpy()
    want = orc.paged_prefill_attn(q.numpy(), kp.numpy(), vp.numpy(), tab[None].numpy(), [L], np.array([0, n]),
                                  1 / d ** 0.5, "f32", "f32")
    assert np.abs(got - want).max() < 2e-6
