"""Pins of the rotary-embedding oracle (CPU).

The reference's rotary code (compiler_fx/modeling_llama.py:150-168, 200-231) is a copy of
transformers' Llama model file and cannot be imported on its own (package-relative imports);
the installed transformers carries the same functions, so they serve as the independent
library routine, next to the float64 closed form and the invariants of a rotation.
"""
import numpy as np
import pytest
import torch

from oracle import rope_oracle as R
from oracle import paged_kv_oracle as P
from helpers import raw

tf_llama = pytest.importorskip("transformers.models.llama.modeling_llama")


def rand_codes(rng, shape, dtype, std=1.0):
    x = (rng.standard_normal(shape) * std).astype(np.float32)
    return R._to_type(x, dtype)


# ------------------------------------------------------------------ closed form and invariants
def test_rotate_half_formula_is_a_complex_rotation():
    rng = np.random.default_rng(0)
    D = 64
    x = rng.standard_normal((5, 3, D))
    th = rng.uniform(-3, 3, size=(5, 1, D // 2))
    emb = np.concatenate([th, th], axis=-1)
    via_formula = x * np.cos(emb) + R.rotate_half(x) * np.sin(emb)
    assert np.allclose(via_formula, R.rope_exact(x, th), rtol=0, atol=1e-13)


def test_rotation_invariants_float64():
    rng = np.random.default_rng(1)
    D = 128
    inv = R.default_inv_freq(D).astype(np.float64)
    q = rng.standard_normal((1, D))
    k = rng.standard_normal((1, D))
    rot = lambda x, p: R.rope_exact(x, (p * inv)[None, :])
    # pair norms are preserved, position 0 is the identity
    r = rot(q, 37)
    assert np.allclose(r[:, :D // 2] ** 2 + r[:, D // 2:] ** 2, q[:, :D // 2] ** 2 + q[:, D // 2:] ** 2)
    assert np.array_equal(rot(q, 0), q)
    # scores depend on the distance only; rotations compose additively
    s = lambda m, n: float((rot(q, m) @ rot(k, n).T)[0, 0])
    assert abs(s(10, 3) - s(107, 100)) < 1e-9 and abs(s(10, 3) - s(3, 10)) > 1e-3
    assert np.allclose(rot(rot(q, 5), 9), rot(q, 14))


def test_default_inv_freq_matches_library_init():
    from transformers import LlamaConfig
    cfg = LlamaConfig(hidden_size=512, num_attention_heads=4, num_key_value_heads=2, num_hidden_layers=1,
                      intermediate_size=64, vocab_size=32, max_position_embeddings=256)
    emb = tf_llama.LlamaRotaryEmbedding(cfg)
    base = cfg.rope_parameters["rope_theta"] if hasattr(cfg, "rope_parameters") else cfg.rope_theta
    got, want = R.default_inv_freq(128, base=base), emb.inv_freq.numpy()
    assert np.abs(got.view(np.int32) - want.view(np.int32)).max() <= 1      # float32 powf vs float64 pow


# ------------------------------------------------------------------ rounding order, bit for bit
@pytest.mark.parametrize("dtype,tdtype", [("bf16", torch.bfloat16), ("f32", torch.float32)])
def test_apply_rope_bit_exact_vs_library(dtype, tdtype):
    rng = np.random.default_rng(2)
    B, H, S, D = 2, 3, 17, 64
    q = torch.from_numpy(rng.standard_normal((B, H, S, D)).astype(np.float32)).to(tdtype)
    k = torch.from_numpy((rng.standard_normal((B, 1, S, D)) * 30).astype(np.float32)).to(tdtype)
    th = torch.from_numpy(rng.uniform(-50, 50, size=(B, S, D // 2)).astype(np.float32))
    emb = torch.cat((th, th), dim=-1)
    cos, sin = emb.cos().to(tdtype), emb.sin().to(tdtype)
    q_ref, k_ref = tf_llama.apply_rotary_pos_emb(q, k, cos, sin)          # unsqueeze_dim = 1
    got_q = R.apply_rope(raw(q), raw(cos)[:, None], raw(sin)[:, None], dtype)
    got_k = R.apply_rope(raw(k), raw(cos)[:, None], raw(sin)[:, None], dtype)
    assert np.array_equal(got_q, raw(q_ref))
    assert np.array_equal(got_k, raw(k_ref))


def test_apply_rope_rounding_order_matters():
    # a fused multiply-add or a float32 intermediate gives different bf16 bits on enough elements:
    # the bit-exact test above would catch either mistake
    rng = np.random.default_rng(3)
    x = rand_codes(rng, (64, 128), "bf16")
    th = rng.uniform(-3, 3, size=(64, 64)).astype(np.float32)
    emb = np.concatenate([th, th], -1)
    c, s = R._to_type(np.cos(emb), "bf16"), R._to_type(np.sin(emb), "bf16")
    stepwise = R.apply_rope(x, c, s, "bf16")
    xf, cf, sf = (R._to_f32(a, "bf16") for a in (x, c, s))
    single = R._to_type(xf * cf + R.rotate_half(xf) * sf, "bf16")
    assert (stepwise != single).mean() > 0.01


# ------------------------------------------------------------------ tables
@pytest.mark.parametrize("dtype,tdtype", [("bf16", torch.bfloat16), ("f32", torch.float32)])
def test_tables_vs_float64_and_library(dtype, tdtype):
    from aicomp_amd import ops
    from transformers import LlamaConfig
    cfg = LlamaConfig(hidden_size=256, num_attention_heads=2, num_key_value_heads=1, num_hidden_layers=1,
                      intermediate_size=64, vocab_size=32, max_position_embeddings=4096)
    mod = tf_llama.LlamaRotaryEmbedding(cfg)
    P_ = 2048
    cos, sin = ops.rotary_tables(mod.inv_freq, P_, tdtype, attention_scaling=mod.attention_scaling, device="cpu")
    # bit for bit the library module's output for positions 0..P-1
    x = torch.zeros(1, 1, dtype=tdtype)
    lc, ls = mod(x, torch.arange(P_)[None, :])
    assert torch.equal(cos, lc[0]) and torch.equal(sin, ls[0])
    # the oracle's float64-based tables agree within one unit in the last place of the type
    oc, os_ = R.rope_tables(mod.inv_freq.numpy(), P_, dtype, mod.attention_scaling)
    for got, want in ((raw(cos), oc), (raw(sin), os_)):
        if dtype == "bf16":
            assert np.abs(got.astype(np.int32) - want.astype(np.int32)).max() <= 1
            assert (got != want).mean() < 0.01
        else:
            assert np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64)).max() <= 2 or \
                np.allclose(got, want, rtol=0, atol=1.2e-7)


# ------------------------------------------------------------------ rotation + append
def test_rope_kv_append_oracle_composes_rotation_and_copy():
    rng = np.random.default_rng(4)
    T, HQ, HKV, D, BS, NB = 9, 4, 2, 32, 16, 3
    q, k, v = (rand_codes(rng, (T, h, D), "bf16") for h in (HQ, HKV, HKV))
    cos, sin = R.rope_tables(R.default_inv_freq(D), 64, "bf16")
    pos = rng.integers(0, 64, size=T)
    pos[2] = 64                                   # no table row: token left alone
    slots = rng.permutation(NB * BS)[:T].astype(np.int64)
    slots[5] = -1                                 # padding: rotated, not stored
    kp = np.full((NB, HKV, BS, D), 0x7fc0, dtype=np.uint16)
    vp = kp.copy()
    q_out = R.rope_kv_append(q, k, v, cos, sin, pos, kp, vp, slots, "bf16")
    for t in range(T):
        if t == 2:
            assert np.array_equal(q_out[t], q[t])
            continue
        want_q = R.apply_rope(q[t], cos[pos[t]][None], sin[pos[t]][None], "bf16")
        assert np.array_equal(q_out[t], want_q)
        if t == 5:
            continue
        b, o = divmod(int(slots[t]), BS)
        assert np.array_equal(kp[b, :, o], R.apply_rope(k[t], cos[pos[t]][None], sin[pos[t]][None], "bf16"))
        assert np.array_equal(vp[b, :, o], v[t])
    touched = np.zeros(NB * BS, dtype=bool)
    touched[[int(s) for i, s in enumerate(slots) if i not in (2, 5)]] = True
    flat = kp.transpose(0, 2, 1, 3).reshape(NB * BS, -1)
    assert (flat[~touched] == 0x7fc0).all()
