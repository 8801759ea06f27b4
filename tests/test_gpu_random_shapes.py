"""Seeded random shapes through the C ABI and the drop-in operator.

Decode and chunked prefill on random head geometries, head dims, block sizes, element types,
ragged contexts and partition sizes against the float64 oracle; random sessions of the operator
(batch, GQA group, views as HF Llama builds them or contiguous, prefill then decode steps and
further chunks) against the restatement of the reference's contiguous cache.
"""
import random

import numpy as np
import pytest
import torch

import test_gpu_prefill as tp
from aicomp_amd import kv_cache as akv
from aicomp_amd import ops
from oracle import contiguous_ref as cref
from helpers import to_f64

pytestmark = pytest.mark.gpu


def _close(got, want, atol, rtol):
    err = np.abs(got - want)
    return bool(((err <= atol) | (err <= rtol * np.abs(want))).all()), float(err.max())


@pytest.mark.parametrize("seed", range(4))
@pytest.mark.parametrize("schedule", ["balanced", "library"])
def test_random_decode_and_prefill_shapes(device, seed, schedule):
    # "library": the library's own choice of decode schedule for small calls (the suite otherwise
    # pins automatic calls to the balanced schedule)
    if schedule == "library":
        ops.set_small_decode_tokens(32768)          # the autouse fixture restores the suite's setting
    rnd = random.Random(100 + seed)
    for trial in range(12):
        nseq = rnd.randint(1, 5)
        g = rnd.choice([1, 2, 4, 8, 16, 3])
        hkv = rnd.choice([1, 2, 4])
        hq = hkv * g
        d = rnd.choice([64, 128, 128, 256])
        bs = 16 if rnd.random() < 0.8 else rnd.choice([8, 32])
        kv = rnd.choice([None, None, torch.float8_e4m3fn]) if d in (64, 128) and bs == 16 else None
        dtype = torch.bfloat16 if kv is not None or rnd.random() < 0.8 else torch.float32
        decode = rnd.random() < 0.4
        if decode:
            priors, news = [rnd.randint(0, 400) for _ in range(nseq)], [1] * nseq
        else:
            priors = [rnd.choice([0, 0, rnd.randint(0, 300)]) for _ in range(nseq)]
            news = [rnd.choice([1, rnd.randint(1, 40), rnd.randint(1, 200)]) for _ in range(nseq)]
        what = (f"seed {seed} trial {trial}: {nseq} seqs, {hq}/{hkv} heads, D {d}, block {bs}, kv {kv}, {dtype}, "
                f"decode={decode}, priors {priors}, news {news}")
        c = tp.build_case(device, priors, news, hq, hkv, d, bs=bs, dtype=dtype, kv_dtype=kv, seed=1000 * seed + trial)
        want = tp.oracle(c)
        if decode:
            out = torch.full_like(c["q"], float("nan"))
            ps = rnd.choice([0, 0, 64, 256]) // bs * bs
            ops.paged_decode_attn(out, c["q"], c["k_pool"], c["v_pool"], c["table"], c["ctx"], c["scale"],
                                  c["ks"], c["vs"], partition_size=ps)
            torch.cuda.synchronize()
            got = to_f64(out)
        else:
            got = to_f64(tp.run(c, max_q_len=rnd.choice([None, max(news)])))
        ok, mx = _close(got, want, *((1e-5, 1e-5) if dtype == torch.float32 else (1e-2, 2e-2)))
        assert ok and np.isfinite(got).all(), f"{what}: max abs err {mx:.3e}"


@pytest.mark.parametrize("seed", range(3))
@pytest.mark.parametrize("schedule", ["balanced", "library"])
def test_random_operator_sessions(device, seed, schedule, host_route):
    if schedule == "library":
        ops.set_small_decode_tokens(32768)          # the autouse fixture restores the suite's setting
    rnd = random.Random(200 + seed)
    torch.manual_seed(200 + seed)
    for trial in range(10):
        B = rnd.choice([1, 1, 2, 3, 5])
        g = rnd.choice([1, 2, 4, 8])
        hkv = rnd.choice([1, 2, 4, 8])
        hq, d = hkv * g, rnd.choice([64, 128])
        dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float32])
        max_seq = rnd.choice([64, 200, 513])
        kw = {"num_kv_groups": g} if rnd.random() < 0.5 else {}
        new = akv.CachedScaledDotProductAttention(0, max_seq_len=max_seq, dtype=dtype, **kw)
        ref = cref.ContiguousCachedAttention(0, max_seq)
        new.enable(); ref.enable()
        pos = 0
        steps = [rnd.randint(1, min(150, max_seq - 5))] + [rnd.choice([1, 1, 1, 1, rnd.randint(2, 20)]) for _ in range(6)]
        what = f"seed {seed} trial {trial}: B {B}, {hq}/{hkv} heads, D {d}, {dtype}, max_seq {max_seq}, {kw}, steps {steps}"
        for n in steps:
            if pos + n > max_seq:
                break
            if rnd.random() < 0.5:      # the way HF Llama hands them over: transposed views
                q = torch.randn(B, n, hq, d).to(dtype).to(device).transpose(1, 2)
                k = (torch.randn(B, n, hkv, d) * 0.5).to(dtype).to(device).transpose(1, 2)
                v = (torch.randn(B, n, hkv, d) * 0.5).to(dtype).to(device).transpose(1, 2)
            else:
                q = torch.randn(B, hq, n, d).to(dtype).to(device)
                k = (torch.randn(B, hkv, n, d) * 0.5).to(dtype).to(device)
                v = (torch.randn(B, hkv, n, d) * 0.5).to(dtype).to(device)
            ke, ve = (k.repeat_interleave(g, 1), v.repeat_interleave(g, 1)) if g > 1 else (k, v)
            got = new(q, ke, ve, attn_mask=None, is_causal=True)
            want = ref(q.float().cpu(), ke.float().cpu(), ve.float().cpu(), attn_mask=None, is_causal=True)
            if pos > 0 and n > 1:
                # a later chunk: this operator masks causally inside the chunk, the reference applies no mask
                mask = torch.ones(n, pos + n, dtype=torch.bool).tril(diagonal=pos)
                want = torch.nn.functional.scaled_dot_product_attention(
                    q.float().cpu(), ref.k[:, :, :pos + n], ref.v[:, :, :pos + n], attn_mask=mask)
            assert got.shape == want.shape, what
            err = (got.float().cpu() - want).abs()
            ok = (err <= 2e-5) if dtype == torch.float32 else ((err <= 1e-2) | (err <= 2e-2 * want.abs()))
            assert bool(ok.all()), f"{what}: n {n} at {pos}: max abs err {err.max().item():.3e}"
            pos += n
        new.disable()


@pytest.mark.parametrize("seed", range(3))
def test_random_sampler_rows(device, seed):
    """Random vocabulary sizes, row shapes (Gaussian, peaked, nearly flat, heavily tied incl. signed
    zeros, masked with -inf), temperatures, top-k / top-p and logit types against the oracle.  A
    probability below the kernel's fixed-point resolution (2^-40 of the row maximum) may be zero."""
    from oracle import sample_oracle as S
    rnd = random.Random(300 + seed)
    for trial in range(40):
        V = rnd.choice([1, 2, 17, 64, 500, 1024, 1025, 5000, 33000])
        B = rnd.choice([1, 3])
        rng = np.random.default_rng(1000 * seed + trial)
        kind = rnd.choice(["gauss", "peaked", "flat", "ties", "masked"])
        x = (rng.standard_normal((B, V)) * rnd.choice([0.5, 2.0, 4.0])).astype(np.float32)
        if kind == "peaked" and V > 40:
            for b in range(B):
                x[b, rng.choice(V, min(30, V // 2), replace=False)] += 12
        elif kind == "flat":
            x = (rng.standard_normal((B, V)) * 0.01).astype(np.float32)
        elif kind == "ties":
            x = (np.round(x * 2) / 2).astype(np.float32)
        elif kind == "masked" and V > 4:
            for b in range(B):
                x[b, rng.choice(V, V * 3 // 4, replace=False)] = -np.inf
        T = rnd.choice([1.0, 0.7, 1.5, 0.3, 5.0])
        top_k = rnd.choice([0, 0, 1, 5, 50, 1000, 2000, V, V + 5])
        top_p = rnd.choice([1.0, 0.9, 0.5, 0.99, 0.0, 0.3])
        dtype = rnd.choice([torch.float32, torch.float32, torch.bfloat16])
        what = f"seed {seed} trial {trial}: V {V}, {kind}, T {T}, top_k {top_k}, top_p {top_p}, {dtype}"
        u = torch.rand(B, generator=torch.Generator().manual_seed(trial))
        xt = torch.from_numpy(x).to(dtype)
        name = "bf16" if dtype == torch.bfloat16 else "f32"
        vals = xt.float().numpy()
        tok, probs = ops.sample_tokens(xt.to(device), T, top_k, top_p, True, u.to(device), return_probs=True)
        tok, probs = tok.cpu().numpy(), probs.cpu().numpy().astype(np.float64)
        for b in range(B):
            want = S.filtered_probs(vals[b], T, top_k, top_p, name)
            margin = S.nucleus_margin(vals[b], T, top_k, top_p, name) if top_p < 1 else np.full(V, np.inf)
            sure = (margin > 2e-5) & ((want > 1e-11) | (want == 0))
            assert np.array_equal((probs[b] > 0)[sure], (want > 0)[sure]), f"{what}, row {b}: kept set differs"
            assert abs(probs[b].sum() - 1) < 1e-5, what
            if np.array_equal(probs[b] > 0, want > 0):
                assert np.allclose(probs[b], want, rtol=3e-5, atol=1e-9), f"{what}, row {b}: probabilities differ"
            cdf, t = np.cumsum(probs[b]), int(tok[b])
            assert probs[b, t] > 0, f"{what}, row {b}: token {t} has no mass"
            lo = cdf[t - 1] if t else 0.0
            assert lo - 1e-6 <= float(u[b]) <= cdf[t] + 1e-6, f"{what}, row {b}: draw outside its CDF step"
