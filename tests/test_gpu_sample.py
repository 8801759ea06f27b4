"""Sampling kernel through the C ABI vs the oracle."""
import numpy as np
import pytest
import torch

from aicomp_amd import ops
from oracle import sample_oracle as S

pytestmark = pytest.mark.gpu
MARGIN = 2e-5          # entries whose preceding mass is this close to top_p may fall on either side


def check_rows(device, x_cpu, temperature, top_k, top_p, dtype=torch.float32, seed=0):
    """Kernel distribution and draw vs the oracle on every row of x_cpu [B, V] (float32 values)."""
    B, V = x_cpu.shape
    g = torch.Generator().manual_seed(seed)
    u = torch.rand(B, generator=g)
    xt = torch.from_numpy(x_cpu).to(dtype)
    name = {torch.bfloat16: "bf16", torch.float16: "f16"}.get(dtype, "f32")
    vals = xt.float().numpy()
    tok, probs = ops.sample_tokens(xt.to(device), temperature, top_k, top_p, True, u.to(device), return_probs=True)
    torch.cuda.synchronize()
    tok, probs = tok.cpu().numpy(), probs.cpu().numpy().astype(np.float64)
    n_marginal = 0
    for b in range(B):
        want = S.filtered_probs(vals[b], temperature, top_k, top_p, name)
        margin = S.nucleus_margin(vals[b], temperature, top_k, top_p, name) if top_p < 1 else np.full(V, np.inf)
        sure = margin > MARGIN
        n_marginal += int((~sure).sum())
        assert np.array_equal((probs[b] > 0)[sure], (want > 0)[sure]), f"row {b}: kept set differs"
        assert abs(probs[b].sum() - 1) < 1e-5
        if np.array_equal(probs[b] > 0, want > 0):
            assert np.allclose(probs[b], want, rtol=2e-5, atol=1e-9), f"row {b}: probabilities differ"
        # the draw: inverse CDF in index order at u[b], up to float rounding at a CDF step
        cdf = np.cumsum(probs[b])
        t = int(tok[b])
        assert probs[b, t] > 0, f"row {b}: token {t} has no mass"
        lo = cdf[t - 1] if t else 0.0
        assert lo - 1e-6 <= float(u[b]) <= cdf[t] + 1e-6, f"row {b}: u={float(u[b])} not in [{lo}, {cdf[t]}]"
    assert n_marginal <= 2 + 0.03 * B * V          # the check above must not be vacuous
    return tok, probs


@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, 0, 1.0), (0.7, 0, 1.0), (1.0, 40, 1.0), (1.0, 0, 0.9),
                                                     (0.8, 50, 0.9), (1.5, 1000, 0.3), (1.0, 7, 0.0),
                                                     (1.0, 100000, 0.9999), (0.5, 1, 0.5)])
def test_distribution_and_draw_match_oracle(device, temperature, top_k, top_p):
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((6, 5000)) * 2.5).astype(np.float32)
    check_rows(device, x, temperature, top_k, top_p)


def test_odd_vocabulary_sizes_and_tiny_rows(device):
    rng = np.random.default_rng(4)
    for V in (1, 2, 63, 64, 65, 1023, 1025, 4097):
        x = (rng.standard_normal((3, V)) * 2).astype(np.float32)
        check_rows(device, x, 0.9, min(5, V), 0.8, seed=V)


def test_bf16_logits(device):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((4, 3000)) * 3).astype(np.float32)
    check_rows(device, x, 0.7, 20, 0.95, dtype=torch.bfloat16)


def test_ties_top_k_keeps_all_top_p_keeps_in_index_order(device):
    x = np.zeros((1, 10), dtype=np.float32)
    _, p = check_rows(device, x, 1.0, 0, 0.35)
    assert (p[0] > 0).tolist() == [True] * 4 + [False] * 6
    x = np.array([[1.0, 3.0, 2.0, 3.0, 2.0, 0.0]], dtype=np.float32)
    _, p = check_rows(device, x, 1.0, 3, 1.0)
    assert (p[0] > 0).tolist() == [False, True, True, True, True, False]
    # a large flat row: every histogram lane hits the same bins
    x = np.full((2, 20000), -1.25, dtype=np.float32)
    _, p = check_rows(device, x, 1.0, 0, 0.5)
    assert (p[0] > 0).sum() in (10000, 10001)
    # top-k on a flat row keeps every tie (more candidates than the kernel's LDS list holds)
    _, p = check_rows(device, x, 1.0, 7, 1.0)
    assert (p[0] > 0).sum() == 20000
    _, p = check_rows(device, x, 1.3, 7, 0.25)
    assert (p[0] > 0).sum() in (5000, 5001)
    # a few distinct values above a flat floor: the candidate list is used
    x[:, 5::1000] = np.linspace(1, 2, 20, dtype=np.float32)
    _, p = check_rows(device, x, 1.0, 12, 1.0)
    assert (p[0] > 0).sum() == 12


def test_greedy_is_argmax_lowest_index(device):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((16, 7001)).astype(np.float32)
    x[3, 100] = x[3, 6000] = 9.0                       # equal maxima: the lower index wins
    xt = torch.from_numpy(x).to(device)
    tok, probs = ops.sample_tokens(xt, do_sample=False, return_probs=True)
    torch.cuda.synchronize()
    assert tok.cpu().tolist() == [S.greedy(r) for r in x] and tok[3].item() == 100
    assert torch.equal(probs.argmax(-1), tok) and (probs.sum(-1) == 1).all()
    tb = ops.sample_tokens(xt.bfloat16(), do_sample=False)
    assert tb.cpu().tolist() == [int(np.argmax(r)) for r in xt.bfloat16().float().cpu().numpy()]


def test_statistics_of_the_draw(device):
    rng = np.random.default_rng(7)
    row = (rng.standard_normal(50) * 1.5).astype(np.float32)
    N = 40000
    x = torch.from_numpy(np.tile(row, (N, 1))).to(device)
    tok = ops.sample_tokens(x, 0.9, 12, 0.9, generator=torch.Generator(device=device).manual_seed(1))
    torch.cuda.synchronize()
    want = S.filtered_probs(row, 0.9, 12, 0.9)
    counts = np.bincount(tok.cpu().numpy(), minlength=50)
    assert (counts[want == 0] == 0).all()
    keep = want > 0
    chi2 = (((counts[keep] - N * want[keep]) ** 2) / (N * want[keep])).sum()
    assert chi2 < 40, f"chi-square {chi2:.1f} over {keep.sum()} categories"     # 99.9 % point for 11 dof is 31.3


def test_reproducible_and_input_untouched(device):
    rng = np.random.default_rng(8)
    x = torch.from_numpy((rng.standard_normal((32, 128256)) * 2).astype(np.float32)).to(device)
    keep = x.clone()
    u = torch.rand(32, device=device)
    a, pa = ops.sample_tokens(x, 0.8, 50, 0.9, uniforms=u, return_probs=True)
    b, pb = ops.sample_tokens(x, 0.8, 50, 0.9, uniforms=u, return_probs=True)
    c = ops.sample_tokens(x, 0.8, 50, 0.9, uniforms=u)
    torch.cuda.synchronize()
    assert torch.equal(a, b) and torch.equal(pa, pb) and torch.equal(a, c) and torch.equal(x, keep)
    assert ((pa > 0).sum(-1) <= 50).all() and torch.allclose(pa.sum(-1), torch.ones(32, device=device), atol=1e-5)
    # three rows of the full-vocabulary batch against the oracle
    xc = x[:3].cpu().numpy()
    for r in range(3):
        want = S.filtered_probs(xc[r], 0.8, 50, 0.9)
        got = pa[r].cpu().numpy().astype(np.float64)
        margin = S.nucleus_margin(xc[r], 0.8, 50, 0.9)
        sure = margin > MARGIN
        assert np.array_equal((got > 0)[sure], (want > 0)[sure])


def test_rejects_bad_arguments(device):
    x = torch.zeros(2, 10, device=device)
    with pytest.raises(RuntimeError):
        ops.sample_tokens(x, temperature=0.0)
    with pytest.raises(RuntimeError):
        ops.sample_tokens(x.double())
    with pytest.raises(RuntimeError):
        ops.sample_tokens(x.cpu())
    with pytest.raises(RuntimeError):
        ops.sample_tokens(x, uniforms=torch.rand(3, device=device))
    with pytest.raises(RuntimeError):
        ops.sample_tokens(x.t())


def test_masked_vocabulary(device):
    """Rows where most of the vocabulary is masked with -inf, the way a constrained decoder hands
    them over: fewer finite logits than top_k, exactly top_k, many more; -inf entries get no mass.
    A row without any finite logit returns the argmax convention (index 0) and an all-zero row."""
    rng = np.random.default_rng(9)
    V = 6000
    x = np.full((5, V), -np.inf, dtype=np.float32)
    for b, n_finite in enumerate([1, 10, 50, 51, 3000]):
        idx = rng.choice(V, n_finite, replace=False)
        x[b, idx] = (rng.standard_normal(n_finite) * 2).astype(np.float32)
    for temperature, top_k, top_p in [(0.8, 50, 0.9), (1.0, 50, 1.0), (1.0, 0, 0.9), (1.0, 0, 1.0), (1.3, 2000, 0.5)]:
        tok, probs = check_rows(device, x, temperature, top_k, top_p)
        assert np.all(probs[~np.isfinite(x)] == 0)
    dead = torch.full((2, 300), float("-inf"), device=device)
    tok, probs = ops.sample_tokens(dead, 0.8, 50, 0.9, True, torch.tensor([0.3, 0.9], device=device), return_probs=True)
    assert tok.tolist() == [0, 0] and float(probs.abs().sum()) == 0.0
    tok = ops.sample_tokens(dead, do_sample=False)
    assert tok.tolist() == [0, 0]


def test_nucleus_without_top_k_routes(device):
    """top-p without top-k takes one of three routes: a short candidate list above a cut near the
    maximum (peaked rows), the full-row walk resumed below the first digit level (a nucleus of
    thousands), or the complete full-row walk (the threshold lies far below the maximum)."""
    rng = np.random.default_rng(11)
    V = 40000
    peaked = (rng.standard_normal((3, V)) * 2).astype(np.float32)
    for b in range(3):
        peaked[b, rng.choice(V, 25, replace=False)] = 12 + rng.standard_normal(25).astype(np.float32) * 3
    broad = (rng.standard_normal((3, V)) * 3.5).astype(np.float32)
    far = np.zeros((2, V), dtype=np.float32)
    far[:, 17] = 13.0                                   # one strong token, the rest tied 13 below it
    far[1, 5000:5100] = 2.0
    for x in (peaked, broad, far):
        for temperature, top_p in [(1.0, 0.9), (0.8, 0.5), (1.3, 0.97)]:
            check_rows(device, x, temperature, 0, top_p)
    check_rows(device, peaked, 0.7, 0, 0.9, dtype=torch.bfloat16)
    check_rows(device, broad, 0.7, 0, 0.9, dtype=torch.bfloat16)


def test_signed_zeros_are_one_value(device):
    """-0.0 and +0.0 compare equal in the reference's float comparisons: when the k-th largest value
    is a zero, both kinds stay, and they tie in the nucleus order."""
    rng = np.random.default_rng(12)
    V = 5000
    x = (np.round(rng.standard_normal((2, V)) * 1.0) / 2).astype(np.float32)     # many -0.0 and +0.0
    assert (np.signbit(x) & (x == 0)).sum() > 100 and (~np.signbit(x) & (x == 0)).sum() > 100
    for temperature, top_k, top_p in [(1.5, 2000, 1.0), (1.5, 2000, 0.9), (1.0, 300, 0.95), (0.7, 0, 0.8)]:
        check_rows(device, x, temperature, top_k, top_p)
