"""Pins of the sampling oracle (CPU)."""
import itertools

import numpy as np
import pytest
import torch

from oracle import sample_oracle as S


def reference_statements(logits, temperature, top_k, top_p):
    """The statements of _sample_token (opt_prime/opt_prime/inference.py:810-840) run by torch's CPU
    kernels in float64; returns the distribution handed to multinomial."""
    logits = logits.clone()
    if temperature != 1.0:
        logits = logits / temperature
    if top_k > 0:
        top_k = min(top_k, logits.size(-1))
        indices_to_remove = logits < torch.topk(logits, top_k)[0][..., -1, None]
        logits[indices_to_remove] = float('-inf')
    if top_p < 1.0:
        sorted_logits, sorted_indices = torch.sort(logits, descending=True)
        cumulative_probs = torch.cumsum(torch.softmax(sorted_logits, dim=-1), dim=-1)
        sorted_indices_to_remove = cumulative_probs > top_p
        sorted_indices_to_remove[..., 1:] = sorted_indices_to_remove[..., :-1].clone()
        sorted_indices_to_remove[..., 0] = 0
        indices_to_remove = sorted_indices_to_remove.scatter(-1, sorted_indices, sorted_indices_to_remove)
        logits[indices_to_remove] = float('-inf')
    return torch.softmax(logits, dim=-1)


@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, 0, 1.0), (0.7, 0, 1.0), (1.0, 5, 1.0), (1.0, 0, 0.9),
                                                     (0.8, 50, 0.9), (1.3, 1000, 0.5), (1.0, 3, 0.0), (2.0, 10**6, 0.999)])
def test_matches_library_ops_on_tie_free_rows(temperature, top_k, top_p):
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((4, 777)) * 3).astype(np.float32)
    # float64 torch ops: the float32 temperature division is applied first, as the oracle does
    xs = np.stack([S.scaled(r, temperature) for r in x])
    want = reference_statements(torch.from_numpy(xs).double(), 1.0, top_k, top_p).numpy()
    for r in range(4):
        got = S.filtered_probs(x[r], temperature, top_k, top_p)
        assert np.array_equal(got > 0, want[r] > 0)
        assert np.allclose(got, want[r], rtol=1e-12, atol=0)


def test_nucleus_rule_independent_formulation():
    # an entry stays iff the total probability of strictly more probable entries is <= top_p
    rng = np.random.default_rng(1)
    for _ in range(50):
        V = int(rng.integers(2, 40))
        x = rng.standard_normal(V).astype(np.float32) * 2
        top_p = float(rng.uniform(0, 1))
        p_all = np.exp(x.astype(np.float64) - x.max())
        p_all /= p_all.sum()
        keep = np.array([p_all[p_all > p_all[i]].sum() <= top_p for i in range(V)])
        got = S.filtered_probs(x, 1.0, 0, top_p)
        margin = S.nucleus_margin(x, 1.0, 0, top_p)
        sure = margin > 1e-12
        assert np.array_equal((got > 0)[sure], keep[sure])
        assert got[np.argmax(x)] > 0                      # the most probable entry always stays


def test_top_k_keeps_ties_and_brute_force():
    x = np.array([1.0, 3.0, 2.0, 3.0, 2.0, 0.0], dtype=np.float32)
    p = S.filtered_probs(x, 1.0, top_k=3)                 # third largest is 2.0: both 2.0 entries stay
    assert (p > 0).tolist() == [False, True, True, True, True, False]
    # brute force: every subset-free definition on all orderings of a tiny row
    for perm in itertools.permutations([0.5, 1.5, 2.5, 3.5]):
        x = np.array(perm, dtype=np.float32)
        for k in range(1, 5):
            p = S.filtered_probs(x, 1.0, top_k=k)
            assert sorted(x[p > 0].tolist()) == sorted(perm)[-k:]


def test_top_p_ties_are_kept_in_index_order():
    x = np.zeros(10, dtype=np.float32)                    # ten equal entries of probability 0.1
    p = S.filtered_probs(x, 1.0, 0, top_p=0.35)           # mass before entry j is 0.1 j <= 0.35 for j = 0..3
    assert (p > 0).tolist() == [True] * 4 + [False] * 6
    assert np.allclose(p[:4], 0.25)


def test_draw_is_inverse_cdf_and_greedy_lowest_index():
    p = np.array([0.0, 0.25, 0.0, 0.5, 0.25])
    assert [S.draw(p, u) for u in (0.0, 0.2499, 0.25, 0.7499, 0.75, 0.9999)] == [1, 1, 3, 3, 4, 4]
    assert S.greedy(np.array([1.0, 7.0, 7.0, 3.0])) == 1
    rng = np.random.default_rng(2)
    counts = np.bincount([S.draw(p, u) for u in rng.random(20000)], minlength=5)
    assert np.abs(counts / 20000 - p).max() < 0.015


def test_bf16_division_is_rounded_to_bf16():
    x = np.array([1.0, 2.0, 3.0], dtype=np.float32)
    s = S.scaled(x, 0.7, "bf16")
    want = (torch.tensor(x).bfloat16() / 0.7).float().numpy()
    assert np.array_equal(s, want)
