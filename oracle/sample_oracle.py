"""CPU oracle for token sampling.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package may import this module.

What it restates, and from where
--------------------------------
``filtered_probs`` follows ``_sample_token`` statement by statement
(``opt_prime/opt_prime/inference.py:786-843``) on one row, in float64 after
the temperature division (which is done in the logits' own type, as there):

* ``:811-812``  ``logits = logits / temperature`` when temperature != 1;
* ``:815-818``  top-k: entries below the k-th largest value become -inf (ties at
  that value stay), ``k = min(top_k, V)``;
* ``:821-837``  top-p: descending sort, softmax, cumulative sum; an entry is
  removed when the cumulative sum *up to and including the previous entry*
  exceeds top_p (the shift by one), the first entry always stays;
* ``:840``      softmax of what is left.

``draw`` replaces ``torch.multinomial`` (``:841``) by the inverse CDF in index
order at a given uniform number: same distribution, caller-supplied randomness.
``greedy`` is ``argmax`` (``:806-808``), lowest index among equal maxima.

Ties in the descending sort are ordered by index (a stable sort); the reference's
``torch.sort`` leaves that order unspecified.

PARITY PINNING STATUS: pinned.  (i) against torch's own CPU ops executing the
reference's statements (topk, sort, cumsum, softmax, scatter are library routines) in
float64 on tie-free rows; (ii) against an independent formulation of the nucleus
rule (an entry stays iff the total probability of strictly more probable entries is
<= top_p); (iii) brute force on tiny vocabularies; the reference's tests hold no
vectors for it.
"""
from __future__ import annotations

import numpy as np

from . import paged_kv_oracle as P


def scaled(logits_row: np.ndarray, temperature: float, dtype: str = "f32") -> np.ndarray:
    """The temperature division in the logits' own type; returns float32 values."""
    x = np.asarray(logits_row, dtype=np.float32)
    if temperature != 1.0:
        x = (x / np.float32(temperature)).astype(np.float32)
        if dtype == "bf16":
            x = P.bf16_bits_to_f32(P.f32_to_bf16_bits(x))
        elif dtype == "f16":
            x = P.f16_bits_to_f32(P.f32_to_f16_bits(x))
    return x


def filtered_probs(logits_row: np.ndarray, temperature: float = 1.0, top_k: int = 0, top_p: float = 1.0,
                   dtype: str = "f32") -> np.ndarray:
    """Distribution the reference samples from, float64 [V]."""
    x = scaled(logits_row, temperature, dtype).astype(np.float64)
    V = x.size
    if top_k > 0:
        k = min(top_k, V)
        kth = np.sort(x)[::-1][k - 1]
        x = np.where(x < kth, -np.inf, x)
    if top_p < 1.0:
        order = np.argsort(-x, kind="stable")
        sx = x[order]
        e = np.exp(sx - sx[0])
        cum = np.cumsum(e / e.sum())
        remove = cum > top_p
        remove[1:] = remove[:-1].copy()
        remove[0] = False
        rm = np.zeros(V, dtype=bool)
        rm[order] = remove
        x = np.where(rm, -np.inf, x)
    e = np.exp(x - x.max())
    return e / e.sum()


def nucleus_margin(logits_row, temperature, top_k, top_p, dtype="f32") -> np.ndarray:
    """|mass before an entry - top_p| for every entry that survives top-k (inf elsewhere):
    entries with a tiny margin may legitimately fall on either side in float arithmetic."""
    x = scaled(logits_row, temperature, dtype).astype(np.float64)
    V = x.size
    if top_k > 0:
        kth = np.sort(x)[::-1][min(top_k, V) - 1]
        x = np.where(x < kth, -np.inf, x)
    order = np.argsort(-x, kind="stable")
    e = np.exp(x[order] - x[order][0])
    p = e / e.sum()
    before = np.concatenate([[0.0], np.cumsum(p)[:-1]])
    out = np.full(V, np.inf)
    out[order] = np.where(np.isfinite(x[order]), np.abs(before - top_p), np.inf)
    out[order[0]] = np.inf                  # the first entry stays whatever top_p is
    return out


def draw(probs: np.ndarray, u: float) -> int:
    """Inverse CDF in index order: the first index whose cumulative probability exceeds u."""
    cdf = np.cumsum(probs)
    return int(min(np.searchsorted(cdf, u * cdf[-1], side="right"), probs.size - 1))


def greedy(logits_row: np.ndarray) -> int:
    return int(np.argmax(np.asarray(logits_row, dtype=np.float32)))
