"""CPU oracle for rotary position embedding + KV append.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package may import this module.

What it restates, and from where
--------------------------------
* ``rope_tables``    - the cos/sin the reference's rotary module produces
  (``compiler_fx/modeling_llama.py:150-168``): ``freqs = position * inv_freq``
  in float32, ``emb = cat(freqs, freqs)``, ``cos(emb) * attention_scaling``,
  cast to the tensor type.  ``default_inv_freq`` is the "default" rope
  initialisation ``1 / base^(2i/D)`` (transformers' ROPE_INIT_FUNCTIONS, a
  third-party dependency of the reference: "transformers 4.46.2",
  ``opt_prime/README.md:47,51``; 5.15.0 is what is installed here).
* ``apply_rope``     - ``rotate_half`` and ``apply_rotary_pos_emb``
  (``compiler_fx/modeling_llama.py:200-231``):
  ``x_embed = (x * cos) + (rotate_half(x) * sin)`` evaluated the way eager
  PyTorch evaluates it in the tensor's own type: every product is rounded to
  that type, then the sum is rounded (no fused multiply-add).  bf16 is handled
  at bit level, float32 with numpy's float32 arithmetic.
* ``rope_kv_append`` - rotation of Q and K followed by the slice-assign append
  (``opt_prime/opt_prime/kv_cache.py:387-388``) of the rotated K and of V
  through ``slot_mapping`` (brute-force loop over rows), optionally quantised
  to e4m3 exactly like ``paged_kv_oracle.kv_append``.

PARITY PINNING STATUS
* apply_rope: pinned.  (i) float64 closed form: each pair (x[j], x[j+D/2]) is
  the complex number x[j] + i x[j+D/2] multiplied by e^{i theta_j}
  (``rope_exact``, written independently with numpy complex arithmetic);
  (ii) invariants: pair norms preserved, position 0 is the identity, scores
  q(m).k(n) depend on m - n only; (iii) the rounding order, bit for bit,
  against ``transformers.models.llama.modeling_llama.apply_rotary_pos_emb``
  run by torch's CPU bf16 / fp32 eager kernels (a library routine with the
  same text as the reference's copy).  The reference's own tests hold no
  vectors for it.
* rope_tables: pinned against float64 cos/sin (within one unit in the last
  place of the tensor type) and, bit for bit, against transformers'
  ``LlamaRotaryEmbedding`` on CPU.
* rope_kv_append: the append part is the already pinned copy.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import numpy as np

from . import paged_kv_oracle as P


def default_inv_freq(head_dim: int, base: float = 10000.0) -> np.ndarray:
    """1 / base^(2i/D), i = 0 .. D/2-1 (the "default" rope type), evaluated in float64 and
    rounded to float32: within one unit in the last place of a float32 powf.  The frequencies
    are a model buffer, i.e. an input of the path, so this only feeds test data."""
    i = np.arange(0, head_dim, 2, dtype=np.float64)
    return (1.0 / (float(base) ** (i / head_dim))).astype(np.float32)


def rope_angles(inv_freq: np.ndarray, positions: Sequence[int]) -> np.ndarray:
    """theta[p, j] = position_p * inv_freq[j] as float32 products, [P, D/2]."""
    pos = np.asarray(positions, dtype=np.float32)
    return (pos[:, None] * np.asarray(inv_freq, dtype=np.float32)[None, :]).astype(np.float32)


def _to_type(x32: np.ndarray, dtype: str) -> np.ndarray:
    """float32 values -> storage codes of ``dtype`` ("f32": float32, "bf16" / "f16": uint16 bits)."""
    if dtype == "f32":
        return x32.astype(np.float32)
    if dtype == "bf16":
        return P.f32_to_bf16_bits(x32.astype(np.float32))
    if dtype == "f16":
        return P.f32_to_f16_bits(x32.astype(np.float32))
    raise ValueError(dtype)


def _to_f32(raw: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "f32":
        return np.asarray(raw, dtype=np.float32)
    if dtype == "bf16":
        return P.bf16_bits_to_f32(np.asarray(raw, dtype=np.uint16))
    if dtype == "f16":
        return P.f16_bits_to_f32(np.asarray(raw, dtype=np.uint16))
    raise ValueError(dtype)


def rope_tables(inv_freq: np.ndarray, num_positions: int, dtype: str,
                attention_scaling: float = 1.0) -> Tuple[np.ndarray, np.ndarray]:
    """cos, sin tables [num_positions, D] as storage codes of ``dtype``.

    cos/sin are evaluated in float64 on the float32 angle and rounded to float32, which can
    differ from a float32 libm by one unit in the last place; tests allow for that.
    """
    th = rope_angles(inv_freq, np.arange(num_positions))
    emb = np.concatenate([th, th], axis=-1).astype(np.float64)
    cos = (np.cos(emb).astype(np.float32) * np.float32(attention_scaling)).astype(np.float32)
    sin = (np.sin(emb).astype(np.float32) * np.float32(attention_scaling)).astype(np.float32)
    return _to_type(cos, dtype), _to_type(sin, dtype)


def rotate_half(x: np.ndarray) -> np.ndarray:
    """(-x2, x1) for x = (x1, x2) split at D/2 (modeling_llama.py:200-204)."""
    h = x.shape[-1] // 2
    return np.concatenate([-x[..., h:], x[..., :h]], axis=-1)


def apply_rope(x_raw: np.ndarray, cos_raw: np.ndarray, sin_raw: np.ndarray, dtype: str) -> np.ndarray:
    """``(x * cos) + (rotate_half(x) * sin)`` with eager per-operation rounding.

    x_raw [..., D] storage codes; cos_raw / sin_raw broadcastable to it.  Returns codes.
    """
    x = _to_f32(x_raw, dtype)
    c = _to_f32(cos_raw, dtype)
    s = _to_f32(sin_raw, dtype)
    rnd = lambda v: _to_f32(_to_type(v, dtype), dtype)
    p1 = rnd(x * c)                       # float32 product of two bf16 values is exact before rounding
    p2 = rnd(rotate_half(x) * s)
    return _to_type((p1 + p2).astype(np.float32), dtype)


def rope_exact(x: np.ndarray, theta: np.ndarray) -> np.ndarray:
    """float64 rotation by complex multiplication: (x1 + i x2) e^{i theta}, theta [..., D/2]."""
    h = x.shape[-1] // 2
    z = (x[..., :h].astype(np.float64) + 1j * x[..., h:].astype(np.float64)) * np.exp(1j * theta.astype(np.float64))
    return np.concatenate([z.real, z.imag], axis=-1)


def rope_kv_append(q_raw: np.ndarray, k_raw: np.ndarray, v_raw: np.ndarray, cos_tab: np.ndarray,
                   sin_tab: np.ndarray, positions: Optional[Sequence[int]], k_pool: np.ndarray,
                   v_pool: np.ndarray, slot_mapping: Sequence[int], dtype: str,
                   k_scale: Optional[np.ndarray] = None, v_scale: Optional[np.ndarray] = None,
                   pool_dtype: Optional[str] = None) -> np.ndarray:
    """Rotate q [T,Hq,D] and k [T,Hkv,D]; append rotated k and v into the pools (in place).

    Returns the rotated q codes.  Tokens whose position has no table row are left alone
    (q returned unchanged, nothing appended), as the kernel documents.
    """
    T = q_raw.shape[0]
    pos = np.arange(T) if positions is None else np.asarray(positions, dtype=np.int64)
    ok = (pos >= 0) & (pos < cos_tab.shape[0])
    safe = np.where(ok, pos, 0)
    cos = cos_tab[safe][:, None, :]
    sin = sin_tab[safe][:, None, :]
    q_rot = apply_rope(q_raw, cos, sin, dtype)
    k_rot = apply_rope(k_raw, cos, sin, dtype)
    q_out = np.where(ok[:, None, None], q_rot, q_raw)
    slots = np.where(ok, np.asarray(slot_mapping, dtype=np.int64), -1)
    P.kv_append(k_rot, v_raw, k_pool, v_pool, slots, k_scale, v_scale,
                pool_dtype=pool_dtype or dtype, in_dtype=dtype)
    return q_out
