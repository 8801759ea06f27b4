"""CPU oracle for the paged KV-cache attention path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package may import this module: it is the checker that
tests, the smoke entry and the bench's cpu_baseline leg compare the HIP path
against.  It is plain numpy (float64 arithmetic, integer bit manipulation for
bf16 / fp8) with pure-Python loops for the byte-copy parts.

What it restates, and from where
--------------------------------
* ``kv_append``          - the slice-assign append of the reference cache,
  ``opt_prime/opt_prime/kv_cache.py:159-160`` (manager mode) and ``:387-388``
  (internal mode): ``cache[:, :, pos:end, :] = new``.  In paged form the
  destination row of token t is ``pool[slot // BS, :, slot % BS, :]``.
* ``paged_decode_attn``  - the decode branch ``kv_cache.py:397-403``:
  ``scaled_dot_product_attention(q, full_k, full_v, attn_mask=None,
  is_causal=False)`` over the whole cached prefix.
* ``paged_prefill_attn`` - the prefill branch ``kv_cache.py:404-415``:
  the same call with ``is_causal=True`` (Lq == Lk there).  For a chunk that
  starts at a prior context P > 0 the mask is bottom-right aligned (query i
  sees keys j <= P + i); at P == 0 this is the reference's mask, at chunk
  length 1 it is the reference's decode.  The reference itself applies no
  mask for P > 0 (``kv_cache.py:363,397-403``), which it never exercises.
* ``repeat_kv_index``    - the head order of HF Llama's ``repeat_kv``
  (``compiler_fx/modeling_llama.py:268-277``): query head h reads KV head
  h // G.

The softmax(QK^T*scale)V arithmetic itself lives in PyTorch, not in the
reference's sources (third-party: torch, "PyTorch >= 2.0.1, officially tested
2.5.0", ``opt_prime/README.md:45``; no lockfile).  The reference has no tests
for this path, so there are no golden vectors to inherit:

PARITY PINNING STATUS
* kv_append: pinned (closed form: a copy; brute-force loop, gather round trip,
  sentinel check, and a golden trace written from the reference's own
  ``kv_cache.py`` state machine, see tests/golden/).
* attention arithmetic: pinned by the mathematics (textbook formula in
  float64, invariants: weights sum to one, L == 1 returns the V row, equal
  keys give the mean of V, shift invariance, split-K merge identity, brute
  force on tiny shapes) and by torch's CPU ``scaled_dot_product_attention``
  as an independent library routine.  Against the reference's *own tests* it
  is "parity unpinned": none exist for this path.
* fp8 e4m3 (not in the reference): pinned against torch's ``float8_e4m3fn``
  cast over all 256 codes and on random data.
* bf16 / fp16 codecs: pinned against torch's casts over all 65 536 codes (decode) and on
  random data, ties, overflow and subnormals (encode).
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import numpy as np

# --------------------------------------------------------------------------
# Number formats (bit-level, so that "bit-exact" means something on the CPU)
# --------------------------------------------------------------------------


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    """uint16 bfloat16 codes -> float32 (exact)."""
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> uint16 bfloat16 codes, round-to-nearest-even, NaN kept quiet."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = (u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    nan = np.isnan(x)
    out = rounded.astype(np.uint16)
    out[nan] = ((u[nan] >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16)
    return out


def f16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    """uint16 IEEE binary16 codes -> float32 (exact): 1 sign, 5 exponent (bias 15), 10 mantissa;
    exponent 0 is subnormal (m * 2^-24), exponent 31 is inf / NaN."""
    b = np.asarray(bits, dtype=np.uint16).astype(np.int64)
    sign = np.where(b & 0x8000, -1.0, 1.0)
    e = (b >> 10) & 0x1F
    m = b & 0x3FF
    with np.errstate(invalid="ignore"):
        v = np.where(e == 0, m * 2.0 ** -24, (1.0 + m / 1024.0) * np.exp2((e - 15).astype(np.float64)))
        v = np.where(e == 31, np.where(m == 0, np.inf, np.nan), v)
    return (sign * v).astype(np.float32)


def f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> uint16 binary16 codes, round to nearest even, overflow to infinity (numpy's
    conversion; pinned against torch's cast in the tests)."""
    with np.errstate(over="ignore"):
        return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def e4m3_code_table() -> np.ndarray:
    """All 256 OCP fp8 e4m3 ("e4m3fn") codes as float32.

    1 sign, 4 exponent (bias 7), 3 mantissa; no infinities; S.1111.111 is NaN;
    exponent 0 is subnormal: value = 2^-6 * m/8.  Maximum finite value 448.
    """
    t = np.zeros(256, dtype=np.float32)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e = (c >> 3) & 0xF
        m = c & 0x7
        if e == 0xF and m == 0x7:
            v = float("nan")
        elif e == 0:
            v = s * (m / 8.0) * 2.0 ** -6
        else:
            v = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        t[c] = v
    return t


_E4M3 = e4m3_code_table()


def e4m3_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return _E4M3[np.asarray(bits, dtype=np.uint8)]


def f32_to_e4m3_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> e4m3 codes: saturate to +-448, round to nearest even.

    Brute force over the 127 non-negative finite codes (monotone table), so a
    mistake in a closed-form rounding rule cannot hide here.
    """
    x = np.asarray(x, dtype=np.float32)
    mag = np.minimum(np.abs(x).astype(np.float64), 448.0)
    pos = _E4M3[:127].astype(np.float64)  # codes 0..126 ascending, 126 -> 448
    hi = np.searchsorted(pos, mag, side="left")  # first code with value >= mag
    hi = np.clip(hi, 0, 126)
    lo = np.clip(hi - 1, 0, 126)
    d_hi = np.abs(pos[hi] - mag)
    d_lo = np.abs(mag - pos[lo])
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & (lo % 2 == 0))
    code = np.where(pick_lo, lo, hi).astype(np.uint8)
    sign = (np.signbit(x)).astype(np.uint8) << 7
    out = code | sign
    out = np.where(np.isnan(x), np.uint8(0x7F), out).astype(np.uint8)
    return out


def decode_elements(raw: np.ndarray, dtype: str) -> np.ndarray:
    """Raw storage array -> float64 values.  dtype in {"f32","bf16","f16","fp8"}."""
    if dtype == "f32":
        return np.asarray(raw, dtype=np.float32).astype(np.float64)
    if dtype == "bf16":
        return bf16_bits_to_f32(raw).astype(np.float64)
    if dtype == "f16":
        return f16_bits_to_f32(raw).astype(np.float64)
    if dtype == "fp8":
        return e4m3_bits_to_f32(raw).astype(np.float64)
    raise ValueError(dtype)


# --------------------------------------------------------------------------
# Paged layout helpers
# --------------------------------------------------------------------------


def slot_of(block_table_row: Sequence[int], t: int, block_size: int) -> int:
    """Physical slot of logical token t: table[t // BS] * BS + t % BS."""
    return int(block_table_row[t // block_size]) * block_size + t % block_size


def gather_context(pool: np.ndarray, block_table_row: Sequence[int], length: int) -> np.ndarray:
    """pool [num_blocks, Hkv, BS, D] -> contiguous [length, Hkv, D] (any dtype).

    The inverse of the append: it rebuilds the ``[:, :, :end, :]`` prefix view
    that ``kv_cache.py:167-170`` hands to the attention call.
    """
    nb, hkv, bs, d = pool.shape
    out = np.empty((length, hkv, d), dtype=pool.dtype)
    for t in range(length):
        blk = int(block_table_row[t // bs])
        out[t] = pool[blk, :, t % bs, :]
    return out


def gather_context_fast(pool: np.ndarray, block_table_row: Sequence[int], length: int) -> np.ndarray:
    """``gather_context`` as one fancy-indexing expression, for full-size batches (tens of
    thousands of tokens per sequence); checked element for element against the token loop above."""
    bs = pool.shape[2]
    t = np.arange(length)
    blk = np.asarray(block_table_row, dtype=np.int64)[t // bs]
    return np.ascontiguousarray(pool[blk, :, t % bs, :])


def repeat_kv_index(num_q_heads: int, num_kv_heads: int) -> np.ndarray:
    """KV head read by each query head (modeling_llama.py:268-277)."""
    g = num_q_heads // num_kv_heads
    return np.arange(num_q_heads) // g


# --------------------------------------------------------------------------
# KV append
# --------------------------------------------------------------------------


def kv_append(
    key: np.ndarray,
    value: np.ndarray,
    k_pool: np.ndarray,
    v_pool: np.ndarray,
    slot_mapping: Sequence[int],
    k_scale: Optional[np.ndarray] = None,
    v_scale: Optional[np.ndarray] = None,
    pool_dtype: Optional[str] = None,
    in_dtype: Optional[str] = None,
) -> None:
    """Scatter new rows key/value [T, Hkv, D] into the pools, in place.

    Same storage type in and out: a raw copy (bit-exact by construction), as
    in ``kv_cache.py:159-160``.  With an fp8 pool the row is quantised:
    code = e4m3(clamp(float32(x) / scale[h], +-448)) with IEEE float32 division.
    Slots < 0 are skipped (padding).
    """
    nb, hkv, bs, d = k_pool.shape
    quant = pool_dtype == "fp8" and in_dtype != "fp8"
    for t, slot in enumerate(slot_mapping):
        slot = int(slot)
        if slot < 0:
            continue
        blk, off = divmod(slot, bs)
        for h in range(hkv):
            if quant:
                kx = decode_elements(key[t, h], in_dtype).astype(np.float32)
                vx = decode_elements(value[t, h], in_dtype).astype(np.float32)
                k_pool[blk, h, off, :] = f32_to_e4m3_bits(kx / np.float32(k_scale[h]))
                v_pool[blk, h, off, :] = f32_to_e4m3_bits(vx / np.float32(v_scale[h]))
            else:
                for j in range(d):  # brute-force element copy
                    k_pool[blk, h, off, j] = key[t, h, j]
                    v_pool[blk, h, off, j] = value[t, h, j]


def kv_append_fast(key, value, k_pool, v_pool, slot_mapping) -> None:
    """Vectorised raw-copy append for large cases (checked against kv_append)."""
    bs = k_pool.shape[2]
    sm = np.asarray(slot_mapping, dtype=np.int64)
    keep = sm >= 0
    blk = sm[keep] // bs
    off = sm[keep] % bs
    k_pool[blk, :, off, :] = key[keep]
    v_pool[blk, :, off, :] = value[keep]


# --------------------------------------------------------------------------
# Attention
# --------------------------------------------------------------------------


def _softmax_rows(s: np.ndarray) -> np.ndarray:
    m = np.max(s, axis=-1, keepdims=True)
    p = np.exp(s - m)
    return p / np.sum(p, axis=-1, keepdims=True)


def attend_contiguous(
    q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, prior: Optional[int] = None
) -> np.ndarray:
    """Textbook attention in float64 on one sequence.

    q [n, Hq, D]; k, v [L, Hkv, D]; returns [n, Hq, D].
    prior is None  -> no mask (decode, kv_cache.py:400-403).
    prior = P >= 0 -> query i sees keys j <= P + i (L == P + n); P == 0 is the
                      reference's ``is_causal=True`` prefill (kv_cache.py:412-415).
    """
    n, hq, d = q.shape
    L, hkv, _ = k.shape
    kvh = repeat_kv_index(hq, hkv)
    out = np.empty((n, hq, d), dtype=np.float64)
    for h in range(hq):
        s = (q[:, h, :] @ k[:, kvh[h], :].T) * scale  # [n, L]
        if prior is not None:
            j = np.arange(L)[None, :]
            i = np.arange(n)[:, None]
            s = np.where(j <= prior + i, s, -np.inf)
        out[:, h, :] = _softmax_rows(s) @ v[:, kvh[h], :]
    return out


def paged_decode_attn(
    query: np.ndarray,
    k_pool: np.ndarray,
    v_pool: np.ndarray,
    block_table: np.ndarray,
    context_lens: Sequence[int],
    scale: float,
    q_dtype: str = "f32",
    kv_dtype: str = "f32",
    k_scale: Optional[np.ndarray] = None,
    v_scale: Optional[np.ndarray] = None,
    gather=gather_context,
) -> np.ndarray:
    """query [B, Hq, D] raw -> float64 [B, Hq, D].  One new token per sequence.

    A sequence with context length 0 yields zeros (nothing to attend to).  ``gather`` is the
    routine that rebuilds a sequence's contiguous prefix (the token loop, or its vectorised twin).
    """
    B, hq, d = query.shape
    out = np.zeros((B, hq, d), dtype=np.float64)
    qf = decode_elements(query, q_dtype)
    for b in range(B):
        L = int(context_lens[b])
        if L == 0:
            continue
        k = decode_elements(gather(k_pool, block_table[b], L), kv_dtype)
        v = decode_elements(gather(v_pool, block_table[b], L), kv_dtype)
        if k_scale is not None:
            k = k * np.asarray(k_scale, dtype=np.float32).astype(np.float64)[None, :, None]
        if v_scale is not None:
            v = v * np.asarray(v_scale, dtype=np.float32).astype(np.float64)[None, :, None]
        out[b] = attend_contiguous(qf[b][None], k, v, scale, prior=None)[0]
    return out


def paged_prefill_attn(
    query: np.ndarray,
    k_pool: np.ndarray,
    v_pool: np.ndarray,
    block_table: np.ndarray,
    context_lens: Sequence[int],
    cu_q_lens: Sequence[int],
    scale: float,
    q_dtype: str = "f32",
    kv_dtype: str = "f32",
    k_scale: Optional[np.ndarray] = None,
    v_scale: Optional[np.ndarray] = None,
    gather=gather_context,
) -> np.ndarray:
    """query [T, Hq, D] raw (chunks concatenated) -> float64 [T, Hq, D].

    Sequence s owns rows cu_q_lens[s]:cu_q_lens[s+1]; its context (prior +
    chunk, chunk rows already appended) has context_lens[s] tokens.
    """
    T, hq, d = query.shape
    out = np.zeros((T, hq, d), dtype=np.float64)
    qf = decode_elements(query, q_dtype)
    for s in range(len(context_lens)):
        r0, r1 = int(cu_q_lens[s]), int(cu_q_lens[s + 1])
        n = r1 - r0
        L = int(context_lens[s])
        if n == 0:
            continue
        k = decode_elements(gather(k_pool, block_table[s], L), kv_dtype)
        v = decode_elements(gather(v_pool, block_table[s], L), kv_dtype)
        if k_scale is not None:
            k = k * np.asarray(k_scale, dtype=np.float32).astype(np.float64)[None, :, None]
        if v_scale is not None:
            v = v * np.asarray(v_scale, dtype=np.float32).astype(np.float64)[None, :, None]
        out[r0:r1] = attend_contiguous(qf[r0:r1], k, v, scale, prior=L - n)
    return out


def attend_bruteforce(q, k, v, scale, prior=None):
    """Scalar-loop attention for tiny shapes; independent of attend_contiguous."""
    n, hq, d = q.shape
    L, hkv, _ = k.shape
    g = hq // hkv
    out = [[[0.0] * d for _ in range(hq)] for _ in range(n)]
    for i in range(n):
        for h in range(hq):
            hk = h // g
            last = L - 1 if prior is None else min(L - 1, prior + i)
            sc = []
            for j in range(last + 1):
                acc = 0.0
                for c in range(d):
                    acc += float(q[i, h, c]) * float(k[j, hk, c])
                sc.append(acc * scale)
            mx = max(sc)
            w = [math.exp(x - mx) for x in sc]
            z = sum(w)
            for c in range(d):
                acc = 0.0
                for j in range(last + 1):
                    acc += w[j] * float(v[j, hk, c])
                out[i][h][c] = acc / z
    return np.array(out, dtype=np.float64)


# --------------------------------------------------------------------------
# Split-K (flash-decoding) merge: closed form
# --------------------------------------------------------------------------


def partition_partial(q, k, v, scale) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """One partition's (m, l, o): row max, sum of exp, normalised output.

    q [Hq, D]; k, v [Lp, Hkv, D].  An empty partition gives (-inf, 0, 0).
    """
    hq, d = q.shape
    Lp, hkv, _ = k.shape
    kvh = repeat_kv_index(hq, hkv)
    m = np.full(hq, -np.inf)
    l = np.zeros(hq)
    o = np.zeros((hq, d))
    if Lp == 0:
        return m, l, o
    for h in range(hq):
        s = (k[:, kvh[h], :] @ q[h]) * scale
        m[h] = s.max()
        p = np.exp(s - m[h])
        l[h] = p.sum()
        o[h] = (p @ v[:, kvh[h], :]) / l[h]
    return m, l, o


def splitk_merge(ms, ls, os_) -> np.ndarray:
    """out = sum_p e^{m_p-m} l_p o_p / sum_p e^{m_p-m} l_p, m = max_p m_p."""
    ms = np.stack(ms)  # [P, Hq]
    ls = np.stack(ls)
    os_ = np.stack(os_)  # [P, Hq, D]
    m = ms.max(axis=0)
    w = np.where(np.isfinite(ms), np.exp(ms - m[None]), 0.0) * ls
    return (w[:, :, None] * os_).sum(axis=0) / w.sum(axis=0)[:, None]


# --------------------------------------------------------------------------
# fp8 KV scales
# --------------------------------------------------------------------------


def absmax_scales(x: np.ndarray) -> np.ndarray:
    """Per-KV-head float32 scale = absmax / 448 over x [T, Hkv, D] (float)."""
    amax = np.abs(np.asarray(x, dtype=np.float32)).max(axis=(0, 2))
    return (amax / np.float32(448.0)).astype(np.float32)
