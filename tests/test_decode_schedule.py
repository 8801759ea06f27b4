"""Host-side model of the balanced decode schedule (aicomp_amd/csrc/decode_mfma.hip,
streamk_decode_kernel / streamk_reduce_kernel): which tiles each wave takes, where it puts its
partials and how the merge finds them.  The kernel itself is checked against the oracle on the
GPU; this file checks what the launch relies on and no output comparison would show until it
breaks: every tile of every (sequence, KV head) row is taken exactly once, no two partials share
a scratch slot, a row's partials sit in consecutive slots from first + sequence to last +
sequence of its head's region, and every slot lies inside the scratch size the library asks for
(the reference has no counterpart: its decode is one SDPA call per step, kv_cache.py:397-403).
"""
import random

import pytest

TILE, BS = 32, 16
SK_MAX_WAVES = 4096


def tiles_of(length, max_blocks, tile=TILE):
    """Tiles of a row: 32 tokens at head_dim 128, 64 tokens (32 pair rows) at head_dim 64."""
    length = min(max(length, 0), max_blocks * BS)
    return (length + tile - 1) // tile


def schedule(context_lens, hkv, num_waves, max_blocks, tile=TILE):
    """-> (segments, head_slots): segments are (kvh, part, seq, first_tile, n_tiles, slot)."""
    B = len(context_lens)
    wph = num_waves // hkv
    prefix = [0]
    for c in context_lens:
        prefix.append(prefix[-1] + tiles_of(c, max_blocks, tile))
    N = prefix[B]
    W = min(wph, N)
    head_slots = wph + B
    segs = []
    for wave in range(num_waves):
        kvh, part = wave % hkv, wave // hkv
        if part >= W:
            continue
        g0, g1 = part * N // W, (part + 1) * N // W
        lo, hi = 0, B                      # prefix[lo] <= g0 < prefix[hi]
        while hi - lo > 1:
            mid = (lo + hi) // 2
            if prefix[mid] <= g0:
                lo = mid
            else:
                hi = mid
        seq, g = lo, g0
        t = g0 - prefix[seq]
        while g < g1 and seq < B:
            row_tiles = prefix[seq + 1] - prefix[seq]
            nt = min(row_tiles - t, g1 - g)
            assert nt >= 1
            segs.append((kvh, part, seq, t, nt, kvh * head_slots + part + seq))
            g += nt
            if g >= g1:
                break
            seq += 1
            while seq < B and prefix[seq + 1] == prefix[seq]:
                seq += 1
            t = 0
    return segs, head_slots


def check(context_lens, hkv, num_waves, max_blocks, tile=TILE):
    B = len(context_lens)
    segs, head_slots = schedule(context_lens, hkv, num_waves, max_blocks, tile)
    # the scratch the library asks for: SK_MAX_WAVES + rows * hkv slots
    limit = SK_MAX_WAVES + B * hkv
    slots = [s[5] for s in segs]
    assert len(set(slots)) == len(slots), "two partials in one slot"
    assert all(0 <= s < limit for s in slots), "slot outside the scratch"
    rows = {}
    for kvh, part, seq, t, nt, slot in segs:
        rows.setdefault((seq, kvh), []).append((t, nt, part, slot))
    for seq in range(B):
        want = tiles_of(context_lens[seq], max_blocks, tile)
        for kvh in range(hkv):
            got = sorted(rows.get((seq, kvh), []))
            if want == 0:
                assert not got
                continue
            # tiles 0 .. want-1 exactly once, in part order
            pos = 0
            for t, nt, part, slot in got:
                assert t == pos
                pos += nt
            assert pos == want
            parts = [g[2] for g in got]
            first, last = parts[0], parts[-1]          # what the main kernel records for the merge
            assert parts == list(range(first, last + 1))
            assert [g[3] for g in got] == [kvh * head_slots + first + seq + i for i in range(len(got))]


@pytest.mark.parametrize("seed", range(6))
def test_random_batches(seed):
    rnd = random.Random(seed)
    for _ in range(60):
        hkv = rnd.choice([1, 2, 3, 4, 5, 8, 12, 16, 64, 256])
        B = rnd.choice([1, 2, 3, 7, 64, 65, 200, 1024])
        max_blocks = rnd.choice([1, 4, 64, 512])
        kind = rnd.random()
        if kind < 0.2:
            lens = [rnd.choice([0, 1, 31, 32, 33]) for _ in range(B)]
        elif kind < 0.4:
            lens = [rnd.randint(0, max_blocks * BS + 40) for _ in range(B)]     # some beyond the table
        else:
            lens = [rnd.randint(1, max_blocks * BS) for _ in range(B)]
        check(lens, hkv, 1024, max_blocks, rnd.choice([32, 64]))


def test_corner_cases():
    check([0] * 5, 8, 1024, 16)                         # nothing to do
    check([1], 8, 1024, 16)                             # one tile, one wave per head
    check([0, 0, 5000, 0, 1, 0], 8, 1024, 512)          # empty sequences between long ones
    check([32 * 128] * 1, 8, 1024, 256)                 # exactly one tile per wave of a head
    check([32 * 129] * 1, 8, 1024, 512)                 # one tile more than waves
    check([8192] * 64, 8, 1024, 512)
    check([100] * 1024, 256, 1024, 8)                   # four waves per head, 1024 rows
    check([100] * 1024, 3, 1024, 8)                     # waves left over (1024 = 3 * 341 + 1)
    check([17] * 10, 8, 4096, 2)                        # the largest launch the scratch is sized for
    check([0, 63, 64, 65, 4096], 8, 1024, 256, tile=64)  # head_dim 64: tiles of 64 tokens
