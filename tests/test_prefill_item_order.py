"""The closed form the prefill kernel uses to rank (chunk, query tile) items by cost
(aicomp_amd/csrc/prefill_mfma.hip, "Which item this workgroup takes"), restated in Python and
checked against a plain sort: every item gets a distinct rank, dearer items first, ties in item
order.  The kernel's own use of it is covered by the GPU prefill tests (every row computed once)."""
import random


def cost(n, ctx, q, p, kt):
    """Tile steps of query tile q (p positions) of a chunk of n new tokens ending at context ctx."""
    prior = ctx - n
    if n <= 0 or prior < 0 or q * p >= n:
        return 0
    return (min(ctx, prior + (q + 1) * p) + kt - 1) // kt


def ranks_by_sort(chunks, p, kt, ntile):
    items = [(cost(n, ctx, q, p, kt), s * ntile + q) for s, (n, ctx) in enumerate(chunks) for q in range(ntile)]
    order = sorted(items, key=lambda x: (-x[0], x[1]))
    rank = {idx: r for r, (_, idx) in enumerate(order)}
    return [rank[i] for i in range(len(items))]


def ranks_closed_form(chunks, p, kt, ntile):
    shift = p.bit_length() - 1
    assert 1 << shift == p
    tiles = [min(ntile, (n + p - 1) // p) if (n > 0 and ctx >= n) else 0 for n, ctx in chunks]

    def count_ge(s, c):      # tiles of chunk s that cost at least c steps (c >= 1)
        n, ctx = chunks[s]
        x = (c - 1) * kt
        if tiles[s] == 0 or ctx <= x:
            return 0
        prior = ctx - n
        return max(0, tiles[s] - (0 if x < prior else (x - prior) >> shift))

    out = []
    for s, (n, ctx) in enumerate(chunks):
        for q in range(ntile):
            work = q < tiles[s]
            c = cost(n, ctx, q, p, kt) if work else 0
            dearer = equal_before = all_work = idle_before = 0
            for s2 in range(len(chunks)):
                ge1, ge0 = count_ge(s2, c + 1), count_ge(s2, max(c, 1))
                dearer += ge1
                if s2 < s:
                    equal_before += ge0 - ge1
                    idle_before += ntile - tiles[s2]
                if s2 == s:
                    equal_before += q - (tiles[s2] - ge0)
                all_work += tiles[s2]
            out.append(dearer + equal_before if work else all_work + idle_before + (q - tiles[s]))
    return out


def test_closed_form_rank_equals_sort():
    rng = random.Random(1)
    for _ in range(3000):
        nseq = rng.randint(2, 7)
        p, kt = rng.choice([4, 8, 16, 32, 64, 128]), rng.choice([32, 64])
        chunks = []
        for _ in range(nseq):
            n = rng.choice([0, 1, rng.randint(1, 300), rng.randint(1, 40)])
            prior = rng.choice([0, rng.randint(0, 500), rng.randint(0, 50)])
            ctx = n + prior if rng.random() < 0.95 else max(0, n - rng.randint(1, 5))     # a few inconsistent ones
            chunks.append((n, ctx))
        ntile = max(1, max((n + p - 1) // p for n, _ in chunks))
        got = ranks_closed_form(chunks, p, kt, ntile)
        assert got == ranks_by_sort(chunks, p, kt, ntile), (chunks, p, kt)
        assert sorted(got) == list(range(nseq * ntile))


def test_dispatch_places_pair_long_with_short():
    """Odd rounds of the dispatch order are reversed, so the two items that share a CU from the
    start (place i and place i + per_round) have ranks i and 2 * per_round - 1 - i."""
    per_round, items = 32, 64
    want = []
    for place in range(items):
        rnd, pos = divmod(place, per_round)
        cnt = min(per_round, items - rnd * per_round)
        want.append(rnd * per_round + (cnt - 1 - pos) if rnd & 1 else place)
    assert sorted(want) == list(range(items))
    assert all(want[i] + want[i + per_round] == 2 * per_round - 1 for i in range(per_round))
