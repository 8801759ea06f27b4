"""Block allocator and step planner (host logic, CPU only).

The planner's index tensors are checked the way the append itself is pinned: writing
each token's signature into a numpy pool through ``slot_mapping`` (the oracle's brute
force append) and gathering it back through ``block_table`` must reproduce every
sequence's history bit for bit, whatever the interleaving of arrivals, chunks,
finishes and preemptions.
"""
import numpy as np
import pytest

from aicomp_amd.block_manager import (BlockAllocator, OutOfBlocks, StepPlanner,
                                      pool_blocks_for_budget)
from oracle import paged_kv_oracle as O

BS = 16


# ------------------------------------------------------------------ allocator
def test_allocator_basic_and_lifo():
    a = BlockAllocator(8, BS)
    assert a.num_free == 8 and a.num_used == 0
    x = a.allocate(3)
    assert x.tolist() == [0, 1, 2]
    y = a.allocate(2)
    assert y.tolist() == [3, 4]
    a.free(x)
    assert a.num_free == 6
    z = a.allocate(2)                     # most recently freed first
    assert set(z.tolist()) <= {0, 1, 2}
    assert a.num_used == 4


def test_allocator_all_or_nothing_and_errors():
    a = BlockAllocator(4, BS)
    a.allocate(3)
    with pytest.raises(OutOfBlocks):
        a.allocate(2)
    assert a.num_free == 1                # the failed request took nothing
    with pytest.raises(ValueError):
        a.free([3])                       # never allocated
    with pytest.raises(ValueError):
        a.free([0, 0])                    # duplicate in one call
    a.free([0])
    with pytest.raises(ValueError):
        a.free([0])                       # double free
    with pytest.raises(ValueError):
        a.free([9])
    with pytest.raises(ValueError):
        a.allocate(-1)
    with pytest.raises(ValueError):
        BlockAllocator(0)
    assert a.allocate(0).size == 0


def test_allocator_random_ownership():
    rng = np.random.default_rng(0)
    a = BlockAllocator(64, BS)
    held = []
    for _ in range(2000):
        if held and rng.random() < 0.5:
            i = rng.integers(len(held))
            a.free(held.pop(i))
        else:
            n = int(rng.integers(0, 9))
            if a.can_allocate(n):
                held.append(a.allocate(n))
            else:
                with pytest.raises(OutOfBlocks):
                    a.allocate(n)
        flat = np.concatenate(held) if held else np.zeros(0, dtype=np.int32)
        assert np.unique(flat).size == flat.size          # no block handed out twice
        assert a.num_used == flat.size and a.num_free == 64 - flat.size


def test_pool_blocks_for_budget():
    import torch
    # Llama-3-8B: 32 layers, 8 KV heads, D 128, bf16 -> 2*32*8*16*128*2 B = 2 MiB per block
    assert pool_blocks_for_budget(200 * 2**30, 32, 8, 128, torch.bfloat16) == 200 * 2**30 // (2 * 2**20)
    assert pool_blocks_for_budget(2**20, 1, 8, 128, torch.float8_e4m3fn) == 2**20 // (2 * 8 * 16 * 128)


# ------------------------------------------------------------------ planner, checked through the oracle
class Sim:
    """Drives a planner with random arrivals / finishes and replays every plan into numpy pools."""

    def __init__(self, planner, hkv=2, d=4, seed=0):
        self.p = planner
        self.rng = np.random.default_rng(seed)
        nb = planner.alloc.num_blocks
        self.k_pool = np.full((nb, hkv, BS, d), -1, dtype=np.int32)
        self.v_pool = np.full((nb, hkv, BS, d), -1, dtype=np.int32)
        self.hist = {}          # seq_id -> list of token signatures cached so far
        self.hkv, self.d = hkv, d
        self.sig = 0

    def token_rows(self, n):
        base = self.sig + np.arange(n, dtype=np.int32)
        self.sig += n
        k = np.broadcast_to((base * 2)[:, None, None], (n, self.hkv, self.d)).copy()
        k += np.arange(self.hkv, dtype=np.int32)[None, :, None] * 1000003
        return k, k + 1

    def apply(self, plan):
        p = self.p
        for sid in plan.preempted:
            self.hist.pop(sid, None)                 # it will be recomputed from scratch
        T = plan.total_new_tokens
        k, v = self.token_rows(T)
        cu = plan.host_cu_q_lens
        assert cu[0] == 0 and cu[-1] == T and (np.diff(cu) == plan.new_lens).all()
        sm = plan.host_slot_mapping
        assert np.unique(sm).size == T, "a slot is written twice in one step"
        assert (plan.new_lens[:plan.num_prefill_seqs] > 1).all() and (plan.new_lens[plan.num_prefill_seqs:] == 1).all()
        O.kv_append(k, v, self.k_pool, self.v_pool, sm)
        owners = {}
        for r, sid in enumerate(plan.seq_ids):
            h = self.hist.setdefault(sid, [])
            n = int(plan.new_lens[r])
            assert plan.host_context_lens[r] == len(h) + n
            for i in range(n):                       # brute-force slot formula
                t = len(h) + i
                assert sm[cu[r] + i] == O.slot_of(plan.host_block_table[r], t, BS)
                assert plan.host_positions[cu[r] + i] == t
            h.extend(k[cu[r]:cu[r] + n, 0, 0].tolist())
            L = len(h)
            assert p.context_len(sid) == L
            # gathering through the table reproduces the history bit for bit
            got = O.gather_context(self.k_pool, plan.host_block_table[r], L)
            assert (got[:, 0, 0] == np.asarray(h, dtype=np.int32)).all()
            gv = O.gather_context(self.v_pool, plan.host_block_table[r], L)
            assert (gv == got + 1).all()
            blocks = p.blocks_of(sid)
            assert len(blocks) == -(-L // BS)
            assert plan.host_block_table[r, :len(blocks)].tolist() == blocks
            for b in blocks:
                assert owners.setdefault(b, sid) == sid
        # device tensors (CPU here) hold the same values as the host copies
        assert (plan.block_table.numpy() == plan.host_block_table).all()
        assert (plan.context_lens.numpy() == plan.host_context_lens).all()
        assert (plan.cu_q_lens.numpy() == plan.host_cu_q_lens).all()
        assert (plan.slot_mapping.numpy() == plan.host_slot_mapping).all()
        assert (plan.positions.numpy() == plan.host_positions).all()
        # pool accounting over every running sequence
        used = set()
        for sid in list(p._row_of):
            b = p.blocks_of(sid)
            assert not (used & set(b)), "two sequences share a block"
            used |= set(b)
        assert len(used) == p.alloc.num_used


def test_planner_prefill_then_decode_matches_oracle():
    p = StepPlanner(check_plans=True, num_blocks=64, max_seqs=8, max_seq_len=256, max_num_batched_tokens=64,
                    prefill_chunk=24, device="cpu")
    sim = Sim(p)
    p.add_request("a", 50, 10)
    p.add_request("b", 17, 10)
    p.add_request("c", 1, 10)             # a one-token prompt is a decode row from the start
    plans = []
    for _ in range(12):
        plan = p.schedule()
        assert plan is not None
        assert plan.total_new_tokens <= 64 and (plan.new_lens <= 24).all()
        sim.apply(plan)
        plans.append(plan)
    # first step: a gets 24, b gets 17, c its single token (a decode row, placed after the chunks)
    assert plans[0].seq_ids == ["a", "b", "c"] and plans[0].new_lens.tolist() == [24, 17, 1]
    assert plans[0].num_prefill_seqs == 2 and plans[0].max_q_len == 24
    # a needs 24+24+2: the 2-token tail is still a chunk; afterwards every row is one token
    assert plans[1].new_lens.tolist()[:1] == [24] and plans[2].new_lens[0] == 2
    assert plans[3].num_prefill_seqs == 0 and sorted(plans[3].seq_ids) == ["a", "b", "c"]
    assert p.num_generated("b") == p.context_len("b") - 17 + 1


def test_planner_completed_and_finish_release_blocks():
    p = StepPlanner(num_blocks=16, max_seqs=4, max_seq_len=64, device="cpu")
    p.add_request(1, 20, 3)
    p.add_request(2, 5, 1)
    sim = Sim(p)
    sim.apply(p.schedule())                       # both prompts ingested, first tokens sampled
    assert p.completed() == [2]                   # max_new_tokens = 1 is reached by the prefill step
    p.finish(2)
    sim.apply(p.schedule())
    sim.apply(p.schedule())
    assert p.completed() == [1] and p.context_len(1) == 22
    assert p.schedule() is None                   # nothing left to run until the caller finishes it
    p.finish(1)
    assert p.alloc.num_used == 0 and not p.has_work()
    with pytest.raises(ValueError):
        p.finish(1)


def test_planner_errors():
    p = StepPlanner(num_blocks=4, max_seqs=2, max_seq_len=64, device="cpu")
    with pytest.raises(ValueError):
        p.add_request("x", 0)
    with pytest.raises(ValueError):
        p.add_request("x", 60, 10)                # longer than max_seq_len
    p.add_request("x", 10)
    with pytest.raises(ValueError):
        p.add_request("x", 10)                    # duplicate id while waiting
    p.schedule()
    with pytest.raises(ValueError):
        p.add_request("x", 10)                    # duplicate id while running
    with pytest.raises(ValueError):
        StepPlanner(num_blocks=4, max_seqs=0, device="cpu")
    q = StepPlanner(num_blocks=2, max_seqs=2, max_seq_len=64, device="cpu")
    with pytest.raises(ValueError):
        q.add_request("y", 40)                    # can never fit two blocks
    p.add_request("w", 5)
    p.finish("w")                                 # finishing a waiting request just drops it
    assert not p.waiting


def test_planner_max_seq_len_overflow_raises():
    p = StepPlanner(num_blocks=8, max_seqs=2, max_seq_len=20, device="cpu")
    p.add_request("s", 19)                        # unbounded generation
    p.schedule()
    p.schedule()                                  # 20 tokens cached
    with pytest.raises(ValueError):
        p.schedule()


def test_planner_token_budget_and_max_seqs():
    p = StepPlanner(check_plans=True, num_blocks=256, max_seqs=3, max_seq_len=512, max_num_batched_tokens=40,
                    prefill_chunk=32, device="cpu")
    sim = Sim(p)
    for i in range(5):
        p.add_request(i, 100)
    for _ in range(40):
        plan = p.schedule()
        assert plan.total_new_tokens <= 40
        assert p.num_running <= 3
        sim.apply(plan)
    assert p.num_running == 3 and len(p.waiting) == 2      # rows are the limit, not blocks
    p.finish(0)
    sim.apply(p.schedule())
    assert 3 in p._row_of


def test_planner_preemption_recomputes_and_everything_finishes():
    # 12 blocks = 192 tokens of pool for sequences that want up to 80 each: evictions are certain
    p = StepPlanner(check_plans=True, num_blocks=12, max_seqs=6, max_seq_len=96, max_num_batched_tokens=64,
                    prefill_chunk=32, device="cpu")
    sim = Sim(p, seed=3)
    want = {}
    for i in range(6):
        prompt = int(sim.rng.integers(10, 40))
        new = int(sim.rng.integers(20, 40))
        want[i] = (prompt, new)
        p.add_request(i, prompt, new)
    done = set()
    for step in range(2000):
        for sid in p.completed():
            prompt, new = want[sid]
            assert p.context_len(sid) == prompt + new - 1      # the last sampled token is never cached
            assert p.num_generated(sid) == new
            p.finish(sid)
            done.add(sid)
            sim.hist.pop(sid, None)
        plan = p.schedule()
        if plan is None:
            break
        sim.apply(plan)
    assert done == set(range(6)), f"unfinished after {step} steps: {set(range(6)) - done}"
    assert p.num_preemptions > 0
    assert p.alloc.num_used == 0 and not p.has_work()


def test_planner_oldest_cannot_be_preempted_raises_when_alone():
    p = StepPlanner(num_blocks=2, max_seqs=2, max_seq_len=64, device="cpu")
    p.add_request("only", 32)                     # exactly fills both blocks
    p.schedule()
    with pytest.raises(OutOfBlocks):
        p.schedule()                              # its first decode token needs a third block


def test_planner_random_soak_against_oracle():
    p = StepPlanner(check_plans=True, num_blocks=48, max_seqs=10, max_seq_len=160, max_num_batched_tokens=96,
                    prefill_chunk=40, device="cpu", staging_depth=2)
    sim = Sim(p, seed=7)
    nxt = 0
    for step in range(400):
        if sim.rng.random() < 0.3:
            prompt = int(sim.rng.integers(1, 90))
            p.add_request(nxt, prompt, int(sim.rng.integers(1, 60)))
            nxt += 1
        for sid in p.completed():
            p.finish(sid)
            sim.hist.pop(sid, None)
        running = list(p._row_of)
        if running and sim.rng.random() < 0.05:            # a client hangs up mid-generation
            sid = running[int(sim.rng.integers(len(running)))]
            p.finish(sid)
            sim.hist.pop(sid, None)
        plan = p.schedule()
        if plan is not None:
            sim.apply(plan)
    assert nxt > 50


def test_check_plan_catches_corrupted_plans():
    """The kernels skip or clamp what lies outside the pool instead of faulting, so a planner bug
    would be silent: the host-side self-check names it before the plan reaches the device."""
    import copy
    from aicomp_amd.block_manager import PlanError, check_plan
    pl = StepPlanner(num_blocks=64, max_seqs=8, max_seq_len=256, max_num_batched_tokens=512, prefill_chunk=64,
                     device="cpu", check_plans=True)
    for i, n in enumerate((40, 70, 5)):
        pl.add_request(i, n)
    plan = pl.schedule()                       # passes its own check
    check_plan(plan, 64, 16)

    def broken(**edit):
        p = copy.copy(plan)
        for k, fn in edit.items():
            a = getattr(plan, k).copy()
            fn(a)
            setattr(p, k, a)
        return p

    def slot_out(a): a[3] = 64 * 16 + 5
    def slot_neg(a): a[0] = -1
    def slot_dup(a): a[1] = a[0]
    def block_out(a): a[1, 0] = 64
    def block_shared(a): a[2, 0] = a[0, 0]
    def ctx_long(a): a[0] = 256 + 16 * 2
    def ctx_short(a): a[1] = 3
    def pos_wrong(a): a[2] += 1
    for edit in (dict(host_slot_mapping=slot_out), dict(host_slot_mapping=slot_neg), dict(host_slot_mapping=slot_dup),
                 dict(host_block_table=block_out), dict(host_block_table=block_shared),
                 dict(host_context_lens=ctx_long), dict(host_context_lens=ctx_short), dict(host_positions=pos_wrong)):
        with pytest.raises(PlanError):
            check_plan(broken(**edit), 64, 16)
    # inside the planner: a corrupted table row is caught by schedule() itself, before the upload
    r = pl._row_of[1]
    pl._tab[r, 0] = 99
    with pytest.raises(PlanError):
        pl.schedule()


def test_check_plan_flag_defaults_to_the_environment(monkeypatch):
    monkeypatch.delenv("AICOMP_CHECK_PLANS", raising=False)
    assert StepPlanner(num_blocks=8, device="cpu").check_plans is False
    monkeypatch.setenv("AICOMP_CHECK_PLANS", "1")
    assert StepPlanner(num_blocks=8, device="cpu").check_plans is True
    assert StepPlanner(num_blocks=8, device="cpu", check_plans=False).check_plans is False


def test_prefill_item_list_names_every_tile_once_most_expensive_first():
    """ops.prefill_items: the order a planner hands to the prefill kernel.  Every query tile that has
    rows appears exactly once (also for a chunk longer than its context, whose rows the kernel zeroes),
    costs (keys of the tile's last row) never rise along the list, and a launch that is resident all
    at once gets its second round from the cheap end."""
    from aicomp_amd import ops
    rng = np.random.default_rng(3)
    for trial in range(50):
        S = int(rng.integers(1, 40))
        new = rng.choice([0, 1, 7, 31, 32, 33, 64, 100, 512], size=S)
        prior = rng.integers(0, 3000, size=S)
        ctx = prior + new
        if trial % 7 == 0 and S > 1:
            ctx[1] = max(0, new[1] - 5)                                   # an inconsistent row
        tile = int(rng.choice([8, 16, 32, 64, 128]))
        items = ops.prefill_items(ctx, new, tile)
        want = {(s, q) for s in range(S) for q in range(-(-int(new[s]) // tile))}
        got = [tuple(x) for x in items.tolist()]
        assert len(got) == len(set(got)) and set(got) == want, trial
        keys = [min(ctx[s], ctx[s] - new[s] + (q + 1) * tile) for s, q in got]
        assert all(a >= b for a, b in zip(keys, keys[1:])), trial
        assert items.dtype == np.int32 and items.shape == (len(want), 2)
    # 512 workgroups on 256 CUs, 8 per item: 32 items per round; the second round runs cheap to expensive
    items = ops.prefill_items([2048], [2048], 32, num_head_groups=8, num_cus=256)
    assert items[:32, 1].tolist() == list(range(63, 31, -1)) and items[32:, 1].tolist() == list(range(0, 32))
    # a larger launch is dispatched as places free up: expensive first throughout
    items = ops.prefill_items([4096], [4096], 32, num_head_groups=8, num_cus=256)
    assert items[:, 1].tolist() == list(range(127, -1, -1))


def _mixed_plan(ctx, new, npre, max_q):
    import torch
    from aicomp_amd.block_manager import StepPlan
    S = len(ctx)
    cu = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    return StepPlan(seq_ids=list(range(S)), num_prefill_seqs=npre, new_lens=np.asarray(new, dtype=np.int32), max_q_len=max_q,
                    total_new_tokens=int(cu[-1]), block_table=torch.zeros(S, 1, dtype=torch.int32),
                    context_lens=torch.tensor(ctx, dtype=torch.int32), cu_q_lens=torch.from_numpy(cu),
                    slot_mapping=None, positions=None, preempted=[], host_context_lens=np.asarray(ctx), host_cu_q_lens=cu)


def test_step_item_list_orders_a_mixed_step_for_one_launch():
    """ops.step_items: every chunk tile and every decode row exactly once; decode rows that are the
    longer items open the list (one CU-round of them, then one of chunk tiles, then alternating,
    each kind longest first); shorter decode rows leave the list in falling cost."""
    from aicomp_amd import ops
    rng = np.random.default_rng(5)
    npre, ndec, tile = 4, 60, 32
    new = [512] * npre + [1] * ndec
    ctx = [int(p) + 512 for p in rng.integers(0, 2049, npre)] + [int(c) for c in rng.integers(513, 4098, ndec)]
    items = ops.step_items(ctx, new, npre, tile, num_head_groups=8, num_cus=256)
    want = {(s, q) for s in range(npre) for q in range(16)} | {(s, 0) for s in range(npre, npre + ndec)}
    got = [tuple(x) for x in items.tolist()]
    assert len(got) == len(set(got)) and set(got) == want and items.dtype == np.int32
    assert all(s >= npre for s, _ in got[:32]) and all(s < npre for s, _ in got[32:64])
    dec_keys = [ctx[s] for s, _ in got if s >= npre]
    assert dec_keys == sorted(dec_keys, reverse=True)                       # each kind longest first
    pre_keys = [min(ctx[s], ctx[s] - 512 + (q + 1) * tile) for s, q in got if s < npre]
    assert pre_keys == sorted(pre_keys, reverse=True)
    kinds = [s >= npre for s, _ in got[64:64 + 2 * min(ndec - 32, 64 - 32)]]
    assert kinds == [True, False] * (len(kinds) // 2)                       # then alternating
    # short decode rows: falling cost over both kinds
    ctx2 = ctx[:npre] + [int(c) for c in rng.integers(2, 300, ndec)]
    items2 = ops.step_items(ctx2, new, npre, tile, num_head_groups=8, num_cus=256)
    keys2 = [min(ctx2[s], ctx2[s] - new[s] + (q + 1) * tile) for s, q in items2.tolist()]
    assert keys2 == sorted(keys2, reverse=True) and {tuple(x) for x in items2.tolist()} == want
    # no decode rows, or no chunks: the chunk order
    assert (ops.step_items(ctx[:npre], new[:npre], npre, tile, 8, 256) == ops.prefill_items(ctx[:npre], new[:npre], tile, 8, 0)).all()


def test_step_plan_sends_only_moderate_decode_parts_through_one_launch():
    """StepPlan.step_items: a list for a mixed step of 16-bit pools whose decode part is within
    the measured bounds, None otherwise (the step then goes through the prefill and decode kernels)."""
    import torch
    q = torch.zeros(1, 32, 128, dtype=torch.bfloat16)
    pool = torch.zeros(1, 8, 16, 128, dtype=torch.bfloat16)
    mixed = lambda ctx_dec, n_dec=8, chunk=512, npre=2: _mixed_plan([chunk + 100] * npre + [ctx_dec] * n_dec,
                                                                   [chunk] * npre + [1] * n_dec, npre, chunk)
    it = mixed(2000).step_items(q, pool)
    assert it is not None and it.shape == (2 * 16 + 8, 2)
    plan = mixed(2000)
    assert plan.step_items(q, pool) is plan.step_items(q, pool)                           # built once per step
    assert mixed(4608).step_items(q, pool) is not None and mixed(4609).step_items(q, pool) is None   # a long decode row
    assert mixed(2000, n_dec=128).step_items(q, pool) is not None and mixed(2000, n_dec=129).step_items(q, pool) is None
    assert mixed(2000, npre=0).step_items(q, pool) is None and mixed(2000, n_dec=0).step_items(q, pool) is None
    assert mixed(2000).step_items(q, pool.to(torch.float8_e4m3fn)) is None                # fp8 pools: own kernels
    assert mixed(2000).step_items(q.float(), pool.float()) is None
    assert mixed(2000, chunk=16).step_items(q, pool) is None                              # one-column-group kernel
    assert mixed(2000).step_items(torch.zeros(1, 32, 256, dtype=torch.bfloat16), torch.zeros(1, 8, 16, 256, dtype=torch.bfloat16)) is None
