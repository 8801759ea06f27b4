"""Benchmark of the paged KV-cache attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]

A step is one pass of the hot path over one synthetic batch of the Llama-3-8B
decode shape (batch 64, 32 query / 8 KV heads, head_dim 128, block 16, context
uniform in [512,4096], bf16): KV append of one token per sequence, then paged
decode attention.  All inputs are resident in HBM before the timed region.
Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
METRIC = "decode-attn HBM GB/s (% peak) + tokens/s, Llama-3-8B paged KV, 1 GPU"



def measured_traffic_bytes():
    """HBM bytes per decode call of the Llama-3-8B shape as the kept rocprofv3 counter summary gives
    them (--pmc FETCH_SIZE / WRITE_SIZE, scaled by what a 1 GiB device copy reads on the same
    counters; main + merge kernel): read from profiles/decode_llama3_8b_decode.md so that the figure
    in the JSON line and the summary cannot drift apart.  None if the summary is missing."""
    import re
    try:
        with open(os.path.join(ROOT, "profiles", "decode_llama3_8b_decode.md")) as f:
            m = re.search(r"Total HBM traffic per call:\s*([0-9.]+)\s*MB", f.read())
        return float(m.group(1)) * 1e6 if m else None
    except OSError:
        return None


def profiled_prefill_cycles():
    """Shader cycles of one prefill launch of the chunked-prefill shape, from the kept rocprofv3
    counter summary (SQ_BUSY_CYCLES / 32 shader engines); None if the summary is missing."""
    import re
    try:
        with open(os.path.join(ROOT, "profiles", "prefill_chunked_prefill_mixed.md")) as f:
            m = re.search(r"([0-9]+) cycles per launch", f.read())
        return int(m.group(1)) if m else None
    except OSError:
        return None


def settled_back_to_back(fn, reps=50, settle_s=0.03):
    """Average duration of `reps` launches of fn queued back to back between two events, after
    `settle_s` of untimed launches (an idle GPU's clock takes that long to ramp up)."""
    import torch
    fn()
    torch.cuda.synchronize()
    tw = time.perf_counter()
    while time.perf_counter() - tw < settle_s:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
    p0, p1 = _events(2)
    p0.record()
    for _ in range(reps):
        fn()
    p1.record()
    torch.cuda.synchronize()
    return p0.elapsed_time(p1) / reps * 1e-3


def _events(n):
    import torch
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def plan_of_workload(w):
    """The workload's step as the plan a StepPlanner would hand to paged_attention_step (chunks
    first, one-token rows after; the workload's own tables and lengths)."""
    import numpy as np
    from aicomp_amd.block_manager import StepPlan
    npre = w.num_prefill_seqs
    return StepPlan(seq_ids=list(range(w.num_seqs)), num_prefill_seqs=npre,
                    new_lens=np.asarray(w.new_list, dtype=np.int32),
                    max_q_len=max(w.new_list[:npre]) if npre else 0, total_new_tokens=int(w.query.shape[0]),
                    block_table=w.block_table, context_lens=w.context_lens, cu_q_lens=w.cu_q_lens,
                    slot_mapping=w.slot_mapping, positions=None, preempted=[],
                    host_context_lens=np.asarray(w.ctx_list), host_cu_q_lens=w.cu_q_lens.cpu().numpy())


def run_decode_config(name, steps, warmup, dev, settle_ms=30.0):
    """Append + decode for one workload; returns timing and algorithmic figures.

    Clock protocol: an idle MI355X takes about 30 ms of continuous work to bring its shader clock
    up, and the launches in between run up to 10-15 % slower (6 % on the Llama-3.2-1B shape, 3 % on
    the headline shape, whose kernel waits for HBM most of the time).  A serving process never sees
    that ramp after its first step, so every timed loop here is preceded by `settle_ms` of the same
    steps, untimed, before the `warmup` steps; the same K steps timed from an idle part (only the
    `warmup` steps before them) are kept beside the figure as `from_idle`."""
    import torch
    from aicomp_amd import ops, workloads
    w = workloads.make_workload(name, device=dev)
    npre = w.num_prefill_seqs
    S = w.num_seqs
    # decode part: the sequences that add one token
    qd = w.query[int(w.cu_q_lens[npre]):].contiguous()
    btd = w.block_table[npre:].contiguous()
    cld = w.context_lens[npre:].contiguous()
    outd = torch.empty_like(qd)
    if npre:
        T_pre = int(w.cu_q_lens[npre])
        qp = w.query[:T_pre].contiguous()
        outp = torch.empty_like(qp)
        btp = w.block_table[:npre].contiguous()
        clp = w.context_lens[:npre].contiguous()
        cup = w.cu_q_lens[:npre + 1].contiguous()
        max_q = max(w.new_list[:npre])

    # new rows of the decode sequences (one per sequence) for the fused append+decode call
    t0_dec = int(w.cu_q_lens[npre])
    nk_dec = w.new_key[t0_dec:].contiguous()
    nv_dec = w.new_value[t0_dec:].contiguous()

    # A model step walks one K/V pool per layer, so no call finds its pool in a cache the previous
    # call filled.  The timed loop does the same: it cycles over several pools ("layers": same
    # tables and lengths, separate allocations), enough of them that a pool has been pushed out of
    # the 256 MB memory-side cache and the L2s by the time its turn comes again.
    pool_bytes = 2 * w.k_pool.numel() * w.k_pool.element_size()
    n_pools = int(min(32, max(3, -(-(1 << 30) // pool_bytes))))
    pools = [(w.k_pool, w.v_pool)] + [(w.k_pool.clone(), w.v_pool.clone()) for _ in range(n_pools - 1)]

    def step(i=0, ev=None):
        kp, vp = pools[i % len(pools)]
        if ev: ev[0].record()
        if npre:
            # mixed step: scatter every new row (chunks and decode tokens), prefill, decode
            ops.kv_append(w.new_key, w.new_value, kp, vp, w.slot_mapping, w.k_scale, w.v_scale)
            if ev: ev[1].record()
            ops.paged_prefill_attn(outp, qp, kp, vp, btp, clp, cup, w.scale, max_q_len=max_q)
            if ev: ev[2].record()
            ops.paged_decode_attn(outd, qd, kp, vp, btd, cld, w.scale, w.k_scale, w.v_scale)
        else:
            # decode step: the append of the 1-token-per-sequence rows is fused into the call
            if ev: ev[1].record()
            ops.paged_decode_attn(outd, qd, kp, vp, btd, cld, w.scale, w.k_scale, w.v_scale,
                                  new_key=nk_dec, new_value=nv_dec)
        if ev: ev[3].record()

    def append_only():
        ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping, w.k_scale, w.v_scale)

    def settle(fn):
        """Untimed steps for settle_ms (a synchronisation every 8 steps keeps the queue short)."""
        t0, i = time.perf_counter(), 0
        while (time.perf_counter() - t0) * 1e3 < settle_ms:
            for _ in range(8):
                fn(i)
                i += 1
            torch.cuda.synchronize()

    def timed_loop(rotate, settled=True):
        """K steps queued back to back between two HIP events on the launch stream: their distance
        / K is the average duration of a step's launches.  A step that has several phases (append,
        prefill, decode) also carries events between the phases, but only on ten of the steps: an
        event costs a few microseconds of stream time."""
        if settled:
            settle(lambda i: step(i if rotate else 0))
        for i in range(warmup):
            step(i if rotate else 0)
        torch.cuda.synchronize()
        stride = max(1, steps // 10)
        evs = {i: _events(4) for i in range(0, steps, stride)} if npre else {}
        r_begin, r_end = _events(2)
        t0 = time.perf_counter()
        r_begin.record()
        for i in range(steps):
            step(i if rotate else 0, evs.get(i))
        r_end.record()
        t_enqueue = time.perf_counter() - t0
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        region = r_begin.elapsed_time(r_end) / steps * 1e-3     # seconds per step, device time line
        return wall, t_enqueue, region, list(evs.values())

    # the same loop over one pool (every step re-reads what the previous one read): kept beside
    # the rotating figure, which is the one the headline uses
    wall_idle, _, region_idle, _ = timed_loop(rotate=True, settled=False)       # straight after set-up
    wall_1, _, region_1, evs_1 = timed_loop(rotate=False)
    wall, t_enqueue, region, evs = timed_loop(rotate=True)
    planned = None
    if npre:
        # The same step the way a step planner's attention call runs it (paged_attention_step: it
        # decides between one launch over all sequences and chunks / decode rows through their own
        # kernels), over the same rotating pools; the three-launch loop above stays for the
        # per-kernel figures.
        from aicomp_amd.block_manager import paged_attention_step
        plan = plan_of_workload(w)
        out_all = torch.empty_like(w.query)
        one_launch = plan.step_items(w.query, w.k_pool) is not None

        def planned_step(i):
            kp, vp = pools[i % len(pools)]
            paged_attention_step(plan, out_all, w.query, w.new_key, w.new_value, kp, vp, w.scale, w.k_scale, w.v_scale)

        settle(planned_step)
        for i in range(warmup):
            planned_step(i)
        torch.cuda.synchronize()
        p0, p1 = _events(2)
        t0 = time.perf_counter()
        p0.record()
        for i in range(steps):
            planned_step(i)
        p1.record()
        torch.cuda.synchronize()
        planned = {"wall": time.perf_counter() - t0, "region": p0.elapsed_time(p1) / steps * 1e-3,
                   "route": "append + one launch of the chunked-prefill kernel over chunks and decode rows" if one_launch
                   else "append + prefill kernel + decode kernels"}
    # the stand-alone append kernel, timed on its own: 20 launches between two events, queued
    # behind ~1 ms of filler work so that the host's launch rate does not enter the figure
    for _ in range(3):
        append_only()
    filler = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    a0, a1 = _events(2)
    for _ in range(4):
        filler.fill_(1)
    a0.record()
    for _ in range(20):
        append_only()
    a1.record()
    rope_fn, rope_bytes = rope_case(w, dev)
    for _ in range(3):
        rope_fn()
    r0, r1 = _events(2)
    for _ in range(4):
        filler.fill_(1)
    r0.record()
    for _ in range(20):
        rope_fn()
    r1.record()
    torch.cuda.synchronize()
    t_rope = r0.elapsed_time(r1) / 20 * 1e-3
    # cold figure: the decode call right after 1 GiB of unrelated writes has gone through L2 and
    # the memory-side cache (the steady-state loop above re-reads the same pool every step)
    cold = []
    for _ in range(8):
        filler.fill_(2)
        c0, c1 = _events(2)
        c0.record()
        ops.paged_decode_attn(outd, qd, w.k_pool, w.v_pool, btd, cld, w.scale, w.k_scale, w.v_scale)
        c1.record()
        cold.append((c0, c1))
    torch.cuda.synchronize()
    t_cold = statistics.median(a.elapsed_time(b) for a, b in cold) * 1e-3
    del filler
    # the same decode step recorded into a HIP graph (ten calls per graph, so that the graph's own
    # launch cost is shared) and replayed: no host launch cost per step (the library allocates
    # nothing and clears nothing, the scratch is passed in)
    GRAPH_CALLS = len(pools) * -(-10 // len(pools))       # whole turns of the pool cycle
    t_graph = None
    if not npre:
        try:
            need = ops.decode_workspace_bytes(S, w.shape.num_q_heads, w.shape.num_kv_heads, w.shape.head_dim,
                                              w.shape.block_size, btd.shape[1], qd.dtype, w.k_pool.dtype)
            ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for i in range(GRAPH_CALLS):
                    ops.paged_decode_attn(outd, qd, *pools[i % len(pools)], btd, cld, w.scale, w.k_scale, w.v_scale,
                                          new_key=nk_dec, new_value=nv_dec, workspace=ws)
            for _ in range(3):
                graph.replay()
            g0, g1 = _events(2)
            g0.record()
            for _ in range(steps):
                graph.replay()
            g1.record()
            torch.cuda.synchronize()
            t_graph = g0.elapsed_time(g1) / (steps * GRAPH_CALLS) * 1e-3
            del graph
        except Exception as e:                              # a bench figure, not a requirement
            print(f"graph replay not measured for {name}: {e}", file=sys.stderr)
    t_app = a0.elapsed_time(a1) / 20 * 1e-3
    t_pre = statistics.mean(e[1].elapsed_time(e[2]) for e in evs) * 1e-3 if npre else 0.0
    t_pre_b2b = 0.0
    if npre:
        # prefill_us and prefill_roofline describe the launch inside the mixed step (events around it,
        # pools rotating).  Beside it, under its own key: launches queued back to back between two
        # events after ~30 ms of untimed ones (the first launches after an idle gap run 10-15 %
        # slower while the clock ramps up; this is the protocol of `--only prefill`, whose
        # rocprofv3 summary under profiles/ it can be compared with).
        t_pre_b2b = settled_back_to_back(
            lambda: ops.paged_prefill_attn(outp, qp, w.k_pool, w.v_pool, btp, clp, cup, w.scale, max_q_len=max_q))
    # a pure decode step is one call (main + merge kernel): its average duration is the region's
    t_dec = statistics.mean(e[2].elapsed_time(e[3]) for e in evs) * 1e-3 if npre else region
    t_dec_1 = statistics.mean(e[2].elapsed_time(e[3]) for e in evs_1) * 1e-3 if npre else region_1
    # A tiny step is bound by the host's launch rate, not by the GPU: the eager figures then measure
    # Python.  They stay what they are (decode_us is what the eager operator path delivers); the
    # call's duration on the GPU, inside the replayed graph, is reported beside them.
    host_bound = (not npre) and t_graph is not None and t_enqueue / steps > 0.9 * region
    mb = btd.shape[1]
    routed_small = (S - npre) * mb * w.shape.block_size <= ops.set_small_decode_tokens(-1)
    res = {
        "workload": name, "ms_per_step": (planned["wall"] if planned else wall) / steps * 1e3,
        "pools_in_rotation": len(pools), "settle_ms": settle_ms,
        "from_idle": {"ms_per_step": wall_idle / steps * 1e3, "device_us_per_step": region_idle * 1e6,
                      "note": "the same K steps after only the W warm-up steps, the part coming out of idle"},
        "single_pool": {"ms_per_step": wall_1 / steps * 1e3, "decode_us": t_dec_1 * 1e6,
                        "decode_frac_hbm_peak": w.decode_kv_bytes() / t_dec_1 / 1e9 / HBM_PEAK_GBS,
                        "note": "the same loop re-reading one pool every step"},
        "host_enqueue_ms_per_step": t_enqueue / steps * 1e3,
        "append_us": t_app * 1e6, "append_bytes": w.append_bytes(),
        "append_GBs": w.append_bytes() / t_app / 1e9,
        "rope_append_us": t_rope * 1e6, "rope_append_bytes": rope_bytes,
        "rope_append_GBs": rope_bytes / t_rope / 1e9,
        "decode_us": t_dec * 1e6, "decode_bytes": w.decode_kv_bytes(),
        "decode_GBs": w.decode_kv_bytes() / t_dec / 1e9,
        "decode_frac_hbm_peak": w.decode_kv_bytes() / t_dec / 1e9 / HBM_PEAK_GBS,
        "decode_tokens_per_s": (S - npre) / t_dec,
        "decode_cold_us": t_cold * 1e6, "decode_cold_GBs": w.decode_kv_bytes() / t_cold / 1e9,
        "decode_graph_replay_us": None if t_graph is None else t_graph * 1e6,
        "decode_graph_replay_GBs": None if t_graph is None else w.decode_kv_bytes() / t_graph / 1e9,
        "host_bound": bool(host_bound),
        "partition_size": ops.decode_partition_size(S - npre, w.shape.num_q_heads, w.shape.num_kv_heads,
                                                    w.shape.head_dim, w.shape.block_size, btd.shape[1],
                                                    qd.dtype, w.k_pool.dtype),
        "kv_dtype": str(w.k_pool.dtype).replace("torch.", ""),
    }
    mfma_shape = (w.shape.head_dim in (64, 128) and w.shape.block_size == 16 and qd.dtype in (torch.bfloat16, torch.float16))
    balanced = mfma_shape and (S - npre) <= 1024 and not routed_small        # the library's own routing rule
    merge = "" if res["partition_size"] >= mb * w.shape.block_size else " + split_reduce_kernel"
    res["roofline"] = {
        "kernel": ("streamk_decode_kernel + streamk_reduce_kernel" if balanced else
                   "paged_decode_mfma_kernel" + merge if mfma_shape else
                   "paged_attn_generic_kernel" + merge),
        "bound": "hbm", "achieved": res["decode_GBs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": res["decode_frac_hbm_peak"], "algorithmic_bytes": res["decode_bytes"], "avg_launch_us": res["decode_us"]}
    if npre:
        res["step_route"] = planned["route"]
        res["step_device_us"] = planned["region"] * 1e6
        res["three_launches"] = {"ms_per_step": wall / steps * 1e3, "device_us": region * 1e6,
                                 "note": "append of all rows, prefill kernel on the chunks, decode kernels on the rows: "
                                         "the loop prefill_us and decode_us are taken from"}
        cyc = profiled_prefill_cycles()
        res.update({"prefill_us": t_pre * 1e6, "prefill_back_to_back_us": t_pre_b2b * 1e6,
                    "prefill_flops": w.prefill_flops(),
                    "prefill_TFLOPs": w.prefill_flops() / t_pre / 1e12,
                    "prefill_frac_mfma_peak": w.prefill_flops() / t_pre / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                    "prefill_back_to_back_frac_mfma_peak": w.prefill_flops() / t_pre_b2b / 1e12 / MFMA_BF16_PEAK_TFLOPS})
        res["prefill_roofline"] = {
            "kernel": "paged_prefill_mfma_kernel", "bound": "mfma", "achieved": res["prefill_TFLOPs"],
            "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": res["prefill_frac_mfma_peak"],
            "algorithmic_flop": res["prefill_flops"], "avg_launch_us": res["prefill_us"],
            "timed": "the launch inside the mixed step, between two events",
            # the launch's length in shader cycles does not depend on the clock the part happens to
            # hold (profiles/prefill_chunked_prefill_mixed.md, SQ_BUSY_CYCLES per shader engine), so
            # cycles / duration is the clock a timing was taken at; the peak assumes 2.4 GHz
            "cycles_per_launch": cyc,
            "clock_GHz_in_step": None if cyc is None else cyc / (t_pre * 1e6) / 1e3,
            "clock_GHz_back_to_back": None if cyc is None else cyc / (t_pre_b2b * 1e6) / 1e3}
    return res, w


def planner_bench(dev):
    """Host cost of planning one decode step for the headline batch (64 sequences, contexts
    uniform in [512, 4096]): free-list growth, block table, context lengths and slots packed
    into one pinned buffer and copied with one asynchronous transfer.  One plan serves every
    layer of a model step."""
    import numpy as np
    import torch
    from aicomp_amd.block_manager import StepPlanner
    rng = np.random.default_rng(0)
    pl = StepPlanner(num_blocks=12000, max_seqs=64, max_seq_len=4608, max_num_batched_tokens=8192,
                     prefill_chunk=512, device=dev)
    for i in range(64):
        pl.add_request(i, int(rng.integers(512, 4097)))
    plan = pl.schedule()
    while plan.num_prefill_seqs:
        plan = pl.schedule()
    torch.cuda.synchronize()
    n = 200
    t0 = time.perf_counter()
    for _ in range(n):
        plan = pl.schedule()
    host = (time.perf_counter() - t0) / n
    torch.cuda.synchronize()
    return {"decode_plan_host_us": host * 1e6, "seqs": plan.num_seqs,
            "h2d_bytes_per_plan": int(16 * plan.total_new_tokens + 4 * (plan.block_table.numel() + 2 * plan.num_seqs + 1)),
            "note": "StepPlanner.schedule() per decode step, including the enqueue of its one H2D copy"}


def small_batch_decode_bench(dev):
    """Decode calls of the size the reference's own engine issues (Llama-3.2-1B heads, 1 to 8
    sequences of 512 and 2048 tokens): GPU time per call, measured over replays of a HIP graph that
    holds 20 calls, so that the host's launch rate stays out of the figure."""
    import math
    import torch
    from aicomp_amd import ops
    hq, hkv, d = 32, 8, 64
    out_rows = []
    for B in (1, 8):
        for ctx in (512, 2048):
            nblk = math.ceil(ctx / 16)
            nb = B * nblk + 1
            g = torch.Generator().manual_seed(0)
            table = torch.randperm(nb - 1, generator=g)[: B * nblk].reshape(B, nblk).to(torch.int32).to(dev)
            k = (torch.randn(nb, hkv, 16, d, device=dev) * 0.5).to(torch.bfloat16)
            v = (torch.randn(nb, hkv, 16, d, device=dev) * 0.5).to(torch.bfloat16)
            q = torch.randn(B, hq, d, device=dev).to(torch.bfloat16)
            o = torch.empty_like(q)
            cl = torch.full((B,), ctx, dtype=torch.int32, device=dev)
            call = lambda: ops.paged_decode_attn(o, q, k, v, table, cl, 1 / math.sqrt(d))
            call()
            torch.cuda.synchronize()
            graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
            with torch.cuda.stream(side):
                call()
                with torch.cuda.graph(graph, stream=side):
                    for _ in range(20):
                        call()
            torch.cuda.synchronize()
            for _ in range(3):
                graph.replay()
            e0, e1 = _events(2)
            e0.record()
            for _ in range(10):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            nbytes = B * (2 * ctx * hkv * d * 2 + 2 * hq * d * 2)
            out_rows.append({"batch": B, "context": ctx, "us_per_call": round(e0.elapsed_time(e1) / 200 * 1e3, 2),
                             "kv_bytes": nbytes})
    return {"shape": "32 query / 8 KV heads, head_dim 64, bf16", "calls": out_rows}


def mixed_step_graph(dev, two_streams):
    """The chunked-prefill mixed step (4 chunks of 512 tokens + 60 decode sequences) recorded into a
    HIP graph of three steps over three K/V pools, and a function that replays it.  Serial: append of
    the chunk rows, prefill, fused append + decode, one after the other.  Two streams: the decode call
    is launched first on one stream and the append + prefill on a second one, forked from and joined
    to the step's stream with events, so that the hardware may run them side by side (a graph keeps
    the host's stream and event calls out of the figure)."""
    import torch
    from aicomp_amd import ops, workloads
    w = workloads.make_workload("chunked_prefill_mixed", device=dev)
    npre = w.num_prefill_seqs
    T = int(w.cu_q_lens[npre])
    qd, btd, cld = w.query[T:].contiguous(), w.block_table[npre:].contiguous(), w.context_lens[npre:].contiguous()
    qp, btp, clp = w.query[:T].contiguous(), w.block_table[:npre].contiguous(), w.context_lens[:npre].contiguous()
    cup = w.cu_q_lens[:npre + 1].contiguous()
    outd, outp = torch.empty_like(qd), torch.empty_like(qp)
    nkd, nvd = w.new_key[T:].contiguous(), w.new_value[T:].contiguous()
    nkp, nvp, smp = w.new_key[:T].contiguous(), w.new_value[:T].contiguous(), w.slot_mapping[:T].contiguous()
    pools = [(w.k_pool, w.v_pool)] + [(w.k_pool.clone(), w.v_pool.clone()) for _ in range(2)]
    s = w.shape
    ws = torch.empty(ops.decode_workspace_bytes(len(w.ctx_list) - npre, s.num_q_heads, s.num_kv_heads, s.head_dim, s.block_size,
                                                btd.shape[1], qd.dtype, w.k_pool.dtype), dtype=torch.uint8, device=dev)
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()

    def decode(kp, vp):
        ops.paged_decode_attn(outd, qd, kp, vp, btd, cld, w.scale, workspace=ws, new_key=nkd, new_value=nvd)

    def prefill(kp, vp):
        ops.kv_append(nkp, nvp, kp, vp, smp)
        ops.paged_prefill_attn(outp, qp, kp, vp, btp, clp, cup, w.scale, max_q_len=max(w.new_list[:npre]))

    def step(i):
        kp, vp = pools[i % 3]
        if not two_streams:
            prefill(kp, vp)
            decode(kp, vp)
            return
        main = torch.cuda.current_stream()
        fork = torch.cuda.Event()
        fork.record(main)
        sa.wait_event(fork)
        sb.wait_event(fork)
        with torch.cuda.stream(sa):
            decode(kp, vp)
        with torch.cuda.stream(sb):
            prefill(kp, vp)
        ja, jb = torch.cuda.Event(), torch.cuda.Event()
        ja.record(sa)
        jb.record(sb)
        main.wait_event(ja)
        main.wait_event(jb)

    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        for i in range(3):
            step(i)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for i in range(3):
                step(i)
    torch.cuda.synchronize()
    return graph.replay, ("decode on one stream, append + prefill on another" if two_streams else "one stream")


def mixed_step_bench(dev, reps=40):
    """Mixed step replayed from a graph, one stream against two (see mixed_step_graph): us per step."""
    import torch
    res = {}
    for name, two in (("one_stream_us", False), ("two_streams_us", True)):
        fn, _ = mixed_step_graph(dev, two)
        for _ in range(5):
            fn()
        e0, e1 = _events(2)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        res[name] = round(e0.elapsed_time(e1) / (3 * reps) * 1e3, 1)
        del fn
        torch.cuda.empty_cache()
    res["note"] = ("graph replays of 3 steps over 3 pools; two streams: decode launched first, append + prefill beside it, "
                   "forked and joined with events")
    return res


def host_cost_bench(dev):
    """Host time of ONE decode call of the drop-in operator at the size the reference's own engine
    runs (batch 1, Llama-3.2-1B heads: 32 / 8, head_dim 64, bf16, K/V arriving expanded by
    repeat_kv): the Python thread's time per call, timed over 1024 calls without a synchronisation
    inside (32 consecutive steps from the stated context, then the position is set back).
    At 600 cached tokens the call is one launch (whole rows), at 1500 two (256-token partitions and
    their merge).  Through each host route to the same C entry point: the CPython function over a
    per-layer handle (the one the operator takes), the registered operator
    (torch.ops.mi355_kv.decode_step) and the ctypes binding."""
    import torch
    from aicomp_amd import kv_cache as akv
    B, hq, g, d = 1, 32, 4, 64
    hkv = hq // g
    mk = lambda n, h: torch.randn(B, h, n, d, device=dev).to(torch.bfloat16)
    res = {"shape": "batch 1, 32 query / 8 KV heads (K/V expanded to 32), head_dim 64, bf16",
           "call": "op(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False)"}
    available = {"fast": akv._FAST is not None, "torch_op": akv._TORCH_DECODE is not None, "ctypes": True}
    for name in ("fast", "torch_op", "ctypes"):
        if not available[name]:
            continue
        saved, akv._route = akv._route, name
        try:
            op = akv.CachedScaledDotProductAttention(0, 2048, num_kv_groups=g)
            op.enable()
            op(mk(1500, hq), mk(1500, hkv).repeat_interleave(g, 1), mk(1500, hkv).repeat_interleave(g, 1), is_causal=True)
            q, k, v = mk(1, hq), mk(1, hkv).repeat_interleave(g, 1), mk(1, hkv).repeat_interleave(g, 1)
            for ctx in (600, 1500):
                for _ in range(200):
                    op.cache_pos = ctx
                    op(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False)
                torch.cuda.synchronize()
                best = None
                for _ in range(5):
                    n = 1024
                    t0 = time.perf_counter()
                    for _ in range(n // 32):
                        op.cache_pos = ctx                    # 32 steps from the stated context, then back
                        for _ in range(32):                   # the call as compiler_fx/modeling_llama.py:607-614 issues it
                            op(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False)
                    host = (time.perf_counter() - t0) / n
                    torch.cuda.synchronize()
                    best = host if best is None else min(best, host)
                res[f"host_us_per_call_{name}_ctx{ctx}"] = round(best * 1e6, 2)
        finally:
            akv._route = saved
    res["route_in_use"] = akv._route
    res["host_us_per_call"] = res[f"host_us_per_call_{akv._route}_ctx600"]
    return res


def sampler_bench(dev, batch=64, vocab=128256, temperature=0.8, top_k=50, top_p=0.9, reps=20):
    """The step after the attention path: one token per row of [64, 128256] fp32 logits with
    temperature / top-k / top-p (opt_prime/opt_prime/inference.py:786-843).  Beside the kernel, the
    reference's own statement sequence run by torch on the same GPU (sort, cumsum, softmax, scatter,
    multinomial) as the figure it replaces."""
    import torch
    from aicomp_amd import ops
    g = torch.Generator(device=dev).manual_seed(0)
    logits = torch.randn(batch, vocab, device=dev, generator=g) * 2.5
    u = torch.rand(batch, device=dev, generator=g)

    def ours():
        return ops.sample_tokens(logits, temperature, top_k, top_p, uniforms=u)

    def eager():
        x = logits.clone() / temperature
        k = min(top_k, x.size(-1))
        x[x < torch.topk(x, k)[0][..., -1, None]] = float("-inf")
        sl, si = torch.sort(x, descending=True)
        cp = torch.cumsum(torch.softmax(sl, dim=-1), dim=-1)
        rm = cp > top_p
        rm[..., 1:] = rm[..., :-1].clone()
        rm[..., 0] = 0
        x[rm.scatter(-1, si, rm)] = float("-inf")
        return torch.multinomial(torch.softmax(x, dim=-1), num_samples=1).squeeze(-1)

    res = {}
    for name, fn in (("kernel_us", ours), ("torch_eager_us", eager)):
        for _ in range(3):
            fn()
        e0, e1 = _events(2)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        res[name] = e0.elapsed_time(e1) / reps * 1e3
    res.update({"batch": batch, "vocab": vocab, "temperature": temperature, "top_k": top_k, "top_p": top_p,
                "dtype": "f32", "logit_bytes": batch * vocab * 4})
    return res


def prefill_shapes_bench(dev, reps=20):
    """The chunked-prefill kernels on shapes with many more workgroups than the named mixed step
    (512 workgroups there, two per CU, bounded by the longest of them): fresh long prompts and a
    batch of chunks with prior context.  Synthetic K/V, 32/8 heads.  Every shape is first run for
    about 30 ms untimed (the clock of an idle GPU takes that long to settle: the first launches after
    a pause run 10-15 % slower), then `reps` launches are timed between two events."""
    import math
    import torch
    from aicomp_amd import ops
    hq, hkv = 32, 8
    out = []
    for nseq, n, prior, d, kvt, qt in ((1, 8192, 0, 128, torch.bfloat16, torch.bfloat16),
                                       (1, 2048, 0, 128, torch.bfloat16, torch.bfloat16),
                                       (4, 4096, 0, 128, torch.bfloat16, torch.bfloat16),
                                       (16, 512, 2048, 128, torch.bfloat16, torch.bfloat16),
                                       (16, 512, 2048, 128, torch.float8_e4m3fn, torch.bfloat16),
                                       (16, 512, 2048, 64, torch.bfloat16, torch.bfloat16),
                                       (16, 512, 2048, 128, torch.float16, torch.float16),
                                       (1, 2048, 0, 128, torch.float32, torch.float32)):
        ctx = prior + n
        nblk = math.ceil(ctx / 16)
        nb = nseq * nblk + 1
        g = torch.Generator().manual_seed(0)
        table = torch.randperm(nb - 1, generator=g)[: nseq * nblk].reshape(nseq, nblk).to(torch.int32).to(dev)
        k = torch.randn(nb, hkv, 16, d, device=dev) * 0.5
        v = torch.randn(nb, hkv, 16, d, device=dev) * 0.5
        ks = vs = None
        if kvt == torch.float8_e4m3fn:
            ks = (k.abs().amax(dim=(0, 2, 3)) / 448).float().contiguous()
            vs = (v.abs().amax(dim=(0, 2, 3)) / 448).float().contiguous()
            k = (k / ks[None, :, None, None]).to(kvt)
            v = (v / vs[None, :, None, None]).to(kvt)
        else:
            k, v = k.to(kvt), v.to(kvt)
        q = torch.randn(nseq * n, hq, d, device=dev).to(qt)
        o = torch.empty_like(q)
        cl = torch.full((nseq,), ctx, dtype=torch.int32, device=dev)
        cu = (torch.arange(nseq + 1, dtype=torch.int32) * n).to(dev)
        call = lambda: ops.paged_prefill_attn(o, q, k, v, table, cl, cu, 1 / math.sqrt(d), max_q_len=n,
                                              k_scale=ks, v_scale=vs)
        call()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.03:
            for _ in range(4):
                call()
            torch.cuda.synchronize()
        e0, e1 = _events(2)
        e0.record()
        for _ in range(reps):
            call()
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) / reps * 1e-3
        flops = nseq * 4 * hq * d * (n * prior + n * (n + 1) / 2)
        f32 = qt == torch.float32
        peak = 157.3 if f32 else MFMA_BF16_PEAK_TFLOPS          # fp32 matrix peak, published
        name = lambda t_: str(t_).replace("torch.", "")
        out.append({"chunks": nseq, "new_tokens": n, "prior": prior, "head_dim": d,
                    "q_dtype": name(qt), "kv_dtype": name(kvt), "us": round(t * 1e6, 1),
                    "TFLOPs": round(flops / t / 1e12, 1),
                    "kernel": "paged_prefill_mfma_f32_kernel" if f32 else "paged_prefill_mfma_kernel",
                    "peak_TFLOPs": peak, "frac_mfma_peak": round(flops / t / 1e12 / peak, 4)})
        del k, v, q, o
        torch.cuda.empty_cache()
    return out


def prefill_ragged_bench(dev, reps=40):
    """Ragged chunk batches (a serving step's shape: many chunks of unlike lengths over unlike
    contexts), once in the order the kernel finds for itself (launch grid, or its own ranking when
    the batch has at most 16 chunks) and once with the (sequence, query tile) pairs ranked by the
    caller, ops.prefill_items: the way block_manager.paged_attention_step and generate() call it.
    The list's upload is outside the timed loop (a planner builds it once per step, with the other
    step tensors); bf16, 32/8 heads, head_dim 128, block 16; same settle protocol as above."""
    import itertools
    import math
    import random
    import torch
    from aicomp_amd import ops
    hq, hkv, d, bs = 32, 8, 128, 16
    rnd = random.Random(0)
    cases = (("32 chunks of 8..512 tokens, priors 0..2048", [rnd.randint(0, 2048) for _ in range(32)],
              [512, 384, 256, 128, 64, 32, 16, 8] * 4),
             ("64 chunks of 64 tokens, priors 0..4096", [rnd.randint(0, 4096) for _ in range(64)], [64] * 64),
             ("4 chunks of 512 + 20 of 48 tokens, priors 0..3000", [rnd.randint(0, 3000) for _ in range(24)],
              [512] * 4 + [48] * 20))
    ncu = torch.cuda.get_device_properties(0).multi_processor_count
    rows = []
    for name, priors, news in cases:
        ctx = [p + n for p, n in zip(priors, news)]
        need = [math.ceil(c / bs) for c in ctx]
        nb = sum(need) + 1
        g = torch.Generator().manual_seed(1)
        perm = torch.randperm(nb - 1, generator=g).to(torch.int32)
        table = torch.zeros(len(ctx), max(need), dtype=torch.int32)
        at = 0
        for s, k_ in enumerate(need):
            table[s, :k_] = perm[at:at + k_]
            at += k_
        table = table.to(dev)
        k = (torch.randn(nb, hkv, bs, d, device=dev) * 0.5).bfloat16()
        v = (torch.randn(nb, hkv, bs, d, device=dev) * 0.5).bfloat16()
        q = torch.randn(sum(news), hq, d, device=dev).bfloat16()
        o = torch.empty_like(q)
        cl = torch.tensor(ctx, dtype=torch.int32, device=dev)
        cu = torch.tensor([0] + list(itertools.accumulate(news)), dtype=torch.int32, device=dev)
        tile = ops.prefill_tile_positions(hq, hkv, d, bs, q.dtype, k.dtype, max(news))
        ops.prefill_items(ctx, news, tile, num_head_groups=hkv, num_cus=ncu)        # numpy's first call
        t0 = time.perf_counter()
        host_items = ops.prefill_items(ctx, news, tile, num_head_groups=hkv, num_cus=ncu)
        rank_us = (time.perf_counter() - t0) * 1e6
        items = torch.from_numpy(host_items).to(dev)
        us = {}
        for label, it in (("grid_order", None), ("item_list", items)):
            call = lambda: ops.paged_prefill_attn(o, q, k, v, table, cl, cu, 1 / math.sqrt(d), max_q_len=max(news),
                                                  items=it)
            call()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            while time.perf_counter() - t0 < 0.03:
                for _ in range(4):
                    call()
                torch.cuda.synchronize()
            e0, e1 = _events(2)
            e0.record()
            for _ in range(reps):
                call()
            e1.record()
            torch.cuda.synchronize()
            us[label] = e0.elapsed_time(e1) / reps * 1e3
        flops = sum(4 * hq * d * (n * p + n * (n + 1) / 2) for p, n in zip(priors, news))
        rows.append({"batch": name, "new_tokens": sum(news), "items": int(host_items.shape[0]),
                     "grid_places": len(news) * math.ceil(max(news) / tile), "tile_positions": tile,
                     "grid_order_us": round(us["grid_order"], 1), "item_list_us": round(us["item_list"], 1),
                     "speedup": round(us["grid_order"] / us["item_list"], 2),
                     "item_list_TFLOPs": round(flops / us["item_list"] / 1e6, 1),
                     "host_ranking_us": round(rank_us, 1)})
        del k, v, q, o
        torch.cuda.empty_cache()
    return rows


def device_info():
    import torch
    p = torch.cuda.get_device_properties(0)
    return {"name": p.name, "arch": getattr(p, "gcnArchName", ""), "compute_units": p.multi_processor_count,
            "hbm_gib": round(p.total_memory / 2**30, 1),
            "hbm_peak_GBs_used": HBM_PEAK_GBS, "mfma_bf16_peak_TFLOPs_used": MFMA_BF16_PEAK_TFLOPS}


def rope_case(w, dev):
    """Fused rotary + append over every new token of a workload: the launch and its algorithmic
    bytes (Q read and written, K and V read, pool rows written, one cos and one sin row, position
    and slot per token)."""
    import torch
    from aicomp_amd import ops
    s = w.shape
    T = w.query.shape[0]
    inv = 1.0 / (500000.0 ** (torch.arange(0, s.head_dim, 2, dtype=torch.float32) / s.head_dim))
    cos, sin = ops.rotary_tables(inv, 8192, w.query.dtype, device=dev)
    pos = torch.empty(T, dtype=torch.int64, device=dev)
    cu = w.cu_q_lens.cpu().tolist()
    cl = w.context_lens.cpu().tolist()
    for i in range(len(cl)):                 # positions of each sequence's new tokens
        n = cu[i + 1] - cu[i]
        pos[cu[i]:cu[i + 1]] = torch.arange(cl[i] - n, cl[i])
    q_out = torch.empty_like(w.query)
    e, ekv = w.query.element_size(), w.k_pool.element_size()
    nbytes = T * (2 * s.num_q_heads * s.head_dim * e + 2 * s.num_kv_heads * s.head_dim * (e + ekv)
                  + 2 * s.head_dim * e + 16)
    fn = lambda: ops.rope_kv_append(w.query, w.new_key, w.new_value, cos, sin, pos, w.k_pool, w.v_pool,
                                    w.slot_mapping, w.k_scale, w.v_scale, query_out=q_out)
    return fn, nbytes


def profile_target(which, steps, warmup, dev, settle_ms=30.0):
    """Launch one kernel of the path repeatedly, for rocprofv3 (--kernel-trace / --pmc).
    "copy" is a plain device copy of exactly 1 GiB: the counter calibration.

    The launches follow the protocol of the bench's back-to-back timings: `warmup` untimed
    launches, then untimed launches for `settle_ms` more (the clock of an idle part takes about
    that long to ramp up), then `steps` launches queued back to back; a summary averages the last
    `steps` dispatches of the trace.  Counter passes use --settle-ms 0 (they serialise launches)."""
    import torch
    from aicomp_amd import ops, workloads

    def drive(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        settled = 0
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < settle_ms:
            for _ in range(8):
                fn()
            settled += 8
            torch.cuda.synchronize()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return f"{warmup} + {settled} untimed launches, then {steps} back to back"
    if which == "copy":
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        how = drive(lambda: dst.copy_(src))
        print(f"copy: {how}; {src.numel()} bytes read + {dst.numel()} bytes written per launch")
        return
    if which == "sample":
        g = torch.Generator(device=dev).manual_seed(0)
        logits = torch.randn(64, 128256, device=dev, generator=g) * 2.5
        u = torch.rand(64, device=dev, generator=g)
        how = drive(lambda: ops.sample_tokens(logits, 0.8, 50, 0.9, uniforms=u))
        print(f"sample: {how}, over [64, 128256] fp32 logits, temperature 0.8, top-k 50, top-p 0.9")
        return
    if which in ("mixed_serial", "mixed_streams"):
        fn, how = mixed_step_graph(dev, two_streams=which == "mixed_streams")
        for _ in range(warmup + steps):
            fn()
        torch.cuda.synchronize()
        print(f"{which}: {warmup + steps} replays of a graph of 3 mixed steps ({how})")
        return
    if which == "mixed_planned":
        # the named mixed step the way paged_attention_step runs it (one pool)
        from aicomp_amd.block_manager import paged_attention_step
        w = workloads.make_workload("chunked_prefill_mixed", device=dev)
        plan = plan_of_workload(w)
        out = torch.empty_like(w.query)
        one = plan.step_items(w.query, w.k_pool) is not None
        how = drive(lambda: paged_attention_step(plan, out, w.query, w.new_key, w.new_value, w.k_pool, w.v_pool, w.scale))
        print(f"mixed_planned (chunked_prefill_mixed): {how}; "
              f"{'append + one launch over chunks and decode rows' if one else 'append + prefill + decode kernels'}")
        return
    if which == "prefill_long":
        # one fresh prompt of 8192 tokens at the Llama-3-8B head shape (a row of prefill_other_shapes)
        import math
        nseq, n, hq, hkv, d = 1, 8192, 32, 8, 128
        nblk = n // 16
        g = torch.Generator().manual_seed(0)
        table = torch.randperm(nblk, generator=g).reshape(1, nblk).to(torch.int32).to(dev)
        k = (torch.randn(nblk + 1, hkv, 16, d, device=dev) * 0.5).to(torch.bfloat16)
        v = (torch.randn(nblk + 1, hkv, 16, d, device=dev) * 0.5).to(torch.bfloat16)
        q = torch.randn(n, hq, d, device=dev).to(torch.bfloat16)
        o = torch.empty_like(q)
        cl = torch.full((1,), n, dtype=torch.int32, device=dev)
        cu = torch.tensor([0, n], dtype=torch.int32, device=dev)
        how = drive(lambda: ops.paged_prefill_attn(o, q, k, v, table, cl, cu, 1 / math.sqrt(d), max_q_len=n))
        print(f"prefill_long: {how}, {4 * hq * d * (n * (n + 1) // 2)} algorithmic flop per launch")
        return
    name = {"decode": "llama3_8b_decode", "append": "chunked_prefill_mixed", "prefill": "chunked_prefill_mixed",
            "decode_fp8": "llama3_70b_decode_fp8", "decode_long": "long_context_skewed",
            "decode_d64": "llama32_1b_decode", "rope": "chunked_prefill_mixed"}[which]
    w = workloads.make_workload(name, device=dev)
    ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping, w.k_scale, w.v_scale)
    npre = w.num_prefill_seqs
    t0 = int(w.cu_q_lens[npre])
    if which.startswith("decode"):
        q = w.query[t0:].contiguous()
        out = torch.empty_like(q)
        bt, cl = w.block_table[npre:].contiguous(), w.context_lens[npre:].contiguous()
        fn = lambda: ops.paged_decode_attn(out, q, w.k_pool, w.v_pool, bt, cl, w.scale, w.k_scale, w.v_scale)
        info = f"{w.decode_kv_bytes()} algorithmic bytes per launch"
    elif which == "append":
        fn = lambda: ops.kv_append(w.new_key, w.new_value, w.k_pool, w.v_pool, w.slot_mapping)
        info = f"{w.append_bytes()} algorithmic bytes per launch"
    elif which == "rope":
        fn, nbytes = rope_case(w, dev)
        info = f"{nbytes} algorithmic bytes per launch"
    else:
        q = w.query[:t0].contiguous()
        out = torch.empty_like(q)
        bt, cl, cu = w.block_table[:npre].contiguous(), w.context_lens[:npre].contiguous(), w.cu_q_lens[:npre + 1].contiguous()
        mq = max(w.new_list[:npre])
        fn = lambda: ops.paged_prefill_attn(out, q, w.k_pool, w.v_pool, bt, cl, cu, w.scale, max_q_len=mq)
        info = f"{w.prefill_flops()} algorithmic flop per launch"
    how = drive(fn)
    print(f"{which} ({name}): {how}, {info}")


def host_threads():
    """torch.set_num_threads(<the host cores this process may use>), called explicitly: os.cpu_count(),
    held to the share the environment grants where it states one (OMP_NUM_THREADS).  Returns the
    thread count torch reports afterwards."""
    import torch
    n = os.cpu_count() or 1
    try:
        n = max(1, min(n, int(os.environ.get("OMP_NUM_THREADS", n))))
    except ValueError:
        pass
    if torch.get_num_threads() != n:
        torch.set_num_threads(n)
    return torch.get_num_threads()


def cpu_baseline(w, budget_s=20.0):
    """The reference's CPU path (gather -> repeat_kv -> contiguous -> SDPA), restated in
    oracle/contiguous_ref.py, timed on the host cores over a bounded sample of the batch."""
    import torch
    from oracle import contiguous_ref as cref
    threads = host_threads()
    npre = w.num_prefill_seqs
    q = w.query[int(w.cu_q_lens[npre]):].cpu()
    bt = w.block_table[npre:].cpu()
    cl = w.context_lens[npre:].cpu()
    kp, vp = w.k_pool.cpu(), w.v_pool.cpu()
    ks = None if w.k_scale is None else w.k_scale.cpu()
    vs = None if w.v_scale is None else w.v_scale.cpu()
    B = q.shape[0]
    n = min(B, 4 if budget_s < 10 else 8)

    def run(nseq):
        t0 = time.perf_counter()
        cref.reference_cpu_decode(q[:nseq], kp, vp, bt[:nseq], cl[:nseq], w.scale, ks, vs,
                                  compute_dtype=q.dtype)
        return time.perf_counter() - t0

    t1 = run(n)
    # sample: as many sequences as fit ~budget with 3 warmups + >= 3 timed repetitions
    per_seq = t1 / n
    nseq = int(max(1, min(B, budget_s / (6 * per_seq))))
    reps = int(max(3, min(10, budget_s / (per_seq * nseq) - 3)))
    for _ in range(3):
        run(nseq)
    ts = sorted(run(nseq) for _ in range(reps))
    med = ts[len(ts) // 2]
    e = w.k_pool.element_size()
    s = w.shape
    byts = sum(2 * L * s.num_kv_heads * s.head_dim * e for L in w.ctx_list[npre:npre + nseq])
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"value": byts / med / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "tokens_per_s": nseq / med,
            "sample": f"first {nseq} of {B} sequences of the same batch, decode attention only "
                      f"(gather blocks -> repeat_kv -> contiguous -> torch SDPA, {str(q.dtype).replace('torch.', '')}), "
                      f"3 warmups, median of {reps}; {med * 1e3:.1f} ms per pass; "
                      f"cpu '{model}', os.cpu_count()={os.cpu_count()}, torch threads={threads}"}


def cpu_prefill_baseline(w):
    """The reference's CPU prefill call (gather -> repeat_kv -> contiguous -> SDPA), restated in
    oracle/contiguous_ref.py, timed on the host cores for the first chunk of the workload."""
    import torch
    from oracle import contiguous_ref as cref
    host_threads()
    n, L = w.new_list[0], w.ctx_list[0]
    q = w.query[: n].cpu()
    bt = w.block_table[0].cpu()
    kp, vp = w.k_pool.cpu(), w.v_pool.cpu()
    run = lambda: cref.reference_cpu_prefill(q, kp, vp, bt, L, w.scale, compute_dtype=q.dtype)
    run()
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        run()
        ts.append(time.perf_counter() - t0)
    med = sorted(ts)[1]
    s = w.shape
    flops = 4 * s.num_q_heads * s.head_dim * (n * (L - n) + n * (n + 1) / 2)
    return {"value": flops / med / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"first chunk of the workload ({n} new tokens over {L - n} prior ones): gather blocks -> repeat_kv -> "
                      f"contiguous -> torch SDPA with the chunk's causal mask, {str(q.dtype).replace('torch.', '')}, "
                      f"1 warm-up, median of 3; {med * 1e3:.1f} ms per pass"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the other workloads")
    ap.add_argument("--only", choices=["decode", "append", "copy", "prefill", "prefill_long", "decode_fp8", "decode_long", "decode_d64", "rope", "sample",
                             "mixed_serial", "mixed_streams", "mixed_planned"],
                    help="profiling target: launch just this kernel --steps times (no JSON line)")
    ap.add_argument("--settle-ms", type=float, default=30.0,
                    help="untimed steps (launches, with --only) for this long before the warm-up and timed ones")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (asked for --gpus {args.gpus}); "
              "the path shards by sequence or by KV head with no communication, but no "
              "multi-GPU code is part of it.", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from aicomp_amd import _lib
    _lib.load()     # fails loudly if the HIP library is missing
    dev = torch.device("cuda:0")

    if args.only:
        profile_target(args.only, args.steps, args.warmup, dev, args.settle_ms)
        return
    main_res, w = run_decode_config("llama3_8b_decode", args.steps, args.warmup, dev, args.settle_ms)
    s = w.shape
    line = {
        "metric": METRIC,
        "value": main_res["decode_bytes"] / (main_res["ms_per_step"] * 1e-3) / 1e9,
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"],
        # untimed steps of the same kind for this long before the W warm-up steps (an idle part's clock
        # takes that long to come up); the K steps timed without them are in "from_idle"
        "settle_ms": args.settle_ms, "from_idle": main_res["from_idle"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "llama3_8b_decode: batch 64, 32 query / 8 KV heads, head_dim 128, "
                               "block 16, context uniform [512,4096] seed 0, bf16; step = KV append "
                               "of 64 rows + paged decode attention (one fused call); consecutive steps "
                               "run over different K/V pools, as the layers of a model do",
                   "batch": s.batch, "partition_size": main_res["partition_size"],
                   "kv_bytes_per_step": main_res["decode_bytes"]},
        "tokens_per_s": s.batch / (main_res["ms_per_step"] * 1e-3),
        "pct_hbm_peak": 100.0 * main_res["decode_bytes"] / (main_res["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "roofline": {"kernel": "streamk_decode_kernel<bf16> (append fused) + streamk_reduce_kernel (one decode call)",
                     "bound": "hbm", "achieved": main_res["decode_GBs"], "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": main_res["decode_GBs"] / HBM_PEAK_GBS,
                     "traffic": measured_traffic_bytes(),
                     "algorithmic_bytes": main_res["decode_bytes"],
                     "avg_launch_us": main_res["decode_us"]},
        "append": {"us": main_res["append_us"], "GB/s": main_res["append_GBs"],
                   "bytes": main_res["append_bytes"]},
        "decode_graph_replay_us": main_res["decode_graph_replay_us"],
        "pools_in_rotation": main_res["pools_in_rotation"],
        "single_pool": main_res["single_pool"],
        "decode_cold": {"us": main_res["decode_cold_us"], "GB/s": main_res["decode_cold_GBs"],
                        "note": "decode call timed right after 1 GiB of unrelated writes"},
        "device": device_info(),
        "step_planner": planner_bench(dev),
        "sampler": sampler_bench(dev),
        "decode_small_batch": small_batch_decode_bench(dev),
        "operator_host_cost": host_cost_bench(dev),
        "mixed_step_streams": mixed_step_bench(dev),
        "prefill_other_shapes": prefill_shapes_bench(dev),
        "prefill_ragged_batches": prefill_ragged_bench(dev),
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(w)
    del w
    torch.cuda.empty_cache()
    if not args.no_extra:
        extra = []
        for name in ("decode_fp32_small", "llama32_1b_decode", "long_context_skewed", "chunked_prefill_mixed",
                     "llama3_70b_decode_fp8"):
            r, ww = run_decode_config(name, args.steps, args.warmup, dev, args.settle_ms)
            if not args.no_cpu:
                # the reference's CPU path on the same batch, in the workload's own dtype (fp32 for
                # the small anchor shape, which is defined on that path); a few seconds each
                r["cpu_baseline"] = cpu_baseline(ww, budget_s=5.0)
                if ww.num_prefill_seqs:
                    r["prefill_cpu_baseline"] = cpu_prefill_baseline(ww)
            del ww
            torch.cuda.empty_cache()
            rnd = lambda v: round(v, 4) if isinstance(v, float) else v
            extra.append({k: ({kk: rnd(vv) for kk, vv in v.items()} if isinstance(v, dict) else rnd(v))
                          for k, v in r.items()})
        line["other_workloads"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
