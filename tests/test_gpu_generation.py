"""End to end on the GPU: a small Llama-shaped model generating through the paged path
(planner -> rotary + append -> chunked prefill / decode kernels) against the same model
recomputing full causal attention with the library's rotary, repeat_kv and SDPA."""
import pytest
import torch

from aicomp_amd.block_manager import StepPlanner
from aicomp_amd.generation import PagedAttentionBackend, ScheduleGeneration
from tiny_llama import TinyLlama

pytestmark = pytest.mark.gpu


def close(got, want, what):
    scale = want.float().abs().max().item()
    err = (got.float() - want.float()).abs().max().item()
    assert err <= 0.04 * scale + 1e-3, f"{what}: max err {err:.4f} vs logits scale {scale:.3f}"


@pytest.mark.parametrize("kv_dtype", [torch.bfloat16, torch.float8_e4m3fn])
def test_generate_matches_full_recompute(device, kv_dtype):
    torch.manual_seed(0)
    m = TinyLlama().to(device).to(torch.bfloat16)
    m.inv_freq = m.inv_freq.float()
    planner = StepPlanner(num_blocks=64, max_seqs=8, max_seq_len=256, max_num_batched_tokens=80,
                          prefill_chunk=32, device=device)
    backend = PagedAttentionBackend(m.layers, 64, m.hkv, m.d, torch.bfloat16, device, kv_dtype=kv_dtype,
                                    inv_freq=m.inv_freq, max_positions=256)
    if kv_dtype == torch.float8_e4m3fn:
        for i in range(m.layers):
            backend.set_scales(i, torch.full((m.hkv,), 8.0 / 448), torch.full((m.hkv,), 8.0 / 448))
    gen = ScheduleGeneration(lambda ids, pos: m.forward_paged(ids, pos, backend), backend, planner)
    lens = [37, 5, 64]
    B, S = len(lens), max(lens)
    prompts = torch.randint(0, 199, (B, S), device=device)
    tol_what = "fp8 pool" if kv_dtype == torch.float8_e4m3fn else "bf16 pool"

    print("prefill", flush=True)
    logits = gen.prefill(prompts, prompt_lens=lens)
    seqs = [prompts[b, :lens[b]].tolist() for b in range(B)]

    def naive_last():
        out = []
        for s in seqs:
            ids = torch.tensor([s], device=device)
            out.append(m.forward_naive(ids)[0, -1])
        return torch.stack(out)

    if kv_dtype == torch.bfloat16:
        close(logits, naive_last(), "prefill logits")
    for step in range(12):
        nxt = logits.argmax(-1)
        for b in range(B):
            seqs[b].append(int(nxt[b]))
        print(f"decode step {step}", flush=True)
        logits = gen.decode_step(nxt[:, None], position=[len(s) - 1 for s in seqs])
        if kv_dtype == torch.bfloat16:
            close(logits, naive_last(), f"decode step {step} ({tol_what})")
    assert [planner.context_len(b) for b in range(B)] == [len(s) for s in seqs]
    if kv_dtype == torch.float8_e4m3fn:
        # quantised K/V: the run must stay finite and close to the unquantised model's distribution
        ref = naive_last()
        assert torch.isfinite(logits).all()
        assert (logits.float() - ref.float()).abs().max().item() <= 0.35 * ref.float().abs().max().item()
    gen.clear_cache()
    assert planner.alloc.num_used == 0


def test_backend_attend_mixed_step_one_launch_equals_separate_kernels(device, monkeypatch):
    """PagedAttentionBackend.attend on a mixed step (a prompt chunk of one sequence beside a decode
    row of another), rotary embedding on: the one-launch route over chunk and decode row against
    the chunk through the prefill kernel and the row through the decode kernel.  Same pools bit for
    bit (both append through the same launch), chunk rows bit for bit, the decode row within the
    attention tolerance (another kernel sums in another order)."""
    from aicomp_amd.block_manager import StepPlan
    hq, hkv, d, layers = 8, 2, 64, 1
    inv = 1.0 / (10000.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))

    def run():
        torch.manual_seed(4)
        planner = StepPlanner(num_blocks=32, max_seqs=4, max_seq_len=256, max_num_batched_tokens=80,
                              prefill_chunk=32, device=device)
        backend = PagedAttentionBackend(layers, 32, hkv, d, torch.bfloat16, device, inv_freq=inv, max_positions=256)
        planner.add_request("a", 100)
        planner.add_request("b", 10)
        outs, routes = [], []
        for step in range(3):
            plan = planner.schedule()
            T = plan.total_new_tokens
            q = torch.randn(T, hq, d, device=device).to(torch.bfloat16)
            k = (torch.randn(T, hkv, d, device=device) * 0.5).to(torch.bfloat16)
            v = (torch.randn(T, hkv, d, device=device) * 0.5).to(torch.bfloat16)
            backend.begin_step(plan)
            outs.append((plan.num_prefill_seqs, plan.num_prefill_tokens, backend.attend(0, q, k, v)))
            routes.append(plan.step_items(q, backend.k_pools[0]) is not None)
        torch.cuda.synchronize()
        return outs, routes, backend.k_pools[0].clone(), backend.v_pools[0].clone()

    one, routes_one, k1, v1 = run()
    assert routes_one == [False, True, True]          # step 0: two chunks; steps 1, 2: a chunk of "a" beside a token of "b"
    monkeypatch.setattr(StepPlan, "ONE_LAUNCH_MAX_ROWS", 0)
    sep, routes_sep, k2, v2 = run()
    assert routes_sep == [False, False, False]
    assert torch.equal(k1.view(torch.int16), k2.view(torch.int16)) and torch.equal(v1.view(torch.int16), v2.view(torch.int16))
    for (npre, t_pre, a), (_, _, b) in zip(one, sep):
        assert torch.isfinite(a.float()).all()
        assert torch.equal(a[:t_pre].view(torch.int16), b[:t_pre].view(torch.int16))
        err = (a[t_pre:].float() - b[t_pre:].float()).abs()
        assert bool(((err <= 1e-2) | (err <= 2e-2 * b[t_pre:].float().abs())).all()), err.max().item()
