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
