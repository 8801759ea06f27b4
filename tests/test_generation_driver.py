"""Host logic of the generation driver (CPU): token shaping, row order, last-row selection."""
import pytest
import torch

from aicomp_amd.block_manager import StepPlanner
from aicomp_amd.generation import ScheduleGeneration


class EchoBackend:
    device = torch.device("cpu")

    def begin_step(self, plan):
        self.plan = plan


def make(budget=16, chunk=8):
    planner = StepPlanner(num_blocks=64, max_seqs=8, max_seq_len=128, max_num_batched_tokens=budget,
                          prefill_chunk=chunk, device="cpu")
    seen = []

    def model(ids, positions):                # "logits" = (token id, position): enough to check the plumbing
        seen.append((ids.clone(), positions.clone()))
        return torch.stack([ids.float(), positions.float()], dim=1)

    return ScheduleGeneration(model, EchoBackend(), planner), planner, seen


def test_prefill_returns_last_position_of_every_prompt():
    gen, planner, seen = make()
    ids = torch.arange(3 * 20).view(3, 20) + 100
    lens = [20, 3, 11]
    out = gen.prefill(ids, prompt_lens=lens)
    assert out.shape == (3, 2)
    for b, n in enumerate(lens):
        assert out[b].tolist() == [float(ids[b, n - 1]), float(n - 1)]
        assert planner.context_len(b) == n
    # every prompt token was fed exactly once, at its own position, in chunks of at most 8 and 16 per step
    fed = {}
    for t_ids, t_pos in seen:
        assert t_ids.numel() <= 16
        for tok, p in zip(t_ids.tolist(), t_pos.tolist()):
            b = (tok - 100) // 20
            assert (tok - 100) % 20 == p and (b, p) not in fed
            fed[(b, p)] = True
    assert len(fed) == sum(lens)


@pytest.mark.parametrize("shape", ["B", "B1", "1B"])
def test_decode_step_token_shapes(shape):
    gen, planner, seen = make()
    gen.prefill(torch.zeros(2, 5, dtype=torch.long), prompt_lens=[5, 2])
    tok = torch.tensor([7, 9])
    tok = {"B": tok, "B1": tok[:, None], "1B": tok[None, :]}[shape]
    out = gen.decode_step(tok)
    assert out.tolist() == [[7.0, 5.0], [9.0, 2.0]]          # each sequence at its own position
    out = gen.decode_step(torch.tensor([1, 2]), position=[6, 3])
    assert out.tolist() == [[1.0, 6.0], [2.0, 3.0]]
    with pytest.raises(ValueError):
        gen.decode_step(torch.tensor([1, 2]), position=6)    # not the cached length of sequence 1
    with pytest.raises(ValueError):
        gen.decode_step(torch.tensor([1, 2, 3]))


def test_clear_cache_releases_blocks_and_prefill_restarts():
    gen, planner, seen = make()
    gen.prefill(torch.zeros(2, 40, dtype=torch.long))
    assert planner.alloc.num_used == 6
    gen.clear_cache()
    assert planner.alloc.num_used == 0 and not planner.has_work()
    out = gen.prefill(torch.ones(1, 4, dtype=torch.long))
    assert out.tolist() == [[1.0, 3.0]]


def test_rotary_tables_must_cover_the_planner_lengths():
    """A token beyond the rotary tables would be neither rotated nor stored by the fused launch:
    the driver refuses a planner that admits longer sequences than the backend's tables hold."""
    planner = StepPlanner(num_blocks=64, max_seqs=8, max_seq_len=128, device="cpu")

    class RopeBackend(EchoBackend):
        cos = torch.zeros(64, 16)

    with pytest.raises(ValueError, match="rotary tables hold 64"):
        ScheduleGeneration(lambda ids, pos: ids, RopeBackend(), planner)
    RopeBackend.cos = torch.zeros(128, 16)
    ScheduleGeneration(lambda ids, pos: ids, RopeBackend(), planner)
