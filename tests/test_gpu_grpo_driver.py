"""GPU parity of the driver-side GRPO helpers against the CPU oracle (fp32, relative 1e-5; masks exact)."""

import pytest
import torch

from oracle import advantage as OA
from rl_amd.algorithms.grpo import _clip_grpo_advantages, compute_and_apply_seq_logprob_error_masking

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _data(b, s, seed, int_masks=True):
    g = torch.Generator().manual_seed(seed)
    prev = torch.randn(b, s, generator=g)
    gen = prev + 0.2 * torch.randn(b, s, generator=g)
    tm = (torch.rand(b, s, generator=g) < 0.8)
    tm[min(2, b - 1)] = False
    sm = (torch.rand(b, generator=g) < 0.9)
    rewards = (torch.rand(b, generator=g) < 0.5).float()
    cast = (lambda t: t.long()) if int_masks else (lambda t: t.float())
    return {"prev_logprobs": prev, "generation_logprobs": gen, "token_mask": cast(tm), "sample_mask": cast(sm)}, rewards


@pytest.mark.parametrize("b,s,int_masks", [(7, 33, True), (64, 4096, False), (1, 2, True)])
@pytest.mark.parametrize("threshold", [None, 1.18])
@pytest.mark.parametrize("where", ["cpu", "cuda"])
def test_seq_logprob_error_masking_matches_oracle(b, s, int_masks, threshold, where):
    data, rewards = _data(b, s, seed=b * s, int_masks=int_masks)
    want, want_mask = OA.seq_logprob_error_masking(data["prev_logprobs"], data["generation_logprobs"], data["token_mask"],
                                                   data["sample_mask"], rewards, threshold)
    td = {k: v.to(where) for k, v in data.items()}
    got = compute_and_apply_seq_logprob_error_masking(td, rewards.to(where), threshold)
    assert set(got) == set(want)
    for k in want:
        assert abs(got[k] - want[k]) <= 1e-5 * abs(want[k]) + 1e-7, (k, got[k], want[k])
    assert isinstance(got["num_masked_seqs"], int)
    if threshold is not None:
        assert td["sample_mask"].device.type == where
        assert torch.equal(td["sample_mask"].cpu().float(), want_mask.float())
    else:
        assert td["sample_mask"] is not None and torch.equal(td["sample_mask"].cpu(), data["sample_mask"])


def test_all_sequences_masked_gives_zeros():
    data, rewards = _data(4, 8, seed=5)
    data["sample_mask"] = torch.zeros(4)
    got = compute_and_apply_seq_logprob_error_masking({k: v.to(DEV) for k, v in data.items()}, rewards.to(DEV), 1.1)
    assert got["max_seq_mult_prob_error"] == 0.0 and got["mean_seq_mult_prob_error"] == 0.0
    assert got["num_masked_seqs"] == 0 and got["masked_correct_pct"] == 0.0


def test_clip_grpo_advantages():
    adv = torch.tensor([[-5.0, 0.5, 7.0]], device=DEV)
    assert torch.equal(_clip_grpo_advantages(adv, {"advantage_clip_low": -2.0, "advantage_clip_high": 3.0}).cpu(),
                       torch.tensor([[-2.0, 0.5, 3.0]]))
    assert _clip_grpo_advantages(adv, {"advantage_clip_low": None, "advantage_clip_high": None}) is adv
