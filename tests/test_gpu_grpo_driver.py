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


# ---- dynamic sampling (DAPO): scenarios of the reference's tests (tests/unit/algorithms/test_grpo.py:1701-1960) ----
def _ds_batch(n, rewards):
    from rl_amd.distributed.batched_data_dict import BatchedDataDict

    logs = [[{"role": "user", "content": f"prompt_{i // 3}"}, {"role": "assistant", "content": f"response_{i}"}] for i in range(n)]
    return BatchedDataDict({"message_log": logs, "task_name": ["math"] * n, "total_reward": torch.tensor(rewards)})


def _ds_config(prompts, gens, max_batches=5, enabled=True):
    from types import SimpleNamespace

    return SimpleNamespace(grpo=SimpleNamespace(use_dynamic_sampling=enabled, num_prompts_per_step=prompts,
                                                num_generations_per_prompt=gens, dynamic_sampling_max_gen_batches=max_batches))


@pytest.mark.parametrize("n", [0, 1, 63, 64, 65, 256, 257, 5000])
def test_nonzero_indices_matches_oracle(n):
    from oracle import advantage as A

    g = torch.Generator().manual_seed(n)
    v = torch.randn(n, generator=g) * (torch.rand(n, generator=g) < 0.5)
    if n > 2:
        v[1] = float("nan")
        v[2] = -0.0
    got = torch.ops.rl_amd.nonzero_indices(v.to(DEV))
    assert got.dtype == torch.int64 and got.tolist() == A.dynamic_sampling_keep_indices(v)


def test_dynamic_sampling_keeps_every_group_with_spread():
    from rl_amd.algorithms.grpo import dynamic_sampling

    batch = _ds_batch(6, [1.0, 0.0, 1.0, 0.5, 0.5, 0.0])
    std = torch.tensor([0.5, 0.5, 0.5, 0.25, 0.25, 0.25])
    baseline = torch.tensor([0.67, 0.67, 0.67, 0.33, 0.33, 0.33])
    out, complete, cache, metrics = dynamic_sampling(batch, std, baseline, 1, _ds_config(2, 3), None)
    assert out.size == 6 and complete is True
    assert torch.allclose(out["std"], std) and torch.allclose(out["baseline"], baseline)
    assert metrics == {"dynamic_sampling_num_discarded_valid_samples": 0}


def test_dynamic_sampling_drops_groups_without_spread():
    from rl_amd.algorithms.grpo import dynamic_sampling

    batch = _ds_batch(6, [1.0, 1.0, 1.0, 0.5, 0.5, 0.0])
    std = torch.tensor([0.0, 0.0, 0.0, 0.25, 0.25, 0.25])
    baseline = torch.tensor([1.0, 1.0, 1.0, 0.33, 0.33, 0.33])
    out, complete, _cache, _ = dynamic_sampling(batch, std, baseline, 1, _ds_config(1, 3), None)
    assert out.size == 3 and complete is True
    assert torch.allclose(out["std"], torch.tensor([0.25, 0.25, 0.25]))
    assert torch.allclose(out["baseline"], torch.tensor([0.33, 0.33, 0.33]))
    assert [out["message_log"][i][0]["content"] for i in range(out.size)] == ["prompt_1"] * 3
    assert torch.allclose(out["filtered_reward"], torch.tensor([0.5, 0.5, 0.0]))


def test_dynamic_sampling_rows_stay_aligned_through_filter_and_cut():
    from rl_amd.algorithms.grpo import dynamic_sampling

    batch = _ds_batch(9, [1.0, 0.0, 1.0, 0.5, 0.0, 0.5, 0.2, 0.6, 0.9])
    batch["mask_sample"] = torch.tensor([False, True, False, True, False, True, False, False, True])
    std = torch.tensor([0.5, 0.5, 0.5, 0.25, 0.25, 0.25, 0.35, 0.35, 0.35])
    baseline = torch.tensor([0.67, 0.67, 0.67, 0.33, 0.33, 0.33, 0.57, 0.57, 0.57])
    out, complete, _, metrics = dynamic_sampling(batch, std, baseline, dynamic_sampling_num_gen_batches=1,
                                                 master_config=_ds_config(2, 3), timer=None)
    assert complete is True and out.size == 6
    assert torch.equal(out["mask_sample"], torch.tensor([False, True, False, True, False, True]))
    assert metrics["dynamic_sampling_num_discarded_valid_samples"] == 3


def test_dynamic_sampling_caches_until_enough_and_gives_up_after_the_limit():
    from rl_amd.algorithms.grpo import dynamic_sampling

    std = torch.tensor([0.4, 0.4, 0.4])
    baseline = torch.tensor([0.5, 0.5, 0.5])
    cfg = _ds_config(2, 3)
    out, complete, cache, _ = dynamic_sampling(_ds_batch(3, [1.0, 0.0, 0.5]), std, baseline, 1, cfg, None)
    assert out.size == 3 and complete is False and cache is not None and cache == out
    out, complete, cache, _ = dynamic_sampling(_ds_batch(3, [1.0, 0.0, 0.5]), std, baseline, 1, cfg, None, cache)
    assert out.size == 6 and complete is True and cache is not None
    # nothing kept: the batch is ignored, the cache is left alone
    out, complete, cache2, _ = dynamic_sampling(_ds_batch(3, [1.0, 1.0, 1.0]), torch.zeros(3), baseline, 2, cfg, None, None)
    assert out.size == 0 and complete is False and cache2 is None
    with pytest.raises(ValueError):
        dynamic_sampling(_ds_batch(3, [1.0, 0.0, 0.5]), std, baseline, 6, cfg, None)
    # switched off: the batch comes back whole, with baseline and std attached
    batch = _ds_batch(3, [1.0, 1.0, 1.0])
    out, complete, _, metrics = dynamic_sampling(batch, torch.zeros(3), baseline, 1, _ds_config(2, 3, enabled=False), None)
    assert out is batch and complete is True and metrics == {} and torch.equal(out["std"], torch.zeros(3))
