"""Pins the advantage oracle to the reference's golden vectors (CPU only)."""

import pytest
import torch

from oracle import advantage as A
from helpers import load_golden

BASE = load_golden("baseline_cases.json")
ADV = load_golden("grpo_adv_cases.json")


@pytest.mark.parametrize("case", BASE["cases"], ids=[c["name"] for c in BASE["cases"]])
def test_baseline_std_golden(case):
    r = torch.tensor(case["rewards"], dtype=torch.float32)
    p = torch.tensor(case["prompts"])
    v = torch.tensor(case["valid"], dtype=torch.float32)
    baseline, std = A.baseline_and_std_per_prompt(p, r, v)
    assert torch.allclose(baseline, torch.tensor(case["baseline"], dtype=torch.float32), rtol=BASE["rtol"])
    if case["std"] is None:
        assert torch.isfinite(std).all()
    else:
        assert torch.allclose(std, torch.tensor(case["std"], dtype=torch.float32), rtol=BASE["rtol"])


def test_baseline_empty():
    b, s = A.baseline_and_std_per_prompt(torch.empty(0, 3, dtype=torch.long), torch.tensor([]), torch.tensor([]))
    assert b.shape == (0,) and s.shape == (0,)


def test_group_ids_brute_force():
    torch.manual_seed(0)
    p = torch.randint(0, 2, (40, 3))
    gid = A.group_ids_by_prompt(p)
    for i in range(40):
        for j in range(40):
            assert (gid[i] == gid[j]).item() == bool((p[i] == p[j]).all())


def test_non_loo_is_plain_mean_and_bessel_std():
    """Without leave-one-out the baseline is the group mean and std the unbiased
    sample std (library routine)."""
    torch.manual_seed(1)
    r = torch.randn(12)
    p = torch.arange(3).repeat_interleave(4).unsqueeze(-1)
    b, s = A.baseline_and_std_per_prompt(p, r, torch.ones(12), leave_one_out_baseline=False)
    for g in range(3):
        grp = r[g * 4 : g * 4 + 4]
        assert torch.allclose(b[g * 4 : g * 4 + 4], grp.mean().expand(4), atol=1e-6)
        assert torch.allclose(s[g * 4 : g * 4 + 4], grp.std(unbiased=True).expand(4), rtol=1e-3)


def test_loo_matches_brute_force():
    torch.manual_seed(2)
    r = torch.randn(10)
    p = torch.tensor([[0]] * 6 + [[7]] * 4)
    b, s = A.baseline_and_std_per_prompt(p, r, torch.ones(10))
    for lo, hi in ((0, 6), (6, 10)):
        for i in range(lo, hi):
            others = torch.cat([r[lo:i], r[i + 1 : hi]])
            assert b[i].item() == pytest.approx(others.mean().item(), abs=1e-6)
            assert s[i].item() == pytest.approx(others.std(unbiased=True).item(), rel=2e-3)


@pytest.mark.parametrize("case", ADV["cases"], ids=[c["name"] for c in ADV["cases"]])
def test_grpo_advantage_golden(case):
    out = A.grpo_advantages(
        torch.tensor(case["prompt_ids"]), torch.tensor(case["rewards"], dtype=torch.float32),
        torch.ones(*case["mask_shape"]), leave_one_out_baseline=False, normalize_rewards=True,
    )
    assert tuple(out.shape) == tuple(case["mask_shape"])
    assert (out == out[:, :1]).all()
    if case["expected_col"] is not None:
        exp = torch.tensor(case["expected_col"], dtype=torch.float32)
        assert torch.allclose(out[:, 0], exp, rtol=case["rtol"], atol=1e-6)
    elif case["name"] == "symmetry":
        assert out[0, 0] < 0 and abs(out[1, 0]) < 1e-5 and out[2, 0] > 0
        assert torch.allclose(out[0], -out[2], rtol=1e-5)
    else:
        assert abs(out.mean()) < 1e-5


def test_seq_logprob_error_masking_brute_force():
    """The restatement against plain Python loops (the reference's tests only mock this function)."""
    import math

    g = torch.Generator().manual_seed(21)
    b, s = 6, 9
    prev = torch.randn(b, s, generator=g)
    gen = prev + 0.3 * torch.randn(b, s, generator=g)
    tm = (torch.rand(b, s, generator=g) < 0.7).long()
    tm[2] = 0  # a sequence without unmasked tokens must not touch the statistics
    sm = torch.tensor([1, 1, 1, 0, 1, 1])
    rewards = torch.tensor([1.0, 0.0, 1.0, 1.0, 1.0, 0.0])
    errs = []
    for i in range(b):
        m = [float(tm[i, t]) * float(sm[i]) for t in range(1, s)]
        den = sum(m)
        num = sum(math.exp(abs(float(gen[i, t + 1] - prev[i, t + 1])) * m[t]) * m[t] for t in range(s - 1))
        errs.append(num / max(den, 1.0) if den > 0 else None)
    valid = [e for e in errs if e is not None]
    got, new_mask = A.seq_logprob_error_masking(prev, gen, tm, sm, rewards, None)
    assert abs(got["max_seq_mult_prob_error"] - max(valid)) < 1e-5
    assert abs(got["mean_seq_mult_prob_error"] - sum(valid) / len(valid)) < 1e-5
    assert abs(got["min_seq_mult_prob_error"] - min(valid)) < 1e-5
    assert got["num_masked_seqs"] == 0 and new_mask is sm
    thr = sorted(valid)[len(valid) // 2]  # masks the sequences strictly above the median
    got, new_mask = A.seq_logprob_error_masking(prev, gen, tm, sm, rewards, thr + 1e-6)
    want_mask = [float(sm[i]) * (1.0 if (errs[i] if errs[i] is not None else 0.0) <= thr + 1e-6 else 0.0) for i in range(b)]
    assert new_mask.tolist() == want_mask
    dropped = [i for i in range(b) if float(sm[i]) - want_mask[i] != 0]
    assert got["num_masked_seqs"] == len(dropped) > 0
    assert abs(got["masked_correct_pct"] - sum(1 for i in dropped if rewards[i] == 1) / len(dropped)) < 1e-6
    kept = [errs[i] for i in range(b) if want_mask[i] and errs[i] is not None]
    assert abs(got["max_seq_mult_prob_error_after_mask"] - max(kept)) < 1e-5
    assert abs(got["min_seq_mult_prob_error_after_mask"] - min(kept)) < 1e-5


def test_dynamic_sampling_keep_indices_brute_force():
    """``oracle.advantage.dynamic_sampling_keep_indices`` against a plain loop, and on the std vectors of the
    reference's tests (``tests/unit/algorithms/test_grpo.py:1733-1736, 1790-1793``)."""
    from oracle import advantage as A

    g = torch.Generator().manual_seed(0)
    v = torch.randn(200, generator=g) * (torch.rand(200, generator=g) < 0.6)
    v[17] = float("nan")
    v[40] = -0.0
    want = [i for i in range(200) if not (v[i].item() == 0.0)]
    assert A.dynamic_sampling_keep_indices(v) == want and 17 in want and 40 not in want
    assert A.dynamic_sampling_keep_indices(torch.tensor([0.5, 0.5, 0.5, 0.25, 0.25, 0.25])) == [0, 1, 2, 3, 4, 5]
    assert A.dynamic_sampling_keep_indices(torch.tensor([0.0, 0.0, 0.0, 0.25, 0.25, 0.25])) == [3, 4, 5]
    assert A.dynamic_sampling_keep_indices(torch.zeros(0)) == []
