"""Oracle: per-prompt group baseline / std and GRPO advantages.

Test infrastructure only (see ``oracle/__init__.py``).

Restates ``nemo_rl/algorithms/utils.py:104-198``
(``calculate_baseline_and_std_per_prompt``) and
``nemo_rl/algorithms/advantage_estimator.py:82-98``
(``GRPOAdvantageEstimator.compute_advantage``).
"""

from __future__ import annotations

import torch


def group_ids_by_prompt(prompts: torch.Tensor) -> torch.Tensor:
    """Group index per row: rows are in one group iff their prompt-token rows
    are exactly equal (``utils.py:132,144``).  Groups are numbered in order of
    first appearance; the numbering itself never reaches the outputs."""
    seen: dict[tuple, int] = {}
    ids = []
    if prompts.shape[0] == 0:
        return torch.zeros(0, dtype=torch.int64)
    for row in prompts.reshape(prompts.shape[0], -1).tolist():
        ids.append(seen.setdefault(tuple(row), len(seen)))
    return torch.tensor(ids, dtype=torch.int64)


def baseline_and_std_per_prompt(
    prompts, rewards, valid_mask, leave_one_out_baseline: bool = True, std_rewards=None
):
    """``utils.py:130-198``.

    For each group with more than one valid sample: ``n = n_valid - loo``;
    ``baseline = M @ (r * valid) / n`` with ``M = 1 - I`` (leave-one-out) or all
    ones; ``E2 = M @ (r_std^2 * valid) / n``; ``std = sqrt((E2 - E1^2) * n/(n-1))``
    with NaN -> 0.  Groups with at most one valid sample: baseline = reward,
    std = 0.  Every member of a group (valid or not) receives the values."""
    if std_rewards is None:
        std_rewards = rewards
    gid = group_ids_by_prompt(prompts)
    baseline = torch.zeros_like(rewards)
    std = torch.zeros_like(rewards)
    loo = int(leave_one_out_baseline)
    for g in range(int(gid.max().item()) + 1 if gid.numel() else 0):
        idx = torch.nonzero(gid == g).squeeze(-1)
        k = idx.numel()
        mix = (1 - torch.eye(k)) if leave_one_out_baseline else torch.ones(k, k)
        v = valid_mask[idx]
        if v.sum() <= 1:
            baseline[idx] = rewards[idx]
            continue
        n = v.float().sum() - loo
        e1 = torch.matmul(mix, rewards[idx] * v) / n
        e1_std = e1 if std_rewards is rewards else torch.matmul(mix, std_rewards[idx] * v) / n
        e2 = torch.matmul(mix, torch.pow(std_rewards[idx], 2) * v) / n
        baseline[idx] = e1
        std[idx] = ((e2 - e1_std.square()) * (n / (n - 1))).sqrt().nan_to_num(0)
    return baseline, std


def grpo_advantages(
    prompt_ids, rewards, mask, leave_one_out_baseline: bool = True, normalize_rewards: bool = True
):
    """``advantage_estimator.py:82-98``: ``adv = r - baseline``; where
    ``std > 0`` divide by ``std + 1e-6``; broadcast to ``mask.shape``."""
    baseline, std = baseline_and_std_per_prompt(
        prompt_ids, rewards, torch.ones_like(rewards), leave_one_out_baseline
    )
    adv = (rewards - baseline).unsqueeze(-1)
    if normalize_rewards:
        nz = std > 0
        adv[nz] = adv[nz] / (std.unsqueeze(-1)[nz] + 1e-6)
    return adv.expand(mask.shape)


def clip_advantages(adv, low=None, high=None):
    """``nemo_rl/algorithms/grpo.py:2302-2313``: optional clamp."""
    if low is None and high is None:
        return adv
    return torch.clamp(adv, min=low, max=high)


def seq_logprob_error_masking(prev_logprobs, generation_logprobs, token_mask, sample_mask, rewards, threshold):
    """``compute_and_apply_seq_logprob_error_masking`` (``nemo_rl/algorithms/grpo.py:2513-2640``)
    restated: returns ``(metrics dict, new sample_mask)``.  The reference's tests only mock this
    function, so it is pinned by brute-force loops on tiny inputs (``tests/test_oracle_advantage.py``)."""
    tm = token_mask[:, 1:].float()
    sm = sample_mask.float()
    lp_error = (generation_logprobs[:, 1:] - prev_logprobs[:, 1:]).abs()
    mask = tm * sm.unsqueeze(-1)
    denom = mask.sum(-1)
    valid = denom > 0
    err = torch.zeros_like(denom)
    stats = [0.0, 0.0, 0.0]
    if valid.any():
        num = (torch.exp(lp_error * mask) * mask).sum(-1)
        err[valid] = num[valid] / denom[valid].clamp(min=1)
        v = err[valid]
        stats = [v.max().item(), v.mean().item(), v.min().item()]
    after = list(stats)
    n_masked, pct, new_mask = 0, 0.0, sample_mask
    if threshold is not None:
        new_mask = (err <= threshold).float() * sm
        diff = sm - new_mask
        n_masked = int(diff.sum().item())
        if n_masked > 0:
            pct = int((rewards.view(-1)[diff.bool()] == 1).sum().item()) / n_masked
        kept = new_mask.bool() & valid
        after = [err[kept].max().item(), err[kept].mean().item(), err[kept].min().item()] if kept.sum() > 0 else [0.0, 0.0, 0.0]
    keys = ["max_seq_mult_prob_error", "mean_seq_mult_prob_error", "min_seq_mult_prob_error",
            "max_seq_mult_prob_error_after_mask", "mean_seq_mult_prob_error_after_mask", "min_seq_mult_prob_error_after_mask"]
    out = dict(zip(keys, stats + after))
    out["num_masked_seqs"] = n_masked
    out["masked_correct_pct"] = pct
    return out, new_mask


def dynamic_sampling_keep_indices(std):
    """``dynamic_sampling`` (``nemo_rl/algorithms/grpo.py:1752-1758``): the rows whose prompt group has a
    non-zero reward spread, ``arange(n)[std != 0.0]`` (ascending; NaN counts as non-zero)."""
    mask = std != 0.0
    return torch.arange(len(mask))[mask].tolist()
