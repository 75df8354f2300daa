"""Helpers around the loss (counterparts of ``nemo_rl/algorithms/utils.py:42-274``).

``calculate_baseline_and_std_per_prompt`` runs the HIP grouping / statistics kernels.  The other
helpers are thin [B, S]-sized tensor expressions kept for API compatibility; inside
``ClippedPGLossFn`` their arithmetic is part of the fused loss kernel instead.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import ops as _ops  # noqa: F401

_OPS = torch.ops.rl_amd


def _gpu_device() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("rl_amd needs an MI355X: no GPU is visible and there is no CPU fallback")
    return torch.device("cuda", torch.cuda.current_device())


def calculate_kl(
    logprobs: torch.Tensor,
    logprobs_reference: torch.Tensor,
    kl_type: str = "k3",
    input_clamp_value: float | None = 20.0,
    output_clamp_value: float | None = 10.0,
    importance_sampling_weights: torch.Tensor | None = None,
) -> torch.Tensor:
    """Per-token k1 / k2 / k3 estimate of KL(policy || reference), ``utils.py:42-101``."""
    logr = logprobs_reference - logprobs
    if input_clamp_value is not None:
        bounded = logr.clamp(min=-input_clamp_value, max=input_clamp_value)
        if importance_sampling_weights is not None:
            importance_sampling_weights = torch.where(
                logr == bounded, importance_sampling_weights, importance_sampling_weights.detach()
            )
        logr = bounded
    if kl_type == "k1":
        kl = -logr
    elif kl_type == "k2":
        kl = torch.square(logr) / 2
    elif kl_type == "k3":
        kl = torch.exp(logr) - 1 - logr
    else:
        raise ValueError(f"Invalid KL type: {kl_type}")
    if importance_sampling_weights is not None:
        kl = importance_sampling_weights * kl
    if output_clamp_value is not None:
        kl = kl.clamp(min=-output_clamp_value, max=output_clamp_value)
    return kl


def masked_mean(
    values: torch.Tensor,
    mask: torch.Tensor,
    dim: Optional[int] = None,
    global_normalization_factor: Optional[torch.Tensor | float] = None,
):
    """``sum(values * mask) / (norm + 1e-8)``, ``utils.py:212-224``."""
    norm = torch.sum(mask, dim=dim) if global_normalization_factor is None else global_normalization_factor
    return torch.sum(values * mask, dim=dim) / (norm + 1e-8)


def mask_out_neg_inf_logprobs(logprobs: torch.Tensor, mask: torch.Tensor, logprobs_name: str) -> torch.Tensor:
    """``utils.py:227-257``: positions that are masked out or infinite become 0 (with the reference's
    warning when valid tokens are affected)."""
    is_inf = torch.isinf(logprobs)
    # both counts in one transfer: the warning is the only reason this function waits for the device at all
    hit, valid = torch.stack([(is_inf & mask.bool()).sum(), mask.sum().to(torch.int64)]).tolist()
    if hit > 0:
        print(
            f"[WARNING]: {hit}/{valid} valid tokens have -inf in {logprobs_name} "
            "(policy top-k/top-p mismatch). Masking out these positions."
        )
    keep = mask * (~is_inf).float()
    return torch.where(keep.bool(), logprobs, 0.0)


def calculate_baseline_and_std_per_prompt(
    prompts: torch.Tensor,
    rewards: torch.Tensor,
    valid_mask: torch.Tensor,
    leave_one_out_baseline: bool = True,
    std_rewards: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``utils.py:104-198``: per-prompt (leave-one-out) baseline and std; results come back on the
    device of ``rewards``.  Inputs that live on the host (the driver's default) are staged to the GPU."""
    baseline, std, _, _ = _group_stats(prompts, rewards, valid_mask, leave_one_out_baseline, std_rewards, False)
    return baseline, std


def _group_stats(prompts, rewards, valid_mask, leave_one_out, std_rewards, normalize):
    home = rewards.device
    dev = home if home.type == "cuda" else _gpu_device()
    if rewards.numel() == 0:
        z = torch.zeros_like(rewards)
        return z, z.clone(), z.clone(), torch.zeros(0, dtype=torch.int32, device=home)
    out = _OPS.group_baseline_std(
        prompts.to(dev, torch.int64),
        rewards.to(dev, torch.float32),
        valid_mask.to(dev, torch.float32),
        None if std_rewards is None or std_rewards is rewards else std_rewards.to(dev, torch.float32),
        bool(leave_one_out),
        bool(normalize),
    )
    baseline, std, adv, group = (t.to(home) for t in out)
    return baseline.to(rewards.dtype), std.to(rewards.dtype), adv.to(rewards.dtype), group
