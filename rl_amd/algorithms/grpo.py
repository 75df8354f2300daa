"""Driver-side pieces of the GRPO step that sit between the rollout and the loss
(``nemo_rl/algorithms/grpo.py``), on the device.

Only the numeric kernels of that file are mirrored: the per-sequence logprob-error mask
(``:2513-2640``) and the advantage clamp (``:2302-2313``).  The training loop, batching and
logging around them stay with the reference.
"""

from __future__ import annotations

from typing import Any, Optional

import torch

from .. import ops  # noqa: F401  (registers torch.ops.rl_amd)


def _device_for(t: torch.Tensor) -> torch.device:
    if t.is_cuda:
        return t.device
    if not torch.cuda.is_available():
        raise RuntimeError("rl_amd: the GRPO kernels run on the GPU only and no GPU is visible")
    return torch.device("cuda", torch.cuda.current_device())


def compute_and_apply_seq_logprob_error_masking(
    train_data: Any,
    rewards: torch.Tensor,
    seq_logprob_error_threshold: Optional[float],
) -> dict:
    """``grpo.py:2513-2640``: per-sequence multiplicative probability error between the generation
    engine's and the policy's logprobs, its max / mean / min, and -- with a threshold -- the updated
    ``train_data["sample_mask"]`` that drops the sequences above it.  One launch pair and one
    device-to-host copy instead of a dozen ``[B, S]`` passes and ``.item()`` calls."""
    token_mask = train_data["token_mask"]
    sample_mask = train_data["sample_mask"]
    dev = _device_for(train_data["prev_logprobs"])
    f32 = lambda t: t.to(device=dev, dtype=torch.float32)  # noqa: E731
    _err, mask_out, record = torch.ops.rl_amd.seq_logprob_error(
        f32(train_data["prev_logprobs"]), f32(train_data["generation_logprobs"]), f32(token_mask), f32(sample_mask).reshape(-1),
        f32(rewards).reshape(-1) if rewards is not None else None,
        float(seq_logprob_error_threshold) if seq_logprob_error_threshold is not None else None)
    rec = record.tolist()
    if seq_logprob_error_threshold is not None:
        train_data["sample_mask"] = mask_out.to(sample_mask.device)
    return {
        "max_seq_mult_prob_error": rec[0],
        "mean_seq_mult_prob_error": rec[1],
        "min_seq_mult_prob_error": rec[2],
        "max_seq_mult_prob_error_after_mask": rec[3],
        "mean_seq_mult_prob_error_after_mask": rec[4],
        "min_seq_mult_prob_error_after_mask": rec[5],
        "num_masked_seqs": int(rec[6]),
        "masked_correct_pct": rec[7],
    }


def _clip_grpo_advantages(advantages: torch.Tensor, grpo_config: Any) -> torch.Tensor:
    """``grpo.py:2302-2313``: clamp normalised advantages when bounds are configured."""
    get = grpo_config.get if hasattr(grpo_config, "get") else lambda k, d=None: getattr(grpo_config, k, d)
    clip_low, clip_high = get("advantage_clip_low", None), get("advantage_clip_high", None)
    if clip_low is not None:
        advantages = advantages.clamp(min=clip_low)
    if clip_high is not None:
        advantages = advantages.clamp(max=clip_high)
    return advantages
