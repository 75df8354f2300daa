"""Driver-side pieces of the GRPO step that sit between the rollout and the loss
(``nemo_rl/algorithms/grpo.py``), on the device.

Only the numeric pieces of that file are mirrored: the per-sequence logprob-error mask
(``:2513-2640``), the advantage clamp (``:2302-2313``) and the dynamic-sampling filter that keeps the
prompt groups with a non-zero reward spread (``:1699-1830``).  The training loop and logging around
them stay with the reference.
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


def _cfg(config: Any, section: str, key: str, default: Any = None) -> Any:
    """``config.section.key`` or ``config[section][key]``, whichever the caller's config type offers."""
    sec = getattr(config, section, None) if not isinstance(config, dict) else config.get(section)
    if sec is None:
        return default
    if isinstance(sec, dict):
        return sec.get(key, default)
    return getattr(sec, key, default)


class _NoTimer:
    def time(self, _name):
        import contextlib

        return contextlib.nullcontext()


def dynamic_sampling(repeated_batch: Any, std: torch.Tensor, baseline: torch.Tensor, dynamic_sampling_num_gen_batches: int,
                     master_config: Any, timer: Any, batch_cache: Any = None):
    """``grpo.py:1699-1830`` (DAPO dynamic sampling): keep the samples whose prompt group has ``std != 0``,
    collect them in ``batch_cache`` across generation batches until ``num_prompts_per_step *
    num_generations_per_prompt`` are available, then cut to exactly that many.

    Returns ``(batch, is_batch_complete, batch_cache, metrics)``.  The selection ``arange(n)[std != 0]``
    is one compaction launch on the device; the bookkeeping is the reference's."""
    is_batch_complete = True
    train_prompts_size = _cfg(master_config, "grpo", "num_prompts_per_step") * _cfg(master_config, "grpo", "num_generations_per_prompt")
    repeated_batch["baseline"] = baseline
    repeated_batch["std"] = std
    total_rewards = repeated_batch["total_reward"]
    metrics: dict = {}
    if not _cfg(master_config, "grpo", "use_dynamic_sampling", False):
        return repeated_batch, is_batch_complete, batch_cache, metrics

    with (timer or _NoTimer()).time("dynamic_sampling"):
        dev = _device_for(std)
        keep = torch.ops.rl_amd.nonzero_indices(std.to(device=dev, dtype=torch.float32).reshape(-1)).tolist()
        filtered = repeated_batch.select_indices(keep)
        filtered["std"] = std[keep]
        filtered["baseline"] = baseline[keep]
        # the unfiltered rewards stay under total_reward, the kept ones go to filtered_reward (``:1764-1767``)
        filtered_rewards = filtered["total_reward"]
        filtered["total_reward"] = total_rewards
        filtered["filtered_reward"] = filtered_rewards
        if filtered.size > 0:
            if batch_cache is not None:
                filtered = type(filtered).from_batches(
                    [batch_cache, filtered],
                    allow_missing_packed_tensors=bool(_cfg(master_config, "grpo", "deduplicate_multimodal_data", False)))
            batch_cache = filtered
        n_kept = filtered.size
        print(f"Detected {n_kept} prompts with non-zero std; {train_prompts_size} are required and used for training.")
        if n_kept < train_prompts_size:
            max_batches = _cfg(master_config, "grpo", "dynamic_sampling_max_gen_batches")
            assert max_batches is not None and max_batches > 0, (
                "When using grpo.use_dynamic_sampling, grpo.dynamic_sampling_max_gen_batches must be > 0"
            )
            if dynamic_sampling_num_gen_batches <= max_batches:
                print(f"Generation sample buffer size: {n_kept} is smaller than train_prompts_size: {train_prompts_size}. "
                      f"Processed {dynamic_sampling_num_gen_batches} batches so far out of {max_batches}.")
                is_batch_complete = False
            else:
                raise ValueError(
                    f"Dynamic sampling has reached the maximum allowed number of batches ({max_batches}). Consider evaluating "
                    "the complexity of your data or adjusting the num_prompts_per_step or num_generations_per_prompt "
                    "parameters to enhance the diversity of the samples."
                )
        else:
            metrics["dynamic_sampling_num_discarded_valid_samples"] = n_kept - train_prompts_size
            filtered = filtered.slice(0, train_prompts_size)
    return filtered, is_batch_complete, batch_cache, metrics
