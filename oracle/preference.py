"""Oracle: preference (reward-model), DPO and per-sample NLL losses.

Test infrastructure only (see ``oracle/__init__.py``).

Restates, with torch autograd supplying every gradient,
``nemo_rl/algorithms/loss/loss_functions.py:818-842`` (``NLLLossFn``, both
branches), ``:877-946`` (``PreferenceLossFn``) and ``:1025-1106``
(``DPOLossFn``).

Pins (``tests/test_oracle_preference.py``): the three closed-form cases of the
reference's own tests (``tests/unit/algorithms/test_loss_functions.py:133-370``:
zero logits against a zero reference give ``-logsigmoid(0)``; the SFT term is
the chosen rows' summed / averaged NLL; with the preference weight at zero the
loss is the rescaled ``NLLLossFn`` value) and a loop-per-pair brute force on
random inputs that includes fractional sample masks, which enter the
preference term squared.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

import torch

from .loss import masked_mean


@dataclass
class DPOConfig:
    """``DPOLossConfig`` (``loss_functions.py:949-954``)."""

    reference_policy_kl_penalty: float = 0.05
    preference_loss_weight: float = 1.0
    sft_loss_weight: float = 0.0
    preference_average_log_probs: bool = False
    sft_average_log_probs: bool = False


def nll_loss_rows(next_token_logprobs, data, average_log_probs: bool = False):
    """``NLLLossFn(..., dpo_loss=True)`` (``loss_functions.py:823-829``): one value per sample."""
    mask = data["token_mask"][:, 1:] * data["sample_mask"].unsqueeze(-1)
    n = torch.sum(mask, -1)
    loss = -torch.sum(next_token_logprobs * mask, dim=-1)
    if average_log_probs:
        loss = loss / n.clamp(min=1)
    return loss, {
        "loss": loss,
        "num_unmasked_tokens": mask.sum().item(),
        "num_valid_samples": data["sample_mask"].sum().item(),
    }


def _preference_terms(rewards, sample_mask, global_valid_seqs, beta: float = 1.0):
    """``PreferenceLossFn._preference_loss`` (``loss_functions.py:881-917``): rows alternate
    chosen / rejected; every mean is normalised by half the global number of valid samples."""
    chosen, rejected = rewards[::2], rewards[1::2]
    per_sample = -torch.nn.functional.logsigmoid(beta * (chosen - rejected)) * sample_mask[::2]
    half = global_valid_seqs / 2
    return (
        masked_mean(per_sample, sample_mask[::2], global_normalization_factor=half),
        masked_mean(chosen > rejected, sample_mask[::2], global_normalization_factor=half),
        masked_mean(chosen, sample_mask[::2], global_normalization_factor=half),
        masked_mean(rejected, sample_mask[1::2], global_normalization_factor=half),
    )


def preference_loss(logits, data: Mapping[str, Any], global_valid_seqs):
    """``PreferenceLossFn.__call__`` (``loss_functions.py:919-946``): ``logits [B, 1]`` are rewards."""
    sample_mask = data["sample_mask"]
    loss, acc, rc, rr = _preference_terms(logits.squeeze(-1), sample_mask, global_valid_seqs)
    return loss, {
        "loss": loss.item(),
        "accuracy": acc.item(),
        "rewards_chosen_mean": rc.item(),
        "rewards_rejected_mean": rr.item(),
        "num_valid_samples": (sample_mask.sum() / 2).item(),
    }


def dpo_loss(cfg: DPOConfig, next_token_logprobs, data: Mapping[str, Any], global_valid_seqs):
    """``DPOLossFn.__call__`` (``loss_functions.py:1034-1106``).  The reference logprobs are read
    at ``[:, :-1]`` (``:1043``), not at ``[:, 1:]`` as in the policy-gradient loss."""
    sample_mask = data["sample_mask"]
    sft_chosen = torch.tensor(0.0)
    if cfg.sft_loss_weight > 0:
        rows, _ = nll_loss_rows(next_token_logprobs, data, cfg.sft_average_log_probs)
        sft_chosen = masked_mean(rows[::2], sample_mask[::2], global_normalization_factor=global_valid_seqs / 2)
    token_mask = data["token_mask"][:, 1:]
    diff = (next_token_logprobs - data["reference_policy_logprobs"][:, :-1]) * token_mask
    rewards = diff.sum(-1)
    if cfg.preference_average_log_probs:
        rewards = rewards / token_mask.sum(-1).clamp(min=1)
    pref, acc, rc, rr = _preference_terms(rewards, sample_mask, global_valid_seqs, cfg.reference_policy_kl_penalty)
    loss = cfg.sft_loss_weight * sft_chosen + cfg.preference_loss_weight * pref
    return loss, {
        "loss": loss.item(),
        "sft_loss": sft_chosen.item(),
        "preference_loss": pref.item(),
        "accuracy": acc.item(),
        "rewards_chosen_mean": rc.item(),
        "rewards_rejected_mean": rr.item(),
        "num_valid_samples": (sample_mask.sum() / 2).item(),
    }
