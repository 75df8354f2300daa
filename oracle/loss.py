"""Oracle: clipped policy-gradient (GRPO family) loss and its helpers.

Test infrastructure only (see ``oracle/__init__.py``).

Restates, with torch autograd supplying every gradient,
``nemo_rl/algorithms/utils.py:42-101`` (``calculate_kl``), ``:212-224``
(``masked_mean``) and ``nemo_rl/algorithms/loss/loss_functions.py:111-164``
(config defaults), ``:228-324`` (constructor checks), ``:374-788`` (the loss).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional

import torch


def masked_mean(values, mask, dim=None, global_normalization_factor=None):
    """``utils.py:219-224``: ``sum(values*mask) / (norm + 1e-8)`` with
    ``norm = sum(mask)`` unless a global factor is given."""
    norm = torch.sum(mask, dim=dim) if global_normalization_factor is None else global_normalization_factor
    return torch.sum(values * mask, dim=dim) / (norm + 1e-8)


def calculate_kl(
    logprobs,
    logprobs_reference,
    kl_type: str = "k3",
    input_clamp_value: Optional[float] = 20.0,
    output_clamp_value: Optional[float] = 10.0,
    importance_sampling_weights=None,
):
    """``utils.py:72-101``.  ``logr = ref - lp``; optional clamp of ``logr`` to
    +-input_clamp, detaching the importance weight wherever the clamp changed
    the value; k1 = -logr, k2 = logr^2/2, k3 = exp(logr) - 1 - logr; times the
    weight; optional clamp of the result to +-output_clamp."""
    logr = logprobs_reference - logprobs
    if input_clamp_value is not None:
        clipped = logr.clamp(min=-input_clamp_value, max=input_clamp_value)
        if importance_sampling_weights is not None:
            importance_sampling_weights = torch.where(
                logr == clipped, importance_sampling_weights, importance_sampling_weights.detach()
            )
        logr = clipped
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


@dataclass
class LossConfig:
    """Field names and defaults of ``ClippedPGLossConfig``
    (``loss_functions.py:111-164``)."""

    disable_ppo_ratio: bool = False
    token_level_loss: bool = True
    sequence_level_importance_ratios: bool = False
    ratio_clip_min: float = 0.2
    ratio_clip_max: float = 0.2
    ratio_clip_c: Optional[float] = None
    reference_policy_kl_penalty: float = 0.01
    reference_policy_kl_type: str = "k3"
    kl_input_clamp_value: Optional[float] = 20.0
    kl_output_clamp_value: Optional[float] = 10.0
    use_kl_in_reward: bool = False
    use_importance_sampling_correction: bool = False
    truncated_importance_sampling_type: Optional[str] = None
    truncated_importance_sampling_ratio: Optional[float] = None
    truncated_importance_sampling_ratio_min: Optional[float] = None
    use_on_policy_kl_approximation: bool = False
    force_on_policy_ratio: bool = False
    use_cispo: bool = False
    positive_example_nll_weight: float = 0.0


def check_config(cfg: LossConfig) -> None:
    """Constructor assertions, ``loss_functions.py:265-324``."""
    if cfg.sequence_level_importance_ratios:
        assert not cfg.token_level_loss
    if cfg.use_cispo:
        assert not cfg.disable_ppo_ratio
        assert not cfg.force_on_policy_ratio
        assert not cfg.sequence_level_importance_ratios
        assert cfg.ratio_clip_c is None
        assert cfg.token_level_loss
    kind = cfg.truncated_importance_sampling_type
    if kind is not None:
        assert cfg.use_importance_sampling_correction
        assert kind in ("tis", "icepop", "seq-mask-tis")
        hi = cfg.truncated_importance_sampling_ratio
        lo = cfg.truncated_importance_sampling_ratio_min
        assert hi is not None and hi > 0
        if lo is not None:
            assert lo <= hi
        if kind in ("icepop", "seq-mask-tis"):
            assert lo is not None
        if kind == "seq-mask-tis":
            assert not cfg.sequence_level_importance_ratios


def _finite_or_zero(x):
    return torch.nan_to_num(x, nan=0.0, posinf=0.0, neginf=0.0)


def clipped_pg_loss(
    cfg: LossConfig,
    next_token_logprobs: torch.Tensor,
    data: Mapping[str, Any],
    global_valid_seqs,
    global_valid_toks,
):
    """``ClippedPGLossFn.__call__`` (``loss_functions.py:382-788``).

    Returns ``(loss, metrics)`` where ``metrics`` holds Python floats."""
    check_config(cfg)
    beta = 0 if cfg.use_kl_in_reward else cfg.reference_policy_kl_penalty  # :240-242
    token_level = cfg.token_level_loss
    kl_type = cfg.reference_policy_kl_type

    lp = next_token_logprobs
    tm = data["token_mask"][:, 1:]
    sm = data["sample_mask"]
    adv = data["advantages"][:, 1:]
    gen = data["generation_logprobs"][:, 1:]
    prev = lp.detach() if cfg.force_on_policy_ratio else data["prev_logprobs"][:, 1:]  # :386-402
    mask = tm * sm.unsqueeze(-1)
    gt, gs = global_valid_toks, global_valid_seqs

    def tok_mean(v):
        return masked_mean(v, mask, global_normalization_factor=gt)

    def seq_mean(v):
        return masked_mean(masked_mean(v, tm, dim=-1), sm, global_normalization_factor=gs)

    # --- diagnostics on (gen, prev), :406-466 ---
    mult_prob_error = tok_mean(torch.exp(torch.abs(gen - prev) * mask)).item()
    gen_kl = tok_mean(calculate_kl(gen, prev, kl_type, None, None)).item()
    policy_kl = tok_mean(calculate_kl(prev, gen, kl_type, None, None)).item()
    log_mix = torch.log(0.5 * torch.exp(prev) + 0.5 * torch.exp(gen))
    kl_prev_mix = torch.exp(prev - log_mix) - (prev - log_mix) - 1
    kl_gen_mix = torch.exp(gen - log_mix) - (gen - log_mix) - 1
    js = tok_mean(0.5 * kl_prev_mix + 0.5 * kl_gen_mix).item()

    # --- KL to the reference policy, :469-517 ---
    if beta != 0:
        ref = data["reference_policy_logprobs"][:, 1:]
        lpu = data.get("curr_logprobs_unfiltered", lp)
        if cfg.use_on_policy_kl_approximation:
            w_kl = torch.exp(lpu - gen)
        else:
            w_kl = torch.exp(lpu - lpu.detach())
        w_kl = _finite_or_zero(w_kl)
        kl = beta * calculate_kl(
            lpu, ref, kl_type, cfg.kl_input_clamp_value, cfg.kl_output_clamp_value, w_kl
        )
        kl = tok_mean(kl) if token_level else seq_mean(kl)
    else:
        kl = torch.tensor(0.0)

    # --- probability ratios, :520-543 ---
    if cfg.force_on_policy_ratio:
        ratios = (lp - lp.detach()).exp()
        ratios_clamped = ratios
    elif not cfg.disable_ppo_ratio:
        log_ratios = lp - prev
        if cfg.sequence_level_importance_ratios:
            per_seq = masked_mean(log_ratios, tm, dim=-1).unsqueeze(-1).exp()
            ratios = per_seq.repeat(1, adv.shape[1])
        else:
            ratios = log_ratios.exp()
        ratios_clamped = ratios.clamp(1.0 - cfg.ratio_clip_min, 1.0 + cfg.ratio_clip_max)
    else:
        ratios = lp
        ratios_clamped = lp

    # --- surrogate, :545-561 ---
    if cfg.use_cispo:
        clip_loss = -adv * ratios_clamped.detach() * lp
    else:
        clip_loss = torch.max(-adv * ratios, -adv * ratios_clamped)
    if cfg.ratio_clip_c is not None:
        assert cfg.ratio_clip_c > 1
        clip_loss = torch.where(adv < 0, torch.min(clip_loss, -adv * cfg.ratio_clip_c), clip_loss)

    # --- off-policy importance weights, :568-676 ---
    extra = {}
    if cfg.sequence_level_importance_ratios:
        w_is = _finite_or_zero(torch.exp(((prev - gen) * mask).sum(dim=-1)).detach()).unsqueeze(-1)
    else:
        w_is = _finite_or_zero(torch.exp(prev - gen))
    hi = cfg.truncated_importance_sampling_ratio
    lo = cfg.truncated_importance_sampling_ratio_min
    kind = cfg.truncated_importance_sampling_type
    if hi is not None:
        if kind == "tis":
            floor = 0.0 if lo is None else lo
            oob = (w_is > hi) | (w_is < floor)
            extra["is_oob_ratio"] = tok_mean(oob.float()).item()
            w_is = torch.clamp(w_is, min=floor, max=hi)
        elif kind == "icepop":
            inside = (w_is >= lo) & (w_is <= hi)
            extra["is_oob_ratio"] = tok_mean((~inside).float()).item()
            w_is = torch.where(inside, w_is, torch.zeros_like(w_is))
        elif kind == "seq-mask-tis":
            geo = torch.exp(masked_mean(_finite_or_zero(prev - gen), tm, dim=-1)).detach()
            seq_keep = ((geo >= lo) & (geo <= hi)).float()
            extra["is_oob_ratio"] = masked_mean(
                1.0 - seq_keep, sm, global_normalization_factor=gs
            ).item()
            w_is = w_is * seq_keep.unsqueeze(-1)
        else:
            raise ValueError(f"Invalid truncated importance sampling type: {kind}")
    w_use = w_is if cfg.use_importance_sampling_correction else torch.ones_like(prev)

    # --- reductions, :678-717 ---
    actor = tok_mean(w_use * clip_loss) if token_level else seq_mean(w_use * clip_loss)
    if cfg.sequence_level_importance_ratios:
        sample_ratio = masked_mean(w_is, sm, global_normalization_factor=gs)
    else:
        sample_ratio = tok_mean(w_is)
    with torch.no_grad():
        entropy = -tok_mean(torch.exp(lp - gen) * lp)

    # --- positive-example NLL, :723-733 ---
    nll = torch.tensor(0.0)
    if cfg.positive_example_nll_weight > 0 and "rewards" in data:
        good = mask * (data["rewards"] > 0).float().unsqueeze(-1)
        n_good = good.sum()
        if n_good > 0:
            nll = masked_mean(-lp, good, global_normalization_factor=n_good)

    loss = actor + kl + cfg.positive_example_nll_weight * nll

    # --- ratio statistics, :736-762 ---
    with torch.no_grad():
        r_mean = tok_mean(ratios.detach()).item()
        rc_mean = tok_mean(ratios_clamped.detach()).item()
        sel = mask.bool()
        r_sel, rc_sel = ratios.detach()[sel], ratios_clamped.detach()[sel]
        if r_sel.numel() > 0:
            r_min, r_max = r_sel.min().item(), r_sel.max().item()
            rc_min, rc_max = rc_sel.min().item(), rc_sel.max().item()
        else:
            r_min = rc_min = float("inf")
            r_max = rc_max = float("-inf")

    metrics = {
        "loss": loss.item(),
        "probs_ratio": r_mean,
        "probs_ratio_clamped": rc_mean,
        "probs_ratio_min": r_min,
        "probs_ratio_max": r_max,
        "probs_ratio_clamped_min": rc_min,
        "probs_ratio_clamped_max": rc_max,
        "kl_penalty": kl.item() / beta if kl else 0,  # :777
        "token_mult_prob_error": mult_prob_error,
        "gen_kl_error": gen_kl,
        "policy_kl_error": policy_kl,
        "js_divergence_error": js,
        "sampling_importance_ratio": sample_ratio.item(),
        "num_valid_samples": sm.sum().item(),
        "approx_entropy": entropy.item(),
        **extra,
        "positive_nll_loss": nll.item(),
    }
    return loss, metrics


_MIN_METRICS = ("probs_ratio_min", "probs_ratio_clamped_min")
_MAX_METRICS = ("probs_ratio_max", "probs_ratio_clamped_max")


def sequence_packing_loss(cfg: LossConfig, packed_logits, data, cu_seqlens, cu_seqlens_padded, global_valid_seqs,
                          global_valid_toks, logprob_fn):
    """``SequencePackingLossWrapper.__call__`` (``loss/wrapper.py:65-166``) around ``prepare_loss_input`` +
    ``ClippedPGLossFn`` at CP = 1: sequence ``i`` owns the packed positions
    ``[cu_padded[i], cu_padded[i+1])``, its data rows are cut to the unpadded length (:87-93), the loss is
    called once per sequence and summed (:136), metrics are summed except the ratio extrema, which are
    combined with min / max while infinite sentinels of empty sequences are skipped (:137-164).
    ``logprob_fn(input_ids, logits)`` is the oracle's next-token logprob."""
    cup = cu_seqlens if cu_seqlens_padded is None else cu_seqlens_padded
    total, merged = 0, {}
    for i in range(len(cu_seqlens) - 1):
        n_real = int(cu_seqlens[i + 1] - cu_seqlens[i])
        start, n_pad = int(cup[i]), int(cup[i + 1] - cup[i])
        row = {k: (v[i : i + 1, :n_real] if isinstance(v, torch.Tensor) and v.ndim > 1 and v.shape[1] > 1 else
                   (v[i : i + 1] if isinstance(v, torch.Tensor) else v)) for k, v in data.items()}
        piece = packed_logits.narrow(1, start, n_pad)
        lp = logprob_fn(row["input_ids"], piece)
        loss, metrics = clipped_pg_loss(cfg, lp, row, global_valid_seqs, global_valid_toks)
        total = total + loss
        for k, v in metrics.items():
            if k in _MIN_METRICS:
                merged.setdefault(k, float("inf"))
                if v not in (float("inf"), float("-inf")):
                    merged[k] = min(merged[k], v)
            elif k in _MAX_METRICS:
                merged.setdefault(k, float("-inf"))
                if v not in (float("inf"), float("-inf")):
                    merged[k] = max(merged[k], v)
            else:
                merged[k] = merged.get(k, 0) + v
    return total, merged


def nll_loss(next_token_logprobs, data, global_valid_toks):
    """``NLLLossFn`` scalar branch (``loss_functions.py:818-842``)."""
    mask = data["token_mask"][:, 1:] * data["sample_mask"].unsqueeze(-1)
    loss = -masked_mean(next_token_logprobs, mask, global_normalization_factor=global_valid_toks)
    return loss, {
        "loss": loss.item(),
        "num_unmasked_tokens": mask.sum().item(),
        "num_valid_samples": data["sample_mask"].sum().item(),
    }
