"""Single-pass path: logits -> clipped-PG loss -> dlogits in one kernel.

``fused_logits_clipped_pg_loss`` does what ``prepare_loss_input`` + ``ClippedPGLossFn`` + the
backward of the logprob op do (``nemo_rl/algorithms/loss/wrapper.py:292-322``), but the logits are
read once and the gradient written once: the kernel keeps each row on chip between the
log-sum-exp and the gradient and evaluates the token's loss terms in between.  The gradient exists
as soon as the forward returns; ``backward`` hands it to autograd, rescaled in place on the device when
the upstream gradient is not the ``loss_scale`` it was computed with.
"""

from __future__ import annotations

from typing import Any, Optional

import torch

from ... import ops as _ops  # noqa: F401
from ..._deferred import pending_temperature
from ..._lib import NRL_TEMP_RCP
from .loss_functions import ClippedPGLossFn, _f32, _global_valid, metrics_record_to_dict

_OPS = torch.ops.rl_amd


def why_not_fusable(loss_fn, logits, data, sampling_params=None) -> Optional[str]:
    """None if the fused kernel covers this call, else the reason it does not."""
    from ..logits_sampling_utils import need_top_k_or_top_p_filtering

    if type(loss_fn) is not ClippedPGLossFn:
        return "not a ClippedPGLossFn"
    if getattr(loss_fn, "use_fused_linear_logprobs", False):
        return "the model already returned logprobs"
    if need_top_k_or_top_p_filtering(sampling_params):
        return "top-k/top-p filtering"
    if loss_fn.sequence_level_importance_ratios and not (loss_fn.disable_ppo_ratio or loss_fn.force_on_policy_ratio):
        return "sequence-level probability ratios"
    if loss_fn.force_on_policy_ratio and (
        loss_fn.sequence_level_importance_ratios or loss_fn.truncated_importance_sampling_type == "seq-mask-tis"
    ):
        return "sequence-level importance weights of the current policy"
    if loss_fn.positive_example_nll_weight > 0 and "rewards" in data:
        return "positive-example NLL term"
    if not isinstance(logits, torch.Tensor) or not logits.is_cuda or logits.dim() != 3:
        return "logits are not a [B, S, V] GPU tensor"
    elt = logits.element_size()
    if logits.dtype not in (torch.float32, torch.bfloat16, torch.float16) or logits.stride(2) != 1:
        return "unsupported logits dtype or layout"
    vocab = logits.shape[2]
    if (vocab * elt) % 16 or vocab * elt > 20480 * 16:
        return "vocabulary row does not fit the on-chip path"
    if logits.data_ptr() % 16 or (logits.stride(0) * elt) % 16 or (logits.stride(1) * elt) % 16:
        return "rows are not 16-byte aligned"
    if logits.shape[1] < data["input_ids"].shape[1]:
        return "logits shorter than input_ids"
    return None


def _rescale(dlogits, grad_loss, loss_scale):
    """The stored gradient was computed for an upstream factor of ``loss_scale``.  Whatever factor autograd
    actually delivers is applied in place by one kernel that reads it from the device: the host never waits
    for its value, no second ``[B, S, V]`` tensor exists, and when the two agree (the normal case) the kernel
    touches no memory."""
    if not isinstance(grad_loss, torch.Tensor) or not grad_loss.is_cuda:
        grad_loss = torch.as_tensor(grad_loss, dtype=torch.float32, device=dlogits.device)
    view = dlogits if dlogits.dim() == 3 else dlogits.unsqueeze(0)
    _OPS.scale_rows_(view, grad_loss, float(loss_scale))
    return dlogits


def _hand_over(ctx, grad_loss):
    dlogits, ctx.dlogits = ctx.dlogits, None
    if dlogits is None:
        raise RuntimeError("the single-pass loss hands its gradient buffer to autograd once; a second backward "
                           "through the same loss needs a new forward")
    return _rescale(dlogits, grad_loss, ctx.loss_scale)


class _FusedLogitsLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, targets, n_inner, prev, gen, ref, adv, token_mask, sample_mask, global_valid, iflags, fparams,
                loss_scale, in_place, temperature):
        x = logits.detach()
        if in_place:
            loss, lp, metrics = _OPS.fused_logits_grpo_loss_(
                x, targets, n_inner, prev, gen, ref, adv, token_mask, sample_mask, global_valid, iflags, fparams, loss_scale,
                temperature, NRL_TEMP_RCP)
            dlogits = x  # the caller declared the logits dead; their storage now holds the gradient
        else:
            loss, dlogits, lp, metrics = _OPS.fused_logits_grpo_loss(
                x, targets, n_inner, prev, gen, ref, adv, token_mask, sample_mask, global_valid, iflags, fparams, loss_scale,
                temperature, NRL_TEMP_RCP)
        ctx.dlogits = dlogits  # an intermediate, neither input nor output: held directly so it can be rescaled in place
        ctx.loss_scale = loss_scale
        ctx.mark_non_differentiable(lp, metrics)
        return loss, lp, metrics

    @staticmethod
    def backward(ctx, grad_loss, _g_lp, _g_metrics):
        return (_hand_over(ctx, grad_loss),) + (None,) * 14


def fused_logits_clipped_pg_loss(
    logits: torch.Tensor,
    data: Any,
    loss_fn: ClippedPGLossFn,
    global_valid_seqs,
    global_valid_toks,
    *,
    loss_scale: float = 1.0,
    in_place: bool = False,
):
    """``(loss, metrics)`` exactly as ``loss_fn(prepare_loss_input(logits, data, loss_fn))`` would return them.

    ``loss_scale`` is the gradient the caller will send into ``loss.backward()`` (1 for a plain
    ``backward()``, ``dp_size * cp_size`` when the worker scales the loss first); with it the stored
    gradient is final and ``backward`` moves no data.  ``in_place=True`` writes the gradient over the
    logits buffer instead of allocating a second ``[B, S, V]`` tensor (the logits are dead after the
    loss in the training step).  The metrics do not include values for masked positions, which are
    never evaluated."""
    reason = why_not_fusable(loss_fn, logits, data)
    if reason is not None:
        raise NotImplementedError(f"fused logits->loss path: {reason}")
    dev = logits.device
    ids = data["input_ids"].to(dev)
    if ids.dtype != torch.int64:
        ids = ids.long()
    n_inner = ids.shape[1] - 1
    beta = loss_fn.reference_policy_kl_penalty
    sample_mask_in = data["sample_mask"]
    prev = None if loss_fn.force_on_policy_ratio else _f32(data["prev_logprobs"][:, 1:], dev)
    ref = _f32(data["reference_policy_logprobs"][:, 1:], dev) if beta != 0 else None
    iflags, fparams = loss_fn._kernel_config(False)
    loss, _lp, metrics = _FusedLogitsLoss.apply(
        logits, ids[:, 1:], n_inner, prev, _f32(data["generation_logprobs"][:, 1:], dev), ref,
        _f32(data["advantages"][:, 1:], dev), _f32(data["token_mask"][:, 1:], dev), _f32(sample_mask_in, dev),
        _global_valid(global_valid_seqs, global_valid_toks, dev), iflags, fparams, float(loss_scale), bool(in_place),
        pending_temperature(logits),  # a divide apply_temperature_scaling left to this kernel
    )
    return loss, metrics_record_to_dict(metrics, loss_fn, sample_mask_in)


class _FusedPackedLogitsLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits2d, targets, cu, unpacked_seqlen, prev, gen, ref, adv, token_mask, sample_mask, global_valid, iflags,
                fparams, loss_scale, temperature):
        loss, dlogits, lp, metrics = _OPS.fused_packed_logits_grpo_loss(
            logits2d.detach(), targets, True, cu, unpacked_seqlen, prev, gen, ref, adv, token_mask, sample_mask, global_valid,
            iflags, fparams, loss_scale, temperature, NRL_TEMP_RCP)
        ctx.dlogits = dlogits  # an intermediate, neither input nor output: held directly so it can be rescaled in place
        ctx.loss_scale = loss_scale
        ctx.mark_non_differentiable(lp, metrics)
        return loss, lp, metrics

    @staticmethod
    def backward(ctx, grad_loss, _g_lp, _g_metrics):
        return (_hand_over(ctx, grad_loss),) + (None,) * 14


def why_not_fusable_packed(loss_fn, logits, data, sampling_params=None) -> Optional[str]:
    """As ``why_not_fusable`` for a packed ``[1, T, V]`` microbatch."""
    if not isinstance(logits, torch.Tensor) or logits.dim() != 3 or logits.shape[0] != 1:
        return "logits are not a packed [1, T, V] tensor"
    probe = dict(data)
    probe["input_ids"] = data["input_ids"][:, :1]  # the shape test of the unpacked path does not apply
    return why_not_fusable(loss_fn, logits, probe, sampling_params)


def fused_packed_logits_clipped_pg_loss(logits, data, loss_fn, cu_seqlens_q, cu_seqlens_q_padded, global_valid_seqs,
                                        global_valid_toks, *, loss_scale: float = 1.0):
    """``SequencePackingFusionLossWrapper.__call__`` (``loss/wrapper.py:169-228``) in one pass over the packed
    logits: ``prepare_packed_loss_input`` + ``ClippedPGLossFn`` + the backward of the packed logprob op."""
    from ...distributed.model_utils import _checked_cu_seqlens
    from .utils import _packed_targets

    reason = why_not_fusable_packed(loss_fn, logits, data)
    if reason is not None:
        raise NotImplementedError(f"fused packed logits->loss path: {reason}")

    dev = logits.device
    input_ids = data["input_ids"]
    x = logits.squeeze(0)
    targets = _packed_targets(input_ids, cu_seqlens_q, cu_seqlens_q_padded, x.shape[0], dev).reshape(-1)
    cu = _checked_cu_seqlens(cu_seqlens_q_padded, x.shape[0], targets.shape[0], dev)
    beta = loss_fn.reference_policy_kl_penalty
    sample_mask_in = data["sample_mask"]
    prev = None if loss_fn.force_on_policy_ratio else _f32(data["prev_logprobs"][:, 1:], dev)
    ref = _f32(data["reference_policy_logprobs"][:, 1:], dev) if beta != 0 else None
    iflags, fparams = loss_fn._kernel_config(False)
    loss, _lp, metrics = _FusedPackedLogitsLoss.apply(
        x, targets, cu, input_ids.shape[1], prev,
        _f32(data["generation_logprobs"][:, 1:], dev), ref, _f32(data["advantages"][:, 1:], dev),
        _f32(data["token_mask"][:, 1:], dev), _f32(sample_mask_in, dev),
        _global_valid(global_valid_seqs, global_valid_toks, dev), iflags, fparams, float(loss_scale),
        pending_temperature(logits),
    )
    return loss, metrics_record_to_dict(metrics, loss_fn, sample_mask_in)
