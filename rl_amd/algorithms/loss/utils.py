"""Turns model output (logits) into the keyword arguments of a loss function
(counterpart of ``nemo_rl/algorithms/loss/utils.py:37-120, 214-385``, LOGPROB input type)."""

from __future__ import annotations

from typing import Any, Optional

import torch

from ...distributed.model_utils import (
    from_parallel_logits_to_logprobs_packed_sequences,
    get_next_token_logprobs_from_logits,
)
from ..logits_sampling_utils import TrainingSamplingParams, need_top_k_or_top_p_filtering
from ..utils import mask_out_neg_inf_logprobs
from .interfaces import LossFunction, LossInputType


def _wants_unfiltered_kl(loss_fn) -> bool:
    return hasattr(loss_fn, "reference_policy_kl_penalty") and loss_fn.reference_policy_kl_penalty != 0


def prepare_loss_input(
    logits: torch.Tensor,
    data: Any,
    loss_fn: LossFunction,
    vocab_parallel_rank: Optional[int] = None,
    vocab_parallel_group: Optional[Any] = None,
    context_parallel_group: Optional[Any] = None,
    sampling_params: Optional[TrainingSamplingParams] = None,
    d2t: Optional[torch.Tensor] = None,
    chunk_size: Optional[int] = None,
) -> tuple[dict[str, Any], Any]:
    """``loss/utils.py:37-120``.  Returns ``({"next_token_logprobs": [B, S-1]}, data)``; with top-k /
    top-p active ``data`` gains ``curr_logprobs_unfiltered`` when the loss has a KL penalty."""
    if loss_fn.input_type != LossInputType.LOGPROB or getattr(loss_fn, "use_fused_linear_logprobs", False):
        # these readers have no fused temperature (the loss takes the logits as they are, or reduces them with
        # kernels that do not scale): a divide left to the kernels by deferred_temperature() is applied here
        from ...temperature import materialise_pending

        logits = materialise_pending(logits)
    if loss_fn.input_type == LossInputType.LOGIT:
        return {"logits": logits}, data
    if loss_fn.input_type == LossInputType.DISTILLATION:  # ``loss/utils.py:122-141``
        from ...distributed.model_utils import get_distillation_topk_logprobs_from_logits

        student, teacher, h_all = get_distillation_topk_logprobs_from_logits(
            student_logits=logits,
            teacher_topk_logits=data["teacher_topk_logits"],
            teacher_topk_indices=data["teacher_topk_indices"],
            zero_outside_topk=loss_fn.zero_outside_topk,
            calculate_entropy=loss_fn.zero_outside_topk and loss_fn.kl_type != "forward",
            vocab_parallel_rank=vocab_parallel_rank,
            vocab_parallel_group=vocab_parallel_group,
            context_parallel_group=context_parallel_group,
        )
        return {"student_topk_logprobs": student, "teacher_topk_logprobs": teacher, "H_all": h_all}, data
    if loss_fn.input_type != LossInputType.LOGPROB:
        raise ValueError(f"Unknown loss function input type: {loss_fn.input_type}")

    def logprobs_with(params, chunk):
        return get_next_token_logprobs_from_logits(
            input_ids=data["input_ids"],
            next_token_logits=logits,
            seq_index=data.get("seq_index", None),
            vocab_parallel_rank=vocab_parallel_rank,
            vocab_parallel_group=vocab_parallel_group,
            context_parallel_group=context_parallel_group,
            sampling_params=params,
            chunk_size=chunk,
        )

    if getattr(loss_fn, "use_fused_linear_logprobs", False):
        # the model forward already produced next-token logprobs (loss/utils.py:77-83)
        logprobs = logits.to(torch.float32)[:, : data["input_ids"].shape[1] - 1]
    else:
        logprobs = logprobs_with(sampling_params, chunk_size)  # loss/utils.py:85-94: the main call chunks

    if need_top_k_or_top_p_filtering(sampling_params):
        mask = data["token_mask"] * data["sample_mask"].unsqueeze(-1)
        logprobs = mask_out_neg_inf_logprobs(logprobs, mask[:, 1:].to(logprobs.device), "curr_logprobs")
        if _wants_unfiltered_kl(loss_fn):
            data["curr_logprobs_unfiltered"] = logprobs_with(None, None)  # :108-118: the unfiltered pass does not
    return {"next_token_logprobs": logprobs}, data


def _pack_input_ids(
    input_ids: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_q_padded: torch.Tensor,
    cp_rank: int = 0,
    cp_size: int = 1,
    roll_shift: int = 0,
) -> torch.Tensor:
    """``loss/utils.py:214-261`` with ``cp_size == 1``: ``[B, S]`` ids -> ``[1, T]`` packed ids.  Each
    sequence fills its padded span (``min(actual_len, S)`` tokens, zero tail) and is rolled inside it.
    The boundaries are read from the host once and the packing is a single gather."""
    if cp_size != 1:
        raise NotImplementedError("context parallelism spans more than one GPU")
    cu = cu_seqlens_q.detach().to("cpu", torch.int64)
    cup = cu_seqlens_q_padded.detach().to("cpu", torch.int64)
    batch, width = input_ids.shape
    total = int(cup[-1])
    span = cup[1:] - cup[:-1]
    n_real = torch.minimum(cu[1:] - cu[:-1], torch.tensor(width))
    seq_of = torch.repeat_interleave(torch.arange(batch), span, output_size=int(span.sum()))
    offset = torch.arange(int(span.sum())) - torch.repeat_interleave(cup[:-1] - cup[0], span)
    src = offset - roll_shift  # element j of the rolled span comes from (j - shift) mod span
    src = torch.remainder(src, span[seq_of].clamp(min=1))
    valid = src < n_real[seq_of]
    dev = input_ids.device
    flat = input_ids[seq_of.to(dev), src.clamp(max=width - 1).to(dev)] * valid.to(dev)
    packed = torch.zeros(total, dtype=input_ids.dtype, device=dev)
    packed[int(cup[0]) : int(cup[0]) + flat.numel()] = flat
    return packed.unsqueeze(0)


def _packed_targets(input_ids: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_q_padded: torch.Tensor,
                    total: int, dev: torch.device) -> torch.Tensor:
    """``_pack_input_ids(..., roll_shift=-1)`` padded to the ``total`` packed positions, ``[1, total]`` on ``dev``,
    by one kernel that reads the boundaries where they are: with boundaries that live on the GPU (as the attention
    kernels need them) the host reads nothing and does not wait for the device."""
    def on_dev(t):
        return t.detach().to(device=dev, dtype=torch.int32).contiguous()

    ids = input_ids.to(dev)
    ids = ids if ids.dtype == torch.int64 else ids.long()
    ids = ids if ids.dim() != 2 or ids.shape[1] <= 1 or ids.stride(1) == 1 else ids.contiguous()
    return torch.ops.rl_amd.pack_input_ids(ids, on_dev(cu_seqlens_q), on_dev(cu_seqlens_q_padded), -1, total).unsqueeze(0)


def prepare_packed_loss_input(
    logits: torch.Tensor,
    data: Any,
    loss_fn: LossFunction,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_q_padded: torch.Tensor,
    vocab_parallel_rank: Optional[int] = None,
    vocab_parallel_group: Optional[Any] = None,
    context_parallel_group: Optional[Any] = None,
    sampling_params: Optional[TrainingSamplingParams] = None,
    chunk_size: Optional[int] = None,
) -> tuple[dict[str, Any], Any]:
    """``loss/utils.py:264-385``: packed ``[1, T, V]`` logits + unpacked ``[B, S]`` data -> logprobs for
    every sequence in one launch."""
    if loss_fn.input_type != LossInputType.LOGPROB:
        raise ValueError(
            f"prepare_packed_loss_input only supports LossInputType.LOGPROB, got {loss_fn.input_type}. "
            "Use SequencePackingLossWrapper with prepare_loss_input for other types."
        )
    input_ids = data["input_ids"]
    rank = vocab_parallel_rank or 0
    vocab = logits.shape[-1]
    targets = _packed_targets(input_ids, cu_seqlens_q, cu_seqlens_q_padded, logits.shape[1], logits.device)

    def logprobs_with(params):
        return from_parallel_logits_to_logprobs_packed_sequences(
            logits,
            targets,
            cu_seqlens_q_padded,
            input_ids.shape[1],
            vocab_start_index=rank * vocab,
            vocab_end_index=(rank + 1) * vocab,
            group=vocab_parallel_group,
            inference_only=False,
            cp_group=context_parallel_group,
            sampling_params=params,
            chunk_size=None,
            target_is_pre_rolled=True,
        )

    logprobs = logprobs_with(sampling_params)
    if need_top_k_or_top_p_filtering(sampling_params):
        mask = data["token_mask"] * data["sample_mask"].unsqueeze(-1)
        logprobs = mask_out_neg_inf_logprobs(logprobs, mask[:, 1:].to(logprobs.device), "curr_logprobs")
        if _wants_unfiltered_kl(loss_fn):
            data["curr_logprobs_unfiltered"] = logprobs_with(None)
    return {"next_token_logprobs": logprobs}, data
