"""Loss wrappers for sequence-packed microbatches
(counterpart of ``nemo_rl/algorithms/loss/wrapper.py:28-228, 292-322``)."""

from __future__ import annotations

import functools
import math
from typing import Any, Callable, Optional

import torch

from .interfaces import LossFunction

_MIN_KEYS = {"probs_ratio_min", "probs_ratio_clamped_min"}
_MAX_KEYS = {"probs_ratio_max", "probs_ratio_clamped_max"}


def _bound_keywords(prepare_fn, base, allowed) -> Optional[dict]:
    """The workers never pass ``prepare_loss_input`` bare: they bind ``sampling_params`` / ``d2t`` /
    ``chunk_size`` with ``functools.partial`` first (``models/megatron/train.py:506-533``,
    ``models/automodel/train.py:624-627``).  Returns the bound keywords when ``prepare_fn`` is ``base`` itself
    or such a partial of it (keywords from ``allowed`` only, no positional arguments), else ``None``."""
    if prepare_fn is base:
        return {}
    if isinstance(prepare_fn, functools.partial) and prepare_fn.func is base and not prepare_fn.args:
        kw = dict(prepare_fn.keywords)
        if set(kw) <= set(allowed):
            return kw
    return None


def _slice_row(data, idx: int):
    if hasattr(data, "slice"):
        return data.slice(idx, idx + 1)
    return {k: (v[idx : idx + 1] if isinstance(v, torch.Tensor) else v) for k, v in data.items()}


class SequencePackingLossWrapper:
    """One loss call per packed sequence (``wrapper.py:28-166``): the logits of sequence ``i`` are the
    slice ``[cu_padded[i], cu_padded[i+1])`` of the packed row, its data tensors are cut to the
    unpadded length; losses and metrics are summed, extrema combined with min / max."""

    def __init__(self, loss_fn: LossFunction, prepare_fn: Callable[..., Any], cu_seqlens_q, cu_seqlens_q_padded=None,
                 vocab_parallel_rank: Optional[int] = None, vocab_parallel_group: Optional[Any] = None,
                 context_parallel_group: Optional[Any] = None):
        self.loss_fn = loss_fn
        self.prepare_fn = prepare_fn
        self.cu_seqlens_q = cu_seqlens_q
        self.cu_seqlens_q_padded = cu_seqlens_q_padded
        self.vocab_parallel_rank = vocab_parallel_rank
        self.vocab_parallel_group = vocab_parallel_group
        self.context_parallel_group = context_parallel_group

    def __call__(self, next_token_logits, data, global_valid_seqs, global_valid_toks):
        cu = [int(v) for v in self.cu_seqlens_q.tolist()]
        cup = cu if self.cu_seqlens_q_padded is None else [int(v) for v in self.cu_seqlens_q_padded.tolist()]
        fused = getattr(self.loss_fn, "use_fused_linear_logprobs", False)
        total, merged = 0, {}
        for i in range(len(cu) - 1):
            n_real, n_pad = cu[i + 1] - cu[i], cup[i + 1] - cup[i]
            row = {
                k: (v[:, :n_real] if isinstance(v, torch.Tensor) and v.ndim > 1 and v.shape[1] > 1 else v)
                for k, v in _slice_row(data, i).items()
            }
            stop = cup[i] + n_pad
            if fused:
                stop = min(stop, next_token_logits.shape[1])
            piece = next_token_logits[:, cup[i] : stop] if fused else next_token_logits.narrow(1, cup[i], n_pad)
            loss_input, row = self.prepare_fn(
                logits=piece, data=row, loss_fn=self.loss_fn, vocab_parallel_rank=self.vocab_parallel_rank,
                vocab_parallel_group=self.vocab_parallel_group, context_parallel_group=self.context_parallel_group,
            )
            loss, metrics = self.loss_fn(
                data=row, global_valid_seqs=global_valid_seqs, global_valid_toks=global_valid_toks, **loss_input
            )
            total = total + loss
            for key, value in metrics.items():
                value = value.item() if isinstance(value, torch.Tensor) and value.ndim == 0 else value
                if key in _MIN_KEYS:
                    merged.setdefault(key, float("inf"))
                    if not math.isinf(value):
                        merged[key] = min(merged[key], value)
                elif key in _MAX_KEYS:
                    merged.setdefault(key, float("-inf"))
                    if not math.isinf(value):
                        merged[key] = max(merged[key], value)
                else:
                    merged[key] = merged.get(key, 0) + value
        return total, merged


class SequencePackingFusionLossWrapper:
    """All packed sequences in one pass (``wrapper.py:169-228``): ``prepare_fn`` (normally
    ``prepare_packed_loss_input``) runs once on the packed logits, then the loss runs once."""

    def __init__(self, loss_fn: LossFunction, prepare_fn: Callable[..., Any], cu_seqlens_q, cu_seqlens_q_padded=None,
                 vocab_parallel_rank: Optional[int] = None, vocab_parallel_group: Optional[Any] = None,
                 context_parallel_group: Optional[Any] = None):
        self.loss_fn = loss_fn
        self.prepare_fn = prepare_fn
        self.cu_seqlens_q = cu_seqlens_q
        self.cu_seqlens_q_padded = cu_seqlens_q if cu_seqlens_q_padded is None else cu_seqlens_q_padded
        self.vocab_parallel_rank = vocab_parallel_rank
        self.vocab_parallel_group = vocab_parallel_group
        self.context_parallel_group = context_parallel_group

    def __call__(self, next_token_logits, data, global_valid_seqs, global_valid_toks):
        from .fused import fused_packed_logits_clipped_pg_loss, why_not_fusable_packed
        from .utils import prepare_packed_loss_input

        # a ClippedPGLossFn whose token gradient needs no other token's logprob: logits -> loss -> gradient
        # in one pass over the packed row, as in wrap_loss_fn_with_input_preparation
        bound = _bound_keywords(self.prepare_fn, prepare_packed_loss_input, ("sampling_params", "chunk_size"))
        if (bound is not None and torch.is_grad_enabled()
                and isinstance(next_token_logits, torch.Tensor) and next_token_logits.requires_grad
                and why_not_fusable_packed(self.loss_fn, next_token_logits, data, bound.get("sampling_params")) is None):
            from ...distributed.model_utils import _group_size

            if _group_size(self.vocab_parallel_group) == 1 and _group_size(self.context_parallel_group) == 1:
                return fused_packed_logits_clipped_pg_loss(
                    next_token_logits, data, self.loss_fn, self.cu_seqlens_q, self.cu_seqlens_q_padded,
                    global_valid_seqs, global_valid_toks)
        loss_input, prepared = self.prepare_fn(
            logits=next_token_logits, data=data, loss_fn=self.loss_fn, cu_seqlens_q=self.cu_seqlens_q,
            cu_seqlens_q_padded=self.cu_seqlens_q_padded, vocab_parallel_rank=self.vocab_parallel_rank,
            vocab_parallel_group=self.vocab_parallel_group, context_parallel_group=self.context_parallel_group,
        )
        return self.loss_fn(
            data=prepared, global_valid_seqs=global_valid_seqs, global_valid_toks=global_valid_toks, **loss_input
        )


def wrap_loss_fn_with_input_preparation(next_token_logits, data, global_valid_seqs, global_valid_toks,
                                        loss_fn: LossFunction, prepare_fn: Callable[..., Any],
                                        vocab_parallel_rank: Optional[int] = None,
                                        vocab_parallel_group: Optional[Any] = None,
                                        context_parallel_group: Optional[Any] = None):
    """``wrapper.py:292-322``: prepare, then call the loss.  When the loss is a ``ClippedPGLossFn`` whose
    per-token gradient does not need other tokens' logprobs and the logits are a plain GPU tensor, both
    steps (and the later backward through the logprob op) run as one fused pass over the logits."""
    from .fused import fused_logits_clipped_pg_loss, why_not_fusable
    from .utils import prepare_loss_input

    # chunk_size only bounds the reference's working set and d2t belongs to the draft-model loss: neither changes
    # what the single pass computes, top-k / top-p filtering (checked by why_not_fusable) does
    bound = _bound_keywords(prepare_fn, prepare_loss_input, ("sampling_params", "d2t", "chunk_size"))
    if (bound is not None and bound.get("d2t") is None and torch.is_grad_enabled()
            and isinstance(next_token_logits, torch.Tensor) and next_token_logits.requires_grad
            and why_not_fusable(loss_fn, next_token_logits, data, bound.get("sampling_params")) is None):
        from ...distributed.model_utils import _group_size

        if _group_size(vocab_parallel_group) == 1 and _group_size(context_parallel_group) == 1:
            return fused_logits_clipped_pg_loss(next_token_logits, data, loss_fn, global_valid_seqs, global_valid_toks)
    loss_input, data = prepare_fn(
        logits=next_token_logits, data=data, loss_fn=loss_fn, vocab_parallel_rank=vocab_parallel_rank,
        vocab_parallel_group=vocab_parallel_group, context_parallel_group=context_parallel_group,
    )
    return loss_fn(data=data, global_valid_seqs=global_valid_seqs, global_valid_toks=global_valid_toks, **loss_input)
