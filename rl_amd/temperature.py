"""Temperature scaling of the model's logits (``apply_temperature_scaling``,
``nemo_rl/models/automodel/train.py:180-194`` and ``nemo_rl/models/megatron/train.py:203-217``).

The reference divides the logits tensor in place, in its own dtype, right after the model forward; the
Megatron worker even drops the return value, so "the tensor the model returned now holds scaled values"
is the contract.  ``apply_temperature_scaling`` here keeps it: one HIP pass ``x * (1 / T)`` over the
tensor (how a GPU ``div_`` by a scalar rounds), differentiable like ``div_``.

That pass costs a full read + write of ``[B, S, V]``.  The logprob kernels can apply the same divide,
with the same rounding of value and gradient, while they stream the row anyway.  Because nothing in
the tensor itself can say "not divided yet" without risking a silently unscaled read elsewhere, a bare
call never does that: only inside ``with deferred_temperature():`` does ``apply_temperature_scaling`` leave the
memory alone and record (storage object, T) for the calling thread, for as long as that storage lives; the logprob / loss entry points of this
package look the logits they are handed up in that record (views of the recorded tensor share its
storage) and divide inside their kernels.  Whoever opens the context promises that, until it closes,
only those entry points read the logits -- as ``forward_with_post_processing_fn`` of the DTensor worker's mirror
does, which knows that a post-processor of this package comes next.  Readers of this package that have no fused
temperature either refuse such logits or, where they sit on a worker's path (``prepare_loss_input`` for a loss that
takes raw logits), apply the divide after all (``materialise_pending``).
"""

from __future__ import annotations

from typing import Any, Optional

import torch

from . import ops  # noqa: F401  (registers torch.ops.rl_amd)
from ._deferred import _state, deferred_temperature, drop_record, pending_temperature, record_temperature  # noqa: F401

_OPS = torch.ops.rl_amd


def _one(device) -> torch.Tensor:
    return torch.ones((), dtype=torch.float32, device=device)


class _DivideInPlace(torch.autograd.Function):
    """``logits.div_(T)`` with GPU rounding: value ``round(x * (1/T))``, gradient ``round(g * (1/T))``."""

    @staticmethod
    def forward(ctx, logits, temperature):
        ctx.mark_dirty(logits)
        ctx.temperature = temperature
        view = logits if logits.dim() == 3 else logits.view(-1, 1, logits.shape[-1])
        _OPS.scale_rows_(view, _one(logits.device), temperature)
        return logits

    @staticmethod
    def backward(ctx, grad):
        g3 = grad if grad.dim() == 3 else grad.reshape(-1, 1, grad.shape[-1])
        if g3.stride(-1) != 1:
            g3 = g3.contiguous()
        return _OPS.scale_rows(g3, _one(grad.device), ctx.temperature).view(grad.shape), None


def _divide_now(logits: torch.Tensor, t: float) -> torch.Tensor:
    if not logits.is_cuda:
        raise RuntimeError("rl_amd runs on the GPU only (got CPU logits); there is no CPU fallback")
    if logits.dim() < 1 or logits.stride(-1) != 1 or not logits.is_contiguous():
        raise ValueError("apply_temperature_scaling expects a contiguous logits tensor")
    if torch.is_grad_enabled() and logits.requires_grad:
        return _DivideInPlace.apply(logits, t)
    view = logits if logits.dim() == 3 else logits.view(-1, 1, logits.shape[-1])
    _OPS.scale_rows_(view, _one(logits.device), t)
    return logits


def apply_temperature_scaling(logits: torch.Tensor, sampling_params: Optional[Any]) -> torch.Tensor:
    """Same contract as the reference function: returns ``logits``, divided in place by the temperature
    when there is one and it is not 1.  Inside ``deferred_temperature()`` the divide is left to the
    logprob kernels instead (see the module text)."""
    if sampling_params is None or sampling_params.temperature == 1.0:
        return logits
    t = float(sampling_params.temperature)
    if getattr(_state, "depth", 0) > 0:
        if not logits.is_cuda:
            raise RuntimeError("deferred_temperature() needs GPU logits")
        record_temperature(logits, t)
        return logits
    return _divide_now(logits, t)


def materialise_pending(logits: Any) -> Any:
    """For a reader without a fused temperature (a loss that takes raw logits, the distillation reductions): a
    divide that ``apply_temperature_scaling`` left to the kernels is applied now, in place and through autograd
    exactly as the eager call would have, and taken off the record.  The tensor must be the whole of the recorded
    storage: dividing a slice would leave the rest of it undivided with nothing on record."""
    if not isinstance(logits, torch.Tensor):
        return logits
    t = pending_temperature(logits)
    if t == 1.0:
        return logits
    if logits.storage_offset() != 0 or logits.numel() * logits.element_size() != logits.untyped_storage().nbytes():
        raise RuntimeError("a view of logits whose temperature divide is still deferred reached a reader that cannot apply "
                           "it; hand over the whole tensor, or divide eagerly outside deferred_temperature()")
    drop_record(logits)
    return _divide_now(logits, t)
