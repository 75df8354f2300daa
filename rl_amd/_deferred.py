"""Per-thread record of temperature divides that ``apply_temperature_scaling`` left to the kernels
(see ``rl_amd/temperature.py``).  No dependencies, so that every layer of the package can consult it."""

from __future__ import annotations

import contextlib
import threading
from typing import Any

import torch

_state = threading.local()


@contextlib.contextmanager
def deferred_temperature():
    """While open (on this thread), ``apply_temperature_scaling`` records the temperature instead of dividing
    and this package's logprob / loss entry points divide inside their kernels.  The record is dropped
    when the context closes; a backward pass started later still uses the temperature its forward saw."""
    _state.depth = getattr(_state, "depth", 0) + 1
    if _state.depth == 1:
        _state.pending = []
    try:
        yield
    finally:
        _state.depth -= 1
        if _state.depth == 0:
            _state.pending = []


def pending_temperature(logits: Any) -> float:
    """The temperature recorded for the tensor ``logits`` is a view of, else 1."""
    if getattr(_state, "depth", 0) == 0 or not isinstance(logits, torch.Tensor) or not _state.pending:
        return 1.0
    key = logits.untyped_storage().data_ptr()
    for ptr, t in reversed(_state.pending):
        if ptr == key:
            return t
    return 1.0


def refuse_pending(logits: Any, what: str) -> None:
    """For entry points that read logits but have no fused temperature: fail instead of reading unscaled values."""
    t = pending_temperature(logits)
    if t != 1.0:
        raise RuntimeError(f"{what} was handed logits whose temperature divide (T={t}) is still deferred; "
                           "it has no fused temperature - call it outside deferred_temperature()")
