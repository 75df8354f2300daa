"""Per-thread record of temperature divides that ``apply_temperature_scaling`` left to the kernels
(see ``rl_amd/temperature.py``).  No dependencies, so that every layer of the package can consult it."""

from __future__ import annotations

import contextlib
import threading
import weakref
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


def record_temperature(logits: torch.Tensor, temperature: float) -> None:
    """Notes that the storage ``logits`` lives in still awaits its divide by ``temperature``.

    The note is tied to the storage *object*, through a weak reference: PyTorch keeps one Python object per
    storage for as long as the storage exists, whichever tensors and views come and go, so the note ends
    with the memory it describes.  An address alone would not do: the caching allocator hands a freed
    block to the next tensor of that size, which would then be divided although nobody asked."""
    entry = (weakref.ref(logits.untyped_storage()), float(temperature), int(logits.shape[-1]), logits.dtype)
    _state.pending = [e for e in _state.pending if e[0]() is not None]
    _state.pending.append(entry)


def pending_temperature(logits: Any) -> float:
    """The temperature recorded for the storage ``logits`` is a view of, else 1.

    A floating-point ``[..., V]`` tensor that is *not* on record while logits of the same width and dtype
    are is refused: it is most likely a copy (``.float()``, ``.contiguous()`` of a strided view, a gather)
    of logits whose divide was put off, and reading it as it is would silently use undivided values."""
    if getattr(_state, "depth", 0) == 0 or not isinstance(logits, torch.Tensor) or not _state.pending:
        return 1.0
    storage = logits.untyped_storage()
    live = [e for e in _state.pending if e[0]() is not None]
    _state.pending = live
    for ref, t, _, _ in reversed(live):
        if ref() is storage:
            return t
    if logits.dim() >= 2 and logits.is_floating_point():
        for _, t, vocab, dtype in live:
            if vocab == logits.shape[-1] and dtype == logits.dtype:
                raise RuntimeError(
                    f"inside deferred_temperature(): logits of shape {tuple(logits.shape)} are not on record although "
                    f"logits of the same width await their divide (T={t}); a copy of deferred logits carries "
                    "undivided values - hand over the tensor apply_temperature_scaling returned (or a view of it), "
                    "or divide eagerly outside the context")
    return 1.0


def drop_record(logits: torch.Tensor) -> None:
    """Forgets what is on record for the storage of ``logits`` (its divide has been applied)."""
    if getattr(_state, "depth", 0) == 0:
        return
    storage = logits.untyped_storage()
    _state.pending = [e for e in _state.pending if e[0]() is not None and e[0]() is not storage]


def refuse_pending(logits: Any, what: str) -> None:
    """For entry points that read logits but have no fused temperature: fail instead of reading unscaled values."""
    t = pending_temperature(logits)
    if t != 1.0:
        raise RuntimeError(f"{what} was handed logits whose temperature divide (T={t}) is still deferred; "
                           "it has no fused temperature - call it outside deferred_temperature()")
