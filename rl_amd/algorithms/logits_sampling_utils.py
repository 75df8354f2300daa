"""Top-k / top-p (nucleus) filtering of training logits
(counterpart of ``nemo_rl/algorithms/logits_sampling_utils.py``)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

# rows per launch hint kept for signature compatibility (``logits_sampling_utils.py:26``); the HIP
# selection kernel works row by row and needs no chunking
TOP_K_TOP_P_CHUNK_SIZE: int = 256


@dataclass
class TrainingSamplingParams:
    """``logits_sampling_utils.py:29-44``: top_k (None or -1 = off), top_p (1.0 = off), temperature."""

    top_k: int | None = None
    top_p: float = 1.0
    temperature: float = 1.0


def _need_top_k_filtering(top_k: int | None) -> bool:
    return top_k is not None and top_k > 0


def _need_top_p_filtering(top_p: float | None) -> bool:
    return top_p is not None and top_p != 1.0


def need_top_k_or_top_p_filtering(sampling_params: Optional[TrainingSamplingParams]) -> bool:
    """``logits_sampling_utils.py:57-66``."""
    if sampling_params is None:
        return False
    return _need_top_k_filtering(sampling_params.top_k) or _need_top_p_filtering(sampling_params.top_p)


def apply_top_k_top_p(
    logits: torch.Tensor,
    top_k: int | None,
    top_p: float,
    chunk_size: int | None = TOP_K_TOP_P_CHUNK_SIZE,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """``logits_sampling_utils.py:254-285``: ``(filtered_logits, keep_mask)`` with ``-inf`` outside the
    kept set; the gradient of the filtered logits is passed through where kept and zero elsewhere."""
    if not _need_top_k_filtering(top_k) and not _need_top_p_filtering(top_p):
        return logits, None
    from ..distributed.sampling_logprob import filter_logits

    return filter_logits(logits, top_k, top_p)
