"""Loss protocol and enums, as in ``nemo_rl/algorithms/loss/interfaces.py:23-110``."""

from __future__ import annotations

import enum
from typing import Any, Protocol

import torch


class LossType(enum.Enum):
    TOKEN_LEVEL = "token_level"
    SEQUENCE_LEVEL = "sequence_level"


class MetricNormalizer(enum.Enum):
    """Which global denominator a returned metric was divided by, so that callers that run the loss
    with placeholder ``global_valid_* = 1`` can rescale the summed fragments afterwards."""

    TOKENS = "tokens"
    SEQUENCES = "sequences"
    NONE = "none"


class LossInputType(enum.Enum):
    LOGIT = "logit"
    LOGPROB = "logprob"
    DISTILLATION = "distillation"
    DISTILLATION_CROSS_TOKENIZER = "distillation_cross_tokenizer"
    DRAFT = "draft"


class LossFunction(Protocol):
    """``loss_fn(data=..., global_valid_seqs=..., global_valid_toks=..., **loss_input) -> (loss, metrics)``."""

    loss_type: LossType
    input_type: LossInputType

    def __call__(
        self, data: Any, global_valid_seqs: torch.Tensor, global_valid_toks: torch.Tensor, **kwargs: Any
    ) -> tuple[torch.Tensor, dict[str, Any]]: ...
