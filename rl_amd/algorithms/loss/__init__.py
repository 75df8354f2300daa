"""Loss functions of the GRPO hot path (counterpart of ``nemo_rl/algorithms/loss/__init__.py``)."""

from .fused import (
    fused_logits_clipped_pg_loss,
    fused_packed_logits_clipped_pg_loss,
    why_not_fusable,
    why_not_fusable_packed,
)
from .interfaces import LossFunction, LossInputType, LossType, MetricNormalizer
from .loss_functions import (
    ClippedPGLossConfig,
    ClippedPGLossFn,
    DistillationLossConfig,
    DistillationLossFn,
    DPOLossConfig,
    DPOLossFn,
    DraftCrossEntropyLossFn,
    NLLLossFn,
    PreferenceLossFn,
)
from .utils import prepare_loss_input, prepare_packed_loss_input
from .wrapper import (
    SequencePackingFusionLossWrapper,
    SequencePackingLossWrapper,
    wrap_loss_fn_with_input_preparation,
)

__all__ = [
    "fused_logits_clipped_pg_loss", "fused_packed_logits_clipped_pg_loss", "why_not_fusable", "why_not_fusable_packed",
    "ClippedPGLossConfig", "ClippedPGLossFn", "DistillationLossConfig", "DistillationLossFn", "DPOLossConfig", "DPOLossFn", "DraftCrossEntropyLossFn", "NLLLossFn", "PreferenceLossFn", "LossFunction", "LossInputType", "LossType",
    "MetricNormalizer", "prepare_loss_input", "prepare_packed_loss_input", "SequencePackingFusionLossWrapper",
    "SequencePackingLossWrapper", "wrap_loss_fn_with_input_preparation",
]
