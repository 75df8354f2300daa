"""Makes the kernels reachable under NeMo-RL's own dotted paths.

``install()`` either registers ``nemo_rl.distributed.model_utils``, ``nemo_rl.algorithms.loss`` (and
its sub-modules), ``nemo_rl.algorithms.loss_functions``, ``nemo_rl.algorithms.utils``,
``nemo_rl.algorithms.logits_sampling_utils``, ``nemo_rl.algorithms.advantage_estimator`` and
``nemo_rl.models.automodel.train`` / ``nemo_rl.models.megatron.train`` (their post-processors and
``apply_temperature_scaling``) as
aliases of the ``rl_amd`` modules (when NeMo-RL is not importable), or replaces the hot-path
attributes of an existing NeMo-RL install in place.
"""

from __future__ import annotations

import importlib
import sys
import types

_ALIASES = {
    "nemo_rl.distributed.model_utils": "rl_amd.distributed.model_utils",
    "nemo_rl.algorithms.logits_sampling_utils": "rl_amd.algorithms.logits_sampling_utils",
    "nemo_rl.algorithms.utils": "rl_amd.algorithms.utils",
    "nemo_rl.algorithms.advantage_estimator": "rl_amd.algorithms.advantage_estimator",
    "nemo_rl.algorithms.loss": "rl_amd.algorithms.loss",
    "nemo_rl.algorithms.loss.interfaces": "rl_amd.algorithms.loss.interfaces",
    "nemo_rl.algorithms.loss.loss_functions": "rl_amd.algorithms.loss.loss_functions",
    "nemo_rl.algorithms.loss.utils": "rl_amd.algorithms.loss.utils",
    "nemo_rl.algorithms.loss.wrapper": "rl_amd.algorithms.loss.wrapper",
    "nemo_rl.algorithms.loss_functions": "rl_amd.algorithms.loss_functions",
    "nemo_rl.models.automodel.train": "rl_amd.models.automodel.train",
    "nemo_rl.models.megatron.train": "rl_amd.models.megatron.train",
    "nemo_rl.algorithms.grpo": "rl_amd.algorithms.grpo",
}

# attributes replaced on a real NeMo-RL install (module -> names)
_PATCHED = {
    "nemo_rl.distributed.model_utils": [
        "DistributedLogprob", "ChunkedDistributedLogprob", "DistributedLogprobWithSampling",
        "ChunkedDistributedLogprobWithSampling", "ChunkedDistributedHiddenStatesToLogprobs",
        "from_parallel_logits_to_logprobs", "from_parallel_logits_to_logprobs_packed_sequences",
        "from_parallel_hidden_states_to_logprobs", "get_next_token_logprobs_from_logits",
        "dtensor_from_parallel_logits_to_logprobs", "get_logprobs_from_vocab_parallel_logits",
        "get_distillation_topk_logprobs_from_logits",
        "ChunkedDistributedEntropy", "ChunkedDistributedGatherLogprob", "DistributedCrossEntropy",
        "_compute_distributed_log_softmax", "_compute_distributed_log_softmax_with_grad",
    ],
    "nemo_rl.algorithms.logits_sampling_utils": ["apply_top_k_top_p"],
    "nemo_rl.algorithms.loss.wrapper": ["wrap_loss_fn_with_input_preparation", "SequencePackingLossWrapper",
                                        "SequencePackingFusionLossWrapper"],
    "nemo_rl.algorithms.loss.utils": ["prepare_loss_input", "prepare_packed_loss_input"],
    "nemo_rl.algorithms.loss.loss_functions": ["ClippedPGLossFn", "NLLLossFn", "PreferenceLossFn", "DPOLossFn", "DistillationLossFn",
                                               "DraftCrossEntropyLossFn"],
    "nemo_rl.algorithms.utils": ["calculate_baseline_and_std_per_prompt", "calculate_kl", "masked_mean",
                                 "mask_out_neg_inf_logprobs"],
    "nemo_rl.models.automodel.train": ["LogprobsPostProcessor", "LossPostProcessor", "apply_temperature_scaling"],
    "nemo_rl.models.megatron.train": ["LogprobsPostProcessor", "LossPostProcessor", "apply_temperature_scaling"],
    "nemo_rl.algorithms.grpo": ["compute_and_apply_seq_logprob_error_masking", "dynamic_sampling"],
    "nemo_rl.algorithms.advantage_estimator": ["GRPOAdvantageEstimator"],
}


def _real_nemo_rl_present() -> bool:
    mod = sys.modules.get("nemo_rl")
    if mod is not None:
        return not getattr(mod, "__rl_amd_alias__", False)
    try:
        return importlib.util.find_spec("nemo_rl") is not None
    except (ImportError, ValueError):
        return False


def install(force_alias: bool = False) -> str:
    """Returns ``"patched"`` or ``"aliased"``."""
    if _real_nemo_rl_present() and not force_alias:
        for target, names in _PATCHED.items():
            dst = importlib.import_module(target)
            src = importlib.import_module(_ALIASES[target])
            for name in names:
                setattr(dst, name, getattr(src, name))
        return "patched"
    for parent in ("nemo_rl", "nemo_rl.distributed", "nemo_rl.algorithms", "nemo_rl.models", "nemo_rl.models.automodel",
                   "nemo_rl.models.megatron"):
        if parent not in sys.modules:
            pkg = types.ModuleType(parent)
            pkg.__path__ = []  # a package, so sub-module imports resolve through sys.modules
            pkg.__rl_amd_alias__ = True
            sys.modules[parent] = pkg
    for alias, real in _ALIASES.items():
        mod = importlib.import_module(real)
        sys.modules[alias] = mod
        parent, _, leaf = alias.rpartition(".")
        setattr(sys.modules[parent], leaf, mod)
    return "aliased"
