"""The DTensor worker's post-processors (``nemo_rl/models/automodel/train.py:540-864``) on the HIP kernels and the
function that feeds them, ``forward_with_post_processing_fn`` (``:308-441``).

The policy worker runs this forward-only pass twice per step (``prev_logprobs`` and
``reference_policy_logprobs``) on the same logits shapes as training.  Here one launch emits the
``[B, S]`` result directly: the logprob of every next token, the zero column in front and the
zeros from ``input_lengths`` on, without reading the logits of padding positions and without the
fp32 ``[B, S, V]`` log-softmax the reference materialises.  One GPU: ``cp_size`` must be 1 and the
logits a plain tensor (no DTensor / TP mesh).
"""

from __future__ import annotations

from typing import Any, Optional

import torch

from .. import _need_single_gpu
from ... import ops  # noqa: F401  (registers torch.ops.rl_amd)
from ..._deferred import pending_temperature
from ..._lib import NRL_TEMP_RCP
from ...algorithms.logits_sampling_utils import TrainingSamplingParams, need_top_k_or_top_p_filtering
from ...algorithms.loss.utils import mask_out_neg_inf_logprobs
from ...distributed import model_utils as MU
from ...temperature import apply_temperature_scaling, deferred_temperature  # noqa: F401


# The model-side helpers of ``forward_with_post_processing_fn`` (``model_forward``, ``extract_logits``,
# ``_needs_kv_cache_for_shared_layers``) and the post-processors this package does not replace
# (``TopkLogitsPostProcessor``, ``FullLogitsPostProcessor``, ``ScorePostProcessor``) are the install's own: they are
# looked up in the globals of the function this one replaces.  A caller without an install may provide them here.
MODEL_HELPERS: Optional[dict] = None


def _helpers() -> dict:
    if MODEL_HELPERS is not None:
        return MODEL_HELPERS
    from ...compat import original

    theirs = original("nemo_rl.models.automodel.train", "forward_with_post_processing_fn")
    if theirs is None:
        raise NotImplementedError("forward_with_post_processing_fn runs the model with the helpers of a NeMo-RL install "
                                  "(model_forward, extract_logits); none is installed and MODEL_HELPERS is not set")
    return theirs.__globals__


def forward_with_post_processing_fn(
    model: Any,
    post_processing_fn: Any,
    processed_mb: Any,
    is_reward_model: bool = False,
    allow_flash_attn_args: bool = True,
    global_valid_seqs: Optional[torch.Tensor] = None,
    global_valid_toks: Optional[torch.Tensor] = None,
    sampling_params: Optional[TrainingSamplingParams] = None,
    sequence_dim: int = 1,
):
    """``models/automodel/train.py:308-441``: model forward, temperature, post-processing; same arguments, same
    ``(result, metrics, processed_mb)``.

    The one difference is where the temperature divide happens.  The reference divides the logits tensor in place
    and hands it to the post-processor, and autograd later sends the gradient back through that divide: two read +
    write passes over ``[B, S, V]``.  When the post-processor is this package's ``LossPostProcessor`` or
    ``LogprobsPostProcessor`` nothing else reads the tensor in between (it is deleted on return), so the divide is
    left to the kernel that reads the logits next (``deferred_temperature``), with the same roundings of value and
    gradient; a loss that takes the raw logits gets them divided after all (``materialise_pending``).  Every other
    post-processor sees the in-place divide."""
    h = _helpers()
    data_dict = processed_mb.data_dict
    processed_inputs = processed_mb.processed_inputs
    kv_cache = h.get("_needs_kv_cache_for_shared_layers")
    outputs = h["model_forward"](model, processed_inputs, is_reward_model=is_reward_model,
                                 allow_flash_attn_args=allow_flash_attn_args,
                                 use_cache=kv_cache(model) if kv_cache is not None else False)
    logits = h["extract_logits"](model, outputs)
    del outputs

    def is_a(name):
        cls = h.get(name)
        return cls is not None and isinstance(post_processing_fn, cls)

    ours = isinstance(post_processing_fn, (LossPostProcessor, LogprobsPostProcessor))
    defer = ours and type(logits) is torch.Tensor and logits.is_cuda
    with (deferred_temperature() if defer else _nothing()):
        if ours or is_a("TopkLogitsPostProcessor") or is_a("FullLogitsPostProcessor"):
            logits = apply_temperature_scaling(logits, sampling_params)
        if isinstance(post_processing_fn, LossPostProcessor):
            result, metrics = post_processing_fn(
                logits=logits, data_dict=data_dict, processed_inputs=processed_inputs, global_valid_seqs=global_valid_seqs,
                global_valid_toks=global_valid_toks, sequence_dim=sequence_dim)
        elif isinstance(post_processing_fn, LogprobsPostProcessor) or is_a("TopkLogitsPostProcessor"):
            result = post_processing_fn(
                logits=logits, data_dict=data_dict, processed_inputs=processed_inputs,
                original_batch_size=processed_mb.original_batch_size, original_seq_len=processed_mb.original_seq_len,
                sequence_dim=sequence_dim)
            if isinstance(post_processing_fn, LogprobsPostProcessor):
                metrics = {"logprobs": result}
            else:
                vals, idx = result
                metrics = {"topk_logits": vals, "topk_indices": idx}
        elif is_a("FullLogitsPostProcessor"):
            result = post_processing_fn(
                logits=logits, data_dict=data_dict, processed_inputs=processed_inputs,
                original_batch_size=processed_mb.original_batch_size, original_seq_len=processed_mb.original_seq_len,
                sequence_dim=sequence_dim)
            metrics = {"full_logits": result}
        elif is_a("ScorePostProcessor"):
            result = post_processing_fn(logits=logits)
            metrics = {"scores": result}
        else:
            raise TypeError(f"Unknown post-processing function type: {type(post_processing_fn)}")
    del logits
    return result, metrics, processed_mb


def _nothing():
    import contextlib

    return contextlib.nullcontext()


class LossPostProcessor:
    """``LossPostProcessor`` of the DTensor worker (``nemo_rl/models/automodel/train.py:540-653``): logits of one
    microbatch -> ``(loss, metrics)``.  Same constructor and call signature as the reference class.

    The reference prepares the loss input and calls the loss as two steps; here the unpacked case goes through
    ``wrap_loss_fn_with_input_preparation``, which does the same two steps unless the loss is a
    ``ClippedPGLossFn`` the single pass covers - then logits -> loss -> gradient is one kernel.  Packed
    microbatches take ``SequencePackingLossWrapper`` with the unpadded boundaries for both arguments, as the
    reference does."""

    def __init__(self, loss_fn: Any, cfg: Any, device_mesh: Any, cp_mesh: Any, tp_mesh: Any, cp_size: int, dp_size: int,
                 enable_seq_packing: bool = False, sampling_params: Optional[TrainingSamplingParams] = None):
        self.loss_fn = loss_fn
        self.cfg = cfg
        self.device_mesh = device_mesh
        self.cp_mesh = cp_mesh
        self.tp_mesh = tp_mesh
        self.cp_size = cp_size
        self.dp_size = dp_size
        self.enable_seq_packing = enable_seq_packing
        self.sampling_params = sampling_params
        _need_single_gpu(cp_size, "LossPostProcessor")

    def __call__(self, logits: torch.Tensor, data_dict: Any, processed_inputs: Any, global_valid_seqs: torch.Tensor,
                 global_valid_toks: torch.Tensor, sequence_dim: int = 1):
        from functools import partial

        from ...algorithms.loss import (
            SequencePackingLossWrapper,
            prepare_loss_input,
            wrap_loss_fn_with_input_preparation,
        )

        if type(logits).__name__ == "DTensor":
            raise NotImplementedError("LossPostProcessor: vocabulary-parallel (DTensor) logits need more than one GPU")
        prepare = partial(prepare_loss_input, sampling_params=self.sampling_params)
        if self.enable_seq_packing:
            cu = processed_inputs.flash_attn_kwargs.cu_seqlens_q
            wrapped = SequencePackingLossWrapper(loss_fn=self.loss_fn, prepare_fn=prepare, cu_seqlens_q=cu,
                                                 cu_seqlens_q_padded=cu)
            return wrapped(logits, data_dict, global_valid_seqs, global_valid_toks)
        loss, metrics = wrap_loss_fn_with_input_preparation(logits, data_dict, global_valid_seqs, global_valid_toks,
                                                            self.loss_fn, prepare)
        if hasattr(metrics, "defer_scaling"):
            # this worker's loop divides every metric by the number of global batches before it calls backward()
            # (``train.py:525-547``): let the mapping record that instead of waiting for the device
            metrics.defer_scaling()
        return loss, metrics


class LogprobsPostProcessor:
    """Same constructor and call signature as the reference class."""

    def __init__(
        self,
        cfg: Any,
        device_mesh: Any,
        cp_mesh: Any,
        tp_mesh: Any,
        cp_size: int,
        enable_seq_packing: bool = False,
        sampling_params: Optional[TrainingSamplingParams] = None,
    ):
        self.cfg = cfg
        self.device_mesh = device_mesh
        self.cp_mesh = cp_mesh
        self.tp_mesh = tp_mesh
        self.cp_size = cp_size
        self.enable_seq_packing = enable_seq_packing
        self.sampling_params = sampling_params
        self.logprob_chunk_size = cfg.get("logprob_chunk_size", None) if hasattr(cfg, "get") else None
        _need_single_gpu(cp_size, "LogprobsPostProcessor")

    def __call__(
        self,
        logits: torch.Tensor,
        data_dict: Any,
        processed_inputs: Any,
        original_batch_size: int,
        original_seq_len: int,
        sequence_dim: int = 1,
    ) -> torch.Tensor:
        """``[batch, seq]`` fp32 token logprobs (``train.py:689-806``)."""
        if type(logits).__name__ == "DTensor":
            raise NotImplementedError("LogprobsPostProcessor: vocabulary-parallel (DTensor) logits need more than one GPU")
        seq_len = processed_inputs.seq_len
        input_ids = processed_inputs.input_ids.to(logits.device)
        filtering = need_top_k_or_top_p_filtering(self.sampling_params)
        with torch.no_grad():
            if self.enable_seq_packing:
                token_logprobs = self._unpack(logits, input_ids, processed_inputs, data_dict, original_batch_size,
                                              original_seq_len, filtering)
            elif filtering:
                lp = MU.from_parallel_logits_to_logprobs(logits, input_ids, 0, logits.shape[-1], None, inference_only=True,
                                                         sampling_params=self.sampling_params)
                token_logprobs = torch.cat([torch.zeros_like(lp[:, :1]), lp], dim=1)
                lengths = torch.as_tensor(data_dict["input_lengths"], device=lp.device).reshape(-1, 1)
                token_logprobs = token_logprobs * (torch.arange(seq_len, device=lp.device)[None, :] < lengths)
            else:
                lengths = torch.as_tensor(data_dict["input_lengths"]).to(device=logits.device, dtype=torch.int64).contiguous()
                temperature = pending_temperature(logits)  # a divide apply_temperature_scaling left to this kernel
                x = logits if logits.stride(-1) == 1 else logits.contiguous()
                token_logprobs = torch.ops.rl_amd.logprob_post_fwd(
                    x, input_ids[:, 1:], lengths, input_ids.shape[1] - 1, 0, x.shape[-1], temperature, NRL_TEMP_RCP)
        if filtering:  # ``train.py:799-804``
            mask = data_dict["token_mask"] * data_dict["sample_mask"].unsqueeze(-1)
            token_logprobs = mask_out_neg_inf_logprobs(token_logprobs, mask.to(token_logprobs.device), "prev_logprobs")
        return token_logprobs

    def _unpack(self, logits, input_ids, processed_inputs, data_dict, batch, seq_len, filtering):
        """Packed ``[1, T, V]`` logits -> ``[batch, seq_len]`` (``train.py:764-778``): sequence ``i`` occupies
        ``cu_seqlens[i] .. cu_seqlens[i+1]``, its first token gets 0 and so does everything past its length."""
        cu = processed_inputs.flash_attn_kwargs.cu_seqlens_q
        cu = torch.as_tensor(cu).to(device=logits.device, dtype=torch.int32)
        lengths = torch.as_tensor(data_dict["input_lengths"]).to(cu.device)
        if cu.numel() != batch + 1 or not bool(((cu[1:] - cu[:-1]) == lengths.to(cu.dtype)).all()):
            raise ValueError("cu_seqlens_q must delimit exactly the input_lengths of the microbatch")
        lp = MU.from_parallel_logits_to_logprobs_packed_sequences(
            logits, input_ids.reshape(-1), cu, seq_len, 0, logits.shape[-1], None, inference_only=True,
            sampling_params=self.sampling_params if filtering else None)
        return torch.cat([torch.zeros_like(lp[:, :1]), lp], dim=1)
