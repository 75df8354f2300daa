"""The Megatron worker's post-processors (``nemo_rl/models/megatron/train.py:442-684``) on the HIP kernels, and
its forward step with the temperature divide left to those kernels (``:220-362``).

The reference classes return a function that the Megatron forward step applies to the model's output
tensor.  ``LogprobsPostProcessor``'s yields ``(dummy_loss, {"logprobs": [B, S]})``: here the plain path is one
forward-only launch that writes the ``[B, S]`` result with its zero column directly, the packed path
is the packed logprob kernel, and top-k / top-p go through the sampling kernels.  One GPU: the
tensor- and context-parallel groups of the reference are of size one, so the vocabulary range is
the whole last axis of the output tensor.
"""

from __future__ import annotations

from typing import Any, Callable, Dict, Optional, Tuple

import torch

from ... import ops  # noqa: F401  (registers torch.ops.rl_amd)
from ..._deferred import drop_record, pending_temperature, record_temperature
from ..._lib import NRL_TEMP_RCP
from ...algorithms.logits_sampling_utils import TrainingSamplingParams, need_top_k_or_top_p_filtering
from ...algorithms.loss.utils import mask_out_neg_inf_logprobs
from ...distributed import model_utils as MU
from ...temperature import apply_temperature_scaling, deferred_temperature  # noqa: F401


class LossPostProcessor:
    """``LossPostProcessor`` of the Megatron worker (``nemo_rl/models/megatron/train.py:442-597``) for one GPU
    (tensor- and context-parallel size 1, so no ``megatron.core`` state is consulted): ``__call__`` returns the
    function the forward step applies to the model's output tensor, ``output -> (loss, metrics)``.

    ``prepare_loss_input`` is bound to ``sampling_params`` / ``d2t`` / ``chunk_size`` with ``functools.partial``
    exactly as the reference binds it, so the wrappers below see what a real worker hands them; a
    ``ClippedPGLossFn`` the single pass covers then runs logits -> loss -> gradient as one kernel.  The loss is
    multiplied by ``num_microbatches`` (``:583-594``, undoing the schedule's averaging); the gradient the single
    pass has already written is rescaled on the device by whatever factor autograd delivers.  The draft-model
    wrapper (``student_logits`` in the data) is not part of this path."""

    def __init__(self, loss_fn: Any, cfg: Any, num_microbatches: int = 1, cp_normalize: bool = True,
                 sampling_params: Optional[TrainingSamplingParams] = None, draft_model: Any = None,
                 prepare_fn: Optional[Callable[..., Any]] = None):
        if draft_model is not None:
            raise NotImplementedError("LossPostProcessor: the draft-model loss is outside this build")
        self.loss_fn = loss_fn
        self.cfg = cfg
        self.num_microbatches = num_microbatches
        self.cp_normalize = cp_normalize
        self.sampling_params = sampling_params
        self.prepare_fn = prepare_fn
        self.d2t = None

    def __call__(self, data_dict: Any, packed_seq_params: Any = None, global_valid_seqs: Optional[torch.Tensor] = None,
                 global_valid_toks: Optional[torch.Tensor] = None) -> Callable[[torch.Tensor], Tuple[torch.Tensor, Dict[str, Any]]]:
        from functools import partial

        from ...algorithms.loss import (
            SequencePackingFusionLossWrapper,
            SequencePackingLossWrapper,
            prepare_loss_input,
            prepare_packed_loss_input,
            wrap_loss_fn_with_input_preparation,
        )

        chunk = self.cfg.get("logprob_chunk_size", None)
        if self.prepare_fn is not None:
            prepare = self.prepare_fn
        else:
            prepare = partial(prepare_loss_input, sampling_params=self.sampling_params, d2t=self.d2t, chunk_size=chunk)
        if "student_logits" in data_dict:
            raise NotImplementedError("LossPostProcessor: the draft-model loss is outside this build")
        if self.cfg["sequence_packing"]["enabled"] and packed_seq_params is not None:
            if self.cfg.get("sequence_packing", {}).get("fuse_loss", False):
                assert self.prepare_fn is None, (
                    "sequence_packing.fuse_loss=true does not support a custom prepare_fn (e.g. the value model's "
                    "value-specific prep). Disable fuse_loss for the value model."
                )
                wrapper_cls = SequencePackingFusionLossWrapper
                prepare = partial(prepare_packed_loss_input, sampling_params=self.sampling_params, chunk_size=chunk)
            else:
                wrapper_cls = SequencePackingLossWrapper
            wrapped = wrapper_cls(loss_fn=self.loss_fn, prepare_fn=prepare, cu_seqlens_q=packed_seq_params.cu_seqlens_q,
                                  cu_seqlens_q_padded=packed_seq_params.cu_seqlens_q_padded, vocab_parallel_rank=0,
                                  vocab_parallel_group=None, context_parallel_group=None)
        else:
            wrapped = partial(wrap_loss_fn_with_input_preparation, loss_fn=self.loss_fn, prepare_fn=prepare,
                              vocab_parallel_rank=0, vocab_parallel_group=None, context_parallel_group=None)
        wrapped = partial(wrapped, data=data_dict, global_valid_seqs=global_valid_seqs, global_valid_toks=global_valid_toks)
        num_microbatches = self.num_microbatches

        def counteract_schedule_averaging(*args, **kwargs):
            loss, metrics = wrapped(*args, **kwargs)
            return loss * num_microbatches, metrics  # context-parallel size 1: no division

        return counteract_schedule_averaging


class LogprobsPostProcessor:
    """Same constructor and call signature as the reference class."""

    def __init__(self, cfg: Any, sampling_params: Optional[TrainingSamplingParams] = None,
                 use_fused_linear_logprobs: bool = False):
        self.cfg = cfg
        self.sampling_params = sampling_params
        self.use_fused_linear_logprobs = use_fused_linear_logprobs

    def __call__(self, data_dict: Any, input_ids: torch.Tensor, cu_seqlens_padded: Optional[torch.Tensor],
                 ) -> Callable[[torch.Tensor], Tuple[torch.Tensor, Dict[str, torch.Tensor]]]:
        unpacked_input_ids = data_dict["input_ids"]
        original_seq_length = unpacked_input_ids.shape[1]
        filtering = need_top_k_or_top_p_filtering(self.sampling_params)
        packing = bool(self.cfg["sequence_packing"]["enabled"])
        chunk = self.cfg.get("logprob_chunk_size", None) if hasattr(self.cfg, "get") else None

        def processor_fn_inner(output_tensor: torch.Tensor):
            with torch.no_grad():
                if self.use_fused_linear_logprobs:  # the model already returned logprobs (``train.py:634-636``)
                    lp = output_tensor.to(torch.float32)[:, : original_seq_length - 1]
                    token_logprobs = torch.cat([torch.zeros_like(lp[:, :1]), lp], dim=1)
                elif packing:
                    vocab = output_tensor.shape[-1]
                    lp = MU.from_parallel_logits_to_logprobs_packed_sequences(
                        output_tensor, target=input_ids, cu_seqlens_padded=cu_seqlens_padded,
                        unpacked_seqlen=original_seq_length, vocab_start_index=0, vocab_end_index=vocab, group=None,
                        inference_only=True, cp_group=None, chunk_size=chunk, sampling_params=self.sampling_params)
                    token_logprobs = torch.cat([torch.zeros_like(lp[:, :1]), lp], dim=1)
                elif filtering:
                    vocab = output_tensor.shape[-1]
                    lp = MU.from_parallel_logits_to_logprobs(
                        output_tensor, target=unpacked_input_ids.to(output_tensor.device), vocab_start_index=0,
                        vocab_end_index=vocab, tp_group=None, inference_only=True, chunk_size=chunk,
                        sampling_params=self.sampling_params)
                    token_logprobs = torch.cat([torch.zeros_like(lp[:, :1]), lp], dim=1)
                else:
                    # logprob of every next token and the zero column in front in one launch; no position is padding
                    temperature = pending_temperature(output_tensor)  # a divide left to this kernel
                    x = output_tensor if output_tensor.stride(-1) == 1 else output_tensor.contiguous()
                    ids = unpacked_input_ids.to(x.device)
                    full = torch.full((ids.shape[0],), ids.shape[1], dtype=torch.int64, device=x.device)
                    token_logprobs = torch.ops.rl_amd.logprob_post_fwd(
                        x, ids[:, 1:], full, ids.shape[1] - 1, 0, x.shape[-1], temperature, NRL_TEMP_RCP)
                if filtering:  # ``train.py:672-677``
                    mask = data_dict["token_mask"] * data_dict["sample_mask"].unsqueeze(-1)
                    token_logprobs = mask_out_neg_inf_logprobs(token_logprobs, mask.to(token_logprobs.device), "prev_logprobs")
            return torch.tensor(0.0, device=token_logprobs.device), {"logprobs": token_logprobs}

        return processor_fn_inner


def _forward_deferring_temperature(post_processing_fn: Any, sampling_params: Any, use_fused_linear_logprobs: bool,
                                   call: Callable[[], Any]) -> Any:
    """Runs the install's forward step (``call``) so that its ``apply_temperature_scaling`` -- this package's, through
    the module global -- records the temperature instead of dividing, and hands the record on to the function the
    step returns, which Megatron-Core's schedule applies to the output tensor next
    (``megatron/core/pipeline_parallel/schedules.py``: ``output_tensor, loss_func = forward_step_func(...)`` and then
    ``loss_func(output_tensor)``).  Only when what follows is a post-processor of this package and the output is
    logits: with ``use_fused_linear_logprobs`` the model returns logprobs, which the reference divides all the same."""
    ours = isinstance(post_processing_fn, (LossPostProcessor, LogprobsPostProcessor))
    if (not ours or sampling_params is None or sampling_params.temperature == 1.0 or use_fused_linear_logprobs):
        return call()
    with deferred_temperature():
        output_tensor, wrapped = call()
        temperature = 1.0
        if type(output_tensor) is torch.Tensor and output_tensor.is_cuda:
            temperature = pending_temperature(output_tensor)
            drop_record(output_tensor)
    if temperature == 1.0:  # nothing was put off (the install's step did not scale this output)
        return output_tensor, wrapped

    def with_the_divide_pending(output: torch.Tensor, *args: Any, **kwargs: Any) -> Any:
        # Whatever the schedule hands over is the step's output or a copy of it: undivided values either way.
        with deferred_temperature():
            record_temperature(output, temperature)
            return wrapped(output, *args, **kwargs)

    return output_tensor, with_the_divide_pending


def forward_with_post_processing_fn(
    data_iterator: Any,
    model: Any,
    post_processing_fn: Any,
    defer_fp32_logits: Optional[bool] = False,
    global_valid_seqs: Optional[torch.Tensor] = None,
    global_valid_toks: Optional[torch.Tensor] = None,
    sampling_params: Optional[TrainingSamplingParams] = None,
    straggler_timer: Any = None,
    draft_model: Any = None,
    enable_hidden_capture: Optional[bool] = False,
    use_fused_linear_logprobs: bool = False,
    use_router_replay: bool = False,
    router_replay_train: bool = False,
) -> Tuple[torch.Tensor, Callable]:
    """``nemo_rl/models/megatron/train.py:220-362`` on a NeMo-RL install: the install's own function does the work
    (the Megatron-Core model forward, router replay, hidden-state capture); this one only decides where the
    temperature divide happens.  The reference scales the output in place (``:336``) and autograd later sends the
    gradient back through that divide, two read + write passes over ``[B, S, V]`` per microbatch; here, when a
    ``LossPostProcessor`` or ``LogprobsPostProcessor`` of this package consumes the output, the kernels that read
    the logits anyway apply the divide, with the same rounding of value and gradient.  The output tensor then keeps
    its undivided values."""
    from ...compat import original

    theirs = original("nemo_rl.models.megatron.train", "forward_with_post_processing_fn")
    if theirs is None:
        raise RuntimeError("forward_with_post_processing_fn of the Megatron worker wraps the function of a NeMo-RL install "
                           "(it needs Megatron-Core's model forward); rl_amd.install() found none to wrap")
    return _forward_deferring_temperature(
        post_processing_fn, sampling_params, use_fused_linear_logprobs,
        lambda: theirs(data_iterator, model, post_processing_fn, defer_fp32_logits=defer_fp32_logits,
                       global_valid_seqs=global_valid_seqs, global_valid_toks=global_valid_toks,
                       sampling_params=sampling_params, straggler_timer=straggler_timer, draft_model=draft_model,
                       enable_hidden_capture=enable_hidden_capture, use_fused_linear_logprobs=use_fused_linear_logprobs,
                       use_router_replay=use_router_replay, router_replay_train=router_replay_train))
