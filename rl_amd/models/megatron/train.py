"""``LogprobsPostProcessor`` of the Megatron worker (``nemo_rl/models/megatron/train.py:599-684``) on the
HIP kernels.

The reference class returns a function that the Megatron forward step applies to the model's output
tensor; that function yields ``(dummy_loss, {"logprobs": [B, S]})``.  Here the plain path is one
forward-only launch that writes the ``[B, S]`` result with its zero column directly, the packed path
is the packed logprob kernel, and top-k / top-p go through the sampling kernels.  One GPU: the
tensor- and context-parallel groups of the reference are of size one, so the vocabulary range is
the whole last axis of the output tensor.
"""

from __future__ import annotations

from typing import Any, Callable, Dict, Optional, Tuple

import torch

from ... import ops  # noqa: F401  (registers torch.ops.rl_amd)
from ..._lib import NRL_TEMP_RCP
from ...algorithms.logits_sampling_utils import TrainingSamplingParams, need_top_k_or_top_p_filtering
from ...algorithms.loss.utils import mask_out_neg_inf_logprobs
from ...distributed import model_utils as MU


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
                    x = output_tensor if output_tensor.stride(-1) == 1 else output_tensor.contiguous()
                    ids = unpacked_input_ids.to(x.device)
                    full = torch.full((ids.shape[0],), ids.shape[1], dtype=torch.int64, device=x.device)
                    token_logprobs = torch.ops.rl_amd.logprob_post_fwd(
                        x, ids[:, 1:], full, ids.shape[1] - 1, 0, x.shape[-1], 1.0, NRL_TEMP_RCP)
                if filtering:  # ``train.py:672-677``
                    mask = data_dict["token_mask"] * data_dict["sample_mask"].unsqueeze(-1)
                    token_logprobs = mask_out_neg_inf_logprobs(token_logprobs, mask.to(token_logprobs.device), "prev_logprobs")
            return torch.tensor(0.0, device=token_logprobs.device), {"logprobs": token_logprobs}

        return processor_fn_inner
