"""Logits -> token log-probabilities on one MI355X.

Single-GPU counterpart of ``nemo_rl/distributed/model_utils.py``: the same public names and
argument lists, with the chain of PyTorch ops (fp32 cast, amax, exp, sum, log, gather and their
backward) replaced by one streaming HIP kernel per direction (``torch.ops.rl_amd.logprob_fwd`` /
``logprob_bwd``).  Tensor-parallel and context-parallel groups are accepted for signature
compatibility but must span a single rank; this build runs on one GPU.

What each function mirrors is cited as ``model_utils.py:<lines>`` of the reference file.
"""

from __future__ import annotations

from typing import Any, Optional

import torch

from .. import ops as _ops  # noqa: F401  (registers torch.ops.rl_amd.*)
from .._deferred import pending_temperature, refuse_pending
from .._lib import NRL_TEMP_RCP
from ..algorithms.logits_sampling_utils import (
    TrainingSamplingParams,
    need_top_k_or_top_p_filtering,
)

_OPS = torch.ops.rl_amd


def _group_size(group) -> int:
    if group is None or not torch.distributed.is_available() or not torch.distributed.is_initialized():
        return 1
    return torch.distributed.get_world_size(group)


def _require_single_rank(group, what: str) -> None:
    n = _group_size(group)
    if n != 1:
        raise NotImplementedError(
            f"{what}: a {n}-rank process group was given; this build computes the full vocabulary on one GPU"
        )


def _to_device(t: torch.Tensor, like: torch.Tensor) -> torch.Tensor:
    return t if t.device == like.device else t.to(like.device)


def _prep_rows(logits, targets):
    if logits.dim() != 3:
        raise ValueError(f"expected logits [B, S, V], got {tuple(logits.shape)}")
    if logits.stride(-1) != 1:
        logits = logits.contiguous()
    targets = _to_device(targets, logits)
    if targets.dtype != torch.int64:
        targets = targets.long()
    return logits, targets


def _fwd_rows(ctx, logits, targets, n_inner, vocab_start, vocab_end, inference_only, temperature):
    """Shared forward: saves the logits (no copy), the targets and one fp32 log-sum-exp per row;
    the softmax is never materialised."""
    if temperature == 1.0:
        temperature = pending_temperature(logits)  # a divide apply_temperature_scaling left to this kernel
    logits, targets = _prep_rows(logits.detach(), targets)
    save = (not inference_only) and ctx.needs_input_grad[0]
    out, lse = _OPS.logprob_fwd(logits, targets, n_inner, vocab_start, vocab_end, temperature, NRL_TEMP_RCP, save)
    if save:
        ctx.save_for_backward(logits, targets, lse)
        ctx.meta = (n_inner, vocab_start, vocab_end, temperature)
    ctx.saved = save
    return out


def _bwd_rows(ctx, grad_out):
    """Shared backward: the gradient comes back in the logits' dtype, rows >= n_inner zeroed."""
    if not ctx.saved:
        raise RuntimeError("backward through a logprob computed with inference_only=True")
    logits, targets, lse = ctx.saved_tensors
    n_inner, vocab_start, vocab_end, temperature = ctx.meta
    grad = grad_out if grad_out.dtype == torch.float32 else grad_out.float()
    return _OPS.logprob_bwd(logits, targets, lse, grad, n_inner, vocab_start, vocab_end, temperature, NRL_TEMP_RCP)


class _RowsLogprob(torch.autograd.Function):
    """logits [B,S,V], targets [B,>=n_inner] (already aligned to the rows) -> fp32 [B,n_inner]."""

    @staticmethod
    def forward(ctx, logits, targets, n_inner, vocab_start, vocab_end, inference_only, temperature):
        return _fwd_rows(ctx, logits, targets, n_inner, vocab_start, vocab_end, inference_only, temperature)

    @staticmethod
    def backward(ctx, grad_out):
        return _bwd_rows(ctx, grad_out), None, None, None, None, None, None


def _rows_logprob(logits, targets, n_inner, vocab_start, vocab_end, inference_only, temperature=1.0):
    return _RowsLogprob.apply(logits, targets, n_inner, vocab_start, vocab_end, inference_only, float(temperature))


class _LogSoftmaxRows(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits):
        refuse_pending(logits, "_compute_distributed_log_softmax")
        x = logits.detach()
        x2 = x.reshape(-1, x.shape[-1])
        if x2.stride(-1) != 1:
            x2 = x2.contiguous()
        out = _OPS.log_softmax_fwd(x2)
        ctx.save_for_backward(out)
        return out.view(logits.shape)

    @staticmethod
    def backward(ctx, grad):
        (out,) = ctx.saved_tensors
        g2 = grad.reshape(out.shape)
        if g2.stride(-1) != 1:
            g2 = g2.contiguous()
        return _OPS.log_softmax_bwd(out, g2.to(out.dtype)).view(grad.shape)


def _compute_distributed_log_softmax_with_grad(vocab_parallel_logits: torch.Tensor, group: Any) -> torch.Tensor:
    """``model_utils.py:33-67`` on one rank: the stable log-softmax of every row, same shape and dtype as the
    input, differentiable.  The arithmetic is fp32 whatever the input dtype (the reference subtracts the
    maximum and exponentiates in the input dtype; its callers on this path cast to fp32 first)."""
    _require_single_rank(group, "_compute_distributed_log_softmax_with_grad")
    return _LogSoftmaxRows.apply(vocab_parallel_logits)


@torch.no_grad()
def _compute_distributed_log_softmax(vocab_parallel_logits: torch.Tensor, group: Any) -> torch.Tensor:
    """``model_utils.py:70-79``: the same without a graph."""
    return _compute_distributed_log_softmax_with_grad(vocab_parallel_logits, group)


class DistributedLogprob(torch.autograd.Function):
    """``model_utils.py:120-207``.  ``apply(logits, target, vocab_start_index, vocab_end_index, group,
    inference_only=False)`` with ``target`` already shifted; every position is computed."""

    @staticmethod
    def forward(ctx, vocab_parallel_logits, target, vocab_start_index, vocab_end_index, group, inference_only=False):
        _require_single_rank(group, "DistributedLogprob")
        return _fwd_rows(
            ctx, vocab_parallel_logits, target, target.shape[1], vocab_start_index, vocab_end_index, inference_only, 1.0
        )

    @staticmethod
    def backward(ctx, *grad_outputs):
        return _bwd_rows(ctx, grad_outputs[0]), None, None, None, None, None


class ChunkedDistributedLogprob(torch.autograd.Function):
    """``model_utils.py:267-380``.  The sequence-chunk loop only bounds the reference's working set;
    the streaming kernel has none, so ``chunk_size`` does not change the launch and chunked and
    unchunked results are bit-identical."""

    @staticmethod
    def forward(ctx, vocab_parallel_logits, target, vocab_start_index, vocab_end_index, chunk_size, tp_group,
                inference_only=False):
        _require_single_rank(tp_group, "ChunkedDistributedLogprob")
        if chunk_size is None or int(chunk_size) < 1:
            raise ValueError(f"chunk_size must be a positive int, got {chunk_size}")
        return _fwd_rows(
            ctx, vocab_parallel_logits, target, target.shape[1], vocab_start_index, vocab_end_index, inference_only, 1.0
        )

    @staticmethod
    def backward(ctx, *grad_outputs):
        return _bwd_rows(ctx, grad_outputs[0]), None, None, None, None, None, None


class DistributedLogprobWithSampling(torch.autograd.Function):
    """``model_utils.py:383-510`` on one rank: ``apply(logits, target, tp_group, top_k, top_p,
    inference_only=False)`` with ``target`` already shifted.  No all-to-all and no sort: the selection
    kernel finds the kept set of every row on chip."""

    @staticmethod
    def forward(ctx, vocab_parallel_logits, target, tp_group, top_k, top_p, inference_only=False):
        from .sampling_logprob import _sampled_fwd

        _require_single_rank(tp_group, "DistributedLogprobWithSampling")
        return _sampled_fwd(ctx, vocab_parallel_logits, target, target.shape[1], top_k, top_p, inference_only)

    @staticmethod
    def backward(ctx, *grad_outputs):
        from .sampling_logprob import _sampled_bwd

        return _sampled_bwd(ctx, grad_outputs[0]), None, None, None, None, None


class ChunkedDistributedLogprobWithSampling(torch.autograd.Function):
    """``model_utils.py:513-719``; ``chunk_size`` bounds the reference's sort buffers and has no effect here."""

    @staticmethod
    def forward(ctx, vocab_parallel_logits, target, tp_group, top_k, top_p, chunk_size, inference_only=False):
        from .sampling_logprob import _sampled_fwd

        _require_single_rank(tp_group, "ChunkedDistributedLogprobWithSampling")
        return _sampled_fwd(ctx, vocab_parallel_logits, target, target.shape[1], top_k, top_p, inference_only)

    @staticmethod
    def backward(ctx, *grad_outputs):
        from .sampling_logprob import _sampled_bwd

        return _sampled_bwd(ctx, grad_outputs[0]), None, None, None, None, None, None


def _get_tokens_on_this_cp_rank(input_ids, cp_rank: int, cp_size: int, seq_dim: int = 1):
    """``model_utils.py:1199-1233`` for the only context-parallel size this build runs with."""
    if cp_size != 1:
        raise NotImplementedError("context parallelism spans more than one GPU")
    return input_ids


def from_parallel_logits_to_logprobs(
    vocab_parallel_logits: torch.Tensor,
    target: torch.Tensor,
    vocab_start_index: int,
    vocab_end_index: int,
    tp_group: Any,
    inference_only: bool = False,
    cp_group: Optional[Any] = None,
    chunk_size: Optional[int] = None,
    sampling_params: Optional[TrainingSamplingParams] = None,
) -> torch.Tensor:
    """``model_utils.py:947-1042``: ``target`` is unshifted ``[B, S]``; returns ``[B, S-1]`` fp32.

    The roll by -1 and the dropped last column become pointer arithmetic: row ``(b, i)`` reads
    ``target[b, i+1]`` and only ``S-1`` rows per sequence are launched.  Logits longer than the
    targets (context-parallel padding in the reference, ``:984-986``) are ignored beyond ``S``."""
    _require_single_rank(tp_group, "from_parallel_logits_to_logprobs")
    _require_single_rank(cp_group, "from_parallel_logits_to_logprobs")
    b, s = target.shape
    if vocab_parallel_logits.shape[1] < s:
        raise ValueError(f"logits cover {vocab_parallel_logits.shape[1]} positions, targets {s}")
    if s - 1 <= 0:  # nothing to predict (a one-token or empty sequence): torch's gather returns an empty result
        return torch.zeros((b, 0), dtype=torch.float32, device=vocab_parallel_logits.device)
    if need_top_k_or_top_p_filtering(sampling_params):
        from .sampling_logprob import rows_logprob_sampled

        return rows_logprob_sampled(
            vocab_parallel_logits, target[:, 1:], s - 1, sampling_params.top_k, sampling_params.top_p, inference_only
        )
    return _rows_logprob(
        vocab_parallel_logits, target[:, 1:], s - 1, vocab_start_index, vocab_end_index, inference_only
    )


def get_next_token_logprobs_from_logits(
    input_ids: torch.Tensor,
    next_token_logits: torch.Tensor,
    seq_index: Optional[torch.Tensor] = None,
    vocab_parallel_rank: Optional[int] = None,
    vocab_parallel_group: Optional[Any] = None,
    context_parallel_group: Optional[Any] = None,
    sampling_params: Optional[TrainingSamplingParams] = None,
    chunk_size: Optional[int] = None,
) -> torch.Tensor:
    """``model_utils.py:1611-1695``.  All three branches of the reference reduce to the same maths
    on one GPU.  The reference first casts the logits to fp32 (``:1648-1649``); the kernel reads
    bf16/fp16 directly and accumulates in fp32, which is the same arithmetic without the copy, and
    autograd receives the gradient already narrowed (one rounding, as the cast's backward does)."""
    if vocab_parallel_group is not None:
        assert vocab_parallel_rank is not None, (
            "vocab_parallel_rank must be provided when vocab_parallel_group is provided"
        )
        _require_single_rank(vocab_parallel_group, "get_next_token_logprobs_from_logits")
    _require_single_rank(context_parallel_group, "get_next_token_logprobs_from_logits")
    if seq_index is not None:
        raise NotImplementedError("seq_index belongs to context-parallel DTensor logits (more than one GPU)")
    if hasattr(next_token_logits, "to_local"):
        next_token_logits = next_token_logits.to_local()
    vocab = next_token_logits.shape[-1]
    rank = vocab_parallel_rank or 0
    inference_only = not (torch.is_grad_enabled() and next_token_logits.requires_grad)
    return from_parallel_logits_to_logprobs(
        next_token_logits,
        input_ids,
        vocab_start_index=rank * vocab,
        vocab_end_index=(rank + 1) * vocab,
        tp_group=vocab_parallel_group,
        inference_only=inference_only,
        cp_group=context_parallel_group,
        chunk_size=None,
        sampling_params=sampling_params,
    )[:, : input_ids.shape[1] - 1]


def _mesh_dim_size(mesh, name: str) -> int:
    names = getattr(mesh, "mesh_dim_names", None)
    if names is None or name not in names:
        return 1
    return int(mesh.shape[names.index(name)])


def dtensor_from_parallel_logits_to_logprobs(
    vocab_parallel_logits: torch.Tensor,
    target: Any,
    vocab_start_index: int,
    vocab_end_index: int,
    tp_group: Any,
    inference_only: bool = False,
    seq_index: Optional[torch.Tensor] = None,
    chunk_size: Optional[int] = None,
    sampling_params: Optional[TrainingSamplingParams] = None,
) -> torch.Tensor:
    """``model_utils.py:839-944``: the DTensor worker's twin of ``from_parallel_logits_to_logprobs``.  ``target``
    may be a DTensor; on one GPU its mesh has no context-parallel extent, so the re-ordering by
    ``seq_index`` (``:880-892``) never applies and the local shard is the whole tensor."""
    if hasattr(target, "to_local"):
        if _mesh_dim_size(target.device_mesh, "cp") > 1:
            raise NotImplementedError("dtensor_from_parallel_logits_to_logprobs: context parallelism needs more than one GPU")
        target = target.to_local()
    if seq_index is not None:
        raise NotImplementedError("seq_index belongs to context-parallel logits (more than one GPU)")
    return from_parallel_logits_to_logprobs(
        vocab_parallel_logits, target, vocab_start_index, vocab_end_index, tp_group, inference_only=inference_only,
        cp_group=None, chunk_size=chunk_size, sampling_params=sampling_params)


def get_logprobs_from_vocab_parallel_logits(
    vocab_parallel_logits: Any,
    input_ids: Any,
    seq_index: Optional[torch.Tensor] = None,
    chunk_size: Optional[int] = None,
    sampling_params: Optional[TrainingSamplingParams] = None,
) -> torch.Tensor:
    """``model_utils.py:1558-1608``: vocabulary-parallel DTensor logits -> ``[B, S-1]`` logprobs.  The rank's
    vocabulary interval comes from the mesh's ``tp`` group (``:1592-1596``), which has one member here."""
    mesh = vocab_parallel_logits.device_mesh
    if seq_index is not None:
        assert _mesh_dim_size(mesh, "cp") >= 1 and "cp" in (mesh.mesh_dim_names or ()), (
            "seq_index must be provided for cp sharded logits"
        )
    tp_group = mesh.get_group("tp")
    _require_single_rank(tp_group, "get_logprobs_from_vocab_parallel_logits")
    tp_rank, tp_size = tp_group.rank(), tp_group.size()
    per_rank = vocab_parallel_logits.shape[-1] // tp_size
    return dtensor_from_parallel_logits_to_logprobs(
        vocab_parallel_logits.to_local(), input_ids, per_rank * tp_rank, (tp_rank + 1) * per_rank, tp_group,
        inference_only=not torch.is_grad_enabled(), seq_index=seq_index, chunk_size=chunk_size,
        sampling_params=sampling_params)


# ------------------------------------------------------------------------------------------------
# packed sequences
# ------------------------------------------------------------------------------------------------
class _PackedLogprob(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits2d, targets1d, pre_rolled, cu_dev, unpacked_seqlen, vocab_start, vocab_end, inference_only,
                temperature):
        save = (not inference_only) and ctx.needs_input_grad[0]
        out, lse = _OPS.logprob_packed_fwd(
            logits2d.detach(), targets1d, pre_rolled, cu_dev, unpacked_seqlen, vocab_start, vocab_end, temperature,
            NRL_TEMP_RCP, save,
        )
        if save:
            ctx.save_for_backward(logits2d.detach(), targets1d, cu_dev, lse)
            ctx.meta = (pre_rolled, unpacked_seqlen, vocab_start, vocab_end, temperature)
        ctx.saved = save
        return out

    @staticmethod
    def backward(ctx, grad_out):
        if not ctx.saved:
            raise RuntimeError("backward through a logprob computed with inference_only=True")
        logits2d, targets1d, cu_dev, lse = ctx.saved_tensors
        pre_rolled, unpacked_seqlen, vocab_start, vocab_end, temperature = ctx.meta
        d = _OPS.logprob_packed_bwd(
            logits2d, targets1d, pre_rolled, cu_dev, unpacked_seqlen, vocab_start, vocab_end, temperature, NRL_TEMP_RCP,
            lse, grad_out.float(),
        )
        return d, None, None, None, None, None, None, None, None


def _checked_cu_seqlens(cu_seqlens_padded: torch.Tensor, total: int, n_targets: int, device) -> torch.Tensor:
    """The sequence boundaries as int32 on the device.  Boundaries that live on the host are checked there (they
    should be non-decreasing and stay inside the packed buffers).  Boundaries that live on the GPU are taken as they
    are, so the host neither reads them nor waits for the device (the reference reads them per sequence): the
    kernels find a position's sequence by bisection, which ends at a span that contains it whatever the order, and
    clamp the target index to the packed row, so bad boundaries give wrong numbers but no stray access."""
    if cu_seqlens_padded.is_cuda:
        if cu_seqlens_padded.dim() != 1 or cu_seqlens_padded.numel() < 1:
            raise ValueError("cu_seqlens_padded must be a 1-D tensor with at least one entry")
        return cu_seqlens_padded.detach().to(device=device, dtype=torch.int32).contiguous()
    host = cu_seqlens_padded.detach().to("cpu", torch.int64)
    if host.dim() != 1 or host.numel() < 1:
        raise ValueError("cu_seqlens_padded must be a 1-D tensor with at least one entry")
    if host.numel() > 1 and bool((host[1:] < host[:-1]).any()):
        raise ValueError("cu_seqlens_padded must be non-decreasing")
    if int(host[0]) < 0 or int(host[-1]) > total or int(host[-1]) > n_targets:
        raise ValueError(
            f"cu_seqlens_padded spans [{int(host[0])}, {int(host[-1])}) but the packed row has {total} positions "
            f"and {n_targets} targets"
        )
    return host.to(torch.int32).to(device)


def from_parallel_logits_to_logprobs_packed_sequences(
    vocab_parallel_logits: torch.Tensor,
    target: torch.Tensor,
    cu_seqlens_padded: torch.Tensor,
    unpacked_seqlen: int,
    vocab_start_index: int,
    vocab_end_index: int,
    group: Any,
    inference_only: bool = False,
    cp_group: Optional[Any] = None,
    chunk_size: Optional[int] = None,
    sampling_params: Optional[TrainingSamplingParams] = None,
    target_is_pre_rolled: bool = False,
) -> torch.Tensor:
    """``model_utils.py:1045-1196``: packed ``[1, T, V]`` logits -> unpacked ``[B, unpacked_seqlen-1]``.

    The per-sequence roll, the dropped last position of every sequence and the unpacking are index
    arithmetic inside the kernel (a binary search of ``cu_seqlens_padded`` per row); positions that
    never reach the output are not read at all."""
    _require_single_rank(group, "from_parallel_logits_to_logprobs_packed_sequences")
    _require_single_rank(cp_group, "from_parallel_logits_to_logprobs_packed_sequences")
    if vocab_parallel_logits.dim() != 3 or vocab_parallel_logits.shape[0] != 1:
        raise ValueError(f"expected packed logits [1, T, V], got {tuple(vocab_parallel_logits.shape)}")
    temperature = pending_temperature(vocab_parallel_logits)  # a divide apply_temperature_scaling left to the kernel
    logits2d = vocab_parallel_logits.squeeze(0)
    if logits2d.stride(-1) != 1:
        logits2d = logits2d.contiguous()
    targets1d = _to_device(target, logits2d).reshape(-1).long().contiguous()
    total = logits2d.shape[0]
    cu_dev = _checked_cu_seqlens(cu_seqlens_padded, total, targets1d.shape[0], logits2d.device)
    if need_top_k_or_top_p_filtering(sampling_params):
        from .sampling_logprob import packed_logprob_sampled

        return packed_logprob_sampled(
            logits2d, targets1d, target_is_pre_rolled, cu_dev, int(unpacked_seqlen), sampling_params.top_k,
            sampling_params.top_p, inference_only, temperature,
        )
    return _PackedLogprob.apply(
        logits2d, targets1d, bool(target_is_pre_rolled), cu_dev, int(unpacked_seqlen), vocab_start_index,
        vocab_end_index, inference_only, temperature,
    )


# ------------------------------------------------------------------------------------------------
# fused lm_head: hidden states -> logprobs
# ------------------------------------------------------------------------------------------------
# Whether the forward keeps its bf16 logits [N, V] for the backward, which then reads them instead of multiplying
# the hidden states and the weights a second time (a quarter of the step's matrix work).  The reference recomputes
# (``model_utils.py:2249-2262``) because its logits are fp32 and its memory 80 GB; here the logits of 65 536 tokens
# x 151 936 ids are 20 GB of 288.  True / False force the choice; "auto" keeps them while they take no more than
# ``LMHEAD_KEEP_FRACTION`` of the memory that is free when the forward runs and, together with the backward's
# workspace, no more than half of it.  The gradients are the same both ways.
LMHEAD_KEEP_LOGITS: Any = "auto"
LMHEAD_KEEP_FRACTION = 0.25


def _keep_lmhead_logits(n_tokens: int, vocab: int, device: torch.device, hidden_size: int = 0) -> bool:
    if LMHEAD_KEEP_LOGITS != "auto":
        return bool(LMHEAD_KEEP_LOGITS)
    need = ((n_tokens + 31) // 32 * 32) * ((vocab + 31) // 32 * 32) * 2
    free, _ = torch.cuda.mem_get_info(device)
    free += torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)  # the allocator's own free blocks
    # (and the backward's own workspace and outputs must still fit comfortably next to them)
    later = 0
    if hidden_size > 0:
        from .. import _lib

        later = _lib.load().nrl_lmhead_bwd_workspace_bytes(n_tokens, hidden_size, vocab) + n_tokens * hidden_size * 4
    return need <= LMHEAD_KEEP_FRACTION * free and need + later <= 0.5 * free


class ChunkedDistributedHiddenStatesToLogprobs(torch.autograd.Function):
    """``model_utils.py:2137-2316`` on one rank: ``apply(hidden [S,B,H], target [B,S] (already shifted),
    output_weight [V,H], vocab_start_index, vocab_end_index, chunk_size, tp_group, inference_only)``
    -> fp32 ``[B,S]``.  The product runs on the bf16 matrix cores with the softmax folded into the
    GEMM epilogue; ``chunk_size`` (the reference's sequence chunk) is not needed to bound memory in the
    forward, and the backward chunks tokens on its own.  See ``LMHEAD_KEEP_LOGITS`` for what the forward saves."""

    @staticmethod
    def forward(ctx, tensor_parallel_hidden_states, target, output_weight_layer, vocab_start_index, vocab_end_index,
                chunk_size, tp_group, inference_only=False):
        _require_single_rank(tp_group, "ChunkedDistributedHiddenStatesToLogprobs")
        hidden = tensor_parallel_hidden_states.detach()
        if hidden.dim() != 3:
            raise ValueError(f"expected hidden states [S, B, H], got {tuple(hidden.shape)}")
        s, b, h = hidden.shape
        hidden2d = hidden.reshape(s * b, h)
        weight = output_weight_layer.detach()
        tgt = _to_device(target, hidden).long().t().contiguous().reshape(-1)  # token order of the hidden rows: (s, b)
        ctx.saved = (not inference_only) and (ctx.needs_input_grad[0] or ctx.needs_input_grad[2])
        keep = ctx.saved and _keep_lmhead_logits(s * b, weight.shape[0], hidden.device, h)
        lp, lse, logits = _OPS.lmhead_logprob_fwd(hidden2d, weight, tgt, vocab_start_index, vocab_end_index, keep)
        if ctx.saved:
            ctx.save_for_backward(hidden2d, weight, tgt, lse, logits)
            ctx.meta = (s, b, h, vocab_start_index, vocab_end_index, tensor_parallel_hidden_states.dtype,
                        output_weight_layer.dtype)
        return lp.view(s, b).t().contiguous()

    @staticmethod
    def backward(ctx, *grad_outputs):
        if not ctx.saved:
            raise RuntimeError("backward through a logprob computed with inference_only=True")
        hidden2d, weight, tgt, lse, logits = ctx.saved_tensors
        s, b, h, v0, v1, h_dtype, w_dtype = ctx.meta
        grad = grad_outputs[0].float().t().contiguous().reshape(-1)
        dh, dw = _OPS.lmhead_logprob_bwd(hidden2d, weight, tgt, lse, grad, v0, v1, logits if logits.numel() else None)
        return dh.view(s, b, h).to(h_dtype), None, dw.to(w_dtype), None, None, None, None, None


def from_parallel_hidden_states_to_logprobs(
    tensor_parallel_hidden_states: torch.Tensor,
    output_weight_layer: torch.Tensor,
    runtime_gather_output: bool,
    target: torch.Tensor,
    vocab_start_index: int,
    vocab_end_index: int,
    tp_group: Any,
    inference_only: bool = False,
    cp_group: Optional[Any] = None,
    chunk_size: Optional[int] = None,
) -> torch.Tensor:
    """``model_utils.py:2106-2134``: hidden ``[S,B,H]`` (sequence first), weight ``[V,H]``, unshifted
    ``target [B,S]`` -> ``[B, S-1]`` fp32."""
    assert _group_size(cp_group) == 1, "Context parallelism is not supported for linear CE fusion loss"
    rolled = target.roll(shifts=-1, dims=-1)
    logprobs = ChunkedDistributedHiddenStatesToLogprobs.apply(
        tensor_parallel_hidden_states, rolled, output_weight_layer, vocab_start_index, vocab_end_index, chunk_size,
        tp_group, inference_only,
    )
    return logprobs[:, :-1]



# ------------------------------------------------------------------------------------------------
# distillation reductions on the same streaming core (TP = 1)
# ------------------------------------------------------------------------------------------------
class ChunkedDistributedEntropy(torch.autograd.Function):
    """``model_utils.py:2023-2103``: ``H_all[b, s] = sum_v p_v log p_v``.  ``chunk_size`` is accepted for
    signature compatibility; a row never leaves the chip, so nothing needs chunking."""

    @staticmethod
    def forward(ctx, vocab_parallel_logits, chunk_size, tp_group, inference_only=False):
        _require_single_rank(tp_group, "ChunkedDistributedEntropy")
        x = vocab_parallel_logits if vocab_parallel_logits.stride(-1) == 1 else vocab_parallel_logits.contiguous()
        h, lse = torch.ops.rl_amd.neg_entropy_fwd(x)
        if not inference_only:
            ctx.save_for_backward(x, lse, h)
        return h

    @staticmethod
    def backward(ctx, *grad_outputs):
        x, lse, h = ctx.saved_tensors
        g = grad_outputs[0].to(torch.float32).contiguous()
        return torch.ops.rl_amd.neg_entropy_bwd(x, lse, h, g), None, None, None


class ChunkedDistributedGatherLogprob(torch.autograd.Function):
    """``model_utils.py:722-836``: log-softmax once, gathered at ``global_indices [B, S, K]``."""

    @staticmethod
    def forward(ctx, vocab_parallel_logits, global_indices, vocab_start_index, vocab_end_index, chunk_size, tp_group,
                inference_only=False):
        _require_single_rank(tp_group, "ChunkedDistributedGatherLogprob")
        x = vocab_parallel_logits if vocab_parallel_logits.stride(-1) == 1 else vocab_parallel_logits.contiguous()
        idx = _to_device(global_indices, x).long().contiguous()
        out, lse = torch.ops.rl_amd.gather_logprob_fwd(x, idx, int(vocab_start_index), int(vocab_end_index))
        if not inference_only:
            ctx.save_for_backward(x, idx, lse)
            ctx.vocab_range = (int(vocab_start_index), int(vocab_end_index))
        return out

    @staticmethod
    def backward(ctx, *grad_outputs):
        x, idx, lse = ctx.saved_tensors
        g = grad_outputs[0].to(torch.float32).contiguous()
        d = torch.ops.rl_amd.gather_logprob_bwd(x, idx, ctx.vocab_range[0], ctx.vocab_range[1], lse, g)
        return d, None, None, None, None, None, None


class DistributedCrossEntropy(torch.autograd.Function):
    """``model_utils.py:209-264``: soft-target cross entropy ``H(p_target, q_student)``; the gradient
    flows to the student logits only."""

    @staticmethod
    def forward(ctx, student_logits, target_logits, group, inference_only=False):
        if student_logits.shape != target_logits.shape:
            raise ValueError(
                "student_logits and target_logits must have the same shape, "
                f"got {student_logits.shape} and {target_logits.shape}."
            )
        _require_single_rank(group, "DistributedCrossEntropy")
        lead = student_logits.shape[:-1]
        x = student_logits.reshape(1, -1, student_logits.shape[-1]) if student_logits.dim() != 3 else student_logits
        y = target_logits.reshape(x.shape) if target_logits.dim() != 3 else target_logits
        x = x if x.stride(-1) == 1 else x.contiguous()
        y = _to_device(y, x)
        ce, lx, ly = torch.ops.rl_amd.soft_cross_entropy_fwd(x, y)
        if not inference_only:
            ctx.save_for_backward(x, y, lx, ly)
            ctx.in_shape = student_logits.shape
        return ce.reshape(lead)

    @staticmethod
    def backward(ctx, *grad_outputs):
        x, y, lx, ly = ctx.saved_tensors
        g = grad_outputs[0].to(torch.float32).reshape(lx.shape).contiguous()
        d = torch.ops.rl_amd.soft_cross_entropy_bwd(x, y, lx, ly, g)
        return d.reshape(ctx.in_shape), None, None, None


class _TopkLogSoftmax(torch.autograd.Function):
    """log_softmax over the K logits of every row at the given vocabulary indices."""

    @staticmethod
    def forward(ctx, logits, indices):
        out = torch.ops.rl_amd.topk_logsoftmax_fwd(logits.detach(), indices)
        ctx.save_for_backward(logits, indices, out)
        return out

    @staticmethod
    def backward(ctx, grad):
        logits, indices, out = ctx.saved_tensors
        return torch.ops.rl_amd.topk_logsoftmax_bwd(logits, indices, out, grad.contiguous().float()), None


def get_distillation_topk_logprobs_from_logits(
    student_logits: torch.Tensor,
    teacher_topk_logits: torch.Tensor,
    teacher_topk_indices: torch.Tensor,
    zero_outside_topk: bool,
    calculate_entropy: bool,
    vocab_parallel_rank: Optional[int] = None,
    vocab_parallel_group: Optional[Any] = None,
    context_parallel_group: Optional[Any] = None,
):
    """``model_utils.py:1856-2020``: the student's log-probabilities at the teacher's top-k ids, the teacher's
    own top-k log-probabilities and (optionally) ``H_all = sum_v p log p`` of the student rows, all cut to the
    next-token alignment ``[:, :-1]``.

    ``zero_outside_topk``: the student entries come from the full-vocabulary log-softmax (streaming gather
    kernel); otherwise from a softmax over just the K gathered logits.  The student's fp32 copy
    (``:1874``) is not made: the kernels read the logits in their dtype and accumulate in fp32."""
    if teacher_topk_indices.shape[-1] <= 0:
        raise ValueError(
            f"topk must be positive, got {teacher_topk_indices.shape[-1]}. "
            "topk=0 is not supported as it would result in empty tensor operations."
        )
    if vocab_parallel_group is not None:
        assert vocab_parallel_rank is not None, (
            "vocab_parallel_rank must be provided when vocab_parallel_group is provided"
        )
        _require_single_rank(vocab_parallel_group, "get_distillation_topk_logprobs_from_logits")
    _require_single_rank(context_parallel_group, "get_distillation_topk_logprobs_from_logits")
    if hasattr(student_logits, "to_local"):
        mesh = student_logits.device_mesh
        _require_single_rank(mesh.get_group("tp"), "get_distillation_topk_logprobs_from_logits")
        if _mesh_dim_size(mesh, "cp") > 1:
            raise NotImplementedError("get_distillation_topk_logprobs_from_logits: context parallelism needs more than one GPU")
        student_logits = student_logits.to_local()
    indices = teacher_topk_indices.to(student_logits.device)
    if indices.dtype != torch.int64:
        indices = indices.long()
    vocab = student_logits.shape[-1]
    seq = student_logits.shape[1]
    H_all = None
    if zero_outside_topk:
        student_topk_logprobs = ChunkedDistributedGatherLogprob.apply(student_logits, indices, 0, vocab, seq, None, False)
        if calculate_entropy:
            H_all = ChunkedDistributedEntropy.apply(student_logits, seq, None, False)
    else:
        student_topk_logprobs = _TopkLogSoftmax.apply(student_logits, indices)
    teacher = teacher_topk_logits.to(student_topk_logprobs.device)
    if teacher.dim() != 3:
        raise ValueError(f"teacher_topk_logits must be [B, S, K], got {tuple(teacher.shape)}")
    if teacher.stride(2) != 1 and teacher.shape[2] > 1:
        teacher = teacher.contiguous()
    teacher_topk_logprobs = torch.ops.rl_amd.topk_logsoftmax_fwd(teacher.detach(), None)
    teacher_topk_logprobs = teacher_topk_logprobs[:, :-1, :]
    student_topk_logprobs = student_topk_logprobs[:, :-1, :]
    if calculate_entropy and H_all is not None:
        H_all = H_all[:, :-1]
    return student_topk_logprobs, teacher_topk_logprobs, H_all
