"""Token logprobs under top-k / top-p filtering (K3), the counterpart of
``DistributedLogprobWithSampling`` / ``ChunkedDistributedLogprobWithSampling``
(``nemo_rl/distributed/model_utils.py:383-719``) and of ``apply_top_k_top_p``
(``nemo_rl/algorithms/logits_sampling_utils.py:254-285``) on one GPU."""

from __future__ import annotations

import torch

from .. import ops as _ops  # noqa: F401
from .._deferred import pending_temperature, refuse_pending
from .._lib import NRL_TEMP_RCP

_OPS = torch.ops.rl_amd

def _norm_k(top_k) -> int:
    return int(top_k) if top_k is not None and top_k > 0 else 0


def _norm_p(top_p) -> float:
    return float(top_p) if top_p is not None else 1.0


def _record_capacity(top_k: int) -> int:
    """Entries per row of the kept-set record the forward leaves for the backward (0: none).  Under a top-k the kept
    set has at most k elements plus ties, a few dozen ids of a 150 000-wide row: with them on record the backward
    writes a gradient row (zeros and those entries) without reading the logits again.  8 bytes per entry and row;
    rows whose kept set is larger fall back to the streaming backward one by one."""
    if 0 < top_k <= 64:
        return 64
    if 0 < top_k <= 128:
        return 128
    return 128 if top_k <= 0 else 0  # top-p alone: peaked rows keep a small nucleus


def _sampled_fwd(ctx, logits, targets, n_inner, top_k, top_p, inference_only, want_unfiltered=False, temperature=1.0):
    """Shared forward of the filtered-logprob autograd functions: saves the logits (no copy), the targets
    and three numbers per row (threshold, tie index, kept log-sum-exp)."""
    if temperature == 1.0:
        temperature = pending_temperature(logits)  # a divide apply_temperature_scaling left to this kernel
    logits = logits.detach()
    if logits.dim() != 3:
        raise ValueError(f"expected logits [B, S, V], got {tuple(logits.shape)}")
    if logits.stride(-1) != 1:
        logits = logits.contiguous()
    targets = targets.to(logits.device)
    if targets.dtype != torch.int64:
        targets = targets.long()
    ctx.saved = (not inference_only) and ctx.needs_input_grad[0]
    capacity = _record_capacity(_norm_k(top_k)) if ctx.saved else 0
    if capacity:
        lp, thr, tie, lse, lpu, *record = _OPS.topk_topp_logprob_fwd_rec(
            logits, targets, n_inner, _norm_k(top_k), _norm_p(top_p), temperature, NRL_TEMP_RCP, want_unfiltered, capacity
        )
    else:
        record = []
        lp, thr, tie, lse, lpu = _OPS.topk_topp_logprob_fwd(
            logits, targets, n_inner, _norm_k(top_k), _norm_p(top_p), temperature, NRL_TEMP_RCP, want_unfiltered
        )
    if ctx.saved:
        ctx.save_for_backward(logits, targets, thr, tie, lse, *record)
        ctx.n_inner = n_inner
        ctx.temperature = temperature
    return (lp, lpu) if want_unfiltered else lp


def _sampled_bwd(ctx, grad_lp):
    if not ctx.saved:
        raise RuntimeError("backward through a logprob computed with inference_only=True")
    logits, targets, thr, tie, lse, *record = ctx.saved_tensors
    return _OPS.topk_topp_logprob_bwd(
        logits, targets, thr, tie, lse, grad_lp.float().contiguous(), ctx.n_inner, ctx.temperature, NRL_TEMP_RCP, *record
    )


class _RowsLogprobSampled(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, targets, n_inner, top_k, top_p, inference_only, temperature):
        return _sampled_fwd(ctx, logits, targets, n_inner, top_k, top_p, inference_only, temperature=temperature)

    @staticmethod
    def backward(ctx, grad_lp):
        return _sampled_bwd(ctx, grad_lp), None, None, None, None, None, None


def rows_logprob_sampled(logits, targets, n_inner, top_k, top_p, inference_only=False, temperature=1.0):
    """logits [B,S,V], targets [B,>=n_inner] aligned with the rows -> fp32 [B,n_inner]; a target outside
    the kept set gives ``-inf`` (``model_utils.py:445-452``)."""
    return _RowsLogprobSampled.apply(logits, targets, n_inner, top_k, top_p, inference_only, float(temperature))


def packed_logprob_sampled(logits2d, targets1d, pre_rolled, cu_dev, unpacked_seqlen, top_k, top_p, inference_only,
                           temperature=1.0):
    """Packed ``[T, V]`` logits under filtering -> unpacked ``[n_seq, unpacked_seqlen-1]``.  Every packed
    position is one row of the selection kernel; the per-sequence roll and the unpacking are index
    tensors built from ``cu_seqlens`` (sizes ``[T]`` and ``[n_seq, L]``)."""
    dev = logits2d.device
    total = logits2d.shape[0]
    cu = cu_dev.to(torch.int64)
    n_seq = cu.shape[0] - 1
    width = unpacked_seqlen - 1
    pos = torch.arange(total, device=dev)
    seq = torch.searchsorted(cu, pos, right=True) - 1
    seq_c = seq.clamp(0, max(n_seq - 1, 0))
    start, stop = cu[seq_c], cu[seq_c + 1] if n_seq > 0 else cu[seq_c]
    inside = (seq >= 0) & (seq < n_seq) & (pos < stop)
    if pre_rolled:
        tgt_idx = pos
    else:
        tgt_idx = torch.where(pos + 1 < stop, pos + 1, start)
    tgt = torch.where(inside, targets1d[tgt_idx.clamp(max=targets1d.shape[0] - 1)], torch.zeros_like(pos))
    lp_flat = rows_logprob_sampled(logits2d.unsqueeze(0), tgt.unsqueeze(0), total, top_k, top_p, inference_only,
                                   temperature)[0]
    # out[s, p] = lp_flat[cu[s] + p] for p < min(len_s - 1, width)
    p = torch.arange(width, device=dev).unsqueeze(0)
    lens = (cu[1:] - cu[:-1]).unsqueeze(-1)
    src = cu[:-1].unsqueeze(-1) + p
    valid = p < (lens - 1)
    gathered = lp_flat[src.clamp(max=max(total - 1, 0))] if total > 0 else torch.zeros((n_seq, width), device=dev)
    return torch.where(valid, gathered, torch.zeros_like(gathered))


class _FilterLogits(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits3d, top_k, top_p):
        x = logits3d.detach()
        _, thr, tie, _, _ = _OPS.topk_topp_logprob_fwd(x, None, x.shape[1], top_k, top_p, 1.0, NRL_TEMP_RCP, False)
        filtered, keep = _OPS.topk_topp_filter(x, thr, tie, 1.0, NRL_TEMP_RCP)
        keep = keep.bool()
        ctx.save_for_backward(keep)
        ctx.mark_non_differentiable(keep)
        return filtered, keep

    @staticmethod
    def backward(ctx, grad_filtered, _grad_keep):
        (keep,) = ctx.saved_tensors
        return grad_filtered * keep, None, None


def filter_logits(logits, top_k, top_p):
    """``apply_top_k_top_p``: filtered logits (``-inf`` outside the kept set) and the boolean keep mask, same
    shape as ``logits``; gradients pass through where kept."""
    refuse_pending(logits, "apply_top_k_top_p")
    shape = logits.shape
    x = logits.reshape(1, -1, shape[-1]) if logits.dim() != 3 else logits
    if x.stride(-1) != 1:
        x = x.contiguous()
    filtered, keep = _FilterLogits.apply(x, _norm_k(top_k), _norm_p(top_p))
    return filtered.reshape(shape), keep.reshape(shape)
