"""Oracle: per-token vocabulary logits -> token log-probabilities.

Test infrastructure only (see ``oracle/__init__.py``).

Single-GPU (TP = CP = 1) restatement of ``nemo_rl/distributed/model_utils.py``:
the collectives at ``:50-54, 61-65, 152-156`` reduce over one rank and vanish.
The backward of the row op restates the reference's hand-written one (it differs from
plain autograd only for targets outside the vocabulary shard); the tests pin it to
torch autograd of ``log_softmax(x).gather(t)`` for in-range targets.
"""

from __future__ import annotations

from typing import Optional

import torch

from . import sampling


def apply_temperature(logits: torch.Tensor, temperature: Optional[float]) -> torch.Tensor:
    """``nemo_rl/models/automodel/train.py:180-194``: ``logits.div_(T)`` in the
    logits' own dtype (bf16 logits are re-rounded to bf16), skipped for T in
    (None, 1).  Returns a new tensor; the reference divides in place."""
    if temperature is None or temperature == 1.0:
        return logits
    return logits / temperature


def stable_log_softmax(x32: torch.Tensor) -> torch.Tensor:
    """``model_utils.py:49-67``: ``m = amax``; ``x - m``; ``sum(exp)``;
    ``(x - m) - log(sum)``, all fp32."""
    m = torch.amax(x32, dim=-1, keepdim=True).detach()
    shifted = x32 - m
    return shifted - shifted.exp().sum(-1, keepdim=True).log()


class _RowsLogprob(torch.autograd.Function):
    """``DistributedLogprob`` on one rank (``model_utils.py:136-207``).  The hand-written backward is
    ``-softmax * g`` for every row plus ``g`` at the target of the rows whose target is inside the
    shard (``:193-197``): a row whose target lies in another shard returns 0 in the forward but still
    receives the softmax term, because the full-vocabulary logprob is the sum over shards."""

    @staticmethod
    def forward(ctx, logits, target, vocab_start, vocab_end):
        outside = (target < vocab_start) | (target >= vocab_end)
        local = (target - vocab_start).masked_fill(outside, 0)
        logp = stable_log_softmax(logits.to(torch.float32))
        picked = torch.gather(logp, -1, local.unsqueeze(-1)).squeeze(-1)
        ctx.save_for_backward(logp.exp(), outside, local)
        return picked.masked_fill(outside, 0.0)

    @staticmethod
    def backward(ctx, grad_output):
        softmax, outside, local = ctx.saved_tensors
        onehot = torch.nn.functional.one_hot(local, num_classes=softmax.shape[-1]) * (~outside).unsqueeze(-1)
        return (onehot.float() - softmax) * grad_output.unsqueeze(-1), None, None, None


def rows_logprob(
    logits: torch.Tensor,
    target: torch.Tensor,
    vocab_start: int = 0,
    vocab_end: Optional[int] = None,
) -> torch.Tensor:
    """``logits [..., V]`` any float dtype, ``target [...]`` int64, already shifted.  Targets outside
    ``[vocab_start, vocab_end)`` give 0 (``model_utils.py:137-150``)."""
    if vocab_end is None:
        vocab_end = vocab_start + logits.shape[-1]
    return _RowsLogprob.apply(logits, target, vocab_start, vocab_end)


def rows_logprob_seq_chunked(logits, target, chunk_size, vocab_start=0, vocab_end=None):
    """``ChunkedDistributedLogprob`` (``model_utils.py:294-323``): the same maths
    in ``chunk_size``-token slices of dim 1, concatenated."""
    seq = logits.shape[1]
    parts = [
        rows_logprob(
            logits[:, lo : lo + chunk_size], target[:, lo : lo + chunk_size], vocab_start, vocab_end
        )
        for lo in range(0, seq, chunk_size)
    ]
    return torch.cat(parts, dim=1)


def rows_logprob_sampled(logits, target, top_k, top_p):
    """``DistributedLogprobWithSampling.forward`` on one rank
    (``model_utils.py:439-452``): filter, fp32 ``log_softmax``, gather.  A target
    outside the kept set yields ``-inf``.  The filter runs in the dtype it is
    given (``:440`` passes the caller's tensor, fp32 on the training path
    because of ``:1648-1649``)."""
    filtered, _ = sampling.apply_top_k_top_p(logits, top_k, top_p)
    logp = torch.log_softmax(filtered.to(torch.float32), dim=-1)
    return torch.gather(logp, -1, target.unsqueeze(-1)).squeeze(-1)


def from_logits_to_logprobs(
    logits: torch.Tensor,
    target: torch.Tensor,
    vocab_start: int = 0,
    vocab_end: Optional[int] = None,
    chunk_size: Optional[int] = None,
    top_k=None,
    top_p: float = 1.0,
) -> torch.Tensor:
    """``from_parallel_logits_to_logprobs`` (``model_utils.py:979-1042``) with
    TP = CP = 1: roll the unshifted ``target [B,S]`` by -1, right-pad it with 0
    when the logits are longer, compute every position, drop the pad and the
    last column -> ``[B, S-1]``."""
    tgt = target.roll(shifts=-1, dims=-1)
    pad = logits.shape[1] - tgt.shape[1]
    if pad > 0:
        tgt = torch.nn.functional.pad(tgt, (0, pad), value=0)
    if sampling.wants_filtering(top_k, top_p):
        out = rows_logprob_sampled(logits, tgt, top_k, top_p)
    elif chunk_size is not None:
        out = rows_logprob_seq_chunked(logits, tgt, chunk_size, vocab_start, vocab_end)
    else:
        out = rows_logprob(logits, tgt, vocab_start, vocab_end)
    if pad > 0:
        out = out[:, :-pad]
    return out[:, :-1]


def next_token_logprobs(input_ids, logits, top_k=None, top_p: float = 1.0):
    """Plain-tensor branch of ``get_next_token_logprobs_from_logits``
    (``model_utils.py:1648-1649, 1677-1693``): fp32 cast, drop the last position,
    filter, ``log_softmax``, gather ``input_ids[:, 1:]``."""
    x = logits.to(torch.float32)[:, :-1]
    x, _ = sampling.apply_top_k_top_p(x, top_k, top_p)
    logp = torch.log_softmax(x, dim=-1)
    return torch.gather(logp, -1, input_ids[:, 1:].unsqueeze(-1)).squeeze(-1)


def pack_input_ids(input_ids, cu_seqlens, cu_seqlens_padded, roll_shift=0):
    """``_pack_input_ids`` (``nemo_rl/algorithms/loss/utils.py:239-261``), CP = 1:
    each sequence is copied (``min(actual_len, S)`` tokens, zero tail) into a
    buffer of its padded length, rolled by ``roll_shift`` inside that span and
    placed at ``cu_seqlens_padded[i]`` -> ``[1, T]``."""
    cu = [int(v) for v in cu_seqlens.tolist()]
    cup = [int(v) for v in cu_seqlens_padded.tolist()]
    packed = torch.zeros(cup[-1], dtype=input_ids.dtype)
    for i in range(input_ids.shape[0]):
        span = cup[i + 1] - cup[i]
        seq = torch.zeros(span, dtype=input_ids.dtype)
        n = min(cu[i + 1] - cu[i], input_ids.shape[1])
        seq[:n] = input_ids[i, :n]
        if roll_shift:
            seq = seq.roll(roll_shift)
        packed[cup[i] : cup[i + 1]] = seq
    return packed.unsqueeze(0)


def packed_logits_to_logprobs(
    logits,
    target,
    cu_seqlens_padded,
    unpacked_seqlen: int,
    vocab_start: int = 0,
    vocab_end: Optional[int] = None,
    chunk_size: Optional[int] = None,
    top_k=None,
    top_p: float = 1.0,
    target_is_pre_rolled: bool = False,
):
    """``from_parallel_logits_to_logprobs_packed_sequences``
    (``model_utils.py:1085-1196``), CP = 1.  ``logits [1,T,V]``; ``target [1,T]``.
    Unless pre-rolled, targets are rolled by -1 inside each sequence's span
    (``:1098-1108``).  The result is unpacked to ``[B, unpacked_seqlen-1]``,
    dropping every sequence's last position and zero-filling (``:1176-1194``)."""
    cup = [int(v) for v in cu_seqlens_padded.tolist()]
    nseq = len(cup) - 1
    tgt = target
    if not target_is_pre_rolled:
        flat = target.squeeze(0)
        rolled = torch.zeros_like(flat)
        for i in range(nseq):
            rolled[cup[i] : cup[i + 1]] = flat[cup[i] : cup[i + 1]].roll(-1)
        tgt = rolled.unsqueeze(0)
    if sampling.wants_filtering(top_k, top_p):
        flat_lp = rows_logprob_sampled(logits, tgt, top_k, top_p)
    elif chunk_size is not None:
        flat_lp = rows_logprob_seq_chunked(logits, tgt, chunk_size, vocab_start, vocab_end)
    else:
        flat_lp = rows_logprob(logits, tgt, vocab_start, vocab_end)
    flat_lp = flat_lp.squeeze(0)
    out = torch.zeros((nseq, unpacked_seqlen - 1), dtype=flat_lp.dtype, device=flat_lp.device)
    rows = []
    for i in range(nseq):
        n = min(max(cup[i + 1] - cup[i] - 1, 0), unpacked_seqlen - 1)
        row = torch.zeros(unpacked_seqlen - 1, dtype=flat_lp.dtype, device=flat_lp.device)
        if n > 0:
            row = torch.cat([flat_lp[cup[i] : cup[i] + n], row[n:]])
        rows.append(row)
    if rows:
        out = torch.stack(rows)
    return out


def mask_out_neg_inf_logprobs(logprobs, mask):
    """``nemo_rl/algorithms/utils.py:246-257`` without the warning print:
    positions that are masked out or hold +-inf become 0."""
    keep = mask * (~torch.isinf(logprobs)).float()
    return torch.where(keep.bool(), logprobs, 0.0)


def logprobs_post_process(logits, input_ids, input_lengths, cu_seqlens=None, original_batch_size=None,
                          original_seq_len=None, top_k=None, top_p: float = 1.0):
    """``LogprobsPostProcessor.__call__`` without TP / CP (``models/automodel/train.py:689-806``):
    fp32 log-softmax + gather of the next token (``_compute_local_logprobs`` ``:808-864``), a zero
    prepended for the first token (``:759-762``), then either the per-sequence unpack of a packed row
    (``:764-778``) or the right-padding mask from ``input_lengths`` (``:779-791``).  Pinned by the
    textbook identity it is written in (``log_softmax`` + ``gather``) and by brute force on tiny
    inputs in ``tests/test_oracle_logprob.py``."""
    nxt = input_ids[:, 1:]
    x = logits[:, : nxt.shape[1]].to(torch.float32)
    if top_k is not None or top_p < 1.0:
        x, _ = sampling.apply_top_k_top_p(x, top_k, top_p)
    lp = torch.log_softmax(x, dim=-1).gather(-1, nxt.unsqueeze(-1)).squeeze(-1)
    lp = torch.cat([torch.zeros_like(lp[:, :1]), lp], dim=1)
    if cu_seqlens is not None:
        out = torch.zeros(original_batch_size, original_seq_len, dtype=lp.dtype, device=lp.device)
        for i in range(original_batch_size):
            start, end = int(cu_seqlens[i]) + 1, int(cu_seqlens[i + 1])
            out[i, 1 : int(input_lengths[i])] = lp[0, start:end]
        return out
    mask = torch.arange(lp.shape[1], device=lp.device)[None, :] < torch.as_tensor(input_lengths, device=lp.device).reshape(-1, 1)
    return lp * mask
