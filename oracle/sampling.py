"""Oracle: top-k / top-p (nucleus) filtering of logits rows.

Test infrastructure only (see ``oracle/__init__.py``).

Follows ``nemo_rl/algorithms/logits_sampling_utils.py:47-66`` (predicates),
``:69-108`` (top-k only), ``:111-210`` (top-k + top-p through an ascending
sort) and ``:213-285`` (gradient = upstream gradient where kept, else zero).
"""

from __future__ import annotations

import torch

NEG_INF = float("-inf")


def wants_top_k(top_k) -> bool:
    # logits_sampling_utils.py:47-49
    return top_k is not None and top_k > 0


def wants_top_p(top_p) -> bool:
    # logits_sampling_utils.py:52-54
    return top_p is not None and top_p != 1.0


def wants_filtering(top_k, top_p) -> bool:
    # logits_sampling_utils.py:57-66
    return wants_top_k(top_k) or wants_top_p(top_p)


def keep_mask_rows(rows: torch.Tensor, top_k, top_p) -> torch.Tensor | None:
    """Boolean keep mask for a 2-D ``[n, V]`` tensor (no gradient).

    top-k only (``:96-100``): keep ``x >= k-th largest`` (ties kept).
    with top-p (``:169-200``): ascending sort; top-k threshold is the value at
    sorted index ``V - k`` with ``>=``; softmax of the top-k-masked sorted row;
    inclusive ascending cumsum; keep where ``cumsum > 1 - top_p``; the largest
    element is always kept; masks are scattered back to vocabulary order.
    """
    if not wants_filtering(top_k, top_p):
        return None
    rows = rows.detach()
    n, vocab = rows.shape
    if not wants_top_p(top_p):
        kth = torch.topk(rows, top_k, dim=-1).values[:, -1:]
        return rows >= kth

    ordered, order = torch.sort(rows, dim=-1, descending=False, stable=True)
    keep_sorted = torch.ones_like(ordered, dtype=torch.bool)
    if wants_top_k(top_k):
        thr = ordered[:, vocab - top_k].unsqueeze(-1)
        keep_sorted = ordered >= thr
        ordered = ordered.masked_fill(~keep_sorted, NEG_INF)
    mass = torch.cumsum(torch.softmax(ordered, dim=-1), dim=-1)
    nucleus = mass > (1 - top_p)
    nucleus[:, -1] = True
    keep_sorted = keep_sorted & nucleus
    keep = torch.empty_like(keep_sorted)
    keep.scatter_(-1, order, keep_sorted)
    return keep


class _MaskedLogits(torch.autograd.Function):
    # logits_sampling_utils.py:213-251: forward fills -inf where not kept,
    # backward zeroes the gradient there.
    @staticmethod
    def forward(ctx, logits, keep):
        ctx.save_for_backward(keep)
        return logits.masked_fill(~keep, NEG_INF)

    @staticmethod
    def backward(ctx, grad):
        (keep,) = ctx.saved_tensors
        return grad.masked_fill(~keep, 0.0), None


def apply_top_k_top_p(logits: torch.Tensor, top_k, top_p, chunk_size=256):
    """Filtered logits (``-inf`` outside the kept set) and the keep mask.

    ``chunk_size`` only bounds the reference's working set
    (``logits_sampling_utils.py:164-204``); rows are independent, so the result
    does not depend on it and the oracle ignores it.
    """
    if not wants_filtering(top_k, top_p):
        return logits, None
    shape = logits.shape
    keep = keep_mask_rows(logits.reshape(-1, shape[-1]), top_k, top_p).reshape(shape)
    return _MaskedLogits.apply(logits, keep), keep
