"""Oracle: fused lm_head -> token log-probabilities (hidden states in, no
materialised full-sequence logits).

Test infrastructure only (see ``oracle/__init__.py``).  Pinned by the identity the
path reduces to: forward == ``log_softmax(hidden @ W.T).gather(target)`` and
backward == torch autograd of that unfused form, chunked == unchunked
(``tests/test_oracle_logprob.py::test_lmhead_equals_unfused_and_autograd``).  The
reference holds no vectors for this path (its only test needs Megatron, two GPUs
and a model download); PARITY UNPINNED only for the rounding of the reference's
dW, which it accumulates per chunk in the weights' dtype.

Restates ``nemo_rl/distributed/model_utils.py:2119-2134`` (roll, drop last
column) and ``:2152-2215, 2240-2291`` (forward / backward per sequence chunk)
for TP = 1.  The reference multiplies in the weights' dtype and softmaxes in
fp32; its dW accumulates chunk contributions in the weights' dtype
(``:2248, 2284-2286``).  This oracle accumulates dW in fp32 (one rounding at
the end) unless ``accumulate_in_weight_dtype`` is set.
"""

from __future__ import annotations

from typing import Optional

import torch

from .logprob import stable_log_softmax


def hidden_to_logprobs_rows(hidden_sbh, weight_vh, target_bs, chunk_size: Optional[int] = None):
    """Forward, ``model_utils.py:2170-2197``.  ``hidden [S,B,H]`` (sequence
    first), ``weight [V,H]``, ``target [B,S]`` already shifted -> ``[B,S]`` fp32."""
    seq = hidden_sbh.shape[0]
    step = seq if chunk_size is None else chunk_size
    parts = []
    for lo in range(0, seq, step):
        logits = torch.matmul(hidden_sbh[lo : lo + step], weight_vh.T)
        logits = logits.to(torch.float32).transpose(0, 1).contiguous()
        logp = stable_log_softmax(logits)
        parts.append(torch.gather(logp, -1, target_bs[:, lo : lo + step].unsqueeze(-1)).squeeze(-1))
    return torch.cat(parts, dim=1)


def hidden_to_logprobs(hidden_sbh, weight_vh, target_bs, chunk_size: Optional[int] = None):
    """``from_parallel_hidden_states_to_logprobs`` (``:2119-2134``): roll the
    unshifted target by -1, compute, drop the last column -> ``[B, S-1]``."""
    rolled = target_bs.roll(shifts=-1, dims=-1)
    return hidden_to_logprobs_rows(hidden_sbh, weight_vh, rolled, chunk_size)[:, :-1]


def hidden_to_logprobs_backward(
    hidden_sbh,
    weight_vh,
    target_bs,
    grad_bs,
    chunk_size: Optional[int] = None,
    accumulate_in_weight_dtype: bool = False,
):
    """Backward, ``model_utils.py:2249-2291``: per chunk recompute logits and
    softmax, ``G = g * (onehot - softmax)`` (fp32), ``dH = G @ W.float()`` (fp32,
    returned ``[S,B,H]``), ``dW += (hidden^T G)^T``."""
    seq, _, width = hidden_sbh.shape
    vocab = weight_vh.shape[0]
    step = seq if chunk_size is None else chunk_size
    d_w = torch.zeros(
        vocab, width, dtype=weight_vh.dtype if accumulate_in_weight_dtype else torch.float32, device=weight_vh.device
    )
    d_h_parts = []
    for lo in range(0, seq, step):
        h = hidden_sbh[lo : lo + step]
        logits = torch.matmul(h, weight_vh.T).to(torch.float32).transpose(0, 1).contiguous()
        p = stable_log_softmax(logits).exp()
        onehot = torch.nn.functional.one_hot(target_bs[:, lo : lo + step], num_classes=vocab)
        g = (onehot.float() - p) * grad_bs[:, lo : lo + step].unsqueeze(-1)
        d_h_parts.append(torch.matmul(g, weight_vh.to(torch.float32)))
        contrib = torch.einsum("bsd,bsv->dv", h.transpose(0, 1).contiguous().float(), g)
        d_w.add_(contrib.transpose(0, 1).contiguous().to(d_w.dtype))
    d_h = torch.cat(d_h_parts, dim=1).transpose(0, 1).contiguous()
    return d_h, d_w.to(weight_vh.dtype)
