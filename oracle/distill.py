"""CPU restatement of the distillation reductions of ``nemo_rl/distributed/model_utils.py`` at TP = 1.

TEST INFRASTRUCTURE ONLY: imported by ``tests/`` (and nothing else); the product never falls back to it.
Each function is the forward of the reference class in plain fp32 PyTorch, differentiated by stock
autograd; the reference's hand-written backward formulas (cited) are what stock autograd yields for these
expressions, which ``tests/test_oracle_distill.py`` checks against the closed forms.
"""

from __future__ import annotations

import torch


def neg_entropy(logits: torch.Tensor) -> torch.Tensor:
    """``ChunkedDistributedEntropy.forward`` (``model_utils.py:2030-2060``): ``sum_v p_v log p_v``
    per row, fp32.  Backward in the reference (``:2062-2103``): ``softmax * (log_probs - H)``."""
    lp = torch.log_softmax(logits.to(torch.float32), dim=-1)
    return (lp.exp() * lp).sum(-1)


def gather_logprob(logits: torch.Tensor, indices: torch.Tensor, vocab_start: int = 0, vocab_end=None) -> torch.Tensor:
    """``ChunkedDistributedGatherLogprob.forward`` (``model_utils.py:733-778``): log-softmax gathered at
    ``indices [B, S, K]`` (global ids; positions outside ``[vocab_start, vocab_end)`` give 0).
    Backward in the reference (``:780-836``): ``-softmax * sum_k g_k + scatter_add(g_k)``."""
    v = logits.shape[-1]
    vocab_end = vocab_start + v if vocab_end is None else vocab_end
    lp = torch.log_softmax(logits.to(torch.float32), dim=-1)
    in_range = (indices >= vocab_start) & (indices < vocab_end)
    li = (indices - vocab_start).clamp(min=0, max=v - 1)
    return torch.gather(lp, -1, li) * in_range.to(lp.dtype)


def soft_cross_entropy(student_logits: torch.Tensor, target_logits: torch.Tensor) -> torch.Tensor:
    """``DistributedCrossEntropy.forward`` (``model_utils.py:216-250``):
    ``-sum_v softmax(target)_v * log_softmax(student)_v``; the target is a constant
    (backward ``:252-264``: ``(q - p) * g`` to the student only)."""
    p = torch.softmax(target_logits.detach().to(torch.float32), dim=-1)
    lq = torch.log_softmax(student_logits.to(torch.float32), dim=-1)
    return -(p * lq).sum(-1)
