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


def distillation_topk_logprobs(student_logits, teacher_topk_logits, teacher_topk_indices, zero_outside_topk: bool,
                               calculate_entropy: bool):
    """Non-distributed branch of ``get_distillation_topk_logprobs_from_logits``
    (``model_utils.py:1856-2020``): fp32 student logits; with ``zero_outside_topk`` the student's entries come
    from the full log-softmax (``:1973-1979``), otherwise from a softmax over the K gathered logits
    (``:1999-2005``); the teacher's from a softmax over its K logits (``:2010``); everything cut to ``[:, :-1]``."""
    if teacher_topk_indices.shape[-1] <= 0:
        raise ValueError("topk must be positive")
    x = student_logits.to(torch.float32)
    h_all = None
    if zero_outside_topk:
        lp = torch.log_softmax(x, dim=-1)
        s = lp.gather(dim=-1, index=teacher_topk_indices)
        if calculate_entropy:
            h_all = (lp.exp() * lp).sum(-1)
    else:
        s = torch.log_softmax(x.gather(dim=-1, index=teacher_topk_indices), dim=-1)
    t = torch.log_softmax(teacher_topk_logits.to(s.dtype), dim=-1)
    return s[:, :-1, :], t[:, :-1, :], (h_all[:, :-1] if h_all is not None else None)


def distillation_loss(kl_type: str, mixed_kl_weight: float, zero_outside_topk: bool, student_topk_logprobs,
                      teacher_topk_logprobs, h_all, data, global_valid_toks, log_infinitesimal: float = -100):
    """``DistillationLossFn.__call__`` (``loss_functions.py:1141-1206``)."""
    sp, tp = student_topk_logprobs.exp(), teacher_topk_logprobs.exp()
    correction = torch.zeros_like(sp[..., 0])
    if zero_outside_topk and kl_type != "forward":
        h_rest = h_all - (sp * student_topk_logprobs).sum(-1)
        p_rest = 1 - sp.sum(-1)
        correction = h_rest - log_infinitesimal * p_rest
        if kl_type == "mixed":
            correction = correction * (1.0 - mixed_kl_weight)
    fwd = tp * (teacher_topk_logprobs - student_topk_logprobs)
    rev = sp * (student_topk_logprobs - teacher_topk_logprobs)
    per = fwd if kl_type == "forward" else rev if kl_type == "reverse" else mixed_kl_weight * fwd + (1.0 - mixed_kl_weight) * rev
    per = per.sum(-1) + correction
    if "token_mask" in data and "sample_mask" in data:
        mask = data["token_mask"][:, 1:][:, : per.shape[1]] * data["sample_mask"].unsqueeze(-1)
        loss = (per * mask).sum() / (global_valid_toks + 1e-8)
    else:
        loss = per.mean()
    return loss, {"loss": float(loss.item()), "num_valid_samples": data["input_ids"].shape[0]}
