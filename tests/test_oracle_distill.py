"""Pins for the distillation oracle: closed forms, the reference's stated backward formulas, brute force."""

import math

import torch

from oracle import distill as D


def test_neg_entropy_closed_forms_and_backward_formula():
    # uniform logits: sum p log p = -log V
    assert torch.allclose(D.neg_entropy(torch.zeros(2, 3, 64)), torch.full((2, 3), -math.log(64.0)), atol=1e-6)
    # a one-hot-like distribution has entropy -> 0
    x = torch.zeros(1, 1, 8)
    x[..., 3] = 50.0
    assert abs(D.neg_entropy(x).item()) < 1e-6
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 4, 37, generator=g, requires_grad=True)
    up = torch.randn(2, 4, generator=g)
    h = D.neg_entropy(x)
    (h * up).sum().backward()
    lp = torch.log_softmax(x.detach(), -1)
    want = lp.exp() * (lp - h.detach().unsqueeze(-1)) * up.unsqueeze(-1)  # model_utils.py:2092-2096
    assert torch.allclose(x.grad, want, atol=1e-6)


def test_gather_logprob_brute_force_and_backward_formula():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 3, 11, generator=g, requires_grad=True)
    idx = torch.randint(0, 11, (2, 3, 4), generator=g)
    idx[0, 0] = torch.tensor([5, 5, 2, 5])  # duplicates accumulate in the backward
    out = D.gather_logprob(x, idx)
    for b in range(2):
        for s in range(3):
            row = x[b, s].tolist()
            lse = math.log(sum(math.exp(v) for v in row))
            for k in range(4):
                assert abs(out[b, s, k].item() - (row[int(idx[b, s, k])] - lse)) < 1e-5
    up = torch.randn(2, 3, 4, generator=g)
    (out * up).sum().backward()
    p = torch.softmax(x.detach(), -1)
    want = -p * up.sum(-1, keepdim=True)
    want.scatter_add_(2, idx, up)  # model_utils.py:812-818
    assert torch.allclose(x.grad, want, atol=1e-6)
    # a vocabulary shard: ids outside [start, end) read as 0
    shard = D.gather_logprob(x.detach()[..., 4:9], idx, vocab_start=4, vocab_end=9)
    assert bool((shard[(idx < 4) | (idx >= 9)] == 0).all())


def test_soft_cross_entropy_identities():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 5, 29, generator=g, requires_grad=True)
    y = torch.randn(3, 5, 29, generator=g)
    ce = D.soft_cross_entropy(x, y)
    # H(p, q) = H(p) + KL(p || q)
    p, lp, lq = torch.softmax(y, -1), torch.log_softmax(y, -1), torch.log_softmax(x.detach(), -1)
    assert torch.allclose(ce, -(p * lp).sum(-1) + (p * (lp - lq)).sum(-1), atol=1e-5)
    # a one-hot teacher reduces it to the ordinary cross entropy
    hard = torch.full((1, 1, 29), -1e4)
    hard[..., 7] = 0.0
    assert torch.allclose(D.soft_cross_entropy(x.detach()[:1, :1], hard),
                          torch.nn.functional.cross_entropy(x.detach()[0, :1], torch.tensor([7])).reshape(1, 1), atol=1e-5)
    up = torch.randn(3, 5, generator=g)
    (ce * up).sum().backward()
    assert torch.allclose(x.grad, (torch.softmax(x.detach(), -1) - p) * up.unsqueeze(-1), atol=1e-6)  # model_utils.py:261-263
