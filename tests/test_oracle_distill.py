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


# ---- top-k distillation loss (oracle pins) ----
def _kd_case(b=2, s=6, v=40, k=8, seed=0):
    g = torch.Generator().manual_seed(seed)
    student = torch.randn(b, s, v, generator=g) * 2
    teacher_full = torch.randn(b, s, v, generator=g) * 2
    t_logits, t_idx = torch.topk(teacher_full, k, dim=-1)
    return student, teacher_full, t_logits, t_idx


def test_topk_logprobs_are_the_textbook_pieces():
    from oracle import distill as D

    student, _full, t_logits, t_idx = _kd_case()
    s_lp, t_lp, h = D.distillation_topk_logprobs(student, t_logits, t_idx, zero_outside_topk=True, calculate_entropy=True)
    full = torch.log_softmax(student, -1)
    assert torch.equal(s_lp, full.gather(-1, t_idx)[:, :-1])
    assert torch.allclose(h, -torch.distributions.Categorical(logits=student).entropy()[:, :-1], atol=1e-5)
    assert torch.allclose(t_lp.exp().sum(-1), torch.ones(2, 5), atol=1e-6)
    s_lp2, _, h2 = D.distillation_topk_logprobs(student, t_logits, t_idx, zero_outside_topk=False, calculate_entropy=False)
    assert h2 is None and torch.allclose(s_lp2.exp().sum(-1), torch.ones(2, 5), atol=1e-6)
    # renormalising the full-vocabulary entries over the top-k gives the restricted softmax
    assert torch.allclose(s_lp2, s_lp - torch.logsumexp(s_lp, -1, keepdim=True), atol=1e-5)


def test_distillation_loss_closed_forms():
    from oracle import distill as D

    student, _full, t_logits, t_idx = _kd_case(seed=1)
    data = {"input_ids": torch.zeros(2, 6, dtype=torch.long)}
    # the same distribution on both sides: every KL is zero
    s_lp, _t, _h = D.distillation_topk_logprobs(student, t_logits, t_idx, False, False)
    for kl in ("forward", "reverse", "mixed"):
        loss, m = D.distillation_loss(kl, 0.3, False, s_lp, s_lp.clone(), None, data, None)
        assert abs(loss.item()) < 1e-7 and m["num_valid_samples"] == 2
    # top-k spanning the whole vocabulary: nothing is outside, the correction vanishes and the reverse KL
    # is the textbook KL(student || teacher)
    v = student.shape[-1]
    idx_all = torch.arange(v).expand(2, 6, v).contiguous()
    teacher_logits = torch.randn(2, 6, v, generator=torch.Generator().manual_seed(5))
    s_lp, t_lp, h = D.distillation_topk_logprobs(student, teacher_logits, idx_all, True, True)
    loss, _ = D.distillation_loss("reverse", 0.5, True, s_lp, t_lp, h, data, None)
    want = torch.nn.functional.kl_div(t_lp, s_lp, log_target=True, reduction="none").sum(-1).mean()
    assert abs(loss.item() - want.item()) < 1e-5
    loss_f, _ = D.distillation_loss("forward", 0.5, True, s_lp, t_lp, h, data, None)
    want_f = torch.nn.functional.kl_div(s_lp, t_lp, log_target=True, reduction="none").sum(-1).mean()
    assert abs(loss_f.item() - want_f.item()) < 1e-5
    loss_m, _ = D.distillation_loss("mixed", 0.25, True, s_lp, t_lp, h, data, None)
    assert abs(loss_m.item() - (0.25 * want_f.item() + 0.75 * want.item())) < 1e-5


def test_distillation_loss_brute_force_with_masks_and_correction():
    import math

    from oracle import distill as D

    student, _full, t_logits, t_idx = _kd_case(b=3, s=5, v=30, k=4, seed=2)
    s_lp, t_lp, h = D.distillation_topk_logprobs(student, t_logits, t_idx, True, True)
    tm = torch.tensor([[0, 1, 1, 0, 1], [0, 0, 1, 1, 1], [0, 1, 1, 1, 1]])
    sm = torch.tensor([1.0, 0.0, 0.5])
    data = {"input_ids": torch.zeros(3, 5, dtype=torch.long), "token_mask": tm, "sample_mask": sm}
    gt = torch.tensor(7.0)
    w = 0.4
    loss, _ = D.distillation_loss("mixed", w, True, s_lp, t_lp, h, data, gt)
    tot = 0.0
    for b in range(3):
        for t in range(4):
            m = tm[b, t + 1].item() * sm[b].item()
            f = r = ssum = sslp = 0.0
            for j in range(4):
                s, u = s_lp[b, t, j].item(), t_lp[b, t, j].item()
                f += math.exp(u) * (u - s)
                r += math.exp(s) * (s - u)
                ssum += math.exp(s)
                sslp += math.exp(s) * s
            corr = (h[b, t].item() - sslp) + 100.0 * (1.0 - ssum)
            tot += (w * f + (1 - w) * r + (1 - w) * corr) * m
    assert abs(loss.item() - tot / (7.0 + 1e-8)) <= 1e-5 * abs(tot / 7.0) + 1e-6
