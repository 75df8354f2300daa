"""GPU parity of the DPO / preference / per-sample NLL kernels against the CPU oracle.  Tolerance:
loss, metrics and gradients 1e-4 relative (stated per assertion)."""

import math

import pytest
import torch

from oracle import logprob as OL
from oracle import preference as P
from rl_amd.algorithms.loss import (
    DPOLossConfig,
    DPOLossFn,
    NLLLossFn,
    PreferenceLossFn,
    prepare_loss_input,
)

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _close(a, b, rel=1e-4, abs_=1e-6):
    return abs(float(a) - float(b)) <= rel * abs(float(b)) + abs_


def _case(b, s, seed, float_masks=True):
    g = torch.Generator().manual_seed(seed)
    lp = -torch.rand((b, s - 1), generator=g) * 4
    ref = -torch.rand((b, s), generator=g) * 4
    tm = (torch.rand((b, s), generator=g) < 0.7)
    tm[:, 0] = False
    if b > 4:
        tm[4] = False
    sm = torch.ones(b)
    if float_masks:
        sm[2:4] = 0.5
    if b > 6:
        sm[6:8] = 0
    if float_masks:
        tm, sm = tm.float(), sm
    else:
        tm, sm = tm.long(), sm.long()
    return lp, {"token_mask": tm, "sample_mask": sm, "reference_policy_logprobs": ref}


CONFIGS = [
    dict(),
    dict(reference_policy_kl_penalty=0.3, preference_loss_weight=0.7, sft_loss_weight=0.2),
    dict(reference_policy_kl_penalty=0.1, sft_loss_weight=0.5, preference_average_log_probs=True, sft_average_log_probs=True),
    dict(reference_policy_kl_penalty=0.0, preference_loss_weight=0.0, sft_loss_weight=1.0),
    dict(reference_policy_kl_penalty=2.0, preference_average_log_probs=True),
]


@pytest.mark.parametrize("cfg", CONFIGS, ids=[str(i) for i in range(len(CONFIGS))])
@pytest.mark.parametrize("b,s,float_masks", [(8, 33, True), (2, 5, False), (64, 700, True)])
def test_dpo_matches_oracle(cfg, b, s, float_masks):
    lp, data = _case(b, s, seed=b * 7 + s, float_masks=float_masks)
    gs = torch.tensor(float(b) - 1.0)
    xo = lp.clone().requires_grad_(True)
    want, wm = P.dpo_loss(P.DPOConfig(**cfg), xo, data, gs)
    want.backward()
    fn = DPOLossFn(DPOLossConfig(**cfg))
    xg = lp.to(DEV).requires_grad_(True)
    got, gm = fn(next_token_logprobs=xg, data={k: v.to(DEV) for k, v in data.items()}, global_valid_seqs=gs.to(DEV),
                 global_valid_toks=torch.tensor(1.0))
    got.backward()
    assert _close(got.item(), want.item()), (got.item(), want.item())
    assert set(gm) == set(wm)
    for k in wm:
        assert _close(gm[k], wm[k]), (k, gm[k], wm[k])
    scale = xo.grad.abs().max().item() + 1e-30
    assert (xg.grad.cpu() - xo.grad).abs().max().item() <= 1e-4 * scale
    assert torch.all(xg.grad.cpu()[data["token_mask"][:, 1:] == 0] == 0)


def test_dpo_reference_closed_forms_through_the_logit_path():
    """The reference's own expectations (``test_loss_functions.py:133-201``) through
    ``prepare_loss_input`` + ``DPOLossFn`` on the GPU."""
    data = {
        "input_ids": torch.arange(8).reshape(2, 4).to(torch.int64).to(DEV),
        "token_mask": torch.tensor([[0, 0, 1, 1], [0, 0, 1, 1]]).to(DEV),
        "sample_mask": torch.tensor([1, 1]).to(DEV),
        "reference_policy_logprobs": torch.zeros((2, 4)).to(DEV),
    }
    logits = torch.zeros((2, 4, 16), device=DEV)
    gs = torch.sum(data["sample_mask"])
    gt = torch.sum(data["token_mask"] * data["sample_mask"].unsqueeze(-1))
    fn = DPOLossFn(DPOLossConfig(reference_policy_kl_penalty=0.0))
    loss_input, d2 = prepare_loss_input(logits, data, fn)
    loss, _ = fn(data=d2, global_valid_seqs=gs, global_valid_toks=gt, **loss_input)
    assert math.isclose(loss.item(), math.log(2.0), rel_tol=1e-6)
    fn = DPOLossFn(DPOLossConfig(reference_policy_kl_penalty=0.0, sft_loss_weight=0.5))
    loss_input, d2 = prepare_loss_input(logits, data, fn)
    loss, m = fn(data=d2, global_valid_seqs=gs, global_valid_toks=gt, **loss_input)
    assert math.isclose(loss.item(), 0.5 * 2 * math.log(16.0) + math.log(2.0), rel_tol=1e-6)
    assert math.isclose(m["sft_loss"], 2 * math.log(16.0), rel_tol=1e-6)


def test_dpo_end_to_end_gradient_reaches_the_logits():
    g = torch.Generator().manual_seed(17)
    b, s, v = 6, 12, 300
    logits = torch.randn((b, s, v), generator=g) * 2
    ids = torch.randint(0, v, (b, s), generator=g)
    _, data = _case(b, s, seed=5)
    data["input_ids"] = ids
    cfg = dict(reference_policy_kl_penalty=0.2, sft_loss_weight=0.3)
    gs = torch.tensor(float(b))
    xo = logits.clone().requires_grad_(True)
    want, _ = P.dpo_loss(P.DPOConfig(**cfg), OL.next_token_logprobs(ids, xo), data, gs)
    want.backward()
    fn = DPOLossFn(DPOLossConfig(**cfg))
    xg = logits.to(DEV).requires_grad_(True)
    loss_input, d2 = prepare_loss_input(xg, {k: t.to(DEV) for k, t in data.items()}, fn)
    got, _ = fn(data=d2, global_valid_seqs=gs.to(DEV), global_valid_toks=torch.tensor(1.0), **loss_input)
    got.backward()
    assert _close(got.item(), want.item())
    scale = xo.grad.abs().max().item()
    assert (xg.grad.cpu() - xo.grad).abs().max().item() <= 1e-4 * scale


def test_dpo_rejects_an_odd_batch():
    lp, data = _case(3, 6, seed=1)
    fn = DPOLossFn(DPOLossConfig())
    with pytest.raises((ValueError, RuntimeError)):
        fn(next_token_logprobs=lp.to(DEV), data={k: v.to(DEV) for k, v in data.items()},
           global_valid_seqs=torch.tensor(3.0), global_valid_toks=None)


@pytest.mark.parametrize("b", [2, 10, 600])
def test_reward_model_preference_loss(b):
    g = torch.Generator().manual_seed(b)
    rewards = torch.randn((b, 1), generator=g) * 3
    sm = (torch.rand(b, generator=g) < 0.8).float()
    sm[:2] = 0.5
    gs = torch.tensor(float(b) - 0.5)
    xo = rewards.clone().requires_grad_(True)
    want, wm = P.preference_loss(xo, {"sample_mask": sm}, gs)
    want.backward()
    xg = rewards.to(DEV).requires_grad_(True)
    got, gm = PreferenceLossFn()(xg, {"sample_mask": sm.to(DEV)}, gs.to(DEV), None)
    got.backward()
    assert _close(got.item(), want.item())
    assert set(gm) == set(wm)
    for k in wm:
        assert _close(gm[k], wm[k]), (k, gm[k], wm[k])
    assert (xg.grad.cpu() - xo.grad).abs().max().item() <= 1e-4 * (xo.grad.abs().max().item() + 1e-30)


@pytest.mark.parametrize("average", [False, True])
def test_per_sample_nll_rows(average):
    lp, data = _case(8, 40, seed=9)
    xo = lp.clone().requires_grad_(True)
    want, wm = P.nll_loss_rows(xo, data, average)
    up = torch.arange(1.0, 9.0)
    (want * up).sum().backward()
    xg = lp.to(DEV).requires_grad_(True)
    got, gm = NLLLossFn()(xg, {k: v.to(DEV) for k, v in data.items()}, None, torch.tensor(1.0), dpo_loss=True,
                          dpo_average_log_probs=average)
    (got * up.to(DEV)).sum().backward()
    torch.testing.assert_close(got.detach().cpu(), want.detach(), rtol=1e-5, atol=1e-6)
    assert gm["loss"] is got
    assert _close(gm["num_unmasked_tokens"], wm["num_unmasked_tokens"]) and _close(gm["num_valid_samples"], wm["num_valid_samples"])
    torch.testing.assert_close(xg.grad.cpu(), xo.grad, rtol=1e-5, atol=1e-7)
