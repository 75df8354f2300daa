"""Pins for ``oracle/preference.py``: the expectations of the reference's own DPO tests
(``tests/unit/algorithms/test_loss_functions.py:133-370``), restated as closed forms on the CPU, and a
loop-per-pair brute force."""

import math

import pytest
import torch

from oracle import logprob as OL
from oracle import loss as O
from oracle import preference as P


def _zero_case():
    """``setup_dpo_loss_test_data`` (``test_loss_functions.py:46-59``), vocab 16, one pair."""
    data = {
        "input_ids": torch.arange(8).reshape(2, 4).to(torch.int64),
        "token_mask": torch.tensor([[0, 0, 1, 1], [0, 0, 1, 1]]),
        "sample_mask": torch.tensor([1, 1]),
        "reference_policy_logprobs": torch.zeros((2, 4)),
    }
    return data, torch.zeros((2, 4, 16))


def test_equal_rewards_give_log_two():
    data, logits = _zero_case()
    lp = OL.next_token_logprobs(data["input_ids"], logits)
    gs = data["sample_mask"].sum()
    loss, m = P.dpo_loss(P.DPOConfig(reference_policy_kl_penalty=0.0), lp, data, gs)
    assert math.isclose(loss.item(), math.log(2.0), rel_tol=1e-6)
    assert m["accuracy"] == 0.0 and m["num_valid_samples"] == 1.0
    # with the SFT term: 0.5 * (two unmasked tokens at log 16 each) + log 2
    loss, m = P.dpo_loss(P.DPOConfig(reference_policy_kl_penalty=0.0, sft_loss_weight=0.5), lp, data, gs)
    assert math.isclose(loss.item(), 0.5 * 2 * math.log(16.0) + math.log(2.0), rel_tol=1e-6)
    assert math.isclose(m["sft_loss"], 2 * math.log(16.0), rel_tol=1e-6)


def test_sft_term_sums_or_averages_the_chosen_rows():
    """``test_dpo_loss_varying_sequence_lengths``: lengths 3, 5, 4, 6, zero logits over 10 ids."""
    b, s, v = 4, 6, 10
    ids = torch.zeros((b, s), dtype=torch.long)
    tm = torch.zeros((b, s))
    for i, n in enumerate((3, 5, 4, 6)):
        ids[i, :n] = torch.arange(n)
        tm[i, :n] = 1.0
    data = {"input_ids": ids, "reference_policy_logprobs": torch.zeros((b, s)), "token_mask": tm, "sample_mask": torch.ones(b)}
    lp = OL.next_token_logprobs(ids, torch.zeros((b, s, v)))
    gs = data["sample_mask"].sum()
    _, m_sum = P.dpo_loss(P.DPOConfig(0.1, 1.0, 0.5, False, False), lp, data, gs)
    _, m_avg = P.dpo_loss(P.DPOConfig(0.1, 1.0, 0.5, True, True), lp, data, gs)
    # chosen rows have 2 and 3 unmasked next tokens, each costing log 10
    assert math.isclose(m_sum["sft_loss"], (2 + 3) * math.log(10.0) / 2, rel_tol=1e-6)
    assert math.isclose(m_avg["sft_loss"], math.log(10.0), rel_tol=1e-6)


def test_sft_only_matches_rescaled_nll():
    """``test_dpo_sft_matches_nll_loss``: with the preference weight at zero the loss is the NLL of
    the chosen rows times (chosen tokens / pairs)."""
    g = torch.Generator().manual_seed(3)
    v, pairs = 8, 2
    ids = torch.randint(0, v, (2 * pairs, 5), generator=g)
    tm = torch.tensor([[0, 0, 1, 1, 0], [0, 0, 1, 1, 1], [0, 1, 1, 1, 1], [0, 1, 1, 1, 0]])
    data = {"input_ids": ids, "token_mask": tm, "sample_mask": torch.tensor([1, 1, 1, 1]),
            "reference_policy_logprobs": torch.randn((4, 5), generator=g)}
    logits = torch.randn((4, 5, v), generator=g)
    lp = OL.next_token_logprobs(ids, logits)
    chosen = {k: t[::2] for k, t in data.items()}
    n_tok = (chosen["token_mask"][:, 1:] * chosen["sample_mask"].unsqueeze(-1)).sum()
    nll, _ = O.nll_loss(lp[::2], chosen, n_tok)
    dpo, _ = P.dpo_loss(P.DPOConfig(0.0, 0.0, 1.0, False, False), lp, data, data["sample_mask"].sum())
    assert math.isclose(dpo.item(), nll.item() * n_tok.item() / pairs, rel_tol=1e-5)


@pytest.mark.parametrize("avg_p,avg_s", [(False, False), (True, False), (False, True), (True, True)])
def test_brute_force_pairs(avg_p, avg_s):
    g = torch.Generator().manual_seed(11 + avg_p + 2 * avg_s)
    b, s = 6, 9
    lp = -torch.rand((b, s - 1), generator=g) * 3
    ref = -torch.rand((b, s), generator=g) * 3
    tm = (torch.rand((b, s), generator=g) < 0.6).float()
    tm[4] = 0                                       # a pair whose chosen row has no token
    sm = torch.tensor([1.0, 1.0, 0.5, 0.5, 1.0, 1.0])  # fractional masks enter the preference term squared
    sm[1] = 0.0                                     # the reference reads only the chosen row's mask for a pair
    data = {"token_mask": tm, "sample_mask": sm, "reference_policy_logprobs": ref}
    beta, wp, ws, gs = 0.3, 0.7, 0.2, 5.0
    loss, m = P.dpo_loss(P.DPOConfig(beta, wp, ws, avg_p, avg_s), lp, data, torch.tensor(gs))
    pref = sft = acc = rc = rr = 0.0
    for p in range(b // 2):
        rew, nll = [], []
        for row in (2 * p, 2 * p + 1):
            r = n = nl = nm = 0.0
            for t in range(s - 1):
                r += (lp[row, t].item() - ref[row, t].item()) * tm[row, t + 1].item()
                n += tm[row, t + 1].item()
                nl -= lp[row, t].item() * tm[row, t + 1].item() * sm[row].item()
                nm += tm[row, t + 1].item() * sm[row].item()
            rew.append(r / max(n, 1.0) if avg_p else r)
            nll.append(nl / max(nm, 1.0) if avg_s else nl)
        w = sm[2 * p].item()
        delta = beta * (rew[0] - rew[1])
        pref += math.log1p(math.exp(-delta)) * w * w
        sft += nll[0] * w
        acc += (rew[0] > rew[1]) * w
        rc += rew[0] * w
        rr += rew[1] * sm[2 * p + 1].item()
    den = gs / 2 + 1e-8
    assert math.isclose(m["preference_loss"], pref / den, rel_tol=1e-5, abs_tol=1e-7)
    assert math.isclose(m["sft_loss"], sft / den, rel_tol=1e-5, abs_tol=1e-7)
    assert math.isclose(loss.item(), (wp * pref + ws * sft) / den, rel_tol=1e-5, abs_tol=1e-7)
    assert math.isclose(m["accuracy"], acc / den, rel_tol=1e-6)
    assert math.isclose(m["rewards_chosen_mean"], rc / den, rel_tol=1e-5, abs_tol=1e-7)
    assert math.isclose(m["rewards_rejected_mean"], rr / den, rel_tol=1e-5, abs_tol=1e-7)
    assert math.isclose(m["num_valid_samples"], sm.sum().item() / 2, rel_tol=1e-6)


def test_reward_model_preference_loss():
    rewards = torch.tensor([[2.0], [1.0], [0.0], [3.0], [1.0], [1.0]])
    sm = torch.tensor([1.0, 1.0, 1.0, 1.0, 0.0, 0.0])
    loss, m = P.preference_loss(rewards, {"sample_mask": sm}, torch.tensor(4.0))
    want = (math.log1p(math.exp(-1.0)) + math.log1p(math.exp(3.0))) / (2 + 1e-8)
    assert math.isclose(loss.item(), want, rel_tol=1e-6)
    assert math.isclose(m["accuracy"], 0.5, rel_tol=1e-6) and math.isclose(m["rewards_chosen_mean"], 1.0, rel_tol=1e-6)
    assert math.isclose(m["rewards_rejected_mean"], 2.0, rel_tol=1e-6) and m["num_valid_samples"] == 2.0


def test_per_sample_nll_rows():
    lp = torch.tensor([[-1.0, -2.0, -3.0], [-0.5, -0.5, -0.5]])
    data = {"token_mask": torch.tensor([[1, 0, 1, 1], [1, 1, 1, 0]]), "sample_mask": torch.tensor([1.0, 0.5])}
    rows, m = P.nll_loss_rows(lp, data)
    assert torch.allclose(rows, torch.tensor([5.0, 0.5]))
    rows, _ = P.nll_loss_rows(lp, data, average_log_probs=True)
    assert torch.allclose(rows, torch.tensor([2.5, 0.5]))   # row 1: 0.5 / clamp(1.0, min=1)
    assert m["num_unmasked_tokens"] == 3.0 and m["num_valid_samples"] == 1.5
