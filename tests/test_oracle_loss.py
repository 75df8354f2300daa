"""Pins the loss oracle to the reference's golden vectors and closed forms
(CPU only)."""

import math

import pytest
import torch

from oracle import loss as O
from helpers import golden_case_to_inputs, load_golden

KL = load_golden("kl_cases.json")
PG = load_golden("clipped_pg_cases.json")


@pytest.mark.parametrize("kl_type", ["k1", "k2", "k3"])
def test_calculate_kl_golden(kl_type):
    v = KL["values"]
    lp, ref = torch.tensor(v["logprobs"]), torch.tensor(v["logprobs_reference"])
    got = O.calculate_kl(lp, ref, kl_type, None, None)
    assert torch.allclose(got, torch.tensor(v["unclamped"][kl_type]), rtol=v["rtol"])
    got = O.calculate_kl(lp, ref, kl_type, 20.0, 10.0)
    assert torch.allclose(got, torch.tensor(v["clamped_in20_out10"][kl_type]), rtol=v["rtol"])


def test_calculate_kl_is_weight_detached_when_input_clamped():
    c = KL["is_detach_when_input_clamped"]
    lp = torch.tensor(c["logprobs"], requires_grad=True)
    w = torch.exp(lp - lp.detach())
    kl = O.calculate_kl(lp, torch.tensor(c["logprobs_reference"]), "k3", c["input_clamp"], None, w)
    torch.testing.assert_close(kl.detach(), torch.tensor(c["expected_kl"]))
    kl.sum().backward()
    torch.testing.assert_close(lp.grad, torch.tensor(c["expected_grad_of_sum"]), atol=1e-6, rtol=1e-6)


def test_calculate_kl_output_clamp_blocks_is_gradient():
    c = KL["output_clamp_blocks_is_gradient"]
    lp = torch.tensor(c["logprobs"], requires_grad=True)
    w = 100.0 * torch.exp(lp - lp.detach())
    kl = O.calculate_kl(lp, torch.tensor(c["logprobs_reference"]), "k3", None, c["output_clamp"], w)
    torch.testing.assert_close(kl.detach(), torch.tensor(c["expected_kl"]))
    kl.sum().backward()
    torch.testing.assert_close(lp.grad, torch.tensor(c["expected_grad_of_sum"]), atol=1e-6, rtol=1e-6)


def test_masked_mean_closed_forms():
    v = torch.tensor([1.0, 2.0, 3.0, 4.0])
    m = torch.zeros(4)
    assert O.masked_mean(v, m).item() == 0.0
    m[0] = 1
    torch.testing.assert_close(O.masked_mean(v, m), torch.tensor(1.0))
    v2 = torch.tensor([[1.0, 2.0], [3.0, 4.0]])
    torch.testing.assert_close(O.masked_mean(v2, torch.zeros(2, 2), dim=1), torch.zeros(2))
    torch.testing.assert_close(
        O.masked_mean(v2, torch.ones(2, 2), global_normalization_factor=8.0), torch.tensor(1.25)
    )


@pytest.mark.parametrize("case", PG["cases"], ids=[c["name"] for c in PG["cases"]])
def test_clipped_pg_golden(case):
    lp, data, gs, gt = golden_case_to_inputs(case)
    cfg = O.LossConfig(**case["cfg"])
    loss, metrics = O.clipped_pg_loss(cfg, lp.clone().requires_grad_(True), data, gs, gt)
    if "expected_loss" in case:
        exp = case["expected_loss"]
        tol = case.get("rtol", 0.0) * abs(exp) + case.get("atol", 1e-6)
        assert abs(loss.item() - exp) <= tol, (loss.item(), exp)
    for k, v in case.get("expected_metrics_exact", {}).items():
        assert metrics[k] == v, (k, metrics[k])
    for k, v in case.get("expected_metrics_approx", {}).items():
        assert metrics[k] == pytest.approx(v, rel=1e-5), (k, metrics[k])
    if case.get("property") == "loss is finite":
        assert math.isfinite(loss.item())


@pytest.mark.parametrize("approx", [False, True])
def test_kl_gradient_includes_sampling_term(approx):
    c = PG["kl_gradient_case"]
    t = lambda k: torch.tensor(c[k])
    z = torch.zeros(1, 1)

    def grad(beta):
        lp = t("curr").clone().requires_grad_(True)
        data = {
            "token_mask": torch.tensor([[0, 1, 1]]), "sample_mask": torch.tensor([1]),
            "advantages": torch.cat([z, t("adv")], -1), "prev_logprobs": torch.cat([z, t("prev")], -1),
            "generation_logprobs": torch.cat([z, t("gen")], -1),
            "reference_policy_logprobs": torch.cat([z, t("ref")], -1),
        }
        cfg = O.LossConfig(reference_policy_kl_penalty=beta, use_on_policy_kl_approximation=approx)
        gt = torch.sum(data["sample_mask"].unsqueeze(-1) * data["token_mask"])
        loss, _ = O.clipped_pg_loss(cfg, lp, data, torch.sum(data["sample_mask"]), gt)
        loss.backward()
        return lp.grad

    got = grad(c["beta"]) - grad(0.0)
    logr = t("ref") - t("curr")
    kl = torch.exp(logr) - 1 - logr
    w = torch.exp(t("curr") - t("gen")) if approx else torch.ones_like(logr)
    torch.testing.assert_close(got, c["beta"] * w * (kl + 1 - torch.exp(logr)) / 2)


@pytest.mark.parametrize("bad", PG["config_asserts"]["must_raise_assertion"])
def test_config_asserts(bad):
    with pytest.raises(AssertionError):
        O.check_config(O.LossConfig(**bad))


def test_zero_mask_gives_exact_zero():
    case = PG["cases"][0]
    lp, data, gs, gt = golden_case_to_inputs(case)
    data["token_mask"] = torch.zeros_like(data["token_mask"])
    gt = torch.sum(data["sample_mask"].unsqueeze(-1) * data["token_mask"])
    loss, m = O.clipped_pg_loss(O.LossConfig(reference_policy_kl_penalty=0.1), lp, data, gs, gt)
    assert loss.item() == 0.0
    assert m["probs_ratio_min"] == float("inf") and m["probs_ratio_max"] == float("-inf")


def test_sample_mask_equals_sub_batch():
    torch.manual_seed(3)
    b, s = 2, 6
    lp = -torch.rand(b, s - 1)
    data = {
        "token_mask": torch.cat([torch.zeros(b, 1, dtype=torch.int64), torch.ones(b, s - 1, dtype=torch.int64)], 1),
        "sample_mask": torch.tensor([1, 0]),
        "advantages": torch.randn(b, s) + 1, "prev_logprobs": torch.randn(b, s) * 0.1 - 0.5,
        "generation_logprobs": torch.randn(b, s) * 0.1 - 0.5,
        "reference_policy_logprobs": torch.randn(b, s) * 0.1 - 0.5,
    }
    cfg = O.LossConfig(reference_policy_kl_penalty=0.1)
    gt = torch.sum(data["sample_mask"].unsqueeze(-1) * data["token_mask"])
    full, _ = O.clipped_pg_loss(cfg, lp, data, data["sample_mask"].sum(), gt)
    sub = {k: v[:1] for k, v in data.items()}
    gt0 = torch.sum(sub["sample_mask"].unsqueeze(-1) * sub["token_mask"])
    only, _ = O.clipped_pg_loss(cfg, lp[:1], sub, sub["sample_mask"].sum(), gt0)
    torch.testing.assert_close(full, only)


def test_diagnostics_against_float64_formulas():
    """The diagnostics the reference never tests numerically: independent
    float64 evaluation of their textbook definitions."""
    torch.manual_seed(11)
    b, s = 3, 9
    lp = -torch.rand(b, s - 1) * 2
    prev = torch.cat([torch.zeros(b, 1), lp + 0.05 * torch.randn(b, s - 1)], 1)
    gen = torch.cat([torch.zeros(b, 1), lp + 0.05 * torch.randn(b, s - 1)], 1)
    tm = torch.ones(b, s, dtype=torch.int64)
    tm[:, 0] = 0
    tm[1, 5:] = 0
    data = {"token_mask": tm, "sample_mask": torch.tensor([1.0, 1.0, 0.0]), "advantages": torch.randn(b, s),
            "prev_logprobs": prev, "generation_logprobs": gen, "reference_policy_logprobs": prev}
    mask = (tm[:, 1:] * data["sample_mask"].unsqueeze(-1)).double()
    n = mask.sum()
    _, m = O.clipped_pg_loss(O.LossConfig(reference_policy_kl_penalty=0.0), lp, data, torch.tensor(2.0), n.float())
    p, g, c = prev[:, 1:].double(), gen[:, 1:].double(), lp.double()
    mean = lambda v: float((v * mask).sum() / n)
    assert m["token_mult_prob_error"] == pytest.approx(mean(torch.exp((g - p).abs())), rel=1e-5)
    assert m["gen_kl_error"] == pytest.approx(mean(torch.exp(p - g) - 1 - (p - g)), rel=1e-3, abs=1e-7)
    assert m["policy_kl_error"] == pytest.approx(mean(torch.exp(g - p) - 1 - (g - p)), rel=1e-3, abs=1e-7)
    mix = 0.5 * (p.exp() + g.exp())
    js = 0.5 * (p.exp() / mix - 1 - (p - mix.log())) + 0.5 * (g.exp() / mix - 1 - (g - mix.log()))
    assert m["js_divergence_error"] == pytest.approx(mean(js), rel=1e-2, abs=1e-7)
    assert m["sampling_importance_ratio"] == pytest.approx(mean(torch.exp(p - g)), rel=1e-5)
    r = torch.exp(c - p)
    assert m["probs_ratio"] == pytest.approx(mean(r), rel=1e-5)
    assert m["probs_ratio_clamped"] == pytest.approx(mean(r.clamp(0.8, 1.2)), rel=1e-5)
    assert m["probs_ratio_min"] == pytest.approx(float(r[mask.bool()].min()), rel=1e-5)
    assert m["probs_ratio_max"] == pytest.approx(float(r[mask.bool()].max()), rel=1e-5)
    assert m["approx_entropy"] == pytest.approx(-mean(torch.exp(c - g) * c), rel=1e-5)
    assert m["num_valid_samples"] == 2.0


def _packed_oracle_case(**kw):
    from helpers import packed_grpo_case

    return packed_grpo_case(dtype=torch.float32, seed=13, **kw)


def test_sequence_packing_loss_equals_one_call_on_the_unpacked_batch():
    """The identity the reference's own test states for its two wrappers
    (``tests/unit/algorithms/test_sequence_packing_fusion.py:190-265``): with global normalisers the per-sequence
    losses add up to the loss of the whole unpacked batch, and so do the gradients."""
    from oracle import logprob as OL

    logits, data, cu, cup, gs, gt = _packed_oracle_case(lens=[9, 5, 12, 7], pads=[3, 1, 0, 5], width=14, vocab=64)
    for cfg in (O.LossConfig(), O.LossConfig(token_level_loss=False, reference_policy_kl_penalty=0.01)):
        x1 = logits.clone().requires_grad_(True)
        l1, m1 = O.sequence_packing_loss(cfg, x1, data, cu, cup, gs, gt, OL.next_token_logprobs)
        l1.backward()
        x2 = logits.clone().requires_grad_(True)
        targets = OL.pack_input_ids(data["input_ids"], cu, cup, roll_shift=-1)
        lp = OL.packed_logits_to_logprobs(x2[:, : int(cup[-1])], targets, cup, 14, target_is_pre_rolled=True)
        l2, m2 = O.clipped_pg_loss(cfg, lp, data, gs, gt)
        l2.backward()
        torch.testing.assert_close(l1, l2, atol=1e-6, rtol=1e-5)
        torch.testing.assert_close(x1.grad, x2.grad, atol=1e-7, rtol=1e-5)
        for k in ("probs_ratio_min", "probs_ratio_max", "probs_ratio_clamped_min", "probs_ratio_clamped_max",
                  "probs_ratio", "token_mult_prob_error", "num_valid_samples"):
            assert m1[k] == pytest.approx(m2[k], rel=1e-5), k


def test_sequence_packing_loss_extrema_skip_empty_sequences():
    """Brute force for the min / max merge (``loss/wrapper.py:145-164``): the merged extrema are the extrema over
    all valid tokens; a sequence without valid tokens contributes its +-inf sentinels, which are skipped; with no
    valid token anywhere the sentinels stay."""
    from oracle import logprob as OL

    logits, data, cu, cup, gs, gt = _packed_oracle_case(lens=[6, 4, 8], pads=[2, 0, 1], width=8, vocab=32, empty_mask_rows=(1,))
    _, m = O.sequence_packing_loss(O.LossConfig(), logits, data, cu, cup, gs, gt, OL.next_token_logprobs)
    ratios = []
    for i in (0, 2):
        n = int(cu[i + 1] - cu[i])
        piece = logits[:, int(cup[i]) : int(cup[i + 1])]
        lp = OL.next_token_logprobs(data["input_ids"][i : i + 1, :n], piece)[0]
        r = torch.exp(lp - data["prev_logprobs"][i, 1:n])
        ratios.append(r[data["token_mask"][i, 1:n] > 0])
    allr = torch.cat(ratios)
    assert m["probs_ratio_min"] == pytest.approx(allr.min().item(), rel=1e-6)
    assert m["probs_ratio_max"] == pytest.approx(allr.max().item(), rel=1e-6)
    assert m["probs_ratio_clamped_min"] == pytest.approx(allr.clamp(0.8, 1.2).min().item(), rel=1e-6)
    data["token_mask"] = torch.zeros_like(data["token_mask"])
    _, m = O.sequence_packing_loss(O.LossConfig(), logits, data, cu, cup, gs, gt, OL.next_token_logprobs)
    assert m["probs_ratio_min"] == float("inf") and m["probs_ratio_max"] == float("-inf")
