"""GPU parity of the two loss helpers that are also called on their own, ``calculate_kl`` and ``masked_mean``
(``nemo_rl/algorithms/utils.py:42-101, 207-224``): the reference's own golden values and gradient cases
(``tests/unit/algorithms/test_loss_functions.py:837-930``), then random inputs against the oracle and its autograd.
fp32 arithmetic on both sides with ``expf`` against torch's ``exp``: the k3 form ``exp(r) - 1 - r`` cancels for small
``r``, so the bound is a few units in the last place of the terms it subtracts (``exp(|r|) + 1 + |r|``), not of the
result."""

import pytest
import torch

from helpers import load_golden
from oracle import loss as OLoss
from rl_amd.algorithms import utils as U

pytestmark = pytest.mark.gpu
DEV = "cuda"
KL = load_golden("kl_cases.json")


@pytest.mark.parametrize("kl_type", ["k1", "k2", "k3"])
def test_calculate_kl_golden_values(kl_type):
    c = KL["values"]
    lp = torch.tensor(c["logprobs"], device=DEV)
    ref = torch.tensor(c["logprobs_reference"], device=DEV)
    got = U.calculate_kl(lp, ref, kl_type=kl_type, input_clamp_value=None, output_clamp_value=None)
    torch.testing.assert_close(got.cpu(), torch.tensor(c["unclamped"][kl_type]), rtol=c["rtol"], atol=0)
    got = U.calculate_kl(lp, ref, kl_type=kl_type)  # input clamp 20, output clamp 10
    torch.testing.assert_close(got.cpu(), torch.tensor(c["clamped_in20_out10"][kl_type]), rtol=c["rtol"], atol=0)


def test_input_clamp_detaches_the_importance_weight():
    c = KL["is_detach_when_input_clamped"]
    lp = torch.tensor(c["logprobs"], device=DEV, requires_grad=True)
    ref = torch.tensor(c["logprobs_reference"], device=DEV)
    w = torch.exp(lp - lp.detach())
    kl = U.calculate_kl(lp, ref, kl_type=c["kl_type"], input_clamp_value=c["input_clamp"],
                        output_clamp_value=c["output_clamp"], importance_sampling_weights=w)
    torch.testing.assert_close(kl.detach().cpu(), torch.tensor(c["expected_kl"]), rtol=1e-5, atol=0)
    kl.sum().backward()
    torch.testing.assert_close(lp.grad.cpu(), torch.tensor(c["expected_grad_of_sum"]), rtol=1e-5, atol=1e-6)


def test_output_clamp_blocks_the_weight_gradient():
    c = KL["output_clamp_blocks_is_gradient"]
    lp = torch.tensor(c["logprobs"], device=DEV, requires_grad=True)
    ref = torch.tensor(c["logprobs_reference"], device=DEV)
    w = 100 * torch.exp(lp - lp.detach())
    kl = U.calculate_kl(lp, ref, kl_type=c["kl_type"], input_clamp_value=c["input_clamp"],
                        output_clamp_value=c["output_clamp"], importance_sampling_weights=w)
    torch.testing.assert_close(kl.detach().cpu(), torch.tensor(c["expected_kl"]))
    kl.sum().backward()
    torch.testing.assert_close(lp.grad.cpu(), torch.tensor(c["expected_grad_of_sum"]))


@pytest.mark.parametrize("kl_type", ["k1", "k2", "k3"])
@pytest.mark.parametrize("clamps", [(None, None), (2.0, None), (None, 1.5), (1.0, 0.8), (20.0, 10.0)])
@pytest.mark.parametrize("weighted", [False, True])
def test_calculate_kl_random_against_the_oracle_and_its_autograd(kl_type, clamps, weighted):
    g = torch.Generator().manual_seed(int(kl_type[1]) * 100 + int(10 * (clamps[0] or 0)) + int(weighted))
    b, s = 5, 131
    lp = (-torch.rand(b, s, generator=g) * 4).requires_grad_(True)
    ref = (-torch.rand(b, s, generator=g) * 4).requires_grad_(True)
    w = (torch.rand(b, s, generator=g) * 2).requires_grad_(True) if weighted else None
    up = torch.randn(b, s, generator=g)
    want = OLoss.calculate_kl(lp, ref, kl_type, clamps[0], clamps[1], w)
    (want * up).sum().backward()
    leaves = [lp, ref] + ([w] if weighted else [])
    want_grads = [t.grad.clone() for t in leaves]
    dev = [t.detach().to(DEV).requires_grad_(True) for t in leaves]
    got = U.calculate_kl(dev[0], dev[1], kl_type, clamps[0], clamps[1], dev[2] if weighted else None)
    assert got.shape == want.shape and got.dtype == torch.float32 and got.is_cuda
    logr = (ref - lp).detach().abs()
    ulps = 8 * 2.0 ** -23 * (logr.exp() + 1 + logr) * (w.detach().abs().clamp(min=1) if weighted else 1)
    assert bool(((got.detach().cpu() - want.detach()).abs() <= ulps).all())
    (got * up.to(DEV)).sum().backward()
    for d, wg in zip(dev, want_grads):
        assert bool(((d.grad.cpu() - wg).abs() <= ulps * up.abs().clamp(min=1)).all())


def test_calculate_kl_broadcasts_and_follows_the_input_dtype_and_device():
    lp = torch.tensor([[-1.0, -2.0, -0.5]], dtype=torch.bfloat16, device=DEV)
    ref = torch.tensor([[-1.5], [-0.25]], dtype=torch.bfloat16, device=DEV)
    got = U.calculate_kl(lp, ref)
    want = OLoss.calculate_kl(lp.float().cpu(), ref.float().cpu())
    assert got.shape == (2, 3) and got.dtype == torch.bfloat16
    torch.testing.assert_close(got.float().cpu(), want.to(torch.bfloat16).float())
    host = U.calculate_kl(lp.float().cpu(), ref.float().cpu())  # the driver's tensors live on the host
    assert host.device.type == "cpu"
    torch.testing.assert_close(host, want, rtol=1e-6, atol=1e-7)
    with pytest.raises(ValueError, match="Invalid KL type"):
        U.calculate_kl(lp, ref, kl_type="k4")


@pytest.mark.parametrize("dim", [None, -1, 0, 1])
@pytest.mark.parametrize("norm", [None, 37.0, "tensor"])
def test_masked_mean_against_the_oracle_and_its_autograd(dim, norm):
    g = torch.Generator().manual_seed(11)
    v = torch.randn(6, 301, generator=g).requires_grad_(True)
    m = (torch.rand(6, 301, generator=g) < 0.6).float()
    m[2] = 0  # a row without any valid token: 0 / 1e-8
    n = torch.tensor(41.0) if norm == "tensor" else norm
    want = OLoss.masked_mean(v, m, dim=dim, global_normalization_factor=n)
    up = torch.randn(want.shape, generator=g)
    (want * up).sum().backward()
    vd = v.detach().to(DEV).requires_grad_(True)
    nd = n.to(DEV) if norm == "tensor" else n
    got = U.masked_mean(vd, m.to(DEV), dim=dim, global_normalization_factor=nd)
    assert got.shape == want.shape and got.is_cuda
    torch.testing.assert_close(got.detach().cpu(), want.detach(), rtol=2e-6, atol=1e-7)
    (got * up.to(DEV)).sum().backward()
    torch.testing.assert_close(vd.grad.cpu(), v.grad, rtol=2e-6, atol=1e-9)


def test_masked_mean_closed_forms_and_mask_broadcast():
    v = torch.tensor([[1.0, 2.0, 3.0, 4.0]], device=DEV)
    assert U.masked_mean(v, torch.tensor([[1, 0, 1, 0]], device=DEV)).item() == pytest.approx(2.0)
    assert U.masked_mean(v, torch.ones(1, 4, device=DEV), global_normalization_factor=5.0).item() == pytest.approx(2.0)
    assert U.masked_mean(v, torch.zeros(1, 4, device=DEV)).item() == 0.0
    rows = torch.arange(12.0, device=DEV).reshape(3, 4)
    got = U.masked_mean(rows, torch.tensor([1.0, 1.0, 0.0, 0.0], device=DEV), dim=-1)   # mask broadcast over the rows
    torch.testing.assert_close(got.cpu(), torch.tensor([0.5, 4.5, 8.5]))
    with pytest.raises(NotImplementedError):
        U.masked_mean(rows, torch.ones(3, 4, device=DEV), dim=(0, 1))


def test_neg_inf_warning_immediate_and_deferred(capsys):
    """``utils.py:227-257``: masked-out and infinite positions become 0 and the warning counts the valid tokens that
    were infinite.  By default the warning is printed once its counts have arrived from the device; with the switch
    off, before the function returns, as in the reference."""
    from oracle import logprob as OL

    lp = torch.tensor([[-1.0, float("-inf"), -2.0, float("-inf")], [-0.5, -0.25, float("-inf"), -3.0]], device=DEV)
    mask = torch.tensor([[1.0, 1.0, 0.0, 0.0], [1.0, 1.0, 1.0, 0.0]], device=DEV)
    want = OL.mask_out_neg_inf_logprobs(lp.cpu(), mask.cpu())
    assert U.DEFER_NEG_INF_WARNING is True
    U.flush_neg_inf_warnings()
    capsys.readouterr()
    U.DEFER_NEG_INF_WARNING = False
    try:
        got = U.mask_out_neg_inf_logprobs(lp, mask, "curr_logprobs")
        assert torch.equal(got.cpu(), want)
        assert "2/5 valid tokens have -inf in curr_logprobs" in capsys.readouterr().out
    finally:
        U.DEFER_NEG_INF_WARNING = True
    got = U.mask_out_neg_inf_logprobs(lp, mask, "prev_logprobs")
    quiet = U.mask_out_neg_inf_logprobs(lp[:, :1], mask[:, :1], "prev_logprobs")  # nothing infinite: no warning
    assert torch.equal(got.cpu(), want) and torch.equal(quiet, lp[:, :1])
    U.flush_neg_inf_warnings()
    out = capsys.readouterr().out
    assert out.count("[WARNING]") == 1 and "2/5 valid tokens have -inf in prev_logprobs" in out
    U.flush_neg_inf_warnings()  # nothing left
    assert capsys.readouterr().out == ""
