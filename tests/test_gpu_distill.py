"""GPU parity of the distillation reductions against the CPU oracle.  Tolerances as for the logprob
kernels: 1e-5 absolute (fp32 logits) / 2e-3 (bf16) on the per-row scalars, gradients within 1e-4 relative of
the fp32 oracle gradient plus the single narrowing to the logits' dtype."""

import pytest
import torch

from oracle import distill as OD
from rl_amd.distributed import model_utils as MU

pytestmark = pytest.mark.gpu
DEV = "cuda"
SHAPES = [(torch.float32, 1000), (torch.float32, 33), (torch.bfloat16, 4096), (torch.bfloat16, 50257), (torch.bfloat16, 151936)]


def _grad_ok(got, want, dtype):
    got = got.float().cpu()
    scale = want.abs().max().item() + 1e-30
    if dtype == torch.float32:
        return (got - want).abs().max().item() <= 1e-4 * scale
    return bool(((got - want).abs() <= want.abs() * (2.0 ** -8 + 1e-4) + 1e-4 * scale + 1e-30).all())


def _tol(dtype):
    return 1e-5 if dtype == torch.float32 else 2e-3


@pytest.mark.parametrize("dtype,vocab", SHAPES)
def test_neg_entropy(dtype, vocab):
    g = torch.Generator().manual_seed(vocab)
    b, s = 2, 5
    logits = (torch.randn(b, s, vocab, generator=g) * 2.5).to(dtype)
    up = torch.randn(b, s, generator=g)
    up[0, 1] = 0
    xo = logits.to(torch.float32, copy=True).requires_grad_(True)
    want = OD.neg_entropy(xo)
    (want * up).sum().backward()
    xg = logits.to(DEV).requires_grad_(True)
    got = MU.ChunkedDistributedEntropy.apply(xg, 2, None)
    assert got.shape == (b, s) and got.dtype == torch.float32
    assert (got.cpu() - want.detach()).abs().max().item() <= 10 * _tol(dtype)  # |H| is up to log V times a logprob error
    (got * up.to(DEV)).sum().backward()
    assert _grad_ok(xg.grad, xo.grad, dtype)
    assert bool((xg.grad[0, 1] == 0).all())


@pytest.mark.parametrize("dtype,vocab", SHAPES)
def test_gather_logprob(dtype, vocab):
    g = torch.Generator().manual_seed(vocab + 1)
    b, s, k = 2, 4, 6
    logits = (torch.randn(b, s, vocab, generator=g) * 2.5).to(dtype)
    idx = torch.randint(0, vocab, (b, s, k), generator=g)
    idx[0, 0, :3] = idx[0, 0, 0]  # duplicates
    up = torch.randn(b, s, k, generator=g)
    xo = logits.to(torch.float32, copy=True).requires_grad_(True)
    want = OD.gather_logprob(xo, idx)
    (want * up).sum().backward()
    xg = logits.to(DEV).requires_grad_(True)
    got = MU.ChunkedDistributedGatherLogprob.apply(xg, idx.to(DEV), 0, vocab, 3, None)
    assert (got.cpu() - want.detach()).abs().max().item() <= _tol(dtype)
    (got * up.to(DEV)).sum().backward()
    assert _grad_ok(xg.grad, xo.grad, dtype)


def test_gather_logprob_vocab_shard_reads_zero_outside():
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(1, 3, 64, generator=g)
    idx = torch.randint(0, 200, (1, 3, 5), generator=g)
    want = OD.gather_logprob(logits, idx, 100, 164)
    got = MU.ChunkedDistributedGatherLogprob.apply(logits.to(DEV), idx.to(DEV), 100, 164, 8, None, True)
    assert (got.cpu() - want).abs().max().item() <= 1e-5
    assert bool((got.cpu()[(idx < 100) | (idx >= 164)] == 0).all())


@pytest.mark.parametrize("dtype,vocab", SHAPES)
def test_soft_cross_entropy(dtype, vocab):
    g = torch.Generator().manual_seed(vocab + 2)
    b, s = 2, 3
    student = (torch.randn(b, s, vocab, generator=g) * 2.5).to(dtype)
    teacher = (torch.randn(b, s, vocab, generator=g) * 2.5).to(dtype)
    up = torch.randn(b, s, generator=g)
    xo = student.to(torch.float32, copy=True).requires_grad_(True)
    want = OD.soft_cross_entropy(xo, teacher.float())
    (want * up).sum().backward()
    xg = student.to(DEV).requires_grad_(True)
    got = MU.DistributedCrossEntropy.apply(xg, teacher.to(DEV), None)
    assert got.shape == (b, s)
    assert (got.cpu() - want.detach()).abs().max().item() <= 10 * _tol(dtype)
    (got * up.to(DEV)).sum().backward()
    assert _grad_ok(xg.grad, xo.grad, dtype)
    with pytest.raises(ValueError):
        MU.DistributedCrossEntropy.apply(xg, teacher.to(DEV)[..., :-1], None)


def test_strided_views_and_odd_alignment():
    g = torch.Generator().manual_seed(4)
    big = torch.randn(2, 6, 1003, generator=g).to(DEV)
    view = big[:, 1:5, 3:1000]  # rows start off a 16-byte boundary, 997 columns
    want = OD.neg_entropy(view.cpu())
    got = MU.ChunkedDistributedEntropy.apply(view, 4, None, True)
    assert (got.cpu() - want).abs().max().item() <= 1e-5


# ---- top-k distillation path: prepare_loss_input(DISTILLATION) + DistillationLossFn ----
def _kd_inputs(b, s, v, k, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    student = (torch.randn(b, s, v, generator=g) * 2).to(dtype)
    teacher_full = torch.randn(b, s, v, generator=g) * 2
    t_logits, t_idx = torch.topk(teacher_full, k, dim=-1)
    tm = (torch.rand(b, s, generator=g) < 0.7).float()
    tm[:, 0] = 0
    sm = torch.ones(b)
    if b > 1:
        sm[1] = 0.5
    if b > 2:
        sm[2] = 0
    data = {"input_ids": torch.zeros(b, s, dtype=torch.long), "token_mask": tm, "sample_mask": sm,
            "teacher_topk_logits": t_logits, "teacher_topk_indices": t_idx}
    gt = (tm[:, 1:] * sm.unsqueeze(-1)).sum()
    return student, data, gt


@pytest.mark.parametrize("kl_type,zero_outside", [("forward", False), ("forward", True), ("reverse", False), ("reverse", True),
                                                  ("mixed", False), ("mixed", True)])
@pytest.mark.parametrize("dtype,v,k,tol", [(torch.float32, 500, 16, 1e-5), (torch.bfloat16, 4096, 64, 2e-3)])
def test_distillation_path_matches_oracle(kl_type, zero_outside, dtype, v, k, tol):
    from oracle import distill as D
    from rl_amd.algorithms.loss import DistillationLossConfig, DistillationLossFn, prepare_loss_input

    student, data, gt = _kd_inputs(4, 9, v, k, dtype, seed=v + k)
    xo = student.to(torch.float32).clone().requires_grad_(True)
    s_lp, t_lp, h = D.distillation_topk_logprobs(xo, data["teacher_topk_logits"], data["teacher_topk_indices"], zero_outside,
                                                 zero_outside and kl_type != "forward")
    want, wm = D.distillation_loss(kl_type, 0.3, zero_outside, s_lp, t_lp, h, data, gt)
    want.backward()

    fn = DistillationLossFn(DistillationLossConfig(kl_type=kl_type, mixed_kl_weight=0.3, zero_outside_topk=zero_outside))
    xg = student.to(DEV).requires_grad_(True)
    ddev = {k_: t.to(DEV) for k_, t in data.items()}
    loss_input, d2 = prepare_loss_input(xg, ddev, fn)
    assert (loss_input["student_topk_logprobs"].detach().cpu() - s_lp.detach()).abs().max().item() <= tol
    assert (loss_input["teacher_topk_logprobs"].cpu() - t_lp).abs().max().item() <= 1e-5
    assert (loss_input["H_all"] is None) == (h is None)
    got, gm = fn(data=d2, global_valid_seqs=None, global_valid_toks=gt.to(DEV), **loss_input)
    got.backward()
    assert abs(got.item() - want.item()) <= (1e-4 if dtype == torch.float32 else 2e-3) * abs(want.item()) + 1e-6
    assert gm["num_valid_samples"] == wm["num_valid_samples"] and abs(gm["loss"] - got.item()) < 1e-7
    scale = xo.grad.abs().max().item() + 1e-30
    diff = (xg.grad.float().cpu() - xo.grad).abs().max().item()
    assert diff <= (1e-4 if dtype == torch.float32 else 2.0 ** -7) * scale
    assert torch.all(xg.grad[:, -1] == 0)  # the last position feeds nothing


def test_distillation_loss_without_masks_and_with_duplicate_indices():
    from oracle import distill as D
    from rl_amd.algorithms.loss import DistillationLossConfig, DistillationLossFn, prepare_loss_input

    student, data, _gt = _kd_inputs(2, 6, 300, 8, torch.float32, seed=3)
    data["teacher_topk_indices"][:, :, 3] = data["teacher_topk_indices"][:, :, 1]  # a repeated id: its gradients add up
    plain = {k: v for k, v in data.items() if k not in ("token_mask", "sample_mask")}
    xo = student.clone().requires_grad_(True)
    s_lp, t_lp, h = D.distillation_topk_logprobs(xo, plain["teacher_topk_logits"], plain["teacher_topk_indices"], False, False)
    want, _ = D.distillation_loss("mixed", 0.5, False, s_lp, t_lp, h, plain, None)
    want.backward()
    fn = DistillationLossFn(DistillationLossConfig())
    xg = student.to(DEV).requires_grad_(True)
    loss_input, d2 = prepare_loss_input(xg, {k: v.to(DEV) for k, v in plain.items()}, fn)
    got, _ = fn(data=d2, global_valid_seqs=None, global_valid_toks=None, **loss_input)
    got.backward()
    assert abs(got.item() - want.item()) <= 1e-4 * abs(want.item()) + 1e-7
    assert (xg.grad.cpu() - xo.grad).abs().max().item() <= 1e-4 * xo.grad.abs().max().item()


def test_distillation_rejects_an_empty_top_k():
    from rl_amd.algorithms.loss import DistillationLossConfig, DistillationLossFn, prepare_loss_input

    fn = DistillationLossFn(DistillationLossConfig())
    data = {"input_ids": torch.zeros(1, 3, dtype=torch.long), "teacher_topk_logits": torch.zeros(1, 3, 0),
            "teacher_topk_indices": torch.zeros(1, 3, 0, dtype=torch.long)}
    with pytest.raises(ValueError):
        prepare_loss_input(torch.zeros(1, 3, 16, device=DEV), data, fn)
    with pytest.raises(AssertionError):
        DistillationLossFn(DistillationLossConfig(kl_type="sideways"))


def test_draft_cross_entropy_loss():
    """``DraftCrossEntropyLossFn`` against the reference's own non-parallel formula
    (``loss_functions.py:96-101``) evaluated on the CPU."""
    from rl_amd.algorithms.loss import DraftCrossEntropyLossFn

    g = torch.Generator().manual_seed(21)
    b, s, v = 3, 7, 1000
    teacher = torch.randn(b, s, v, generator=g) * 2
    student = torch.randn(b, s, v, generator=g) * 2
    tm = (torch.rand(b, s, generator=g) < 0.7).float()
    sm = torch.tensor([1.0, 0.0, 0.5])
    gt = (tm * sm.unsqueeze(-1)).sum()
    xo = student.clone().requires_grad_(True)
    per_token = OD.soft_cross_entropy(xo, teacher)
    want = (per_token * tm * sm.unsqueeze(-1)).sum() / (gt + 1e-8)
    want.backward()
    xg = student.to(DEV).requires_grad_(True)
    got = DraftCrossEntropyLossFn()(teacher.to(DEV), xg, tm.to(DEV), {"sample_mask": sm.to(DEV)}, None, gt.to(DEV))
    got.backward()
    assert abs(got.item() - want.item()) <= 1e-4 * abs(want.item())
    assert (xg.grad.cpu() - xo.grad).abs().max().item() <= 1e-4 * xo.grad.abs().max().item()
    assert torch.all(xg.grad[1] == 0)
