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
