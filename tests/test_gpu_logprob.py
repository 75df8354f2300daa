"""GPU parity: HIP logits -> logprob kernels against the CPU oracle.

Tolerances (from the parity contract): logprobs within 1e-5 absolute for fp32 logits and 2e-3 for
bf16/fp16 logits; gradients within 1e-4 relative (fp32), and for 16-bit logits within half a unit
in the last place of the fp32 oracle gradient (the single narrowing) plus that 1e-4."""

import pytest
import torch

from oracle import logprob as OL
from rl_amd.distributed import model_utils as MU

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _oracle_fwd_bwd(logits_cpu, ids_cpu, g_cpu, **kw):
    x = logits_cpu.to(torch.float32, copy=True).requires_grad_(True)  # exact upcast: the fp32 gradient before narrowing
    lp = OL.from_logits_to_logprobs(x, ids_cpu, **kw)
    (lp * g_cpu).sum().backward()
    return lp.detach(), x.grad


def _check_grad(got, want_f32, dtype):
    got = got.float().cpu()
    scale = want_f32.abs().max().item() + 1e-30
    if dtype == torch.float32:
        assert (got - want_f32).abs().max().item() <= 1e-4 * scale
    else:
        ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
        floor = 2.0 ** -24 if dtype == torch.float16 else 1e-30  # fp16 subnormal spacing
        bound = want_f32.abs() * (ulp + 1e-4) + 1e-4 * scale * ulp + floor
        assert bool(((got - want_f32).abs() <= bound).all())
        same = (got == want_f32.to(dtype).float()).float().mean().item()
        assert same > 0.99, same


@pytest.mark.parametrize("dtype,vocab,atol", [
    (torch.float32, 32000, 1e-5), (torch.float32, 1000, 1e-5), (torch.float32, 33, 1e-5), (torch.float32, 8, 1e-5),
    (torch.bfloat16, 151936, 2e-3), (torch.bfloat16, 50257, 2e-3), (torch.bfloat16, 33, 2e-3),
    (torch.float16, 4099, 2e-3),
])
def test_logprob_fwd_bwd_matches_oracle(dtype, vocab, atol):
    g = torch.Generator().manual_seed(vocab)
    b, s = 2, 9
    logits = (torch.randn(b, s, vocab, generator=g) * 2).to(dtype)
    ids = torch.randint(0, vocab, (b, s), generator=g)
    up = torch.randn(b, s - 1, generator=g)
    up[0, 2] = 0.0
    want_lp, want_grad = _oracle_fwd_bwd(logits, ids, up)

    x = logits.to(DEV).requires_grad_(True)
    lp = MU.from_parallel_logits_to_logprobs(x, ids.to(DEV), 0, vocab, None)
    assert lp.shape == (b, s - 1) and lp.dtype == torch.float32
    assert (lp.cpu() - want_lp).abs().max().item() <= atol
    (lp * up.to(DEV)).sum().backward()
    assert x.grad.dtype == dtype and x.grad.shape == x.shape
    _check_grad(x.grad, want_grad.float(), dtype)
    assert torch.all(x.grad[:, -1] == 0) and torch.all(x.grad[0, 2] == 0)
    # rows with an in-range target sum to zero (softmax - onehot)
    assert x.grad.float().sum(-1).abs().max().item() <= (1e-5 if dtype == torch.float32 else 2e-2) * up.abs().max().item()


def test_spiked_logits_times_100_stay_finite():
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(2, 6, 1024, generator=g) * 100
    ids = torch.zeros(2, 6, dtype=torch.long)
    want = OL.from_logits_to_logprobs(logits, ids)
    got = MU.from_parallel_logits_to_logprobs(logits.to(DEV), ids.to(DEV), 0, 1024, None).cpu()
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("fill", ["-inf", "min"])
def test_masked_vocabulary_runs_contribute_nothing(dtype, fill):
    """Long runs of -inf (or the dtype's most negative value) in a row, including at its start where a
    lane sees nothing finite first, must not disturb the log-sum-exp or the gradient."""
    g = torch.Generator().manual_seed(15)
    vocab = 6144
    logits = torch.randn(2, 5, vocab, generator=g).to(dtype)
    val = float("-inf") if fill == "-inf" else torch.finfo(dtype).min
    logits[..., :2048] = val
    logits[..., 4000:4100] = val
    ids = torch.randint(2048, 4000, (2, 5), generator=g)
    up = torch.randn(2, 4, generator=g)
    want_lp, want_grad = _oracle_fwd_bwd(logits, ids, up)
    x = logits.to(DEV).requires_grad_(True)
    got = MU.from_parallel_logits_to_logprobs(x, ids.to(DEV), 0, vocab, None)
    (got * up.to(DEV)).sum().backward()
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.cpu(), want_lp, rtol=0, atol=1e-5 if dtype == torch.float32 else 2e-3)
    assert torch.isfinite(x.grad).all()
    assert (x.grad[..., :2048] == 0).all() and (x.grad[..., 4000:4100] == 0).all()
    _check_grad(x.grad[:, :-1], want_grad[:, :-1], dtype)


def test_out_of_shard_targets():
    g = torch.Generator().manual_seed(6)
    logits = torch.randn(1, 5, 16, generator=g)
    ids = torch.tensor([[0, 3, 20, 40, 16]])  # shard covers [16, 32)
    want_lp, want_grad = _oracle_fwd_bwd(logits, ids, torch.ones(1, 4), vocab_start=16, vocab_end=32)
    x = logits.to(DEV).requires_grad_(True)
    lp = MU.from_parallel_logits_to_logprobs(x, ids.to(DEV), 16, 32, None)
    torch.testing.assert_close(lp.cpu(), want_lp, rtol=0, atol=1e-5)
    assert lp[0, 0].item() == 0.0 and lp[0, 2].item() == 0.0
    lp.sum().backward()
    torch.testing.assert_close(x.grad.cpu(), want_grad, rtol=1e-4, atol=1e-6)


def test_autograd_classes_match_reference_call_convention():
    g = torch.Generator().manual_seed(7)
    vocab = 257
    logits = torch.randn(2, 8, vocab, generator=g)
    tgt = torch.randint(0, vocab, (2, 8), generator=g)  # already shifted: all S positions are computed
    want = OL.rows_logprob(logits, tgt)
    x = logits.to(DEV).requires_grad_(True)
    a = MU.DistributedLogprob.apply(x, tgt.to(DEV), 0, vocab, None, False)
    c = MU.ChunkedDistributedLogprob.apply(x, tgt.to(DEV), 0, vocab, 3, None, False)
    assert a.shape == (2, 8)
    torch.testing.assert_close(a.cpu(), want, rtol=0, atol=1e-5)
    assert torch.equal(a, c)  # chunking never changes a bit
    ga, = torch.autograd.grad(a.sum(), x)
    gc, = torch.autograd.grad(c.sum(), x)
    assert torch.equal(ga, gc)
    xo = logits.clone().requires_grad_(True)
    OL.rows_logprob(xo, tgt).sum().backward()
    torch.testing.assert_close(ga.cpu(), xo.grad, rtol=1e-4, atol=1e-6)
    with torch.no_grad():
        inf_only = MU.DistributedLogprob.apply(logits.to(DEV), tgt.to(DEV), 0, vocab, None, True)
    assert torch.equal(inf_only, a.detach())


def test_next_token_front_door_and_strided_views():
    g = torch.Generator().manual_seed(8)
    vocab = 1001  # odd: bf16 rows start at 2-byte offsets, exercising the unaligned head/tail path
    big = (torch.randn(3, 7, vocab + 3, generator=g)).to(torch.bfloat16)
    logits = big[:, :, 1 : vocab + 1]  # non-contiguous rows, contiguous vocab axis
    ids = torch.randint(0, vocab, (3, 7), generator=g)
    want = OL.next_token_logprobs(ids, logits)
    xg = big.to(DEV)[:, :, 1 : vocab + 1].requires_grad_(True)
    got = MU.get_next_token_logprobs_from_logits(ids, xg)  # ids on the host, like the reference allows
    assert (got.cpu() - want).abs().max().item() <= 2e-3
    got.sum().backward()
    xo = logits.to(torch.float32, copy=True).requires_grad_(True)
    OL.next_token_logprobs(ids, xo).sum().backward()
    _check_grad(xg.grad, xo.grad, torch.bfloat16)


def test_batch_invariance_bitwise():
    g = torch.Generator().manual_seed(9)
    vocab = 151936
    logits = (torch.randn(4, 5, vocab, generator=g) * 3).to(torch.bfloat16).to(DEV)
    ids = torch.randint(0, vocab, (4, 5), generator=g).to(DEV)
    full = MU.from_parallel_logits_to_logprobs(logits, ids, 0, vocab, None)
    for b in range(4):
        one = MU.from_parallel_logits_to_logprobs(logits[b : b + 1], ids[b : b + 1], 0, vocab, None)
        assert torch.equal(one[0], full[b])
    again = MU.from_parallel_logits_to_logprobs(logits, ids, 0, vocab, None)
    assert torch.equal(again, full)


def test_empty_and_single_position_inputs():
    x = torch.zeros(0, 4, 16, device=DEV)
    out = MU.from_parallel_logits_to_logprobs(x, torch.zeros(0, 4, dtype=torch.long, device=DEV), 0, 16, None)
    assert out.shape == (0, 3)
    x = torch.zeros(2, 1, 16, device=DEV)
    out = MU.from_parallel_logits_to_logprobs(x, torch.zeros(2, 1, dtype=torch.long, device=DEV), 0, 16, None)
    assert out.shape == (2, 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pre_rolled", [False, True])
def test_packed_sequences_match_oracle(dtype, pre_rolled):
    # lengths of the reference's own test (tests/unit/distributed/test_model_utils.py:254-434) + padding + empty
    g = torch.Generator().manual_seed(10)
    lens, pads = [24, 48, 0, 16, 40], [24, 48, 0, 20, 40]
    vocab, smax = 515, 48
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    cup = torch.tensor([0] + torch.tensor(pads).cumsum(0).tolist(), dtype=torch.int32)
    ids = torch.zeros(len(lens), smax, dtype=torch.int64)
    for i, n in enumerate(lens):
        ids[i, :n] = torch.randint(0, vocab, (n,), generator=g)
    total = int(cup[-1])
    logits = (torch.randn(1, total, vocab, generator=g) * 2).to(dtype)
    targets = OL.pack_input_ids(ids, cu, cup, roll_shift=-1 if pre_rolled else 0)
    up = torch.randn(len(lens), smax - 1, generator=g)

    xo = logits.to(torch.float32, copy=True).requires_grad_(True)
    want = OL.packed_logits_to_logprobs(xo, targets, cup, smax, target_is_pre_rolled=pre_rolled)
    (want * up).sum().backward()

    xg = logits.to(DEV).requires_grad_(True)
    got = MU.from_parallel_logits_to_logprobs_packed_sequences(
        xg, targets.to(DEV), cup.to(DEV), smax, 0, vocab, None, target_is_pre_rolled=pre_rolled)
    assert got.shape == (len(lens), smax - 1)
    assert (got.cpu() - want.detach()).abs().max().item() <= (1e-5 if dtype == torch.float32 else 2e-3)
    (got * up.to(DEV)).sum().backward()
    _check_grad(xg.grad, xo.grad.float(), dtype)


def test_packed_rejects_bad_boundaries():
    x = torch.zeros(1, 8, 16, device=DEV)
    t = torch.zeros(1, 8, dtype=torch.long, device=DEV)
    with pytest.raises(ValueError):
        MU.from_parallel_logits_to_logprobs_packed_sequences(x, t, torch.tensor([0, 5, 12]), 8, 0, 16, None)
    with pytest.raises(ValueError):
        MU.from_parallel_logits_to_logprobs_packed_sequences(x, t, torch.tensor([0, 5, 3]), 8, 0, 16, None)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fused_temperature_matches_in_place_divide(dtype):
    """The kernel's fused temperature reproduces logits.div_(T) done in the logits' dtype (GPU
    semantics: multiply by the fp32 reciprocal, round to the dtype)."""
    from rl_amd._lib import NRL_TEMP_DIV, NRL_TEMP_RCP

    g = torch.Generator().manual_seed(11)
    vocab, t = 4096, 0.7
    logits = (torch.randn(2, 5, vocab, generator=g) * 3).to(dtype)
    ids = torch.randint(0, vocab, (2, 5), generator=g)
    xg, idg = logits.to(DEV), ids.to(DEV)
    for mode, scaled in ((NRL_TEMP_DIV, logits / t), (NRL_TEMP_RCP, (logits.float() * (1.0 / torch.tensor(t))).to(dtype))):
        want = OL.rows_logprob(scaled, ids)
        got, lse = torch.ops.rl_amd.logprob_fwd(xg, idg, 5, 0, vocab, t, mode, True)
        assert (got.cpu() - want).abs().max().item() <= 1e-5  # same rounded inputs -> fp32-level agreement


@pytest.mark.parametrize("dtype,vocab", [(torch.float32, 2003), (torch.float32, 4096), (torch.bfloat16, 4099), (torch.float16, 777)])
def test_materialised_log_softmax_and_its_gradient(dtype, vocab):
    """``_compute_distributed_log_softmax[_with_grad]`` (``model_utils.py:33-79``) at TP = 1 against the
    oracle's restatement: values within 1e-5 (fp32) or one unit in the last place of the narrow dtype,
    gradient ``g - softmax * sum(g)`` against torch autograd of the oracle."""
    g = torch.Generator().manual_seed(vocab)
    x = (torch.randn(3, 5, vocab, generator=g) * 2.5).to(dtype)
    up = torch.randn(3, 5, vocab, generator=g).to(dtype)
    xo = x.float().clone().requires_grad_(True)
    want = OL.stable_log_softmax(xo)
    (want * up.float()).sum().backward()
    xg = x.to(DEV).requires_grad_(True)
    got = MU._compute_distributed_log_softmax_with_grad(xg, None)
    assert got.dtype == dtype and got.shape == x.shape
    (got.float() * up.to(DEV).float()).sum().backward()
    gv, wv = got.detach().float().cpu(), want.detach()
    if dtype == torch.float32:
        assert (gv - wv).abs().max().item() <= 1e-5
        scale = xo.grad.abs().max().item()
        assert (xg.grad.cpu() - xo.grad).abs().max().item() <= 1e-4 * scale
    else:
        ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
        assert bool(((gv - wv).abs() <= wv.abs() * ulp + 1e-6).all())
        # the saved output is in the narrow dtype, so softmax = exp(y) carries its rounding (|y| * ulp relative)
        scale = xo.grad.abs().max().item()
        assert (xg.grad.float().cpu() - xo.grad).abs().max().item() <= 20 * ulp * scale
    with torch.no_grad():
        same = MU._compute_distributed_log_softmax(x.to(DEV), None)
    assert torch.equal(same, got.detach()) and not same.requires_grad
    # a view with a padded row stride goes through without a copy of the values changing
    wide = torch.zeros(4, vocab + 8, dtype=dtype)
    wide[:, :vocab] = x[0, :4]
    sl = MU._compute_distributed_log_softmax(wide.to(DEV)[:, :vocab], None)
    assert torch.equal(sl.cpu(), got.detach().cpu()[0, :4])
