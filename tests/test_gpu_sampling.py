"""GPU parity: top-k / top-p filtered logprobs (K3) against the CPU oracle.

The oracle filters in fp32 (the training path casts the logits first); tolerances as for the
unfiltered logprobs.  Exact ties at the top-p boundary follow the documented rule (ascending
stable order: larger vocabulary indices survive), which is also what the oracle's stable sort does."""

import math

import pytest
import torch

from oracle import logprob as OL
from oracle import loss as O
from oracle import sampling as OS
from rl_amd.algorithms.logits_sampling_utils import TrainingSamplingParams, apply_top_k_top_p
from rl_amd.algorithms.loss import ClippedPGLossConfig, ClippedPGLossFn, prepare_loss_input
from rl_amd.distributed import model_utils as MU

pytestmark = pytest.mark.gpu
DEV = "cuda"

CASES = [(10, 1.0), (None, 0.9), (10, 0.9), (50, 0.95), (1, 1.0), (300, 0.5), (None, 0.3)]


def _check_grad(got, want_f32, dtype):
    got = got.float().cpu()
    scale = want_f32.abs().max().item() + 1e-30
    if dtype == torch.float32:
        assert (got - want_f32).abs().max().item() <= 1e-4 * scale
    else:
        ulp = 2.0 ** -8
        assert bool(((got - want_f32).abs() <= want_f32.abs() * (ulp + 1e-4) + 1e-4 * scale * ulp + 1e-30).all())


@pytest.mark.parametrize("k,p", CASES)
@pytest.mark.parametrize("dtype,vocab", [(torch.float32, 2003), (torch.bfloat16, 4096)])
def test_sampled_logprob_fwd_bwd_matches_oracle(k, p, dtype, vocab):
    g = torch.Generator().manual_seed(vocab + (k or 0))
    b, s = 2, 7
    logits = (torch.randn(b, s, vocab, generator=g) * 2.5).to(dtype)
    ids = torch.randint(0, vocab, (b, s), generator=g)
    # make most targets likely tokens so that a good share of them survives the filter
    top = logits.float().argmax(-1)
    ids[:, 1:] = torch.where(torch.rand(b, s - 1, generator=g) < 0.7, top[:, :-1], ids[:, 1:])
    up = torch.randn(b, s - 1, generator=g)
    xo = logits.to(torch.float32, copy=True).requires_grad_(True)
    want = OL.from_logits_to_logprobs(xo, ids, top_k=k, top_p=p)
    fin = torch.isfinite(want)
    assert fin.any()
    (torch.where(fin, want, torch.zeros_like(want)) * up).sum().backward()

    xg = logits.to(DEV).requires_grad_(True)
    got = MU.from_parallel_logits_to_logprobs(xg, ids.to(DEV), 0, vocab, None,
                                              sampling_params=TrainingSamplingParams(top_k=k, top_p=p))
    gc = got.cpu()
    assert torch.equal(torch.isfinite(gc), fin)            # the same targets are filtered out
    assert torch.all(gc[~fin] == -math.inf)
    assert (gc[fin] - want.detach()[fin]).abs().max().item() <= (1e-5 if dtype == torch.float32 else 2e-3)
    (torch.where(fin.to(DEV), got, torch.zeros_like(got)) * up.to(DEV)).sum().backward()
    _check_grad(xg.grad, xo.grad, dtype)
    # nothing outside the kept set receives gradient
    keep = OS.keep_mask_rows(logits.float().reshape(-1, vocab), k, p).reshape(b, s, vocab)
    assert torch.all(xg.grad.cpu()[:, :-1][~keep[:, :-1]] == 0)


@pytest.mark.parametrize("k,p", [(10, 1.0), (None, 0.9), (10, 0.9)])
def test_apply_top_k_top_p_standalone(k, p):
    g = torch.Generator().manual_seed(21)
    x = torch.randn(3, 5, 1500, generator=g) * 2
    want_f, want_keep = OS.apply_top_k_top_p(x, k, p)
    xg = x.to(DEV).requires_grad_(True)
    got_f, got_keep = apply_top_k_top_p(xg, k, p)
    assert got_keep.dtype == torch.bool and got_keep.shape == x.shape
    assert torch.equal(got_keep.cpu(), want_keep)
    assert torch.equal(got_f.detach().cpu(), want_f)
    assert torch.equal(got_keep, ~torch.isinf(got_f))
    up = torch.randn(3, 5, 1500, generator=g).to(DEV)
    torch.where(got_keep, got_f, torch.zeros_like(got_f)).mul(up).sum().backward()
    assert torch.equal(xg.grad.cpu(), (up.cpu() * want_keep))
    # switched off: the input comes back untouched
    same, none = apply_top_k_top_p(xg, None, 1.0)
    assert same is xg and none is None


def test_ties_at_the_boundaries():
    vocab = 64
    row = torch.full((vocab,), -5.0)
    row[[3, 17, 40]] = 2.0          # three-way tie for the 2nd..4th largest
    row[9] = 3.0
    x = row.view(1, 1, vocab).repeat(1, 2, 1)
    # top-k = 2 keeps every value tied with the 2nd largest
    _, keep = apply_top_k_top_p(x.to(DEV), 2, 1.0)
    assert sorted(torch.nonzero(keep[0, 0]).flatten().tolist()) == [3, 9, 17, 40]
    # top-p cutting through the tie keeps the larger indices first, like a stable ascending sort
    for p in (0.45, 0.65, 0.85):
        want_f, want_keep = OS.apply_top_k_top_p(x, None, p)
        _, keep = apply_top_k_top_p(x.to(DEV), None, p)
        assert torch.equal(keep.cpu(), want_keep), p


def test_c4_slice_bf16_temperature_topk_topp():
    """benchmark config 4 at reduced rows: V=151936 bf16, T=0.7 (divide in bf16), top_k=50, top_p=0.95."""
    g = torch.Generator().manual_seed(1004)
    vocab, b, s = 151936, 2, 6
    logits = (torch.randn(b, s, vocab, generator=g) * 3).to(torch.bfloat16)
    ids = torch.randint(0, vocab, (b, s), generator=g)
    scaled = (logits.float() * (1.0 / torch.tensor(0.7))).to(torch.bfloat16)   # what the GPU in-place divide yields
    top = scaled.float().argmax(-1)
    ids[:, 1:] = torch.where(torch.rand(b, s - 1, generator=g) < 0.8, top[:, :-1], ids[:, 1:])
    want = OL.from_logits_to_logprobs(scaled.float(), ids, top_k=50, top_p=0.95)
    got = MU.from_parallel_logits_to_logprobs(scaled.to(DEV), ids.to(DEV), 0, vocab, None,
                                              sampling_params=TrainingSamplingParams(top_k=50, top_p=0.95)).cpu()
    fin = torch.isfinite(want)
    assert torch.equal(torch.isfinite(got), fin) and fin.any()
    assert (got[fin] - want[fin]).abs().max().item() <= 2e-3
    # fused temperature at the op level gives the same rows from the unscaled logits
    from rl_amd._lib import NRL_TEMP_RCP

    lp, *_ = torch.ops.rl_amd.topk_topp_logprob_fwd(logits.to(DEV), ids[:, 1:].to(DEV), s - 1, 50, 0.95, 0.7, NRL_TEMP_RCP, False)
    assert torch.equal(lp.cpu(), got)


def test_flat_distribution_under_top_p_alone_fails_loudly():
    x = torch.zeros(1, 2, 151936, device=DEV)   # every token tied: the nucleus is ~144k tokens wide
    ids = torch.zeros(1, 2, dtype=torch.long, device=DEV)
    with pytest.raises(RuntimeError, match="candidate list"):
        MU.from_parallel_logits_to_logprobs(x, ids, 0, 151936, None, sampling_params=TrainingSamplingParams(top_p=0.95))


def test_prepare_loss_input_with_sampling_and_kl():
    """loss/utils.py:97-118 of the reference: filtered logprobs with -inf masked to 0, plus unfiltered
    logprobs for the KL term; end-to-end loss and dlogits against the oracle."""
    g = torch.Generator().manual_seed(31)
    b, s, vocab = 3, 12, 777
    logits = torch.randn(b, s, vocab, generator=g) * 2
    ids = torch.randint(0, vocab, (b, s), generator=g)
    top = logits.argmax(-1)
    ids[:, 1:] = torch.where(torch.rand(b, s - 1, generator=g) < 0.6, top[:, :-1], ids[:, 1:])
    tm = torch.ones(b, s, dtype=torch.int64)
    tm[:, :3] = 0
    data = {"input_ids": ids, "token_mask": tm, "sample_mask": torch.ones(b), "advantages": torch.randn(b, s, generator=g),
            "prev_logprobs": -torch.rand(b, s, generator=g), "generation_logprobs": -torch.rand(b, s, generator=g),
            "reference_policy_logprobs": -torch.rand(b, s, generator=g) * 5}
    gs, gt = torch.tensor(float(b)), (tm[:, 1:]).sum().float()
    k, p = 20, 0.9
    xo = logits.clone().requires_grad_(True)
    lp_f = OL.next_token_logprobs(ids, xo, top_k=k, top_p=p)
    lp_f = OL.mask_out_neg_inf_logprobs(lp_f, (tm[:, 1:] * 1.0))
    lp_u = OL.next_token_logprobs(ids, xo)
    want, wm = O.clipped_pg_loss(O.LossConfig(reference_policy_kl_penalty=0.05), lp_f, {**data, "curr_logprobs_unfiltered": lp_u}, gs, gt)
    want.backward()

    fn = ClippedPGLossFn(ClippedPGLossConfig(reference_policy_kl_penalty=0.05))
    xg = logits.to(DEV).requires_grad_(True)
    ddev = {kk: v.to(DEV) for kk, v in data.items()}
    loss_input, ddev = prepare_loss_input(xg, ddev, fn, sampling_params=TrainingSamplingParams(top_k=k, top_p=p))
    assert "curr_logprobs_unfiltered" in ddev
    got, gm = fn(data=ddev, global_valid_seqs=gs.to(DEV), global_valid_toks=gt.to(DEV), **loss_input)
    got.backward()
    assert abs(got.item() - want.item()) <= 1e-4 * abs(want.item()) + 1e-6
    for kk in wm:
        assert abs(float(gm[kk]) - float(wm[kk])) <= 1e-4 * abs(float(wm[kk])) + 1e-6, kk
    scale = xo.grad.abs().max().item()
    assert (xg.grad.cpu() - xo.grad).abs().max().item() <= 1e-4 * scale


@pytest.mark.parametrize("pre_rolled", [False, True])
def test_packed_sequences_with_sampling(pre_rolled):
    g = torch.Generator().manual_seed(41)
    lens, vocab, smax = [9, 14, 0, 6], 600, 14
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    ids = torch.zeros(len(lens), smax, dtype=torch.int64)
    for i, n in enumerate(lens):
        ids[i, :n] = torch.randint(0, vocab, (n,), generator=g)
    logits = torch.randn(1, int(cu[-1]), vocab, generator=g) * 2
    targets = OL.pack_input_ids(ids, cu, cu, roll_shift=-1 if pre_rolled else 0)
    want = OL.packed_logits_to_logprobs(logits, targets, cu, smax, top_k=15, top_p=0.9, target_is_pre_rolled=pre_rolled)
    got = MU.from_parallel_logits_to_logprobs_packed_sequences(
        logits.to(DEV), targets.to(DEV), cu.to(DEV), smax, 0, vocab, None,
        sampling_params=TrainingSamplingParams(top_k=15, top_p=0.9), target_is_pre_rolled=pre_rolled).cpu()
    fin = torch.isfinite(want)
    assert torch.equal(torch.isfinite(got), fin)
    assert (got[fin] - want[fin]).abs().max().item() <= 1e-5


def test_sampling_autograd_classes():
    g = torch.Generator().manual_seed(51)
    vocab = 999
    x = torch.randn(2, 6, vocab, generator=g) * 2
    t = x.argmax(-1)
    want = OL.rows_logprob_sampled(x, t, 10, 0.9)
    xg = x.to(DEV).requires_grad_(True)
    a = MU.DistributedLogprobWithSampling.apply(xg, t.to(DEV), None, 10, 0.9, False)
    c = MU.ChunkedDistributedLogprobWithSampling.apply(xg, t.to(DEV), None, 10, 0.9, 2, False)
    assert torch.equal(a, c)
    torch.testing.assert_close(a.cpu(), want, rtol=0, atol=1e-5)
    ga, = torch.autograd.grad(a.sum(), xg)
    xo = x.clone().requires_grad_(True)
    OL.rows_logprob_sampled(xo, t, 10, 0.9).sum().backward()
    torch.testing.assert_close(ga.cpu(), xo.grad, rtol=1e-4, atol=1e-6)
