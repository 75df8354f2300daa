"""GPU parity of the single-pass path (logits -> loss -> dlogits in one kernel) against the
three-kernel HIP path and the CPU oracle.  Tolerances: loss / metrics 1e-4 relative, gradients as in
``test_gpu_logprob.py``."""

import math

import pytest
import torch

from oracle import logprob as OL
from oracle import loss as O
from rl_amd.algorithms.loss import (
    ClippedPGLossConfig,
    ClippedPGLossFn,
    fused_logits_clipped_pg_loss,
    prepare_loss_input,
    why_not_fusable,
    wrap_loss_fn_with_input_preparation,
)

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _batch(b, s, vocab, dtype, seed, float_masks=False):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(b, s, vocab, generator=g) * 2.5).to(dtype)
    ids = torch.randint(0, vocab, (b, s), generator=g)
    cur = OL.next_token_logprobs(ids, logits.float())
    pad = lambda t: torch.cat([torch.zeros(b, 1), t], 1)  # noqa: E731
    tm = torch.zeros(b, s, dtype=torch.float32 if float_masks else torch.int64)
    for i in range(b):
        tm[i, int(torch.randint(1, s - 2, (1,), generator=g)):] = 1
    if b > 2:
        tm[2] = 0
    sm = torch.ones(b, dtype=torch.float32 if float_masks else torch.int64)
    if b > 1:
        sm[1] = 0
    prev = pad(cur + 0.05 * torch.randn(b, s - 1, generator=g))
    data = {"input_ids": ids, "token_mask": tm, "sample_mask": sm,
            "advantages": torch.randn(b, 1, generator=g).expand(b, s).contiguous(), "prev_logprobs": prev,
            "generation_logprobs": pad(cur + 0.05 * torch.randn(b, s - 1, generator=g)),
            "reference_policy_logprobs": pad(cur + 0.05 * torch.randn(b, s - 1, generator=g))}
    gs = sm.sum()
    gt = (tm[:, 1:] * sm.unsqueeze(-1)).sum()
    return logits, data, gs, gt


def _close(a, b, rel=1e-4, abs_=1e-6):
    if math.isinf(a) or math.isinf(b):
        return a == b
    return abs(a - b) <= rel * abs(b) + abs_


FUSABLE = [
    dict(),
    dict(reference_policy_kl_penalty=0.0, ratio_clip_min=0.2, ratio_clip_max=0.28),
    dict(reference_policy_kl_penalty=0.05, reference_policy_kl_type="k2", use_on_policy_kl_approximation=True),
    dict(token_level_loss=False, reference_policy_kl_penalty=0.001),
    dict(ratio_clip_c=3.0, use_importance_sampling_correction=True),
    dict(use_cispo=True),
    dict(disable_ppo_ratio=True),
    dict(force_on_policy_ratio=True),
    dict(use_importance_sampling_correction=True, truncated_importance_sampling_type="tis", truncated_importance_sampling_ratio=1.02),
    dict(use_importance_sampling_correction=True, truncated_importance_sampling_type="seq-mask-tis",
         truncated_importance_sampling_ratio=1.01, truncated_importance_sampling_ratio_min=0.99),
    dict(token_level_loss=False, use_importance_sampling_correction=True, sequence_level_importance_ratios=True,
         disable_ppo_ratio=True),
]


@pytest.mark.parametrize("cfg", FUSABLE, ids=[str(i) for i in range(len(FUSABLE))])
@pytest.mark.parametrize("dtype,vocab", [(torch.float32, 2000), (torch.bfloat16, 4096)])
def test_fused_matches_oracle_and_unfused(cfg, dtype, vocab):
    logits, data, gs, gt = _batch(4, 24, vocab, dtype, seed=len(cfg) + vocab)
    xo = logits.to(torch.float32, copy=True).requires_grad_(True)
    want, wm = O.clipped_pg_loss(O.LossConfig(**cfg), OL.next_token_logprobs(data["input_ids"], xo), data, gs, gt)
    want.backward()

    fn = ClippedPGLossFn(ClippedPGLossConfig(**cfg))
    ddev = {k: v.to(DEV) for k, v in data.items()}
    xg = logits.to(DEV).requires_grad_(True)
    assert why_not_fusable(fn, xg, ddev) is None
    got, gm = fused_logits_clipped_pg_loss(xg, ddev, fn, gs.to(DEV), gt.to(DEV))
    got.backward()
    assert _close(got.item(), want.item()), (got.item(), want.item())
    assert set(gm) == set(wm)
    for k in wm:
        assert _close(float(gm[k]), float(wm[k]), rel=1e-4, abs_=1e-6), (k, gm[k], wm[k])

    xu = logits.to(DEV).requires_grad_(True)
    loss_input, d2 = prepare_loss_input(xu, dict(ddev), fn)
    un, um = fn(data=d2, global_valid_seqs=gs.to(DEV), global_valid_toks=gt.to(DEV), **loss_input)
    un.backward()
    assert _close(got.item(), un.item(), rel=1e-5)
    scale = xo.grad.abs().max().item() + 1e-30
    gf, gu = xg.grad.float().cpu(), xu.grad.float().cpu()
    if dtype == torch.float32:
        assert (gf - xo.grad).abs().max().item() <= 1e-4 * scale
        # the two paths sum the exponentials in different orders; d loss / d logprob amplifies that
        # ulp-level logprob difference wherever the KL term nearly cancels
        assert (gf - gu).abs().max().item() <= 1e-4 * scale
    else:
        ulp = 2.0 ** -8
        assert bool(((gf - xo.grad).abs() <= xo.grad.abs() * (ulp + 1e-4) + 1e-4 * scale * ulp + 1e-30).all())
        assert (gf == gu).float().mean().item() > 0.995
    # masked tokens and the dropped last position receive exactly zero
    mask = (data["token_mask"][:, 1:] * data["sample_mask"].unsqueeze(-1)) != 0
    assert torch.all(gf[:, :-1][~mask] == 0) and torch.all(gf[:, -1] == 0)


def test_fused_rows_with_masked_vocabulary_runs():
    """-inf runs in the logits (start of the row included) leave the single pass finite and equal to
    the three-pass path."""
    logits, data, gs, gt = _batch(3, 17, 6144, torch.bfloat16, seed=77)
    logits[..., :2048] = float("-inf")
    logits[..., 5000:5100] = float("-inf")
    data["input_ids"] = data["input_ids"] % 2000 + 2100
    cur = torch.cat([torch.zeros(3, 1), OL.next_token_logprobs(data["input_ids"], logits.float())], 1)
    for k in ("prev_logprobs", "generation_logprobs", "reference_policy_logprobs"):
        data[k] = cur + 0.03
    fn = ClippedPGLossFn(ClippedPGLossConfig())
    ddev = {k: v.to(DEV) for k, v in data.items()}
    xg = logits.to(DEV).requires_grad_(True)
    got, _ = fused_logits_clipped_pg_loss(xg, ddev, fn, gs.to(DEV), gt.to(DEV))
    got.backward()
    xu = logits.to(DEV).requires_grad_(True)
    loss_input, d2 = prepare_loss_input(xu, dict(ddev), fn)
    un, _ = fn(data=d2, global_valid_seqs=gs.to(DEV), global_valid_toks=gt.to(DEV), **loss_input)
    un.backward()
    assert torch.isfinite(got) and torch.isfinite(xg.grad).all()
    assert _close(got.item(), un.item(), rel=1e-5)
    assert (xg.grad[..., :2048] == 0).all()
    assert (xg.grad.float() == xu.grad.float()).float().mean().item() > 0.995


def test_fused_in_place_and_loss_scale():
    logits, data, gs, gt = _batch(3, 16, 1024, torch.bfloat16, seed=5)
    fn = ClippedPGLossFn(ClippedPGLossConfig())
    ddev = {k: v.to(DEV) for k, v in data.items()}
    x1 = logits.to(DEV).requires_grad_(True)
    l1, _ = fused_logits_clipped_pg_loss(x1, ddev, fn, gs.to(DEV), gt.to(DEV))
    (g1,) = torch.autograd.grad(l1, x1)
    # the upstream gradient is folded in at forward time ...
    x2 = logits.to(DEV).requires_grad_(True)
    l2, _ = fused_logits_clipped_pg_loss(x2, ddev, fn, gs.to(DEV), gt.to(DEV), loss_scale=4.0)
    (g2,) = torch.autograd.grad(l2 * 4.0, x2)
    assert l1.item() == l2.item()
    torch.testing.assert_close(g2.float(), g1.float() * 4.0, rtol=2 ** -7, atol=0)
    # ... or applied afterwards when it was not announced
    x3 = logits.to(DEV).requires_grad_(True)
    l3, _ = fused_logits_clipped_pg_loss(x3, ddev, fn, gs.to(DEV), gt.to(DEV))
    (g3,) = torch.autograd.grad(l3 * 4.0, x3)
    torch.testing.assert_close(g3.float(), g1.float() * 4.0, rtol=2 ** -7, atol=0)
    # in place: the logits buffer ends up holding the gradient
    base = logits.to(DEV)
    leaf = base.clone().requires_grad_(True)
    work = leaf * 1                      # a non-leaf, like a model output
    l4, _ = fused_logits_clipped_pg_loss(work, ddev, fn, gs.to(DEV), gt.to(DEV), in_place=True)
    (g4,) = torch.autograd.grad(l4, leaf)
    assert l4.item() == l1.item() and torch.equal(g4, g1)


def test_unfusable_configs_fall_back_in_the_wrapper():
    logits, data, gs, gt = _batch(3, 12, 512, torch.float32, seed=9)
    ddev = {k: v.to(DEV) for k, v in data.items()}
    gspo = ClippedPGLossFn(ClippedPGLossConfig(token_level_loss=False, sequence_level_importance_ratios=True))
    assert why_not_fusable(gspo, logits.to(DEV), ddev) is not None
    on_policy_seq = ClippedPGLossFn(ClippedPGLossConfig(token_level_loss=False, sequence_level_importance_ratios=True,
                                                        force_on_policy_ratio=True))
    assert why_not_fusable(on_policy_seq, logits.to(DEV), ddev) is not None
    with pytest.raises(NotImplementedError):
        fused_logits_clipped_pg_loss(logits.to(DEV).requires_grad_(True), ddev, gspo, gs, gt)
    for fn in (gspo, ClippedPGLossFn(ClippedPGLossConfig())):
        xw = logits.to(DEV).requires_grad_(True)
        lw, mw = wrap_loss_fn_with_input_preparation(xw, dict(ddev), gs.to(DEV), gt.to(DEV), fn, prepare_loss_input)
        lw.backward()
        xu = logits.to(DEV).requires_grad_(True)
        li, d2 = prepare_loss_input(xu, dict(ddev), fn)
        lu, mu = fn(data=d2, global_valid_seqs=gs.to(DEV), global_valid_toks=gt.to(DEV), **li)
        lu.backward()
        assert _close(lw.item(), lu.item(), rel=1e-5)
        assert set(mw) == set(mu)
        torch.testing.assert_close(xw.grad, xu.grad, rtol=1e-4, atol=1e-9)


@pytest.mark.parametrize("dtype,vocab", [
    (torch.bfloat16, 151936),  # 19 slots of 1024 16-byte vectors: the 16-register-slot instantiation
    (torch.bfloat16, 110000),  # 14 slots: 12 register slots
    (torch.bfloat16, 80000),   # 10 slots: 8 register slots
    (torch.float32, 50256),    # 13 slots: 12 register slots
    (torch.float32, 32000),    # 8 slots: 4 register slots, the last one exactly full
    (torch.float32, 81920),    # the longest fp32 row the on-chip path takes
])
def test_fused_row_lengths(dtype, vocab):
    logits, data, gs, gt = _batch(3, 40, vocab, dtype, seed=1002)
    data["sample_mask"][1] = 1  # more live rows than one pass of a small grid would take in one step
    gs = data["sample_mask"].sum()
    gt = (data["token_mask"][:, 1:] * data["sample_mask"].unsqueeze(-1)).sum()
    fn = ClippedPGLossFn(ClippedPGLossConfig())
    ddev = {k: v.to(DEV) for k, v in data.items()}
    xg = logits.to(DEV).requires_grad_(True)
    got, gm = fused_logits_clipped_pg_loss(xg, ddev, fn, gs.to(DEV), gt.to(DEV))
    got.backward()
    xo = logits.to(torch.float32, copy=True).requires_grad_(True)
    want, wm = O.clipped_pg_loss(O.LossConfig(), OL.next_token_logprobs(data["input_ids"], xo), data, gs, gt)
    want.backward()
    assert _close(got.item(), want.item())
    for k in wm:
        assert _close(float(gm[k]), float(wm[k]), rel=2e-4, abs_=1e-6), (k, gm[k], wm[k])
    scale = xo.grad.abs().max().item()
    err = (xg.grad.float().cpu() - xo.grad).abs()
    if dtype == torch.float32:
        assert err.max().item() <= 1e-4 * scale
    else:  # one narrowing to bf16 on top of the 1e-4
        assert bool((err <= xo.grad.abs() * (2.0 ** -8 + 1e-4) + 1e-4 * scale * 2.0 ** -8 + 1e-30).all())


def _packed_case(lens, pads, width, vocab, dtype, seed, tail=0):
    """Unpacked ``[B, width]`` loss data plus the packed ``[1, T, V]`` logits of the same sequences:
    sequence i holds ``lens[i]`` tokens inside a span of ``lens[i] + pads[i]`` packed positions,
    ``tail`` unused positions follow the last span."""
    b = len(lens)
    g = torch.Generator().manual_seed(seed)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    cup = torch.tensor([0] + list((torch.tensor(lens) + torch.tensor(pads)).cumsum(0)), dtype=torch.int32)
    total = int(cup[-1]) + tail
    logits = (torch.randn(1, total, vocab, generator=g) * 2.5).to(dtype)
    ids = torch.zeros(b, width, dtype=torch.int64)
    tm = torch.zeros(b, width, dtype=torch.int64)
    for i, n in enumerate(lens):
        ids[i, :n] = torch.randint(0, vocab, (n,), generator=g)
        if n > 2:
            tm[i, int(torch.randint(1, n - 1, (1,), generator=g)):n] = 1
    sm = torch.ones(b, dtype=torch.int64)
    if b > 2:
        sm[1] = 0
    targets = OL.pack_input_ids(ids, cu, cup, roll_shift=-1)
    cur = OL.packed_logits_to_logprobs(logits.float()[:, : int(cup[-1])], targets, cup, width, target_is_pre_rolled=True)
    pad = lambda t: torch.cat([torch.zeros(b, 1), t], 1)  # noqa: E731
    noise = lambda: 0.05 * torch.randn(b, width - 1, generator=g)  # noqa: E731
    data = {"input_ids": ids, "token_mask": tm, "sample_mask": sm,
            "advantages": torch.randn(b, 1, generator=g).expand(b, width).contiguous(),
            "prev_logprobs": pad(cur + noise()), "generation_logprobs": pad(cur + noise()),
            "reference_policy_logprobs": pad(cur + noise())}
    gs = sm.sum()
    gt = (tm[:, 1:] * sm.unsqueeze(-1)).sum()
    return logits, data, cu, cup, gs, gt


PACKED_SHAPES = [
    dict(lens=[9, 5, 12, 7], pads=[0, 0, 0, 0], width=12),
    dict(lens=[9, 5, 12, 7], pads=[3, 1, 0, 5], width=14, tail=6),
    dict(lens=[6, 0, 10, 1, 8], pads=[2, 4, 0, 3, 0], width=10),   # an empty and a one-token sequence
]


@pytest.mark.parametrize("cfg", [FUSABLE[0], FUSABLE[2], FUSABLE[3], FUSABLE[7], FUSABLE[9], FUSABLE[10]],
                         ids=["0", "2", "3", "7", "9", "10"])
@pytest.mark.parametrize("shape", PACKED_SHAPES, ids=["tight", "padded", "ragged"])
@pytest.mark.parametrize("dtype,vocab", [(torch.float32, 2000), (torch.bfloat16, 4096)])
def test_fused_packed_matches_oracle_and_three_pass(cfg, shape, dtype, vocab):
    from rl_amd.algorithms.loss import SequencePackingFusionLossWrapper, prepare_packed_loss_input
    from rl_amd.algorithms.loss.fused import fused_packed_logits_clipped_pg_loss, why_not_fusable_packed

    logits, data, cu, cup, gs, gt = _packed_case(vocab=vocab, dtype=dtype, seed=31 + len(cfg) + vocab, **shape)
    width = data["input_ids"].shape[1]
    xo = logits.to(torch.float32, copy=True).requires_grad_(True)
    targets = OL.pack_input_ids(data["input_ids"], cu, cup, roll_shift=-1)
    lp = OL.packed_logits_to_logprobs(xo[:, : int(cup[-1])], targets, cup, width, target_is_pre_rolled=True)
    want, wm = O.clipped_pg_loss(O.LossConfig(**cfg), lp, data, gs, gt)
    want.backward()

    fn = ClippedPGLossFn(ClippedPGLossConfig(**cfg))
    ddev = {k: v.to(DEV) for k, v in data.items()}
    xg = logits.to(DEV).requires_grad_(True)
    assert why_not_fusable_packed(fn, xg, ddev) is None
    got, gm = fused_packed_logits_clipped_pg_loss(xg, ddev, fn, cu.to(DEV), cup.to(DEV), gs.to(DEV), gt.to(DEV))
    got.backward()
    assert _close(got.item(), want.item()), (got.item(), want.item())
    assert set(gm) == set(wm)
    for k in wm:
        assert _close(float(gm[k]), float(wm[k]), rel=1e-4, abs_=1e-6), (k, gm[k], wm[k])

    # the three-pass packed path on the same inputs; the wrapper itself takes the single pass
    xu = logits.to(DEV).requires_grad_(True)
    loss_input, d2 = prepare_packed_loss_input(xu, dict(ddev), fn, cu.to(DEV), cup.to(DEV))
    un, _ = fn(data=d2, global_valid_seqs=gs.to(DEV), global_valid_toks=gt.to(DEV), **loss_input)
    un.backward()
    xw = logits.to(DEV).requires_grad_(True)
    wrapped = SequencePackingFusionLossWrapper(fn, prepare_packed_loss_input, cu.to(DEV), cup.to(DEV))
    lw, mw = wrapped(xw, dict(ddev), gs.to(DEV), gt.to(DEV))
    lw.backward()
    assert lw.item() == got.item() and torch.equal(xw.grad, xg.grad) and set(mw) == set(wm)
    assert _close(got.item(), un.item(), rel=1e-5)

    scale = xo.grad.abs().max().item() + 1e-30
    gf, gu = xg.grad.float().cpu(), xu.grad.float().cpu()
    if dtype == torch.float32:
        assert (gf - xo.grad).abs().max().item() <= 1e-4 * scale
        assert (gf - gu).abs().max().item() <= 1e-4 * scale
    else:
        ulp = 2.0 ** -8
        assert bool(((gf - xo.grad).abs() <= xo.grad.abs() * (ulp + 1e-4) + 1e-4 * scale * ulp + 1e-30).all())
        assert (gf == gu).float().mean().item() > 0.995
    # rows that feed no token (padding inside a span, every sequence's last position, the unused tail,
    # masked tokens) receive exactly zero
    live = torch.zeros(logits.shape[1], dtype=torch.bool)
    w = data["token_mask"][:, 1:] * data["sample_mask"].unsqueeze(-1)
    for i in range(len(cup) - 1):
        n = min(max(int(cup[i + 1] - cup[i]) - 1, 0), width - 1)
        live[int(cup[i]) : int(cup[i]) + n] = w[i, :n] != 0
    assert torch.all(gf[0][~live] == 0)


def test_fused_packed_full_rows():
    """A packed microbatch at a real vocabulary (19 on-chip slots) with more live rows than workgroups."""
    from rl_amd.algorithms.loss import prepare_packed_loss_input
    from rl_amd.algorithms.loss.fused import fused_packed_logits_clipped_pg_loss

    lens = [70, 33, 120, 64, 90, 17, 101, 55]
    logits, data, cu, cup, gs, gt = _packed_case(lens, [2, 7, 0, 0, 6, 7, 3, 1], 128, 151936, torch.bfloat16, seed=8)
    fn = ClippedPGLossFn(ClippedPGLossConfig())
    ddev = {k: v.to(DEV) for k, v in data.items()}
    xg = logits.to(DEV).requires_grad_(True)
    got, gm = fused_packed_logits_clipped_pg_loss(xg, ddev, fn, cu.to(DEV), cup.to(DEV), gs.to(DEV), gt.to(DEV))
    got.backward()
    xu = logits.to(DEV).requires_grad_(True)
    loss_input, d2 = prepare_packed_loss_input(xu, dict(ddev), fn, cu.to(DEV), cup.to(DEV))
    un, um = fn(data=d2, global_valid_seqs=gs.to(DEV), global_valid_toks=gt.to(DEV), **loss_input)
    un.backward()
    assert _close(got.item(), un.item(), rel=1e-5)
    for k in um:
        if k not in ("probs_ratio_min", "probs_ratio_max", "probs_ratio_clamped_min", "probs_ratio_clamped_max"):
            assert _close(float(gm[k]), float(um[k]), rel=1e-4, abs_=1e-6), (k, gm[k], um[k])
    assert (xg.grad.float() == xu.grad.float()).float().mean().item() > 0.995
    lp_want = OL.packed_logits_to_logprobs(logits.float(), OL.pack_input_ids(data["input_ids"], cu, cup, roll_shift=-1),
                                           cup, 128, target_is_pre_rolled=True)
    got_lp = loss_input["next_token_logprobs"].detach().float().cpu()
    assert (got_lp - lp_want).abs().max().item() <= 2e-3


def test_fused_packed_rejects_what_it_cannot_take():
    from rl_amd.algorithms.loss.fused import fused_packed_logits_clipped_pg_loss, why_not_fusable_packed

    logits, data, cu, cup, gs, gt = _packed_case([5, 6], [0, 0], 8, 512, torch.float32, seed=3)
    ddev = {k: v.to(DEV) for k, v in data.items()}
    gspo = ClippedPGLossFn(ClippedPGLossConfig(token_level_loss=False, sequence_level_importance_ratios=True))
    assert why_not_fusable_packed(gspo, logits.to(DEV), ddev) is not None
    with pytest.raises(NotImplementedError):
        fused_packed_logits_clipped_pg_loss(logits.to(DEV).requires_grad_(True), ddev, gspo, cu, cup, gs, gt)
    fn = ClippedPGLossFn(ClippedPGLossConfig())
    with pytest.raises(ValueError):   # boundaries that leave the packed row
        fused_packed_logits_clipped_pg_loss(logits.to(DEV).requires_grad_(True), ddev, fn, cu,
                                            torch.tensor([0, 5, 40], dtype=torch.int32), gs, gt)


def test_step_metrics_hold_the_same_values_as_the_eager_dictionary():
    from rl_amd.algorithms.loss.loss_functions import PendingMetric, StepMetrics

    logits, data, gs, gt = _batch(3, 20, 4096, torch.bfloat16, seed=77)
    ddev = {k: v.to(DEV) for k, v in data.items()}
    fn = ClippedPGLossFn(ClippedPGLossConfig())
    fn.lazy_metrics = False
    eager_loss, eager = fused_logits_clipped_pg_loss(logits.to(DEV).requires_grad_(True), ddev, fn, gs.to(DEV), gt.to(DEV))
    assert type(eager) is dict
    fn.lazy_metrics = True                   # the default
    x = logits.to(DEV).requires_grad_(True)
    lazy_loss, lazy = fused_logits_clipped_pg_loss(x, ddev, fn, gs.to(DEV), gt.to(DEV))
    assert isinstance(lazy, StepMetrics) and isinstance(lazy, dict)
    lazy_loss.backward()                     # more work goes onto the stream before the record is looked at
    torch.ops.rl_amd.logprob_fwd(logits.to(DEV), ddev["input_ids"], 20, 0, 4096, 1.0, 1, False)
    assert lazy == eager and dict(lazy.items()) == eager and lazy_loss.item() == eager_loss.item()
    assert list(lazy) == list(eager) and all(type(v) in (float, int) for v in lazy.values())
    # the three-pass loss returns the same kind of mapping
    loss_input, d2 = prepare_loss_input(logits.to(DEV), dict(ddev), fn)
    _, m3 = fn(data=d2, global_valid_seqs=gs.to(DEV), global_valid_toks=gt.to(DEV), **loss_input)
    assert isinstance(m3, StepMetrics) and set(m3) == set(eager)


def test_the_worker_loop_does_not_wait_for_the_device_between_loss_and_backward(monkeypatch):
    """The DTensor worker divides every metric but the extrema by the number of global batches right after the loss
    call and only then calls ``backward`` (``models/automodel/train.py:525-547``).  With the metrics of a call still on
    their way that loop must not wait for the device: no event or stream synchronisation happens before ``backward``
    is queued, and what is read afterwards is the eager value divided by the same number."""
    from rl_amd.algorithms.loss.loss_functions import PendingMetric

    logits, data, gs, gt = _batch(4, 64, 32768, torch.bfloat16, seed=78)
    ddev = {k: v.to(DEV) for k, v in data.items()}
    gsd, gtd = gs.to(DEV), gt.to(DEV)
    fn = ClippedPGLossFn(ClippedPGLossConfig())
    fn.lazy_metrics = False
    _, eager = fused_logits_clipped_pg_loss(logits.to(DEV).requires_grad_(True), ddev, fn, gsd, gtd)
    fn.lazy_metrics = True
    xs = [logits.to(DEV).requires_grad_(True) for _ in range(3)]
    torch.cuda.synchronize()

    waits = []
    real_event_sync, real_sync = torch.cuda.Event.synchronize, torch.cuda.synchronize
    monkeypatch.setattr(torch.cuda.Event, "synchronize", lambda self: (waits.append("event"), real_event_sync(self))[1])
    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a, **k: (waits.append("device"), real_sync(*a, **k))[1])
    monkeypatch.setattr(torch.Tensor, "item", lambda self: (waits.append("item"), self.tolist())[1])
    num_global_batches = 4
    collected = []
    torch.cuda._sleep(400_000_000)                     # keeps the device busy (about 0.2 s) while the host runs the loop
    from rl_amd.models.automodel.train import LossPostProcessor

    post = LossPostProcessor(fn, {}, None, None, None, 1, 1)   # the DTensor worker's post-processor announces the scaling
    for x in xs:                                       # three microbatches queued back to back
        loss, metrics = post(logits=x, data_dict=ddev, processed_inputs=None, global_valid_seqs=gsd, global_valid_toks=gtd)
        for k in metrics.keys():
            if "_min" in k or "_max" in k:
                continue
            metrics[k] /= num_global_batches
        (loss * 2).backward()
        collected.append(metrics)
    assert waits == [], waits                          # nothing waited while the device was still working
    pending = sum(isinstance(v, PendingMetric) for v in dict.values(collected[-1]))
    monkeypatch.undo()
    assert pending > 0                                 # (the last call's record had indeed not arrived)
    for metrics in collected:
        metrics["lr"] = 1e-5
        assert metrics["num_valid_samples"] > 0
        for k, v in metrics.items():
            if k == "lr":
                continue
            want = eager[k] if ("_min" in k or "_max" in k) else eager[k] / num_global_batches
            assert type(v) in (float, int) and v == want, (k, v, want)
