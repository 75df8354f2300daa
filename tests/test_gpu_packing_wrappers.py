"""GPU parity of the two sequence-packing loss wrappers and of the forms in which the policy workers hand
them their ``prepare_fn``.

``SequencePackingLossWrapper`` (one loss call per packed sequence; the default packing path of both
workers) and ``SequencePackingFusionLossWrapper`` (one call for the whole packed row) must agree with each
other and with the oracle on loss, dlogits and the merged metrics: the reference pins fused == unfused, loss
and gradient, to 1e-5 (``tests/unit/algorithms/test_sequence_packing_fusion.py:190-265``), with the lengths
used below."""

import math
from functools import partial

import pytest
import torch

from helpers import packed_grpo_case
from oracle import logprob as OL
from oracle import loss as O
from rl_amd.algorithms.logits_sampling_utils import TrainingSamplingParams
from rl_amd.algorithms.loss import (
    ClippedPGLossConfig,
    ClippedPGLossFn,
    SequencePackingFusionLossWrapper,
    SequencePackingLossWrapper,
    prepare_loss_input,
    prepare_packed_loss_input,
    wrap_loss_fn_with_input_preparation,
)

pytestmark = pytest.mark.gpu
DEV = "cuda"
EXTREMA = ("probs_ratio_min", "probs_ratio_max", "probs_ratio_clamped_min", "probs_ratio_clamped_max")


def _close(a, b, rel=1e-4, abs_=1e-6):
    if math.isinf(a) or math.isinf(b):
        return a == b
    return abs(a - b) <= rel * abs(b) + abs_


def _to_dev(data):
    return {k: v.to(DEV) for k, v in data.items()}


def _oracle(cfg, logits, data, cu, cup, gs, gt):
    xo = logits.to(torch.float32, copy=True).requires_grad_(True)
    want, wm = O.sequence_packing_loss(O.LossConfig(**cfg), xo, data, cu, cup, gs, gt, OL.next_token_logprobs)
    want.backward()
    return want, wm, xo.grad


def _check_grad(got, want, dtype):
    scale = want.abs().max().item() + 1e-30
    got = got.float().cpu()
    if dtype == torch.float32:
        # the reference's own bound for fused == unfused: atol = rtol = 1e-5
        assert bool(((got - want).abs() <= 1e-5 + 1e-5 * want.abs()).all()), (got - want).abs().max().item()
        assert (got - want).abs().max().item() <= 1e-4 * scale
    else:
        ulp = 2.0 ** -8
        assert bool(((got - want).abs() <= want.abs() * (ulp + 1e-4) + 1e-4 * scale * ulp + 1e-30).all())


CASES = {
    # the reference test's lengths at max_seq_len 512 (128, 256, 170, 384), spans padded to multiples of 8 so that
    # cu_seqlens_q_padded != cu_seqlens_q
    "reference_lengths": dict(lens=[128, 256, 170, 384], pads=[0, 0, 6, 0], width=512, vocab=512),
    # a sequence without any valid token (its extrema are the +-inf sentinels the merge must skip), a sequence
    # whose sample is masked out, an empty and a one-token sequence, unused positions behind the last span
    "ragged": dict(lens=[9, 5, 12, 0, 1, 7], pads=[3, 1, 0, 2, 3, 5], width=14, vocab=640, tail=6,
                   empty_mask_rows=(1,), dead_rows=(2,)),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("cfg", [dict(), dict(token_level_loss=False, reference_policy_kl_penalty=0.001),
                                 dict(reference_policy_kl_penalty=0.0, ratio_clip_min=0.2, ratio_clip_max=0.28)],
                         ids=["default", "sequence_level_kl", "dapo"])
@pytest.mark.parametrize("case", list(CASES), ids=list(CASES))
def test_per_sequence_wrapper_fused_wrapper_and_oracle_agree(case, cfg, dtype):
    spec = CASES[case]
    logits, data, cu, cup, gs, gt = packed_grpo_case(dtype=dtype, seed=77, float_masks=(case == "reference_lengths"),
                                                     **spec)
    want, wm, want_grad = _oracle(cfg, logits, data, cu, cup, gs, gt)
    fn = ClippedPGLossFn(ClippedPGLossConfig(**cfg))
    ddev = _to_dev(data)

    x1 = logits.to(DEV).requires_grad_(True)
    unfused = SequencePackingLossWrapper(fn, prepare_loss_input, cu.to(DEV), cup.to(DEV))
    l1, m1 = unfused(x1, dict(ddev), gs.to(DEV), gt.to(DEV))
    l1.backward()

    x2 = logits.to(DEV).requires_grad_(True)
    fused = SequencePackingFusionLossWrapper(fn, prepare_packed_loss_input, cu.to(DEV), cup.to(DEV))
    l2, m2 = fused(x2, dict(ddev), gs.to(DEV), gt.to(DEV))
    l2.backward()

    assert x1.grad.abs().sum().item() > 0 and x2.grad.abs().sum().item() > 0
    tol = 1e-5 if dtype == torch.float32 else 1e-4
    assert abs(l1.item() - l2.item()) <= tol + tol * abs(l2.item()), (l1.item(), l2.item())
    assert abs(l1.item() - want.item()) <= tol + tol * abs(want.item()), (l1.item(), want.item())
    _check_grad(x1.grad[0], want_grad[0], dtype)
    _check_grad(x2.grad[0], want_grad[0], dtype)
    if dtype == torch.float32:
        assert bool(((x1.grad - x2.grad).abs() <= 1e-5 + 1e-5 * x2.grad.abs()).all())

    # merged metrics of the per-sequence wrapper against the oracle's merge (sums, and min / max that skip the
    # infinite sentinels of sequences without valid tokens)
    assert set(m1) == set(wm)
    for k in wm:
        assert _close(float(m1[k]), float(wm[k]), rel=2e-4, abs_=2e-6), (k, m1[k], wm[k])
    # the one-call wrapper reports the same extrema and the same additive metrics wherever per-sequence sums and
    # the whole-batch value coincide (everything normalised by the global counts)
    for k in EXTREMA + ("loss", "probs_ratio", "probs_ratio_clamped", "token_mult_prob_error", "approx_entropy"):
        assert _close(float(m2[k]), float(m1[k]), rel=2e-4, abs_=2e-6), (k, m2[k], m1[k])
    if case == "ragged":
        assert all(math.isfinite(float(m1[k])) for k in EXTREMA)


def test_per_sequence_wrapper_keeps_sentinels_when_no_sequence_has_valid_tokens():
    logits, data, cu, cup, gs, gt = packed_grpo_case([6, 4], [2, 0], 8, 256, torch.float32, seed=5, empty_mask_rows=(0, 1))
    fn = ClippedPGLossFn(ClippedPGLossConfig())
    x = logits.to(DEV).requires_grad_(True)
    loss, m = SequencePackingLossWrapper(fn, prepare_loss_input, cu.to(DEV), cup.to(DEV))(
        x, _to_dev(data), gs.to(DEV), torch.ones((), device=DEV))
    assert loss.item() == 0.0
    assert m["probs_ratio_min"] == float("inf") and m["probs_ratio_max"] == float("-inf")
    assert m["probs_ratio_clamped_min"] == float("inf") and m["probs_ratio_clamped_max"] == float("-inf")


def _count_calls(monkeypatch, name):
    import rl_amd.algorithms.loss.fused as F

    calls = []
    real = getattr(F, name)

    def counted(*a, **k):
        calls.append(1)
        return real(*a, **k)

    monkeypatch.setattr(F, name, counted)
    return calls


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_prepare_fn_bound_like_the_workers_reaches_the_single_pass(monkeypatch, dtype):
    """The Megatron worker binds ``prepare_loss_input`` with ``functools.partial(sampling_params=, d2t=,
    chunk_size=)`` (``models/megatron/train.py:506-513``), the DTensor worker with ``sampling_params=`` only
    (``models/automodel/train.py:624-627``).  Both forms must take the single pass and agree with the
    three-pass path spelled out."""
    from helpers import synthetic_grpo_batch

    w = synthetic_grpo_batch(2, 3, 40, 4096, seed=9, logits_dtype=dtype)
    b, s = w["input_ids"].shape
    g = w["generator"]
    data = {"input_ids": w["input_ids"], "token_mask": w["token_mask"], "sample_mask": w["sample_mask"],
            "advantages": torch.randn(b, 1, generator=g).expand(b, s).contiguous(),
            "prev_logprobs": -3 + 0.3 * torch.randn(b, s, generator=g),
            "generation_logprobs": -3 + 0.3 * torch.randn(b, s, generator=g),
            "reference_policy_logprobs": -3 + 0.3 * torch.randn(b, s, generator=g)}
    gs = w["sample_mask"].sum().to(DEV)
    gt = (w["token_mask"][:, 1:] * w["sample_mask"].unsqueeze(-1)).sum().float().to(DEV)
    fn = ClippedPGLossFn(ClippedPGLossConfig())
    ddev = _to_dev(data)
    params = TrainingSamplingParams(top_k=None, top_p=1.0, temperature=1.0)

    x3 = w["logits"].to(DEV).requires_grad_(True)
    loss_input, d3 = prepare_loss_input(x3, dict(ddev), fn, sampling_params=params, chunk_size=16)
    l3, m3 = fn(data=d3, global_valid_seqs=gs, global_valid_toks=gt, **loss_input)
    l3.backward()

    calls = _count_calls(monkeypatch, "fused_logits_clipped_pg_loss")
    for bound in (partial(prepare_loss_input, sampling_params=params, d2t=None, chunk_size=16),
                  partial(prepare_loss_input, sampling_params=params),
                  partial(prepare_loss_input, sampling_params=None, d2t=None, chunk_size=None)):
        n = len(calls)
        x = w["logits"].to(DEV).requires_grad_(True)
        l, m = wrap_loss_fn_with_input_preparation(x, dict(ddev), gs, gt, fn, bound, vocab_parallel_rank=0,
                                                   vocab_parallel_group=None, context_parallel_group=None)
        l.backward()
        assert len(calls) == n + 1, "the bound prepare_fn did not reach the single pass"
        assert _close(l.item(), l3.item(), rel=1e-5)
        for k in m3:
            if k not in EXTREMA:
                assert _close(float(m[k]), float(m3[k]), rel=1e-4, abs_=1e-6), (k, m[k], m3[k])
        if dtype == torch.float32:
            assert (x.grad - x3.grad).abs().max().item() <= 1e-4 * x3.grad.abs().max().item()
        else:
            assert (x.grad == x3.grad).float().mean().item() > 0.995
    # filtering, a draft-token map or a foreign prepare_fn keep the general path
    n = len(calls)
    for bound in (partial(prepare_loss_input, sampling_params=TrainingSamplingParams(top_k=5, top_p=1.0, temperature=1.0)),
                  partial(prepare_loss_input, d2t=torch.zeros(1)),
                  lambda **kw: prepare_loss_input(**kw)):
        if isinstance(bound, partial) and bound.keywords.get("d2t") is not None:
            continue  # LossInputType.DRAFT is not built; only the dispatch matters here
        x = w["logits"].to(DEV).requires_grad_(True)
        wrap_loss_fn_with_input_preparation(x, dict(ddev), gs, gt, fn, bound)
    assert len(calls) == n


def test_packed_prepare_fn_bound_like_the_megatron_worker_reaches_the_single_pass(monkeypatch):
    """``partial(prepare_packed_loss_input, sampling_params=, chunk_size=)`` as in ``models/megatron/train.py:529-533``."""
    logits, data, cu, cup, gs, gt = packed_grpo_case([9, 5, 12, 7], [3, 1, 0, 5], 14, 2048, torch.bfloat16, seed=3)
    fn = ClippedPGLossFn(ClippedPGLossConfig(token_level_loss=False, reference_policy_kl_penalty=0.001))
    ddev = _to_dev(data)
    calls = _count_calls(monkeypatch, "fused_packed_logits_clipped_pg_loss")
    bound = partial(prepare_packed_loss_input, sampling_params=TrainingSamplingParams(top_k=None, top_p=1.0, temperature=0.7),
                    chunk_size=1024)
    x = logits.to(DEV).requires_grad_(True)
    l, m = SequencePackingFusionLossWrapper(fn, bound, cu.to(DEV), cup.to(DEV), 0, None, None)(x, dict(ddev), gs.to(DEV), gt.to(DEV))
    l.backward()
    assert len(calls) == 1
    xu = logits.to(DEV).requires_grad_(True)
    loss_input, d2 = bound(logits=xu, data=dict(ddev), loss_fn=fn, cu_seqlens_q=cu.to(DEV), cu_seqlens_q_padded=cup.to(DEV))
    lu, _ = fn(data=d2, global_valid_seqs=gs.to(DEV), global_valid_toks=gt.to(DEV), **loss_input)
    lu.backward()
    assert _close(l.item(), lu.item(), rel=1e-5)
    assert (x.grad == xu.grad).float().mean().item() > 0.995


@pytest.mark.parametrize("factor", [1.0, 3.0, 0.37])
def test_upstream_gradient_other_than_the_loss_scale_is_applied_on_the_device(factor):
    """``loss * factor`` after the loss returned (what both workers do, ``models/automodel/train.py:547``,
    ``models/megatron/train.py:590-592``): the gradient the single pass has already written is rescaled in
    place by the factor autograd delivers, whatever it is."""
    from helpers import synthetic_grpo_batch
    from rl_amd.algorithms.loss import fused_logits_clipped_pg_loss

    w = synthetic_grpo_batch(2, 2, 24, 2048, seed=4, logits_dtype=torch.float32)
    b, s = w["input_ids"].shape
    g = w["generator"]
    data = {"input_ids": w["input_ids"], "token_mask": w["token_mask"], "sample_mask": w["sample_mask"],
            "advantages": torch.randn(b, s, generator=g), "prev_logprobs": -3 + 0.3 * torch.randn(b, s, generator=g),
            "generation_logprobs": -3 + 0.3 * torch.randn(b, s, generator=g),
            "reference_policy_logprobs": -3 + 0.3 * torch.randn(b, s, generator=g)}
    gs = w["sample_mask"].sum()
    gt = (w["token_mask"][:, 1:] * w["sample_mask"].unsqueeze(-1)).sum().float()
    xo = w["logits"].clone().requires_grad_(True)
    want, _ = O.clipped_pg_loss(O.LossConfig(), OL.next_token_logprobs(data["input_ids"], xo), data, gs, gt)
    (want * factor).backward()
    fn = ClippedPGLossFn(ClippedPGLossConfig())
    x = w["logits"].to(DEV).requires_grad_(True)
    loss, _ = fused_logits_clipped_pg_loss(x, _to_dev(data), fn, gs.to(DEV), gt.to(DEV))
    (loss * factor).backward()
    assert (x.grad.cpu() - xo.grad).abs().max().item() <= 1e-4 * xo.grad.abs().max().item()
    with pytest.raises(RuntimeError, match="once"):
        x2 = w["logits"].to(DEV).requires_grad_(True)
        loss2, _ = fused_logits_clipped_pg_loss(x2, _to_dev(data), fn, gs.to(DEV), gt.to(DEV))
        loss2.backward(retain_graph=True)
        loss2.backward()


def test_megatron_loss_post_processor_counteracts_the_schedule_averaging():
    """The mirror of the Megatron worker's ``LossPostProcessor`` (``models/megatron/train.py:442-597``) on one
    GPU: loss and gradient are ``num_microbatches`` times the plain ones, packed (both wrappers) and unpacked."""
    from rl_amd.models.megatron.train import LossPostProcessor

    class Packed:
        def __init__(self, cu, cup):
            self.cu_seqlens_q, self.cu_seqlens_q_padded = cu, cup

    logits, data, cu, cup, gs, gt = packed_grpo_case([9, 5, 12, 7], [3, 1, 0, 5], 14, 1024, torch.float32, seed=21)
    cfg = dict(reference_policy_kl_penalty=0.01)
    want, _, want_grad = _oracle(cfg, logits, data, cu, cup, gs, gt)
    fn = ClippedPGLossFn(ClippedPGLossConfig(**cfg))
    for fuse in (False, True):
        post = LossPostProcessor(fn, {"sequence_packing": {"enabled": True, "fuse_loss": fuse}, "logprob_chunk_size": None},
                                 num_microbatches=3)
        x = logits.to(DEV).requires_grad_(True)
        loss, _ = post(_to_dev(data), Packed(cu.to(DEV), cup.to(DEV)), gs.to(DEV), gt.to(DEV))(x)
        loss.backward()
        assert _close(loss.item(), 3 * want.item(), rel=1e-5)
        assert (x.grad.cpu() - 3 * want_grad).abs().max().item() <= 1e-4 * 3 * want_grad.abs().max().item()


@pytest.mark.parametrize("roll", [0, -1, 1, -5])
@pytest.mark.parametrize("cu_on_gpu", [True, False])
def test_device_id_packing_matches_the_oracle(roll, cu_on_gpu):
    """The packing kernel (ids [B, S] -> one packed row, rolled inside every padded span, read from boundaries that
    stay on the device) against the oracle's loop per sequence: padded spans, an empty sequence, a recorded length
    beyond the row width, a first boundary above zero and packed rows longer than the last boundary."""
    from oracle import logprob as OLP

    g = torch.Generator().manual_seed(3)
    ids = torch.randint(1, 50, (4, 12), generator=g)
    cases = [
        (ids, [0, 5, 17, 17, 26], [0, 8, 24, 24, 36], 36),
        (ids, [0, 5, 17, 17, 26], [0, 8, 24, 24, 36], 50),
        (ids[:2], [0, 5, 20], [0, 8, 24], 24),
        (ids[:3], [3, 9, 9, 21], [4, 12, 12, 24], 31),
        (ids[:1], [0, 1], [0, 1], 1),
    ]
    for rows, cu, cup, total in cases:
        cu_t, cup_t = torch.tensor(cu), torch.tensor(cup)
        want = OLP.pack_input_ids(rows, cu_t, cup_t, roll_shift=roll).reshape(-1)
        want = torch.nn.functional.pad(want, (0, total - want.numel()))
        where = DEV if cu_on_gpu else "cpu"
        got = torch.ops.rl_amd.pack_input_ids(rows.to(DEV), cu_t.to(DEV, torch.int32), cup_t.to(DEV, torch.int32), roll, total)
        assert torch.equal(got.cpu(), want), (cu, cup, total)
        if roll == -1:
            from rl_amd.algorithms.loss.utils import _packed_targets

            via = _packed_targets(rows.to(DEV), cu_t.to(where), cup_t.to(where), total, torch.device(DEV))
            assert via.shape == (1, total) and torch.equal(via.cpu().reshape(-1), want)
