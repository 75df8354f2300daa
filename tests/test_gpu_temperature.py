"""Temperature scaling on the GPU: the in-place mirror of ``apply_temperature_scaling``
(``nemo_rl/models/automodel/train.py:180-194``), the same divide fused into the logprob kernels, and the
gradient through it.

The reference divides the logits tensor in place in its own dtype, so both the scaled logit and, through
autograd, the gradient are rounded to that dtype: ``dx = round(round(d) / T)``.  The oracle spells the chain
out on the CPU with torch autograd, once per rounding convention: ``x / T`` (how the CPU divides) and
``x * fp32(1 / T)`` (how a GPU ``div_`` by a scalar is evaluated)."""

import pytest
import torch

from oracle import logprob as OL
from oracle import loss as O
from rl_amd import ops  # noqa: F401
from rl_amd._lib import NRL_TEMP_DIV, NRL_TEMP_RCP
from rl_amd.algorithms.logits_sampling_utils import TrainingSamplingParams
from rl_amd.temperature import apply_temperature_scaling, deferred_temperature, pending_temperature

pytestmark = pytest.mark.gpu
DEV = "cuda"
T = 0.7
MODES = [(NRL_TEMP_DIV, "div"), (NRL_TEMP_RCP, "rcp")]


def _scaled(x, mode):
    """The reference's divide as a differentiable CPU expression in x's dtype."""
    if mode == NRL_TEMP_DIV:
        return x / T
    rcp = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(T, dtype=torch.float32)
    return (x.float() * rcp).to(x.dtype)


def _ulp(dtype):
    return {torch.float32: 2.0 ** -23, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]


def _check_twice_rounded(got, want, dtype):
    """Gradients that went through two roundings to ``dtype``: bit-equal almost everywhere; where the fp32 values
    under the roundings differ in the last bits a result may land one unit of ``dtype`` away."""
    got, want = got.float().cpu(), want.float()
    scale = want.abs().max().item()
    assert scale > 0
    if dtype == torch.float32:
        assert (got - want).abs().max().item() <= 1e-4 * scale
        return
    assert (got == want).float().mean().item() > 0.98
    assert bool(((got - want).abs() <= want.abs() * 2 * _ulp(dtype) + 1e-6 * scale).all())


def _inputs(dtype, vocab, seed, b=2, s=6):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(b, s, vocab, generator=g) * 3).to(dtype)
    ids = torch.randint(0, vocab, (b, s), generator=g)
    up = torch.randn(b, s, generator=g)
    up[0, 1] = 0.0  # a masked row: its gradient row must be exactly zero
    return logits, ids, up


@pytest.mark.parametrize("mode,_name", MODES, ids=[m[1] for m in MODES])
@pytest.mark.parametrize("dtype,vocab", [(torch.bfloat16, 4096), (torch.float16, 2000), (torch.float32, 1003)])
def test_logprob_backward_with_fused_temperature(dtype, vocab, mode, _name):
    logits, ids, up = _inputs(dtype, vocab, 21)
    xo = logits.clone().requires_grad_(True)
    want = OL.rows_logprob(_scaled(xo, mode).float(), ids)
    (want * up).sum().backward()
    xg, idg = logits.to(DEV), ids.to(DEV)
    got, lse = torch.ops.rl_amd.logprob_fwd(xg, idg, ids.shape[1], 0, vocab, T, mode, True)
    assert (got.cpu() - want.detach()).abs().max().item() <= 1e-5
    d = torch.ops.rl_amd.logprob_bwd(xg, idg, lse, up.to(DEV), ids.shape[1], 0, vocab, T, mode)
    _check_twice_rounded(d, xo.grad, dtype)
    assert torch.all(d[0, 1] == 0)


@pytest.mark.parametrize("mode,_name", MODES, ids=[m[1] for m in MODES])
@pytest.mark.parametrize("top_k,top_p", [(50, 0.95), (10, 1.0), (None, 0.9)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_filtered_logprob_backward_with_fused_temperature(dtype, top_k, top_p, mode, _name):
    vocab = 4096
    logits, ids, up = _inputs(dtype, vocab, 33)
    # targets the filter keeps, so that the logprobs are finite and every row has a one-hot term
    ids = logits.float().argmax(-1)
    xo = logits.clone().requires_grad_(True)
    want = OL.rows_logprob_sampled(_scaled(xo, mode).float(), ids, top_k, top_p)
    (want * up).sum().backward()
    xg, idg = logits.to(DEV), ids.to(DEV)
    k = top_k or 0
    lp, thr, tie, lse, _ = torch.ops.rl_amd.topk_topp_logprob_fwd(xg, idg, ids.shape[1], k, top_p, T, mode, False)
    assert (lp.cpu() - want.detach()).abs().max().item() <= 1e-5
    d = torch.ops.rl_amd.topk_topp_logprob_bwd(xg, idg, thr, tie, lse, up.to(DEV), ids.shape[1], T, mode)
    _check_twice_rounded(d, xo.grad, dtype)
    assert torch.all(d[0, 1] == 0)


def _loss_data(b, s, cur, g):
    pad = lambda t: torch.cat([torch.zeros(b, 1), t], 1)  # noqa: E731
    tm = torch.ones(b, s, dtype=torch.int64)
    tm[:, 0] = 0
    tm[0, 2] = 0
    sm = torch.ones(b, dtype=torch.int64)
    data = {"token_mask": tm, "sample_mask": sm, "advantages": torch.randn(b, 1, generator=g).expand(b, s).contiguous(),
            "prev_logprobs": pad(cur + 0.05 * torch.randn(b, s - 1, generator=g)),
            "generation_logprobs": pad(cur + 0.05 * torch.randn(b, s - 1, generator=g)),
            "reference_policy_logprobs": pad(cur + 0.05 * torch.randn(b, s - 1, generator=g))}
    return data, sm.sum().float(), (tm[:, 1:] * sm.unsqueeze(-1)).sum().float()


@pytest.mark.parametrize("mode,_name", MODES, ids=[m[1] for m in MODES])
@pytest.mark.parametrize("dtype,vocab", [(torch.bfloat16, 4096), (torch.bfloat16, 151936), (torch.float32, 2048)])
def test_single_pass_loss_with_fused_temperature(dtype, vocab, mode, _name):
    from rl_amd.algorithms.loss import ClippedPGLossConfig, ClippedPGLossFn
    from rl_amd.algorithms.loss.loss_functions import _f32, _global_valid

    b, s = 2, 6
    logits, ids, _ = _inputs(dtype, vocab, 45, b, s)
    g = torch.Generator().manual_seed(46)
    xo = logits.clone().requires_grad_(True)
    lp = OL.next_token_logprobs(ids, _scaled(xo, mode).float())
    data, gs, gt = _loss_data(b, s, lp.detach(), g)
    data["input_ids"] = ids
    cfg = dict(reference_policy_kl_penalty=0.01)
    want, wm = O.clipped_pg_loss(O.LossConfig(**cfg), lp, data, gs, gt)
    want.backward()
    fn = ClippedPGLossFn(ClippedPGLossConfig(**cfg))
    iflags, fparams = fn._kernel_config(False)
    d = {k: v.to(DEV) for k, v in data.items()}
    loss, dlogits, got_lp, metrics = torch.ops.rl_amd.fused_logits_grpo_loss(
        logits.to(DEV), d["input_ids"][:, 1:], s - 1, _f32(d["prev_logprobs"][:, 1:], DEV),
        _f32(d["generation_logprobs"][:, 1:], DEV), _f32(d["reference_policy_logprobs"][:, 1:], DEV),
        _f32(d["advantages"][:, 1:], DEV), _f32(d["token_mask"][:, 1:], DEV), _f32(d["sample_mask"], DEV),
        _global_valid(gs, gt, DEV), iflags, fparams, 1.0, T, mode)
    assert abs(loss.item() - want.item()) <= 1e-4 * abs(want.item()) + 1e-6
    live = (data["token_mask"][:, 1:] > 0)
    # identical rounded inputs on both sides, so far inside the 2e-3 allowed for 16-bit logits: what is left is the
    # fp32 summation order over the vocabulary (logprobs near -20 at V = 151936)
    assert ((got_lp.cpu() - lp.detach()).abs() * live).max().item() <= (1e-5 if dtype == torch.float32 else 1e-4)
    _check_twice_rounded(dlogits, xo.grad, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(2, 5, 4096), (1, 7, 1003), (3, 640)])
def test_apply_temperature_scaling_is_the_in_place_gpu_divide(dtype, shape):
    """Bit for bit what ``logits.div_(T)`` gives on the GPU (the reference's own statement), in place, returning
    the same tensor; and the same gradient as ``div_`` through a non-leaf tensor."""
    g = torch.Generator().manual_seed(3)
    base = (torch.randn(*shape, generator=g) * 4).to(dtype).to(DEV)
    params = TrainingSamplingParams(top_k=None, top_p=1.0, temperature=T)
    want = base.clone().div_(T)
    x = base.clone()
    out = apply_temperature_scaling(x, params)
    assert out is x and out.data_ptr() == x.data_ptr()
    assert torch.equal(out, want)

    up = torch.randn(*shape, generator=g).to(dtype).to(DEV)
    leaf_a = base.clone().requires_grad_(True)
    (leaf_a * 1).div_(T).mul(up).sum().backward()
    leaf_b = base.clone().requires_grad_(True)
    hidden = leaf_b * 1
    scaled = apply_temperature_scaling(hidden, params)
    assert scaled.data_ptr() == hidden.data_ptr()
    scaled.mul(up).sum().backward()
    assert torch.equal(leaf_b.grad, leaf_a.grad)


def test_apply_temperature_scaling_leaves_logits_alone_without_a_temperature():
    """``tests/unit/models/megatron/test_train.py:170-210``: no sampling params or T = 1 -> untouched."""
    x = torch.randn(2, 3, 64, device=DEV)
    keep = x.clone()
    assert apply_temperature_scaling(x, None) is x and torch.equal(x, keep)
    assert apply_temperature_scaling(x, TrainingSamplingParams(top_k=None, top_p=1.0, temperature=1.0)) is x
    assert torch.equal(x, keep)
    apply_temperature_scaling(x, TrainingSamplingParams(top_k=None, top_p=1.0, temperature=2.0))
    assert torch.equal(x, keep / 2.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_deferred_temperature_matches_the_eager_divide(dtype):
    """Inside ``deferred_temperature()`` the logits stay untouched and the logprob entry points divide in their
    kernels: same logprobs as after the eager in-place divide (the rounded inputs are identical), same
    gradient with respect to the undivided logits up to the two roundings; views of the tensor are
    recognised; readers without a fused temperature refuse."""
    from rl_amd.algorithms.logits_sampling_utils import apply_top_k_top_p
    from rl_amd.distributed.model_utils import get_next_token_logprobs_from_logits

    vocab = 4096
    logits, ids, up = _inputs(dtype, vocab, 61, 2, 8)
    params = TrainingSamplingParams(top_k=None, top_p=1.0, temperature=T)
    up = up[:, :-1].to(DEV)

    leaf_e = logits.to(DEV).requires_grad_(True)
    eager = get_next_token_logprobs_from_logits(ids.to(DEV), apply_temperature_scaling(leaf_e * 1, params))
    (eager * up).sum().backward()

    leaf_d = logits.to(DEV).requires_grad_(True)
    with deferred_temperature():
        hidden = leaf_d * 1
        keep = hidden.detach().clone()
        out = apply_temperature_scaling(hidden, params)
        assert out is hidden and torch.equal(hidden.detach(), keep)
        assert pending_temperature(hidden) == T and pending_temperature(hidden[:, :-1]) == T
        with pytest.raises(RuntimeError, match="not on record"):   # same width, never went through the function
            pending_temperature(leaf_d)
        deferred = get_next_token_logprobs_from_logits(ids.to(DEV), out)
        sliced = get_next_token_logprobs_from_logits(ids[:, :5].to(DEV), out[:, :5])
        with pytest.raises(RuntimeError, match="deferred"):
            apply_top_k_top_p(out, 5, 1.0)
    assert pending_temperature(hidden) == 1.0
    (deferred * up).sum().backward()  # after the context closed: the forward's temperature is what counts
    assert torch.equal(deferred, eager)
    assert torch.equal(sliced, eager[:, :4])
    _check_twice_rounded(leaf_d.grad, leaf_e.grad.cpu(), dtype)

    # top-k / top-p, and the single pass through the workers' wrapper, under the same deferral
    from functools import partial

    from rl_amd.algorithms.loss import ClippedPGLossConfig, ClippedPGLossFn, prepare_loss_input, wrap_loss_fn_with_input_preparation

    filt = TrainingSamplingParams(top_k=50, top_p=0.95, temperature=T)
    want = get_next_token_logprobs_from_logits(ids.to(DEV), apply_temperature_scaling(logits.to(DEV), filt), sampling_params=filt)
    with deferred_temperature():
        x = apply_temperature_scaling(logits.to(DEV), filt)
        got = get_next_token_logprobs_from_logits(ids.to(DEV), x, sampling_params=filt)
    assert torch.equal(got, want)

    g = torch.Generator().manual_seed(62)
    data, gs, gt = _loss_data(2, 8, eager.detach().cpu(), g)
    data["input_ids"] = ids
    ddev = {k: v.to(DEV) for k, v in data.items()}
    fn = ClippedPGLossFn(ClippedPGLossConfig())
    prep = partial(prepare_loss_input, sampling_params=params)
    leaf_1 = logits.to(DEV).requires_grad_(True)
    l1, _ = wrap_loss_fn_with_input_preparation(apply_temperature_scaling(leaf_1 * 1, params), dict(ddev), gs.to(DEV), gt.to(DEV), fn, prep)
    l1.backward()
    leaf_2 = logits.to(DEV).requires_grad_(True)
    with deferred_temperature():
        l2, _ = wrap_loss_fn_with_input_preparation(apply_temperature_scaling(leaf_2 * 1, params), dict(ddev), gs.to(DEV), gt.to(DEV), fn, prep)
    l2.backward()
    assert abs(l1.item() - l2.item()) <= 1e-6 * abs(l1.item()) + 1e-7
    _check_twice_rounded(leaf_2.grad, leaf_1.grad.cpu(), dtype)


def test_a_recycled_address_is_not_divided():
    """The record of a deferred divide ends with the storage it was made for: a tensor that the caching
    allocator places at the address of freed deferred logits has no temperature and its logprobs are those of
    the undivided values."""
    from rl_amd.distributed.model_utils import get_next_token_logprobs_from_logits

    vocab = 4096
    logits, ids, _ = _inputs(torch.bfloat16, vocab, 63, 2, 8)
    params = TrainingSamplingParams(top_k=None, top_p=1.0, temperature=T)
    plain = get_next_token_logprobs_from_logits(ids.to(DEV), logits.to(DEV))
    with deferred_temperature():
        a = apply_temperature_scaling(logits.to(DEV), params)
        address = a.data_ptr()
        assert pending_temperature(a) == T
        divided = get_next_token_logprobs_from_logits(ids.to(DEV), a)
        torch.cuda.synchronize()
        del a
        b = torch.empty_like(logits, device=DEV)          # same size: the allocator hands the freed block back
        b.copy_(logits)
        if b.data_ptr() != address:  # (an allocator configured not to hand a freed block back: nothing to test)
            pytest.skip("the caching allocator did not reuse the freed block")
        assert pending_temperature(b) == 1.0
        again = get_next_token_logprobs_from_logits(ids.to(DEV), b)
    assert torch.equal(again, plain) and not torch.equal(divided, plain)


@pytest.mark.parametrize("what", ["loss", "logprobs", "fused_linear", "foreign"])
def test_megatron_forward_step_leaves_the_divide_to_the_kernels(what):
    """The Megatron worker's forward step scales the model output in place and drops the return value
    (``nemo_rl/models/megatron/train.py:336``); Megatron-Core's schedule then applies the function the step returned
    to that output.  Wrapped by this package, the step of an install (a stand-in here: model call, the scaling, the
    dispatch on the post-processor's type) records the temperature instead, the output keeps its undivided values and
    the returned function divides inside the kernels: same loss, metrics and logprobs as after the in-place divide,
    the gradient equal up to its two roundings.  With ``use_fused_linear_logprobs`` (the output holds logprobs, which
    the reference divides all the same) and for a post-processor that is not this package's the step runs as it is."""
    from rl_amd.algorithms.loss import ClippedPGLossConfig, ClippedPGLossFn
    from rl_amd.models.megatron import train as MT

    dtype, vocab, b, s = torch.bfloat16, 4096, 2, 8
    logits, ids, _ = _inputs(dtype, vocab, 71, b, s)
    params = TrainingSamplingParams(top_k=None, top_p=1.0, temperature=T)
    g = torch.Generator().manual_seed(72)
    base_lp = torch.log_softmax((logits.float() * (1 / T)), -1)[:, :-1].gather(-1, ids[:, 1:, None])[..., 0]
    data, gs, gt = _loss_data(b, s, base_lp, g)
    data["input_ids"] = ids
    ddev = {k: v.to(DEV) for k, v in data.items()}
    cfg = {"sequence_packing": {"enabled": False}}

    class Foreign:  # stands for the install's TopkLogitsPostProcessor: reads the scaled tensor itself
        def __call__(self, data_dict, **kwargs):
            return lambda output: (output.float().sum(), {})

    def post_processor():
        if what == "loss":
            return MT.LossPostProcessor(ClippedPGLossFn(ClippedPGLossConfig()), cfg, sampling_params=params)
        if what == "foreign":
            return Foreign()
        return MT.LogprobsPostProcessor(cfg, sampling_params=params, use_fused_linear_logprobs=what == "fused_linear")

    def install_step(data_iterator, model, post_processing_fn, sampling_params=None, global_valid_seqs=None,
                     global_valid_toks=None, **unused):
        mb = next(data_iterator)
        output = model(mb)
        MT.apply_temperature_scaling(output, sampling_params)  # in place, return value dropped
        if isinstance(post_processing_fn, MT.LossPostProcessor):
            return output, post_processing_fn(data_dict=mb, packed_seq_params=None, global_valid_seqs=global_valid_seqs,
                                              global_valid_toks=global_valid_toks)
        if isinstance(post_processing_fn, MT.LogprobsPostProcessor):
            return output, post_processing_fn(data_dict=mb, input_ids=mb["input_ids"], cu_seqlens_padded=None)
        return output, post_processing_fn(data_dict=mb)

    def run(deferring):
        leaf = logits.to(DEV).requires_grad_(what == "loss")
        post = post_processor()
        step = lambda: install_step(iter([dict(ddev)]), lambda mb: leaf * 1, post, sampling_params=params,  # noqa: E731
                                    global_valid_seqs=gs.to(DEV), global_valid_toks=gt.to(DEV))
        if deferring:
            output, fn = MT._forward_deferring_temperature(post, params, what == "fused_linear", step)
        else:
            output, fn = step()
        raw = output.detach().clone()
        first, second = fn(output)
        if what == "loss":
            first.backward()
        return raw, first, second, leaf.grad

    raw_e, first_e, second_e, grad_e = run(False)
    raw_d, first_d, second_d, grad_d = run(True)
    assert not torch.equal(raw_e, logits.to(DEV))            # the reference's way: the output holds divided values
    if what in ("loss", "logprobs"):
        assert torch.equal(raw_d, logits.to(DEV))            # the output kept its undivided values
    else:
        assert torch.equal(raw_d, raw_e)                     # nothing was put off
    if what == "loss":
        assert abs(first_e.item() - first_d.item()) <= 1e-6 * abs(first_e.item()) + 1e-7
        for k in second_e:
            a, c = float(second_e[k]), float(second_d[k])
            assert abs(a - c) <= 1e-5 * abs(a) + 1e-7, k
        _check_twice_rounded(grad_d, grad_e.cpu(), dtype)
    elif what == "foreign":
        assert torch.equal(first_e, first_d)
    else:
        assert torch.equal(second_e["logprobs"], second_d["logprobs"])
