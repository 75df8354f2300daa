"""Clipped policy-gradient loss (GRPO / PPO-clip / DAPO clip-higher / REINFORCE / GSPO / CISPO)
and the NLL loss, computed by the fused HIP loss kernel.

Counterpart of ``nemo_rl/algorithms/loss/loss_functions.py:111-842``: same configuration fields,
constructor checks, call signature, returned metrics and ``metric_normalizations`` table.  One
call is two kernel launches and one device->host copy of the metrics record, instead of a few
dozen element-wise kernels and a synchronisation per metric.
"""

from __future__ import annotations

from typing import Any, Optional

import torch
from pydantic import BaseModel

from ... import ops as _ops  # noqa: F401
from ..._lib import METRIC_SLOTS, NRL_TIS
from .interfaces import LossFunction, LossInputType, LossType, MetricNormalizer

_OPS = torch.ops.rl_amd
_KL_TYPES = {"k1": 1, "k2": 2, "k3": 3}


class ClippedPGLossConfig(BaseModel, extra="allow"):
    """Field names and defaults of the reference configuration (``loss_functions.py:111-164``)."""

    disable_ppo_ratio: bool = False
    token_level_loss: bool = True
    sequence_level_importance_ratios: bool = False
    ratio_clip_min: float = 0.2
    ratio_clip_max: float = 0.2
    ratio_clip_c: Optional[float] = None
    reference_policy_kl_penalty: float = 0.01
    reference_policy_kl_type: str = "k3"
    kl_input_clamp_value: Optional[float] = 20.0
    kl_output_clamp_value: Optional[float] = 10.0
    use_kl_in_reward: bool = False
    use_importance_sampling_correction: bool = False
    truncated_importance_sampling_type: Optional[str] = None
    truncated_importance_sampling_ratio: Optional[float] = None
    truncated_importance_sampling_ratio_min: Optional[float] = None
    use_on_policy_kl_approximation: bool = False
    force_on_policy_ratio: bool = False
    use_cispo: bool = False
    positive_example_nll_weight: float = 0.0


def _gpu_for(t: torch.Tensor) -> torch.device:
    if t.is_cuda:
        return t.device
    if not torch.cuda.is_available():
        raise RuntimeError("rl_amd needs an MI355X: no GPU is visible and there is no CPU fallback")
    return torch.device("cuda", torch.cuda.current_device())


def _f32(t, dev):
    return t.to(device=dev, dtype=torch.float32)


def _global_valid(seqs, toks, dev) -> torch.Tensor:
    parts = []
    for v in (seqs, toks):
        if isinstance(v, torch.Tensor):
            parts.append(v.detach().reshape(()).to(device=dev, dtype=torch.float32))
        else:
            parts.append(torch.tensor(float(v), dtype=torch.float32, device=dev))
    return torch.stack(parts)


class PendingMetric:
    """One value of a ``StepMetrics`` mapping whose record has not been read yet.

    It stands for ``record[key]`` times the factors it has been multiplied or divided by since: ``value / n`` and
    ``value * n`` with a plain number give another ``PendingMetric`` and touch nothing (that is what the DTensor
    worker does to every metric right after the loss call, ``models/automodel/train.py:525-533``); every other use
    -- ``float()``, comparison, addition, formatting, pickling -- waits for the record and continues with the
    ``float``."""

    __slots__ = ("_owner", "_key", "_steps")

    def __init__(self, owner, key, steps=()):
        self._owner, self._key, self._steps = owner, key, steps

    def _value(self):
        v = self._owner._resolve()[self._key]
        for divide, n in self._steps:
            v = v / n if divide else v * n
        return v

    def _scaled(self, divide, n):
        if type(n) in (int, float):
            return PendingMetric(self._owner, self._key, self._steps + ((divide, n),))
        return self._value() / n if divide else self._value() * n

    def __truediv__(self, n): return self._scaled(True, n)
    def __mul__(self, n): return self._scaled(False, n)
    __rmul__ = __mul__
    def __rtruediv__(self, n): return n / self._value()
    def __add__(self, o): return self._value() + o
    def __radd__(self, o): return o + self._value()
    def __sub__(self, o): return self._value() - o
    def __rsub__(self, o): return o - self._value()
    def __neg__(self): return -self._value()
    def __pos__(self): return self._value()
    def __abs__(self): return abs(self._value())
    def __pow__(self, o): return self._value() ** o
    def __float__(self): return float(self._value())
    def __int__(self): return int(self._value())
    def __bool__(self): return bool(self._value())
    def __round__(self, n=None): return round(self._value(), n)
    def __eq__(self, o): return self._value() == o
    def __ne__(self, o): return self._value() != o
    def __lt__(self, o): return self._value() < o
    def __le__(self, o): return self._value() <= o
    def __gt__(self, o): return self._value() > o
    def __ge__(self, o): return self._value() >= o
    def __hash__(self): return hash(self._value())
    def __repr__(self): return repr(self._value())
    def __str__(self): return str(self._value())
    def __format__(self, spec): return format(self._value(), spec)
    def __reduce__(self):
        v = self._value()
        return (type(v), (v,))


class StepMetrics(dict):
    """The metrics of a loss call: a ``dict`` whose values arrive from the device behind the stream.

    The reference ends every loss call with about fifteen ``.item()`` calls, each of which stalls the host until
    the device has caught up.  Here the 24-float record of a call travels to pinned host memory behind the kernels
    and the host waits for it only when a value is first needed: ``metrics[key]``, ``items()``, ``values()``,
    ``get()``, ``pop()``, ``copy()``, ``repr()``, comparison, ``json.dumps`` and pickling all wait once, and from then
    on the mapping holds plain numbers.  A Megatron worker reads its metrics after ``forward_backward_func`` has
    returned, by when the records have long arrived, so it never waits.

    The DTensor worker does touch them earlier: ``metrics[k] /= num_global_batches`` between the loss call and
    ``backward()`` (``models/automodel/train.py:525-547``).  For that caller, which the ``LossPostProcessor`` of that
    worker's mirror announces with ``defer_scaling()``, ``metrics[key]`` hands out a ``PendingMetric`` while the record
    is still on its way and ``metrics[key] = ...`` stores whatever it is given, so the division is recorded instead of
    waited for and the backward pass and the next microbatch are queued while the device is still busy.  Without
    that announcement every value that leaves the mapping is a plain number, whatever the timing.
    ``loss_fn.lazy_metrics = False`` gives a plain ``dict`` filled before the call returns instead."""

    def __init__(self, keys, fetch):
        super().__init__()
        self._fetch = fetch
        self._record = None
        self._pending_ok = False
        for key in keys:
            dict.__setitem__(self, key, PendingMetric(self, key))

    def defer_scaling(self):
        """From now on ``metrics[key]`` may hand out a ``PendingMetric`` (see the class text).  Returns ``self``."""
        self._pending_ok = True
        return self

    def _resolve(self) -> dict:
        if self._record is None:
            self._record = self._fetch()
            self._fetch = None
            for key, value in list(dict.items(self)):
                if isinstance(value, PendingMetric):
                    dict.__setitem__(self, key, value._value())
        return self._record

    def _settle(self, wait: bool):
        if self._record is None and (wait or self._fetch.ready()):
            self._resolve()

    def __getitem__(self, key):
        self._settle(not self._pending_ok)
        return dict.__getitem__(self, key)

    def __setitem__(self, key, value):
        if isinstance(value, PendingMetric) and self._record is not None:
            value = value._value()
        dict.__setitem__(self, key, value)

    def items(self): self._settle(True); return dict.items(self)
    def values(self): self._settle(True); return dict.values(self)
    def get(self, key, default=None): self._settle(True); return dict.get(self, key, default)
    def pop(self, *args): self._settle(True); return dict.pop(self, *args)
    def popitem(self): self._settle(True); return dict.popitem(self)
    def setdefault(self, key, default=None): self._settle(True); return dict.setdefault(self, key, default)
    def copy(self): self._settle(True); return dict(dict.items(self))
    def __iter__(self): self._settle(not self._pending_ok); return dict.__iter__(self)   # (dict(metrics) comes this way)
    def __eq__(self, other): self._settle(True); return dict.__eq__(self, other)
    def __ne__(self, other): self._settle(True); return dict.__ne__(self, other)
    def __or__(self, other): self._settle(True); return dict.__or__(dict(dict.items(self)), other)
    def __repr__(self): self._settle(True); return dict.__repr__(self)
    def __reduce_ex__(self, protocol): self._settle(True); return (dict, (dict(dict.items(self)),))
    __hash__ = None


def fetch_later(record: torch.Tensor):
    """Starts the copy of a small device record to pinned host memory on the current stream and returns a function
    that waits for that copy alone (not for work enqueued afterwards) and yields the values as a list; its
    ``ready()`` says without waiting whether the copy has arrived."""
    if not record.is_cuda:
        values = record.tolist
        fetch = lambda: values()  # noqa: E731
        fetch.ready = lambda: True
        return fetch
    host = torch.empty(record.shape, dtype=record.dtype, pin_memory=True)
    host.copy_(record, non_blocking=True)
    done = torch.cuda.Event()
    done.record()

    def fetch():
        if not done.query():
            done.synchronize()
        return host.tolist()

    fetch.ready = done.query
    return fetch


def metrics_record_to_dict(metrics: torch.Tensor, loss_fn, sample_mask_in: torch.Tensor) -> dict:
    """The kernels' metrics record -> the dictionary ``ClippedPGLossFn`` returns (``loss_functions.py:767-788``).
    Fetching the record is the one device -> host wait of a loss call; it is put off until the values are needed
    (``StepMetrics``) unless ``loss_fn.lazy_metrics`` is switched off."""
    beta = loss_fn.reference_policy_kl_penalty
    with_oob = loss_fn.truncated_importance_sampling_ratio is not None
    as_float = sample_mask_in.is_floating_point()
    values = fetch_later(metrics)
    keys = ["loss", "probs_ratio", "probs_ratio_clamped", "probs_ratio_min", "probs_ratio_max", "probs_ratio_clamped_min",
            "probs_ratio_clamped_max", "kl_penalty", "token_mult_prob_error", "gen_kl_error", "policy_kl_error",
            "js_divergence_error", "sampling_importance_ratio", "num_valid_samples", "approx_entropy"]
    if with_oob:
        keys.append("is_oob_ratio")
    keys.append("positive_nll_loss")

    def build():
        m = values()
        get = lambda name: m[METRIC_SLOTS[name]]  # noqa: E731
        out = {key: get(key) for key in keys if key not in ("kl_penalty", "num_valid_samples")}
        out["kl_penalty"] = get("kl") / beta if (beta != 0 and get("kl") != 0) else 0
        n_valid = get("num_valid_samples")
        out["num_valid_samples"] = n_valid if as_float else int(n_valid)
        return {key: out[key] for key in keys}

    build.ready = values.ready
    return StepMetrics(keys, build) if getattr(loss_fn, "lazy_metrics", True) else build()


class _FusedLoss(torch.autograd.Function):
    """loss, metrics = kernel(lp, lpu, ...); the kernel also returns d loss / d lp (and / d lpu), so the
    backward is a scalar multiply."""

    @staticmethod
    def forward(ctx, lp, lpu, prev, gen, ref, adv, token_mask, sample_mask, correct, global_valid, iflags, fparams):
        loss, dlp, dlpu, metrics = _OPS.grpo_loss(
            lp.detach(), None if lpu is None else lpu.detach(), prev, gen, ref, adv, token_mask, sample_mask, correct,
            global_valid, iflags, fparams,
        )
        ctx.save_for_backward(dlp, dlpu)
        ctx.has_lpu = lpu is not None and dlpu.numel() > 0
        ctx.mark_non_differentiable(metrics)
        return loss, metrics

    @staticmethod
    def backward(ctx, grad_loss, _grad_metrics):
        dlp, dlpu = ctx.saved_tensors
        g_lp = dlp * grad_loss if ctx.needs_input_grad[0] else None
        g_lpu = dlpu * grad_loss if (ctx.has_lpu and ctx.needs_input_grad[1]) else None
        return (g_lp, g_lpu) + (None,) * 10


class ClippedPGLossFn(LossFunction):
    """Generalised clipped policy-gradient loss with KL regularisation.

    ``L = E_t[max(-A r, -A clip(r, 1-eps_lo, 1+eps_hi))] + beta * KL(pi || pi_ref)`` with the variants
    selected by the configuration flags (see ``ClippedPGLossConfig``).

    The metrics come back as a ``StepMetrics`` dictionary, which waits for the device when its values are first
    needed rather than before the call returns; ``lazy_metrics = False`` (not in the reference; set it on the
    instance) gives a plain dictionary filled at once."""

    lazy_metrics = True

    input_type = LossInputType.LOGPROB

    def __init__(self, cfg, use_fused_linear_logprobs: bool = False):
        if isinstance(cfg, dict):
            cfg = ClippedPGLossConfig(**cfg)
        self.use_fused_linear_logprobs = use_fused_linear_logprobs
        self.disable_ppo_ratio = cfg.disable_ppo_ratio
        self.ratio_clip_min = cfg.ratio_clip_min
        self.ratio_clip_max = cfg.ratio_clip_max
        self.ratio_clip_c = cfg.ratio_clip_c
        self.reference_policy_kl_penalty = cfg.reference_policy_kl_penalty if not cfg.use_kl_in_reward else 0
        self.reference_policy_kl_type = cfg.reference_policy_kl_type
        self.kl_input_clamp_value = cfg.kl_input_clamp_value
        self.kl_output_clamp_value = cfg.kl_output_clamp_value
        self.use_importance_sampling_correction = cfg.use_importance_sampling_correction
        self.truncated_importance_sampling_type = cfg.truncated_importance_sampling_type
        self.truncated_importance_sampling_ratio = cfg.truncated_importance_sampling_ratio
        self.truncated_importance_sampling_ratio_min = cfg.truncated_importance_sampling_ratio_min
        self.use_on_policy_kl_approximation = cfg.use_on_policy_kl_approximation
        self.force_on_policy_ratio = cfg.force_on_policy_ratio
        self.sequence_level_importance_ratios = cfg.sequence_level_importance_ratios
        self.positive_example_nll_weight = cfg.positive_example_nll_weight
        self.use_cispo = cfg.use_cispo
        self.loss_type = LossType.TOKEN_LEVEL if cfg.token_level_loss else LossType.SEQUENCE_LEVEL
        self._check_flags()
        self.metric_normalizations = self._normalizations()

    # -- constructor checks, loss_functions.py:265-324 ------------------------------------------
    def _check_flags(self) -> None:
        if self.sequence_level_importance_ratios:
            assert self.loss_type == LossType.SEQUENCE_LEVEL, (
                "sequence-level importance sampling (e.g. GSPO) is mutually exclusive with token-level loss"
            )
        if self.use_cispo:
            assert not self.disable_ppo_ratio, "use_cispo is incompatible with disable_ppo_ratio"
            assert not self.force_on_policy_ratio, "use_cispo is incompatible with force_on_policy_ratio"
            assert not self.sequence_level_importance_ratios, (
                "use_cispo is incompatible with sequence_level_importance_ratios"
            )
            assert self.ratio_clip_c is None, "use_cispo is incompatible with dual clipping (ratio_clip_c)"
            assert self.loss_type == LossType.TOKEN_LEVEL, "use_cispo requires token_level_loss=True"
        kind = self.truncated_importance_sampling_type
        if kind is not None:
            assert self.use_importance_sampling_correction, (
                "truncated importance sampling is only supported when use_importance_sampling_correction is True"
            )
            assert kind in ("tis", "icepop", "seq-mask-tis"), (
                f"truncated_importance_sampling_type must be 'tis', 'icepop', or 'seq-mask-tis', got {kind}"
            )
            hi, lo = self.truncated_importance_sampling_ratio, self.truncated_importance_sampling_ratio_min
            assert hi is not None and hi > 0, "truncated_importance_sampling_ratio should be positive"
            if lo is not None:
                assert lo <= hi, (
                    "truncated_importance_sampling_ratio_min must be <= truncated_importance_sampling_ratio"
                )
            if kind in ("icepop", "seq-mask-tis"):
                assert lo is not None, (
                    "truncated_importance_sampling_ratio_min should be set when "
                    "truncated_importance_sampling_type is 'icepop' or 'seq-mask-tis'"
                )
            if kind == "seq-mask-tis":
                assert not self.sequence_level_importance_ratios, (
                    "seq-mask-tis is incompatible with sequence_level_importance_ratios=True"
                )

    # -- per-metric denominators, loss_functions.py:331-372 --------------------------------------
    def _normalizations(self) -> dict[str, MetricNormalizer]:
        tok, seq, none = MetricNormalizer.TOKENS, MetricNormalizer.SEQUENCES, MetricNormalizer.NONE
        like_grad = tok if self.loss_type == LossType.TOKEN_LEVEL else seq
        table = {"loss": like_grad, "kl_penalty": like_grad}
        for key in ("probs_ratio", "probs_ratio_clamped", "token_mult_prob_error", "gen_kl_error",
                    "policy_kl_error", "js_divergence_error", "approx_entropy"):
            table[key] = tok
        table["sampling_importance_ratio"] = seq if self.sequence_level_importance_ratios else tok
        for key in ("num_valid_samples", "positive_nll_loss", "probs_ratio_min", "probs_ratio_max",
                    "probs_ratio_clamped_min", "probs_ratio_clamped_max"):
            table[key] = none
        if self.truncated_importance_sampling_type is not None:
            table["is_oob_ratio"] = seq if self.truncated_importance_sampling_type == "seq-mask-tis" else tok
        return table

    def _kernel_config(self, has_nll: bool) -> tuple[list[int], list[float]]:
        kind = self.truncated_importance_sampling_type
        if self.truncated_importance_sampling_ratio is not None and kind not in ("tis", "icepop", "seq-mask-tis"):
            raise ValueError(f"Invalid truncated importance sampling type: {kind}")
        if self.reference_policy_kl_type not in _KL_TYPES:
            raise ValueError(f"Invalid KL type: {self.reference_policy_kl_type}")
        if self.ratio_clip_c is not None:
            assert self.ratio_clip_c > 1, (
                f"ratio_clip_c must exceed 1 representing a lower bound of the ratios, got {self.ratio_clip_c}."
            )
        use_tis = self.truncated_importance_sampling_ratio is not None
        lo = self.truncated_importance_sampling_ratio_min
        iflags = [
            int(self.loss_type == LossType.TOKEN_LEVEL), int(self.disable_ppo_ratio), int(self.force_on_policy_ratio),
            int(self.use_cispo), int(self.sequence_level_importance_ratios),
            int(self.use_importance_sampling_correction), int(self.use_on_policy_kl_approximation),
            NRL_TIS[kind] if use_tis else 0, _KL_TYPES[self.reference_policy_kl_type],
            int(self.reference_policy_kl_penalty != 0), int(self.kl_input_clamp_value is not None),
            int(self.kl_output_clamp_value is not None), int(self.ratio_clip_c is not None), int(has_nll),
        ]
        fparams = [
            self.ratio_clip_min, self.ratio_clip_max, self.ratio_clip_c or 0.0, float(self.reference_policy_kl_penalty),
            self.kl_input_clamp_value or 0.0, self.kl_output_clamp_value or 0.0,
            self.truncated_importance_sampling_ratio or 0.0, 0.0 if lo is None else lo,
            float(self.positive_example_nll_weight),
        ]
        return iflags, fparams

    def __call__(
        self,
        next_token_logprobs: torch.Tensor,
        data: Any,
        global_valid_seqs: torch.Tensor,
        global_valid_toks: torch.Tensor,
    ) -> tuple[torch.Tensor, dict]:
        """``loss_functions.py:374-788``.  ``data`` is any mapping with the reference's keys."""
        lp_in = next_token_logprobs
        home = lp_in.device
        dev = _gpu_for(lp_in)
        beta = self.reference_policy_kl_penalty

        sample_mask_in = data["sample_mask"]
        lp = _f32(lp_in, dev)
        token_mask = _f32(data["token_mask"][:, 1:], dev)
        sample_mask = _f32(sample_mask_in, dev)
        adv = _f32(data["advantages"][:, 1:], dev)
        prev = None if self.force_on_policy_ratio else _f32(data["prev_logprobs"][:, 1:], dev)
        gen = _f32(data["generation_logprobs"][:, 1:], dev)
        ref = lpu = None
        if beta != 0:
            ref = _f32(data["reference_policy_logprobs"][:, 1:], dev)
            unfiltered = data.get("curr_logprobs_unfiltered", None)
            if unfiltered is not None and unfiltered is not lp_in:
                lpu = _f32(unfiltered, dev)
        correct = None
        has_nll = self.positive_example_nll_weight > 0 and "rewards" in data
        if has_nll:
            correct = (data["rewards"] > 0).to(device=dev, dtype=torch.float32)
        iflags, fparams = self._kernel_config(has_nll)

        loss, metrics = _FusedLoss.apply(
            lp, lpu, prev, gen, ref, adv, token_mask, sample_mask, correct,
            _global_valid(global_valid_seqs, global_valid_toks, dev), iflags, fparams,
        )
        if home != dev:
            loss = loss.to(home)
        return loss, metrics_record_to_dict(metrics, self, sample_mask_in)


class _FusedNll(torch.autograd.Function):
    @staticmethod
    def forward(ctx, lp, token_mask, sample_mask, global_valid):
        loss, dlp, metrics = _OPS.nll_loss(lp.detach(), token_mask, sample_mask, global_valid)
        ctx.save_for_backward(dlp)
        ctx.mark_non_differentiable(metrics)
        return loss, metrics

    @staticmethod
    def backward(ctx, grad_loss, _grad_metrics):
        (dlp,) = ctx.saved_tensors
        return dlp * grad_loss, None, None, None


class NLLLossFn(LossFunction):
    """Negative log-likelihood over the masked tokens (``loss_functions.py:791-842``): the scalar loss,
    or with ``dpo_loss=True`` one value per sample."""

    loss_type = LossType.TOKEN_LEVEL
    input_type = LossInputType.LOGPROB

    def __init__(self, use_fused_linear_logprobs: bool = False):
        self.use_fused_linear_logprobs = use_fused_linear_logprobs
        self.metric_normalizations = {
            "loss": MetricNormalizer.TOKENS,
            "num_unmasked_tokens": MetricNormalizer.NONE,
            "num_valid_samples": MetricNormalizer.NONE,
        }

    def __call__(self, next_token_logprobs, data, global_valid_seqs, global_valid_toks,
                 dpo_loss: bool = False, dpo_average_log_probs: bool = False):
        if dpo_loss:
            return self._per_sample(next_token_logprobs, data, dpo_average_log_probs)
        home = next_token_logprobs.device
        dev = _gpu_for(next_token_logprobs)
        sample_mask_in, token_mask_in = data["sample_mask"], data["token_mask"]
        loss, metrics = _FusedNll.apply(
            _f32(next_token_logprobs, dev), _f32(token_mask_in[:, 1:], dev), _f32(sample_mask_in, dev),
            _global_valid(1.0, global_valid_toks, dev),
        )
        if home != dev:
            loss = loss.to(home)
        m = metrics.cpu().tolist()
        integral = not (sample_mask_in.is_floating_point() or token_mask_in.is_floating_point())
        return loss, {
            "loss": m[0],
            "num_unmasked_tokens": int(m[1]) if integral else m[1],
            "num_valid_samples": m[2] if sample_mask_in.is_floating_point() else int(m[2]),
        }


    def _per_sample(self, next_token_logprobs, data, average_log_probs):
        """``dpo_loss=True`` (``loss_functions.py:823-829``): ``loss [B]``, summed (or averaged) over each sample's tokens."""
        home = next_token_logprobs.device
        dev = _gpu_for(next_token_logprobs)
        loss, totals = _NllRows.apply(_f32(next_token_logprobs, dev), _f32(data["token_mask"][:, 1:], dev),
                                      _f32(data["sample_mask"], dev), bool(average_log_probs))
        if home != dev:
            loss = loss.to(home)
        t = totals.cpu().tolist()
        return loss, {"loss": loss, "num_unmasked_tokens": t[0], "num_valid_samples": t[1]}


class _NllRows(torch.autograd.Function):
    @staticmethod
    def forward(ctx, lp, token_mask, sample_mask, average):
        rows, den, totals = _OPS.nll_rows_fwd(lp.detach(), token_mask, sample_mask, average)
        ctx.save_for_backward(token_mask, sample_mask, den)
        ctx.mark_non_differentiable(totals)
        return rows, totals

    @staticmethod
    def backward(ctx, grad_rows, _grad_totals):
        token_mask, sample_mask, den = ctx.saved_tensors
        return _OPS.nll_rows_bwd(grad_rows.contiguous().float(), token_mask, sample_mask, den), None, None, None


class _Preference(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rewards, sample_mask, global_valid):
        loss, drewards, metrics = _OPS.preference_loss(rewards.detach(), sample_mask, global_valid)
        ctx.save_for_backward(drewards)
        ctx.mark_non_differentiable(metrics)
        return loss, metrics

    @staticmethod
    def backward(ctx, grad_loss, _grad_metrics):
        (drewards,) = ctx.saved_tensors
        return drewards * grad_loss, None, None


class PreferenceLossFn(LossFunction):
    """Reward-model preference loss ``-E[log sigmoid(r_chosen - r_rejected)]`` over rows that alternate
    chosen / rejected (``loss_functions.py:853-946``)."""

    loss_type = LossType.SEQUENCE_LEVEL
    input_type = LossInputType.LOGIT

    def split_output_tensor(self, tensor):
        return tensor[::2], tensor[1::2]

    def __call__(self, logits, data, global_valid_seqs, global_valid_toks):
        home = logits.device
        dev = _gpu_for(logits)
        loss, metrics = _Preference.apply(_f32(logits.squeeze(-1), dev), _f32(data["sample_mask"], dev),
                                          _global_valid(global_valid_seqs, 1.0, dev))
        if home != dev:
            loss = loss.to(home)
        m = metrics.cpu().tolist()
        return loss, {"loss": m[0], "accuracy": m[1], "rewards_chosen_mean": m[2], "rewards_rejected_mean": m[3],
                      "num_valid_samples": m[4]}


class DPOLossConfig(BaseModel, extra="allow"):
    """Field names and defaults of ``loss_functions.py:949-954``."""

    reference_policy_kl_penalty: float = 0.05
    preference_loss_weight: float = 1.0
    sft_loss_weight: float = 0.0
    preference_average_log_probs: bool = False
    sft_average_log_probs: bool = False


class _Dpo(torch.autograd.Function):
    @staticmethod
    def forward(ctx, lp, ref, token_mask, sample_mask, global_valid, beta, w_pref, w_sft, avg_pref, avg_sft):
        loss, dlp, metrics = _OPS.dpo_loss(lp.detach(), ref, token_mask, sample_mask, global_valid, beta, w_pref, w_sft,
                                           avg_pref, avg_sft)
        ctx.save_for_backward(dlp)
        ctx.mark_non_differentiable(metrics)
        return loss, metrics

    @staticmethod
    def backward(ctx, grad_loss, _grad_metrics):
        (dlp,) = ctx.saved_tensors
        return (dlp * grad_loss,) + (None,) * 9


class DPOLossFn(PreferenceLossFn):
    """Direct preference optimisation on token logprobs (``loss_functions.py:966-1106``): preference
    term on the summed (or averaged) logprob margins against the reference policy, plus an optional
    SFT term on the chosen rows.  Rewards, both terms and the gradient come from one fused call."""

    loss_type = LossType.SEQUENCE_LEVEL
    input_type = LossInputType.LOGPROB

    def __init__(self, cfg, use_fused_linear_logprobs: bool = False):
        get = cfg.get if isinstance(cfg, dict) else lambda k, d=None: getattr(cfg, k, d)  # noqa: E731
        defaults = DPOLossConfig()
        for name in DPOLossConfig.model_fields:
            setattr(self, name, get(name, getattr(defaults, name)))
        self.use_fused_linear_logprobs = use_fused_linear_logprobs
        self.sft_loss = NLLLossFn(use_fused_linear_logprobs=use_fused_linear_logprobs)

    def __call__(self, next_token_logprobs, data, global_valid_seqs, global_valid_toks):
        if self.sft_loss_weight > 0 and global_valid_toks is None:
            raise AssertionError("global_valid_toks must be provided for SFT loss")
        home = next_token_logprobs.device
        dev = _gpu_for(next_token_logprobs)
        loss, metrics = _Dpo.apply(
            _f32(next_token_logprobs, dev), _f32(data["reference_policy_logprobs"][:, :-1], dev),
            _f32(data["token_mask"][:, 1:], dev), _f32(data["sample_mask"], dev), _global_valid(global_valid_seqs, 1.0, dev),
            float(self.reference_policy_kl_penalty), float(self.preference_loss_weight), float(self.sft_loss_weight),
            bool(self.preference_average_log_probs), bool(self.sft_average_log_probs),
        )
        if home != dev:
            loss = loss.to(home)
        m = metrics.cpu().tolist()
        return loss, {"loss": m[0], "sft_loss": m[1], "preference_loss": m[2], "accuracy": m[3], "rewards_chosen_mean": m[4],
                      "rewards_rejected_mean": m[5], "num_valid_samples": m[6]}


class DistillationLossConfig(BaseModel, extra="allow"):
    """Field names and defaults of ``loss_functions.py:1109-1112``."""

    kl_type: str = "mixed"
    mixed_kl_weight: float = 0.5
    zero_outside_topk: bool = False


class _DistillTopk(torch.autograd.Function):
    @staticmethod
    def forward(ctx, student_lp, teacher_lp, h_all, token_mask, sample_mask, global_valid_toks, kl_type, w, zero_outside, log_inf):
        loss, d_s, d_h = _OPS.distill_topk_loss(student_lp.detach(), teacher_lp.detach(), None if h_all is None else h_all.detach(),
                                                token_mask, sample_mask, global_valid_toks, kl_type, w, zero_outside, log_inf)
        ctx.save_for_backward(d_s, d_h)
        ctx.has_h = h_all is not None and d_h.numel() > 0
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        d_s, d_h = ctx.saved_tensors
        return (d_s * grad_loss, None, d_h * grad_loss if ctx.has_h else None) + (None,) * 7


class DistillationLossFn(LossFunction):
    """Top-k distillation loss (``loss_functions.py:1124-1206``): forward, reverse or mixed KL between the
    teacher's and the student's top-k log-probabilities per token, optionally with the correction for the
    student's mass outside the top-k, masked mean over the tokens.  One fused call returns the loss and
    the gradients with respect to the student's top-k log-probabilities and ``H_all``."""

    loss_type = LossType.TOKEN_LEVEL
    input_type = LossInputType.DISTILLATION
    _KL = {"forward": 0, "reverse": 1, "mixed": 2}

    def __init__(self, cfg):
        get = cfg.get if isinstance(cfg, dict) else lambda k, d=None: getattr(cfg, k, d)  # noqa: E731
        defaults = DistillationLossConfig()
        self.kl_type = get("kl_type", defaults.kl_type)
        self.mixed_kl_weight = get("mixed_kl_weight", defaults.mixed_kl_weight)
        self.zero_outside_topk = get("zero_outside_topk", defaults.zero_outside_topk)
        self.log_infinitesimal = -100
        assert self.kl_type in ["forward", "reverse", "mixed"], "Invalid KL type"
        assert self.mixed_kl_weight >= 0 and self.mixed_kl_weight <= 1, (
            "Invalid mixed KL weight"
        )

    def __call__(self, student_topk_logprobs, teacher_topk_logprobs, H_all, data, global_valid_seqs, global_valid_toks):
        home = student_topk_logprobs.device
        dev = _gpu_for(student_topk_logprobs)
        token_mask = sample_mask = valid = None
        if "token_mask" in data and "sample_mask" in data:
            n = student_topk_logprobs.shape[1]
            token_mask = _f32(data["token_mask"][:, 1:][:, :n], dev)
            sample_mask = _f32(data["sample_mask"], dev)
            valid = _global_valid(1.0, global_valid_toks, dev)[1:]
        loss = _DistillTopk.apply(
            _f32(student_topk_logprobs, dev), _f32(teacher_topk_logprobs, dev), None if H_all is None else _f32(H_all, dev),
            token_mask, sample_mask, valid, self._KL[self.kl_type], float(self.mixed_kl_weight), bool(self.zero_outside_topk),
            float(self.log_infinitesimal),
        )
        if home != dev:
            loss = loss.to(home)
        return loss, {"loss": float(loss.item()), "num_valid_samples": data["input_ids"].shape[0]}


class DraftCrossEntropyLossFn(LossFunction):
    """Soft-target cross entropy for draft-model training (``loss_functions.py:66-108``): per token
    ``-sum_v softmax(teacher)_v log_softmax(student)_v`` from one streaming pass over both logit
    tensors, then the masked mean over the tokens."""

    loss_type = LossType.TOKEN_LEVEL
    input_type = LossInputType.DRAFT

    def __init__(self, vocab_parallel_group: Optional[Any] = None):
        self.vocab_parallel_group = vocab_parallel_group

    def __call__(self, teacher_logits, student_logits, token_mask, data, global_valid_seqs, global_valid_toks):
        from ...distributed.model_utils import DistributedCrossEntropy

        per_token = DistributedCrossEntropy.apply(student_logits, teacher_logits, self.vocab_parallel_group, False)
        dev = per_token.device
        # masked_mean(x, mask, Gt) = sum(x * mask) / (Gt + 1e-8): the NLL kernel's reduction with the sign flipped
        nll, _metrics = _FusedNll.apply(per_token, _f32(token_mask, dev), _f32(data["sample_mask"], dev),
                                        _global_valid(1.0, global_valid_toks, dev))
        return -nll
