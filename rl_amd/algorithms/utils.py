"""Helpers around the loss (counterparts of ``nemo_rl/algorithms/utils.py:42-274``).

``calculate_baseline_and_std_per_prompt`` runs the HIP grouping / statistics kernels, ``calculate_kl`` and
``masked_mean`` their own small kernels (inside ``ClippedPGLossFn`` the same arithmetic is part of the fused loss
kernel instead).  ``mask_out_neg_inf_logprobs`` is [B, S]-sized tensor plumbing around the reference's warning.
"""

from __future__ import annotations

import atexit
from typing import Optional

import torch

from .. import ops as _ops  # noqa: F401

_OPS = torch.ops.rl_amd


def _install_original(name: str):
    """The function of this name that an existing NeMo-RL install had before ``rl_amd.install()`` replaced it."""
    from ..compat import original

    return original("nemo_rl.algorithms.utils", name)


def _host_only(*tensors) -> bool:
    """Host tensors in a process that sees no GPU (the GRPO driver of a multi-node run)."""
    return not torch.cuda.is_available() and all(t is None or not t.is_cuda for t in tensors)


def _gpu_device() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("rl_amd needs an MI355X: no GPU is visible and there is no CPU fallback")
    return torch.device("cuda", torch.cuda.current_device())


_KL_TYPES = {"k1": 1, "k2": 2, "k3": 3}


def _staged(t: torch.Tensor, dev: torch.device) -> torch.Tensor:
    """fp32, contiguous, on the GPU (host tensors, the driver's default, are copied over)."""
    return t.detach().to(device=dev, dtype=torch.float32).contiguous()


class _CalculateKl(torch.autograd.Function):
    @staticmethod
    def forward(ctx, lp, ref, weights, kl_type, input_clamp, output_clamp, out_dtype, out_device):
        dev = lp.device if lp.is_cuda else _gpu_device()
        parts = torch.broadcast_tensors(*[t for t in (lp, ref, weights) if t is not None])
        staged = [_staged(t, dev) for t in parts]
        lp32, ref32 = staged[0], staged[1]
        w32 = staged[2] if weights is not None else None
        ctx.save_for_backward(lp32, ref32, w32)
        ctx.cfg = (kl_type, input_clamp, output_clamp)
        ctx.inputs = [(t.shape, t.dtype, t.device) if t is not None else None for t in (lp, ref, weights)]
        out = _OPS.calculate_kl(lp32, ref32, w32, kl_type, input_clamp, output_clamp)
        return out.to(device=out_device, dtype=out_dtype)

    @staticmethod
    def backward(ctx, grad):
        lp32, ref32, w32 = ctx.saved_tensors
        need = ctx.needs_input_grad[:3]
        g = _staged(grad.expand(lp32.shape), lp32.device)
        grads = _OPS.calculate_kl_bwd(g, lp32, ref32, w32, *ctx.cfg, need[0], need[1], bool(need[2] and w32 is not None))
        out = []
        for wanted, d, meta in zip(need, grads, ctx.inputs):
            if not wanted or meta is None:
                out.append(None)
                continue
            shape, dtype, device = meta
            out.append(d.sum_to_size(shape).to(device=device, dtype=dtype) if tuple(d.shape) != tuple(shape) else d.to(device=device, dtype=dtype))
        return (*out, None, None, None, None, None)


def calculate_kl(
    logprobs: torch.Tensor,
    logprobs_reference: torch.Tensor,
    kl_type: str = "k3",
    input_clamp_value: float | None = 20.0,
    output_clamp_value: float | None = 10.0,
    importance_sampling_weights: torch.Tensor | None = None,
) -> torch.Tensor:
    """Per-token k1 / k2 / k3 estimate of KL(policy || reference), ``utils.py:42-101``: one elementwise HIP kernel
    (the arithmetic of the loss kernel's KL term) with its gradient kernel behind autograd.  Computed in fp32 and
    returned in the inputs' promoted dtype, on the device of ``logprobs``."""
    if kl_type not in _KL_TYPES:
        raise ValueError(f"Invalid KL type: {kl_type}")
    tensors = [t for t in (logprobs, logprobs_reference, importance_sampling_weights) if t is not None]
    theirs = _install_original("calculate_kl")
    if theirs is not None and (_host_only(*tensors) or any(t.dtype == torch.float64 for t in tensors)):
        # on an install: what the kernels do not cover (a driver process without a GPU, double precision)
        # stays with the function the install came with
        return theirs(logprobs, logprobs_reference, kl_type, input_clamp_value, output_clamp_value,
                      importance_sampling_weights)
    out_dtype = tensors[0].dtype
    for t in tensors[1:]:
        out_dtype = torch.promote_types(out_dtype, t.dtype)
    return _CalculateKl.apply(
        logprobs, logprobs_reference, importance_sampling_weights, _KL_TYPES[kl_type],
        None if input_clamp_value is None else float(input_clamp_value),
        None if output_clamp_value is None else float(output_clamp_value), out_dtype, logprobs.device,
    )


class _MaskedMeanRows(torch.autograd.Function):
    @staticmethod
    def forward(ctx, values2d, mask2d, norm):
        out, denom = _OPS.masked_mean_rows(values2d, mask2d, norm)
        ctx.save_for_backward(mask2d, denom)
        return out

    @staticmethod
    def backward(ctx, grad):
        mask2d, denom = ctx.saved_tensors
        return _OPS.masked_mean_rows_bwd(grad.contiguous().float(), mask2d, denom), None, None


def masked_mean(
    values: torch.Tensor,
    mask: torch.Tensor,
    dim: Optional[int] = None,
    global_normalization_factor: Optional[torch.Tensor | float] = None,
):
    """``sum(values * mask) / (norm + 1e-8)``, ``utils.py:207-224``, over everything (``dim=None``) or one axis: a
    row-reduction HIP kernel (sums carried in double) and its gradient kernel for ``values``.  The mask and the
    normalisation factor are constants of the gradient, as in every use the reference makes of this function."""
    norm = global_normalization_factor
    not_covered = None
    if dim is not None and not isinstance(dim, int):
        not_covered = "masked_mean reduces over everything or over one axis"
    elif mask.requires_grad or (isinstance(norm, torch.Tensor) and norm.requires_grad):
        not_covered = "masked_mean differentiates with respect to the values only"
    elif isinstance(norm, torch.Tensor) and norm.numel() != 1:
        not_covered = "the normalisation factor must be one value"
    theirs = _install_original("masked_mean")
    if theirs is not None and (not_covered or _host_only(values, mask) or values.dtype == torch.float64):
        # on an install: argument forms no caller on the hot path uses, a driver process without a GPU and
        # double precision stay with the function the install came with
        return theirs(values, mask, dim, global_normalization_factor)
    if not_covered:
        raise NotImplementedError(not_covered)
    out_dtype = torch.promote_types(values.dtype, mask.dtype)
    if isinstance(norm, torch.Tensor):
        out_dtype = torch.promote_types(out_dtype, norm.dtype)
    if not out_dtype.is_floating_point:
        out_dtype = torch.float32
    dev = values.device if values.is_cuda else _gpu_device()
    v, m = torch.broadcast_tensors(values, mask)
    if dim is None:
        v2, m2, out_shape = v.reshape(1, -1), m.reshape(1, -1), ()
    else:
        v, m = v.movedim(dim, -1), m.movedim(dim, -1)
        out_shape = tuple(v.shape[:-1])
        v2, m2 = v.reshape(-1, v.shape[-1]), m.reshape(-1, m.shape[-1])
    v2 = v2.to(device=dev, dtype=torch.float32).contiguous()
    m2 = _staged(m2, dev)
    norm_t = None if norm is None else torch.as_tensor(norm, dtype=torch.float32).detach().to(dev).reshape(1)
    out = _MaskedMeanRows.apply(v2, m2, norm_t)
    return out.reshape(out_shape).to(device=values.device, dtype=out_dtype)


# The warning of ``mask_out_neg_inf_logprobs`` needs two counts from the device.  The reference fetches them and
# prints before it returns, which stalls the caller's thread until the forward pass has finished, once per
# microbatch.  Here the counts travel to pinned host memory behind the stream and the same line is printed once they
# have arrived -- at a later call, at ``flush_neg_inf_warnings()`` or when the interpreter exits -- so the caller keeps
# queueing work (the backward, the next microbatch).  ``DEFER_NEG_INF_WARNING = False`` prints before returning.
DEFER_NEG_INF_WARNING = True
_pending_warnings: list = []  # (event, pinned int64[2], name)


def _warn_neg_inf(hit: int, valid: int, logprobs_name: str) -> None:
    if hit > 0:
        print(
            f"[WARNING]: {hit}/{valid} valid tokens have -inf in {logprobs_name} "
            "(policy top-k/top-p mismatch). Masking out these positions."
        )


def flush_neg_inf_warnings(wait: bool = True) -> None:
    """Prints the deferred warnings whose counts have arrived, oldest first; with ``wait`` all of them."""
    while _pending_warnings:
        event, counts, name = _pending_warnings[0]
        if not wait and not event.query():
            return
        event.synchronize()
        _pending_warnings.pop(0)
        _warn_neg_inf(int(counts[0]), int(counts[1]), name)


atexit.register(flush_neg_inf_warnings)


def mask_out_neg_inf_logprobs(logprobs: torch.Tensor, mask: torch.Tensor, logprobs_name: str) -> torch.Tensor:
    """``utils.py:227-257``: positions that are masked out or infinite become 0 (with the reference's
    warning when valid tokens are affected)."""
    is_inf = torch.isinf(logprobs)
    # both counts in one transfer: the warning is the only reason this function waits for the device at all
    counts = torch.stack([(is_inf & mask.bool()).sum(), mask.sum().to(torch.int64)])
    if DEFER_NEG_INF_WARNING and counts.is_cuda:
        flush_neg_inf_warnings(wait=False)
        host = torch.empty(2, dtype=torch.int64, pin_memory=True)
        host.copy_(counts, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        _pending_warnings.append((event, host, logprobs_name))
    else:
        hit, valid = counts.tolist()
        _warn_neg_inf(hit, valid, logprobs_name)
    keep = mask * (~is_inf).float()
    return torch.where(keep.bool(), logprobs, 0.0)


def calculate_baseline_and_std_per_prompt(
    prompts: torch.Tensor,
    rewards: torch.Tensor,
    valid_mask: torch.Tensor,
    leave_one_out_baseline: bool = True,
    std_rewards: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``utils.py:104-198``: per-prompt (leave-one-out) baseline and std; results come back on the
    device of ``rewards``.  Inputs that live on the host (the driver's default) are staged to the GPU."""
    theirs = _install_original("calculate_baseline_and_std_per_prompt")
    if theirs is not None and _host_only(prompts, rewards, valid_mask, std_rewards):
        return theirs(prompts, rewards, valid_mask, leave_one_out_baseline, std_rewards)  # a driver without a GPU
    baseline, std, _, _ = _group_stats(prompts, rewards, valid_mask, leave_one_out_baseline, std_rewards, False)
    return baseline, std


def _group_stats(prompts, rewards, valid_mask, leave_one_out, std_rewards, normalize):
    home = rewards.device
    dev = home if home.type == "cuda" else _gpu_device()
    if rewards.numel() == 0:
        z = torch.zeros_like(rewards)
        return z, z.clone(), z.clone(), torch.zeros(0, dtype=torch.int32, device=home)
    out = _OPS.group_baseline_std(
        prompts.to(dev, torch.int64),
        rewards.to(dev, torch.float32),
        valid_mask.to(dev, torch.float32),
        None if std_rewards is None or std_rewards is rewards else std_rewards.to(dev, torch.float32),
        bool(leave_one_out),
        bool(normalize),
    )
    baseline, std, adv, group = (t.to(home) for t in out)
    return baseline.to(rewards.dtype), std.to(rewards.dtype), adv.to(rewards.dtype), group
