"""PyTorch custom ops (``torch.ops.rl_amd.*``) over the C-ABI HIP library.

PyTorch supplies device memory and the current stream; every computation is a kernel in
``librl_amd_hip.so``.  Each op validates shapes on the host before a launch and raises on
anything the kernels do not assume (CPU tensors, non-contiguous vocabulary axis, wrong dtype).
"""

from __future__ import annotations

import ctypes as C
import os

import torch

from . import _lib
from ._deferred import refuse_pending

_DTYPES = {torch.float32: _lib.NRL_F32, torch.bfloat16: _lib.NRL_BF16, torch.float16: _lib.NRL_F16}

_LIB = torch.library.Library("rl_amd", "DEF")

# Optional per-launch timing: an object with ``start(name)`` / ``stop(name)`` that records events on
# the current stream around a kernel launch (used by the benchmark harness); None in normal use.
KERNEL_TIMER = None


class _timed:
    def __init__(self, name):
        self.name = name

    def __enter__(self):
        if KERNEL_TIMER is not None:
            KERNEL_TIMER.start(self.name)

    def __exit__(self, *exc):
        if KERNEL_TIMER is not None:
            KERNEL_TIMER.stop(self.name)
        return False


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t) -> C.c_void_p:
    return C.c_void_p(0 if t is None else t.data_ptr())


def _need_gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("rl_amd ops run on the GPU only (got a CPU tensor); there is no CPU fallback")


_PHASE = 1 << 21          # large device allocations start on 2 MiB boundaries
# where in that period the gradient buffer starts, relative to the logits (NRL_GRAD_PHASE overrides, for tuning)
_GRAD_PHASE = int(os.environ.get("NRL_GRAD_PHASE", "0x1B0000"), 0) % _PHASE
_PHASED_MIN_BYTES = 64 << 20


def _grad_buffer(shape, like: torch.Tensor) -> torch.Tensor:
    """An uninitialised tensor of ``shape`` in ``like``'s dtype for a kernel that streams ``like`` in and the
    new tensor out at the same time.  The kernels read and write rows at a fixed distance from each other, and
    how fast HBM serves the two streams together depends on that distance modulo the address interleave: with
    both buffers on 2 MiB boundaries a 256 KiB row (V = 131072 bf16) loses 5 - 17 %, and distances of 64 - 256
    KiB lose 8 % at V = 151936.  Starting the output 1.69 MiB into the period was at or near the best measured
    for both, so large outputs are placed there inside a slightly larger allocation."""
    n = 1
    for d in shape:
        n *= int(d)
    nbytes = n * like.element_size()
    if nbytes < _PHASED_MIN_BYTES:
        return torch.empty(tuple(shape), dtype=like.dtype, device=like.device)
    flat = torch.empty((nbytes + _PHASE,), dtype=torch.uint8, device=like.device)
    off = (like.data_ptr() + _GRAD_PHASE - flat.data_ptr()) % _PHASE
    off -= off % 256  # keeps every row start as aligned as in a fresh allocation
    return flat[off:off + nbytes].view(like.dtype).view(tuple(shape))



def _dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported logits dtype {t.dtype}") from None


def _rows(logits, targets, n_inner, vocab_start, vocab_end, temperature, temp_mode) -> _lib.NrlRows:
    """logits [B, S, V] (unit stride on V), targets [B, >= n_inner] int64 view."""
    if logits.dim() != 3 or targets.dim() != 2:
        raise ValueError(f"expected logits [B,S,V] and targets [B,S'], got {tuple(logits.shape)}, {tuple(targets.shape)}")
    if logits.stride(2) != 1 and logits.shape[2] > 1:
        raise ValueError("the vocabulary axis of the logits must be contiguous")
    if targets.dtype != torch.int64:
        raise ValueError(f"targets must be int64, got {targets.dtype}")
    b, s, v = logits.shape
    if targets.shape[0] != b or n_inner > s or n_inner > targets.shape[1] or n_inner < 0:
        raise ValueError(
            f"rows [{b}, {n_inner}] do not fit logits {tuple(logits.shape)} / targets {tuple(targets.shape)}"
        )
    r = _lib.NrlRows()
    r.logits = logits.data_ptr()
    r.dtype = _dtype_code(logits)
    r.n_outer, r.n_inner, r.vocab = b, n_inner, v
    r.stride_outer, r.stride_inner = logits.stride(0), logits.stride(1)
    r.targets = targets.data_ptr()
    r.tgt_stride_outer, r.tgt_stride_inner = targets.stride(0), targets.stride(1)
    r.vocab_start, r.vocab_end = vocab_start, vocab_end
    r.temperature, r.temp_mode = temperature, temp_mode
    return r


# ------------------------------------------------------------------------------------------------
# K1 / K2
# ------------------------------------------------------------------------------------------------
_LIB.define(
    "logprob_fwd(Tensor logits, Tensor targets, int n_inner, int vocab_start, int vocab_end, "
    "float temperature, int temp_mode, bool save_lse) -> (Tensor, Tensor)"
)
_LIB.define(
    "logprob_bwd(Tensor logits, Tensor targets, Tensor lse, Tensor grad, int n_inner, int vocab_start, "
    "int vocab_end, float temperature, int temp_mode) -> Tensor"
)
_LIB.define(
    "logprob_bwd_(Tensor(a!) logits, Tensor targets, Tensor lse, Tensor grad, int n_inner, int vocab_start, "
    "int vocab_end, float temperature, int temp_mode) -> ()"
)


def _logprob_fwd(logits, targets, n_inner, vocab_start, vocab_end, temperature, temp_mode, save_lse):
    _need_gpu(logits, targets)
    rows = _rows(logits, targets, n_inner, vocab_start, vocab_end, temperature, temp_mode)
    b = logits.shape[0]
    with torch.cuda.device(logits.device):
        out = torch.empty((b, n_inner), dtype=torch.float32, device=logits.device)
        lse = torch.empty((b, n_inner) if save_lse else (0,), dtype=torch.float32, device=logits.device)
        with _timed("logprob_fwd"):
            code = _lib.load().nrl_logprob_fwd(C.byref(rows), _ptr(out), _ptr(lse if save_lse else None), _stream())
    _lib.check(code, "nrl_logprob_fwd")
    return out, lse


def _logprob_bwd(logits, targets, lse, grad, n_inner, vocab_start, vocab_end, temperature, temp_mode, in_place=False):
    _need_gpu(logits, targets, lse, grad)
    rows = _rows(logits, targets, n_inner, vocab_start, vocab_end, temperature, temp_mode)
    b, s, v = logits.shape
    if tuple(lse.shape) != (b, n_inner) or not lse.is_contiguous() or lse.dtype != torch.float32:
        raise ValueError("lse must be a contiguous fp32 [B, n_inner] tensor")
    if tuple(grad.shape) != (b, n_inner) or grad.dtype != torch.float32:
        raise ValueError(f"grad must be fp32 [B, n_inner], got {grad.dtype} {tuple(grad.shape)}")
    with torch.cuda.device(logits.device):
        d = logits if in_place else _grad_buffer((b, s, v), logits)
        with _timed("logprob_bwd"):
            code = _lib.load().nrl_logprob_bwd(
                C.byref(rows), _ptr(lse), _ptr(grad), grad.stride(0), grad.stride(1),
                _ptr(d), s, d.stride(0), d.stride(1), _stream(),
            )
    _lib.check(code, "nrl_logprob_bwd")
    return d


def _logprob_bwd_inplace(logits, targets, lse, grad, n_inner, vocab_start, vocab_end, temperature, temp_mode):
    """The gradient overwrites the logits buffer (for callers that no longer need the logits)."""
    _logprob_bwd(logits, targets, lse, grad, n_inner, vocab_start, vocab_end, temperature, temp_mode, in_place=True)


_LIB.define(
    "logprob_post_fwd(Tensor logits, Tensor targets, Tensor lengths, int n_inner, int vocab_start, int vocab_end, "
    "float temperature, int temp_mode) -> Tensor"
)


def _logprob_post_fwd(logits, targets, lengths, n_inner, vocab_start, vocab_end, temperature, temp_mode):
    """[B, n_inner + 1] forward-only logprobs: zero column in front, zeros from each sequence's length on."""
    _need_gpu(logits, targets, lengths)
    rows = _rows(logits, targets, n_inner, vocab_start, vocab_end, temperature, temp_mode)
    b = logits.shape[0]
    if lengths.dtype != torch.int64 or tuple(lengths.shape) != (b,) or not lengths.is_contiguous():
        raise ValueError("lengths must be a contiguous int64 [B] tensor")
    with torch.cuda.device(logits.device):
        out = torch.empty((b, n_inner + 1), dtype=torch.float32, device=logits.device)
        with _timed("logprob_post_fwd"):
            code = _lib.load().nrl_logprob_post_fwd(C.byref(rows), _ptr(lengths), _ptr(out), _stream())
    _lib.check(code, "nrl_logprob_post_fwd")
    return out


_LIB.define("scale_rows_(Tensor(a!) x, Tensor factor, float divisor) -> ()")
_LIB.define("scale_rows(Tensor x, Tensor factor, float divisor) -> Tensor")


def _scale_rows(x, factor, divisor, in_place=False):
    """``x * (factor / divisor)`` for a ``[B, S, V]`` tensor and a device scalar ``factor``, in ``x``'s dtype.  The
    host does not wait for the factor's value; in place, a factor equal to the divisor touches no memory."""
    _need_gpu(x, factor)
    if x.dim() != 3 or (x.stride(2) != 1 and x.shape[2] > 1):
        raise ValueError(f"expected [B, S, V] with a contiguous last axis, got {tuple(x.shape)} strides {x.stride()}")
    if factor.numel() != 1:
        raise ValueError("factor must hold one element")
    f = factor.detach().reshape(1).to(torch.float32)
    b, s, v = x.shape
    with torch.cuda.device(x.device):
        out = x if in_place else torch.empty((b, s, v), dtype=x.dtype, device=x.device)
        with _timed("scale_rows"):
            code = _lib.load().nrl_scale_rows(_ptr(x), _ptr(out), _dtype_code(x), b, s, v, x.stride(0), x.stride(1),
                                              out.stride(0), out.stride(1), _ptr(f), float(divisor), _stream())
    _lib.check(code, "nrl_scale_rows")
    return out


def _scale_rows_inplace(x, factor, divisor):
    _scale_rows(x, factor, divisor, in_place=True)


for _name, _fn in (("logprob_fwd", _logprob_fwd), ("logprob_bwd", _logprob_bwd), ("logprob_bwd_", _logprob_bwd_inplace),
                   ("logprob_post_fwd", _logprob_post_fwd), ("scale_rows_", _scale_rows_inplace), ("scale_rows", _scale_rows)):
    _LIB.impl(_name, _fn, "CUDA")
    _LIB.impl(_name, _fn, "CPU")  # raises: there is no CPU path


# ------------------------------------------------------------------------------------------------
# packed sequences
# ------------------------------------------------------------------------------------------------
_LIB.define("pack_input_ids(Tensor input_ids, Tensor cu_seqlens, Tensor cu_seqlens_padded, int roll_shift, int total) -> Tensor")


def _pack_input_ids(input_ids, cu_seqlens, cu_seqlens_padded, roll_shift, total):
    """``[B, S]`` int64 ids -> packed ``[total]`` ids; the boundaries are int32 ``[B + 1]`` device tensors that the
    host never reads."""
    _need_gpu(input_ids, cu_seqlens, cu_seqlens_padded)
    if input_ids.dim() != 2 or input_ids.dtype != torch.int64 or (input_ids.shape[1] > 1 and input_ids.stride(1) != 1):
        raise ValueError("input_ids must be int64 [B, S] with a contiguous last axis")
    b, s = input_ids.shape
    for t in (cu_seqlens, cu_seqlens_padded):
        if t.dtype != torch.int32 or tuple(t.shape) != (b + 1,) or not t.is_contiguous():
            raise ValueError(f"sequence boundaries must be contiguous int32 [{b + 1}] tensors")
    with torch.cuda.device(input_ids.device):
        out = torch.empty((int(total),), dtype=torch.int64, device=input_ids.device)
        code = _lib.load().nrl_pack_input_ids(_ptr(input_ids), b, s, input_ids.stride(0) if b > 1 else max(s, 1), _ptr(cu_seqlens),
                                              _ptr(cu_seqlens_padded), int(roll_shift), _ptr(out), int(total), _stream())
    _lib.check(code, "nrl_pack_input_ids")
    return out


_LIB.impl("pack_input_ids", _pack_input_ids, "CUDA")
_LIB.impl("pack_input_ids", _pack_input_ids, "CPU")

_LIB.define(
    "logprob_packed_fwd(Tensor logits, Tensor targets, bool pre_rolled, Tensor cu_seqlens, int unpacked_seqlen, "
    "int vocab_start, int vocab_end, float temperature, int temp_mode, bool save_lse) -> (Tensor, Tensor)"
)
_LIB.define(
    "logprob_packed_bwd(Tensor logits, Tensor targets, bool pre_rolled, Tensor cu_seqlens, int unpacked_seqlen, "
    "int vocab_start, int vocab_end, float temperature, int temp_mode, Tensor lse, Tensor grad) -> Tensor"
)


def _check_packed(logits, targets, cu_seqlens, unpacked_seqlen):
    _need_gpu(logits, targets, cu_seqlens)
    if logits.dim() != 2 or (logits.stride(1) != 1 and logits.shape[1] > 1):
        raise ValueError("packed logits must be [T, V] with a contiguous vocabulary axis")
    if targets.dtype != torch.int64 or targets.dim() != 1 or not targets.is_contiguous():
        raise ValueError("packed targets must be a contiguous int64 [T] tensor")
    if targets.shape[0] < logits.shape[0]:
        raise ValueError(f"{targets.shape[0]} targets for {logits.shape[0]} packed positions")
    if cu_seqlens.dtype != torch.int32 or cu_seqlens.dim() != 1 or not cu_seqlens.is_contiguous():
        raise ValueError("cu_seqlens must be a contiguous int32 [n_seq+1] tensor")
    if cu_seqlens.shape[0] < 1 or unpacked_seqlen < 1:
        raise ValueError("cu_seqlens needs at least one entry and unpacked_seqlen >= 1")


def _logprob_packed_fwd(logits, targets, pre_rolled, cu_seqlens, unpacked_seqlen, vocab_start, vocab_end,
                        temperature, temp_mode, save_lse):
    _check_packed(logits, targets, cu_seqlens, unpacked_seqlen)
    t, v = logits.shape
    n_seq = cu_seqlens.shape[0] - 1
    with torch.cuda.device(logits.device):
        out = torch.empty((n_seq, unpacked_seqlen - 1), dtype=torch.float32, device=logits.device)
        lse = torch.empty((t,) if save_lse else (0,), dtype=torch.float32, device=logits.device)
        lib = _lib.load()
        with _timed("logprob_packed_fwd"):
            code = lib.nrl_logprob_packed_fwd(
                _ptr(logits), _dtype_code(logits), t, v, logits.stride(0), _ptr(targets), int(pre_rolled),
                _ptr(cu_seqlens), n_seq, unpacked_seqlen, vocab_start, vocab_end, temperature, temp_mode,
                _ptr(out), _ptr(lse if save_lse else None), _stream(),
            )
    _lib.check(code, "nrl_logprob_packed_fwd")
    return out, lse


def _logprob_packed_bwd(logits, targets, pre_rolled, cu_seqlens, unpacked_seqlen, vocab_start, vocab_end,
                        temperature, temp_mode, lse, grad):
    _check_packed(logits, targets, cu_seqlens, unpacked_seqlen)
    _need_gpu(lse, grad)
    t, v = logits.shape
    n_seq = cu_seqlens.shape[0] - 1
    if tuple(lse.shape) != (t,) or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise ValueError("lse must be a contiguous fp32 [T] tensor")
    if tuple(grad.shape) != (n_seq, unpacked_seqlen - 1) or grad.dtype != torch.float32:
        raise ValueError("grad must be fp32 [n_seq, unpacked_seqlen-1]")
    grad = grad.contiguous()
    with torch.cuda.device(logits.device):
        d = _grad_buffer((t, v), logits)
        lib = _lib.load()
        with _timed("logprob_packed_bwd"):
            code = lib.nrl_logprob_packed_bwd(
                _ptr(logits), _dtype_code(logits), t, v, logits.stride(0), _ptr(targets), int(pre_rolled),
                _ptr(cu_seqlens), n_seq, unpacked_seqlen, vocab_start, vocab_end, temperature, temp_mode,
                _ptr(lse), _ptr(grad), _ptr(d), d.stride(0), _stream(),
            )
    _lib.check(code, "nrl_logprob_packed_bwd")
    return d


for _name, _fn in (("logprob_packed_fwd", _logprob_packed_fwd), ("logprob_packed_bwd", _logprob_packed_bwd)):
    _LIB.impl(_name, _fn, "CUDA")
    _LIB.impl(_name, _fn, "CPU")


# ------------------------------------------------------------------------------------------------
# K3: top-k / top-p
# ------------------------------------------------------------------------------------------------
_LIB.define("log_softmax_fwd(Tensor logits) -> Tensor")
_LIB.define("log_softmax_bwd(Tensor logprobs, Tensor grad) -> Tensor")


def _rows2d(t, name):
    if t.dim() != 2 or (t.stride(1) != 1 and t.shape[1] > 1):
        raise ValueError(f"{name} must be [rows, V] with a contiguous vocabulary axis")
    return t


def _log_softmax_fwd(logits):
    """[rows, V] -> log-softmax in the same dtype (fp32 arithmetic)."""
    _need_gpu(logits)
    _rows2d(logits, "logits")
    n, v = logits.shape
    with torch.cuda.device(logits.device):
        out = _grad_buffer((n, v), logits)
        with _timed("log_softmax_fwd"):
            code = _lib.load().nrl_log_softmax_fwd(_ptr(logits), _dtype_code(logits), n, v, logits.stride(0) if n > 1 else v,
                                                   _ptr(out), v, _stream())
    _lib.check(code, "nrl_log_softmax_fwd")
    return out


def _log_softmax_bwd(logprobs, grad):
    _need_gpu(logprobs, grad)
    _rows2d(logprobs, "logprobs")
    _rows2d(grad, "grad")
    if grad.shape != logprobs.shape or grad.dtype != logprobs.dtype:
        raise ValueError("grad must have the shape and dtype of the log-probabilities")
    n, v = logprobs.shape
    with torch.cuda.device(logprobs.device):
        dx = _grad_buffer((n, v), logprobs)
        with _timed("log_softmax_bwd"):
            code = _lib.load().nrl_log_softmax_bwd(_ptr(logprobs), _dtype_code(logprobs), n, v, logprobs.stride(0) if n > 1 else v,
                                                   _ptr(grad), grad.stride(0) if n > 1 else v, _ptr(dx), v, _stream())
    _lib.check(code, "nrl_log_softmax_bwd")
    return dx


for _name, _fn in (("log_softmax_fwd", _log_softmax_fwd), ("log_softmax_bwd", _log_softmax_bwd)):
    _LIB.impl(_name, _fn, "CUDA")
    _LIB.impl(_name, _fn, "CPU")

_LIB.define(
    "topk_topp_logprob_fwd(Tensor logits, Tensor? targets, int n_inner, int top_k, float top_p, float temperature, "
    "int temp_mode, bool want_unfiltered) -> (Tensor, Tensor, Tensor, Tensor, Tensor)"
)
_LIB.define(
    "topk_topp_logprob_fwd_rec(Tensor logits, Tensor targets, int n_inner, int top_k, float top_p, float temperature, "
    "int temp_mode, bool want_unfiltered, int capacity) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)"
)
_LIB.define(
    "topk_topp_logprob_bwd(Tensor logits, Tensor targets, Tensor thr, Tensor tie, Tensor lse_kept, Tensor grad, "
    "int n_inner, float temperature, int temp_mode, Tensor? kept_n=None, Tensor? kept_idx=None, Tensor? kept_x=None) -> Tensor"
)
_LIB.define(
    "topk_topp_filter(Tensor logits, Tensor thr, Tensor tie, float temperature, int temp_mode) -> (Tensor, Tensor)"
)


def _topk_topp_logprob_fwd(logits, targets, n_inner, top_k, top_p, temperature, temp_mode, want_unfiltered, capacity=0):
    """-> (logprob [B,n] (empty without targets), thr, tie, lse_kept, unfiltered logprob (or empty)) and, with a
    capacity, the record of the kept sets (count [B,n], indices and scaled logits [B,n,capacity]) that lets the
    backward write a gradient row without reading the logits."""
    _need_gpu(logits, targets)
    b, s, v = logits.shape
    dummy = targets if targets is not None else torch.zeros((b, max(n_inner, 1)), dtype=torch.int64, device=logits.device)
    rows = _rows(logits, dummy, n_inner, 0, v, temperature, temp_mode)
    if targets is None:
        rows.targets = 0
    dev = logits.device
    with torch.cuda.device(dev):
        f32 = dict(dtype=torch.float32, device=dev)
        lp = torch.empty((b, n_inner) if targets is not None else (0,), **f32)
        thr = torch.empty((b, n_inner), **f32)
        tie = torch.empty((b, n_inner), dtype=torch.int32, device=dev)
        lse = torch.empty((b, n_inner), **f32)
        lpu = torch.empty((b, n_inner) if want_unfiltered else (0,), **f32)
        rec = None
        if capacity > 0:
            rec = (torch.empty((b, n_inner), dtype=torch.int32, device=dev),
                   torch.empty((b, n_inner, capacity), dtype=torch.int32, device=dev),
                   torch.empty((b, n_inner, capacity), **f32))
        with _timed("topk_topp_fwd"):
            code = _lib.load().nrl_topk_topp_logprob_fwd(
                C.byref(rows), int(top_k), float(top_p), _ptr(lp if targets is not None else None), _ptr(thr), _ptr(tie),
                _ptr(lse), _ptr(lpu if want_unfiltered else None), None, _ptr(rec[0] if rec else None),
                _ptr(rec[1] if rec else None), _ptr(rec[2] if rec else None), int(capacity), _stream(),
            )
    _lib.check(code, "nrl_topk_topp_logprob_fwd")
    if capacity > 0:
        return (lp, thr, tie, lse, lpu) + rec
    return lp, thr, tie, lse, lpu


def _topk_topp_logprob_fwd_rec(logits, targets, n_inner, top_k, top_p, temperature, temp_mode, want_unfiltered, capacity):
    if capacity < 1:
        raise ValueError("the kept-set record needs a capacity of at least 1")
    return _topk_topp_logprob_fwd(logits, targets, n_inner, top_k, top_p, temperature, temp_mode, want_unfiltered, capacity)


def _topk_topp_logprob_bwd(logits, targets, thr, tie, lse_kept, grad, n_inner, temperature, temp_mode, kept_n=None,
                           kept_idx=None, kept_x=None):
    _need_gpu(logits, targets, thr, tie, lse_kept, grad, kept_n, kept_idx, kept_x)
    b, s, v = logits.shape
    rows = _rows(logits, targets, n_inner, 0, v, temperature, temp_mode)
    for t, name in ((thr, "thr"), (tie, "tie"), (lse_kept, "lse_kept")):
        if tuple(t.shape) != (b, n_inner) or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous [B, n_inner] tensor")
    if thr.dtype != torch.float32 or lse_kept.dtype != torch.float32 or tie.dtype != torch.int32:
        raise ValueError("thr / lse_kept must be fp32 and tie int32")
    if tuple(grad.shape) != (b, n_inner) or grad.dtype != torch.float32:
        raise ValueError("grad must be fp32 [B, n_inner]")
    capacity = 0
    if kept_n is not None:
        if kept_idx is None or kept_x is None:
            raise ValueError("the kept-set record is (count, indices, values): all three or none")
        capacity = kept_idx.shape[-1]
        ok = (kept_n.dtype == torch.int32 and kept_idx.dtype == torch.int32 and kept_x.dtype == torch.float32
              and tuple(kept_n.shape) == (b, n_inner) and tuple(kept_idx.shape) == (b, n_inner, capacity)
              and tuple(kept_x.shape) == (b, n_inner, capacity)
              and kept_n.is_contiguous() and kept_idx.is_contiguous() and kept_x.is_contiguous() and capacity >= 1)
        if not ok:
            raise ValueError("kept-set record: int32 [B, n], int32 [B, n, capacity], fp32 [B, n, capacity], contiguous")
    with torch.cuda.device(logits.device):
        d = _grad_buffer((b, s, v), logits)
        with _timed("topk_topp_bwd"):
            code = _lib.load().nrl_topk_topp_logprob_bwd(
                C.byref(rows), _ptr(thr), _ptr(tie), _ptr(lse_kept), _ptr(grad), grad.stride(0), grad.stride(1),
                _ptr(kept_n), _ptr(kept_idx), _ptr(kept_x), capacity, _ptr(d), s, d.stride(0), d.stride(1), _stream(),
            )
    _lib.check(code, "nrl_topk_topp_logprob_bwd")
    return d


def _topk_topp_filter(logits, thr, tie, temperature, temp_mode):
    _need_gpu(logits, thr, tie)
    b, s, v = logits.shape
    dummy = torch.zeros((b, max(s, 1)), dtype=torch.int64, device=logits.device)
    rows = _rows(logits, dummy, s, 0, v, temperature, temp_mode)
    rows.targets = 0
    if tuple(thr.shape) != (b, s) or tuple(tie.shape) != (b, s) or not thr.is_contiguous() or not tie.is_contiguous():
        raise ValueError("thr / tie must be contiguous [B, S]")
    with torch.cuda.device(logits.device):
        out = torch.empty((b, s, v), dtype=logits.dtype, device=logits.device)
        keep = torch.empty((b, s, v), dtype=torch.uint8, device=logits.device)
        code = _lib.load().nrl_topk_topp_filter(
            C.byref(rows), _ptr(thr), _ptr(tie), _ptr(out), out.stride(0), out.stride(1), _ptr(keep), _stream()
        )
    _lib.check(code, "nrl_topk_topp_filter")
    return out, keep


for _name, _fn in (("topk_topp_logprob_fwd", _topk_topp_logprob_fwd), ("topk_topp_logprob_fwd_rec", _topk_topp_logprob_fwd_rec),
                   ("topk_topp_logprob_bwd", _topk_topp_logprob_bwd),
                   ("topk_topp_filter", _topk_topp_filter)):
    _LIB.impl(_name, _fn, "CUDA")
    _LIB.impl(_name, _fn, "CPU")


# ------------------------------------------------------------------------------------------------
# K4
# ------------------------------------------------------------------------------------------------
_LIB.define(
    "grpo_loss(Tensor lp, Tensor? lpu, Tensor? prev, Tensor gen, Tensor? ref, Tensor adv, Tensor token_mask, "
    "Tensor sample_mask, Tensor? correct_mask, Tensor global_valid, int[] iflags, float[] fparams) "
    "-> (Tensor, Tensor, Tensor, Tensor)"
)
_LIB.define(
    "nll_loss(Tensor lp, Tensor token_mask, Tensor sample_mask, Tensor global_valid) -> (Tensor, Tensor, Tensor)"
)

_CFG_INT = [n for n, _ in _lib.NrlGrpoCfg._fields_[:14]]
_CFG_FLT = [n for n, _ in _lib.NrlGrpoCfg._fields_[14:]]


def _rowmat(t, b, n, name):
    """fp32 [B, n] with unit column stride -> (tensor kept alive, row stride)."""
    if t is None:
        return None, 0
    if t.dtype != torch.float32 or tuple(t.shape) != (b, n):
        raise ValueError(f"{name} must be fp32 [{b}, {n}], got {t.dtype} {tuple(t.shape)}")
    if n > 1 and t.stride(1) != 1:
        t = t.contiguous()
    return t, (t.stride(0) if b > 1 else n)


def _vec(t, b, name):
    if t is None:
        return None
    if t.dtype != torch.float32 or tuple(t.shape) != (b,):
        raise ValueError(f"{name} must be fp32 [{b}], got {t.dtype} {tuple(t.shape)}")
    return t.contiguous()


def _grpo_inputs(lp, lpu, prev, gen, ref, adv, token_mask, sample_mask, correct_mask, global_valid):
    _need_gpu(lp, lpu, prev, gen, ref, adv, token_mask, sample_mask, correct_mask, global_valid)
    if lp.dim() != 2:
        raise ValueError(f"logprobs must be [B, S-1], got {tuple(lp.shape)}")
    b, n = lp.shape
    keep = []
    inp = _lib.NrlGrpoInputs()
    inp.batch, inp.sm1 = b, n
    for field, t in (("lp", lp), ("lpu", lpu), ("prev", prev), ("gen", gen), ("ref", ref), ("adv", adv),
                     ("token_mask", token_mask)):
        t, stride = _rowmat(t, b, n, field)
        keep.append(t)
        setattr(inp, field, 0 if t is None else t.data_ptr())
        setattr(inp, field + "_stride", stride)
    sm, cm = _vec(sample_mask, b, "sample_mask"), _vec(correct_mask, b, "correct_mask")
    if global_valid.dtype != torch.float32 or tuple(global_valid.shape) != (2,):
        raise ValueError("global_valid must be fp32 [2] = (valid_seqs, valid_toks)")
    gv = global_valid.contiguous()
    keep += [sm, cm, gv]
    inp.sample_mask = sm.data_ptr()
    inp.correct_mask = 0 if cm is None else cm.data_ptr()
    inp.global_valid = gv.data_ptr()
    return inp, keep, b, n


def _grpo_loss(lp, lpu, prev, gen, ref, adv, token_mask, sample_mask, correct_mask, global_valid, iflags, fparams):
    if len(iflags) != len(_CFG_INT) or len(fparams) != len(_CFG_FLT):
        raise ValueError("malformed loss configuration")
    inp, keep, b, n = _grpo_inputs(lp, lpu, prev, gen, ref, adv, token_mask, sample_mask, correct_mask, global_valid)
    cfg = _lib.NrlGrpoCfg()
    for name, v in zip(_CFG_INT, iflags):
        setattr(cfg, name, int(v))
    for name, v in zip(_CFG_FLT, fparams):
        setattr(cfg, name, float(v))
    lib = _lib.load()
    dev = lp.device
    split = lpu is not None and cfg.has_kl
    with torch.cuda.device(dev):
        loss = torch.empty((), dtype=torch.float32, device=dev)
        dlp = torch.empty((b, n), dtype=torch.float32, device=dev)
        dlpu = torch.empty((b, n) if split else (0,), dtype=torch.float32, device=dev)
        metrics = torch.empty((_lib.NRL_GRPO_N_METRICS,), dtype=torch.float32, device=dev)
        ws_bytes = lib.nrl_grpo_loss_workspace_bytes(b)
        ws = torch.empty((ws_bytes // 8,), dtype=torch.float64, device=dev)
        with _timed("grpo_loss"):
            code = lib.nrl_grpo_loss_fwd_bwd(
                C.byref(cfg), C.byref(inp), _ptr(loss), _ptr(dlp), _ptr(dlpu if split else None), _ptr(metrics),
                _ptr(ws), ws_bytes, _stream(),
            )
    _lib.check(code, "nrl_grpo_loss_fwd_bwd")
    del keep
    return loss, dlp, dlpu, metrics


_LIB.define(
    "fused_logits_grpo_loss(Tensor logits, Tensor targets, int n_inner, Tensor? prev, Tensor gen, Tensor? ref, Tensor adv, "
    "Tensor token_mask, Tensor sample_mask, Tensor global_valid, int[] iflags, float[] fparams, float loss_scale, "
    "float temperature, int temp_mode) -> (Tensor, Tensor, Tensor, Tensor)"
)
_LIB.define(
    "fused_logits_grpo_loss_(Tensor(a!) logits, Tensor targets, int n_inner, Tensor? prev, Tensor gen, Tensor? ref, Tensor adv, "
    "Tensor token_mask, Tensor sample_mask, Tensor global_valid, int[] iflags, float[] fparams, float loss_scale, "
    "float temperature, int temp_mode) -> (Tensor, Tensor, Tensor)"
)


def _fused_logits_grpo_loss(logits, targets, n_inner, prev, gen, ref, adv, token_mask, sample_mask, global_valid, iflags,
                            fparams, loss_scale, temperature, temp_mode, in_place=False):
    """-> (loss, dlogits, logprobs [B, n_inner], metrics).  ``temperature`` != 1 divides the logits inside the
    pass the way an in-place ``div_`` of the tensor would have rounded them (``temp_mode``: on the GPU or the CPU)."""
    if len(iflags) != len(_CFG_INT) or len(fparams) != len(_CFG_FLT):
        raise ValueError("malformed loss configuration")
    _need_gpu(logits, targets)
    b, s, v = logits.shape
    rows = _rows(logits, targets, n_inner, 0, v, float(temperature), int(temp_mode))
    dev = logits.device
    lp_shape = torch.empty((b, n_inner), dtype=torch.float32, device=dev)
    inp, keep, _, _ = _grpo_inputs(lp_shape, None, prev, gen, ref, adv, token_mask, sample_mask, None, global_valid)
    cfg = _lib.NrlGrpoCfg()
    for name, val in zip(_CFG_INT, iflags):
        setattr(cfg, name, int(val))
    for name, val in zip(_CFG_FLT, fparams):
        setattr(cfg, name, float(val))
    lib = _lib.load()
    with torch.cuda.device(dev):
        loss = torch.empty((), dtype=torch.float32, device=dev)
        metrics = torch.empty((_lib.NRL_GRPO_N_METRICS,), dtype=torch.float32, device=dev)
        d = logits if in_place else _grad_buffer((b, s, v), logits)
        ws_bytes = lib.nrl_fused_workspace_bytes(b, n_inner)
        ws = torch.empty(((ws_bytes + 7) // 8,), dtype=torch.float64, device=dev)
        with _timed("fused_logits_loss"):
            code = lib.nrl_fused_logits_grpo_loss(
                C.byref(rows), C.byref(cfg), C.byref(inp), float(loss_scale), _ptr(d), s, d.stride(0), d.stride(1),
                _ptr(lp_shape), _ptr(loss), _ptr(metrics), _ptr(ws), ws.numel() * 8, _stream(),
            )
    if code == -2:
        raise NotImplementedError(lib.nrl_last_error().decode(errors="replace"))
    _lib.check(code, "nrl_fused_logits_grpo_loss")
    del keep
    return loss, d, lp_shape, metrics


def _fused_logits_grpo_loss_inplace(logits, targets, n_inner, prev, gen, ref, adv, token_mask, sample_mask, global_valid,
                                    iflags, fparams, loss_scale, temperature, temp_mode):
    loss, _, lp, metrics = _fused_logits_grpo_loss(logits, targets, n_inner, prev, gen, ref, adv, token_mask, sample_mask,
                                                   global_valid, iflags, fparams, loss_scale, temperature, temp_mode,
                                                   in_place=True)
    return loss, lp, metrics


for _name, _fn in (("fused_logits_grpo_loss", _fused_logits_grpo_loss), ("fused_logits_grpo_loss_", _fused_logits_grpo_loss_inplace)):
    _LIB.impl(_name, _fn, "CUDA")
    _LIB.impl(_name, _fn, "CPU")

_LIB.define(
    "fused_packed_logits_grpo_loss(Tensor logits, Tensor targets, bool pre_rolled, Tensor cu_seqlens, int unpacked_seqlen, "
    "Tensor? prev, Tensor gen, Tensor? ref, Tensor adv, Tensor token_mask, Tensor sample_mask, Tensor global_valid, "
    "int[] iflags, float[] fparams, float loss_scale, float temperature, int temp_mode) "
    "-> (Tensor, Tensor, Tensor, Tensor)"
)


def _fused_packed_logits_grpo_loss(logits, targets, pre_rolled, cu_seqlens, unpacked_seqlen, prev, gen, ref, adv, token_mask,
                                   sample_mask, global_valid, iflags, fparams, loss_scale, temperature, temp_mode):
    """Packed [T, V] logits -> (loss, dlogits [T, V], logprobs [n_seq, unpacked_seqlen - 1], metrics)."""
    if len(iflags) != len(_CFG_INT) or len(fparams) != len(_CFG_FLT):
        raise ValueError("malformed loss configuration")
    _check_packed(logits, targets, cu_seqlens, unpacked_seqlen)
    t, v = logits.shape
    n_seq, n_inner = cu_seqlens.shape[0] - 1, unpacked_seqlen - 1
    rows = _lib.NrlRows()
    rows.logits = logits.data_ptr()
    rows.dtype = _dtype_code(logits)
    rows.n_outer, rows.n_inner, rows.vocab = 1, t, v
    rows.stride_outer, rows.stride_inner = 0, logits.stride(0)
    rows.targets = targets.data_ptr()
    rows.tgt_stride_outer, rows.tgt_stride_inner = 0, 1
    rows.vocab_start, rows.vocab_end = 0, v
    rows.temperature, rows.temp_mode = float(temperature), int(temp_mode)
    dev = logits.device
    lp = torch.empty((n_seq, n_inner), dtype=torch.float32, device=dev)
    inp, keep, _, _ = _grpo_inputs(lp, None, prev, gen, ref, adv, token_mask, sample_mask, None, global_valid)
    cfg = _lib.NrlGrpoCfg()
    for name, val in zip(_CFG_INT, iflags):
        setattr(cfg, name, int(val))
    for name, val in zip(_CFG_FLT, fparams):
        setattr(cfg, name, float(val))
    lib = _lib.load()
    with torch.cuda.device(dev):
        loss = torch.empty((), dtype=torch.float32, device=dev)
        metrics = torch.empty((_lib.NRL_GRPO_N_METRICS,), dtype=torch.float32, device=dev)
        d = _grad_buffer((t, v), logits)
        ws_bytes = lib.nrl_fused_packed_workspace_bytes(n_seq, n_inner, t)
        ws = torch.empty(((ws_bytes + 7) // 8,), dtype=torch.float64, device=dev)
        with _timed("fused_packed_logits_loss"):
            code = lib.nrl_fused_packed_logits_grpo_loss(
                C.byref(rows), int(pre_rolled), _ptr(cu_seqlens), n_seq, C.byref(cfg), C.byref(inp), float(loss_scale),
                _ptr(d), d.stride(0), _ptr(lp), _ptr(loss), _ptr(metrics), _ptr(ws), ws.numel() * 8, _stream(),
            )
    if code == -2:
        raise NotImplementedError(lib.nrl_last_error().decode(errors="replace"))
    _lib.check(code, "nrl_fused_packed_logits_grpo_loss")
    del keep
    return loss, d, lp, metrics


_LIB.impl("fused_packed_logits_grpo_loss", _fused_packed_logits_grpo_loss, "CUDA")
_LIB.impl("fused_packed_logits_grpo_loss", _fused_packed_logits_grpo_loss, "CPU")


def _nll_loss(lp, token_mask, sample_mask, global_valid):
    inp, keep, b, n = _grpo_inputs(lp, None, None, None, None, None, token_mask, sample_mask, None, global_valid)
    lib = _lib.load()
    dev = lp.device
    with torch.cuda.device(dev):
        loss = torch.empty((), dtype=torch.float32, device=dev)
        dlp = torch.empty((b, n), dtype=torch.float32, device=dev)
        metrics = torch.empty((3,), dtype=torch.float32, device=dev)
        ws_bytes = lib.nrl_grpo_loss_workspace_bytes(b)
        ws = torch.empty((ws_bytes // 8,), dtype=torch.float64, device=dev)
        code = lib.nrl_nll_loss_fwd_bwd(C.byref(inp), _ptr(loss), _ptr(dlp), _ptr(metrics), _ptr(ws), ws_bytes, _stream())
    _lib.check(code, "nrl_nll_loss_fwd_bwd")
    del keep
    return loss, dlp, metrics


for _name, _fn in (("grpo_loss", _grpo_loss), ("nll_loss", _nll_loss)):
    _LIB.impl(_name, _fn, "CUDA")
    _LIB.impl(_name, _fn, "CPU")


# the loss helpers that are also called on their own (KL in the reward, mean reward)
_LIB.define("calculate_kl(Tensor lp, Tensor ref, Tensor? weights, int kl_type, float? input_clamp, float? output_clamp) -> Tensor")
_LIB.define(
    "calculate_kl_bwd(Tensor grad, Tensor lp, Tensor ref, Tensor? weights, int kl_type, float? input_clamp, "
    "float? output_clamp, bool need_lp, bool need_ref, bool need_weights) -> (Tensor, Tensor, Tensor)"
)
_LIB.define("masked_mean_rows(Tensor values, Tensor mask, Tensor? norm) -> (Tensor, Tensor)")
_LIB.define("masked_mean_rows_bwd(Tensor grad, Tensor mask, Tensor denom) -> Tensor")


def _flat_f32(*tensors):
    for t in tensors:
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous()):
            raise ValueError("expected contiguous fp32 tensors")
    shapes = {tuple(t.shape) for t in tensors if t is not None}
    if len(shapes) > 1:
        raise ValueError(f"shapes differ: {sorted(shapes)}")


def _clamp_args(value):
    return (0, 0.0) if value is None else (1, float(value))


def _calculate_kl(lp, ref, weights, kl_type, input_clamp, output_clamp):
    _need_gpu(lp, ref, weights)
    _flat_f32(lp, ref, weights)
    out = torch.empty_like(lp)
    with torch.cuda.device(lp.device):
        code = _lib.load().nrl_calculate_kl(_ptr(lp), _ptr(ref), _ptr(weights), lp.numel(), int(kl_type),
                                            *_clamp_args(input_clamp), *_clamp_args(output_clamp), _ptr(out), _stream())
    _lib.check(code, "nrl_calculate_kl")
    return out


def _calculate_kl_bwd(grad, lp, ref, weights, kl_type, input_clamp, output_clamp, need_lp, need_ref, need_weights):
    _need_gpu(grad, lp, ref, weights)
    _flat_f32(grad, lp, ref, weights)
    empty = lp.new_empty(0)
    d_lp = torch.empty_like(lp) if need_lp else None
    d_ref = torch.empty_like(lp) if need_ref else None
    d_w = torch.empty_like(lp) if need_weights and weights is not None else None
    with torch.cuda.device(lp.device):
        code = _lib.load().nrl_calculate_kl_bwd(_ptr(grad), _ptr(lp), _ptr(ref), _ptr(weights), lp.numel(), int(kl_type),
                                                *_clamp_args(input_clamp), *_clamp_args(output_clamp), _ptr(d_lp),
                                                _ptr(d_ref), _ptr(d_w), _stream())
    _lib.check(code, "nrl_calculate_kl_bwd")
    return tuple(empty if t is None else t for t in (d_lp, d_ref, d_w))


def _masked_mean_rows(values, mask, norm):
    _need_gpu(values, mask, norm)
    _flat_f32(values, mask)
    if values.dim() != 2:
        raise ValueError(f"expected [rows, cols], got {tuple(values.shape)}")
    if norm is not None and (norm.numel() != 1 or norm.dtype != torch.float32):
        raise ValueError("the normalisation factor must be one fp32 value")
    rows, cols = values.shape
    out = values.new_empty(rows)
    denom = values.new_empty(rows)
    with torch.cuda.device(values.device):
        code = _lib.load().nrl_masked_mean(_ptr(values), _ptr(mask), rows, cols, _ptr(norm), 0.0, int(norm is not None),
                                           _ptr(out), _ptr(denom), _stream())
    _lib.check(code, "nrl_masked_mean")
    return out, denom


def _masked_mean_rows_bwd(grad, mask, denom):
    _need_gpu(grad, mask, denom)
    rows, cols = mask.shape
    out = torch.empty_like(mask)
    with torch.cuda.device(mask.device):
        code = _lib.load().nrl_masked_mean_bwd(_ptr(grad), _ptr(mask), _ptr(denom), rows, cols, _ptr(out), _stream())
    _lib.check(code, "nrl_masked_mean_bwd")
    return out


for _name, _fn in (("calculate_kl", _calculate_kl), ("calculate_kl_bwd", _calculate_kl_bwd),
                   ("masked_mean_rows", _masked_mean_rows), ("masked_mean_rows_bwd", _masked_mean_rows_bwd)):
    _LIB.impl(_name, _fn, "CUDA")
    _LIB.impl(_name, _fn, "CPU")


_LIB.define("topk_logsoftmax_fwd(Tensor logits, Tensor? indices) -> Tensor")
_LIB.define("topk_logsoftmax_bwd(Tensor logits, Tensor indices, Tensor logprobs, Tensor grad) -> Tensor")
_LIB.define(
    "distill_topk_loss(Tensor student_logprobs, Tensor teacher_logprobs, Tensor? h_all, Tensor? token_mask, "
    "Tensor? sample_mask, Tensor? global_valid_toks, int kl_type, float mixed_kl_weight, bool zero_outside_topk, "
    "float log_infinitesimal) -> (Tensor, Tensor, Tensor)"
)


def _topk_logsoftmax_fwd(logits, indices):
    """log_softmax over the K logits at ``indices`` [B, S, K] of every row (or over the whole last axis)."""
    _need_gpu(logits, indices)
    rows = _plain_rows(logits)
    b, s, v = logits.shape
    if indices is not None:
        indices = _gather_indices(logits, indices)
    k = v if indices is None else indices.shape[2]
    with torch.cuda.device(logits.device):
        out = torch.empty((b, s, k), dtype=torch.float32, device=logits.device)
        code = _lib.load().nrl_topk_logsoftmax_fwd(C.byref(rows), _ptr(indices), k, _ptr(out), _stream())
    _lib.check(code, "nrl_topk_logsoftmax_fwd")
    return out


def _topk_logsoftmax_bwd(logits, indices, logprobs, grad):
    _need_gpu(logits, indices, logprobs, grad)
    rows = _plain_rows(logits)
    indices = _gather_indices(logits, indices)
    b, s, k = indices.shape
    for name, t in (("logprobs", logprobs), ("grad", grad)):
        if t.dtype != torch.float32 or tuple(t.shape) != (b, s, k):
            raise ValueError(f"{name} must be fp32 [{b}, {s}, {k}], got {t.dtype} {tuple(t.shape)}")
    logprobs, grad = logprobs.contiguous(), grad.contiguous()
    with torch.cuda.device(logits.device):
        d = _grad_buffer(logits.shape, logits)
        code = _lib.load().nrl_topk_logsoftmax_bwd(C.byref(rows), _ptr(indices), k, _ptr(logprobs), _ptr(grad), _ptr(d),
                                                   d.stride(0), d.stride(1), _stream())
    _lib.check(code, "nrl_topk_logsoftmax_bwd")
    return d


def _distill_topk_loss(student_logprobs, teacher_logprobs, h_all, token_mask, sample_mask, global_valid_toks, kl_type,
                       mixed_kl_weight, zero_outside_topk, log_infinitesimal):
    """-> (loss, d loss / d student_logprobs [B, n, K], d loss / d h_all [B, n] (empty without the correction))."""
    _need_gpu(student_logprobs, teacher_logprobs, h_all, token_mask, sample_mask, global_valid_toks)
    if student_logprobs.dim() != 3 or student_logprobs.shape != teacher_logprobs.shape:
        raise ValueError(f"student / teacher logprobs must both be [B, n, K], got {tuple(student_logprobs.shape)} and "
                         f"{tuple(teacher_logprobs.shape)}")
    if student_logprobs.dtype != torch.float32 or teacher_logprobs.dtype != torch.float32:
        raise ValueError("top-k logprobs must be fp32")
    b, n, k = student_logprobs.shape
    sl, tl = student_logprobs.contiguous(), teacher_logprobs.contiguous()
    correct = bool(zero_outside_topk) and kl_type != 0
    if correct:
        if h_all is None:
            raise ValueError("H_all is required when zero_outside_topk is set and the KL is not the forward one")
        h_all = _row_scalar(h_all, b, n, "H_all")
    tm, tm_stride = (None, 0) if token_mask is None else _rowmat(token_mask, b, n, "token_mask")
    sm = _vec(sample_mask, b, "sample_mask")
    if tm is not None and (sm is None or global_valid_toks is None):
        raise ValueError("token_mask needs sample_mask and global_valid_toks")
    gv = None if global_valid_toks is None else global_valid_toks.reshape(-1)[:1].to(torch.float32).contiguous()
    lib = _lib.load()
    dev = sl.device
    with torch.cuda.device(dev):
        loss = torch.empty((), dtype=torch.float32, device=dev)
        d_s = torch.empty((b, n, k), dtype=torch.float32, device=dev)
        d_h = torch.empty((b, n) if correct else (0,), dtype=torch.float32, device=dev)
        ws_bytes = lib.nrl_distill_topk_loss_workspace_bytes(b, n)
        ws = torch.empty(((ws_bytes + 7) // 8,), dtype=torch.float64, device=dev)
        code = lib.nrl_distill_topk_loss_fwd_bwd(
            _ptr(sl), _ptr(tl), _ptr(h_all if correct else None), _ptr(tm), tm_stride, _ptr(sm), _ptr(gv), b, n, k, int(kl_type),
            float(mixed_kl_weight), int(bool(zero_outside_topk)), float(log_infinitesimal), _ptr(loss), _ptr(d_s),
            _ptr(d_h if correct else None), _ptr(ws), ws.numel() * 8, _stream(),
        )
    _lib.check(code, "nrl_distill_topk_loss_fwd_bwd")
    return loss, d_s, d_h


for _name, _fn in (("topk_logsoftmax_fwd", _topk_logsoftmax_fwd), ("topk_logsoftmax_bwd", _topk_logsoftmax_bwd),
                   ("distill_topk_loss", _distill_topk_loss)):
    _LIB.impl(_name, _fn, "CUDA")
    _LIB.impl(_name, _fn, "CPU")


_LIB.define("nonzero_indices(Tensor values) -> Tensor")


def _nonzero_indices(values):
    """Ascending int64 indices of the non-zero entries of a 1-D fp32 tensor."""
    _need_gpu(values)
    if values.dim() != 1 or values.dtype != torch.float32:
        raise ValueError(f"values must be fp32 [n], got {values.dtype} {tuple(values.shape)}")
    v = values.contiguous()
    n = v.shape[0]
    dev = v.device
    with torch.cuda.device(dev):
        idx = torch.empty((max(n, 1),), dtype=torch.int32, device=dev)
        count = torch.empty((1,), dtype=torch.int32, device=dev)
        code = _lib.load().nrl_nonzero_indices(_ptr(v), n, _ptr(idx), _ptr(count), _stream())
    _lib.check(code, "nrl_nonzero_indices")
    return idx[: int(count.item())].to(torch.int64)


_LIB.impl("nonzero_indices", _nonzero_indices, "CUDA")
_LIB.impl("nonzero_indices", _nonzero_indices, "CPU")


# ------------------------------------------------------------------------------------------------
# preference losses (DPO, reward model) and the per-sample NLL rows
# ------------------------------------------------------------------------------------------------
_LIB.define("nll_rows_fwd(Tensor lp, Tensor token_mask, Tensor sample_mask, bool average) -> (Tensor, Tensor, Tensor)")
_LIB.define("nll_rows_bwd(Tensor grad_rows, Tensor token_mask, Tensor sample_mask, Tensor den) -> Tensor")
_LIB.define(
    "dpo_loss(Tensor lp, Tensor? ref, Tensor token_mask, Tensor sample_mask, Tensor global_valid, float beta, "
    "float preference_loss_weight, float sft_loss_weight, bool preference_average_log_probs, bool sft_average_log_probs) "
    "-> (Tensor, Tensor, Tensor)"
)
_LIB.define("preference_loss(Tensor rewards, Tensor sample_mask, Tensor global_valid) -> (Tensor, Tensor, Tensor)")


def _lp_and_masks(lp, token_mask, sample_mask):
    _need_gpu(lp, token_mask, sample_mask)
    if lp.dim() != 2:
        raise ValueError(f"logprobs must be [B, S-1], got {tuple(lp.shape)}")
    b, n = lp.shape
    lp, lp_stride = _rowmat(lp, b, n, "logprobs")
    tm, tm_stride = _rowmat(token_mask, b, n, "token_mask")
    return b, n, lp, lp_stride, tm, tm_stride, _vec(sample_mask, b, "sample_mask")


def _nll_rows_fwd(lp, token_mask, sample_mask, average):
    """-> (per-sample loss [B], divisor [B], (num_unmasked_tokens, num_valid_samples))."""
    b, n, lp, lp_stride, tm, tm_stride, sm = _lp_and_masks(lp, token_mask, sample_mask)
    dev = lp.device
    with torch.cuda.device(dev):
        rows = torch.empty((b,), dtype=torch.float32, device=dev)
        den = torch.empty((b,), dtype=torch.float32, device=dev)
        totals = torch.empty((2,), dtype=torch.float32, device=dev)
        ws = torch.empty((max(b, 1),), dtype=torch.float32, device=dev)
        code = _lib.load().nrl_nll_rows_fwd(_ptr(lp), lp_stride, _ptr(tm), tm_stride, _ptr(sm), b, n, int(average), _ptr(rows),
                                            _ptr(den), _ptr(totals), _ptr(ws), ws.numel() * 4, _stream())
    _lib.check(code, "nrl_nll_rows_fwd")
    return rows, den, totals


def _nll_rows_bwd(grad_rows, token_mask, sample_mask, den):
    _need_gpu(grad_rows, token_mask, sample_mask, den)
    b, n = token_mask.shape
    tm, tm_stride = _rowmat(token_mask, b, n, "token_mask")
    g, sm, den = _vec(grad_rows, b, "grad_rows"), _vec(sample_mask, b, "sample_mask"), _vec(den, b, "den")
    dev = tm.device
    with torch.cuda.device(dev):
        dlp = torch.empty((b, n), dtype=torch.float32, device=dev)
        code = _lib.load().nrl_nll_rows_bwd(_ptr(g), _ptr(tm), tm_stride, _ptr(sm), _ptr(den), b, n, _ptr(dlp), _stream())
    _lib.check(code, "nrl_nll_rows_bwd")
    return dlp


def _dpo_loss(lp, ref, token_mask, sample_mask, global_valid, beta, preference_loss_weight, sft_loss_weight,
              preference_average_log_probs, sft_average_log_probs):
    """-> (loss, d loss / d logprobs [B, n], metrics[7])."""
    _need_gpu(ref, global_valid)
    b, n, lp, lp_stride, tm, tm_stride, sm = _lp_and_masks(lp, token_mask, sample_mask)
    ref, ref_stride = _rowmat(ref, b, n, "reference_policy_logprobs")
    if global_valid.dtype != torch.float32 or global_valid.numel() < 1:
        raise ValueError("global_valid must be an fp32 tensor whose first element is the number of valid sequences")
    gv = global_valid.contiguous()
    lib = _lib.load()
    dev = lp.device
    with torch.cuda.device(dev):
        loss = torch.empty((), dtype=torch.float32, device=dev)
        dlp = torch.empty((b, n), dtype=torch.float32, device=dev)
        metrics = torch.empty((7,), dtype=torch.float32, device=dev)
        ws_bytes = lib.nrl_dpo_workspace_bytes(b)
        ws = torch.empty(((ws_bytes + 3) // 4,), dtype=torch.float32, device=dev)
        code = lib.nrl_dpo_loss_fwd_bwd(
            _ptr(lp), lp_stride, _ptr(ref), ref_stride, _ptr(tm), tm_stride, _ptr(sm), _ptr(gv), b, n, float(beta),
            float(preference_loss_weight), float(sft_loss_weight), int(preference_average_log_probs),
            int(sft_average_log_probs), _ptr(loss), _ptr(dlp), _ptr(metrics), _ptr(ws), ws.numel() * 4, _stream(),
        )
    _lib.check(code, "nrl_dpo_loss_fwd_bwd")
    return loss, dlp, metrics


def _preference_loss(rewards, sample_mask, global_valid):
    """-> (loss, d loss / d rewards [B], metrics[5])."""
    _need_gpu(rewards, sample_mask, global_valid)
    if rewards.dim() != 1:
        raise ValueError(f"rewards must be [B], got {tuple(rewards.shape)}")
    b = rewards.shape[0]
    r, sm = _vec(rewards, b, "rewards"), _vec(sample_mask, b, "sample_mask")
    if global_valid.dtype != torch.float32 or global_valid.numel() < 1:
        raise ValueError("global_valid must be an fp32 tensor whose first element is the number of valid sequences")
    gv = global_valid.contiguous()
    dev = r.device
    with torch.cuda.device(dev):
        loss = torch.empty((), dtype=torch.float32, device=dev)
        dr = torch.zeros((b,), dtype=torch.float32, device=dev)
        metrics = torch.empty((5,), dtype=torch.float32, device=dev)
        code = _lib.load().nrl_preference_loss_fwd_bwd(_ptr(r), _ptr(sm), _ptr(gv), b, _ptr(loss), _ptr(dr), _ptr(metrics),
                                                       _stream())
    _lib.check(code, "nrl_preference_loss_fwd_bwd")
    return loss, dr, metrics


for _name, _fn in (("nll_rows_fwd", _nll_rows_fwd), ("nll_rows_bwd", _nll_rows_bwd), ("dpo_loss", _dpo_loss),
                   ("preference_loss", _preference_loss)):
    _LIB.impl(_name, _fn, "CUDA")
    _LIB.impl(_name, _fn, "CPU")


# ------------------------------------------------------------------------------------------------
# K5
# ------------------------------------------------------------------------------------------------
_LIB.define(
    "group_baseline_std(Tensor prompts, Tensor rewards, Tensor valid, Tensor? std_rewards, bool leave_one_out, "
    "bool normalize) -> (Tensor, Tensor, Tensor, Tensor)"
)


def _group_baseline_std(prompts, rewards, valid, std_rewards, leave_one_out, normalize):
    _need_gpu(prompts, rewards, valid, std_rewards)
    if prompts.dim() == 1:
        prompts = prompts.unsqueeze(-1)
    if prompts.dim() != 2 or prompts.dtype != torch.int64:
        raise ValueError(f"prompts must be int64 [B, Sp], got {prompts.dtype} {tuple(prompts.shape)}")
    b, sp = prompts.shape
    if sp > 1 and prompts.stride(1) != 1:
        prompts = prompts.contiguous()
    rewards, valid, std_rewards = _vec(rewards, b, "rewards"), _vec(valid, b, "valid_mask"), _vec(std_rewards, b, "std_rewards")
    lib = _lib.load()
    dev = rewards.device
    with torch.cuda.device(dev):
        baseline = torch.empty((b,), dtype=torch.float32, device=dev)
        std = torch.empty((b,), dtype=torch.float32, device=dev)
        adv = torch.empty((b,), dtype=torch.float32, device=dev)
        group = torch.empty((b,), dtype=torch.int32, device=dev)
        ws_bytes = lib.nrl_group_workspace_bytes(b)
        ws = torch.empty(((ws_bytes + 7) // 8,), dtype=torch.float64, device=dev)
        code = lib.nrl_group_baseline_std(
            _ptr(prompts), b, sp, prompts.stride(0) if b > 1 else sp, _ptr(rewards), _ptr(valid), _ptr(std_rewards),
            int(leave_one_out), int(normalize), _ptr(baseline), _ptr(std), _ptr(adv), _ptr(group), _ptr(ws),
            ws.numel() * 8, _stream(),
        )
    _lib.check(code, "nrl_group_baseline_std")
    return baseline, std, adv, group


_LIB.impl("group_baseline_std", _group_baseline_std, "CUDA")
_LIB.impl("group_baseline_std", _group_baseline_std, "CPU")

_LIB.define(
    "seq_logprob_error(Tensor prev, Tensor gen, Tensor token_mask, Tensor sample_mask, Tensor? rewards, "
    "float? threshold) -> (Tensor, Tensor, Tensor)"
)


def _seq_logprob_error(prev, gen, token_mask, sample_mask, rewards, threshold):
    """-> (per-sequence error [B], sample mask after the threshold [B], 8-float record)."""
    _need_gpu(prev, gen, token_mask, sample_mask, rewards)
    if prev.dim() != 2 or gen.shape != prev.shape or token_mask.shape != prev.shape:
        raise ValueError("prev_logprobs, generation_logprobs and token_mask must share one [B, S] shape")
    b, s = prev.shape

    def rows(t, name):
        t = t.to(torch.float32)
        if s > 1 and t.stride(1) != 1:
            t = t.contiguous()
        return t

    prev, gen, token_mask = rows(prev, "prev"), rows(gen, "gen"), rows(token_mask, "token_mask")
    sample_mask = _vec(sample_mask, b, "sample_mask")
    rewards = _vec(rewards, b, "rewards") if rewards is not None else None
    lib = _lib.load()
    dev = prev.device
    with torch.cuda.device(dev):
        err = torch.empty((b,), dtype=torch.float32, device=dev)
        mask_out = torch.empty((b,), dtype=torch.float32, device=dev)
        record = torch.empty((8,), dtype=torch.float32, device=dev)
        ws = torch.empty((max(b, 1),), dtype=torch.float32, device=dev)
        code = lib.nrl_seq_logprob_error(
            _ptr(prev), prev.stride(0) if b > 1 else s, _ptr(gen), gen.stride(0) if b > 1 else s,
            _ptr(token_mask), token_mask.stride(0) if b > 1 else s, _ptr(sample_mask), _ptr(rewards), b, s,
            int(threshold is not None), float(threshold) if threshold is not None else 0.0,
            _ptr(err), _ptr(mask_out), _ptr(record), _ptr(ws), ws.numel() * 4, _stream(),
        )
    _lib.check(code, "nrl_seq_logprob_error")
    return err, mask_out, record


_LIB.impl("seq_logprob_error", _seq_logprob_error, "CUDA")
_LIB.impl("seq_logprob_error", _seq_logprob_error, "CPU")


# ------------------------------------------------------------------------------------------------
# distillation reductions (negative entropy, gathered logprobs, soft-target cross entropy)
# ------------------------------------------------------------------------------------------------
_LIB.define("neg_entropy_fwd(Tensor logits) -> (Tensor, Tensor)")
_LIB.define("neg_entropy_bwd(Tensor logits, Tensor lse, Tensor h, Tensor grad) -> Tensor")
_LIB.define("gather_logprob_fwd(Tensor logits, Tensor indices, int vocab_start, int vocab_end) -> (Tensor, Tensor)")
_LIB.define("gather_logprob_bwd(Tensor logits, Tensor indices, int vocab_start, int vocab_end, Tensor lse, Tensor grad) -> Tensor")
_LIB.define("soft_cross_entropy_fwd(Tensor student, Tensor teacher) -> (Tensor, Tensor, Tensor)")
_LIB.define("soft_cross_entropy_bwd(Tensor student, Tensor teacher, Tensor lse_student, Tensor lse_teacher, Tensor grad) -> Tensor")


def _plain_rows(logits, vocab_start=0, vocab_end=None):
    """nrl_rows for kernels that take no targets: logits [B, S, V] with a contiguous vocabulary axis."""
    if logits.dim() != 3:
        raise ValueError(f"expected logits [B, S, V], got {tuple(logits.shape)}")
    if logits.stride(2) != 1 and logits.shape[2] > 1:
        raise ValueError("the vocabulary axis of the logits must be contiguous")
    refuse_pending(logits, "this op")
    b, s, v = logits.shape
    r = _lib.NrlRows()
    r.logits = logits.data_ptr()
    r.dtype = _dtype_code(logits)
    r.n_outer, r.n_inner, r.vocab = b, s, v
    r.stride_outer, r.stride_inner = logits.stride(0), logits.stride(1)
    r.targets = None
    r.tgt_stride_outer = r.tgt_stride_inner = 0
    r.vocab_start, r.vocab_end = vocab_start, (vocab_start + v if vocab_end is None else vocab_end)
    r.temperature, r.temp_mode = 1.0, _lib.NRL_TEMP_RCP
    return r


def _row_scalar(t, b, s, name):
    if t.dtype != torch.float32 or tuple(t.shape) != (b, s):
        raise ValueError(f"{name} must be fp32 [{b}, {s}], got {t.dtype} {tuple(t.shape)}")
    return t.contiguous()


def _neg_entropy_fwd(logits):
    _need_gpu(logits)
    rows = _plain_rows(logits)
    b, s, _ = logits.shape
    with torch.cuda.device(logits.device):
        h = torch.empty((b, s), dtype=torch.float32, device=logits.device)
        lse = torch.empty((b, s), dtype=torch.float32, device=logits.device)
        with _timed("neg_entropy_fwd"):
            code = _lib.load().nrl_neg_entropy_fwd(C.byref(rows), _ptr(h), _ptr(lse), _stream())
    _lib.check(code, "nrl_neg_entropy_fwd")
    return h, lse


def _neg_entropy_bwd(logits, lse, h, grad):
    _need_gpu(logits, lse, h, grad)
    rows = _plain_rows(logits)
    b, s, _ = logits.shape
    lse, h, grad = _row_scalar(lse, b, s, "lse"), _row_scalar(h, b, s, "h"), _row_scalar(grad, b, s, "grad")
    with torch.cuda.device(logits.device):
        d = _grad_buffer(logits.shape, logits)
        with _timed("neg_entropy_bwd"):
            code = _lib.load().nrl_neg_entropy_bwd(C.byref(rows), _ptr(lse), _ptr(h), _ptr(grad), _ptr(d), d.stride(0), d.stride(1), _stream())
    _lib.check(code, "nrl_neg_entropy_bwd")
    return d


def _gather_indices(logits, indices):
    b, s, _ = logits.shape
    if indices.dtype != torch.int64 or indices.dim() != 3 or tuple(indices.shape[:2]) != (b, s):
        raise ValueError(f"indices must be int64 [{b}, {s}, K], got {indices.dtype} {tuple(indices.shape)}")
    return indices.contiguous()


def _gather_logprob_fwd(logits, indices, vocab_start, vocab_end):
    _need_gpu(logits, indices)
    rows = _plain_rows(logits, vocab_start, vocab_end)
    indices = _gather_indices(logits, indices)
    b, s, k = indices.shape
    with torch.cuda.device(logits.device):
        out = torch.empty((b, s, k), dtype=torch.float32, device=logits.device)
        lse = torch.empty((b, s), dtype=torch.float32, device=logits.device)
        with _timed("gather_logprob_fwd"):
            code = _lib.load().nrl_gather_logprob_fwd(C.byref(rows), _ptr(indices), k, _ptr(out), _ptr(lse), _stream())
    _lib.check(code, "nrl_gather_logprob_fwd")
    return out, lse


def _gather_logprob_bwd(logits, indices, vocab_start, vocab_end, lse, grad):
    _need_gpu(logits, indices, lse, grad)
    rows = _plain_rows(logits, vocab_start, vocab_end)
    indices = _gather_indices(logits, indices)
    b, s, k = indices.shape
    lse = _row_scalar(lse, b, s, "lse")
    if grad.dtype != torch.float32 or tuple(grad.shape) != (b, s, k):
        raise ValueError(f"grad must be fp32 [{b}, {s}, {k}], got {grad.dtype} {tuple(grad.shape)}")
    grad = grad.contiguous()
    with torch.cuda.device(logits.device):
        d = _grad_buffer(logits.shape, logits)
        with _timed("gather_logprob_bwd"):
            code = _lib.load().nrl_gather_logprob_bwd(C.byref(rows), _ptr(indices), k, _ptr(lse), _ptr(grad), _ptr(d),
                                                      d.stride(0), d.stride(1), _stream())
    _lib.check(code, "nrl_gather_logprob_bwd")
    return d


def _teacher_like(student, teacher):
    if teacher.shape != student.shape:
        raise ValueError(f"student_logits and target_logits must have the same shape, got {tuple(student.shape)} and {tuple(teacher.shape)}.")
    if teacher.dtype != student.dtype:
        teacher = teacher.to(student.dtype)
    if teacher.stride(2) != 1 and teacher.shape[2] > 1:
        teacher = teacher.contiguous()
    return teacher


def _soft_cross_entropy_fwd(student, teacher):
    _need_gpu(student, teacher)
    rows = _plain_rows(student)
    teacher = _teacher_like(student, teacher)
    b, s, _ = student.shape
    with torch.cuda.device(student.device):
        ce, lx, ly = (torch.empty((b, s), dtype=torch.float32, device=student.device) for _ in range(3))
        with _timed("soft_cross_entropy_fwd"):
            code = _lib.load().nrl_soft_cross_entropy_fwd(C.byref(rows), _ptr(teacher), teacher.stride(0), teacher.stride(1),
                                                          _ptr(ce), _ptr(lx), _ptr(ly), _stream())
    _lib.check(code, "nrl_soft_cross_entropy_fwd")
    return ce, lx, ly


def _soft_cross_entropy_bwd(student, teacher, lse_student, lse_teacher, grad):
    _need_gpu(student, teacher, lse_student, lse_teacher, grad)
    rows = _plain_rows(student)
    teacher = _teacher_like(student, teacher)
    b, s, _ = student.shape
    lx, ly, grad = _row_scalar(lse_student, b, s, "lse_student"), _row_scalar(lse_teacher, b, s, "lse_teacher"), _row_scalar(grad, b, s, "grad")
    with torch.cuda.device(student.device):
        d = _grad_buffer(student.shape, student)
        with _timed("soft_cross_entropy_bwd"):
            code = _lib.load().nrl_soft_cross_entropy_bwd(C.byref(rows), _ptr(teacher), teacher.stride(0), teacher.stride(1),
                                                          _ptr(lx), _ptr(ly), _ptr(grad), _ptr(d), d.stride(0), d.stride(1), _stream())
    _lib.check(code, "nrl_soft_cross_entropy_bwd")
    return d


for _name, _fn in (("neg_entropy_fwd", _neg_entropy_fwd), ("neg_entropy_bwd", _neg_entropy_bwd),
                   ("gather_logprob_fwd", _gather_logprob_fwd), ("gather_logprob_bwd", _gather_logprob_bwd),
                   ("soft_cross_entropy_fwd", _soft_cross_entropy_fwd), ("soft_cross_entropy_bwd", _soft_cross_entropy_bwd)):
    _LIB.impl(_name, _fn, "CUDA")
    _LIB.impl(_name, _fn, "CPU")


# ------------------------------------------------------------------------------------------------
# K6: fused lm_head
# ------------------------------------------------------------------------------------------------
_LIB.define(
    "lmhead_logprob_fwd(Tensor hidden, Tensor weight, Tensor targets, int vocab_start, int vocab_end, bool keep_logits=False) "
    "-> (Tensor, Tensor, Tensor)"
)
_LIB.define(
    "lmhead_logprob_bwd(Tensor hidden, Tensor weight, Tensor targets, Tensor lse, Tensor grad, int vocab_start, "
    "int vocab_end, Tensor? logits=None) -> (Tensor, Tensor)"
)


def _check_lmhead(hidden, weight, targets):
    _need_gpu(hidden, weight, targets)
    if hidden.dim() != 2 or weight.dim() != 2 or hidden.shape[1] != weight.shape[1]:
        raise ValueError(f"expected hidden [N,H] and weight [V,H], got {tuple(hidden.shape)}, {tuple(weight.shape)}")
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise ValueError("the fused lm_head path runs on bf16 hidden states and weights")
    if hidden.shape[1] % 8:
        raise ValueError("the hidden size must be a multiple of 8")
    if targets.dtype != torch.int64 or tuple(targets.shape) != (hidden.shape[0],) or not targets.is_contiguous():
        raise ValueError("targets must be a contiguous int64 [N] tensor")
    hidden = hidden if hidden.stride(1) == 1 and hidden.stride(0) % 8 == 0 and hidden.data_ptr() % 16 == 0 else hidden.contiguous()
    weight = weight if weight.stride(1) == 1 and weight.stride(0) % 8 == 0 and weight.data_ptr() % 16 == 0 else weight.contiguous()
    return hidden, weight


def _ws(nbytes, dev):
    return torch.empty(((nbytes + 255) // 256 * 32,), dtype=torch.float64, device=dev)  # 256-byte granules


def _lmhead_logprob_fwd(hidden, weight, targets, vocab_start, vocab_end, keep_logits=False):
    """-> (logprobs [N], log-sum-exps [N], the bf16 logits kept for the backward or an empty tensor).  The kept
    logits are a flat buffer in the layout the kernels exchange (``lmhead_unpack_kept_logits`` turns it into
    ``[N, V]``)."""
    hidden, weight = _check_lmhead(hidden, weight, targets)
    n, h = hidden.shape
    v = weight.shape[0]
    lib = _lib.load()
    dev = hidden.device
    with torch.cuda.device(dev):
        lp = torch.empty((n,), dtype=torch.float32, device=dev)
        lse = torch.empty((n,), dtype=torch.float32, device=dev)
        logits = torch.empty((lib.nrl_lmhead_kept_logits_bytes(n, v) // 2,), dtype=torch.bfloat16, device=dev) if keep_logits else None
        nbytes = lib.nrl_lmhead_fwd_workspace_bytes(n, v)
        ws = _ws(nbytes, dev)
        with _timed("lmhead_fwd"):
            code = lib.nrl_lmhead_logprob_fwd(
                _ptr(hidden), n, h, hidden.stride(0), _ptr(weight), v, weight.stride(0), _ptr(targets), vocab_start,
                vocab_end, _ptr(lp), _ptr(lse), _ptr(logits), 0 if logits is None else logits.numel() * 2, _ptr(ws),
                ws.numel() * 8, _stream(),
            )
    _lib.check(code, "nrl_lmhead_logprob_fwd")
    return lp, lse, (logits if keep_logits else lp.new_empty(0, dtype=torch.bfloat16))


def _lmhead_logprob_bwd(hidden, weight, targets, lse, grad, vocab_start, vocab_end, logits=None):
    hidden, weight = _check_lmhead(hidden, weight, targets)
    _need_gpu(lse, grad, logits)
    n, h = hidden.shape
    v = weight.shape[0]
    for t, name in ((lse, "lse"), (grad, "grad")):
        if t.dtype != torch.float32 or tuple(t.shape) != (n,) or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous fp32 [N] tensor")
    if logits is not None and logits.numel() == 0 and n * v > 0:
        logits = None
    lib = _lib.load()
    if logits is not None:
        if (logits.dtype != torch.bfloat16 or logits.dim() != 1 or not logits.is_contiguous() or logits.data_ptr() % 16
                or logits.numel() * 2 != lib.nrl_lmhead_kept_logits_bytes(n, v)):
            raise ValueError("kept logits must be the bf16 buffer the forward returned for these shapes")
    dev = hidden.device
    with torch.cuda.device(dev):
        dh = torch.empty((n, h), dtype=torch.float32, device=dev)
        dw = torch.empty((v, h), dtype=torch.bfloat16, device=dev)
        nbytes = lib.nrl_lmhead_bwd_workspace_bytes(n, h, v)
        ws = _ws(nbytes, dev)
        with _timed("lmhead_bwd"):
            code = lib.nrl_lmhead_logprob_bwd(
                _ptr(hidden), n, h, hidden.stride(0), _ptr(weight), v, weight.stride(0), _ptr(targets), vocab_start,
                vocab_end, _ptr(lse), _ptr(grad), _ptr(logits), 0 if logits is None else logits.numel() * 2, _ptr(dh), h,
                _ptr(dw), h, _ptr(ws), ws.numel() * 8, _stream(),
            )
    _lib.check(code, "nrl_lmhead_logprob_bwd")
    return dh, dw


def lmhead_unpack_kept_logits(kept: torch.Tensor, n_tokens: int, vocab: int) -> torch.Tensor:
    """The kept logits of ``lmhead_logprob_fwd`` as a bf16 ``[N, V]`` tensor (a copy, for inspection: the backward
    reads the buffer as it is).  The buffer holds blocks of 32 ids x 32 tokens, ``ceil(V / 32)`` per token block; a
    block is ``[p][h][token % 32][q][e]`` with id ``16 p + 8 q + 4 h + e``."""
    n_tb, n_vb = (n_tokens + 31) // 32, (vocab + 31) // 32
    blocks = kept.view(n_tb, n_vb, 2, 2, 32, 2, 4)  # tb, vb, p, h, token, q, e
    rows = blocks.permute(0, 4, 1, 2, 5, 3, 6).reshape(n_tb * 32, n_vb * 32)  # (tb, token) x (vb, p, q, h, e)
    return rows[:n_tokens, :vocab].contiguous()


for _name, _fn in (("lmhead_logprob_fwd", _lmhead_logprob_fwd), ("lmhead_logprob_bwd", _lmhead_logprob_bwd)):
    _LIB.impl(_name, _fn, "CUDA")
    _LIB.impl(_name, _fn, "CPU")
