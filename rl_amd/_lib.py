"""ctypes binding of ``librl_amd_hip.so`` (declared in ``include/nrl_hip.h``).

The library is the only compute path of this package: if it is missing the loader raises, it
never falls back to another implementation.
"""

from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "librl_amd_hip.so")

NRL_F32, NRL_BF16, NRL_F16 = 0, 1, 2
NRL_TEMP_DIV, NRL_TEMP_RCP = 0, 1
NRL_TIS = {None: 0, "tis": 1, "icepop": 2, "seq-mask-tis": 3}
NRL_GRPO_N_METRICS = 24
NRL_GRPO_STATIC_MAX_BATCH = 8192

METRIC_SLOTS = {
    "loss": 0, "probs_ratio": 1, "probs_ratio_clamped": 2, "probs_ratio_min": 3, "probs_ratio_max": 4,
    "probs_ratio_clamped_min": 5, "probs_ratio_clamped_max": 6, "kl": 7, "token_mult_prob_error": 8,
    "gen_kl_error": 9, "policy_kl_error": 10, "js_divergence_error": 11, "sampling_importance_ratio": 12,
    "num_valid_samples": 13, "approx_entropy": 14, "is_oob_ratio": 15, "positive_nll_loss": 16,
    "actor_loss": 17, "n_masked_tokens": 18,
}


class NrlRows(C.Structure):
    _fields_ = [
        ("logits", C.c_void_p), ("dtype", C.c_int32),
        ("n_outer", C.c_int64), ("n_inner", C.c_int64), ("vocab", C.c_int64),
        ("stride_outer", C.c_int64), ("stride_inner", C.c_int64),
        ("targets", C.c_void_p), ("tgt_stride_outer", C.c_int64), ("tgt_stride_inner", C.c_int64),
        ("vocab_start", C.c_int64), ("vocab_end", C.c_int64),
        ("temperature", C.c_float), ("temp_mode", C.c_int32),
    ]


class NrlGrpoCfg(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "token_level_loss", "disable_ppo_ratio", "force_on_policy_ratio", "use_cispo",
        "sequence_level_importance_ratios", "use_importance_sampling_correction",
        "use_on_policy_kl_approximation", "tis_type", "kl_type", "has_kl", "has_kl_input_clamp",
        "has_kl_output_clamp", "has_dual_clip", "has_nll")] + [(n, C.c_float) for n in (
        "ratio_clip_min", "ratio_clip_max", "ratio_clip_c", "kl_beta", "kl_input_clamp",
        "kl_output_clamp", "tis_max", "tis_min", "nll_weight")]


class NrlGrpoInputs(C.Structure):
    _fields_ = [
        ("batch", C.c_int64), ("sm1", C.c_int64),
        ("lp", C.c_void_p), ("lp_stride", C.c_int64),
        ("lpu", C.c_void_p), ("lpu_stride", C.c_int64),
        ("prev", C.c_void_p), ("prev_stride", C.c_int64),
        ("gen", C.c_void_p), ("gen_stride", C.c_int64),
        ("ref", C.c_void_p), ("ref_stride", C.c_int64),
        ("adv", C.c_void_p), ("adv_stride", C.c_int64),
        ("token_mask", C.c_void_p), ("token_mask_stride", C.c_int64),
        ("sample_mask", C.c_void_p), ("correct_mask", C.c_void_p), ("global_valid", C.c_void_p),
    ]


_I64, _I32, _F, _P = C.c_int64, C.c_int32, C.c_float, C.c_void_p

# name -> (restype, argtypes); mirrors include/nrl_hip.h one to one
SIGNATURES = {
    "nrl_version": (C.c_int, []),
    "nrl_last_error": (C.c_char_p, []),
    "nrl_logprob_fwd": (C.c_int, [C.POINTER(NrlRows), _P, _P, _P]),
    "nrl_logprob_post_fwd": (C.c_int, [C.POINTER(NrlRows), _P, _P, _P]),
    "nrl_logprob_bwd": (C.c_int, [C.POINTER(NrlRows), _P, _P, _I64, _I64, _P, _I64, _I64, _I64, _P]),
    "nrl_scale_rows": (C.c_int, [_P, _P, _I32, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P, _F, _P]),
    "nrl_pack_input_ids": (C.c_int, [_P, _I64, _I64, _I64, _P, _P, _I64, _P, _I64, _P]),
    "nrl_logprob_packed_fwd": (C.c_int, [_P, _I32, _I64, _I64, _I64, _P, _I32, _P, _I64, _I64, _I64, _I64, _F, _I32, _P, _P, _P]),
    "nrl_logprob_packed_bwd": (C.c_int, [_P, _I32, _I64, _I64, _I64, _P, _I32, _P, _I64, _I64, _I64, _I64, _F, _I32, _P, _P, _P, _I64, _P]),
    "nrl_log_softmax_fwd": (C.c_int, [_P, C.c_int32, _I64, _I64, _I64, _P, _I64, _P]),
    "nrl_log_softmax_bwd": (C.c_int, [_P, C.c_int32, _I64, _I64, _I64, _P, _I64, _P, _I64, _P]),
    "nrl_topk_topp_logprob_fwd": (C.c_int, [C.POINTER(NrlRows), _I64, _F, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I64, _P]),
    "nrl_topk_topp_logprob_bwd": (C.c_int, [C.POINTER(NrlRows), _P, _P, _P, _P, _I64, _I64, _P, _P, _P, _I64, _P, _I64, _I64, _I64, _P]),
    "nrl_topk_topp_filter": (C.c_int, [C.POINTER(NrlRows), _P, _P, _P, _I64, _I64, _P, _P]),
    "nrl_grpo_loss_workspace_bytes": (_I64, [_I64]),
    "nrl_grpo_loss_fwd_bwd": (C.c_int, [C.POINTER(NrlGrpoCfg), C.POINTER(NrlGrpoInputs), _P, _P, _P, _P, _P, _I64, _P]),
    "nrl_grpo_loss_fwd_bwd_static": (C.c_int, [C.POINTER(NrlGrpoCfg), C.POINTER(NrlGrpoInputs), _P, _P, _P, _P, _P]),
    "nrl_fused_workspace_bytes": (_I64, [_I64, _I64]),
    "nrl_fused_packed_workspace_bytes": (_I64, [_I64, _I64, _I64]),
    "nrl_fused_logits_grpo_loss": (C.c_int, [C.POINTER(NrlRows), C.POINTER(NrlGrpoCfg), C.POINTER(NrlGrpoInputs), _F, _P, _I64,
                                             _I64, _I64, _P, _P, _P, _P, _I64, _P]),
    "nrl_fused_packed_logits_grpo_loss": (C.c_int, [C.POINTER(NrlRows), C.c_int32, _P, _I64, C.POINTER(NrlGrpoCfg),
                                                    C.POINTER(NrlGrpoInputs), _F, _P, _I64, _P, _P, _P, _P, _I64, _P]),
    "nrl_nll_loss_fwd_bwd": (C.c_int, [C.POINTER(NrlGrpoInputs), _P, _P, _P, _P, _I64, _P]),
    "nrl_calculate_kl": (C.c_int, [_P, _P, _P, _I64, _I32, _I32, _F, _I32, _F, _P, _P]),
    "nrl_calculate_kl_bwd": (C.c_int, [_P, _P, _P, _P, _I64, _I32, _I32, _F, _I32, _F, _P, _P, _P, _P]),
    "nrl_masked_mean": (C.c_int, [_P, _P, _I64, _I64, _P, _F, _I32, _P, _P, _P]),
    "nrl_masked_mean_bwd": (C.c_int, [_P, _P, _P, _I64, _I64, _P, _P]),
    "nrl_topk_logsoftmax_fwd": (C.c_int, [C.POINTER(NrlRows), _P, _I64, _P, _P]),
    "nrl_topk_logsoftmax_bwd": (C.c_int, [C.POINTER(NrlRows), _P, _I64, _P, _P, _P, _I64, _I64, _P]),
    "nrl_distill_topk_loss_workspace_bytes": (_I64, [_I64, _I64]),
    "nrl_distill_topk_loss_fwd_bwd": (C.c_int, [_P, _P, _P, _P, _I64, _P, _P, _I64, _I64, _I64, C.c_int32, _F, C.c_int32, _F,
                                                _P, _P, _P, _P, _I64, _P]),
    "nrl_nll_rows_fwd": (C.c_int, [_P, _I64, _P, _I64, _P, _I64, _I64, C.c_int32, _P, _P, _P, _P, _I64, _P]),
    "nrl_nll_rows_bwd": (C.c_int, [_P, _P, _I64, _P, _P, _I64, _I64, _P, _P]),
    "nrl_dpo_workspace_bytes": (_I64, [_I64]),
    "nrl_dpo_loss_fwd_bwd": (C.c_int, [_P, _I64, _P, _I64, _P, _I64, _P, _P, _I64, _I64, _F, _F, _F, C.c_int32, C.c_int32,
                                       _P, _P, _P, _P, _I64, _P]),
    "nrl_preference_loss_fwd_bwd": (C.c_int, [_P, _P, _P, _I64, _P, _P, _P, _P]),
    "nrl_neg_entropy_fwd": (C.c_int, [C.POINTER(NrlRows), _P, _P, _P]),
    "nrl_neg_entropy_bwd": (C.c_int, [C.POINTER(NrlRows), _P, _P, _P, _P, _I64, _I64, _P]),
    "nrl_gather_logprob_fwd": (C.c_int, [C.POINTER(NrlRows), _P, _I64, _P, _P, _P]),
    "nrl_gather_logprob_bwd": (C.c_int, [C.POINTER(NrlRows), _P, _I64, _P, _P, _P, _I64, _I64, _P]),
    "nrl_soft_cross_entropy_fwd": (C.c_int, [C.POINTER(NrlRows), _P, _I64, _I64, _P, _P, _P, _P]),
    "nrl_soft_cross_entropy_bwd": (C.c_int, [C.POINTER(NrlRows), _P, _I64, _I64, _P, _P, _P, _P, _I64, _I64, _P]),
    "nrl_nonzero_indices": (C.c_int, [_P, _I64, _P, _P, _P]),
    "nrl_seq_logprob_error": (C.c_int, [_P, _I64, _P, _I64, _P, _I64, _P, _P, _I64, _I64, C.c_int32, C.c_float, _P, _P, _P, _P, _I64, _P]),
    "nrl_lmhead_fwd_workspace_bytes": (_I64, [_I64, _I64]),
    "nrl_lmhead_kept_logits_bytes": (_I64, [_I64, _I64]),
    "nrl_lmhead_logprob_fwd": (C.c_int, [_P, _I64, _I64, _I64, _P, _I64, _I64, _P, _I64, _I64, _P, _P, _P, _I64, _P, _I64, _P]),
    "nrl_lmhead_bwd_workspace_bytes": (_I64, [_I64, _I64, _I64]),
    "nrl_lmhead_logprob_bwd": (C.c_int, [_P, _I64, _I64, _I64, _P, _I64, _I64, _P, _I64, _I64, _P, _P, _P, _I64, _P, _I64, _P, _I64, _P, _I64, _P]),
    "nrl_group_workspace_bytes": (_I64, [_I64]),
    "nrl_group_baseline_std": (C.c_int, [_P, _I64, _I64, _I64, _P, _P, _P, _I32, _I32, _P, _P, _P, _P, _P, _I64, _P]),
}

_lib = None


ABI_VERSION = 111  # nrl_version() of the library these signatures describe


def load() -> C.CDLL:
    """Load the HIP library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m rl_amd.build` (hipcc, gfx950). "
            "rl_amd has no other compute path."
        )
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    built = lib.nrl_version()
    if built != ABI_VERSION:  # a library of another signature set would be called with the wrong arguments
        raise RuntimeError(
            f"{LIB_PATH} has ABI version {built}, these bindings are for {ABI_VERSION}: rebuild it with `python -m rl_amd.build`"
        )
    _lib = lib
    return lib


class NrlError(RuntimeError):
    pass


def check(code: int, what: str) -> None:
    """Map a negative return code to a Python exception (ValueError for bad arguments)."""
    if code == 0:
        return
    msg = load().nrl_last_error().decode(errors="replace")
    text = f"{what} failed ({code}): {msg}"
    if code in (-1, -4):
        raise ValueError(text)
    raise NrlError(text)
