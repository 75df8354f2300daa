"""Shared builders for the parity tests (golden cases -> tensors, synthetic
benchmark-style workloads)."""

from __future__ import annotations

import json
import os

import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_golden(name: str):
    with open(os.path.join(GOLDEN, name)) as fh:
        return json.load(fh)


def _t(rows, dtype=torch.float32):
    return torch.tensor([[float(v) for v in r] for r in rows], dtype=dtype)


def golden_case_to_inputs(case, device="cpu", mask_dtype=torch.int64):
    """Golden ClippedPG case -> (next_token_logprobs [B,S-1], data dict of [B,S]
    tensors, global_valid_seqs, global_valid_toks).  Position 0 is masked."""
    ref_key = next(k for k in ("adv", "curr", "curr_exp", "gen") if k in case)
    b, sm1 = len(case[ref_key]), len(case[ref_key][0])

    def full(key, exp_key=None):
        out = torch.zeros(b, sm1 + 1)
        if key in case:
            out[:, 1:] = _t(case[key])
        elif exp_key and exp_key in case:
            out[:, 1:] = torch.log(_t(case[exp_key]))
        return out.to(device)

    if "curr" in case:
        curr = _t(case["curr"])
    else:
        curr = torch.log(_t(case["curr_exp"]))
    token_mask = torch.ones(b, sm1 + 1, dtype=mask_dtype)
    token_mask[:, 0] = 0
    if "token_mask" in case:
        token_mask = torch.tensor(case["token_mask"], dtype=mask_dtype)
    sample_mask = torch.ones(b, dtype=mask_dtype)
    data = {
        "input_ids": torch.zeros(b, sm1 + 1, dtype=torch.int64).to(device),
        "token_mask": token_mask.to(device),
        "sample_mask": sample_mask.to(device),
        "advantages": full("adv"),
        "prev_logprobs": full("prev", "prev_exp"),
        "generation_logprobs": full("gen"),
        "reference_policy_logprobs": full("ref"),
    }
    gs = torch.sum(data["sample_mask"])
    gt = torch.sum(data["sample_mask"].unsqueeze(-1) * data["token_mask"])
    return curr.to(device), data, gs, gt


def exact_logits_for_logprobs(target_lp, input_ids, vocab):
    """Logits whose log-softmax at the next-token ids equals ``target_lp``
    ([B, S-1], values <= 0): the target logit is 0 and one other logit is
    ``log(exp(-lp) - 1)``, the rest are -100 (lp == 0 -> a single +100 spike)."""
    b, sm1 = target_lp.shape
    logits = torch.full((b, sm1 + 1, vocab), -100.0)
    for i in range(b):
        for j in range(sm1):
            tok = int(input_ids[i, j + 1])
            lp = float(target_lp[i, j])
            if abs(lp) < 1e-8:
                logits[i, j, tok] = 100.0
            else:
                logits[i, j, tok] = 0.0
                logits[i, j, (tok + 1) % vocab] = float(torch.log(torch.exp(torch.tensor(-lp)) - 1.0))
    return logits


def synthetic_grpo_batch(n_prompts, group, seq, vocab, seed, logits_dtype=torch.float32,
                         logit_std=2.0, min_resp=None, spike_p=0.0, spike=8.0):
    """benchmark-style synthetic step input on the CPU (fp32 generated, then cast)."""
    g = torch.Generator().manual_seed(seed)
    b = n_prompts * group
    logits = (torch.randn(b, seq, vocab, generator=g) * logit_std)
    ids = torch.randint(0, vocab, (b, seq), generator=g)
    if spike_p > 0:
        hit = torch.rand(b, seq, generator=g) < spike_p
        nxt = ids.roll(-1, dims=-1)
        logits.scatter_add_(-1, nxt.unsqueeze(-1), (hit.float() * spike).unsqueeze(-1))
    logits = logits.to(logits_dtype)
    lo = min_resp if min_resp is not None else max(1, seq // 8)
    resp = torch.randint(lo, seq + 1, (b,), generator=g)
    pos = torch.arange(seq).unsqueeze(0)
    token_mask = (pos >= (seq - resp).unsqueeze(-1)).to(torch.int64)
    token_mask[:, 0] = 0
    sample_mask = torch.ones(b, dtype=torch.float32)
    rewards = (torch.rand(b, generator=g) < 0.5).float()
    prompt_ids = torch.arange(n_prompts).repeat_interleave(group).unsqueeze(-1) * torch.ones(1, 4, dtype=torch.int64)
    return {
        "logits": logits, "input_ids": ids, "token_mask": token_mask, "sample_mask": sample_mask,
        "rewards": rewards, "prompt_ids": prompt_ids, "generator": g,
    }


def packed_grpo_case(lens, pads, width, vocab, dtype, seed, tail=0, empty_mask_rows=(), dead_rows=(), float_masks=False):
    """Unpacked ``[B, width]`` loss data plus the packed ``[1, T, V]`` logits of the same sequences (CPU):
    sequence i holds ``lens[i]`` tokens inside a span of ``lens[i] + pads[i]`` packed positions, ``tail``
    unused positions follow.  ``empty_mask_rows`` get an all-zero token mask, ``dead_rows`` a zero sample mask.
    Returns (logits, data, cu_seqlens, cu_seqlens_padded, global_valid_seqs, global_valid_toks)."""
    b = len(lens)
    g = torch.Generator().manual_seed(seed)
    lens_t, pads_t = torch.tensor(lens), torch.tensor(pads)
    cu = torch.cat([torch.zeros(1, dtype=torch.int64), lens_t.cumsum(0)]).to(torch.int32)
    cup = torch.cat([torch.zeros(1, dtype=torch.int64), (lens_t + pads_t).cumsum(0)]).to(torch.int32)
    total = int(cup[-1]) + tail
    logits = (torch.randn(1, total, vocab, generator=g) * 2.5).to(dtype)
    ids = torch.zeros(b, width, dtype=torch.int64)
    mdt = torch.float32 if float_masks else torch.int64
    tm = torch.zeros(b, width, dtype=mdt)
    for i, n in enumerate(lens):
        ids[i, :n] = torch.randint(0, vocab, (n,), generator=g)
        if n > 2 and i not in empty_mask_rows:
            tm[i, int(torch.randint(1, n - 1, (1,), generator=g)):n] = 1
    sm = torch.ones(b, dtype=mdt)
    for i in dead_rows:
        sm[i] = 0
    from oracle import logprob as OL

    targets = OL.pack_input_ids(ids, cu, cup, roll_shift=-1)
    cur = OL.packed_logits_to_logprobs(logits.float()[:, : int(cup[-1])], targets, cup, width, target_is_pre_rolled=True)
    near = lambda: torch.cat([torch.zeros(b, 1), cur + 0.05 * torch.randn(b, width - 1, generator=g)], 1)  # noqa: E731
    data = {"input_ids": ids, "token_mask": tm, "sample_mask": sm,
            "advantages": torch.randn(b, 1, generator=g).expand(b, width).contiguous(),
            "prev_logprobs": near(), "generation_logprobs": near(), "reference_policy_logprobs": near()}
    gs = sm.sum().float()
    gt = (tm[:, 1:] * sm.unsqueeze(-1)).sum().float()
    return logits, data, cu, cup, gs, gt


# A stand-in for a NeMo-RL install: a few lines per module, written for this test, that reproduce how the
# reference binds its hot-path names -- package re-exports (``algorithms/loss/__init__.py:15-41``), by-name
# imports in the driver (``algorithms/grpo.py:32-59``), the workers (``models/automodel/train.py:44-48``,
# ``models/megatron/train.py:39-50``, the latter needing Megatron-Core) and the loss module
# (``algorithms/loss/loss_functions.py:26``), and an enum comparison outside the replaced code
# (``models/automodel/data.py:422``).
_STUB_INSTALL = {
    "nemo_rl/__init__.py": "",
    "nemo_rl/distributed/__init__.py": "",
    "nemo_rl/distributed/model_utils.py": "\n".join(
        f"def {n}(*a, **k):\n    return 'reference'" for n in (
            "from_parallel_logits_to_logprobs", "from_parallel_logits_to_logprobs_packed_sequences",
            "from_parallel_hidden_states_to_logprobs", "get_next_token_logprobs_from_logits",
            "dtensor_from_parallel_logits_to_logprobs", "get_logprobs_from_vocab_parallel_logits",
            "get_distillation_topk_logprobs_from_logits", "_compute_distributed_log_softmax",
            "_compute_distributed_log_softmax_with_grad", "allgather_cp_sharded_tensor")
    ) + "\n" + "\n".join(
        f"class {n}:\n    origin = 'reference'" for n in (
            "DistributedLogprob", "ChunkedDistributedLogprob", "DistributedLogprobWithSampling",
            "ChunkedDistributedLogprobWithSampling", "ChunkedDistributedHiddenStatesToLogprobs",
            "ChunkedDistributedEntropy", "ChunkedDistributedGatherLogprob", "DistributedCrossEntropy")
    ) + "\n",
    "nemo_rl/algorithms/__init__.py": "",
    "nemo_rl/algorithms/utils.py": "\n".join(
        f"def {n}(*a, **k):\n    return 'reference'" for n in (
            "calculate_kl", "masked_mean", "calculate_baseline_and_std_per_prompt", "mask_out_neg_inf_logprobs",
            "set_seed")) + "\n",
    "nemo_rl/algorithms/logits_sampling_utils.py": (
        "class TrainingSamplingParams:\n    pass\n"
        "def need_top_k_or_top_p_filtering(p):\n    return False\n"
        "def apply_top_k_top_p(*a, **k):\n    return 'reference'\n"),
    "nemo_rl/algorithms/advantage_estimator.py": (
        "from nemo_rl.algorithms.utils import calculate_baseline_and_std_per_prompt\n"
        "class GRPOAdvantageEstimator:\n    origin = 'reference'\n"
        "class ReinforcePlusPlusAdvantageEstimator:\n    origin = 'reference'\n"),
    "nemo_rl/algorithms/loss/__init__.py": (
        "from nemo_rl.algorithms.loss.loss_functions import (\n"
        "    ClippedPGLossConfig, ClippedPGLossFn, DistillationLossFn, DPOLossFn, DraftCrossEntropyLossFn,\n"
        "    MseValueLossFn, NLLLossFn, PreferenceLossFn)\n"
        "from nemo_rl.algorithms.loss.utils import prepare_loss_input, prepare_packed_loss_input\n"
        "from nemo_rl.algorithms.loss.wrapper import (\n"
        "    SequencePackingFusionLossWrapper, SequencePackingLossWrapper, wrap_loss_fn_with_input_preparation)\n"),
    "nemo_rl/algorithms/loss/interfaces.py": (
        "import enum\n"
        "class LossType(enum.Enum):\n    TOKEN_LEVEL = 'token_level'\n    SEQUENCE_LEVEL = 'sequence_level'\n"
        "class MetricNormalizer(enum.Enum):\n    TOKENS = 'tokens'\n    SEQUENCES = 'sequences'\n    NONE = 'none'\n"
        "class LossInputType(enum.Enum):\n    LOGIT = 'logit'\n    LOGPROB = 'logprob'\n"
        "    DISTILLATION = 'distillation'\n    DISTILLATION_CROSS_TOKENIZER = 'distillation_cross_tokenizer'\n"
        "    DRAFT = 'draft'\n"
        "class LossFunction:\n    pass\n"),
    "nemo_rl/algorithms/loss/loss_functions.py": (
        "from nemo_rl.algorithms.loss.interfaces import LossFunction, LossInputType, LossType\n"
        "from nemo_rl.algorithms.utils import calculate_kl, masked_mean\n"
        "ClippedPGLossConfig = dict\n"
        + "".join(f"class {n}(LossFunction):\n    origin = 'reference'\n    input_type = LossInputType.LOGPROB\n"
                  f"    def __init__(self, *a, **k):\n        self.loss_type = LossType.TOKEN_LEVEL\n"
                  for n in ("ClippedPGLossFn", "NLLLossFn", "PreferenceLossFn", "DPOLossFn", "DistillationLossFn",
                            "DraftCrossEntropyLossFn"))
        + "class MseValueLossFn(LossFunction):\n    def __call__(self, *a):\n        return masked_mean(*a)\n"),
    "nemo_rl/algorithms/loss/utils.py": (
        "from nemo_rl.distributed.model_utils import (\n"
        "    from_parallel_logits_to_logprobs_packed_sequences, get_next_token_logprobs_from_logits)\n"
        "def prepare_loss_input(*a, **k):\n    return 'reference'\n"
        "def prepare_packed_loss_input(*a, **k):\n    return 'reference'\n"),
    "nemo_rl/algorithms/loss/wrapper.py": (
        "def wrap_loss_fn_with_input_preparation(*a, **k):\n    return 'reference'\n"
        "class SequencePackingLossWrapper:\n    origin = 'reference'\n"
        "class SequencePackingFusionLossWrapper:\n    origin = 'reference'\n"),
    "nemo_rl/algorithms/grpo.py": (
        "from nemo_rl.algorithms.advantage_estimator import GRPOAdvantageEstimator, ReinforcePlusPlusAdvantageEstimator\n"
        "from nemo_rl.algorithms.loss import ClippedPGLossConfig, ClippedPGLossFn\n"
        "from nemo_rl.algorithms.loss.interfaces import LossFunction\n"
        "from nemo_rl.algorithms.utils import calculate_baseline_and_std_per_prompt, set_seed\n"
        "def dynamic_sampling(*a, **k):\n    return 'reference'\n"
        "def compute_and_apply_seq_logprob_error_masking(*a, **k):\n    return 'reference'\n"
        "def setup(cfg):\n    return ClippedPGLossFn(cfg)\n"),
    "nemo_rl/models/__init__.py": "",
    "nemo_rl/models/automodel/__init__.py": "",
    "nemo_rl/models/automodel/data.py": (
        "from nemo_rl.algorithms.loss.interfaces import LossType\n"
        "def normalises_by_tokens(loss_fn):\n"
        "    return hasattr(loss_fn, 'loss_type') and loss_fn.loss_type == LossType.TOKEN_LEVEL\n"),
    "nemo_rl/models/automodel/train.py": (
        "from nemo_rl.algorithms.logits_sampling_utils import TrainingSamplingParams, apply_top_k_top_p\n"
        "from nemo_rl.algorithms.loss import SequencePackingLossWrapper, prepare_loss_input\n"
        "from nemo_rl.algorithms.utils import mask_out_neg_inf_logprobs\n"
        "from nemo_rl.distributed.model_utils import allgather_cp_sharded_tensor, get_logprobs_from_vocab_parallel_logits\n"
        "def apply_temperature_scaling(*a, **k):\n    return 'reference'\n"
        "class LossPostProcessor:\n    origin = 'reference'\n"
        "class LogprobsPostProcessor:\n    origin = 'reference'\n"
        "class TopkLogitsPostProcessor:\n    def __call__(self, logits, **k):\n        return logits.topk(2).values, logits.topk(2).indices\n"
        "class FullLogitsPostProcessor:\n    def __call__(self, logits, **k):\n        return logits\n"
        "class ScorePostProcessor:\n    def __call__(self, logits):\n        return logits.sum(-1)\n"
        "def _needs_kv_cache_for_shared_layers(model):\n    return False\n"
        "def model_forward(model, processed_inputs, is_reward_model=False, allow_flash_attn_args=True, use_cache=False):\n"
        "    return model(processed_inputs)\n"
        "def extract_logits(model, outputs):\n    return outputs['logits']\n"
        "def forward_with_post_processing_fn(*a, **k):\n    return 'reference'\n"
        "def automodel_forward_backward(model, mb, fn, **k):\n    return forward_with_post_processing_fn(model, fn, mb, **k)\n"
        "def is_loss_step(fn):\n    return isinstance(fn, LossPostProcessor)\n"),
    "nemo_rl/models/megatron/__init__.py": "",
    "nemo_rl/models/megatron/train.py": (
        "from megatron.core.models.gpt import GPTModel\n"
        "from nemo_rl.algorithms.loss import wrap_loss_fn_with_input_preparation\n"
        "def apply_temperature_scaling(*a, **k):\n    return 'reference'\n"
        "class LossPostProcessor:\n    origin = 'reference'\n"
        "class LogprobsPostProcessor:\n    origin = 'reference'\n"
        "class TopkLogitsPostProcessor:\n    def __call__(self, data_dict):\n        return lambda output: ('topk', output)\n"
        "def forward_with_post_processing_fn(data_iterator, model, post_processing_fn, sampling_params=None, **k):\n"
        "    mb = next(data_iterator)\n"
        "    output = model(mb)\n"
        "    apply_temperature_scaling(output, sampling_params)\n"
        "    return output, post_processing_fn(data_dict=mb)\n"
        "def megatron_forward_backward(model, data_iterator, fn, **k):\n"
        "    return forward_with_post_processing_fn(data_iterator, model, fn, **k)\n"),
    "driver_script.py": (
        "from nemo_rl.algorithms.loss import ClippedPGLossFn\n"
        "from nemo_rl.algorithms.utils import masked_mean\n"),
}


# a stand-in for Megatron-Core, just enough for the stand-in Megatron worker module to import
_STUB_MEGATRON = {
    "megatron/__init__.py": "",
    "megatron/core/__init__.py": "",
    "megatron/core/models/__init__.py": "",
    "megatron/core/models/gpt.py": "class GPTModel:\n    pass\n",
}


def write_stub_install(tmp_path, with_megatron: bool = False) -> str:
    """Writes the stand-in install under ``tmp_path`` and returns the ``PYTHONPATH`` a child process needs to
    import it next to this repository.  ``with_megatron`` adds a stand-in ``megatron.core``, so that the Megatron
    worker module of the stand-in imports."""
    files = dict(_STUB_INSTALL, **(_STUB_MEGATRON if with_megatron else {}))
    for rel, text in files.items():
        path = tmp_path / rel
        path.parent.mkdir(parents=True, exist_ok=True)
        path.write_text(text)
    here = os.path.dirname(os.path.abspath(__file__))
    return os.pathsep.join([str(tmp_path), os.path.dirname(here), here])
