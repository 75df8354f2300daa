"""CPU-only tests of the host-side mirror of the reference interface."""

import pytest
import torch

import rl_amd
from helpers import load_golden, write_stub_install
from oracle import logprob as OL
from rl_amd.algorithms.loss import (
    ClippedPGLossConfig,
    ClippedPGLossFn,
    LossInputType,
    LossType,
    MetricNormalizer,
    NLLLossFn,
)
from rl_amd.algorithms.loss.utils import _pack_input_ids
from rl_amd.algorithms.logits_sampling_utils import TrainingSamplingParams, need_top_k_or_top_p_filtering

PG = load_golden("clipped_pg_cases.json")


@pytest.mark.parametrize("bad", PG["config_asserts"]["must_raise_assertion"])
def test_constructor_asserts(bad):
    with pytest.raises(AssertionError):
        ClippedPGLossFn(ClippedPGLossConfig(**bad))


def test_tis_min_above_max_message():
    cfg = ClippedPGLossConfig(
        use_importance_sampling_correction=True, truncated_importance_sampling_type="tis",
        truncated_importance_sampling_ratio=1.0, truncated_importance_sampling_ratio_min=2.0,
    )
    with pytest.raises(AssertionError, match="truncated_importance_sampling_ratio_min must be <= truncated_importance_sampling_ratio"):
        ClippedPGLossFn(cfg)


def test_metric_normalizations_table():
    # tests/unit/algorithms/test_loss_functions.py:2688-2765 of the reference
    n = ClippedPGLossFn(ClippedPGLossConfig()).metric_normalizations
    assert n["loss"] is MetricNormalizer.TOKENS and n["kl_penalty"] is MetricNormalizer.TOKENS
    assert n["sampling_importance_ratio"] is MetricNormalizer.TOKENS
    for k in ("probs_ratio", "probs_ratio_clamped", "token_mult_prob_error", "gen_kl_error", "policy_kl_error",
              "js_divergence_error", "approx_entropy"):
        assert n[k] is MetricNormalizer.TOKENS
    for k in ("num_valid_samples", "positive_nll_loss", "probs_ratio_min", "probs_ratio_max"):
        assert n[k] is MetricNormalizer.NONE
    assert "is_oob_ratio" not in n
    n = ClippedPGLossFn(ClippedPGLossConfig(token_level_loss=False, sequence_level_importance_ratios=True,
                                            use_importance_sampling_correction=True)).metric_normalizations
    assert n["loss"] is MetricNormalizer.SEQUENCES and n["sampling_importance_ratio"] is MetricNormalizer.SEQUENCES
    assert n["token_mult_prob_error"] is MetricNormalizer.TOKENS
    n = ClippedPGLossFn(ClippedPGLossConfig(
        token_level_loss=True, use_importance_sampling_correction=True,
        truncated_importance_sampling_type="seq-mask-tis", truncated_importance_sampling_ratio=2.0,
        truncated_importance_sampling_ratio_min=0.5)).metric_normalizations
    assert n["loss"] is MetricNormalizer.TOKENS and n["is_oob_ratio"] is MetricNormalizer.SEQUENCES
    n = ClippedPGLossFn(ClippedPGLossConfig(
        token_level_loss=False, use_importance_sampling_correction=True,
        truncated_importance_sampling_type="tis", truncated_importance_sampling_ratio=2.0)).metric_normalizations
    assert n["loss"] is MetricNormalizer.SEQUENCES and n["is_oob_ratio"] is MetricNormalizer.TOKENS
    n = NLLLossFn().metric_normalizations
    assert n["loss"] is MetricNormalizer.TOKENS and n["num_unmasked_tokens"] is MetricNormalizer.NONE


def test_loss_attributes_and_pickle():
    import pickle

    fn = ClippedPGLossFn(ClippedPGLossConfig(use_kl_in_reward=True), use_fused_linear_logprobs=True)
    assert fn.input_type is LossInputType.LOGPROB and fn.loss_type is LossType.TOKEN_LEVEL
    assert fn.reference_policy_kl_penalty == 0 and fn.use_fused_linear_logprobs
    clone = pickle.loads(pickle.dumps(fn))  # the driver ships the loss object to every worker
    assert clone.ratio_clip_min == fn.ratio_clip_min and clone.metric_normalizations == fn.metric_normalizations


def test_sampling_predicates():
    assert not need_top_k_or_top_p_filtering(None)
    assert not need_top_k_or_top_p_filtering(TrainingSamplingParams())
    assert not need_top_k_or_top_p_filtering(TrainingSamplingParams(top_k=-1, top_p=1.0))
    assert need_top_k_or_top_p_filtering(TrainingSamplingParams(top_k=5))
    assert need_top_k_or_top_p_filtering(TrainingSamplingParams(top_p=0.9))


@pytest.mark.parametrize("roll", [0, -1])
def test_pack_input_ids_matches_oracle(roll):
    torch.manual_seed(0)
    ids = torch.randint(1, 50, (4, 12))
    cu = torch.tensor([0, 5, 17, 17, 26])       # lengths 5, 12, 0, 9
    cup = torch.tensor([0, 8, 24, 24, 36])      # padded to multiples of 4 (with an empty sequence)
    got = _pack_input_ids(ids, cu, cup, roll_shift=roll)
    assert torch.equal(got, OL.pack_input_ids(ids, cu, cup, roll_shift=roll))
    # a sequence whose recorded length exceeds the row width copies only the real tokens
    cu2, cup2 = torch.tensor([0, 5, 20]), torch.tensor([0, 8, 24])
    assert torch.equal(_pack_input_ids(ids[:2], cu2, cup2, roll_shift=roll),
                       OL.pack_input_ids(ids[:2], cu2, cup2, roll_shift=roll))


def test_install_aliases_reference_paths():
    assert rl_amd.install() in ("aliased", "patched")
    import nemo_rl.algorithms.loss_functions as short
    from nemo_rl.algorithms.loss import ClippedPGLossFn as A
    from nemo_rl.algorithms.loss.loss_functions import ClippedPGLossFn as B
    from nemo_rl.distributed.model_utils import from_parallel_logits_to_logprobs  # noqa: F401
    from nemo_rl.algorithms.utils import calculate_baseline_and_std_per_prompt  # noqa: F401
    from nemo_rl.algorithms.advantage_estimator import GRPOAdvantageEstimator  # noqa: F401

    assert A is B is short.ClippedPGLossFn is ClippedPGLossFn


def test_multi_rank_groups_are_rejected(monkeypatch):
    from rl_amd.distributed import model_utils as mu

    monkeypatch.setattr(mu, "_group_size", lambda g: 2 if g == "tp2" else 1)
    with pytest.raises(NotImplementedError, match="one GPU"):
        mu.from_parallel_logits_to_logprobs(torch.zeros(1, 2, 4), torch.zeros(1, 2, dtype=torch.long), 0, 4, "tp2")


def _step_metrics(record, arrived):
    from rl_amd.algorithms.loss.loss_functions import StepMetrics

    calls = []

    def fetch():
        calls.append(1)
        return dict(record)

    fetch.ready = lambda: arrived[0]
    return StepMetrics(list(record), fetch), calls


def test_step_metrics_wait_only_when_values_are_needed():
    import json
    import pickle

    from rl_amd.algorithms.loss.loss_functions import PendingMetric

    record = {"loss": 0.5, "probs_ratio_max": 3.0, "num_valid_samples": 4}
    # as returned by the loss: nothing is fetched until a value is needed, and every value that leaves is a number
    m, calls = _step_metrics(record, [False])
    assert isinstance(m, dict) and calls == [] and len(m) == 3 and "loss" in m and list(m.keys()) == list(record)
    m["lr"] = 1e-5
    assert calls == []
    assert type(m["loss"]) is float and calls == [1]
    m, calls = _step_metrics(record, [False])
    assert dict(m) == record and all(type(v) in (float, int) for v in dict(m).values()) and calls == [1]
    m, calls = _step_metrics(record, [False])
    assert {**m} == record and calls == [1]

    # announced by the DTensor worker's post-processor: what that worker does between the loss call and backward()
    # fetches nothing
    arrived = [False]
    m, calls = _step_metrics(record, arrived)
    assert m.defer_scaling() is m
    for k in m.keys():
        if "_min" in k or "_max" in k:
            continue
        m[k] /= 4
    m["lr"] = 1e-5
    assert calls == [] and len(m) == 4
    assert isinstance(m["loss"], PendingMetric) and calls == []
    # the first real use fetches once; afterwards the mapping holds plain numbers
    assert m["num_valid_samples"] > 0 and calls == [1]
    assert dict.__getitem__(m, "loss") == 0.125 and type(dict.__getitem__(m, "loss")) is float
    assert m == {"loss": 0.125, "probs_ratio_max": 3.0, "num_valid_samples": 1.0, "lr": 1e-5} and calls == [1]
    assert json.loads(json.dumps(m))["loss"] == 0.125
    # ... and a record that has arrived by the first touch gives numbers at once
    m, calls = _step_metrics(record, [True])
    m.defer_scaling()
    assert type(m["loss"]) is float and calls == [1]

    # every way of handing the values out wholesale waits, once, announced or not
    for announce in (False, True):
        for use in (lambda x: list(x.items()), lambda x: list(x.values()), lambda x: x.get("loss"), lambda x: repr(x),
                    lambda x: x == record, lambda x: x.copy(), lambda x: x.pop("loss"), lambda x: x.setdefault("b", 2),
                    lambda x: json.dumps(x), lambda x: pickle.dumps(x), lambda x: x | {"a": 1},
                    lambda x: float(x["loss"]), lambda x: x["loss"] + 1, lambda x: f"{x['loss']:.3f}", lambda x: x["loss"] < 1):
            m, calls = _step_metrics(record, [False])
            if announce:
                m.defer_scaling()
            use(m)
            assert calls == [1], use
    m, calls = _step_metrics(record, [False])
    restored = pickle.loads(pickle.dumps(m))
    assert type(restored) is dict and restored == record
    # values that escaped before the record arrived still resolve by themselves, scaled as recorded
    m, calls = _step_metrics(record, [False])
    m.defer_scaling()
    early = {k: m[k] for k in m.keys()}
    scaled = early["loss"] / 2 * 3
    assert calls == [] and scaled == 0.75 and calls == [1] and pickle.loads(pickle.dumps(early["loss"])) == 0.5
    assert early["num_valid_samples"] / torch.tensor(2.0) == torch.tensor(2.0)   # a non-number operand resolves at once


_STUB_CHECK = r"""
import json, sys
import torch
import driver_script
import nemo_rl.algorithms.grpo as grpo
import nemo_rl.algorithms.loss as pkg
import nemo_rl.algorithms.loss.loss_functions as lf
import nemo_rl.algorithms.loss.interfaces as itf
import nemo_rl.models.automodel.train as train
import nemo_rl.models.automodel.data as data
import nemo_rl.algorithms.advantage_estimator as ae
import rl_amd
from rl_amd import compat

mode = rl_amd.install()
again = rl_amd.install()


def _forward_dispatch(train):
    # post-processors this package leaves alone keep working through the replaced forward function (no temperature
    # here: the in-place divide needs a GPU)
    import types

    mb = types.SimpleNamespace(data_dict={}, processed_inputs="inputs", original_batch_size=1, original_seq_len=3)
    x = torch.arange(12.0).view(1, 3, 4)
    model = lambda inputs: {"logits": x}
    score, m1, back = train.automodel_forward_backward(model, mb, train.ScorePostProcessor())
    (vals, idx), m2, _ = train.forward_with_post_processing_fn(model, train.TopkLogitsPostProcessor(), mb, sampling_params=None)
    full, m3, _ = train.forward_with_post_processing_fn(model, train.FullLogitsPostProcessor(), mb)
    try:
        train.forward_with_post_processing_fn(model, object(), mb)
        unknown = False
    except TypeError:
        unknown = True
    return (back is mb and torch.equal(score, x.sum(-1)) and torch.equal(m1["scores"], score) and torch.equal(vals, x.topk(2).values)
            and set(m2) == {"topk_logits", "topk_indices"} and full is x and m3["full_logits"] is x and unknown)

import rl_amd.algorithms.loss as mine
import rl_amd.algorithms.utils as mu
import rl_amd.algorithms.advantage_estimator as mae
import rl_amd.models.automodel.train as mtrain
import nemo_rl.algorithms.loss_functions as short

fn = grpo.setup({"token_level_loss": True})
seq = pkg.ClippedPGLossFn({"token_level_loss": False})
out = {
    "mode": [mode, again],
    "skipped": compat.skipped_modules(),
    "pkg.ClippedPGLossFn": pkg.ClippedPGLossFn is mine.ClippedPGLossFn,
    "lf.ClippedPGLossFn": lf.ClippedPGLossFn is mine.ClippedPGLossFn,
    "grpo.ClippedPGLossFn": grpo.ClippedPGLossFn is mine.ClippedPGLossFn,
    "short.ClippedPGLossFn": short.ClippedPGLossFn is mine.ClippedPGLossFn,
    "script.ClippedPGLossFn": driver_script.ClippedPGLossFn is mine.ClippedPGLossFn,
    "script.masked_mean": driver_script.masked_mean is mu.masked_mean,
    "grpo.GRPOAdvantageEstimator": grpo.GRPOAdvantageEstimator is mae.GRPOAdvantageEstimator,
    "grpo.baseline": grpo.calculate_baseline_and_std_per_prompt is mu.calculate_baseline_and_std_per_prompt,
    "ae.baseline": ae.calculate_baseline_and_std_per_prompt is mu.calculate_baseline_and_std_per_prompt,
    "grpo.untouched": grpo.ReinforcePlusPlusAdvantageEstimator.origin == "reference" and grpo.set_seed() == "reference",
    "grpo.dynamic_sampling": grpo.dynamic_sampling.__module__.startswith("rl_amd."),
    "pkg.prepare_loss_input": pkg.prepare_loss_input is mine.prepare_loss_input,
    "pkg.wrap": pkg.wrap_loss_fn_with_input_preparation is mine.wrap_loss_fn_with_input_preparation,
    "pkg.fusion_wrapper": pkg.SequencePackingFusionLossWrapper is mine.SequencePackingFusionLossWrapper,
    "train.prepare_loss_input": train.prepare_loss_input is mine.prepare_loss_input,
    "train.SequencePackingLossWrapper": train.SequencePackingLossWrapper is mine.SequencePackingLossWrapper,
    "train.apply_top_k_top_p": train.apply_top_k_top_p.__module__.startswith("rl_amd."),
    "train.mask_out": train.mask_out_neg_inf_logprobs is mu.mask_out_neg_inf_logprobs,
    "train.LossPostProcessor": train.LossPostProcessor is mtrain.LossPostProcessor,
    "train.isinstance": train.is_loss_step(object.__new__(mtrain.LossPostProcessor)),
    "train.get_logprobs": train.get_logprobs_from_vocab_parallel_logits.__module__.startswith("rl_amd."),
    "train.untouched": train.allgather_cp_sharded_tensor() == "reference",
    "train.forward": train.forward_with_post_processing_fn is mtrain.forward_with_post_processing_fn,
    "train.forward dispatches": _forward_dispatch(train),
    "lf.calculate_kl": lf.calculate_kl is mu.calculate_kl,
    "lf.masked_mean": lf.masked_mean is mu.masked_mean,
    "driver builds ours": type(fn) is mine.ClippedPGLossFn,
    "enum.loss_type": fn.loss_type is itf.LossType.TOKEN_LEVEL and seq.loss_type is itf.LossType.SEQUENCE_LEVEL,
    "enum.input_type": fn.input_type is itf.LossInputType.LOGPROB
                       and mine.DistillationLossFn.input_type is itf.LossInputType.DISTILLATION,
    "enum.normalizer": fn.metric_normalizations["loss"] is itf.MetricNormalizer.TOKENS
                       and fn.metric_normalizations["num_valid_samples"] is itf.MetricNormalizer.NONE,
    "enum.compare outside": data.normalises_by_tokens(fn) and not data.normalises_by_tokens(seq),
    "enum.exports": mine.LossType is itf.LossType and mine.MetricNormalizer is itf.MetricNormalizer,
    "uncovered forms go to the install": mu.masked_mean(torch.ones(2, 3), torch.ones(2, 3), (0, 1)) == "reference"
                                         and mu.masked_mean(torch.ones(3, dtype=torch.float64), torch.ones(3)) == "reference",
    "driver without a GPU": torch.cuda.is_available() or (
        mu.masked_mean(torch.ones(3), torch.ones(3)) == "reference"
        and mu.calculate_kl(torch.zeros(3), torch.zeros(3)) == "reference"
        and mu.calculate_baseline_and_std_per_prompt(torch.zeros(2, 2, dtype=torch.long), torch.zeros(2), torch.ones(2)) == "reference"),
    "fusable but for the logits": mine.why_not_fusable(fn, None, {}) == "logits are not a [B, S, V] GPU tensor",
}
print("RESULT " + json.dumps(out))
"""


def _run_against_stub_install(tmp_path):
    import json
    import os
    import subprocess
    import sys

    env = dict(os.environ, PYTHONPATH=write_stub_install(tmp_path))
    done = subprocess.run([sys.executable, "-c", _STUB_CHECK], env=env, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-3000:]
    line = [l for l in done.stdout.splitlines() if l.startswith("RESULT ")][-1]
    return json.loads(line[len("RESULT "):])


def test_install_rebinds_an_existing_install_by_identity(tmp_path):
    got = _run_against_stub_install(tmp_path)
    assert got.pop("mode") == ["patched", "patched"]
    assert got.pop("skipped") == ["nemo_rl.models.megatron.train"]      # Megatron-Core is not installed
    wrong = [k for k, v in got.items() if v is not True]
    assert not wrong, wrong


_STUB_MEGATRON_CHECK = r"""
import json
import torch
import nemo_rl.models.megatron.train as mtrain
import rl_amd
from rl_amd import compat
import rl_amd.models.megatron.train as mine

before = [mtrain.forward_with_post_processing_fn]
mode = rl_amd.install()
# a post-processor this package does not replace: the install's own step runs, its scaling included (a GPU is not
# needed for that: the stand-in's apply_temperature_scaling was replaced, and this package's returns CPU logits
# untouched only when there is no temperature)
x = torch.arange(6.0).view(1, 2, 3)
output, fn = mtrain.megatron_forward_backward(lambda mb: x, iter([{"k": 1}]), mtrain.TopkLogitsPostProcessor(), sampling_params=None)
out = {
    "mode": mode,
    "skipped": compat.skipped_modules(),
    "forward replaced": mtrain.forward_with_post_processing_fn is mine.forward_with_post_processing_fn,
    "original kept": compat.original("nemo_rl.models.megatron.train", "forward_with_post_processing_fn") is before[0],
    "LossPostProcessor": mtrain.LossPostProcessor is mine.LossPostProcessor,
    "LogprobsPostProcessor": mtrain.LogprobsPostProcessor is mine.LogprobsPostProcessor,
    "apply_temperature_scaling": mtrain.apply_temperature_scaling is mine.apply_temperature_scaling,
    "passes through": output is x and fn(output) == ("topk", x),
}
print("RESULT " + json.dumps(out))
"""


def test_install_wraps_the_megatron_forward_step(tmp_path):
    """With Megatron-Core importable the Megatron worker module of an install is patched too: its forward step is
    wrapped (the original stays reachable for the wrapper), its post-processors and ``apply_temperature_scaling`` are
    replaced, and a post-processor that stays the install's own runs through the wrapper unchanged."""
    import json
    import os
    import subprocess
    import sys

    env = dict(os.environ, PYTHONPATH=write_stub_install(tmp_path, with_megatron=True))
    done = subprocess.run([sys.executable, "-c", _STUB_MEGATRON_CHECK], env=env, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-3000:]
    got = json.loads([l for l in done.stdout.splitlines() if l.startswith("RESULT ")][-1][len("RESULT "):])
    assert got.pop("mode") == "patched" and got.pop("skipped") == []
    wrong = [k for k, v in got.items() if v is not True]
    assert not wrong, wrong


def test_deferred_temperature_record_dies_with_its_storage_and_refuses_copies():
    import numpy as np

    from rl_amd._deferred import deferred_temperature, pending_temperature, record_temperature

    block = np.zeros(4 * 6 * 32, dtype=np.float32)              # one piece of memory, two storages in turn
    with deferred_temperature():
        a = torch.from_numpy(block).view(4, 6, 32)
        record_temperature(a, 0.7)
        assert pending_temperature(a) == 0.7 and pending_temperature(a[:, :-1]) == 0.7
        assert pending_temperature(a.detach().view(24, 32)) == 0.7
        with pytest.raises(RuntimeError, match="not on record"):
            pending_temperature(a.clone())                      # a copy carries undivided values
        assert pending_temperature(a.double()) == 1.0           # another dtype / width is somebody else's tensor
        assert pending_temperature(torch.zeros(4, 6, 16)) == 1.0
        view = a[1]
        del a                                                   # the storage lives on through the view
        assert pending_temperature(view) == 0.7
        address = view.untyped_storage().data_ptr()
        del view                                                # now it is gone, and its record with it
        b = torch.from_numpy(block).view(4, 6, 32)              # a new storage at the same address
        assert b.untyped_storage().data_ptr() == address
        assert pending_temperature(b) == 1.0
        record_temperature(b, 0.5)
        assert pending_temperature(b) == 0.5
    assert pending_temperature(b) == 1.0
