"""``rl_amd.install()`` on an existing install, on the GPU: a loss built through the install's own package
path and the worker's ``functools.partial`` of the install's ``prepare_loss_input`` reaches the single pass.

The install is the stand-in of ``helpers.write_stub_install`` (the reference's import statements, no
reference code); it runs in a child process because ``install()`` rebinds modules for the whole process."""

import json
import subprocess
import sys

import pytest

from helpers import write_stub_install

pytestmark = pytest.mark.gpu

_CHECK = r"""
import json
from functools import partial

import torch

import nemo_rl.algorithms.grpo as grpo                    # binds the originals by name, as the driver does
import nemo_rl.algorithms.loss as _pkg_before
before = [_pkg_before.prepare_loss_input]               # in a list: install() rebinds module globals, this script's too
import nemo_rl.models.automodel.train as train
import rl_amd

mode = rl_amd.install()
import nemo_rl.algorithms.loss as pkg
from rl_amd.algorithms.loss import fused, why_not_fusable
from helpers import synthetic_grpo_batch
from oracle import logprob as OL
from oracle import loss as O

dev = torch.device("cuda:0")
w = synthetic_grpo_batch(2, 2, 40, 4096, seed=7, logits_dtype=torch.float32, logit_std=2.0)
ids, logits = w["input_ids"], w["logits"]
b, s = ids.shape
xo = logits.clone().requires_grad_(True)
lpo = OL.next_token_logprobs(ids, xo)
noise = lambda: torch.cat([torch.zeros(b, 1), lpo.detach() + 0.05 * torch.randn(b, s - 1, generator=w["generator"])], 1)
data = {"input_ids": ids, "token_mask": w["token_mask"], "sample_mask": w["sample_mask"],
        "advantages": torch.randn(b, s, generator=w["generator"]), "prev_logprobs": noise(),
        "generation_logprobs": noise(), "reference_policy_logprobs": noise()}
gs = w["sample_mask"].sum()
gt = (w["token_mask"][:, 1:] * w["sample_mask"].unsqueeze(-1)).sum()
want, _ = O.clipped_pg_loss(O.LossConfig(), lpo, data, gs, gt)
want.backward()

fn = grpo.setup({})                                       # the driver's constructor call
xg = logits.to(dev).requires_grad_(True)
ddev = {k: v.to(dev) for k, v in data.items()}
calls = []
real = fused.fused_logits_clipped_pg_loss
fused.fused_logits_clipped_pg_loss = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
got, metrics = pkg.wrap_loss_fn_with_input_preparation(
    xg, ddev, gs.to(dev), gt.to(dev), fn, partial(train.prepare_loss_input, sampling_params=None))
got.backward()
print("RESULT " + json.dumps({
    "mode": mode,
    "rebinding": before[0] is not pkg.prepare_loss_input and train.prepare_loss_input is pkg.prepare_loss_input,
    "fusable": why_not_fusable(fn, xg, ddev),
    "single_pass_calls": len(calls),
    "loss": [got.item(), want.item()],
    "metric_loss": float(metrics["loss"]),
    "grad_err": (xg.grad.cpu() - xo.grad).abs().max().item(),
    "grad_scale": xo.grad.abs().max().item(),
}))
"""


def test_patched_install_reaches_the_single_pass(tmp_path):
    import os

    env = dict(os.environ, PYTHONPATH=write_stub_install(tmp_path))
    done = subprocess.run([sys.executable, "-c", _CHECK], env=env, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    got = json.loads([l for l in done.stdout.splitlines() if l.startswith("RESULT ")][-1][len("RESULT "):])
    assert got["mode"] == "patched" and got["rebinding"] is True
    assert got["fusable"] is None and got["single_pass_calls"] == 1
    loss, want = got["loss"]
    assert abs(loss - want) <= 1e-4 * abs(want) + 1e-6
    assert abs(got["metric_loss"] - want) <= 1e-4 * abs(want) + 1e-6
    assert got["grad_err"] <= 1e-4 * got["grad_scale"]


_FORWARD_CHECK = r"""
import json, types
import torch

import nemo_rl.models.automodel.train as train
import nemo_rl.algorithms.loss as pkg
import nemo_rl.algorithms.loss.interfaces as itf
import rl_amd

rl_amd.install()
from rl_amd.algorithms.logits_sampling_utils import TrainingSamplingParams
from rl_amd.temperature import apply_temperature_scaling
from helpers import synthetic_grpo_batch

dev = torch.device("cuda:0")
T = 0.7
w = synthetic_grpo_batch(2, 2, 40, 4096, seed=11, logits_dtype=torch.bfloat16, logit_std=3.0)
ids, base = w["input_ids"], w["logits"]
b, s = ids.shape
g = w["generator"]
noise = lambda: torch.cat([torch.zeros(b, 1), -torch.rand(b, s - 1, generator=g) * 4], 1)
data = {"input_ids": ids, "token_mask": w["token_mask"], "sample_mask": w["sample_mask"],
        "advantages": torch.randn(b, s, generator=g), "prev_logprobs": noise(), "generation_logprobs": noise(),
        "reference_policy_logprobs": noise(), "input_lengths": torch.full((b,), s)}
ddev = {k: v.to(dev) for k, v in data.items()}
gs = w["sample_mask"].sum().to(dev)
gt = (w["token_mask"][:, 1:] * w["sample_mask"].unsqueeze(-1)).sum().to(dev)
params = TrainingSamplingParams(top_k=None, top_p=1.0, temperature=T)


class Model:
    # stands for the network: its output is a non-leaf tensor that depends on a parameter
    def __init__(self):
        self.weight = base.to(dev).requires_grad_(True)
    def __call__(self, inputs):
        self.out = self.weight * 1
        return {"logits": self.out}


def microbatch():
    inputs = types.SimpleNamespace(seq_len=s, input_ids=ids.to(dev), flash_attn_kwargs=None)
    return types.SimpleNamespace(data_dict=dict(ddev), processed_inputs=inputs, original_batch_size=b, original_seq_len=s)


fn = pkg.ClippedPGLossFn({})
post = train.LossPostProcessor(fn, {}, None, None, None, 1, 1, False, params)

# the worker's way: through the replaced forward function
m1 = Model()
loss1, metrics1, _ = train.forward_with_post_processing_fn(m1, post, microbatch(), global_valid_seqs=gs, global_valid_toks=gt,
                                                           sampling_params=params)
untouched = torch.equal(m1.out.detach().view(torch.int16), base.to(dev).view(torch.int16))
loss1.backward()

# the reference's sequence spelled out: divide in place, then the post-processor
m2 = Model()
logits = apply_temperature_scaling(m2(None)["logits"], params)
divided = not torch.equal(m2.out.detach().view(torch.int16), base.to(dev).view(torch.int16))
loss2, metrics2 = post(logits=logits, data_dict=dict(ddev), processed_inputs=microbatch().processed_inputs,
                       global_valid_seqs=gs, global_valid_toks=gt)
loss2.backward()

# forward-only logprobs through the same function
lpp = train.LogprobsPostProcessor({}, None, None, None, 1, False, params)
with torch.no_grad():
    lp1, _, _ = train.forward_with_post_processing_fn(Model(), lpp, microbatch(), sampling_params=params)
    m4 = Model()
    lp2 = lpp(logits=apply_temperature_scaling(m4(None)["logits"], params), data_dict=dict(ddev),
              processed_inputs=microbatch().processed_inputs, original_batch_size=b, original_seq_len=s)


# a loss that takes the raw logits (not this package's): it must be handed divided values
class RawLogitsLoss:
    loss_type = itf.LossType.TOKEN_LEVEL
    input_type = itf.LossInputType.LOGIT
    def __call__(self, data, global_valid_seqs, global_valid_toks, logits):
        self.seen = logits.detach().clone()
        return logits.float().mean(), {}


raw = RawLogitsLoss()
m5 = Model()
loss5, _, _ = train.forward_with_post_processing_fn(m5, train.LossPostProcessor(raw, {}, None, None, None, 1, 1, False, params),
                                                    microbatch(), global_valid_seqs=gs, global_valid_toks=gt, sampling_params=params)
loss5.backward()
m6 = Model()
want5 = apply_temperature_scaling(m6(None)["logits"], params)
want5.float().mean().backward()

g1, g2 = m1.weight.grad.float(), m2.weight.grad.float()
print("RESULT " + json.dumps({
    "untouched": untouched, "divided": divided,
    "loss": [loss1.item(), loss2.item()],
    "metric": [float(metrics1["loss"]), float(metrics2["loss"])],
    "grad_equal_share": (g1 == g2).float().mean().item(),
    "grad_err": (g1 - g2).abs().max().item(), "grad_scale": g2.abs().max().item(),
    "logprobs_equal": torch.equal(lp1, lp2),
    "raw_sees_divided": torch.equal(raw.seen.view(torch.int16), want5.detach().view(torch.int16)),
    "raw_grad_equal": torch.equal(m5.weight.grad.view(torch.int16), m6.weight.grad.view(torch.int16)),
}))
"""


def test_the_replaced_forward_function_leaves_the_divide_to_the_kernels(tmp_path):
    """``forward_with_post_processing_fn`` of the DTensor worker, replaced on an install: with this package's loss and
    logprob post-processors the logits are never divided in memory (the kernels apply T), with the results of the
    reference's divide-then-post-process sequence; a loss that takes raw logits receives divided ones, gradient
    included."""
    import os

    env = dict(os.environ, PYTHONPATH=write_stub_install(tmp_path))
    done = subprocess.run([sys.executable, "-c", _FORWARD_CHECK], env=env, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    got = json.loads([l for l in done.stdout.splitlines() if l.startswith("RESULT ")][-1][len("RESULT "):])
    assert got["untouched"] is True and got["divided"] is True
    a, b = got["loss"]
    assert abs(a - b) <= 1e-6 * abs(b) + 1e-7
    a, b = got["metric"]
    assert abs(a - b) <= 1e-6 * abs(b) + 1e-7
    assert got["grad_equal_share"] > 0.98 and got["grad_err"] <= 2.0 ** -7 * got["grad_scale"]
    assert got["logprobs_equal"] is True
    assert got["raw_sees_divided"] is True and got["raw_grad_equal"] is True
