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
