"""GPU parity: fused lm_head -> logprob (K6, bf16 MFMA) against the CPU oracle.

The reference's matmul returns bf16 logits; two correct implementations can round an individual
logit to neighbouring bf16 values when their fp32 accumulation orders differ, so a logprob may be off
by one bf16 step of its logit (~2^-8 |x|) on a small fraction of tokens.  Checked here: at least 99 %
of the tokens within 2e-3 of the oracle and all within one bf16 step.

Gradients: the reference forms ``G = g * (onehot - softmax)`` and both backward products in fp32
(``model_utils.py:2263-2286``).  The kernels multiply on the bf16 matrix cores with fp32 accumulation (``W`` and
the hidden states are bf16 already) and narrow ``G`` to bf16 once (round to nearest even, relative error at most
2^-8 per element) - except the one-hot term of dH, ``g * W[target]``, the one large entry of a row of ``G``,
which is added in fp32.  The error of an output element is therefore bounded by the narrowing of the terms it
sums: ``|dH - dH_fp32| <= 2^-8 * (|g * softmax| @ |W|)`` and ``|dW - dW_fp32| <= 2^-8 * ((|g * softmax| + |G|)^T @
|hidden|)`` (the target's entry of ``G^T`` is ``bf16(g + bf16(-g * softmax))``: both narrowings count, which matters
for a confident token, where ``|G| = |g| (1 - p)`` is far smaller than the softmax part it is the difference of)
element by element, to which the checks add as much again for logits that round to the neighbouring bf16 value
under another accumulation order, 1e-4 of the largest entry for the fp32 accumulation, and for dW its final
narrowing to bf16.  The fp32 ``dhidden_out`` of the C ABI is what is compared, not its bf16 cast; on the flat
distributions of random weights it comes out at about 1e-5 of the fp32 oracle (Frobenius), checked at 1e-4."""

import pytest
import torch

from oracle import lmhead as OH
from oracle import logprob as OL
from rl_amd import ops
from rl_amd.distributed import model_utils as MU

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _make(s, b, h, v, seed, w_std=0.05):
    g = torch.Generator().manual_seed(seed)
    hid = torch.randn(s, b, h, generator=g).to(torch.bfloat16)
    w = (torch.randn(v, h, generator=g) * w_std).to(torch.bfloat16)
    ids = torch.randint(0, v, (b, s), generator=g)
    return hid, w, ids, g


@pytest.mark.parametrize("s,b,h,v", [(40, 3, 64, 1000), (300, 1, 128, 777), (257, 2, 72, 4099), (64, 8, 256, 32000)])
def test_lmhead_forward_matches_oracle(s, b, h, v):
    hid, w, ids, _ = _make(s, b, h, v, seed=s + v)
    want = OH.hidden_to_logprobs(hid, w, ids)                     # bf16 matmul, fp32 softmax
    exact = OL.from_logits_to_logprobs((hid.float() @ w.float().T).transpose(0, 1), ids)
    got = MU.from_parallel_hidden_states_to_logprobs(hid.to(DEV), w.to(DEV), False, ids.to(DEV), 0, v, None).cpu()
    assert got.shape == (b, s - 1) and got.dtype == torch.float32
    err = (got - want).abs()
    logit_scale = (hid.float() @ w.float().T).abs().max().item()
    assert (err <= 2e-3).float().mean().item() >= 0.99, err.max().item()
    assert err.max().item() <= 2.0 ** -7 * logit_scale + 2e-3
    assert (got - exact).abs().max().item() <= 2.0 ** -7 * logit_scale + 2e-3


def test_lmhead_out_of_range_targets_give_zero():
    hid, w, ids, _ = _make(16, 2, 64, 512, seed=3)
    ids[:, 3] = 600
    got = MU.from_parallel_hidden_states_to_logprobs(hid.to(DEV), w.to(DEV), False, ids.to(DEV), 0, 512, None).cpu()
    assert torch.all(got[:, 2] == 0)


def narrowing_bounds(hid_rows, w, targets, up_rows):
    """fp32 oracle gradients of the rows ``hid_rows [n, H]`` plus the element-wise bounds stated in the module
    text: (dH, dW, bound_dH, bound_dW)."""
    logits = (hid_rows @ w.T).float()                                 # bf16 matmul, as the reference's
    p = torch.softmax(logits, -1)
    grad = (torch.nn.functional.one_hot(targets, w.shape[0]).float() - p) * up_rows.unsqueeze(-1)
    d_h = grad @ w.float()
    d_w = grad.T @ hid_rows.float()
    eps = 2.0 ** -7                                                   # 2^-8 narrowing of G, as much again for flipped logits
    soft = p * up_rows.abs().unsqueeze(-1)                            # the part of G that dH takes through bf16
    b_h = eps * (soft @ w.float().abs()) + 1e-4 * d_h.abs().max()
    b_w = eps * ((soft + grad.abs()).T @ hid_rows.float().abs()) + 1e-4 * d_w.abs().max() + 2.0 ** -8 * d_w.abs()
    return d_h, d_w, b_h, b_w


@pytest.mark.parametrize("s,b,h,v", [(40, 3, 64, 1000), (130, 2, 128, 2500), (96, 4, 256, 8192)])
def test_lmhead_backward_matches_oracle(s, b, h, v):
    hid, w, ids, g = _make(s, b, h, v, seed=7 * s)
    up = torch.randn(b, s, generator=g) * 1e-3
    up[:, -1] = 0
    up[0, 5] = 0
    rolled = ids.roll(-1, -1)
    want_dh, want_dw = OH.hidden_to_logprobs_backward(hid, w, rolled, up)   # fp32 accumulation, dW narrowed once
    hg = hid.to(DEV).requires_grad_(True)
    wg = w.to(DEV).requires_grad_(True)
    lp = MU.from_parallel_hidden_states_to_logprobs(hg, wg, False, ids.to(DEV), 0, v, None)
    (lp * up[:, :-1].to(DEV)).sum().backward()
    assert hg.grad.dtype == torch.bfloat16 and hg.grad.shape == hid.shape
    assert wg.grad.dtype == torch.bfloat16 and wg.grad.shape == w.shape

    # the kernel's own outputs through the op that wraps the C ABI: fp32 dH [N, H], bf16 dW [V, H]
    hid2d = hid.reshape(s * b, h)
    tgt = rolled.t().contiguous().reshape(-1)                          # token order of the hidden rows: (s, b)
    up_rows = up.t().contiguous().reshape(-1)
    _, lse, none = torch.ops.rl_amd.lmhead_logprob_fwd(hid2d.to(DEV), w.to(DEV), tgt.to(DEV), 0, v)
    assert none.numel() == 0
    dh, dw = torch.ops.rl_amd.lmhead_logprob_bwd(hid2d.to(DEV), w.to(DEV), tgt.to(DEV), lse, up_rows.to(DEV), 0, v)
    assert dh.dtype == torch.float32
    o_dh, o_dw, b_dh, b_dw = narrowing_bounds(hid2d, w, tgt, up_rows)
    torch.testing.assert_close(o_dh.view(s, b, h), want_dh, rtol=1e-5, atol=1e-9)   # the two oracle spellings agree
    err_h, err_w = (dh.cpu() - o_dh).abs(), (dw.float().cpu() - o_dw).abs()
    assert bool((err_h <= b_dh).all()), (err_h / b_dh).max().item()
    assert bool((err_w <= b_dw).all()), (err_w / b_dw).max().item()
    # the measured size of that error: well under the bound, and two orders under the 1e-2 the reference allows
    # between its fused and unfused paths (tests/unit/models/policy/test_megatron_worker.py:2571-2658)
    assert (err_h.norm() / o_dh.norm()).item() <= 1e-4
    assert ((dw.float().cpu() - o_dw).norm() / o_dw.norm()).item() <= 3e-3
    assert bool((hg.grad.float().cpu() == dh.cpu().view(s, b, h).to(torch.bfloat16).float()).all())


def test_lmhead_equals_unfused_path_on_gpu():
    """Fused and unfused HIP paths agree (the reference's only test of this path compares the two)."""
    s, b, h, v = 96, 2, 128, 5000
    hid, w, ids, _ = _make(s, b, h, v, seed=11)
    hd, wd, idd = hid.to(DEV), w.to(DEV), ids.to(DEV)
    fused = MU.from_parallel_hidden_states_to_logprobs(hd, wd, False, idd, 0, v, None)
    logits = torch.matmul(hd, wd.T).transpose(0, 1).contiguous()   # [B,S,V] bf16, library GEMM
    unfused = MU.from_parallel_logits_to_logprobs(logits, idd, 0, v, None)
    err = (fused - unfused).abs()
    assert (err <= 2e-3).float().mean().item() >= 0.99
    assert err.max().item() <= 1e-2


def _bwd_through_the_op(hid2d, w, tgt, up_rows, keep=False):
    v = w.shape[0]
    _, lse, logits = torch.ops.rl_amd.lmhead_logprob_fwd(hid2d.to(DEV), w.to(DEV), tgt.to(DEV), 0, v, keep)
    return torch.ops.rl_amd.lmhead_logprob_bwd(hid2d.to(DEV), w.to(DEV), tgt.to(DEV), lse, up_rows.to(DEV), 0, v,
                                               logits if keep else None)


@pytest.mark.parametrize("keep", [False, True])
@pytest.mark.parametrize("live", ["none", "one", "last_only"])
def test_lmhead_backward_runs_on_live_tokens_only(live, keep):
    """The backward products run on the tokens with a non-zero upstream gradient (the others have a zero row in the
    logits' gradient): no such token, a single one, and one at the very end."""
    g = torch.Generator().manual_seed(5)
    n, h, v = 300, 64, 1000
    hid = torch.randn(n, h, generator=g).to(torch.bfloat16)
    w = (torch.randn(v, h, generator=g) * 0.05).to(torch.bfloat16)
    tgt = torch.randint(0, v, (n,), generator=g)
    up = torch.zeros(n)
    if live == "one":
        up[137] = 0.5
    elif live == "last_only":
        up[n - 1] = -0.25
    dh, dw = _bwd_through_the_op(hid, w, tgt, up, keep)
    o_dh, o_dw, b_dh, b_dw = narrowing_bounds(hid, w, tgt, up)
    if live == "none":
        assert bool((dh == 0).all()) and bool((dw.float() == 0).all())
        return
    assert bool((dh.cpu()[up == 0] == 0).all())
    assert bool(((dh.cpu() - o_dh).abs() <= b_dh).all()) and bool(((dw.float().cpu() - o_dw).abs() <= b_dw).all())


@pytest.mark.parametrize("keep", [False, True])
def test_lmhead_backward_live_tokens_across_the_chunk_boundary(keep):
    """More live tokens than one backward chunk holds (16384), ending in a partial chunk whose length is not a
    multiple of the 64-wide K slab; masked tokens scattered in between."""
    g = torch.Generator().manual_seed(6)
    n, h, v = 20011, 64, 520
    hid = torch.randn(n, h, generator=g).to(torch.bfloat16)
    w = (torch.randn(v, h, generator=g) * 0.05).to(torch.bfloat16)
    tgt = torch.randint(0, v, (n,), generator=g)
    up = torch.randn(n, generator=g) * 1e-3
    up[torch.rand(n, generator=g) < 0.1] = 0.0
    assert 16384 < int((up != 0).sum()) < n and int((up != 0).sum()) % 64 != 0
    dh, dw = _bwd_through_the_op(hid, w, tgt, up, keep)
    o_dh, o_dw, b_dh, b_dw = narrowing_bounds(hid, w, tgt, up)
    assert bool((dh.cpu()[up == 0] == 0).all())
    assert bool(((dh.cpu() - o_dh).abs() <= b_dh).all())
    assert bool(((dw.float().cpu() - o_dw).abs() <= b_dw).all())
    assert ((dh.cpu() - o_dh).norm() / o_dh.norm()).item() <= 1e-4


@pytest.mark.parametrize("n,h,v", [(300, 64, 1000), (257, 72, 4099), (515, 128, 777), (64, 256, 32000)])
def test_lmhead_kept_logits_are_the_rounded_product_and_give_the_same_gradients(n, h, v):
    """With ``keep_logits`` the forward leaves the bf16 logits and the backward reads them instead of recomputing
    the product: the kept values are the product rounded to bf16 (to one bf16 step of the fp32 product, the same
    latitude as the logprobs), logprobs and log-sum-exps do not change, and the gradients equal those of the
    recomputing backward -- bit for bit, as both take their softmax from the same rounded logits -- and stay within
    the oracle's narrowing bounds.  Vocabulary sizes that are not a multiple of 8 and token counts that are not a
    multiple of the 128-wide tile are among the cases."""
    g = torch.Generator().manual_seed(n + v)
    hid = torch.randn(n, h, generator=g).to(torch.bfloat16)
    w = (torch.randn(v, h, generator=g) * 0.05).to(torch.bfloat16)
    tgt = torch.randint(0, v, (n,), generator=g)
    up = torch.randn(n, generator=g) * 1e-3
    up[torch.rand(n, generator=g) < 0.2] = 0.0
    hd, wd, td, ud = hid.to(DEV), w.to(DEV), tgt.to(DEV), up.to(DEV)
    lp0, lse0, _ = torch.ops.rl_amd.lmhead_logprob_fwd(hd, wd, td, 0, v)
    lp1, lse1, kept = torch.ops.rl_amd.lmhead_logprob_fwd(hd, wd, td, 0, v, True)
    logits = ops.lmhead_unpack_kept_logits(kept, n, v)
    assert logits.shape == (n, v) and logits.dtype == torch.bfloat16
    assert bool((lp0 == lp1).all()) and bool((lse0 == lse1).all())
    exact = hid.float() @ w.float().T
    step = 2.0 ** -8 * exact.abs() + 1e-30
    assert bool(((logits.float().cpu() - exact).abs() <= step * 1.01 + 1e-6 * exact.abs().max()).all())
    # the log-sum-exp of the kept logits is the one the forward reported
    torch.testing.assert_close(torch.logsumexp(logits.float(), -1), lse1, rtol=0, atol=2e-5)
    dh0, dw0 = torch.ops.rl_amd.lmhead_logprob_bwd(hd, wd, td, lse0, ud, 0, v)
    dh1, dw1 = torch.ops.rl_amd.lmhead_logprob_bwd(hd, wd, td, lse1, ud, 0, v, kept)
    o_dh, o_dw, b_dh, b_dw = narrowing_bounds(hid, w, tgt, up)
    assert bool(((dh1.cpu() - o_dh).abs() <= b_dh).all()) and bool(((dw1.float().cpu() - o_dw).abs() <= b_dw).all())
    assert bool((dh0 == dh1).all()) and bool((dw0 == dw1).all())


@pytest.mark.parametrize("keep", [True, False, "auto"])
def test_lmhead_autograd_with_and_without_kept_logits(keep, monkeypatch):
    s, b, h, v = 130, 2, 128, 2500
    hid, w, ids, g = _make(s, b, h, v, seed=21)
    up = torch.randn(b, s - 1, generator=g) * 1e-3
    monkeypatch.setattr(MU, "LMHEAD_KEEP_LOGITS", False)
    h0, w0 = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    lp0 = MU.from_parallel_hidden_states_to_logprobs(h0, w0, False, ids.to(DEV), 0, v, None)
    (lp0 * up.to(DEV)).sum().backward()
    monkeypatch.setattr(MU, "LMHEAD_KEEP_LOGITS", keep)
    h1, w1 = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    lp1 = MU.from_parallel_hidden_states_to_logprobs(h1, w1, False, ids.to(DEV), 0, v, None)
    (lp1 * up.to(DEV)).sum().backward()
    assert bool((lp0 == lp1).all()) and bool((h0.grad == h1.grad).all()) and bool((w0.grad == w1.grad).all())
    with torch.no_grad():   # nothing is kept when no gradient can be asked for
        MU.from_parallel_hidden_states_to_logprobs(hid.to(DEV), w.to(DEV), False, ids.to(DEV), 0, v, None, inference_only=True)


@pytest.mark.parametrize("keep", [False, True])
def test_lmhead_backward_on_confident_tokens(keep):
    """Peaked distributions (the target's probability close to 1, as for most tokens of a trained policy): the
    target's gradient entry ``g (1 - p)`` is the small difference of two large terms, one of which went through bf16;
    the element-wise bounds hold there too, and a vocabulary of one id (probability exactly 1) gives gradients of
    rounding size only."""
    g = torch.Generator().manual_seed(9)
    n, h, v = 200, 64, 300
    hid = torch.randn(n, h, generator=g).to(torch.bfloat16)
    w = (torch.randn(v, h, generator=g) * 0.05).to(torch.bfloat16)
    tgt = torch.randint(0, v, (n,), generator=g)
    hid[50:] = (w[tgt[50:]].float() * 150.0).to(torch.bfloat16)     # rows aligned with their target's weights: p -> 1
    up = torch.randn(n, generator=g) * 1e-2
    p_t = torch.softmax((hid @ w.T).float(), -1).gather(-1, tgt[:, None])[:, 0]
    assert float(p_t[50:].median()) > 0.99
    dh, dw = _bwd_through_the_op(hid, w, tgt, up, keep)
    o_dh, o_dw, b_dh, b_dw = narrowing_bounds(hid, w, tgt, up)
    assert bool(((dh.cpu() - o_dh).abs() <= b_dh).all()) and bool(((dw.float().cpu() - o_dw).abs() <= b_dw).all())
    one = torch.zeros(n, dtype=torch.long)
    dh1, dw1 = _bwd_through_the_op(hid, w[:1].contiguous(), one, up, keep)
    o_dh1, o_dw1, b_dh1, b_dw1 = narrowing_bounds(hid, w[:1], one, up)
    assert bool(((dh1.cpu() - o_dh1).abs() <= b_dh1).all()) and bool(((dw1.float().cpu() - o_dw1).abs() <= b_dw1).all())


_ALIGN_SCRIPT = r"""
import sys, torch
sys.path.insert(0, sys.argv[1])
from rl_amd import ops
g = torch.Generator().manual_seed(5)
n, h, v = 2600, 128, 9000      # 11 token tiles x several vocabulary splits: whole and partial XCD patches
hid = torch.randn(n, h, generator=g).to(torch.bfloat16).cuda()
w = (torch.randn(v, h, generator=g) * 0.05).to(torch.bfloat16).cuda()
tgt = torch.randint(0, v, (n,), generator=g).cuda()
out = []
for keep in (False, True):
    lp, lse, kept = torch.ops.rl_amd.lmhead_logprob_fwd(hid, w, tgt, 0, v, keep)
    if keep:
        kept = ops.lmhead_unpack_kept_logits(kept, n, v)   # (the buffer's padding is not written)
    out += [lp.cpu(), lse.cpu(), kept.cpu()]
torch.save(out, sys.argv[2])
"""


def _forward_in_child(tmp_dir, name, extra_env):
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = tmp_dir / "fwd.py"
    script.write_text(_ALIGN_SCRIPT)
    child_env = {k: v for k, v in os.environ.items() if not k.startswith("NRL_LMHEAD_ALIGN")}
    child_env.update(extra_env)
    out = tmp_dir / f"{name}.pt"
    done = subprocess.run([sys.executable, str(script), root, str(out)], env=child_env, capture_output=True, text=True,
                          timeout=240)
    assert done.returncode == 0, done.stderr[-2000:]
    return torch.load(out, weights_only=True)


@pytest.fixture(scope="module")
def default_forward(tmp_path_factory):
    return _forward_in_child(tmp_path_factory.mktemp("lmhead_align"), "default", {})


@pytest.mark.parametrize("env", [{"NRL_LMHEAD_ALIGN": "0"}, {"NRL_LMHEAD_ALIGN": "1"}, {"NRL_LMHEAD_ALIGN": "3"},
                                 {"NRL_LMHEAD_ALIGN_SPINS": "0"}, {"NRL_LMHEAD_ALIGN": "2", "NRL_LMHEAD_ALIGN_SPINS": "1"}])
def test_lmhead_forward_is_the_same_however_its_workgroups_wait_for_each_other(env, default_forward, tmp_path):
    """The forward's workgroups that share an L2 wait for each other before their first tile (the default), before every
    N-th tile, or never (``NRL_LMHEAD_ALIGN``); a workgroup that is not joined within ``NRL_LMHEAD_ALIGN_SPINS`` polls
    walks on alone (0: every workgroup gives up at once).  None of this touches the arithmetic: logprobs, log-sum-exps
    and kept logits are bit-identical.  The settings are read once per process, hence the child processes."""
    variant = _forward_in_child(tmp_path, "variant", env)
    assert len(variant) == len(default_forward) == 6
    for a, b in zip(default_forward, variant):
        assert a.shape == b.shape
        if a.dtype == torch.bfloat16:
            a, b = a.view(torch.int16), b.view(torch.int16)
        assert bool((a == b).all())
