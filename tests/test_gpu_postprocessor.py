"""GPU parity of the forward-only LogprobsPostProcessor path against the CPU oracle (tolerances: 1e-5
for fp32 logits, 2e-3 for bf16)."""

from types import SimpleNamespace

import pytest
import torch

from oracle import logprob as OL
from rl_amd.algorithms.logits_sampling_utils import TrainingSamplingParams
from rl_amd.models.automodel import LogprobsPostProcessor

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _pp(packing=False, params=None):
    return LogprobsPostProcessor({"logprob_chunk_size": None}, None, None, None, 1, enable_seq_packing=packing, sampling_params=params)


@pytest.mark.parametrize("dtype,vocab,tol", [(torch.float32, 1000, 1e-5), (torch.bfloat16, 151936, 2e-3), (torch.float32, 33, 1e-5)])
def test_right_padded_batch_matches_oracle(dtype, vocab, tol):
    g = torch.Generator().manual_seed(vocab)
    b, s = 4, 12
    logits = (torch.randn(b, s, vocab, generator=g) * 2).to(dtype)
    ids = torch.randint(0, vocab, (b, s), generator=g)
    lengths = torch.tensor([12, 1, 7, 2])
    want = OL.logprobs_post_process(logits, ids, lengths)
    # poison the padding rows: they must not be read, and must come out as exact zeros
    poisoned = logits.clone()
    for i, n in enumerate(lengths.tolist()):
        poisoned[i, max(n - 1, 0):] = float("nan")
    got = _pp()(poisoned.to(DEV), {"input_lengths": lengths}, SimpleNamespace(seq_len=s, input_ids=ids), b, s)
    assert got.shape == (b, s) and got.dtype == torch.float32
    assert torch.isfinite(got).all()
    assert (got.cpu() - want).abs().max().item() <= tol
    assert bool((got[:, 0] == 0).all())
    for i, n in enumerate(lengths.tolist()):
        assert bool((got[i, n:] == 0).all())
    # bit-identical to the training-side logprobs of the same rows (batch invariance)
    from rl_amd.distributed import model_utils as MU

    train = MU.from_parallel_logits_to_logprobs(logits.to(DEV), ids.to(DEV), 0, vocab, None)
    assert torch.equal(train[0], got[0, 1:])


def test_packed_row_matches_oracle():
    g = torch.Generator().manual_seed(11)
    lens, vocab, smax = [9, 1, 14, 6], 777, 16
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    total = int(cu[-1])
    logits = (torch.randn(1, total, vocab, generator=g) * 2)
    packed_ids = torch.randint(0, vocab, (1, total), generator=g)
    want = OL.logprobs_post_process(logits, packed_ids, torch.tensor(lens), cu_seqlens=cu, original_batch_size=len(lens),
                                    original_seq_len=smax)
    pi = SimpleNamespace(seq_len=total, input_ids=packed_ids, flash_attn_kwargs=SimpleNamespace(cu_seqlens_q=cu))
    got = _pp(packing=True)(logits.to(DEV), {"input_lengths": torch.tensor(lens)}, pi, len(lens), smax)
    assert got.shape == (len(lens), smax)
    assert (got.cpu() - want).abs().max().item() <= 1e-5
    with pytest.raises(ValueError):
        _pp(packing=True)(logits.to(DEV), {"input_lengths": torch.tensor([9, 2, 13, 6])}, pi, len(lens), smax)


def test_top_k_top_p_and_neg_inf_masking():
    g = torch.Generator().manual_seed(12)
    b, s, vocab = 3, 10, 2048
    logits = torch.randn(b, s, vocab, generator=g) * 3
    ids = torch.randint(0, vocab, (b, s), generator=g)
    ids[:, 1:] = torch.where(torch.rand(b, s - 1, generator=g) < 0.7, logits.argmax(-1)[:, :-1], ids[:, 1:])
    lengths = torch.tensor([10, 6, 10])
    tm = (torch.arange(s)[None, :] < lengths[:, None]).float()  # padding is masked, as the driver builds it
    data = {"input_lengths": lengths, "token_mask": tm, "sample_mask": torch.ones(b)}
    want = OL.logprobs_post_process(logits, ids, lengths, top_k=20, top_p=0.9)
    want = OL.mask_out_neg_inf_logprobs(want, data["token_mask"] * data["sample_mask"].unsqueeze(-1))
    params = TrainingSamplingParams(top_k=20, top_p=0.9)
    got = _pp(params=params)(logits.to(DEV), {k: v.to(DEV) for k, v in data.items()}, SimpleNamespace(seq_len=s, input_ids=ids), b, s)
    assert torch.isfinite(got).all()
    assert (got.cpu() - want).abs().max().item() <= 1e-5


def test_more_than_one_gpu_is_refused():
    with pytest.raises(NotImplementedError):
        LogprobsPostProcessor({}, None, None, None, 2)


# ---- the Megatron worker's post-processor (returns a function of the output tensor) ----
def _mpp(packing=False, params=None, fused=False):
    from rl_amd.models.megatron import LogprobsPostProcessor as MegatronPP

    return MegatronPP({"sequence_packing": {"enabled": packing}, "logprob_chunk_size": None}, params, fused)


@pytest.mark.parametrize("dtype,vocab,tol", [(torch.float32, 1000, 1e-5), (torch.bfloat16, 32000, 2e-3)])
def test_megatron_plain_path_matches_oracle(dtype, vocab, tol):
    g = torch.Generator().manual_seed(vocab + 1)
    b, s = 3, 11
    logits = (torch.randn(b, s, vocab, generator=g) * 2).to(dtype)
    ids = torch.randint(0, vocab, (b, s), generator=g)
    want = torch.cat([torch.zeros(b, 1), OL.next_token_logprobs(ids, logits.float())], 1)
    fn = _mpp()({"input_ids": ids.to(DEV)}, ids.to(DEV), None)
    loss, out = fn(logits.to(DEV))
    got = out["logprobs"]
    assert loss.item() == 0.0 and got.shape == (b, s) and got.dtype == torch.float32
    assert (got.cpu() - want).abs().max().item() <= tol and bool((got[:, 0] == 0).all())


def test_megatron_packed_path_matches_oracle():
    g = torch.Generator().manual_seed(12)
    lens, pads, vocab, smax = [9, 2, 14, 6], [3, 2, 0, 1], 500, 16
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    cup = torch.tensor([0] + (torch.tensor(lens) + torch.tensor(pads)).cumsum(0).tolist(), dtype=torch.int32)
    total = int(cup[-1])
    ids = torch.zeros(len(lens), smax, dtype=torch.int64)
    for i, n in enumerate(lens):
        ids[i, :n] = torch.randint(0, vocab, (n,), generator=g)
    packed_ids = OL.pack_input_ids(ids, cu, cup)
    logits = torch.randn(1, total, vocab, generator=g) * 2
    lp = OL.packed_logits_to_logprobs(logits, packed_ids, cup, smax)
    want = torch.cat([torch.zeros(len(lens), 1), lp], 1)
    fn = _mpp(packing=True)({"input_ids": ids.to(DEV)}, packed_ids.to(DEV), cup.to(DEV))
    _, out = fn(logits.to(DEV))
    assert out["logprobs"].shape == (len(lens), smax)
    assert (out["logprobs"].cpu() - want).abs().max().item() <= 1e-5


def test_megatron_fused_linear_and_top_k_paths():
    g = torch.Generator().manual_seed(13)
    b, s, vocab = 2, 9, 400
    ids = torch.randint(0, vocab, (b, s), generator=g)
    # the model already returned logprobs: cut to S - 1 columns and prepend the zero column
    given = -torch.rand(b, s + 3, generator=g)
    _, out = _mpp(fused=True)({"input_ids": ids.to(DEV)}, ids.to(DEV), None)(given.to(DEV))
    assert torch.equal(out["logprobs"].cpu(), torch.cat([torch.zeros(b, 1), given[:, : s - 1]], 1))
    # top-k: logprobs of filtered-out tokens are -inf in the oracle and masked to 0 where the mask is 0
    logits = torch.randn(b, s, vocab, generator=g) * 3
    params = TrainingSamplingParams(top_k=20, top_p=1.0, temperature=1.0)
    tm = torch.ones(b, s, dtype=torch.int64)
    sm = torch.ones(b, dtype=torch.int64)
    want = torch.cat([torch.zeros(b, 1), OL.next_token_logprobs(ids, logits, top_k=20, top_p=1.0)], 1)
    kept = torch.isfinite(want)
    data = {"input_ids": ids.to(DEV), "token_mask": (tm * kept).to(DEV), "sample_mask": sm.to(DEV)}
    _, out = _mpp(params=params)(data, ids.to(DEV), None)(logits.to(DEV))
    got = out["logprobs"].cpu()
    assert (got[kept] - want[kept]).abs().max().item() <= 1e-5 and bool((got[~kept] == 0).all())
