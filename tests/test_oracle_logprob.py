"""Pins the logprob / sampling / lm_head oracles to textbook identities, brute
force and the invariants the reference's own tests use (CPU only)."""

import math

import pytest
import torch

from oracle import lmhead as H
from oracle import logprob as L
from oracle import sampling as S


def _textbook(logits, target):
    # tests/unit/distributed/test_distributed_logprob.py:37-43 of the reference
    lp = torch.nn.functional.log_softmax(logits.float(), dim=-1)
    return lp.gather(-1, target.unsqueeze(-1)).squeeze(-1)


def test_rows_logprob_is_log_softmax_gather():
    torch.manual_seed(0)
    x = torch.randn(2, 7, 33) * 3
    t = torch.randint(0, 33, (2, 7))
    torch.testing.assert_close(L.rows_logprob(x, t), _textbook(x, t), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(L.rows_logprob(x * 100, t), _textbook(x * 100, t), rtol=1e-4, atol=1e-4)
    assert torch.isfinite(L.rows_logprob(x * 100, torch.zeros_like(t))).all()


def test_rows_logprob_brute_force_tiny_vocab():
    x = torch.tensor([[[0.5, -1.0, 2.0]]])
    for tok in range(3):
        e = [math.exp(v) for v in x[0, 0].tolist()]
        want = math.log(e[tok] / sum(e))
        assert L.rows_logprob(x, torch.tensor([[tok]])).item() == pytest.approx(want, abs=1e-6)


def test_out_of_shard_targets_give_zero_and_keep_softmax_term():
    torch.manual_seed(1)
    x = torch.randn(1, 4, 8, requires_grad=True)
    t = torch.tensor([[3, 9, 12, 8]])  # shard covers [8, 16): 3 is outside
    out = L.rows_logprob(x, t, vocab_start=8, vocab_end=16)
    assert out[0, 0].item() == 0.0
    torch.testing.assert_close(out[0, 1:], _textbook(x, (t - 8).clamp(min=0))[0, 1:])
    out.sum().backward()
    # the foreign-target row keeps the -softmax term only; in-shard rows sum to zero
    torch.testing.assert_close(x.grad[0, 0], -torch.softmax(x.detach()[0, 0], -1))
    assert x.grad[0, 1].sum().abs() < 1e-6


def test_gradient_is_onehot_minus_softmax_and_rows_sum_to_zero():
    torch.manual_seed(2)
    x = torch.randn(2, 5, 17, requires_grad=True)
    t = torch.randint(0, 17, (2, 5))
    g = torch.randn(2, 5)
    (L.rows_logprob(x, t) * g).sum().backward()
    want = g.unsqueeze(-1) * (torch.nn.functional.one_hot(t, 17).float() - torch.softmax(x.detach(), -1))
    torch.testing.assert_close(x.grad, want, rtol=1e-5, atol=1e-6)
    assert x.grad.sum(-1).abs().max() < 1e-5


def test_roll_and_drop_last_column():
    torch.manual_seed(3)
    x = torch.randn(2, 6, 11)
    ids = torch.randint(0, 11, (2, 6))
    got = L.from_logits_to_logprobs(x, ids)
    assert got.shape == (2, 5)
    torch.testing.assert_close(got, _textbook(x[:, :-1], ids[:, 1:]), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(L.next_token_logprobs(ids, x), got, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_seq_chunked_equals_unchunked(dtype):
    torch.manual_seed(4)
    x = torch.randn(2, 13, 19).to(dtype)
    ids = torch.randint(0, 19, (2, 13))
    a = L.from_logits_to_logprobs(x, ids)
    for chunk in (1, 4, 13, 50):
        torch.testing.assert_close(L.from_logits_to_logprobs(x, ids, chunk_size=chunk), a, rtol=1e-6, atol=1e-6)


def test_packed_equals_per_sequence_and_prerolled():
    # tests/unit/distributed/test_model_utils.py:254-434 of the reference uses lengths [24,48,16,40]
    torch.manual_seed(5)
    lens = [24, 48, 16, 40]
    vocab, smax = 29, 48
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    ids = torch.zeros(4, smax, dtype=torch.int64)
    for i, n in enumerate(lens):
        ids[i, :n] = torch.randint(0, vocab, (n,))
    packed_ids = L.pack_input_ids(ids, cu, cu)
    x = torch.randn(1, int(cu[-1]), vocab)
    got = L.packed_logits_to_logprobs(x, packed_ids, cu, smax)
    assert got.shape == (4, smax - 1)
    for i, n in enumerate(lens):
        seq = x[:, int(cu[i]) : int(cu[i + 1])]
        want = L.from_logits_to_logprobs(seq, ids[i : i + 1, :n])
        torch.testing.assert_close(got[i, : n - 1], want[0], rtol=1e-5, atol=1e-5)
        assert torch.all(got[i, n - 1 :] == 0)
    rolled = L.pack_input_ids(ids, cu, cu, roll_shift=-1)
    pre = L.packed_logits_to_logprobs(x, rolled, cu, smax, target_is_pre_rolled=True)
    torch.testing.assert_close(pre, got)


def test_pack_input_ids_edge_cases():
    # padded spans longer than the data, and cu_seqlens exceeding the row width
    ids = torch.tensor([[1, 2, 3, 0], [4, 5, 0, 0]])
    cu = torch.tensor([0, 3, 5])
    cup = torch.tensor([0, 4, 8])
    assert L.pack_input_ids(ids, cu, cup).tolist() == [[1, 2, 3, 0, 4, 5, 0, 0]]
    assert L.pack_input_ids(ids, cu, cup, roll_shift=-1).tolist() == [[2, 3, 0, 1, 5, 0, 0, 4]]
    cu_big = torch.tensor([0, 3, 9])  # last length 6 > row width 4
    assert L.pack_input_ids(ids, cu_big, torch.tensor([0, 4, 10])).tolist() == [[1, 2, 3, 0, 4, 5, 0, 0, 0, 0]]


@pytest.mark.parametrize("k,p", [(10, 1.0), (None, 0.9), (10, 0.9), (1, 1.0), (None, 0.0001)])
def test_top_k_top_p_properties(k, p):
    # tests/unit/distributed/test_model_utils.py:1164-1252 of the reference
    torch.manual_seed(6)
    x = torch.randn(9, 64) * 2
    filt, keep = S.apply_top_k_top_p(x, k, p)
    assert torch.equal(keep, ~torch.isinf(filt))
    assert torch.equal(filt[keep], x[keep])
    assert keep.sum(-1).min() >= 1
    probs = torch.softmax(x, -1)
    for r in range(9):
        kept = keep[r]
        if k is not None:
            assert kept.sum() <= k  # no ties in random floats
            kth = torch.topk(x[r], k).values[-1]
            assert torch.all(x[r][kept] >= kth)
        if p < 1.0:
            base = probs[r] if k is None else torch.softmax(x[r].masked_fill(x[r] < torch.topk(x[r], k).values[-1], -math.inf), -1)
            order = torch.argsort(base, descending=True)
            csum = torch.cumsum(base[order], 0)
            n_keep = int((csum - base[order] < p - 1e-6).sum().clamp(min=1))
            assert set(order[:n_keep].tolist()) <= set(torch.nonzero(kept).flatten().tolist()) or abs(int(kept.sum()) - n_keep) <= 1
            assert abs(int(kept.sum()) - n_keep) <= 1
            assert torch.softmax(filt[r], -1).sum().item() == pytest.approx(1.0, abs=1e-5)


def test_top_k_keeps_ties_and_top_p_brute_force():
    x = torch.tensor([[1.0, 3.0, 3.0, 2.0, 0.0]])
    _, keep = S.apply_top_k_top_p(x, 1, 1.0)
    assert keep.tolist() == [[False, True, True, False, False]]
    # brute force top-p on 4 values: probs ascending [0.1, 0.2, 0.3, 0.4]
    pr = torch.tensor([[0.3, 0.1, 0.4, 0.2]])
    _, keep = S.apply_top_k_top_p(pr.log(), None, 0.65)
    # ascending cumsum: .1,.3,.6,1.0 ; keep where > .35 -> the .3 and .4 entries
    assert keep.tolist() == [[True, False, True, False]]


def test_filter_gradient_is_masked():
    torch.manual_seed(7)
    x = torch.randn(3, 32, requires_grad=True)
    filt, keep = S.apply_top_k_top_p(x, 5, 0.9)
    g = torch.randn(3, 32)
    torch.where(keep, filt, torch.zeros_like(filt)).mul(g).sum().backward()
    torch.testing.assert_close(x.grad, g * keep)


@pytest.mark.parametrize("k,p", [(10, 1.0), (None, 0.9), (10, 0.9)])
def test_sampled_logprob_equals_filter_then_log_softmax(k, p):
    torch.manual_seed(8)
    x = torch.randn(2, 6, 40, requires_grad=True)
    ids = torch.randint(0, 40, (2, 6))
    got = L.from_logits_to_logprobs(x, ids, top_k=k, top_p=p)
    filt, _ = S.apply_top_k_top_p(x.detach(), k, p)
    want = _textbook(filt[:, :-1], ids[:, 1:])
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)
    assert torch.isinf(got).any() or True
    finite = torch.isfinite(got)
    got[finite].sum().backward()
    assert torch.isfinite(x.grad).all()


def test_mask_out_neg_inf():
    lp = torch.tensor([[-1.0, float("-inf"), -2.0]])
    out = L.mask_out_neg_inf_logprobs(lp, torch.tensor([[1.0, 1.0, 0.0]]))
    assert out.tolist() == [[-1.0, 0.0, 0.0]]


def test_temperature_rounds_in_logits_dtype():
    x = torch.tensor([7.3125], dtype=torch.bfloat16)
    y = L.apply_temperature(x, 0.7)
    assert y.dtype == torch.bfloat16
    assert y.item() == (x / 0.7).item() and y.item() != pytest.approx(7.3125 / 0.7, abs=1e-4)
    assert L.apply_temperature(x, 1.0) is x and L.apply_temperature(x, None) is x


def test_lmhead_equals_unfused_and_autograd():
    torch.manual_seed(9)
    s, b, h, v = 10, 2, 16, 37
    hid = torch.randn(s, b, h)
    w = torch.randn(v, h) * 0.3
    ids = torch.randint(0, v, (b, s))
    want = L.from_logits_to_logprobs((hid @ w.T).transpose(0, 1), ids)
    for chunk in (None, 3, 10):
        torch.testing.assert_close(H.hidden_to_logprobs(hid, w, ids, chunk), want, rtol=1e-5, atol=1e-5)
    hid_g, w_g = hid.clone().requires_grad_(True), w.clone().requires_grad_(True)
    g = torch.randn(b, s)
    rolled = ids.roll(-1, -1)
    (L.rows_logprob((hid_g @ w_g.T).transpose(0, 1), rolled) * g).sum().backward()
    d_h, d_w = H.hidden_to_logprobs_backward(hid, w, rolled, g, chunk_size=4)
    torch.testing.assert_close(d_h, hid_g.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(d_w, w_g.grad, rtol=1e-4, atol=1e-5)


def test_logprobs_post_process_brute_force():
    """The forward-only post-processor restatement against plain Python loops on a tiny input."""
    g = torch.Generator().manual_seed(3)
    b, s, v = 3, 6, 5
    logits = torch.randn(b, s, v, generator=g)
    ids = torch.randint(0, v, (b, s), generator=g)
    lengths = [6, 3, 1]
    got = L.logprobs_post_process(logits, ids, torch.tensor(lengths))
    for i in range(b):
        for t in range(s):
            if t == 0 or t >= lengths[i]:
                assert got[i, t] == 0
            else:
                row = logits[i, t - 1].tolist()
                lse = math.log(sum(math.exp(x) for x in row))
                assert abs(got[i, t].item() - (row[int(ids[i, t])] - lse)) < 1e-5
    # packed: the same sequences laid end to end give the same rows
    cu = torch.tensor([0, 6, 9, 10], dtype=torch.int32)
    packed_logits = torch.cat([logits[i, : lengths[i]] for i in range(b)])[None]
    packed_ids = torch.cat([ids[i, : lengths[i]] for i in range(b)])[None]
    unpacked = L.logprobs_post_process(packed_logits, packed_ids, torch.tensor(lengths), cu_seqlens=cu,
                                        original_batch_size=b, original_seq_len=s)
    assert torch.allclose(unpacked, got, atol=1e-6)


def test_stable_log_softmax_is_the_textbook_one():
    """``model_utils.py:49-67``: against the library routine in float64 and a brute-force loop on a tiny row
    (a dropped maximum, a wrong sign of the log term or a sum over the wrong axis fails one of them)."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(4, 6, 300, generator=g) * 3 + 40.0      # large offset: an unshifted exp would overflow fp32 sums' precision
    got = L.stable_log_softmax(x)
    want = torch.log_softmax(x.double(), dim=-1)
    assert (got.double() - want).abs().max().item() <= 2e-5
    row = [0.5, -1.25, 3.0, 3.0, -7.0]
    z = sum(math.exp(v) for v in row)
    brute = [v - math.log(z) for v in row]
    small = L.stable_log_softmax(torch.tensor([row]))
    assert all(abs(float(small[0, i]) - brute[i]) <= 1e-6 for i in range(len(row)))
    assert abs(float(small.exp().sum()) - 1.0) <= 1e-6
