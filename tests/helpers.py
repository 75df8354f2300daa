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
