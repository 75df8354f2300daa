#!/usr/bin/env python3
"""Benchmark of the GRPO logprob + loss hot path on one MI355X.

One step = one pass of the hot path over one synthetic batch of the workload: for every
microbatch, logits -> token logprobs (K1), clipped-PG loss forward+backward (K4), dlogits (K2),
through the public API (``prepare_loss_input`` -> ``ClippedPGLossFn`` -> autograd).  Inputs are
resident in HBM before the timed region.  Prints ONE JSON line.

Default workload (benchmark config 2): 16 prompts x 8 generations = 128 sequences x 4096 tokens,
V = 151936, bf16 logits ~ N(0,3) with a +8 spike at the target id with p = 0.3, prompt prefix
U[256,1024] masked out; run as microbatches of 16 sequences (19.9 GB of logits each).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# HBM bytes per launch of the dominant kernel measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (scaled by the same counters on a 4 GiB copy), valid for one microbatch of the named workload
MEASURED_TRAFFIC_BYTES = {
    "c2": 16.90e9 + 19.95e9,  # fused_logits_loss_kernel
    "c4": 14.72e9 + 19.92e9,  # topk_topp_stream_kernel (backward): rows of masked tokens are zero-filled unread
    "c4_fwd": 23.54e9,        # topk_topp_fwd_kernel: the row once plus the re-read of the chunks that reach the bound
    "c5": 33.41e9 + 34.38e9,  # fused_logits_loss_kernel, packed
    # lmhead_fwd_kernel: L2 fills (W and hidden-state tiles re-fetched by every 4 x 8 patch of tiles that uses
    # them; 114 GB if the workgroups of a patch stayed in step) + the partial log-sum-exp records written
    "c3_fwd": 207.8e9 + 1.28e9,
}
THREE_PASS_BWD_TRAFFIC_BYTES = {"c2": 16.83e9 + 19.92e9}  # logprob_bwd_kernel

WORKLOADS = {
    # name: (sequences, seq_len, vocab, dtype, sequences per microbatch, logit std, spike p)
    "c2": dict(seqs=128, seq_len=4096, vocab=151936, dtype="bf16", mb_seqs=16, std=3.0, spike_p=0.3,
               desc="benchmark config 2: 16 prompts x 8 = 128 seq x 4096 tok, V=151936 bf16, fwd+bwd to dlogits"),
    "c3": dict(seqs=16, seq_len=4096, vocab=151936, dtype="bf16", mb_seqs=16, std=0.0, spike_p=0.0, hidden=4096,
               desc="benchmark config 3: fused lm_head + logprob, hidden [65536,4096] bf16, W [151936,4096] bf16, fwd+bwd (dH, dW)"),
    "c4": dict(seqs=64, seq_len=8192, vocab=151936, dtype="bf16", mb_seqs=8, std=3.0, spike_p=0.0, temperature=0.7,
               top_k=50, top_p=0.95,
               desc="benchmark config 4: 64 seq x 8192 tok, V=151936 bf16, T=0.7, top_k=50, top_p=0.95, DAPO clip-higher, no KL"),
    "distill": dict(seqs=8, seq_len=4096, vocab=151936, dtype="bf16", mb_seqs=8, std=3.0, spike_p=0.0, topk=64,
                    desc="distillation reductions on 8 x 4096 rows, V=151936 bf16: negative entropy, 64 gathered logprobs, soft cross entropy"),
    "c5": dict(seqs=0, seq_len=131072, vocab=131072, dtype="bf16", mb_seqs=0, std=3.0, spike_p=0.0,
               desc="benchmark config 5: sequences of U[2048,32768] tokens packed into one 131072-token row, V=131072 bf16, "
                    "sequence-level-normalised loss, k3 KL beta=0.001, fwd+bwd to dlogits"),
    "post": dict(seqs=16, seq_len=4096, vocab=151936, dtype="bf16", mb_seqs=16, std=3.0, spike_p=0.0,
                 desc="forward-only LogprobsPostProcessor (prev / reference logprobs): 16 seq x 4096 tok right-padded to "
                      "lengths U[2048,4096], V=151936 bf16"),
    "c1": dict(seqs=32, seq_len=512, vocab=32000, dtype="f32", mb_seqs=32, std=2.0, spike_p=0.0,
               desc="benchmark config 1: 8 prompts x 4 = 32 seq x 512 tok, V=32000 fp32"),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--seqs", type=int, default=None, help="override the number of sequences (smaller test runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 4 GiB device-to-device copy (reference point for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target duration of the CPU baseline sample")
    return ap.parse_args()


class EventTimer:
    """Records HIP events on the current stream around each kernel launch of the timed region."""

    def __init__(self, torch):
        self.torch = torch
        self.open = {}
        self.pairs = {}

    def start(self, name):
        ev = self.torch.cuda.Event(enable_timing=True)
        ev.record()
        self.open[name] = ev

    def stop(self, name):
        ev = self.torch.cuda.Event(enable_timing=True)
        ev.record()
        self.pairs.setdefault(name, []).append((self.open.pop(name), ev))

    def summary(self):
        out = {}
        for name, pairs in self.pairs.items():
            ms = [a.elapsed_time(b) for a, b in pairs]
            out[name] = dict(launches=len(ms), avg_ms=sum(ms) / len(ms), total_ms=sum(ms))
        return out


def make_microbatch(torch, w, n_seq, seed, dev):
    """Synthetic microbatch generated on the GPU (the CPU-generated variant of the same recipe is what
    the parity tests use)."""
    g = torch.Generator(device=dev).manual_seed(seed)
    s, v = w["seq_len"], w["vocab"]
    dtype = torch.bfloat16 if w["dtype"] == "bf16" else torch.float32
    logits = torch.empty((n_seq, s, v), dtype=dtype, device=dev)
    logits.normal_(0.0, w["std"], generator=g)
    ids = torch.randint(0, v, (n_seq, s), generator=g, device=dev)
    if w["spike_p"] > 0:
        hit = (torch.rand((n_seq, s - 1), generator=g, device=dev) < w["spike_p"]).to(dtype) * 8.0
        view = logits[:, :-1]
        idx = ids[:, 1:].unsqueeze(-1)
        view.scatter_add_(-1, idx, hit.unsqueeze(-1))
    lo, hi = (256, 1024) if s >= 2048 else (max(1, s // 8), max(2, s // 4))
    prefix = torch.randint(lo, hi + 1, (n_seq,), generator=g, device=dev)
    token_mask = (torch.arange(s, device=dev).unsqueeze(0) >= prefix.unsqueeze(-1)).to(torch.int64)
    token_mask[:, 0] = 0
    sample_mask = torch.ones(n_seq, dtype=torch.float32, device=dev)
    adv = torch.randn((n_seq, 1), generator=g, device=dev).expand(n_seq, s).contiguous()
    # prev / generation / reference logprobs = current-policy logprobs + N(0, 0.05), as in a real step
    # where the policy has moved only slightly since the rollout
    from rl_amd.distributed.model_utils import get_next_token_logprobs_from_logits

    with torch.no_grad():
        cur = get_next_token_logprobs_from_logits(ids, logits)
    cur = torch.cat([torch.zeros((n_seq, 1), device=dev), cur], dim=1)
    noise = lambda: cur + 0.05 * torch.randn((n_seq, s), generator=g, device=dev)  # noqa: E731
    prev = noise()
    return dict(logits=logits, data={
        "input_ids": ids, "token_mask": token_mask, "sample_mask": sample_mask, "advantages": adv,
        "prev_logprobs": prev, "generation_logprobs": prev, "reference_policy_logprobs": noise(),
    })


def cpu_baseline(torch, w, seconds):
    """The oracle (pure PyTorch restatement of the reference op sequence) on the host cores, on a
    bounded sample of the same workload: real vocabulary and dtype, fewer rows."""
    from oracle import logprob as OL
    from oracle import loss as O

    cores = os.cpu_count() or 1
    threads = min(cores, 16)
    torch.set_num_threads(threads)
    dtype = torch.bfloat16 if w["dtype"] == "bf16" else torch.float32
    v = w["vocab"]

    def run(n_seq, s):
        g = torch.Generator().manual_seed(1002)
        logits = (torch.randn(n_seq, s, v, generator=g) * w["std"]).to(dtype).requires_grad_(True)
        ids = torch.randint(0, v, (n_seq, s), generator=g)
        base = -torch.rand(n_seq, s, generator=g) * 3
        tm = torch.ones(n_seq, s, dtype=torch.int64)
        tm[:, : s // 8] = 0
        data = {"token_mask": tm, "sample_mask": torch.ones(n_seq), "advantages": torch.randn(n_seq, 1, generator=g).expand(n_seq, s),
                "prev_logprobs": base, "generation_logprobs": base, "reference_policy_logprobs": base + 0.05}
        t0 = time.perf_counter()
        lp = OL.next_token_logprobs(ids, logits)
        loss, _ = O.clipped_pg_loss(O.LossConfig(), lp, data, torch.tensor(float(n_seq)), tm[:, 1:].sum().float())
        loss.backward()
        return time.perf_counter() - t0

    s, n_seq = 64, 64
    run(1, s)  # warm-up
    times = []
    while sum(times) < seconds or len(times) < 3:
        times.append(run(n_seq, s))
    times.sort()
    t = times[len(times) // 2]
    rows = n_seq * s
    return dict(value=rows / t, unit="tokens/s", cores=threads, kind="port",
                sample=f"{rows} rows of V={v} {w['dtype']} per iteration, oracle fwd+loss+bwd, median of {len(times)} "
                       f"iterations ({sum(times):.1f} s total), {threads} threads of {cores} host cores")


MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16


def bench_topk(args, torch, w):
    """Config 4: top-k / top-p filtered training logprobs -> DAPO loss -> dlogits (K3 forward + backward)."""
    from rl_amd import ops
    from rl_amd.algorithms.logits_sampling_utils import TrainingSamplingParams
    from rl_amd.algorithms.loss import ClippedPGLossConfig, ClippedPGLossFn, prepare_loss_input

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.seqs:
        w["seqs"] = args.seqs
        w["mb_seqs"] = min(w["mb_seqs"], args.seqs)
    n_mb = (w["seqs"] + w["mb_seqs"] - 1) // w["mb_seqs"]
    mb_bytes = w["mb_seqs"] * w["seq_len"] * w["vocab"] * 2
    free, _ = torch.cuda.mem_get_info()
    n_buf = max(1, min(n_mb, int((free * 0.9 - mb_bytes * 1.5) // mb_bytes)))
    params = TrainingSamplingParams(top_k=w["top_k"], top_p=w["top_p"])
    fn = ClippedPGLossFn(ClippedPGLossConfig(ratio_clip_min=0.2, ratio_clip_max=0.28, reference_policy_kl_penalty=0.0))
    mbs = []
    for i in range(n_buf):
        m = make_microbatch(torch, dict(w, spike_p=0.0), w["mb_seqs"], 4004 + i, dev)
        # logits.div_(T) in bf16, as the worker does before the loss; targets mostly the argmax so that they survive the filter
        m["logits"].mul_(1.0 / w["temperature"])
        top = torch.stack([m["logits"][b].float().argmax(-1) for b in range(w["mb_seqs"])])
        keep = torch.rand(top[:, :-1].shape, device=dev) < 0.8
        m["data"]["input_ids"][:, 1:] = torch.where(keep, top[:, :-1], m["data"]["input_ids"][:, 1:])
        with torch.no_grad():
            from rl_amd.distributed.model_utils import get_next_token_logprobs_from_logits
            cur = get_next_token_logprobs_from_logits(m["data"]["input_ids"], m["logits"], sampling_params=params)
        cur = torch.cat([torch.zeros((w["mb_seqs"], 1), device=dev), torch.nan_to_num(cur, neginf=0.0)], dim=1)
        for k in ("prev_logprobs", "generation_logprobs"):
            m["data"][k] = cur + 0.05 * torch.randn_like(cur)
        m["data"].pop("reference_policy_logprobs", None)
        mbs.append(m)
    tot_seqs = torch.tensor(float(w["seqs"]), device=dev)
    tot_toks = (sum(m["data"]["token_mask"][:, 1:].sum() for m in mbs) * (n_mb / n_buf)).float()

    def step():
        for i in range(n_mb):
            m = mbs[i % n_buf]
            logits = m["logits"].requires_grad_(True)
            loss_input, data = prepare_loss_input(logits, m["data"], fn, sampling_params=params)
            loss, _ = fn(data=data, global_valid_seqs=tot_seqs, global_valid_toks=tot_toks, **loss_input)
            (d,) = torch.autograd.grad(loss, logits)
            del d, loss, loss_input

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer = EventTimer(torch)
    ops.KERNEL_TIMER = timer
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ops.KERNEL_TIMER = None
    k = timer.summary()
    nan = dict(avg_ms=float("nan"))
    fwd, bwd = k.get("topk_topp_fwd", nan), k.get("topk_topp_bwd", nan)
    rows = w["mb_seqs"] * w["seq_len"]
    row_bytes = w["vocab"] * 2
    tokens = w["seqs"] * w["seq_len"]
    fwd_gbs = row_bytes * w["mb_seqs"] * (w["seq_len"] - 1) / (fwd["avg_ms"] * 1e-3) / 1e9
    bwd_gbs = 2 * row_bytes * rows / (bwd["avg_ms"] * 1e-3) / 1e9
    print(json.dumps({
        "metric": "top-k/top-p filtered logprob + DAPO loss fwd/bwd tokens/s at V=151936; % of HBM peak",
        "value": tokens * args.steps / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w["desc"], "sequences": w["seqs"], "seq_len": w["seq_len"], "vocab": w["vocab"],
                   "microbatches": n_mb, "resident_logit_buffers": n_buf},
        "algorithmic_bytes_per_token": 3 * row_bytes,
        "hbm_frac_end_to_end": 3 * row_bytes * tokens * args.steps / elapsed / 1e9 / HBM_PEAK_GBS,
        "roofline": {"bound": "hbm", "kernel": "topk_topp_stream_kernel (backward)", "achieved": bwd_gbs, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": bwd_gbs / HBM_PEAK_GBS,
                     "traffic": MEASURED_TRAFFIC_BYTES["c4"] if not args.seqs else None, "avg_launch_ms": bwd["avg_ms"],
                     "algorithmic_bytes_per_launch": 2 * row_bytes * rows},
        "roofline_fwd": {"bound": "hbm", "kernel": "topk_topp_fwd_kernel", "achieved": fwd_gbs, "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": fwd_gbs / HBM_PEAK_GBS, "avg_launch_ms": fwd["avg_ms"],
                         "traffic": MEASURED_TRAFFIC_BYTES["c4_fwd"] if not args.seqs else None},
        "kernel_ms": {n: round(v["avg_ms"], 4) for n, v in k.items()},
    }))


def bench_distill(args, torch, w):
    """Negative entropy, gathered logprobs and soft-target cross entropy, forward + backward each."""
    from rl_amd import ops
    from rl_amd.distributed import model_utils as MU

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    b, s, v, k = w["seqs"], w["seq_len"], w["vocab"], w["topk"]
    g = torch.Generator(device=dev).manual_seed(6006)
    student = torch.empty((b, s, v), dtype=torch.bfloat16, device=dev).normal_(0.0, w["std"], generator=g)
    teacher = torch.empty((b, s, v), dtype=torch.bfloat16, device=dev).normal_(0.0, w["std"], generator=g)
    idx = torch.randint(0, v, (b, s, k), generator=g, device=dev)
    up2 = torch.randn((b, s), generator=g, device=dev)
    up3 = torch.randn((b, s, k), generator=g, device=dev)

    def step():
        x = student.requires_grad_(True)
        (d,) = torch.autograd.grad((MU.ChunkedDistributedEntropy.apply(x, s, None) * up2).sum(), x)
        del d
        (d,) = torch.autograd.grad((MU.ChunkedDistributedGatherLogprob.apply(x, idx, 0, v, s, None) * up3).sum(), x)
        del d
        (d,) = torch.autograd.grad((MU.DistributedCrossEntropy.apply(x, teacher, None) * up2).sum(), x)
        del d

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer = EventTimer(torch)
    ops.KERNEL_TIMER = timer
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ops.KERNEL_TIMER = None
    km = timer.summary()
    tensor_bytes = b * s * v * 2
    passes = {"neg_entropy_fwd": 1, "neg_entropy_bwd": 2, "gather_logprob_fwd": 1, "gather_logprob_bwd": 2,
              "soft_cross_entropy_fwd": 2, "soft_cross_entropy_bwd": 3}
    kernels = {n: {"avg_launch_ms": round(km[n]["avg_ms"], 4), "algorithmic_bytes_per_launch": passes[n] * tensor_bytes,
                   "achieved_GBps": passes[n] * tensor_bytes / (km[n]["avg_ms"] * 1e-3) / 1e9,
                   "frac_of_hbm_peak": passes[n] * tensor_bytes / (km[n]["avg_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS}
               for n in passes if n in km}
    worst = min(kernels, key=lambda n: kernels[n]["frac_of_hbm_peak"])
    print(json.dumps({
        "metric": "distillation reductions fwd/bwd tokens/s at V=151936 (three losses per token); % of HBM peak",
        "value": 3 * b * s * args.steps / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "config": {"workload": w["desc"]},
        "roofline": {"bound": "hbm", "kernel": worst, "achieved": kernels[worst]["achieved_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": kernels[worst]["frac_of_hbm_peak"], "traffic": None},
        "kernels": kernels,
    }))


def bench_post(args, torch, w):
    """The forward-only post-processor the policy worker runs for prev_logprobs and reference_policy_logprobs."""
    from types import SimpleNamespace

    from rl_amd import ops
    from rl_amd.models.automodel.train import LogprobsPostProcessor

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    b, s, v = w["seqs"], w["seq_len"], w["vocab"]
    g = torch.Generator(device=dev).manual_seed(7007)
    logits = torch.empty((b, s, v), dtype=torch.bfloat16, device=dev).normal_(0.0, w["std"], generator=g)
    ids = torch.randint(0, v, (b, s), generator=g, device=dev)
    lengths = torch.randint(s // 2, s + 1, (b,), generator=g, device=dev)
    pp = LogprobsPostProcessor({"logprob_chunk_size": None}, None, None, None, 1)
    inputs = SimpleNamespace(seq_len=s, input_ids=ids)

    def step():
        return pp(logits, {"input_lengths": lengths}, inputs, b, s)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer = EventTimer(torch)
    ops.KERNEL_TIMER = timer
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ops.KERNEL_TIMER = None
    km = timer.summary()
    live_rows = int((lengths - 1).clamp(min=0).sum().item())   # rows 0 .. length-2 of a sequence are read
    alg = live_rows * v * 2
    k_ms = km["logprob_post_fwd"]["avg_ms"]
    gbs = alg / (k_ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "forward-only token logprobs (post-processor) tokens/s at V=151936; % of HBM peak",
        "value": b * s * args.steps / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w["desc"], "sequences": b, "seq_len": s, "vocab": v, "rows_read": live_rows},
        "roofline": {"bound": "hbm", "kernel": "logprob_post_fwd_kernel", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs / HBM_PEAK_GBS, "traffic": None, "avg_launch_ms": k_ms, "algorithmic_bytes_per_launch": alg},
        "kernel_ms": {k: round(x["avg_ms"], 4) for k, x in km.items()},
    }))


def bench_packed(args, torch, w):
    """One packed row through SequencePackingFusionLossWrapper (single pass), then the three-pass packed path."""
    from rl_amd import ops
    from rl_amd.algorithms.loss import (ClippedPGLossConfig, ClippedPGLossFn, SequencePackingFusionLossWrapper,
                                        prepare_packed_loss_input)
    from rl_amd.distributed.model_utils import from_parallel_logits_to_logprobs_packed_sequences

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    total, v = w["seq_len"], w["vocab"]
    g = torch.Generator(device=dev).manual_seed(5005)
    lens = []
    while sum(lens) < total:
        lens.append(min(int(torch.randint(2048, 32769, (1,), generator=g, device=dev)), total - sum(lens)))
    nseq, smax = len(lens), max(lens)
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=dev)
    logits = torch.empty((1, total, v), dtype=torch.bfloat16, device=dev).normal_(0.0, w["std"], generator=g)
    ids = torch.randint(0, v, (nseq, smax), generator=g, device=dev)
    in_seq = torch.arange(smax, device=dev).unsqueeze(0) < torch.tensor(lens, device=dev).unsqueeze(-1)
    ids = ids * in_seq
    prefix = torch.randint(256, 1025, (nseq, 1), generator=g, device=dev)
    token_mask = ((torch.arange(smax, device=dev).unsqueeze(0) >= prefix) & in_seq).to(torch.int64)
    fn = ClippedPGLossFn(ClippedPGLossConfig(token_level_loss=False, reference_policy_kl_penalty=0.001))
    with torch.no_grad():
        targets = torch.cat([ids[i, : lens[i]].roll(-1) for i in range(nseq)]).unsqueeze(0)
        cur = from_parallel_logits_to_logprobs_packed_sequences(logits, targets, cu, smax, 0, v, None,
                                                                target_is_pre_rolled=True)
    cur = torch.cat([torch.zeros((nseq, 1), device=dev), cur], dim=1)
    noise = lambda: cur + 0.05 * torch.randn((nseq, smax), generator=g, device=dev)  # noqa: E731
    prev = noise()
    data = {"input_ids": ids, "token_mask": token_mask, "sample_mask": torch.ones(nseq, device=dev),
            "advantages": torch.randn((nseq, 1), generator=g, device=dev).expand(nseq, smax).contiguous(),
            "prev_logprobs": prev, "generation_logprobs": prev, "reference_policy_logprobs": noise()}
    gs = torch.tensor(float(nseq), device=dev)
    gt = token_mask[:, 1:].sum().float()
    live_rows = int(gt.item())
    wrapped = SequencePackingFusionLossWrapper(fn, prepare_packed_loss_input, cu, cu)

    def step():
        x = logits.requires_grad_(True)
        loss, _m = wrapped(x, data, gs, gt)
        (d,) = torch.autograd.grad(loss, x)
        del d, loss

    def three_pass_step():
        x = logits.requires_grad_(True)
        loss_input, prepared = prepare_packed_loss_input(x, data, fn, cu, cu)
        loss, _m = fn(data=prepared, global_valid_seqs=gs, global_valid_toks=gt, **loss_input)
        (d,) = torch.autograd.grad(loss, x)
        del d, loss, loss_input

    def timed(fn_step):
        for _ in range(args.warmup):
            fn_step()
        torch.cuda.synchronize()
        timer = EventTimer(torch)
        ops.KERNEL_TIMER = timer
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn_step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ops.KERNEL_TIMER = None
        return dt, timer.summary()

    elapsed, km = timed(step)
    row_bytes = v * 2
    # a live row is read once and its gradient written once; a row that feeds no token is only zero-filled
    alg = live_rows * 2 * row_bytes + (total - live_rows) * row_bytes
    fk = km["fused_packed_logits_loss"]["avg_ms"]
    gbs = alg / (fk * 1e-3) / 1e9
    out = {
        "metric": "GRPO logprob+loss fwd/bwd tokens/s, packed 131072-token row at V=131072; % of HBM peak",
        "value": total * args.steps / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w["desc"], "sequences": nseq, "packed_tokens": total, "vocab": v, "loss_tokens": live_rows,
                   "api": "SequencePackingFusionLossWrapper(ClippedPGLossFn, prepare_packed_loss_input)(logits, batch, ...) + "
                          "autograd.grad -> nrl_fused_packed_logits_grpo_loss"},
        "roofline": {"bound": "hbm", "kernel": "fused_logits_loss_kernel (packed)", "achieved": gbs, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC_BYTES["c5"], "avg_launch_ms": fk,
                     "algorithmic_bytes_per_launch": alg},
        "kernel_ms": {k: round(x["avg_ms"], 4) for k, x in km.items()},
    }
    t_elapsed, tk = timed(three_pass_step)
    out["three_pass"] = {
        "value": total * args.steps / t_elapsed, "unit": "tokens/s", "ms_per_step": t_elapsed / args.steps * 1e3,
        "api": "prepare_packed_loss_input -> nrl_logprob_packed_fwd; ClippedPGLossFn -> nrl_grpo_loss_fwd_bwd; "
               "backward -> nrl_logprob_packed_bwd",
        "kernel_ms": {k: round(x["avg_ms"], 4) for k, x in tk.items()},
    }
    print(json.dumps(out))


def bench_lmhead(args, torch, w):
    """Config 3: hidden states -> logprobs -> loss -> (dH, dW) through the fused MFMA path."""
    from rl_amd import ops
    from rl_amd.algorithms.loss import ClippedPGLossConfig, ClippedPGLossFn
    from rl_amd.distributed.model_utils import from_parallel_hidden_states_to_logprobs

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    b, s, h, v = (args.seqs or w["seqs"]), w["seq_len"], w["hidden"], w["vocab"]
    g = torch.Generator(device=dev).manual_seed(1003)
    hidden = torch.randn((s, b, h), generator=g, device=dev).to(torch.bfloat16).requires_grad_(True)
    weight = (torch.randn((v, h), generator=g, device=dev) * 0.02).to(torch.bfloat16).requires_grad_(True)
    ids = torch.randint(0, v, (b, s), generator=g, device=dev)
    with torch.no_grad():
        cur = from_parallel_hidden_states_to_logprobs(hidden, weight, False, ids, 0, v, None, inference_only=True)
    cur = torch.cat([torch.zeros((b, 1), device=dev), cur], dim=1)
    prev = cur + 0.05 * torch.randn((b, s), generator=g, device=dev)
    tm = (torch.arange(s, device=dev).unsqueeze(0) >= torch.randint(256, 1025, (b, 1), generator=g, device=dev)).long()
    data = {"input_ids": ids, "token_mask": tm, "sample_mask": torch.ones(b, device=dev),
            "advantages": torch.randn((b, 1), generator=g, device=dev).expand(b, s).contiguous(),
            "prev_logprobs": prev, "generation_logprobs": prev,
            "reference_policy_logprobs": cur + 0.05 * torch.randn((b, s), generator=g, device=dev)}
    fn = ClippedPGLossFn(ClippedPGLossConfig(), use_fused_linear_logprobs=True)
    gs, gt = torch.tensor(float(b), device=dev), tm[:, 1:].sum().float()

    def step():
        lp = from_parallel_hidden_states_to_logprobs(hidden, weight, False, ids, 0, v, None)
        loss, _ = fn(next_token_logprobs=lp, data=data, global_valid_seqs=gs, global_valid_toks=gt)
        dh, dw = torch.autograd.grad(loss, (hidden, weight))
        del dh, dw

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer = EventTimer(torch)
    ops.KERNEL_TIMER = timer
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ops.KERNEL_TIMER = None
    k = timer.summary()
    n = b * s
    fwd_ms, bwd_ms = k["lmhead_fwd"]["avg_ms"], k["lmhead_bwd"]["avg_ms"]
    fwd_tf = 2.0 * n * h * v / (fwd_ms * 1e-3) / 1e12
    bwd_alg_tf = 4.0 * n * h * v / (bwd_ms * 1e-3) / 1e12       # dH + dW
    bwd_exec_tf = 6.0 * n * h * v / (bwd_ms * 1e-3) / 1e12      # + recomputed logits
    result = {
        "metric": "fused lm_head + GRPO loss fwd/bwd tokens/s; % of bf16 MFMA peak",
        "value": n * args.steps / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w["desc"], "tokens": n, "hidden": h, "vocab": v},
        "roofline": {"bound": "mfma", "kernel": "lmhead_fwd_kernel", "achieved": fwd_tf, "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": fwd_tf / MFMA_BF16_PEAK_TFLOPS, "traffic": MEASURED_TRAFFIC_BYTES["c3_fwd"] if not args.seqs else None,
                     "avg_launch_ms": fwd_ms},
        "roofline_bwd": {"bound": "mfma", "kernel": "lmhead backward (grad + dH + dW GEMMs)", "achieved": bwd_alg_tf,
                         "achieved_incl_recompute": bwd_exec_tf, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": bwd_alg_tf / MFMA_BF16_PEAK_TFLOPS, "avg_launch_ms": bwd_ms},
        "algorithmic_tflops_end_to_end": 6.0 * n * h * v * args.steps / elapsed / 1e12,
        "kernel_ms": {kk: round(vv["avg_ms"], 4) for kk, vv in k.items()},
    }
    print(json.dumps(result))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)
    import torch

    from rl_amd import _lib, ops
    from rl_amd.algorithms.loss import ClippedPGLossConfig, ClippedPGLossFn, prepare_loss_input

    _lib.load()
    w = dict(WORKLOADS[args.workload])
    if args.workload == "c3":
        return bench_lmhead(args, torch, w)
    if args.workload == "c4":
        return bench_topk(args, torch, w)
    if args.workload == "distill":
        return bench_distill(args, torch, w)
    if args.workload == "c5":
        return bench_packed(args, torch, w)
    if args.workload == "post":
        return bench_post(args, torch, w)
    if args.seqs:
        w["seqs"] = args.seqs
        w["mb_seqs"] = min(w["mb_seqs"], args.seqs)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    elt = 2 if w["dtype"] == "bf16" else 4
    n_mb = (w["seqs"] + w["mb_seqs"] - 1) // w["mb_seqs"]
    mb_bytes = w["mb_seqs"] * w["seq_len"] * w["vocab"] * elt
    free, _total = torch.cuda.mem_get_info()
    # logits of every microbatch stay resident if they fit next to one gradient buffer; otherwise
    # the microbatches cycle through as many distinct buffers as fit
    n_buf = max(1, min(n_mb, int((free * 0.9 - mb_bytes * 1.2) // mb_bytes)))
    mbs = [make_microbatch(torch, w, w["mb_seqs"], 1002 + i, dev) for i in range(n_buf)]
    torch.cuda.synchronize()

    fn = ClippedPGLossFn(ClippedPGLossConfig())  # eps 0.2/0.2, k3 KL beta 0.01, token-level mean
    tot_seqs = torch.tensor(float(w["seqs"]), device=dev)
    tot_toks = sum((m["data"]["token_mask"][:, 1:].sum() for m in mbs)) * (n_mb / n_buf)
    tot_toks = tot_toks.float()

    from rl_amd.algorithms.loss import wrap_loss_fn_with_input_preparation

    def step():
        # the drop-in call: logits + batch -> loss; dispatches to the single-pass kernel when the loss
        # configuration allows it (this one does), and autograd hands back d loss / d logits
        for i in range(n_mb):
            m = mbs[i % n_buf]
            logits = m["logits"].requires_grad_(True)
            loss, _metrics = wrap_loss_fn_with_input_preparation(logits, m["data"], tot_seqs, tot_toks, fn, prepare_loss_input)
            (dlogits,) = torch.autograd.grad(loss, logits)
            del dlogits, loss

    def three_pass_step():
        # the reference's call structure spelled out: logprobs (pass 1), loss on logprobs, backward (passes 2+3)
        for i in range(n_mb):
            m = mbs[i % n_buf]
            logits = m["logits"].requires_grad_(True)
            loss_input, data = prepare_loss_input(logits, m["data"], fn)
            loss, _metrics = fn(data=data, global_valid_seqs=tot_seqs, global_valid_toks=tot_toks, **loss_input)
            (dlogits,) = torch.autograd.grad(loss, logits)
            del dlogits, loss, loss_input

    def timed(fn_step):
        for _ in range(args.warmup):
            fn_step()
        torch.cuda.synchronize()
        timer = EventTimer(torch)
        ops.KERNEL_TIMER = timer
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn_step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ops.KERNEL_TIMER = None
        return dt, timer.summary()

    elapsed, kernels = timed(step)
    tokens_per_step = w["seqs"] * w["seq_len"]
    rows_per_launch = w["mb_seqs"] * w["seq_len"]
    row_bytes = w["vocab"] * elt
    nan = dict(avg_ms=float("nan"))
    fk = kernels.get("fused_logits_loss", nan)
    alg_launch = 2 * row_bytes * rows_per_launch  # every logit read once, every gradient element written once
    f_gbs = alg_launch / (fk["avg_ms"] * 1e-3) / 1e9
    result = {
        "metric": "GRPO logprob+loss fwd/bwd tokens/s at V=151936; % of HBM peak",
        "value": tokens_per_step * args.steps / elapsed,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w["dtype"],
        "data": "synthetic",
        "config": {"workload": w["desc"], "sequences": w["seqs"], "seq_len": w["seq_len"], "vocab": w["vocab"],
                   "microbatches": n_mb, "resident_logit_buffers": n_buf,
                   "loss": "ClippedPGLoss eps=0.2/0.2, k3 KL beta=0.01, token-level",
                   "api": "wrap_loss_fn_with_input_preparation(logits, batch, ...) + autograd.grad -> "
                          "nrl_fused_logits_grpo_loss (seq stats + single pass + term reduce + finish)"},
        "algorithmic_bytes_per_token": 2 * row_bytes,
        "hbm_frac_end_to_end": 2 * row_bytes * tokens_per_step * args.steps / elapsed / 1e9 / HBM_PEAK_GBS,
        "roofline": {"bound": "hbm", "kernel": "fused_logits_loss_kernel", "achieved": f_gbs, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": f_gbs / HBM_PEAK_GBS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload) if not args.seqs else None,
                     "avg_launch_ms": fk["avg_ms"], "algorithmic_bytes_per_launch": alg_launch},
        "kernel_ms": {k: round(v["avg_ms"], 4) for k, v in kernels.items()},
    }
    # ---- the three-pass path (its own row: 3 * V * sizeof per token) ----
    t_elapsed, t_kernels = timed(three_pass_step)
    bwd = t_kernels.get("logprob_bwd", nan)
    fwd = t_kernels.get("logprob_fwd", nan)
    bwd_gbs = 2 * row_bytes * rows_per_launch / (bwd["avg_ms"] * 1e-3) / 1e9
    fwd_gbs = row_bytes * w["mb_seqs"] * (w["seq_len"] - 1) / (fwd["avg_ms"] * 1e-3) / 1e9
    result["three_pass"] = {
        "value": tokens_per_step * args.steps / t_elapsed, "unit": "tokens/s", "ms_per_step": t_elapsed / args.steps * 1e3,
        "api": "prepare_loss_input -> nrl_logprob_fwd; ClippedPGLossFn -> nrl_grpo_loss_fwd_bwd; backward -> nrl_logprob_bwd",
        "algorithmic_bytes_per_token": 3 * row_bytes,
        "hbm_frac_end_to_end": 3 * row_bytes * tokens_per_step * args.steps / t_elapsed / 1e9 / HBM_PEAK_GBS,
        "roofline_bwd": {"bound": "hbm", "kernel": "logprob_bwd_kernel", "achieved": bwd_gbs, "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": bwd_gbs / HBM_PEAK_GBS, "avg_launch_ms": bwd["avg_ms"],
                         "traffic": THREE_PASS_BWD_TRAFFIC_BYTES.get(args.workload) if not args.seqs else None,
                         "algorithmic_bytes_per_launch": 2 * row_bytes * rows_per_launch},
        "roofline_fwd": {"bound": "hbm", "kernel": "logprob_fwd_kernel", "achieved": fwd_gbs, "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": fwd_gbs / HBM_PEAK_GBS, "avg_launch_ms": fwd["avg_ms"]},
        "kernel_ms": {k: round(v["avg_ms"], 4) for k, v in t_kernels.items()},
    }
    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.float32, device=dev).fill_(1.0)  # 4 GiB
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        result["copy_calibration_bytes"] = src.numel() * 4
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(torch, w, args.cpu_seconds)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
