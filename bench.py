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
import contextlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

def source_fingerprint(name):
    """First 12 hex digits of the SHA-256 of ``rl_amd/csrc/<name>``: what a row of the traffic table is tied to."""
    import hashlib

    try:
        with open(os.path.join(ROOT, "rl_amd", "csrc", name), "rb") as fh:
            return hashlib.sha256(fh.read()).hexdigest()[:12]
    except OSError:
        return None


def load_measured_traffic():
    """HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, from the committed table
    ``profiles/measured_traffic.md`` (key -> dict(kernel, read, write, profile)).  Each row names the profile summary
    it was taken from and the kernel's source file with that file's fingerprint at the time of the measurement; a
    row whose source has changed since is dropped here, so the JSON line says ``traffic: null`` instead of quoting
    bytes that belong to another version of the kernel."""
    table = {}
    path = os.path.join(ROOT, "profiles", "measured_traffic.md")
    try:
        with open(path) as fh:
            for line in fh:
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) == 7 and cells[0] not in ("key", "---") and not set(cells[0]) <= set("-"):
                    try:
                        name, _, stamp = cells[5].partition("@")
                        if source_fingerprint(name.strip()) != stamp.strip():
                            continue
                        table[cells[0]] = dict(kernel=cells[1], shape=cells[2], read=float(cells[3]), write=float(cells[4]),
                                               profile=cells[6])
                    except ValueError:
                        pass
    except OSError:
        pass
    return table


MEASURED_TRAFFIC = load_measured_traffic()


def hbm_roofline(kernel, alg_bytes, avg_ms, traffic_key=None, **extra):
    """The roofline record of an HBM-bound kernel: ``achieved`` = algorithmic bytes / average launch time;
    ``traffic`` = measured bytes per launch (or None when no profile covers this launch shape) and
    ``frac_measured`` = those bytes / the same time / peak."""
    gbs = alg_bytes / (avg_ms * 1e-3) / 1e9
    rec = {"bound": "hbm", "kernel": kernel, "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
           "traffic": None, "avg_launch_ms": avg_ms, "algorithmic_bytes_per_launch": alg_bytes}
    row = MEASURED_TRAFFIC.get(traffic_key) if traffic_key else None
    if row is not None:
        moved = row["read"] + row["write"]
        rec["traffic"] = moved
        rec["frac_measured"] = moved / (avg_ms * 1e-3) / 1e9 / HBM_PEAK_GBS
        rec["traffic_profile"] = row["profile"]
    rec.update(extra)
    return rec


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
    "c1": dict(seqs=32, seq_len=512, vocab=32000, dtype="f32", mb_seqs=32, std=2.0, spike_p=0.0, group=4, response_suffix=64,
               desc="benchmark config 1: 8 prompts x 4 = 32 seq x 512 tok, V=32000 fp32, response suffix U[64,512], Bernoulli "
                    "rewards -> group-normalised advantages"),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--seqs", type=int, default=None, help="override the number of sequences (smaller test runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true",
                    help="skip the baseline legs (oracle on the host cores, oracle's op sequence on the GPU, copy bandwidth)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 4 GiB device-to-device copy (reference point for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target duration of the CPU baseline sample")
    ap.add_argument("--source-fingerprints", action="store_true",
                    help="print the fingerprints of the kernel sources (for the rows of profiles/measured_traffic.md) and exit")
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
    if w.get("response_suffix"):   # config 1: the response is a suffix of random length U[64, S]
        prefix = s - torch.randint(w["response_suffix"], s + 1, (n_seq,), generator=g, device=dev)
    else:
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


def timed(torch, ops, args, step):
    """W untimed steps, then K timed ones bracketed by synchronisation; HIP events around every kernel launch of
    the timed region (on the stream the ops launch on).  -> (seconds, per-kernel summary)."""
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer = EventTimer(torch)
    ops.KERNEL_TIMER = timer
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ops.KERNEL_TIMER = None
    return dt, timer.summary()


# ------------------------------------------------------------------------------------------------
# Baseline legs: the oracle (the CPU restatement of the reference's op sequence) on the host cores, the same
# op sequence with stock torch ops on the GPU, and the device's copy bandwidth.  Reported next to the
# measurement; none of it is on the product path.
# ------------------------------------------------------------------------------------------------
def oracle_sample(torch, w, kind, device, rows):
    """One bounded sample of workload ``w`` for the oracle on ``device``: -> (run, rows, unit text).  ``run()`` does one
    forward (+ loss + backward where the workload has one) of the reference's op sequence on about ``rows``
    rows of the real vocabulary and dtype; inputs are built once, outside the timed call."""
    from oracle import distill as OD
    from oracle import lmhead as OH
    from oracle import logprob as OL
    from oracle import loss as O

    g = torch.Generator().manual_seed(1002)
    dtype = torch.bfloat16 if w["dtype"] == "bf16" else torch.float32
    v = w["vocab"]
    s = 64 if rows >= 64 else rows
    n_seq = max(1, rows // s)
    rows = n_seq * s

    def loss_data(n, width, beta_ref=True):
        base = -torch.rand(n, width, generator=g) * 3
        tm = torch.ones(n, width, dtype=torch.int64)
        tm[:, : max(1, width // 8)] = 0
        d = {"token_mask": tm, "sample_mask": torch.ones(n), "advantages": torch.randn(n, 1, generator=g).expand(n, width).contiguous(),
             "prev_logprobs": base, "generation_logprobs": base.clone()}
        if beta_ref:
            d["reference_policy_logprobs"] = base + 0.05
        return {k: t.to(device) for k, t in d.items()}, torch.tensor(float(n), device=device), tm[:, 1:].sum().float().to(device)

    if kind == "lmhead":
        h = w["hidden"]
        hidden = torch.randn(s, n_seq, h, generator=g).to(torch.bfloat16).to(device).requires_grad_(True)
        weight = (torch.randn(v, h, generator=g) * 0.02).to(torch.bfloat16).to(device).requires_grad_(True)
        ids = torch.randint(0, v, (n_seq, s), generator=g).to(device)
        data, gs, gt = loss_data(n_seq, s)

        def run():
            hidden.grad = weight.grad = None
            lp = OH.hidden_to_logprobs(hidden, weight, ids)
            loss, _ = O.clipped_pg_loss(O.LossConfig(), lp, data, gs, gt)
            loss.backward()

        return run, rows, f"{rows} tokens, H={h}, V={v} bf16: hidden -> logprobs -> loss -> (dH, dW) by autograd"

    std = w["std"] or 1.0
    logits = (torch.randn(n_seq, s, v, generator=g) * std).to(dtype).to(device)
    ids = torch.randint(0, v, (n_seq, s), generator=g).to(device)
    if kind == "post":
        lengths = torch.randint(s // 2, s + 1, (n_seq,), generator=g).to(device)

        def run():
            with torch.no_grad():
                OL.logprobs_post_process(logits, ids, lengths)

        return run, rows, f"{rows} rows of V={v} {w['dtype']}: forward-only fp32 log-softmax + gather + padding mask"
    if kind == "distill":
        teacher = (torch.randn(n_seq, s, v, generator=g) * std).to(dtype).to(device)
        idx = torch.randint(0, v, (n_seq, s, w["topk"]), generator=g).to(device)
        x = logits.requires_grad_(True)

        def run():
            x.grad = None
            (OD.neg_entropy(x).sum() + OD.gather_logprob(x, idx).sum() + OD.soft_cross_entropy(x, teacher).sum()).backward()

        return run, rows, f"{rows} rows of V={v} {w['dtype']}: negative entropy + {w['topk']} gathered logprobs + soft cross entropy, fwd+bwd"
    x = logits.requires_grad_(True)
    if kind == "topk":
        ids = logits.float().argmax(-1).roll(1, -1)  # next-token targets that survive the filter
        data, gs, gt = loss_data(n_seq, s, beta_ref=False)
        cfg = O.LossConfig(ratio_clip_min=0.2, ratio_clip_max=0.28, reference_policy_kl_penalty=0.0)

        def run():
            x.grad = None
            scaled = OL.apply_temperature(x, w["temperature"])
            lp = OL.next_token_logprobs(ids, scaled, top_k=w["top_k"], top_p=w["top_p"])
            mask = (data["token_mask"] * data["sample_mask"].unsqueeze(-1))[:, 1:]
            lp = OL.mask_out_neg_inf_logprobs(lp, mask)
            loss, _ = O.clipped_pg_loss(cfg, lp, data, gs, gt)
            loss.backward()

        return run, rows, (f"{rows} rows of V={v} bf16: div_(T) -> top-k/top-p by full sort -> log-softmax -> gather -> DAPO loss -> "
                           "backward")
    if kind == "packed":
        cu = torch.arange(0, rows + 1, s, dtype=torch.int32)
        data, gs, gt = loss_data(n_seq, s)
        packed = x.reshape(1, rows, v)
        cfg = O.LossConfig(token_level_loss=False, reference_policy_kl_penalty=0.001)

        def run():
            x.grad = None
            targets = OL.pack_input_ids(ids.cpu(), cu, cu, roll_shift=-1).to(device)
            lp = OL.packed_logits_to_logprobs(packed, targets, cu, s, target_is_pre_rolled=True)
            loss, _ = O.clipped_pg_loss(cfg, lp, data, gs, gt)
            loss.backward()

        return run, rows, f"{rows} packed rows ({n_seq} sequences) of V={v} bf16: packed logprobs -> sequence-level loss -> backward"
    data, gs, gt = loss_data(n_seq, s)

    def run():
        x.grad = None
        lp = OL.next_token_logprobs(ids, x)
        loss, _ = O.clipped_pg_loss(O.LossConfig(), lp, data, gs, gt)
        loss.backward()

    return run, rows, f"{rows} rows of V={v} {w['dtype']}: logprobs -> clipped-PG loss (k3 KL) -> backward to dlogits"


def cpu_baseline(torch, w, kind, seconds, rows):
    """The oracle on the host cores of the GPU box: median of at least two iterations after one warm-up, bounded
    to about ``seconds`` of work."""
    cores = os.cpu_count() or 1
    threads = min(cores, 16)  # the box's CPU share for one GPU
    torch.set_num_threads(threads)
    run, rows, what = oracle_sample(torch, w, kind, "cpu", rows)
    t0 = time.perf_counter()
    run()  # warm-up
    first = time.perf_counter() - t0
    times = []
    while (sum(times) + first < seconds and len(times) < 25) or len(times) < 2:
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    t = times[len(times) // 2]
    return dict(value=rows / t, unit="tokens/s", cores=threads, kind="port",
                sample=f"{what}; median of {len(times)} iterations after one warm-up ({sum(times) + first:.1f} s in all), "
                       f"{threads} threads of {cores} host cores")


def reference_on_gpu(torch, w, kind, rows):
    """The same op sequence (the oracle's restatement of the reference) with stock torch-ROCm ops on the device:
    what a worker gets from the reference's Python on this GPU without this library."""
    try:
        run, rows, what = oracle_sample(torch, w, kind, "cuda", rows)
        run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        n = 3
        for _ in range(n):
            run()
        torch.cuda.synchronize()
        t = (time.perf_counter() - t0) / n
        peak = torch.cuda.max_memory_allocated()
        return dict(value=rows / t, unit="tokens/s", sample=f"{what}; stock torch ops on the GPU, mean of {n} iterations after one warm-up",
                    ms_per_iteration=t * 1e3)
    except Exception as exc:  # a baseline leg must never take the measurement down with it
        return dict(value=None, unit="tokens/s", error=f"{type(exc).__name__}: {exc}"[:300])
    finally:
        torch.cuda.empty_cache()


def copy_bandwidth(torch, dev):
    """Read + write GB/s of a 4 GiB device-to-device copy (HIP events), the practical ceiling of a kernel that
    streams one tensor in and another out."""
    src = torch.empty(1 << 30, dtype=torch.float32, device=dev).fill_(1.0)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(3):
        dst.copy_(src)
    b.record()
    torch.cuda.synchronize()
    ms = a.elapsed_time(b) / 3
    del src, dst
    torch.cuda.empty_cache()
    return 2 * (1 << 32) / (ms * 1e-3) / 1e9


def read_write_ceiling(torch, logits, ids, read_bytes, write_bytes):
    """What this device delivers to the two halves of a gradient kernel taken apart, on the bench's own buffers:
    a pure read of the logits (the forward logprob kernel, K1) and a pure write of a gradient buffer of the same
    shape (the backward logprob kernel with every upstream gradient zero: rows are zero-filled, nothing is read).
    ``mixed_bound_ms`` = the launch's read bytes at the read rate plus its written bytes at the write rate: the time
    a read + write kernel of that launch would take if the two streams did not disturb each other."""
    ops = torch.ops.rl_amd
    b, s, v = logits.shape
    elt = logits.element_size()
    n = s - 1
    targets = ids[:, 1:]

    def ms_of(fn, reps=3):
        fn()
        torch.cuda.synchronize()
        a, z = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        z.record()
        torch.cuda.synchronize()
        return a.elapsed_time(z) / reps

    with torch.no_grad():
        lse = torch.zeros((b, n), dtype=torch.float32, device=logits.device)
        zero = torch.zeros((b, n), dtype=torch.float32, device=logits.device)
        read_ms = ms_of(lambda: ops.logprob_fwd(logits, targets, n, 0, v, 1.0, 1, False))
        write_ms = ms_of(lambda: ops.logprob_bwd(logits, targets, lse, zero, n, 0, v, 1.0, 1))
    read_gbs = b * n * v * elt / (read_ms * 1e-3) / 1e9
    write_gbs = b * s * v * elt / (write_ms * 1e-3) / 1e9
    torch.cuda.empty_cache()
    return {"read_bandwidth_GBps": read_gbs, "write_bandwidth_GBps": write_gbs,
            "mixed_bound_ms": (read_bytes / read_gbs + write_bytes / write_gbs) / 1e6,
            "mixed_bound_bytes": {"read": read_bytes, "written": write_bytes}}


def worker_scaling(metrics, num_global_batches=1):
    """What the DTensor worker does with the metrics of a microbatch between the loss call and ``backward()``
    (``nemo_rl/models/automodel/train.py:525-533``)."""
    for k in metrics.keys():
        if "_min" in k or "_max" in k:
            continue
        metrics[k] /= num_global_batches
    return metrics


def read_metrics(collected):
    """The DTensor worker's look at the metrics of its microbatches after the step: every value of every record."""
    return [dict(m.items()) for m in collected]


def megatron_metrics(collected, num_global_batches=1):
    """What the Megatron worker does with the metrics of its microbatches after ``forward_backward_func`` has returned
    (``models/policy/workers/megatron_policy_worker.py:1004-1022``): a new dictionary per microbatch, every value read."""
    out = []
    for x in collected:
        scaled = {}
        for k in x.keys():
            scaled[k] = x[k] if ("_min" in k or "_max" in k) else x[k] / num_global_batches
        out.append(scaled)
    return out


def dtensor_worker(torch):
    """The DTensor worker's own call sequence around the loss, ``forward_with_post_processing_fn(model, LossPostProcessor,
    microbatch, ...)`` (``models/automodel/train.py:308-441, 593-653``), with the bench's resident logits standing for the
    model's output: -> ``(module, run(post, logits, data, global_valid_seqs, global_valid_toks, sampling_params))``."""
    import types

    from rl_amd.models.automodel import train as AT

    AT.MODEL_HELPERS = {"model_forward": lambda model, inputs, **kw: model(inputs), "extract_logits": lambda model, out: out}

    def run(post, logits, data, seqs, toks, sampling_params=None):
        b, s = logits.shape[0], logits.shape[1]
        mb = types.SimpleNamespace(data_dict=data, processed_inputs=None, original_batch_size=b, original_seq_len=s)
        loss, metrics, _ = AT.forward_with_post_processing_fn(lambda inputs: logits, post, mb, global_valid_seqs=seqs,
                                                              global_valid_toks=toks, sampling_params=sampling_params)
        return loss, metrics

    return AT, run


def finish(result, args, torch, w, kind, cpu_rows, gpu_rows):
    """Adds the baseline legs to a workload's record and prints the one JSON line."""
    if not args.no_cpu_baseline:
        dev = torch.device("cuda:0")
        torch.cuda.empty_cache()
        free, _ = torch.cuda.mem_get_info()
        if free > (10 << 30):
            gbs = copy_bandwidth(torch, dev)
            result["copy_bandwidth_GBps"] = gbs
            roof = result.get("roofline", {})
            if roof.get("bound") == "hbm" and roof.get("achieved"):
                roof["copy_bandwidth_frac"] = roof["achieved"] / gbs
        result["reference_on_gpu"] = reference_on_gpu(torch, w, kind, gpu_rows)
        result["cpu_baseline"] = cpu_baseline(torch, w, kind, args.cpu_seconds, cpu_rows)
    print(json.dumps(result), file=_JSON_OUT, flush=True)


MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16


def bench_topk(args, torch, w):
    """Config 4: temperature 0.7 + top-k / top-p filtered training logprobs -> DAPO loss -> dlogits (K3 forward +
    backward).  Headline: the DTensor worker's sequence, ``forward_with_post_processing_fn`` with a ``LossPostProcessor``
    (model output -> ``apply_temperature_scaling`` -> ``prepare_loss_input`` -> loss), with no switch of this package
    set; the function leaves the temperature divide to the kernels because this package's post-processor reads the
    logits next.  Rows of their own: the -inf warning printed at once, the divide as an in-place pass of its own (the Megatron
    worker's step), the backward without the kept-set record, and a forward over flat rows."""
    from functools import partial

    from rl_amd import ops
    from rl_amd.algorithms.logits_sampling_utils import TrainingSamplingParams
    from rl_amd.algorithms.loss import ClippedPGLossConfig, ClippedPGLossFn, prepare_loss_input
    from rl_amd.distributed.model_utils import get_next_token_logprobs_from_logits
    from rl_amd.temperature import apply_temperature_scaling, deferred_temperature

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.seqs:
        w["seqs"] = args.seqs
        w["mb_seqs"] = min(w["mb_seqs"], args.seqs)
    n_mb = (w["seqs"] + w["mb_seqs"] - 1) // w["mb_seqs"]
    mb_bytes = w["mb_seqs"] * w["seq_len"] * w["vocab"] * 2
    free, _ = torch.cuda.mem_get_info()
    n_buf = max(1, min(n_mb, int((free * 0.9 - mb_bytes * 2.6) // mb_bytes)))
    params = TrainingSamplingParams(top_k=w["top_k"], top_p=w["top_p"], temperature=w["temperature"])
    prepare = partial(prepare_loss_input, sampling_params=params)  # as the DTensor worker binds it
    fn = ClippedPGLossFn(ClippedPGLossConfig(ratio_clip_min=0.2, ratio_clip_max=0.28, reference_policy_kl_penalty=0.0))
    mbs = []
    for i in range(n_buf):
        m = make_microbatch(torch, dict(w, spike_p=0.0), w["mb_seqs"], 4004 + i, dev)
        # targets mostly the argmax so that they survive the filter
        top = torch.stack([m["logits"][b].float().argmax(-1) for b in range(w["mb_seqs"])])
        keep = torch.rand(top[:, :-1].shape, device=dev) < 0.8
        m["data"]["input_ids"][:, 1:] = torch.where(keep, top[:, :-1], m["data"]["input_ids"][:, 1:])
        with torch.no_grad(), deferred_temperature():
            cur = get_next_token_logprobs_from_logits(m["data"]["input_ids"], apply_temperature_scaling(m["logits"], params),
                                                      sampling_params=params)
        cur = torch.cat([torch.zeros((w["mb_seqs"], 1), device=dev), torch.nan_to_num(cur, neginf=0.0)], dim=1)
        for k in ("prev_logprobs", "generation_logprobs"):
            m["data"][k] = cur + 0.05 * torch.randn_like(cur)
        m["data"].pop("reference_policy_logprobs", None)
        mbs.append(m)
    tot_seqs = torch.tensor(float(w["seqs"]), device=dev)
    tot_toks = (sum(m["data"]["token_mask"][:, 1:].sum() for m in mbs) * (n_mb / n_buf)).float()

    class _ModelOutput(torch.autograd.Function):
        """Hands the resident logits buffer out as a non-leaf tensor, as a model's forward would: the worker's
        in-place ``logits.div_(T)`` is only legal on such a tensor.  No copy; the gradient stops here."""

        @staticmethod
        def forward(ctx, buffer, anchor):
            return buffer.detach()

        @staticmethod
        def backward(ctx, grad):
            return None, grad.new_zeros(())

    anchor = torch.zeros((), device=dev, requires_grad=True)
    one = torch.ones((), device=dev)
    restore_events = []

    AT, _ = dtensor_worker(torch)   # the DTensor worker's own sequence, the resident logits standing for the model's output
    import types

    post = AT.LossPostProcessor(fn, {}, None, None, None, 1, 1, False, params)

    def step(defer=True):
        collected = []
        for i in range(n_mb):
            m = mbs[i % n_buf]
            if defer:
                # (the function leaves the divide to the kernels by itself: this package's post-processor comes next)
                mb = types.SimpleNamespace(data_dict=m["data"], processed_inputs=None, original_batch_size=w["mb_seqs"],
                                           original_seq_len=w["seq_len"])
                loss, metrics, _ = AT.forward_with_post_processing_fn(
                    lambda inputs: _ModelOutput.apply(m["logits"], anchor), post, mb, global_valid_seqs=tot_seqs,
                    global_valid_toks=tot_toks, sampling_params=params)
            else:
                # apply_temperature_scaling called on its own, outside the workers' forward functions: in place
                out = _ModelOutput.apply(m["logits"], anchor)
                logits = apply_temperature_scaling(out, params)
                loss_input, data = prepare(logits=logits, data=m["data"], loss_fn=fn)
                loss, metrics = fn(data=data, global_valid_seqs=tot_seqs, global_valid_toks=tot_toks, **loss_input)
                del loss_input, logits, out
            collected.append(worker_scaling(metrics) if defer else metrics)
            torch.autograd.grad(loss, anchor)
            del loss
            if not defer:
                # Not part of the step: the bench keeps its logits resident, so after an in-place divide it multiplies
                # them back (a worker gets fresh logits from its model).  Timed with events and taken off the clock.
                a, z = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                torch.ops.rl_amd.scale_rows_(m["logits"], one, 1.0 / w["temperature"])
                z.record()
                restore_events.append((a, z))
        if defer:
            read_metrics(collected)
        else:
            megatron_metrics(collected)

    def timed_eager():
        """-> (seconds without the restoring passes, kernel summary)."""
        restore_events.clear()
        total, k = timed(torch, ops, args, lambda: step(defer=False))
        restore_ms = sum(a.elapsed_time(z) for a, z in restore_events[-args.steps * n_mb:])
        k.get("scale_rows", {}).pop("total_ms", None)
        return total - restore_ms * 1e-3, k, restore_ms / (args.steps * n_mb)

    # The headline is the DTensor worker's sequence with no switch of this package set.  Rows of their own: the same
    # with the warning about valid tokens whose logprob is -inf printed before mask_out_neg_inf_logprobs returns, as the
    # reference prints it (one wait per microbatch), and the divide as a pass of its own.
    from rl_amd.algorithms import utils as AU

    elapsed, k = timed(torch, ops, args, step)
    AU.flush_neg_inf_warnings()
    AU.DEFER_NEG_INF_WARNING = False
    try:
        o_elapsed, ok_ = timed(torch, ops, args, step)
    finally:
        AU.DEFER_NEG_INF_WARNING = True
    # the same step with the backward streaming the logits again instead of using the forward's record of the kept sets
    from rl_amd.distributed import sampling_logprob as SL

    record_capacity = SL._record_capacity
    SL._record_capacity = lambda top_k: 0
    try:
        s_elapsed, sk = timed(torch, ops, args, step)
    finally:
        SL._record_capacity = record_capacity
    # last, because the in-place divides and their restoring passes leave the logits a few roundings off
    e_elapsed, ek, restore_avg_ms = timed_eager()
    nan = dict(avg_ms=float("nan"))
    fwd, bwd = k.get("topk_topp_fwd", nan), k.get("topk_topp_bwd", nan)
    rows = w["mb_seqs"] * w["seq_len"]
    row_bytes = w["vocab"] * 2
    tokens = w["seqs"] * w["seq_len"]
    full = not args.seqs

    def row(seconds, kernels, note):
        return {"value": tokens * args.steps / seconds, "unit": "tokens/s", "ms_per_step": seconds / args.steps * 1e3,
                "hbm_frac_end_to_end": 2 * row_bytes * tokens * args.steps / seconds / 1e9 / HBM_PEAK_GBS,
                "kernel_ms": {n: round(v["avg_ms"], 4) for n, v in kernels.items()}, "note": note}

    result = {
        "metric": "top-k/top-p filtered logprob + DAPO loss fwd/bwd tokens/s at V=151936; % of HBM peak",
        "value": tokens * args.steps / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w["desc"], "sequences": w["seqs"], "seq_len": w["seq_len"], "vocab": w["vocab"],
                   "microbatches": n_mb, "resident_logit_buffers": n_buf,
                   "api": "forward_with_post_processing_fn(model, LossPostProcessor(ClippedPGLossFn, sampling_params), microbatch, "
                          "..., sampling_params) of the DTensor worker, then metrics[k] /= num_global_batches and backward, per "
                          "microbatch; every metrics record read after the last one; no rl_amd-specific switch is set",
                   "temperature": "apply_temperature_scaling inside that function; because this package's post-processor reads "
                                  "the logits next, the divide is applied by the kernels (bf16 rounding of a GPU div_, value and "
                                  "gradient) instead of a pass over the logits",
                   "neg_inf_warning": "printed when its two counts have arrived from the device (the package's default)"},
        # the forward reads a row once; the backward writes the gradient row (zeros and the <= 64 kept entries the
        # forward left on record) without reading the logits again
        "algorithmic_bytes_per_token": 2 * row_bytes,
        "hbm_frac_end_to_end": 2 * row_bytes * tokens * args.steps / elapsed / 1e9 / HBM_PEAK_GBS,
        "roofline": hbm_roofline("fill_zero_flat_kernel + topk_topp_stream_kernel (backward from the kept-set record: write only)", row_bytes * rows,
                                 bwd["avg_ms"], "c4" if full else None),
        "roofline_fwd": hbm_roofline("topk_topp_fwd_kernel", row_bytes * w["mb_seqs"] * (w["seq_len"] - 1), fwd["avg_ms"],
                                     "c4_fwd" if full else None),
        "kernel_ms": {n: round(v["avg_ms"], 4) for n, v in k.items()},
        "immediate_warning": row(o_elapsed, ok_, "DEFER_NEG_INF_WARNING = False: mask_out_neg_inf_logprobs waits for its two counts and "
                                                 "prints the warning before it returns, once per microbatch"),
        "in_place_divide": dict(
            row(e_elapsed, ek, "apply_temperature_scaling called on its own (outside the workers' forward functions): one "
                               "in-place pass over the logits, and a second pass when autograd sends the gradient back through it"),
            roofline=hbm_roofline("scale_rows_kernel (the eager divide and its backward; also the restoring pass)",
                                  2 * row_bytes * rows, ek.get("scale_rows", nan)["avg_ms"]),
            clock="wall clock of the steps minus the event-timed passes that multiply the resident logits back after each "
                  "in-place divide (%.3f ms each; a worker's logits come fresh from its model)" % restore_avg_ms),
        "streaming_backward": {
            "value": tokens * args.steps / s_elapsed, "unit": "tokens/s", "ms_per_step": s_elapsed / args.steps * 1e3,
            "kernel_ms": {n: round(v["avg_ms"], 4) for n, v in sk.items()},
            "roofline": hbm_roofline("topk_topp_stream_kernel (backward reading the logits)", 2 * row_bytes * rows,
                                     sk.get("topk_topp_bwd", nan)["avg_ms"], "c4_streaming" if full else None),
            "note": "without the kept-set record: the backward streams every live row again (3 x V bytes per token)"},
    }
    if not args.no_cpu_baseline:
        result.update(read_write_ceiling(torch, mbs[0]["logits"].detach(), mbs[0]["data"]["input_ids"],
                                         read_bytes=rows * row_bytes, write_bytes=rows * row_bytes))
    del mbs
    torch.cuda.empty_cache()
    # ---- flat rows: top-p alone over N(0, 1) logits (an early-training policy) -- every row's nucleus is far wider
    # than the on-chip candidate list, so every row is finished by the radix descent of topk_topp_wide_kernel ----
    flat_rows = w["mb_seqs"] * w["seq_len"] if full else min(4096, w["mb_seqs"] * w["seq_len"])
    gen = torch.Generator(device=dev).manual_seed(4044)
    flat = torch.empty((1, flat_rows + 1, w["vocab"]), dtype=torch.bfloat16, device=dev).normal_(0.0, 1.0, generator=gen)
    flat_ids = torch.randint(0, w["vocab"], (1, flat_rows + 1), generator=gen, device=dev)
    flat_params = TrainingSamplingParams(top_k=None, top_p=w["top_p"], temperature=1.0)

    def flat_step():
        with torch.no_grad():
            get_next_token_logprobs_from_logits(flat_ids, flat, sampling_params=flat_params)

    f_elapsed, fk = timed(torch, ops, args, flat_step)
    f_ms = fk.get("topk_topp_fwd", nan)["avg_ms"]
    result["c4_flat"] = {
        "value": flat_rows * args.steps / f_elapsed, "unit": "tokens/s", "ms_per_step": f_elapsed / args.steps * 1e3,
        "rows": flat_rows, "us_per_row": f_ms * 1e3 / flat_rows,
        "roofline": hbm_roofline("topk_topp_fwd_kernel + topk_topp_wide_kernel (every row wide)", row_bytes * flat_rows, f_ms,
                                 "c4_flat" if flat_rows == 65536 and w["vocab"] == 151936 else None),
        "note": "forward only: top_p=%.2f alone on bf16 N(0,1) logits; the kept set of every row (~10^5 ids) exceeds the "
                "4096-entry candidate list, so the forward marks the row and the wide kernel finds threshold, tie index and "
                "kept log-sum-exp in three more passes over the row (two key digits + the tie search); algorithmic bytes = "
                "one read of the row" % w["top_p"]}
    del flat
    finish(result, args, torch, w, "topk", cpu_rows=256, gpu_rows=2048)


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

    elapsed, km = timed(torch, ops, args, step)
    tensor_bytes = b * s * v * 2
    passes = {"neg_entropy_fwd": 1, "neg_entropy_bwd": 2, "gather_logprob_fwd": 1, "gather_logprob_bwd": 2,
              "soft_cross_entropy_fwd": 2, "soft_cross_entropy_bwd": 3}
    kernels = {n: {"avg_launch_ms": round(km[n]["avg_ms"], 4), "algorithmic_bytes_per_launch": passes[n] * tensor_bytes,
                   "achieved_GBps": passes[n] * tensor_bytes / (km[n]["avg_ms"] * 1e-3) / 1e9,
                   "frac_of_hbm_peak": passes[n] * tensor_bytes / (km[n]["avg_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS}
               for n in passes if n in km}
    worst = min(kernels, key=lambda n: kernels[n]["frac_of_hbm_peak"])
    result = {
        "metric": "distillation reductions fwd/bwd tokens/s at V=151936 (three losses per token); % of HBM peak",
        "value": 3 * b * s * args.steps / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "config": {"workload": w["desc"]},
        "roofline": hbm_roofline(worst, passes[worst] * tensor_bytes, km[worst]["avg_ms"]),
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        ids0 = torch.zeros(student.shape[:2], dtype=torch.int64, device=student.device)
        nbytes = student.numel() * student.element_size()
        result.update(read_write_ceiling(torch, student.detach(), ids0, read_bytes=nbytes, write_bytes=nbytes))
    del student, teacher
    finish(result, args, torch, w, "distill", cpu_rows=512, gpu_rows=2048)


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

    elapsed, km = timed(torch, ops, args, step)
    live_rows = int((lengths - 1).clamp(min=0).sum().item())   # rows 0 .. length-2 of a sequence are read
    result = {
        "metric": "forward-only token logprobs (post-processor) tokens/s at V=151936; % of HBM peak",
        "value": b * s * args.steps / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w["desc"], "sequences": b, "seq_len": s, "vocab": v, "rows_read": live_rows},
        "roofline": hbm_roofline("logprob_post_fwd_kernel", live_rows * v * 2, km["logprob_post_fwd"]["avg_ms"]),
        "kernel_ms": {k: round(x["avg_ms"], 4) for k, x in km.items()},
    }
    if not args.no_cpu_baseline:
        result.update(read_write_ceiling(torch, logits, ids, read_bytes=result["roofline"]["algorithmic_bytes_per_launch"],
                                         write_bytes=0))
    del logits
    finish(result, args, torch, w, "post", cpu_rows=4096, gpu_rows=4096)


def bench_packed(args, torch, w):
    """One packed row through SequencePackingFusionLossWrapper (single pass), then the three-pass packed path."""
    from functools import partial

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
    # prepare_fn bound as the Megatron worker binds it (models/megatron/train.py:529-533)
    prepare = partial(prepare_packed_loss_input, sampling_params=None, chunk_size=None)
    wrapped = SequencePackingFusionLossWrapper(fn, prepare, cu, cu, 0, None, None)

    def step():
        x = logits.requires_grad_(True)
        loss, metrics = wrapped(x, data, gs, gt)      # the Megatron worker's wrapper: its metrics are read after the schedule
        (d,) = torch.autograd.grad(loss, x)
        del d, loss
        megatron_metrics([metrics])

    def three_pass_step():
        x = logits.requires_grad_(True)
        loss_input, prepared = prepare_packed_loss_input(x, data, fn, cu, cu)
        loss, metrics = fn(data=prepared, global_valid_seqs=gs, global_valid_toks=gt, **loss_input)
        (d,) = torch.autograd.grad(loss, x)
        del d, loss, loss_input
        megatron_metrics([metrics])

    elapsed, km = timed(torch, ops, args, step)
    row_bytes = v * 2
    # a live row is read once and its gradient written once; a row that feeds no token is only zero-filled
    alg = live_rows * 2 * row_bytes + (total - live_rows) * row_bytes
    out = {
        "metric": "GRPO logprob+loss fwd/bwd tokens/s, packed 131072-token row at V=131072; % of HBM peak",
        "value": total * args.steps / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w["desc"], "sequences": nseq, "packed_tokens": total, "vocab": v, "loss_tokens": live_rows,
                   "api": "SequencePackingFusionLossWrapper(ClippedPGLossFn, partial(prepare_packed_loss_input, ...))(logits, batch, "
                          "...) + autograd.grad -> nrl_fused_packed_logits_grpo_loss"},
        "hbm_frac_end_to_end": alg * args.steps / elapsed / 1e9 / HBM_PEAK_GBS,
        "roofline": hbm_roofline("fused_logits_loss_kernel (packed)", alg, km["fused_packed_logits_loss"]["avg_ms"], "c5"),
        "kernel_ms": {k: round(x["avg_ms"], 4) for k, x in km.items()},
    }
    t_elapsed, tk = timed(torch, ops, args, three_pass_step)
    out["three_pass"] = {
        "value": total * args.steps / t_elapsed, "unit": "tokens/s", "ms_per_step": t_elapsed / args.steps * 1e3,
        "api": "prepare_packed_loss_input -> nrl_logprob_packed_fwd; ClippedPGLossFn -> nrl_grpo_loss_fwd_bwd; "
               "backward -> nrl_logprob_packed_bwd",
        "kernel_ms": {k: round(x["avg_ms"], 4) for k, x in tk.items()},
    }
    if not args.no_cpu_baseline:
        out.update(read_write_ceiling(torch, logits.detach(), torch.zeros((1, total), dtype=torch.int64, device=dev),
                                      read_bytes=live_rows * row_bytes, write_bytes=total * row_bytes))
    del logits
    finish(out, args, torch, w, "packed", cpu_rows=2048, gpu_rows=4096)


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
        loss, metrics = fn(next_token_logprobs=lp, data=data, global_valid_seqs=gs, global_valid_toks=gt)
        dh, dw = torch.autograd.grad(loss, (hidden, weight))
        del dh, dw
        megatron_metrics([metrics])                # the fused lm_head is the Megatron worker's path

    from rl_amd.distributed import model_utils as MU

    # The forward keeps its bf16 logits when they fit ("auto": a quarter of the free memory; 19.9 GB at this shape)
    # and the backward reads them instead of multiplying a second time.  The reference's way, recomputing, is its
    # own row below.
    n = b * s
    kept = MU._keep_lmhead_logits(n, v, dev, h)
    elapsed, k = timed(torch, ops, args, step)
    fwd_ms, bwd_ms = k["lmhead_fwd"]["avg_ms"], k["lmhead_bwd"]["avg_ms"]
    MU.LMHEAD_KEEP_LOGITS = not kept
    elapsed_other, k_other = timed(torch, ops, args, step)
    MU.LMHEAD_KEEP_LOGITS = "auto"
    fwd_tf = 2.0 * n * h * v / (fwd_ms * 1e-3) / 1e12
    # the backward products run on the tokens that carry a gradient only (masked prompt tokens and each
    # sequence's last position have a zero row in the logits' gradient)
    live = float(gt.item()) / n
    products = 2.0 if kept else 3.0                                       # dH, dW (+ the recomputed logits)
    bwd_alg_tf = 4.0 * n * h * v / (bwd_ms * 1e-3) / 1e12                 # dH + dW of every token, the algorithmic count
    bwd_exec_tf = 2.0 * products * live * n * h * v / (bwd_ms * 1e-3) / 1e12   # what the matrix cores execute, live tokens
    fills = MEASURED_TRAFFIC.get("c3_fwd_kept" if kept else "c3_fwd") if not args.seqs else None
    result = {
        "metric": "fused lm_head + GRPO loss fwd/bwd tokens/s; % of bf16 MFMA peak",
        "value": n * args.steps / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w["desc"], "tokens": n, "hidden": h, "vocab": v,
                   "logits": ("bf16 logits kept by the forward for the backward (%.1f GB)" % (n * v * 2 / 1e9)) if kept
                             else "recomputed in the backward"},
        "roofline": {"bound": "mfma", "kernel": "lmhead_fwd_kernel", "achieved": fwd_tf, "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": fwd_tf / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": (fills["read"] + fills["write"]) if fills else None,
                     "traffic_profile": fills["profile"] if fills else None, "avg_launch_ms": fwd_ms},
        "roofline_bwd": {"bound": "mfma", "kernel": "lmhead backward (grad + dH + dW GEMMs)", "achieved": bwd_alg_tf,
                         "executed": bwd_exec_tf, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": bwd_alg_tf / MFMA_BF16_PEAK_TFLOPS, "frac_executed": bwd_exec_tf / MFMA_BF16_PEAK_TFLOPS,
                         "live_token_fraction": live, "avg_launch_ms": bwd_ms,
                         "note": "achieved counts dH + dW of all tokens (4 N H V); executed counts the products the matrix "
                                 "cores run (dH, dW and, when the logits are not kept, their recomputation), on the tokens "
                                 "with a non-zero gradient only"},
        ("recompute" if kept else "kept_logits"): {
            "tokens_per_s": n * args.steps / elapsed_other, "ms_per_step": elapsed_other / args.steps * 1e3,
            "kernel_ms": {kk: round(vv["avg_ms"], 4) for kk, vv in k_other.items()},
            "note": "the same step with LMHEAD_KEEP_LOGITS = %s" % (not kept)},
        "algorithmic_tflops_end_to_end": 6.0 * n * h * v * args.steps / elapsed / 1e12,
        "kernel_ms": {kk: round(vv["avg_ms"], 4) for kk, vv in k.items()},
    }
    del hidden, weight
    finish(result, args, torch, w, "lmhead", cpu_rows=1024, gpu_rows=1024)


# The one JSON line goes to the process's stdout; whatever the measured code prints on the way (the reference's
# warning about -inf logprobs under top-k / top-p, for one) goes to stderr.
_JSON_OUT = sys.stdout


def main():
    with contextlib.redirect_stdout(sys.stderr):
        try:
            return _main()
        finally:
            # warnings whose counts were still on their way are printed here, not after the JSON line at exit
            utils = sys.modules.get("rl_amd.algorithms.utils")
            if utils is not None:
                utils.flush_neg_inf_warnings()


def _main():
    args = parse_args()
    if args.source_fingerprints:
        import glob

        for path in sorted(glob.glob(os.path.join(ROOT, "rl_amd", "csrc", "*.hip"))):
            print("%s@%s" % (os.path.basename(path), source_fingerprint(os.path.basename(path))), file=_JSON_OUT)
        return
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
    # No switch of this package is set: the step is the worker's loop -- loss, the per-metric division by the number
    # of global batches, backward, per microbatch -- followed by one read of every microbatch's metrics.
    tot_seqs = torch.tensor(float(w["seqs"]), device=dev)
    tot_toks = sum((m["data"]["token_mask"][:, 1:].sum() for m in mbs)) * (n_mb / n_buf)
    tot_toks = tot_toks.float()

    from functools import partial

    from rl_amd.algorithms.advantage_estimator import AdvEstimatorConfig, GRPOAdvantageEstimator
    from rl_amd.algorithms.loss import fused_logits_clipped_pg_loss, wrap_loss_fn_with_input_preparation

    # prepare_fn bound as the Megatron worker binds it (models/megatron/train.py:506-513)
    prepare = partial(prepare_loss_input, sampling_params=None, d2t=None, chunk_size=None)
    grouped = None
    if w.get("group"):  # config 1: advantages come from Bernoulli(0.5) rewards through the per-prompt group baseline
        g = torch.Generator(device=dev).manual_seed(1001)
        n_prompts = w["seqs"] // w["group"]
        grouped = dict(
            prompts=torch.arange(n_prompts, device=dev).repeat_interleave(w["group"]).unsqueeze(-1).expand(-1, 8).contiguous(),
            rewards=(torch.rand((w["seqs"],), generator=g, device=dev) < 0.5).float(),
            estimator=GRPOAdvantageEstimator(AdvEstimatorConfig(), None))

    AT, worker_call = dtensor_worker(torch)
    post = AT.LossPostProcessor(fn, {}, None, None, None, 1, 1)

    def step():
        # the DTensor worker's sequence: its forward function hands the logits to the LossPostProcessor, which calls
        # wrap_loss_fn_with_input_preparation(..., partial(prepare_loss_input, sampling_params=...)); that dispatches to
        # the single-pass kernel when the loss configuration allows it (this one does), and autograd hands back
        # d loss / d logits
        collected = []
        for i in range(n_mb):
            m = mbs[i % n_buf]
            if grouped is not None:
                m["data"]["advantages"] = grouped["estimator"].compute_advantage(grouped["prompts"], grouped["rewards"],
                                                                                 m["data"]["token_mask"])
            logits = m["logits"].requires_grad_(True)
            loss, metrics = worker_call(post, logits, m["data"], tot_seqs, tot_toks)
            collected.append(worker_scaling(metrics))
            (dlogits,) = torch.autograd.grad(loss, logits)
            del dlogits, loss
        read_metrics(collected)

    def three_pass_step():
        # the reference's call structure spelled out: logprobs (pass 1), loss on logprobs, backward (passes 2+3)
        collected = []
        for i in range(n_mb):
            m = mbs[i % n_buf]
            logits = m["logits"].requires_grad_(True)
            loss_input, data = prepare_loss_input(logits, m["data"], fn)
            loss, metrics = fn(data=data, global_valid_seqs=tot_seqs, global_valid_toks=tot_toks, **loss_input)
            collected.append(metrics)
            (dlogits,) = torch.autograd.grad(loss, logits)
            del dlogits, loss, loss_input
        megatron_metrics(collected)

    def in_place_step():
        # the gradient written over the logits (the logits are dead after the loss in a training step): no second
        # [B, S, V] buffer, and the read and the write of a row hit the same DRAM pages
        collected = []
        for i in range(n_mb):
            m = mbs[i % n_buf]
            logits = m["logits"].requires_grad_(True)
            loss, metrics = fused_logits_clipped_pg_loss(logits, m["data"], fn, tot_seqs, tot_toks, in_place=True)
            collected.append(metrics)
            (dlogits,) = torch.autograd.grad(loss, logits)
            del dlogits, loss
        megatron_metrics(collected)

    elapsed, kernels = timed(torch, ops, args, step)
    tokens_per_step = w["seqs"] * w["seq_len"]
    rows_per_launch = w["mb_seqs"] * w["seq_len"]
    row_bytes = w["vocab"] * elt
    nan = dict(avg_ms=float("nan"))
    fk = kernels.get("fused_logits_loss", nan)
    alg_launch = 2 * row_bytes * rows_per_launch  # every logit read once, every gradient element written once
    full = not args.seqs
    result = {
        "metric": "GRPO logprob+loss fwd/bwd tokens/s at V=%d; %% of HBM peak" % w["vocab"],
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
                   "metrics": "all diagnostics computed per microbatch; after every loss call the worker's metrics[k] /= "
                              "num_global_batches, after the last microbatch every value of every record is read (inside the "
                              "timed step); no rl_amd-specific switch is set",
                   "api": "forward_with_post_processing_fn(model, LossPostProcessor(ClippedPGLossFn), microbatch, ...) of the DTensor "
                          "worker -> wrap_loss_fn_with_input_preparation(logits, batch, ..., prepare_fn=partial(prepare_loss_input, "
                          "sampling_params=)) + autograd.grad -> nrl_fused_logits_grpo_loss (seq stats + single pass + term "
                          "reduce + finish)"},
        "algorithmic_bytes_per_token": 2 * row_bytes,
        "hbm_frac_end_to_end": 2 * row_bytes * tokens_per_step * args.steps / elapsed / 1e9 / HBM_PEAK_GBS,
        "roofline": hbm_roofline("fused_logits_loss_kernel", alg_launch, fk["avg_ms"], args.workload if full else None),
        "kernel_ms": {k: round(v["avg_ms"], 4) for k, v in kernels.items()},
    }
    # ---- the same step with a plain dictionary filled before every loss call returns ----
    fn.lazy_metrics = False
    e_elapsed, e_kernels = timed(torch, ops, args, step)
    fn.lazy_metrics = True
    result["eager_metrics"] = {
        "value": tokens_per_step * args.steps / e_elapsed, "unit": "tokens/s", "ms_per_step": e_elapsed / args.steps * 1e3,
        "hbm_frac_end_to_end": 2 * row_bytes * tokens_per_step * args.steps / e_elapsed / 1e9 / HBM_PEAK_GBS,
        "note": "ClippedPGLossFn.lazy_metrics = False: a plain dict filled before the call returns (one device -> host wait "
                "per microbatch)",
    }
    # ---- the three-pass path (its own row: 3 * V * sizeof per token) ----
    t_elapsed, t_kernels = timed(torch, ops, args, three_pass_step)
    bwd = t_kernels.get("logprob_bwd", nan)
    fwd = t_kernels.get("logprob_fwd", nan)
    result["three_pass"] = {
        "value": tokens_per_step * args.steps / t_elapsed, "unit": "tokens/s", "ms_per_step": t_elapsed / args.steps * 1e3,
        "api": "prepare_loss_input -> nrl_logprob_fwd; ClippedPGLossFn -> nrl_grpo_loss_fwd_bwd; backward -> nrl_logprob_bwd",
        "algorithmic_bytes_per_token": 3 * row_bytes,
        "hbm_frac_end_to_end": 3 * row_bytes * tokens_per_step * args.steps / t_elapsed / 1e9 / HBM_PEAK_GBS,
        "roofline_bwd": hbm_roofline("logprob_bwd_kernel", 2 * row_bytes * rows_per_launch, bwd["avg_ms"],
                                     args.workload + "_three_pass_bwd" if full else None),
        "roofline_fwd": hbm_roofline("logprob_fwd_kernel", row_bytes * w["mb_seqs"] * (w["seq_len"] - 1), fwd["avg_ms"],
                                     args.workload + "_three_pass_fwd" if full else None),
        "kernel_ms": {k: round(v["avg_ms"], 4) for k, v in t_kernels.items()},
    }
    # ---- the single pass writing the gradient over the logits (last: it consumes the logits) ----
    i_elapsed, i_kernels = timed(torch, ops, args, in_place_step)
    ik = i_kernels.get("fused_logits_loss", nan)
    result["in_place"] = {
        "value": tokens_per_step * args.steps / i_elapsed, "unit": "tokens/s", "ms_per_step": i_elapsed / args.steps * 1e3,
        "api": "fused_logits_clipped_pg_loss(..., in_place=True): dlogits aliases the logits",
        "hbm_frac_end_to_end": 2 * row_bytes * tokens_per_step * args.steps / i_elapsed / 1e9 / HBM_PEAK_GBS,
        "roofline": hbm_roofline("fused_logits_loss_kernel (dlogits over logits)", alg_launch, ik["avg_ms"]),
    }
    if not args.no_cpu_baseline:
        live = float(mbs[0]["data"]["token_mask"][:, 1:].sum().item())
        result.update(read_write_ceiling(torch, mbs[0]["logits"].detach(), mbs[0]["data"]["input_ids"],
                                         read_bytes=live * row_bytes, write_bytes=rows_per_launch * row_bytes))
    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.float32, device=dev).fill_(1.0)  # 4 GiB
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        result["copy_calibration_bytes"] = src.numel() * 4
        del src, dst
    del mbs
    small = w["vocab"] < 100000
    finish(result, args, torch, w, "loss", cpu_rows=(w["seqs"] * w["seq_len"] if small else 4096),
           gpu_rows=(w["seqs"] * w["seq_len"] if small else 4096))


if __name__ == "__main__":
    main()
