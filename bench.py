#!/usr/bin/env python3
"""Benchmark of the ring-attention hot path on one MI355X.

One "step" is one forward + backward pass of the whole emulated ring over one batch of
synthetic q/k/v/dO already resident in HBM.  Prints ONE JSON line (rank 0 = the only rank).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3b|C3a|C2|C5|C4]

`value` is algorithmic TFLOP/s of fwd+bwd: 14 * D * P * B * H / time, where P is the number of
unmasked (query, key) pairs per (batch, head).  Recompute GEMMs of the split dQ kernel, the
softmax, delta and casts are not counted.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ring-attention-jax-pallas_amd"))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X published dense bf16 MFMA peak

# HBM bytes per launch (read + written) of the step kernels, measured with
# `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of this script (`--copy-probe` gives the
# 1 GiB copy the counters are scaled by: FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).  Profiler counters
# cannot be read from inside a timed run, so the figures are carried here.
MEASURED_HBM_BYTES_PER_LAUNCH = {
    "C3b": {"fwd_step_kernel": 1.492e9, "dkdv_kernel": 2.412e9, "dq_kernel": 1.429e9},
}

WORKLOADS = {
    # name: (B, H, D, S, ring, bias, std, description)
    "C3b": dict(B=1, H=32, D=128, S=131072, n=8, bias="causal", std=1.0,
                desc="S=131072 as 8 shards x 16384, H=32, D=128, causal, whole ring on one GPU"),
    "C3a": dict(B=1, H=32, D=128, S=131072, n=8, bias="causal", std=1.0, only_rank=7,
                desc="rank 7's share of C3b: Lq=16384 over 8 KV shards of 16384, causal"),
    "C2": dict(B=2, H=16, D=128, S=8192, n=8, bias="causal", std=1.0,
               desc="B=2, H=16, D=128, S=8192 as 8 shards x 1024, causal"),
    "C5": dict(B=1, H=8, D=128, S=65536, n=8, bias="window", window=4096, std=0.5,
               desc="B=1, H=8, D=128, S=65536 as 8 shards x 8192, causal window 4096"),
    "C4": dict(B=1, H=16, D=128, S=32768, n=4, bias="segment+alibi", std=1.0, mean_seg=2048,
               desc="B=1, H=16, D=128, S=32768 as 4 shards x 8192, geometric segments (mean 2048) + ALiBi"),
}


def pair_count(kind, window, q_off, kv_off, Lq, Lk):
    """Unmasked (query, key) pairs of one shard pair under a positional mask (closed form per row)."""
    import numpy as np
    i = np.arange(Lq, dtype=np.int64) + q_off
    hi = np.full(Lq, kv_off + Lk - 1, dtype=np.int64)
    lo = np.full(Lq, kv_off, dtype=np.int64)
    if kind in ("causal", "window"):
        hi = np.minimum(hi, i)
    if kind == "window":
        lo = np.maximum(lo, i - window + 1)
    return int(np.maximum(hi - lo + 1, 0).sum())


class EventTimer:
    """Brackets each kernel launch with events on the stream the kernels are enqueued on."""
    split_bwd = True

    def __init__(self, torch):
        self.torch = torch
        self.records = []

    class _Span:
        def __init__(self, owner, key):
            self.owner, self.key = owner, key

        def __enter__(self):
            t = self.owner.torch
            self.a = t.cuda.Event(enable_timing=True)
            self.b = t.cuda.Event(enable_timing=True)
            self.a.record(t.cuda.current_stream())
            return self

        def __exit__(self, *exc):
            self.b.record(self.owner.torch.cuda.current_stream())
            self.owner.records.append((self.key, self.a, self.b))
            return False

    def span(self, kind, qs, ks):
        return self._Span(self, (kind, qs, ks))

    def results(self):
        self.torch.cuda.synchronize()
        return [(key, a.elapsed_time(b)) for key, a, b in self.records]


def mfma_ceiling(torch, dev):
    """bf16 MFMA rate of a loop of nothing but v_mfma_f32_32x32x16_bf16 with operands that toggle
    like real data, one wave per SIMD on every compute unit, ~15 ms per launch: what the board's
    power management leaves of the published peak.  Reported next to `roofline`, never used in it."""
    import ctypes as C
    from ring_attention import _lib
    lib = _lib.load()
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    iters = 100000
    sink = torch.empty(cus * 256, device=dev, dtype=torch.float32)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    best = 0.0
    for rep in range(4):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(torch.cuda.current_stream())
        _lib.check("ra_probe_mfma_rate", lib.ra_probe_mfma_rate(sink.data_ptr(), cus, iters, 1, stream))
        b.record(torch.cuda.current_stream())
        torch.cuda.synchronize()
        if rep:  # the first launch runs while the clock is still ramping
            best = max(best, cus * 4 * iters * 8 * 32768.0 / (a.elapsed_time(b) * 1e-3) / 1e12)
    return {"value": round(best, 1), "unit": "TFLOP/s", "frac_of_published_peak": round(best / PEAK_BF16_TFLOPS, 4),
            "what": "v_mfma_f32_32x32x16_bf16 only, random operands in registers, one wave per SIMD, all CUs"}


def cpu_baseline(D):
    """The numpy restatement of the reference algorithm, timed on the host cores on a bounded
    sample of the workload (same head dim, causal, fp32): H=8, S=16384 as 4 shards of 4096."""
    import numpy as np
    from oracle import ring_oracle as R
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = os.cpu_count() or 1
    H, S, n = 8, 16384, 4
    q, k, v, do = R.make_inputs(0, 1, S, S, H, D)
    pos = np.broadcast_to(np.arange(S), (1, S))
    fn = R.make_bias_fn(causal=True)
    t0 = time.perf_counter()
    out, lse = R.ring_attention(q, k, v, n, fn, {"q_positions": pos}, {"kv_positions": pos},
                                dtype=np.float32, skip_masked_steps=True)
    R.ring_attention_bwd(q, k, v, out, lse, do, n, fn, {"q_positions": pos}, {"kv_positions": pos},
                         dtype=np.float32)
    dt = time.perf_counter() - t0
    flops = 14.0 * D * (S * (S + 1) / 2) * H
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": int(threads), "kind": "port",
            "sample": f"numpy fp32 restatement of ring_attention fwd+bwd, B=1 H={H} D={D} S={S} as {n} "
                      f"shards, causal, {dt:.1f} s wall",
            "seconds": dt}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default="C3b", choices=sorted(WORKLOADS))
    ap.add_argument("--impl", default="hip", choices=["hip", "hip_fused"],
                    help="hip: one launch per ring step (the headline); hip_fused: one launch per ring pass, "
                         "the kernels walk the shards themselves (no per-kernel roofline in that mode)")
    ap.add_argument("--graph", action="store_true",
                    help="capture one fwd+bwd pass of the ring in a HIP graph and time its replays (pays where "
                         "launches are short: C2); no per-kernel roofline in that mode")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-timing", action="store_true")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain elementwise copy of 1 GiB (calibrates HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE GPU: the ring is emulated on a single MI355X and there is no "
              "multi-GPU path in this build (got --gpus %d)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import ring_attention as ra
    from ring_attention import ring as rr

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    w = WORKLOADS[args.workload]
    B, H, D, S, n = w["B"], w["H"], w["D"], w["S"], w["n"]
    L = S // n
    gen = torch.Generator(device=dev)
    gen.manual_seed(0)
    mk = lambda: (torch.randn((B, S, H, D), generator=gen, device=dev, dtype=torch.float32) * w["std"]).to(torch.bfloat16)
    q, k, v = mk(), mk(), mk()
    do = torch.randn((B, S, H, D), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    sm_scale = 1.0 / math.sqrt(D)

    q_kw = kv_kw = None
    seg_np = None
    if w["bias"] == "causal":
        fn = ra.causal_bias()
    elif w["bias"] == "window":
        fn = ra.sliding_window_bias(w["window"])
    else:
        rng = np.random.default_rng(0)
        seg_np = np.zeros((B, S), dtype=np.int32)
        for b in range(B):
            pos, sid = 0, 0
            while pos < S:
                ln = int(rng.geometric(1.0 / w["mean_seg"]))
                seg_np[b, pos:pos + ln] = sid
                pos += ln
                sid += 1
        seg = torch.from_numpy(seg_np).to(dev)
        fn = ra.segment_bias() + ra.alibi_bias(ra.alibi_slopes(H))
        q_kw, kv_kw = {"q_segment_ids": seg}, {"kv_segment_ids": seg}
    plan = rr._RingPlan(q, k, n, fn, q_kw, kv_kw)

    # unmasked pairs per (q shard, kv shard), per (batch, head) on average
    pairs = {}
    for qs in range(n):
        for ks in range(n):
            if seg_np is not None:
                tot = 0
                for b in range(B):
                    cq = np.bincount(seg_np[b, qs * L:(qs + 1) * L])
                    ck = np.bincount(seg_np[b, ks * L:(ks + 1) * L])
                    m_ = min(len(cq), len(ck))
                    tot += int((cq[:m_].astype(np.int64) * ck[:m_]).sum())
                pairs[(qs, ks)] = tot / B
            else:
                pairs[(qs, ks)] = pair_count(w["bias"], w.get("window", 0), qs * L, ks * L, L, L)
    only_rank = w.get("only_rank")
    if only_rank is not None:
        # one device's real share: its query shard against all KV shards (forward), and the
        # same (q, kv) pairs in the backward pass
        raise SystemExit("C3a is measured through C3b's per-launch records; run --workload C3b")
    P = sum(pairs.values())
    flops_fwd = 4.0 * D * P * B * H
    flops_bwd = 10.0 * D * P * B * H

    ev = lambda: torch.cuda.Event(enable_timing=True)

    fused = args.impl == "hip_fused"
    ring_fwd = rr._ring_forward_fused if fused else rr._ring_forward
    ring_bwd = rr._ring_backward_fused if fused else rr._ring_backward
    if fused:
        args.no_kernel_timing = True

    def one_step(marks=None):
        if marks is not None:
            marks[0].record()
        out, lse = ring_fwd(q, k, v, plan, sm_scale, torch.bfloat16)
        if marks is not None:
            marks[1].record()
        grads = ring_bwd(q, k, v, out, lse, do, plan, sm_scale)
        if marks is not None:
            marks[2].record()
        return out, grads

    for _ in range(args.warmup):
        one_step()
    torch.cuda.synchronize()
    if args.graph:
        args.no_kernel_timing = True
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            one_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            held = one_step()
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ms_per_step = dt * 1e3 / args.steps
        # the split is that of one eager pass (events cannot sit inside a replayed graph)
        m = [ev(), ev(), ev()]
        one_step(m)
        torch.cuda.synchronize()
        share = m[0].elapsed_time(m[1]) / m[0].elapsed_time(m[2])
        fwd_ms, bwd_ms = ms_per_step * share, ms_per_step * (1.0 - share)
    else:
        marks = [[ev(), ev(), ev()] for _ in range(args.steps)]
        t0 = time.perf_counter()
        for i in range(args.steps):
            one_step(marks[i])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ms_per_step = dt * 1e3 / args.steps
        fwd_ms = sum(m[0].elapsed_time(m[1]) for m in marks) / args.steps
        bwd_ms = sum(m[1].elapsed_time(m[2]) for m in marks) / args.steps
    value = (flops_fwd + flops_bwd) / (ms_per_step * 1e-3) / 1e12

    result = {
        "metric": "fwd+bwd attention TFLOP/s and % of bf16 MFMA peak, 1 MI355X",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {w['desc']}", "B": B, "H": H, "D": D, "S": S,
                   "ring_size": n, "bias": w["bias"], "unmasked_pairs_per_head": P,
                   "launches": ("one per ring pass" if fused else "one per ring step") +
                               (", replayed from a captured HIP graph" if args.graph else "")},
        "pct_of_bf16_peak": round(100.0 * value / PEAK_BF16_TFLOPS, 2),
        "fwd": {"ms": round(fwd_ms, 3), "tflops": round(flops_fwd / fwd_ms / 1e9, 2),
                "pct_of_bf16_peak": round(100.0 * flops_fwd / fwd_ms / 1e9 / PEAK_BF16_TFLOPS, 2)},
        "bwd": {"ms": round(bwd_ms, 3), "tflops": round(flops_bwd / bwd_ms / 1e9, 2),
                "pct_of_bf16_peak": round(100.0 * flops_bwd / bwd_ms / 1e9 / PEAK_BF16_TFLOPS, 2)},
    }

    # per-kernel timing: one more pass with every launch bracketed by events on the launch stream
    if not args.no_kernel_timing:
        timer = EventTimer(torch)
        out, lse = rr._ring_forward(q, k, v, plan, sm_scale, torch.bfloat16, timer=timer)
        rr._ring_backward(q, k, v, out, lse, do, plan, sm_scale, timer=timer)
        recs = timer.results()
        # algorithmic flops of each kernel per unmasked pair: forward QK^T + PV = 4D; the dK/dV
        # kernel S, dP, dV, dK = 8D; the dQ kernel's own product = 2D (its S/dP recompute is
        # overhead and not counted)
        per_pair = {"fwd": 4.0 * D, "bwd_dkdv": 8.0 * D, "bwd_dq": 2.0 * D}
        names = {"fwd": "fwd_step_kernel", "bwd_dkdv": "dkdv_kernel", "bwd_dq": "dq_kernel"}
        kern = {}
        for (kind, qs, ks), ms in recs:
            if pairs[(qs, ks)] == 0:
                continue
            d = kern.setdefault(kind, {"ms": 0.0, "flops": 0.0, "launches": 0})
            d["ms"] += ms
            d["flops"] += per_pair[kind] * pairs[(qs, ks)] * B * H
            d["launches"] += 1
        kernels = {}
        for kind, d in kern.items():
            kernels[names[kind]] = {
                "launches": d["launches"], "avg_ms": round(d["ms"] / d["launches"], 4),
                "algorithmic_tflop_per_launch": round(d["flops"] / d["launches"] / 1e12, 4),
                "achieved_tflops": round(d["flops"] / d["ms"] / 1e9, 2)}
        dom = max(kern, key=lambda kk: kern[kk]["ms"])
        ach = kern[dom]["flops"] / kern[dom]["ms"] / 1e9
        result["roofline"] = {"bound": "mfma", "kernel": names[dom], "achieved": round(ach, 2),
                              "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                              "frac": round(ach / PEAK_BF16_TFLOPS, 4),
                              "traffic": MEASURED_HBM_BYTES_PER_LAUNCH.get(args.workload, {}).get(names[dom])}
        result["kernels"] = kernels
        # rank 7's share (the last query shard against all 8 KV shards)
        if args.workload == "C3b":
            r7 = [(key, ms) for key, ms in recs if key[1] == n - 1]
            f_ms = sum(ms for key, ms in r7 if key[0] == "fwd")
            b_ms = sum(ms for key, ms in r7 if key[0] != "fwd")
            P7 = sum(pairs[(n - 1, ks)] for ks in range(n))
            result["rank7_share"] = {"fwd_tflops": round(4.0 * D * P7 * B * H / f_ms / 1e9, 2),
                                     "bwd_tflops": round(10.0 * D * P7 * B * H / b_ms / 1e9, 2)}

    if not args.no_kernel_timing:
        result["mfma_ceiling"] = mfma_ceiling(torch, dev)

    if args.copy_probe:
        # a kernel of known traffic (reads 1 GiB, writes 1 GiB) for scaling profiler byte counters
        src = torch.ones(1 << 28, device=dev, dtype=torch.float32)
        for _ in range(3):
            dst = src * 1.0
        torch.cuda.synchronize()
        del src, dst

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(D)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
