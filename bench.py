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

CSRC = os.path.join(ROOT, "ring-attention-jax-pallas_amd", "csrc")


def csrc_digest():
    """Digest of the kernel sources: a stored profiler figure is only quoted while it matches."""
    import hashlib
    h = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".h")):
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def stored_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 counter summary of this
    workload (profiles/<workload>_hbm_traffic.txt, written by --pmc-summary).  Profiler counters
    cannot be read from inside a timed run; the summary carries the digest of the kernel sources
    it was measured on, and a figure measured on other sources is not quoted (None)."""
    path = os.path.join(ROOT, "profiles", f"{workload.lower()}_hbm_traffic.txt")
    if not os.path.exists(path):
        return None
    digest, table = None, {}
    with open(path) as f:
        for line in f:
            t = line.split()
            if line.startswith("csrc-digest:"):
                digest = t[1]
            elif len(t) == 3 and t[0] == "bytes-per-launch":
                table[t[1]] = float(t[2])
    if digest != csrc_digest():
        return None
    return table.get(kernel)


def pmc_summary(workload, fetch_csv, write_csv):
    """Text summary of two rocprofv3 --pmc runs of `bench.py --copy-probe` (FETCH_SIZE, WRITE_SIZE).
    Both counters are scaled by what they read for the 1 GiB elementwise copy of --copy-probe."""
    import csv
    from collections import defaultdict

    def read(path, counter):
        tot, cnt = defaultdict(float), defaultdict(int)
        with open(path) as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] != counter:
                    continue
                tot[row["Kernel_Name"]] += float(row["Counter_Value"])
                cnt[row["Kernel_Name"]] += 1
        return {k: (tot[k] / cnt[k], cnt[k]) for k in tot}

    fetch, write = read(fetch_csv, "FETCH_SIZE"), read(write_csv, "WRITE_SIZE")
    # the copy probe: the kernel outside this library whose writes are closest to 1 GiB per launch
    gib_kib = float(1 << 20)
    probe = [k for k in fetch if "ra::" not in k and k in write]
    pk = min(probe, key=lambda k: abs(write[k][0] - gib_kib), default=None)
    if pk is None or abs(write[pk][0] - gib_kib) > 0.2 * gib_kib:
        raise SystemExit("no copy-probe kernel in the counter files: run bench.py with --copy-probe")
    f_scale = gib_kib / fetch[pk][0]
    w_scale = gib_kib / write[pk][0]
    out = [f"rocprofv3 HBM byte counters, workload {workload}: one fwd+bwd pass of the ring",
           "commands (from /tmp, TMPDIR=/tmp, R = repository root, OUT = an output directory), one counter per run:",
           f"  rocprofv3 --pmc FETCH_SIZE --output-format csv -d $OUT/pmc_fetch -o f -- python3 $R/bench.py --workload {workload} --steps 1 --warmup 0 --no-cpu-baseline --no-kernel-timing --copy-probe",
           f"  rocprofv3 --pmc WRITE_SIZE --output-format csv -d $OUT/pmc_write -o w -- python3 $R/bench.py --workload {workload} --steps 1 --warmup 0 --no-cpu-baseline --no-kernel-timing --copy-probe",
           f"  python3 $R/bench.py --workload {workload} --pmc-summary <f_counter_collection.csv> <w_counter_collection.csv>",
           f"calibration kernel (reads 1 GiB, writes 1 GiB): {pk[:60]}",
           f"  FETCH_SIZE reads {fetch[pk][0]:.0f} KiB -> scale {f_scale:.3f};  WRITE_SIZE reads {write[pk][0]:.0f} KiB -> scale {w_scale:.3f}",
           f"csrc-digest: {csrc_digest()}",
           "", f"{'kernel':<44}{'n':>5}{'FETCH KiB':>14}{'WRITE KiB':>14}{'read GB':>10}{'written GB':>12}"]
    rows = []
    for k in sorted(fetch):
        if not k.startswith("ra::") and "ra::" not in k:
            continue
        fa, n = fetch[k]
        wa = write.get(k, (0.0, 0))[0]
        rd, wr = fa * f_scale * 1024.0, wa * w_scale * 1024.0
        short = k.split("(")[0].replace("void ", "")
        out.append(f"{short:<44}{n:>5}{fa:>14.0f}{wa:>14.0f}{rd / 1e9:>10.3f}{wr / 1e9:>12.3f}")
        rows.append((short, rd + wr))
    out.append("")
    out.append("HBM bytes per launch (read + written, scaled); bench.py quotes these as roofline.traffic:")
    for short, tot in rows:
        out.append(f"bytes-per-launch {short.replace('ra::', '').split('<')[0]} {tot:.4e}")
    return "\n".join(out) + "\n"


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
    # the reference's general bias_fn contract (ring.py:107,186): a Python callable that returns the
    # dense additive [b, 1, lq, lk] block of one (query shard, key/value shard) pair - here the
    # document mask of C4 - which the kernels stream from HBM (4 bytes per score and kernel)
    "CALLABLE": dict(B=1, H=16, D=128, S=32768, n=4, bias="callable", std=1.0, mean_seg=2048,
                     desc="B=1, H=16, D=128, S=32768 as 4 shards x 8192, a callable bias_fn returning the dense "
                          "[b, 1, lq, lk] document mask (geometric segments, mean 2048)"),
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
    path = os.path.join(os.path.dirname(_lib.LIB_PATH), "libringattn_probe.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build the kernels first (__graft_entry__.build())")
    lib = C.CDLL(path)
    lib.ra_probe_mfma_rate.restype = C.c_int
    lib.ra_probe_mfma_rate.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    iters = 100000
    sink = torch.empty(cus * 256, device=dev, dtype=torch.float32)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    best = 0.0
    for rep in range(4):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(torch.cuda.current_stream())
        rc = lib.ra_probe_mfma_rate(sink.data_ptr(), cus, iters, 1, stream)
        if rc:
            raise RuntimeError(f"ra_probe_mfma_rate failed with code {rc}")
        b.record(torch.cuda.current_stream())
        torch.cuda.synchronize()
        if rep:  # the first launch runs while the clock is still ramping
            best = max(best, cus * 4 * iters * 8 * 32768.0 / (a.elapsed_time(b) * 1e-3) / 1e12)
    return {"value": round(best, 1), "unit": "TFLOP/s", "frac_of_published_peak": round(best / PEAK_BF16_TFLOPS, 4),
            "what": "v_mfma_f32_32x32x16_bf16 only, random operands in registers, one wave per SIMD, all CUs"}


def coissue_probe(torch, dev):
    """Table of the co-issue probe of libringattn_probe.so: shader-clock cycles per v_mfma_f32_32x32x16_bf16 and
    SIMD when every MFMA of a loop is followed by a fixed group of other instructions, at one and at two waves
    per SIMD (32 = the matrix pipe is busy all the time).  One workgroup per compute unit; a workgroup's time is that
    of its slowest wave, the table holds the median over workgroups."""
    import ctypes as C
    from ring_attention import _lib
    path = os.path.join(os.path.dirname(_lib.LIB_PATH), "libringattn_probe.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build the kernels first (__graft_entry__.build())")
    lib = C.CDLL(path)
    lib.ra_probe_coissue_cases.restype = C.c_int
    lib.ra_probe_coissue_what.restype = C.c_char_p
    lib.ra_probe_coissue_what.argtypes = [C.c_int]
    lib.ra_probe_coissue.restype = C.c_int
    lib.ra_probe_coissue.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    iters = 20000
    cycles = torch.zeros(cus * 8, device=dev, dtype=torch.int64)
    src = torch.zeros(cus * 16384, device=dev, dtype=torch.uint8)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    lines = [f"cycles of the shader clock per v_mfma_f32_32x32x16_bf16 and SIMD; loop of 8 MFMAs x {iters} trips, "
             f"{cus} workgroups (slowest wave of each, median over workgroups)",
             f"{'behind every MFMA':<84}{'1 wave/SIMD':>12}{'2 waves/SIMD':>13}"]
    for c in range(lib.ra_probe_coissue_cases()):
        row = []
        for waves in (4, 8):
            for n in (200, iters):  # a short launch first: code and clocks warm
                rc = lib.ra_probe_coissue(cycles.data_ptr(), c, waves, cus, n, src.data_ptr(), stream)
                if rc:
                    raise RuntimeError(f"ra_probe_coissue failed with code {rc}")
                torch.cuda.synchronize()
            # the SIMD's older wave is served first and finishes early: a workgroup's time is its slowest wave's
            med = cycles[:cus * waves].view(cus, waves).max(dim=1).values.float().median().item()
            row.append(med / (iters * 8) / (waves // 4))
        lines.append(f"{lib.ra_probe_coissue_what(c).decode():<84}{row[0]:>12.1f}{row[1]:>13.1f}")
    return "\n".join(lines) + "\n"


def cpu_baseline(D, config="sample"):
    """The numpy restatement of the reference algorithm (fp32, causal) timed on the host cores:
    a bounded sample with the workload's head dim (H=8, S=16384 as 4 shards of 4096), or
    benchmark config C1 (forward only) or C2 (forward + backward) in full."""
    import numpy as np
    from oracle import ring_oracle as R
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = os.cpu_count() or 1
    B, H, S, n, bwd = {"sample": (1, 8, 16384, 4, True), "C1": (1, 4, 1024, 4, False),
                       "C2": (2, 16, 8192, 8, True)}[config]
    if config == "C1":
        D = 64
    elif config == "C2":
        D = 128
    q, k, v, do = R.make_inputs(0, B, S, S, H, D)
    pos = np.broadcast_to(np.arange(S), (B, S))
    fn = R.make_bias_fn(causal=True)
    reps = 20 if config == "C1" else 1  # C1 takes milliseconds
    t0 = time.perf_counter()
    for _ in range(reps):
        out, lse = R.ring_attention(q, k, v, n, fn, {"q_positions": pos}, {"kv_positions": pos},
                                    dtype=np.float32, skip_masked_steps=True)
        if bwd:
            R.ring_attention_bwd(q, k, v, out, lse, do, n, fn, {"q_positions": pos}, {"kv_positions": pos},
                                 dtype=np.float32)
    dt = (time.perf_counter() - t0) / reps
    flops = (14.0 if bwd else 4.0) * D * (S * (S + 1) / 2) * H * B
    what = "fwd+bwd" if bwd else "fwd"
    label = "a bounded sample" if config == "sample" else f"config {config} in full"
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": int(threads), "kind": "port",
            "sample": f"numpy fp32 restatement of ring_attention {what} on {label}: B={B} H={H} D={D} S={S} as "
                      f"{n} shards, causal, {dt:.3g} s wall",
            "seconds": dt}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default: 3 for the 0.5 s steps of C3b / C3a, 20 for the millisecond steps of "
                         "the small workloads, whose first launches would otherwise dominate the clock)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default: 1, small workloads 3)")
    ap.add_argument("--workload", default="C3b", choices=sorted(WORKLOADS))
    ap.add_argument("--impl", default="hip", choices=["hip", "hip_fused"],
                    help="hip: one launch per ring step (the headline: what a real ring does, where the next shard "
                         "is not there yet); hip_fused: the whole ring per launch, what ring_attention picks by "
                         "default on one GPU (no per-kernel roofline in that mode)")
    ap.add_argument("--graph", action="store_true",
                    help="capture one fwd+bwd pass of the ring in a HIP graph and time its replays (pays where "
                         "launches are short: C2); no per-kernel roofline in that mode")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-timing", action="store_true")
    ap.add_argument("--cpu-baseline-config", default="sample", choices=["sample", "C1", "C2"],
                    help="what the CPU restatement is timed on: a bounded sample with the workload's head dim "
                         "(default, ~20 s), or benchmark config C1 / C2 in full")
    ap.add_argument("--pmc-summary", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: turn the counter_collection.csv files of two rocprofv3 --pmc runs of this "
                         "script (FETCH_SIZE, WRITE_SIZE; both with --copy-probe) into the text summary kept "
                         "under profiles/ and print it")
    ap.add_argument("--no-dense-summary", action="store_true",
                    help="CALLABLE: hand the step kernels the dense blocks without their summaries (ra_dense_map), "
                         "so that they read every block in full: the streaming rate of the dense-bias kernels")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain elementwise copy of 1 GiB (calibrates HBM byte counters)")
    ap.add_argument("--coissue-probe", action="store_true",
                    help="no workload: print the table of what fits in the shadow of an MFMA (instruction groups "
                         "behind every MFMA of a loop, cycles per MFMA) and exit")
    args = ap.parse_args()
    if args.pmc_summary:
        sys.stdout.write(pmc_summary(args.workload, *args.pmc_summary))
        return
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
    if args.coissue_probe:
        sys.stdout.write(coissue_probe(torch, dev))
        return
    w = WORKLOADS[args.workload]
    small = args.workload in ("C2", "C4", "C5", "CALLABLE")
    if args.steps is None:
        args.steps = 20 if small else 3
    if args.warmup is None:
        args.warmup = 3 if small else 1
    B, H, D, S, n = w["B"], w["H"], w["D"], w["S"], w["n"]
    L = S // n
    # q, k, v ~ N(0, std^2), dO ~ N(0, 1) from numpy.random.default_rng(0) in fp32, rounded to bf16
    # (round to nearest even) on the device: the same stream, draw for draw, as the oracle's
    # make_inputs(0, B, S, S, H, D, std), generated in pieces to bound host memory
    rng0 = np.random.default_rng(0)

    def mk(std):
        t = torch.empty(B * S * H * D, device=dev, dtype=torch.bfloat16)
        piece = 1 << 26
        for a0 in range(0, t.numel(), piece):
            x = rng0.standard_normal(min(piece, t.numel() - a0), dtype=np.float32)
            if std != 1.0:
                x *= np.float32(std)
            t[a0:a0 + x.size] = torch.from_numpy(x).to(dev).to(torch.bfloat16)
        return t.view(B, S, H, D)

    q, k, v = mk(w["std"]), mk(w["std"]), mk(w["std"])
    do = mk(1.0)
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
        if w["bias"] == "callable":
            if args.no_dense_summary:
                from ring_attention import bias as rbias
                rbias.DENSE_SUMMARY = False

            def fn(q_segment_ids, kv_segment_ids):  # the form of ring_test.py:226-233, head-broadcast
                same = q_segment_ids[:, :, None] == kv_segment_ids[:, None, :]
                return torch.where(same, 0.0, float("-inf"))[:, None]
        else:
            fn = ra.segment_bias() + ra.alibi_bias(ra.alibi_slopes(H))
        q_kw, kv_kw = {"q_segment_ids": seg}, {"kv_segment_ids": seg}
    # every step below asks for its plan the way a call of ring_attention does (a small cache keyed
    # on shapes, ring size and bias arrays), so the timed steps carry the host work of a real call
    get_plan = lambda: rr._plan_for(q, k, n, fn, q_kw, kv_kw)
    plan = get_plan()

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
        # one device's real share: its query shard against all key/value shards in the forward
        # pass and the same (query shard, key/value shard) pairs in the backward pass
        P = sum(pairs[(only_rank, ks)] for ks in range(n))
    else:
        P = sum(pairs.values())
    flops_fwd = 4.0 * D * P * B * H
    flops_bwd = 10.0 * D * P * B * H

    ev = lambda: torch.cuda.Event(enable_timing=True)

    fused = args.impl == "hip_fused"
    ring_fwd = rr._ring_forward_fused if fused else rr._ring_forward
    ring_bwd = rr._ring_backward_fused if fused else rr._ring_backward
    if fused:
        args.no_kernel_timing = True

    if only_rank is not None:
        if fused or args.graph:
            raise SystemExit("--workload C3a runs launch per step, eagerly")
        args.no_kernel_timing = True
        r = only_rank
        qr, dor = rr._shard_bhld(q, r, L), rr._shard_bhld(do, r, L)
        carry = rr.init_carry(B, H, L, D, dev)
        out_r = torch.empty((B, L, H, D), dtype=torch.bfloat16, device=dev).permute(0, 2, 1, 3)
        lse_r = torch.empty((B, H, L), dtype=torch.float32, device=dev)
        delta_r = torch.empty((B, H, L), dtype=torch.float32, device=dev)
        dq_acc = torch.empty((B, H, L, D), dtype=torch.float32, device=dev)
        dk_acc, dv_acc = torch.empty_like(dq_acc), torch.empty_like(dq_acc)
        dq_r = torch.empty((B, L, H, D), dtype=torch.bfloat16, device=dev).permute(0, 2, 1, 3)
        dk, dv = torch.empty_like(k), torch.empty_like(v)
        order = [(r - t) % n for t in range(n)]  # the key/value shards as they arrive at device r

    def rank_step(marks=None):
        if marks is not None:
            marks[0].record()
        rr.reset_carry(*carry)
        for s_ in order:
            rr.fwd_block(qr, rr._shard_bhld(k, s_, L), rr._shard_bhld(v, s_, L), plan.block_bias(r, s_), *carry, sm_scale)
        rr.finalize_carry(*carry, out_r, lse_r)
        if marks is not None:
            marks[1].record()
        rr.precompute_delta(out_r, dor, delta_r)
        dq_acc.zero_()
        for s_ in order:
            dk_acc.zero_()
            dv_acc.zero_()
            rr._bwd_step(qr, rr._shard_bhld(k, s_, L), rr._shard_bhld(v, s_, L), dor, lse_r, delta_r, dq_acc,
                         dk_acc, dv_acc, plan.block_bias(r, s_), sm_scale)
            rr._finalize_grad(dk_acc, rr._shard_bhld(dk, s_, L))
            rr._finalize_grad(dv_acc, rr._shard_bhld(dv, s_, L))
        rr._finalize_grad(dq_acc, dq_r)
        if marks is not None:
            marks[2].record()
        return out_r, (dq_r, dk, dv)

    def one_step(marks=None):
        if only_rank is not None:
            return rank_step(marks)
        if marks is not None:
            marks[0].record()
        plan = get_plan()
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
        if w["bias"] == "callable" and not args.no_dense_summary:
            # Every block goes through one summary pass (ra_dense_map, inside the forward launch's
            # bracket and again in the backward step's: the callable is called once per loop,
            # ring.py:107,186); the step kernels then leave out what is -inf throughout and read the
            # block only where it is not zero: matrix work over the unmasked pairs, as in the other
            # workloads.
            ach = kern[dom]["flops"] / kern[dom]["ms"] / 1e9
            result["roofline"] = {"bound": "mfma", "kernel": names[dom] + "<D, 2> with the block's summary",
                                  "achieved": round(ach, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                  "frac": round(ach / PEAK_BF16_TFLOPS, 4), "traffic": None}
            for kind in kern:
                ev_ = [ms for (k2, qs, ks), ms in recs if k2 == kind]
                kernels[names[kind]]["avg_ms_all_launches"] = round(sum(ev_) / len(ev_), 4)
            k_ms = sum(ms for _, ms in recs)
            result["host_and_torch_ms_per_step"] = round(ms_per_step - k_ms, 3)
            result["step_kernels_ms_per_step"] = round(k_ms, 3)
        elif w["bias"] == "callable":
            # the kernels stream the dense [b, 1, lq, lk] fp32 block: 4 bytes per (query, key) position
            # and launch if the heads of a launch share one pass over it, next to which the bf16
            # operands and fp32 carries of the step are small: HBM bound
            every = [ms for (kind, qs, ks), ms in recs if kind == dom]
            bytes_launch = 4.0 * B * L * L
            avg_ms = sum(every) / len(every)
            ach = bytes_launch / (avg_ms * 1e-3) / 1e9
            result["roofline"] = {"bound": "hbm", "kernel": names[dom] + "<D, 2>", "achieved": round(ach, 1),
                                  "peak": 8000.0, "unit": "GB/s", "frac": round(ach / 8000.0, 4), "traffic": None,
                                  "algorithmic_bytes_per_launch": bytes_launch, "avg_ms_all_launches": round(avg_ms, 4)}
            for kind in kern:
                ev_ = [ms for (k2, qs, ks), ms in recs if k2 == kind]
                kernels[names[kind]]["avg_ms_all_launches"] = round(sum(ev_) / len(ev_), 4)
                kernels[names[kind]]["dense_bias_gbps"] = round(bytes_launch / (sum(ev_) / len(ev_) * 1e-3) / 1e9, 1)
            k_ms = sum(ms for _, ms in recs)
            result["host_and_torch_ms_per_step"] = round(ms_per_step - k_ms, 3)
            result["step_kernels_ms_per_step"] = round(k_ms, 3)
        else:
            ach = kern[dom]["flops"] / kern[dom]["ms"] / 1e9
            result["roofline"] = {"bound": "mfma", "kernel": names[dom], "achieved": round(ach, 2),
                                  "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                  "frac": round(ach / PEAK_BF16_TFLOPS, 4),
                                  "traffic": stored_traffic(args.workload, names[dom])}
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
        result["cpu_baseline"] = cpu_baseline(D, args.cpu_baseline_config)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
