#!/usr/bin/env python3
"""Headline benchmark: prefill dispatch + combine on one MI355X, with the decode and rank-share shapes and the W4A8
expert FFN measured beside it.

A step is one pass of the hot path over one synthetic batch at the prefill shape
(T=4096, H=7168, 256 experts, top-8 with Zipf(1.2) popularity, seed 0):
  layout (counts / prefix / stable permutation, with the host read-back of R that a fresh dispatch
  needs) -> FP8 e4m3 dispatch with the per-128 quantiser fused into the expand-permute ->
  combine of BF16 gradients N(0,1) [R,H] (the backward of dispatch).
`value` is the algorithmic HBM bytes of dispatch + combine per second of wall time of that step.

Every kernel is then timed by itself with HIP events on the stream it is launched on, two ways: with the caches
flushed before every launch by a 256 MiB fill (the reference's protocol, deep_ep/utils/testing.py:27-35; at least 20
warm-ups and 100 launches: mean / min / p50 / p95) and back to back.  `roofline` is the dominant kernel under the
flush protocol.  Prints ONE JSON line.

Other modes:
  --ingest-pmc FETCH.csv WRITE.csv   turn two rocprofv3 --pmc counter files of this command (run with --calibrate-copy)
                                     into profiles/hbm_traffic.json, which `roofline.traffic` is read from
  --protocol PRESET                  the reference's generic benchmark workloads (benchmarks/_config.py) through this
                                     library: one `measured` record per operation in the v1 result schema
"""

from __future__ import annotations

import argparse
import contextlib
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = 5000.0  # MI355X dense FP8 (the mixed FP8 x FP4 MFMA issues at the FP8 cadence)
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
FLUSH_BYTES = 256 << 20


def algorithmic_bytes(tokens, hidden, topk, rows):
    """Bytes each kernel must move (no padding, no re-reads)."""
    idx = tokens * topk * 8
    dispatch = tokens * hidden * 2 + tokens * topk * 4 + rows * hidden + rows * (hidden // 128) * 4 + rows * 4
    combine = rows * hidden * 2 + tokens * topk * 4 + tokens * hidden * 2
    layout = idx + 2 * tokens * topk * 4
    return dict(layout=layout, dispatch=dispatch, combine=combine)


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


class Timer:
    """Device times of one launch closure, HIP events on torch's current stream (the one ops launches on)."""

    def __init__(self, torch, iters, warmups):
        self.torch = torch
        self.iters = max(1, iters)
        self.warmups = max(1, warmups)
        self.flush = None
        self.cycles_per_us = None

    def spin_cycles_per_us(self):
        """How many `torch.cuda._sleep` cycles make one microsecond on this GPU (measured once)."""
        if self.cycles_per_us is None:
            torch = self.torch
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda._sleep(100_000)
            start.record()
            torch.cuda._sleep(2_000_000)
            stop.record()
            torch.cuda.synchronize()
            self.cycles_per_us = 2_000_000 / (start.elapsed_time(stop) * 1000.0)
        return self.cycles_per_us

    @staticmethod
    @contextlib.contextmanager
    def no_collector():
        """The timed loops run without Python's cyclic garbage collector: a full collection over the benchmark's heap
        takes tens of milliseconds and would land in whichever launch happens to trigger it."""
        was_enabled = gc.isenabled()
        gc.disable()
        try:
            yield
        finally:
            if was_enabled:
                gc.enable()

    def back_to_back(self, fn, head_start=False):
        """Average microseconds over `iters` launches queued without gaps.  head_start: the GPU is kept busy first by a
        spin kernel (no memory traffic that the timed kernels would have to wait out) for as long as the host needs to
        queue all the launches, measured on the warm-up launches, so that a kernel shorter than its Python launch path
        is still timed back to back."""
        torch = self.torch
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(self.warmups):
            fn()
        host_us = (time.perf_counter() - t0) * 1e6 / self.warmups
        torch.cuda.synchronize()
        if head_start and hasattr(torch.cuda, "_sleep"):
            torch.cuda._sleep(int(self.spin_cycles_per_us() * host_us * self.iters * 1.5) + 100_000)
        with self.no_collector():
            start.record()
            for _ in range(self.iters):
                fn()
            stop.record()
            torch.cuda.synchronize()
        return start.elapsed_time(stop) * 1000.0 / self.iters

    def flushed(self, fn, read_sweep=False):
        """Per-launch times with the caches flushed before every launch: by a 256 MiB fill (which leaves the caches full
        of dirty lines that are written back while the timed kernel runs), or, read_sweep, by a read-only pass over
        the same 256 MiB (which evicts as much and leaves nothing to write back)."""
        torch = self.torch
        if self.flush is None:
            self.flush = torch.zeros(FLUSH_BYTES, dtype=torch.uint8, device="cuda")
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(self.iters)]
        for _ in range(self.warmups):
            fn()
        with self.no_collector():
            for start, stop in pairs:
                if read_sweep:
                    self.flush.view(torch.int64).sum()
                else:
                    self.flush.zero_()
                start.record()
                fn()
                stop.record()
            torch.cuda.synchronize()
        times = sorted(a.elapsed_time(b) * 1000.0 for a, b in pairs)
        pick = lambda q: times[min(len(times) - 1, int(q * len(times)))]
        return dict(mean=sum(times) / len(times), min=times[0], p50=pick(0.5), p95=pick(0.95))

    def drained(self, fn):
        """Mean microseconds of [launch, read-only sweep of 256 MiB] after such a sweep, minus a sweep that follows a
        sweep: the launch with whatever it leaves in the caches for later (dirty lines of write-through or cached
        stores, which the next kernel would have to write back) charged to it."""
        torch = self.torch
        if self.flush is None:
            self.flush = torch.zeros(FLUSH_BYTES, dtype=torch.uint8, device="cuda")
        sweep = lambda: self.flush.view(torch.int64).sum()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(3):
            sweep()
        start.record()
        for _ in range(self.iters):
            sweep()
        stop.record()
        torch.cuda.synchronize()
        alone = start.elapsed_time(stop) * 1000.0 / self.iters
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(self.iters)]
        with self.no_collector():
            for begin, end in pairs:
                sweep()
                begin.record()
                fn()
                sweep()
                end.record()
            torch.cuda.synchronize()
        return sum(a.elapsed_time(b) * 1000.0 for a, b in pairs) / len(pairs) - alone

    def kernel(self, fn, nbytes, head_start=False, extra=None, read_sweep=False, drain=False):
        """One `kernels` entry: flushed statistics, the back-to-back figure, and GB/s of both against 8 TB/s.
        read_sweep: also the statistics after a read-only flush (`after_read_sweep_us`); drain: and with the sweep that
        follows charged to the launch (`after_read_sweep_with_drain_us`)."""
        warm = self.back_to_back(fn, head_start)
        cold = self.flushed(fn)
        if read_sweep:
            swept = self.flushed(fn, read_sweep=True)
            extra = dict(extra or {}, after_read_sweep_us=swept, frac_after_read_sweep=nbytes / swept["mean"] / 1e3 / HBM_PEAK_GBS)
        if drain:
            with_drain = self.drained(fn)
            extra = dict(extra or {}, after_read_sweep_with_drain_us=with_drain,
                         frac_after_read_sweep_with_drain=nbytes / with_drain / 1e3 / HBM_PEAK_GBS)
        entry = dict(
            bytes=nbytes,
            us=cold["mean"],
            flushed_us=cold,
            back_to_back_us=warm,
            GBps=nbytes / cold["mean"] / 1e3,
            frac_of_8TBps=nbytes / cold["mean"] / 1e3 / HBM_PEAK_GBS,
            GBps_back_to_back=nbytes / warm / 1e3,
            frac_back_to_back=nbytes / warm / 1e3 / HBM_PEAK_GBS,
        )
        if extra:
            entry.update(extra)
        return entry


def cpu_baseline(x, idx, w, grads, cfg):
    """The reference CPU path (torch CPU, all host threads) on the same full batch: 3 warm-ups + 10 timed passes."""
    import torch

    from oracle import baseline

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)

    def step():
        counts, psum, r2row, r2route = baseline.layout(idx, cfg["experts"])
        baseline.dispatch_fp8(x, w, r2route, cfg["topk"])
        baseline.combine(grads[: r2route.numel()], r2row)
        return r2route.numel()

    for _ in range(3):
        rows = step()
    times = []
    for _ in range(10):
        t0 = time.perf_counter_ns()
        step()
        times.append((time.perf_counter_ns() - t0) / 1e9)
    mean = sum(times) / len(times)
    nbytes = algorithmic_bytes(cfg["tokens"], cfg["hidden"], cfg["topk"], rows)
    moved = nbytes["dispatch"] + nbytes["combine"]
    return dict(
        value=moved / mean / 1e9,
        unit="GB/s",
        cores=cores,
        kind="port",
        sample=f"the full batch ({cfg['tokens']} tokens, {rows} rows), 3 warm-ups + 10 timed passes, mean {mean * 1e3:.1f} ms "
        f"(min {min(times) * 1e3:.1f}) per pass of layout + FP8 quantise + expand + combine, torch CPU "
        f"{torch.get_num_threads()} threads, {cpu_model()}",
    )


def megamoe_cpu_baseline(hidden, inter):
    """The reference's CPU form of the expert FFN (reference.py:84-89) on dequantised fp32 operands, the two
    contractions by torch.matmul: one expert, a sample of 256 of its rows, 3 warm-ups + 10 timed passes."""
    import numpy as np
    import torch

    from oracle import baseline

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    rows = 256
    rng = np.random.default_rng(0)
    x = torch.from_numpy(rng.normal(size=(rows, hidden)).astype(np.float32))
    w1 = torch.from_numpy((rng.normal(size=(2 * inter, hidden)) * 0.02).astype(np.float32))
    w2 = torch.from_numpy((rng.normal(size=(hidden, inter)) * 0.02).astype(np.float32))
    for _ in range(3):
        baseline.megamoe_expert_forward(x, w1, w2)
    times = []
    for _ in range(10):
        t0 = time.perf_counter_ns()
        baseline.megamoe_expert_forward(x, w1, w2)
        times.append((time.perf_counter_ns() - t0) / 1e9)
    mean = sum(times) / len(times)
    flops = 2.0 * rows * hidden * 2 * inter + 2.0 * rows * inter * hidden
    return dict(
        value=flops / mean / 1e12,
        unit="TFLOP/s",
        cores=cores,
        kind="port",
        sample=f"{rows} rows of one expert (H={hidden}, I={inter}: {flops / 1e9:.1f} GFLOP), dense fp32 weights as the oracle "
        f"materialises them, 3 warm-ups + 10 timed passes, mean {mean * 1e3:.1f} ms, torch CPU {torch.get_num_threads()} "
        f"threads, {cpu_model()}",
    )


def megamoe_shape(torch, ops, timer, tokens, experts, local, topk, weight_sets, hidden=7168, inter=2048, served_only=False):
    """One W4A8 forward shape: (back-to-back us, flushed statistics, rows that reach a local expert, FLOPs).  Random codes
    and constant scale bytes: the time does not depend on the values.  FLOPs = 2*R*H*2I + 2*R*I*H for the R rows."""
    dev = "cuda"
    gen = torch.Generator().manual_seed(0)
    idx = torch.multinomial(torch.ones(tokens, experts), topk, generator=gen).to(torch.int32).to(dev)
    w = torch.softmax(torch.randn(tokens, topk, generator=gen), -1).to(dev)
    x_codes = torch.randint(0, 120, (tokens, hidden), dtype=torch.uint8, generator=gen).to(dev).view(torch.float8_e4m3fn)
    x_scales = torch.full((tokens, hidden // 32), 127, dtype=torch.uint8, device=dev)
    sets = []
    for _ in range(weight_sets):
        w1 = torch.randint(0, 256, (local, 2 * inter, hidden // 2), dtype=torch.uint8, device=dev)
        s1 = torch.full((local, 2 * inter, ops.megamoe_prepared_shape(2 * inter, hidden, True)[2]), 119, dtype=torch.uint8, device=dev)
        w2 = torch.randint(0, 256, (local, hidden, inter // 2), dtype=torch.uint8, device=dev)
        s2 = torch.full((local, hidden, ops.megamoe_prepared_shape(hidden, inter, False)[2]), 119, dtype=torch.uint8, device=dev)
        sets.append((w1, s1, w2, s2))
    ws = ops.Workspace(ops.megamoe_workspace_bytes(tokens, topk, hidden, inter, local))
    ws.tune("megamoe_served_only", int(served_only))
    y = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)
    counts = torch.empty((local,), dtype=torch.int32, device=dev)
    calls = [0]

    def run():
        w1, s1, w2, s2 = sets[calls[0] % len(sets)]
        calls[0] += 1
        ops.megamoe_forward(ws, x_codes, x_scales, idx, w, w1, s1, w2, s2, experts, 0, local, y, counts)

    us = timer.back_to_back(run)
    cold = timer.flushed(run)
    rows = int(counts.sum().item())
    flops = 2.0 * rows * hidden * 2 * inter + 2.0 * rows * inter * hidden
    ws.destroy()
    return us, cold, rows, flops


def megamoe_bench(torch, ops, timer, with_cpu):
    """W4A8 fused expert FFN, H=7168, I=2048.  The headline shape is one EP64 rank's share: 64 source ranks x 256 tokens,
    384 experts of which 6 are local, top-8 uniform routing (about 2000 rows), with three weight sets used in turn
    (3 x 132 MB, more than the 256 MB memory-side cache) so that the GEMMs stream their weights from HBM as they do
    between the layers of a model.  `large_batch` is the same kernels where tile quantisation and fixed costs stop
    mattering: 8192 tokens x top-8 over 32 local experts (65 536 rows)."""
    hidden, inter = 7168, 2048
    us, cold, rows, flops = megamoe_shape(torch, ops, timer, 64 * 256, 384, 6, 8, weight_sets=3)
    result = {
        "workload": "EP64 rank share: 16384 candidate tokens, 6 of 384 experts local, top-8, H=7168, I=2048, "
        "MXFP8 activations x MXFP4 weights (random codes, constant scale bytes), three weight sets in turn; layout + "
        "GMM1(+SwiGLU+requant) + GMM2 + weighted reduce into [16384,7168] (rows of unserved tokens zero-filled)",
        "rows": rows,
        "us_forward": us,
        "flushed_us": cold,
        "gflop": flops / 1e9,
        "tflops_forward": flops / us / 1e6,
        "roofline": {"bound": "mfma", "achieved": flops / us / 1e6, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops / us / 1e6 / MFMA_PEAK_TFLOPS,
                     "note": "whole forward (4 launches), back to back; per-kernel GEMM times are in profiles/"},
    }
    us, cold, rows, flops = megamoe_shape(torch, ops, timer, 64 * 256, 384, 6, 8, weight_sets=3, served_only=True)
    result["served_only"] = {
        "workload": "the same rank share with the rows of y left untouched whose token no local expert serves (what the rank "
        "owes an EP job: other ranks produce those rows); nothing is zero-filled, by the GEMM's idle workgroups or the reduce",
        "rows": rows, "us_forward": us, "flushed_us": cold, "tflops_forward": flops / us / 1e6,
        "frac_of_fp8_peak": flops / us / 1e6 / MFMA_PEAK_TFLOPS,
    }
    big = Timer(torch, max(1, timer.iters // 5), max(1, timer.warmups // 5))
    big.flush, big.cycles_per_us = timer.flush, timer.cycles_per_us
    us, cold, rows, flops = megamoe_shape(torch, ops, big, 8192, 32, 32, 8, weight_sets=1)
    result["large_batch"] = {
        "workload": "8192 tokens x top-8, all 32 experts local (65 536 rows), one weight set (705 MB); whole forward",
        "rows": rows, "us_forward": us, "flushed_us": cold, "gflop": flops / 1e9, "tflops_forward": flops / us / 1e6,
        "frac_of_fp8_peak": flops / us / 1e6 / MFMA_PEAK_TFLOPS,
    }
    us, cold, rows, flops = megamoe_shape(torch, ops, timer, 512, 256, 32, 8, weight_sets=1)
    weight_bytes = 32 * (2 * inter * hidden + hidden * inter) // 2
    result["decode_share"] = {
        "workload": "512 tokens x top-8, 32 of 256 experts local (about 16 rows per expert): the GEMMs are bound by streaming "
        "their 705 MB of FP4 weights (64-row tiles, non-temporal weight copies); whole forward",
        "rows": rows, "us_forward": us, "flushed_us": cold, "weight_bytes": weight_bytes,
        "weights_GBps_forward": weight_bytes / us / 1e3, "frac_of_8TBps": weight_bytes / us / 1e3 / HBM_PEAK_GBS,
    }
    # the MX activation quantiser the public API runs when it is given BF16 rows (per-32 e8m0 scales)
    xb = torch.randn(64 * 256, hidden, device="cuda").bfloat16()
    result["mx_quant"] = timer.kernel(lambda: ops.mx_quant(xb), xb.numel() * 3 + xb.numel() // 32)
    result["mx_quant"]["workload"] = "BF16 [16384,7168] -> e4m3 codes + e8m0 scale per 32"
    del xb
    if with_cpu:
        result["cpu_baseline"] = megamoe_cpu_baseline(hidden, inter)
    return result


def decode_kernels(torch, ops, cases, timer):
    """Decode shape (T=128, H=7168, 256 experts, top-8 uniform, all experts local): BF16 dispatch with expand +
    weighted combine, and their layout."""
    dev = "cuda"
    x, idx, w, cfg = cases.make_inputs("C2", seed=0)
    tokens, hidden, topk, experts = cfg["tokens"], cfg["hidden"], cfg["topk"], cfg["experts"]
    xd, idxd, wd = x.to(dev), idx.to(dev), w.to(dev)
    ws = ops.Workspace(1 << 20)
    lay = ops.layout(ws, idxd, experts)
    _, rows = ops.layout_wait(ws)
    r2row, r2route = lay["route_to_row"], lay["row_to_route"]
    recv, _, recv_w = ops.dispatch_copy(xd, None, wd, r2row, r2route, rows)
    out = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)
    dispatch_bytes = tokens * hidden * 2 + tokens * topk * 8 + rows * hidden * 2 + rows * 4
    combine_bytes = rows * hidden * 2 + rows * 4 + tokens * topk * 4 + tokens * hidden * 2
    entries = {
        "layout": timer.kernel(lambda: ops.layout(ws, idxd, experts), tokens * topk * 16, head_start=True),
        "dispatch_bf16": timer.kernel(lambda: ops.dispatch_copy(xd, None, wd, r2row, r2route, rows), dispatch_bytes, head_start=True),
        "combine_weighted": timer.kernel(lambda: ops.combine(recv, r2row, recv_w, out=out), combine_bytes, head_start=True),
        # what a fresh dispatch of this size runs: layout and payload in one launch
        "layout_dispatch_bf16_one_launch": timer.kernel(
            lambda: ops.layout_dispatch_small(ws, idxd, xd, None, wd, experts), dispatch_bytes + tokens * topk * 8, head_start=True),
    }
    ws.destroy()
    return {"workload": f"decode: T={tokens}, H={hidden}, {experts} experts, top-{topk} uniform, {rows} rows", "kernels": entries}


def rank_share_kernels(torch, ops, cases, timer):
    """One EP64 rank's receive share (64 x 256 candidate tokens, 6 of 384 experts local): layout, fused FP8 dispatch
    of the rows that hit a local expert, weighted combine back into [16384,H]."""
    dev = "cuda"
    x, idx, w, cfg = cases.make_inputs("C4", seed=0)
    tokens, hidden, topk, experts, local = cfg["tokens"], cfg["hidden"], cfg["topk"], cfg["experts"], cfg["num_local"]
    xd, idxd, wd = x.to(dev), idx.to(dev), w.to(dev)
    ws = ops.Workspace(1 << 20)
    lay = ops.layout(ws, idxd, experts, 0, local)
    _, rows = ops.layout_wait(ws, local)
    r2row, r2route = lay["route_to_row"], lay["row_to_route"]
    recv_w = ops.dispatch_quant_fp8(xd, wd, r2row, r2route, rows)[2]
    y = torch.randn(rows, hidden, generator=torch.Generator().manual_seed(1)).bfloat16().to(dev)
    out = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)
    served = int((r2row >= 0).any(dim=1).sum().item())
    dispatch_bytes = tokens * topk * 8 + rows * hidden * 2 + rows * (hidden + (hidden // 128) * 4 + 4)
    combine_bytes = rows * hidden * 2 + rows * 4 + tokens * topk * 4 + served * hidden * 2
    zero_fill = (tokens - served) * hidden * 2
    entries = {
        "layout": timer.kernel(lambda: ops.layout(ws, idxd, experts, 0, local), tokens * topk * 16, head_start=True),
        "dispatch_fp8_quant": timer.kernel(lambda: ops.dispatch_quant_fp8(xd, wd, r2row, r2route, rows), dispatch_bytes, head_start=True),
        "combine_weighted": timer.kernel(
            lambda: ops.combine(y, r2row, recv_w, out=out), combine_bytes,
            extra={"zero_fill_bytes": zero_fill,
                   "note": "rows of unserved tokens are zero-filled, not skipped: the kernel also writes zero_fill_bytes, "
                   "which `bytes` (rows read plus served rows written) leaves out"}),
    }
    entries["combine_weighted"]["GBps_with_zero_fill"] = (combine_bytes + zero_fill) / entries["combine_weighted"]["us"] / 1e3
    entries["combine_weighted_served_only"] = timer.kernel(
        lambda: ops.combine(y, r2row, recv_w, out=out, served_only=True), combine_bytes, head_start=True,
        extra={"note": "rows of unserved tokens are skipped (dpep_combine_served): what the rank does for its share of an EP "
               "job, where those tokens get their rows from other ranks"})
    ws.destroy()
    return {"workload": f"EP64 rank share: {tokens} candidate tokens, {local} of {experts} experts local, top-{topk} uniform, "
            f"H={hidden}, {rows} rows, {served} served tokens", "kernels": entries}


def read_traffic(kernel):
    """HBM bytes per launch of `kernel` from profiles/hbm_traffic.json (written by --ingest-pmc), or None.  The file
    keys its entries "<kernel> @<grid size>"; of several grids of one kernel the one that moved most is the
    benchmark's own shape (the counter runs skip the smaller workloads)."""
    try:
        table = json.load(open(TRAFFIC_FILE))
    except (OSError, ValueError):
        return None
    found = [entry for name, entry in table.get("kernels", {}).items() if name.rsplit(" @", 1)[0] == kernel and not name.endswith("]")]
    return max((entry["hbm_bytes"] for entry in found), default=None)


def ingest_pmc(fetch_csv, write_csv, extra=()):
    """Two rocprofv3 --pmc runs of `bench.py --calibrate-copy --no-extra-shapes` (FETCH_SIZE, then WRITE_SIZE; KiB per
    dispatch) -> profiles/hbm_traffic.json.  Both counters are scaled by what they read for the calibration copy, whose
    traffic is known: [32768,7168] BF16 rows through dispatch_copy_row_kernel = 458 752 KiB read and as much written."""
    import csv
    import re

    def averages(path, counter):
        sums, calls = {}, {}
        for row in csv.DictReader(open(path)):
            if row.get("Counter_Name") != counter or "dpep::" not in row["Kernel_Name"]:
                continue
            name = row["Kernel_Name"].replace("void ", "").replace("dpep::(anonymous namespace)::", "")
            name = re.sub(r"\(.*", "", name).strip() + " @" + row["Grid_Size"]
            sums[name] = sums.get(name, 0.0) + float(row["Counter_Value"])
            calls[name] = calls.get(name, 0) + 1
        return {name: sums[name] / calls[name] for name in sums}, calls

    (fetch, calls), (write, _) = averages(fetch_csv, "FETCH_SIZE"), averages(write_csv, "WRITE_SIZE")
    known_kib = 32768 * 7168 * 2 / 1024
    copy = [name for name in fetch if name.startswith("dispatch_copy_row_kernel") and name in write]
    if len(copy) != 1:
        raise SystemExit("the counter files must hold one shape of dispatch_copy_row_kernel: run bench.py with "
                         "--calibrate-copy --no-extra-shapes")
    fetch_scale, write_scale = known_kib / fetch[copy[0]], known_kib / write[copy[0]]
    kernels = {}
    for name in sorted(set(fetch) & set(write)):
        read_bytes, written = fetch[name] * fetch_scale * 1024, write[name] * write_scale * 1024
        kernels[name] = dict(dispatches=calls[name], fetch_kib=fetch[name], write_kib=write[name], hbm_read_bytes=round(read_bytes),
                             hbm_written_bytes=round(written), hbm_bytes=round(read_bytes + written))
    # Counter passes of a single workload (`bench.py --megamoe-only SHAPE`): scaled by the same factors, keyed
    # "<kernel> @<grid size> [SHAPE]", so that a kernel that runs in several workloads has an entry for each.
    for fetch_more, write_more, label in extra:
        (fetch_x, calls_x), (write_x, _) = averages(fetch_more, "FETCH_SIZE"), averages(write_more, "WRITE_SIZE")
        for name in sorted(set(fetch_x) & set(write_x)):
            read_bytes, written = fetch_x[name] * fetch_scale * 1024, write_x[name] * write_scale * 1024
            kernels[f"{name} [{label}]"] = dict(dispatches=calls_x[name], fetch_kib=fetch_x[name], write_kib=write_x[name],
                                                hbm_read_bytes=round(read_bytes), hbm_written_bytes=round(written),
                                                hbm_bytes=round(read_bytes + written))
    table = dict(source="rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs) of `python3 bench.py --steps 5 --warmup 2 "
                 "--kernel-iters 5 --kernel-warmup 2 --no-cpu-baseline --no-extra-shapes --calibrate-copy`; KiB per dispatch, "
                 "averaged over the dispatches of each kernel and grid size (keys: '<kernel> @<grid size>'); most launches "
                 "follow a 256 MiB cache flush, so inputs come from HBM",
                 fetch_scale=fetch_scale, write_scale=write_scale, calibration_kib=known_kib, kernels=kernels)
    json.dump(table, open(TRAFFIC_FILE, "w"), indent=1, sort_keys=True)
    print(f"wrote {TRAFFIC_FILE}: {len(kernels)} kernels, scale factors {fetch_scale:.3f} / {write_scale:.3f}")


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=100)
    parser.add_argument("--warmup", type=int, default=20)
    parser.add_argument("--kernel-iters", type=int, default=100, help="timed launches per kernel (each protocol)")
    parser.add_argument("--kernel-warmup", type=int, default=20, help="untimed launches per kernel before them")
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-megamoe", action="store_true", help="skip the W4A8 expert-FFN measurement")
    parser.add_argument("--no-extra-shapes", action="store_true", help="skip the decode and rank-share kernel timings")
    parser.add_argument("--calibrate-copy", action="store_true",
                        help="also launch a plain copy of known size (identity dispatch of [32768,7168] BF16: 469.76 MB "
                        "read + 469.76 MB written) so that rocprofv3 FETCH_SIZE / WRITE_SIZE can be scaled")
    parser.add_argument("--dispatch-stores", choices=("through", "streaming", "cached"),
                        help="store policy of the dispatch kernels (default: the library's, streaming)")
    parser.add_argument("--megamoe-only", choices=("rank_share", "served_only", "large_batch", "decode_share"),
                        help="run nothing but that W4A8 forward shape (for counter and trace runs of one workload) and print "
                        "its figures")
    parser.add_argument("--ingest-pmc", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"))
    parser.add_argument("--ingest-extra", nargs=3, action="append", default=[], metavar=("FETCH_CSV", "WRITE_CSV", "LABEL"),
                        help="with --ingest-pmc: two more counter files, of `bench.py --megamoe-only LABEL`")
    parser.add_argument("--protocol", metavar="PRESET", help="run the reference's generic benchmark workload PRESET "
                        "(smoke, decode, prefill) and print one `measured` record per operation")
    args = parser.parse_args()
    if args.ingest_pmc:
        ingest_pmc(*args.ingest_pmc, extra=args.ingest_extra)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU's share; --gpus must be 1 (no multi-GPU path in this build)", file=sys.stderr)
        sys.exit(2)

    import torch

    from deepep_amd import ops
    from oracle import cases

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.protocol:
        from deepep_amd import protocol_bench

        for record in protocol_bench.run(args.protocol, torch, ops, iters=args.kernel_iters, warmups=args.kernel_warmup):
            print(json.dumps(record))
        return

    if args.megamoe_only:
        timer = Timer(torch, args.kernel_iters, args.kernel_warmup)
        shapes = {"rank_share": (64 * 256, 384, 6, 8, 3, False), "served_only": (64 * 256, 384, 6, 8, 3, True),
                  "large_batch": (8192, 32, 32, 8, 1, False), "decode_share": (512, 256, 32, 8, 1, False)}
        tokens, experts, local, topk, sets, served = shapes[args.megamoe_only]
        us, cold, rows, flops = megamoe_shape(torch, ops, timer, tokens, experts, local, topk, weight_sets=sets, served_only=served)
        print(json.dumps({"workload": args.megamoe_only, "rows": rows, "us_forward": us, "flushed_us": cold,
                          "tflops_forward": flops / us / 1e6, "frac_of_fp8_peak": flops / us / 1e6 / MFMA_PEAK_TFLOPS}))
        return
    if args.dispatch_stores:
        ops.dispatch_store_policy(args.dispatch_stores)
    x, idx, w, cfg = cases.make_inputs("C3", seed=0)
    tokens, hidden, topk, experts = cfg["tokens"], cfg["hidden"], cfg["topk"], cfg["experts"]
    rows_expected = tokens * topk
    grads = torch.randn(rows_expected, hidden, generator=torch.Generator().manual_seed(1)).bfloat16()
    xd, idxd, wd, gd = x.to(dev), idx.to(dev), w.to(dev), grads.to(dev)
    ws = ops.Workspace(max(ops.layout_workspace_bytes(tokens, topk, experts), 1 << 20))

    def step():
        # as ElasticBuffer.dispatch does when every expert is local: the payload kernel is queued behind the layout
        # into outputs of T*K rows, and the host synchronisation that yields R (to narrow them) runs meanwhile
        lay = ops.layout(ws, idxd, experts)
        full = ops.dispatch_quant_fp8(xd, wd, lay["route_to_row"], lay["row_to_route"], None)
        _, rows = ops.layout_wait(ws)
        recv = tuple(t[:rows] for t in full)
        out = ops.combine(gd[:rows], lay["route_to_row"])
        return rows, recv, out

    for _ in range(args.warmup):
        rows, _, _ = step()
    torch.cuda.synchronize()
    with Timer.no_collector():
        t0 = time.perf_counter()
        for _ in range(args.steps):
            rows, _, _ = step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    nbytes = algorithmic_bytes(tokens, hidden, topk, rows)
    moved = nbytes["dispatch"] + nbytes["combine"]

    # Per-kernel device time (HIP events on the launch stream), same inputs.
    timer = Timer(torch, args.kernel_iters, args.kernel_warmup)
    lay = ops.layout(ws, idxd, experts)
    r2row, r2route = lay["route_to_row"], lay["row_to_route"]
    grows = gd[:rows]
    out_buf = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)
    q_pre, s_pre = ops.cast_to_fp8(xd)  # the reference semantic: the caller quantises, dispatch moves codes and scales
    recv_w = ops.dispatch_quant_fp8(xd, wd, r2row, r2route, rows)[2]
    bf16_dispatch_bytes = tokens * hidden * 2 + tokens * topk * 4 + rows * hidden * 2 + rows * 4
    copy_dispatch_bytes = tokens * (hidden + (hidden // 128) * 4) + tokens * topk * 4 + rows * (hidden + (hidden // 128) * 4 + 4)
    kernels = {
        "layout": timer.kernel(lambda: ops.layout(ws, idxd, experts), nbytes["layout"], head_start=True, read_sweep=True),
        "dispatch_fp8_quant": timer.kernel(lambda: ops.dispatch_quant_fp8(xd, wd, r2row, r2route, rows), nbytes["dispatch"], read_sweep=True, drain=True),
        "dispatch_fp8_copy": timer.kernel(lambda: ops.dispatch_copy(q_pre, s_pre, wd, r2row, r2route, rows), copy_dispatch_bytes, read_sweep=True),
        "dispatch_bf16": timer.kernel(lambda: ops.dispatch_copy(xd, None, wd, r2row, r2route, rows), bf16_dispatch_bytes, read_sweep=True),
        "combine": timer.kernel(lambda: ops.combine(grows, r2row, out=out_buf), nbytes["combine"], read_sweep=True),
        "combine_weighted": timer.kernel(lambda: ops.combine(grows, r2row, recv_w, out=out_buf), nbytes["combine"] + rows * 4, read_sweep=True),
    }
    # The same fused dispatch under the write-through store policy: it ends sooner behind a read sweep because the
    # memory-side cache takes its rows, and leaves their write-back to whatever runs next (`..._with_drain_us`).
    before = ops.dispatch_store_policy("through")
    kernels["dispatch_fp8_quant_write_through"] = timer.kernel(
        lambda: ops.dispatch_quant_fp8(xd, wd, r2row, r2route, rows), nbytes["dispatch"], read_sweep=True, drain=True,
        extra={"note": "not the default: dpep_dispatch_store_policy(DPEP_STORE_THROUGH)"})
    ops.dispatch_store_policy(before)
    # the stand-alone quantiser on the batch's tokens and the dequantiser on its dispatched rows (checking-side kernels of
    # the reference: per_token_cast_to_fp8 / per_token_cast_back)
    recv_q, recv_s, _ = ops.dispatch_copy(q_pre, s_pre, None, r2row, r2route, rows)
    scale_bytes = (hidden // 128) * 4
    kernels["cast_to_fp8"] = timer.kernel(lambda: ops.cast_to_fp8(xd), tokens * (3 * hidden + scale_bytes), head_start=True)
    kernels["cast_back"] = timer.kernel(lambda: ops.cast_back(recv_q, recv_s), rows * (3 * hidden + scale_bytes))
    del recv_q, recv_s

    dominant = kernels["combine"]
    result = {
        "metric": "dispatch+combine HBM GB/s (T=4096,H=7168,k=8)",
        "value": moved / (ms_per_step * 1e-3) / 1e9,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "prefill: T=4096, H=7168, 256 experts, top-8 Zipf(1.2), seed 0; step = layout (+R read-back) "
            "+ FP8 e4m3 dispatch with fused per-128 quant + BF16 combine of N(0,1) grads [R,H]",
            "tokens": tokens,
            "hidden": hidden,
            "topk": topk,
            "experts": experts,
            "rows": rows,
            "bytes_per_step": moved,
            "kernel_timing": f"{args.kernel_warmup} warm-ups + {args.kernel_iters} launches per kernel and protocol; "
            "`us` / `GBps` / `frac_of_8TBps` are the cache-flushed mean (256 MiB fill before every launch), "
            "`back_to_back_us` / `frac_back_to_back` the same launches queued without gaps, `after_read_sweep_us` the "
            "launches after a read-only pass over 256 MiB (caches evicted, no dirty lines left to write back: "
            "`frac_after_read_sweep`)",
        },
        "roofline": {
            "kernel": "combine_kernel<0, false>",
            "bound": "hbm",
            "achieved": dominant["GBps"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": dominant["frac_of_8TBps"],
            "protocol": "mean of cache-flushed launches (256 MiB fill before each); back to back: "
            f"{dominant['GBps_back_to_back']:.0f} GB/s = {dominant['frac_back_to_back']:.3f}",
            # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by a plain copy of known
            # size; read from the file `--ingest-pmc` writes
            "traffic": read_traffic("combine_kernel<0, false>"),
        },
        "kernels": kernels,
        "dispatch_plus_combine_us": kernels["dispatch_fp8_quant"]["us"] + kernels["combine"]["us"],
        "dispatch_plus_combine_frac_of_8TBps": moved / (kernels["dispatch_fp8_quant"]["us"] + kernels["combine"]["us"]) / 1e3 / HBM_PEAK_GBS,
        "dispatch_stores": ops.dispatch_store_policy(),
    }
    # the same sum under the two other protocols; the fill figure above also pays for writing back the fill's own dirty
    # lines, which leave the caches while the timed kernel runs
    for key, pick in (("after_read_sweep", lambda k: k["after_read_sweep_us"]["mean"]), ("back_to_back", lambda k: k["back_to_back_us"])):
        both = pick(kernels["dispatch_fp8_quant"]) + pick(kernels["combine"])
        result[f"dispatch_plus_combine_{key}_us"] = both
        result[f"dispatch_plus_combine_{key}_frac_of_8TBps"] = moved / both / 1e3 / HBM_PEAK_GBS
    if args.calibrate_copy:
        ident = torch.arange(rows, dtype=torch.int32, device=dev)
        for _ in range(5):
            ops.dispatch_copy(gd[:rows], None, None, ident.view(rows, 1), ident, rows)
        torch.cuda.synchronize()
    ws.destroy()
    del gd, grows, out_buf, q_pre, s_pre
    if not args.no_extra_shapes:
        result["decode"] = decode_kernels(torch, ops, cases, timer)
        result["rank_share"] = rank_share_kernels(torch, ops, cases, timer)
    if not args.no_megamoe:
        result["megamoe"] = megamoe_bench(torch, ops, timer, not args.no_cpu_baseline)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(x, idx, w, grads, cfg)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
