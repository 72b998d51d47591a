#!/usr/bin/env python3
"""Headline benchmark: prefill dispatch + combine on one MI355X.

A step is one pass of the hot path over one synthetic batch at the prefill shape
(T=4096, H=7168, 256 experts, top-8 with Zipf(1.2) popularity, seed 0):
  layout (counts / prefix / stable permutation, with the host read-back of R that a fresh dispatch
  needs) -> FP8 e4m3 dispatch with the per-128 quantiser fused into the expand-permute ->
  combine of BF16 gradients N(0,1) [R,H] (the backward of dispatch).
`value` is the algorithmic HBM bytes of dispatch + combine per second of wall time of that step.
Prints ONE JSON line.
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

HBM_PEAK_GBS = 8000.0


def algorithmic_bytes(tokens, hidden, topk, rows):
    """Bytes each kernel must move (no padding, no re-reads)."""
    idx = tokens * topk * 8
    dispatch = tokens * hidden * 2 + tokens * topk * 4 + rows * hidden + rows * (hidden // 128) * 4 + rows * 4
    combine = rows * hidden * 2 + tokens * topk * 4 + tokens * hidden * 2
    layout = idx + 2 * tokens * topk * 4
    return dict(layout=layout, dispatch=dispatch, combine=combine)


def time_kernel(fn, iters, torch, head_start=None):
    """Average device time of `fn` in microseconds, HIP events on the stream the kernels run on.  `head_start`: the
    GPU is kept busy first (a spin kernel of about 2 ms where torch offers one, else fills of that tensor), so that
    the host queues launches meanwhile and a kernel shorter than its Python launch path is still timed back to back."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    if head_start is not None:
        if hasattr(torch.cuda, "_sleep"):
            torch.cuda._sleep(4_000_000)  # cycles; no memory traffic that the timed kernels would have to wait out
        else:
            for _ in range(8):
                head_start.zero_()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1000.0 / iters


def time_kernel_cold(fn, iters, torch, flush):
    """Per-launch device times with the caches flushed before every launch (a 256 MiB fill, the way the
    reference's flush_l2_cache does, deep_ep/utils/testing.py:27-35): mean / min / p50 / p95 in microseconds."""
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    fn()
    for start, stop in pairs:
        flush.zero_()
        start.record()
        fn()
        stop.record()
    torch.cuda.synchronize()
    times = sorted(a.elapsed_time(b) * 1000.0 for a, b in pairs)
    pick = lambda q: times[min(len(times) - 1, int(q * len(times)))]
    return dict(mean=sum(times) / len(times), min=times[0], p50=pick(0.5), p95=pick(0.95))


def cpu_baseline(x, idx, w, grads, cfg, nbytes):
    """The reference CPU path (torch CPU, all host threads) on the same inputs."""
    import torch

    from oracle import baseline

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    tokens = min(cfg["tokens"], 1024)  # bounded sample: the first 1024 tokens of the same batch
    xs, ids, ws = x[:tokens], idx[:tokens], w[:tokens]

    def step():
        counts, psum, r2row, r2route = baseline.layout(ids, cfg["experts"])
        baseline.dispatch_fp8(xs, ws, r2route, cfg["topk"])
        baseline.combine(grads[: r2route.numel()], r2row)
        return r2route.numel()

    rows = step()
    times = []
    for _ in range(5):
        t0 = time.perf_counter_ns()
        step()
        times.append((time.perf_counter_ns() - t0) / 1e9)
    mean = sum(times) / len(times)
    sample_bytes = algorithmic_bytes(tokens, cfg["hidden"], cfg["topk"], rows)
    moved = sample_bytes["dispatch"] + sample_bytes["combine"]
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return dict(
        value=moved / mean / 1e9,
        unit="GB/s",
        cores=cores,
        kind="port",
        sample=f"first {tokens} tokens of the same batch ({rows} rows), 1 warm-up + 5 timed passes, "
        f"mean {mean * 1e3:.1f} ms per pass, torch CPU {torch.get_num_threads()} threads, {model}",
    )


MFMA_PEAK_TFLOPS = 5000.0  # MI355X dense FP8 (the mixed FP8 x FP4 MFMA issues at the FP8 cadence)


def megamoe_bench(torch, ops, dev, iters):
    """W4A8 fused expert FFN for one EP64 rank's share: 64 source ranks x 256 tokens, 384 experts of which
    6 are local, top-8 uniform routing (about 2048 rows), H=7168, I=2048.  Random codes: the arithmetic
    does not depend on the values.  FLOPs = 2*R*H*2I + 2*R*I*H for the R rows that reach a local expert."""
    tokens, hidden, inter, experts, local, topk = 64 * 256, 7168, 2048, 384, 6, 8
    gen = torch.Generator().manual_seed(0)
    idx = torch.multinomial(torch.ones(tokens, experts), topk, generator=gen).to(torch.int32).to(dev)
    w = torch.softmax(torch.randn(tokens, topk, generator=gen), -1).to(dev)
    x_codes = torch.randint(0, 120, (tokens, hidden), dtype=torch.uint8, generator=gen).to(dev).view(torch.float8_e4m3fn)
    x_scales = torch.full((tokens, hidden // 32), 127, dtype=torch.uint8, device=dev)
    # Three weight sets used in turn (3 x 132 MB, more than the 256 MB memory-side cache), so that the GEMMs
    # stream their weights from HBM as they do between the layers of a model.
    sets = []
    for _ in range(3):
        w1 = torch.randint(0, 256, (local, 2 * inter, hidden // 2), dtype=torch.uint8, device=dev)
        s1 = torch.full((local, 2 * inter, ops.megamoe_prepared_scale_cols(hidden)), 119, dtype=torch.uint8, device=dev)
        w2 = torch.randint(0, 256, (local, hidden, inter // 2), dtype=torch.uint8, device=dev)
        s2 = torch.full((local, hidden, ops.megamoe_prepared_scale_cols(inter)), 119, dtype=torch.uint8, device=dev)
        sets.append((w1, s1, w2, s2))
    ws = ops.Workspace(ops.megamoe_workspace_bytes(tokens, topk, hidden, inter, local))
    y = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)
    counts = torch.empty((local,), dtype=torch.int32, device=dev)
    calls = [0]

    def run():
        w1, s1, w2, s2 = sets[calls[0] % len(sets)]
        calls[0] += 1
        ops.megamoe_forward(ws, x_codes, x_scales, idx, w, w1, s1, w2, s2, experts, 0, local, y, counts)

    us = time_kernel(run, iters, torch)
    rows = int(counts.sum().item())
    flops = 2.0 * rows * hidden * 2 * inter + 2.0 * rows * inter * hidden
    ws.destroy()
    return {
        "workload": "EP64 rank share: 16384 candidate tokens, 6 of 384 experts local, top-8, H=7168, I=2048, "
        "MXFP8 activations x MXFP4 weights, three weight sets in turn; layout + GMM1(+SwiGLU+requant) + GMM2 + "
        "weighted reduce",
        "rows": rows,
        "us_forward": us,
        "gflop": flops / 1e9,
        "tflops_forward": flops / us / 1e6,
        "roofline": {"bound": "mfma", "achieved": flops / us / 1e6, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops / us / 1e6 / MFMA_PEAK_TFLOPS,
                     "note": "whole forward (4 launches); per-kernel GEMM times are in profiles/"},
    }


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=10)
    parser.add_argument("--kernel-iters", type=int, default=50)
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-megamoe", action="store_true", help="skip the W4A8 expert-FFN measurement")
    parser.add_argument("--calibrate-copy", action="store_true",
                        help="also launch a plain copy of known size (identity dispatch of [32768,7168] BF16: 469.76 MB "
                        "read + 469.76 MB written) so that rocprofv3 FETCH_SIZE / WRITE_SIZE can be scaled")
    args = parser.parse_args()
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
    t0 = time.perf_counter()
    for _ in range(args.steps):
        rows, _, _ = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    nbytes = algorithmic_bytes(tokens, hidden, topk, rows)
    moved = nbytes["dispatch"] + nbytes["combine"]

    # Per-kernel device time (HIP events on the launch stream), same inputs.
    lay = ops.layout(ws, idxd, experts)
    r2row, r2route = lay["route_to_row"], lay["row_to_route"]
    grows = gd[:rows]
    out_buf = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)
    it = args.kernel_iters
    recv_w = ops.dispatch_quant_fp8(xd, wd, r2row, r2route, rows)[2]
    head_start = torch.empty(1 << 30, dtype=torch.uint8, device=dev)  # 8 fills of 1 GiB: about 1.4 ms
    us = dict(
        layout=time_kernel(lambda: ops.layout(ws, idxd, experts), min(it, 40), torch, head_start),
        dispatch_fp8_quant=time_kernel(lambda: ops.dispatch_quant_fp8(xd, wd, r2row, r2route, rows), it, torch),
        dispatch_bf16=time_kernel(lambda: ops.dispatch_copy(xd, None, wd, r2row, r2route, rows), it, torch),
        combine=time_kernel(lambda: ops.combine(grows, r2row, out=out_buf), it, torch),
        combine_weighted=time_kernel(lambda: ops.combine(grows, r2row, recv_w, out=out_buf), it, torch),
    )
    del head_start
    flush = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
    cold = dict(
        dispatch_fp8_quant=time_kernel_cold(lambda: ops.dispatch_quant_fp8(xd, wd, r2row, r2route, rows), 30, torch, flush),
        combine=time_kernel_cold(lambda: ops.combine(grows, r2row, out=out_buf), 30, torch, flush),
    )
    del flush
    bf16_dispatch_bytes = tokens * hidden * 2 + tokens * topk * 4 + rows * hidden * 2 + rows * 4
    kernels = {
        "layout": dict(us=us["layout"], bytes=nbytes["layout"]),
        "dispatch_fp8_quant": dict(us=us["dispatch_fp8_quant"], bytes=nbytes["dispatch"]),
        "dispatch_bf16": dict(us=us["dispatch_bf16"], bytes=bf16_dispatch_bytes),
        "combine": dict(us=us["combine"], bytes=nbytes["combine"]),
        "combine_weighted": dict(us=us["combine_weighted"], bytes=nbytes["combine"] + rows * 4),
    }
    for entry in kernels.values():
        entry["GBps"] = entry["bytes"] / entry["us"] / 1e3
        entry["frac_of_8TBps"] = entry["GBps"] / HBM_PEAK_GBS

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
        },
        "roofline": {
            "kernel": "combine_kernel<0, false>",
            "bound": "hbm",
            "achieved": dominant["GBps"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": dominant["GBps"] / HBM_PEAK_GBS,
            # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a plain copy of known
            # size (factors 1.991 / 1.000): 468.7 MB read + 58.7 MB written (profiles/prefill_hbm_traffic_pmc.md)
            "traffic": 527.5e6,
        },
        "kernels": kernels,
        "kernels_cache_flushed_us": cold,
        "dispatch_plus_combine_us": us["dispatch_fp8_quant"] + us["combine"],
    }
    if args.calibrate_copy:
        ident = torch.arange(rows, dtype=torch.int32, device=dev)
        for _ in range(5):
            ops.dispatch_copy(gd[:rows], None, None, ident.view(rows, 1), ident, rows)
        torch.cuda.synchronize()
    if not args.no_megamoe:
        result["megamoe"] = megamoe_bench(torch, ops, dev, args.kernel_iters)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(x, idx, w, grads, cfg, nbytes)
    ws.destroy()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
