"""The reference's generic benchmark protocol through this library, on one GPU.

Restates what a native adapter has to share with the reference's framework-free planner (benchmarks/_config.py):
the workload description and its limits (:14-93), the deterministic inputs ``route_for_token`` / ``hidden_value`` /
``weight_value`` (:149-167), the logical byte count ``traffic`` (:170-206), the rank aggregation of latency samples
(benchmarks/_utils.py:68-88) and the version-1 result record (benchmarks/results/README.md).  ``run`` measures a
workload with ``ElasticBuffer`` under the reference's timing boundary (host call to device output ready,
``perf_counter_ns``, reused inputs, no cache flush; _utils.py:17-42) and returns ``measured`` records.

One GPU holds one rank's receive share.  With ``world_size`` 1 the measured workload is the configured one.  With more
ranks the tokens of all source ranks are flattened (rank-major) and rank 0's share is measured: the record keeps the
reference's aggregate ``traffic`` for the configuration and states the share's own bytes, which the bandwidth uses.
"""

from __future__ import annotations

import hashlib
import json
import math
import statistics
import time
from dataclasses import asdict, dataclass, replace
from datetime import datetime, timezone

SCHEMA_VERSION = 1


@dataclass(frozen=True)
class Workload:
    """Fields, defaults and limits of the reference's ``Config`` (the ones the expanded elastic path uses)."""

    api: str = "elastic"
    operation: str = "dispatch"      # dispatch | combine | roundtrip
    dtype: str = "bf16"              # dispatch input; combine always receives BF16
    layout: str = "expanded"
    dispatch_mode: str = "fresh"     # fresh | cached
    world_size: int = 1
    tokens_per_rank: tuple = (31,)
    hidden: int = 256
    topk: int = 2
    experts: int = 8
    alignment: int = 1
    with_weights: bool = True
    route: str = "balanced"          # balanced | skew | masked | duplicate
    seed: int = 0
    warmup: int = 10
    iterations: int = 50

    def validate(self) -> "Workload":
        allowed = dict(api=("elastic",), operation=("dispatch", "combine", "roundtrip"), dtype=("bf16", "fp8"),
                       layout=("expanded",), dispatch_mode=("fresh", "cached"),
                       route=("balanced", "skew", "masked", "duplicate"))
        for name, values in allowed.items():
            if getattr(self, name) not in values:
                raise ValueError(f"{name} must be one of {values}")
        ranges = dict(world_size=(1, 1024), hidden=(1, 65536), topk=(1, 256), experts=(1, 65536), seed=(0, 2**31 - 1),
                      warmup=(0, 10000), iterations=(1, 10000), alignment=(1, 1))
        for name, (low, high) in ranges.items():
            value = getattr(self, name)
            if type(value) is not int or not low <= value <= high:
                raise ValueError(f"{name} must be an integer in [{low}, {high}]")
        if type(self.with_weights) is not bool:
            raise ValueError("with_weights must be boolean")
        counts = self.tokens_per_rank
        if not isinstance(counts, (list, tuple)) or len(counts) != self.world_size or any(
            type(t) is not int or not 0 <= t <= 1048576 for t in counts
        ):
            raise ValueError("tokens_per_rank must contain one nonnegative integer per rank")
        if not 1 <= sum(counts) <= 1048576:
            raise ValueError("total tokens must be in [1, 1048576]")
        if self.experts % self.world_size or self.topk > self.experts:
            raise ValueError("experts must divide across ranks and topk must not exceed experts")
        if self.dtype == "fp8" and self.hidden % 128:
            raise ValueError("FP8 per-128-column scaling requires hidden divisible by 128")
        if self.operation == "combine" and self.dispatch_mode == "cached":
            raise ValueError("dispatch_mode=cached applies to dispatch or roundtrip")
        return self

    def to_dict(self) -> dict:
        fields = asdict(self)
        fields["tokens_per_rank"] = list(self.tokens_per_rank)
        return fields

    def fingerprint(self) -> str:
        return hashlib.sha256(json.dumps(self.to_dict(), sort_keys=True).encode()).hexdigest()

    def required_capabilities(self) -> list:
        needs = {self.api, "dispatch", self.layout, self.dtype, "route_" + self.route}
        if self.operation != "dispatch":
            needs.add("combine")
        if self.operation == "roundtrip":
            needs.add("roundtrip")
        if self.dispatch_mode == "cached":
            needs.add("cached")
        if len(set(self.tokens_per_rank)) > 1:
            needs.add("unequal_tokens")
        if 0 in self.tokens_per_rank:
            needs.add("zero_tokens")
        if self.world_size == 1:
            needs.add("single_rank")
        if self.with_weights:
            needs.add("weights")
        return sorted(needs)


PRESETS = {
    # the reference's smoke workload (benchmarks/configs/smoke.json) on one rank, and this build's headline shapes
    "smoke": Workload(tokens_per_rank=(31,), hidden=256, topk=2, experts=8),
    "decode": Workload(operation="roundtrip", tokens_per_rank=(128,), hidden=7168, topk=8, experts=256, iterations=100, warmup=20),
    "prefill": Workload(operation="roundtrip", dtype="fp8", tokens_per_rank=(4096,), hidden=7168, topk=8, experts=256,
                        iterations=100, warmup=20),
    "rank_share": Workload(operation="roundtrip", dtype="fp8", world_size=64, tokens_per_rank=(256,) * 64, hidden=7168, topk=8,
                           experts=384, iterations=100, warmup=20),
}


# ---- deterministic inputs (integer formulas shared with the reference's planner) -----------------------------------
def route_for_token(w: Workload, rank: int, token: int) -> tuple:
    ids = [(w.seed + rank * 17 + token * 7 + slot) % w.experts for slot in range(w.topk)]
    if w.route == "skew":
        ids = [e % (w.experts // w.world_size) for e in ids]
    elif w.route == "duplicate" and w.topk > 1:
        ids[1] = ids[0]
    elif w.route == "masked":
        ids = [-1 if (w.seed + rank + token + slot) % 5 == 0 else e for slot, e in enumerate(ids)]
    return tuple(ids)


def hidden_value(w: Workload, rank: int, token: int, column: int) -> float:
    """Exactly BF16-representable."""
    return ((w.seed + rank * 13 + token * 7 + column) % 127 - 63) / 16.0


def weight_value(w: Workload, rank: int, token: int, slot: int) -> float:
    return ((w.seed + rank * 19 + token * 7 + slot * 3) % 127) / 128.0


def traffic(w: Workload, receiver=None) -> dict:
    """Useful payload bytes (rows x hidden x element size; no scales, indices, weights or padding), per source rank and
    in total for the selected operation.  ``receiver``: count only the rows that go to that rank's experts."""
    w.validate()
    per_rank = w.experts // w.world_size
    rows = []
    for rank, tokens in enumerate(w.tokens_per_rank):
        count = 0
        for token in range(tokens):
            for expert in route_for_token(w, rank, token):
                if expert >= 0 and (receiver is None or expert // per_rank == receiver):
                    count += 1
        rows.append(count)
    forward = [n * w.hidden * (1 if w.dtype == "fp8" else 2) for n in rows]
    backward = [n * w.hidden * 2 for n in rows]
    chosen = dict(dispatch=forward, combine=backward, roundtrip=[a + b for a, b in zip(forward, backward)])[w.operation]
    return {
        "definition": "aggregate_useful_hidden_payload_bytes_v1",
        "includes": ["local_routes", "valid_route_multiplicity"],
        "excludes": ["padding", "fp8_scales", "indices", "weights", "protocol", "link_retransmission"],
        "rows_per_source_rank": rows,
        "dispatch_bytes_per_source_rank": forward,
        "combine_bytes_per_source_rank": backward,
        "effective_bytes": sum(chosen),
    }


def aggregate_samples(samples, world_size: int, iterations: int):
    """Rank-major, iteration-aligned samples -> (per-iteration maximum over ranks, statistics of those maxima;
    nearest-rank percentiles)."""
    if type(world_size) is not int or type(iterations) is not int or min(world_size, iterations) < 1:
        raise ValueError("world_size and iterations must be positive integers")
    if not isinstance(samples, (tuple, list)) or len(samples) != world_size:
        raise ValueError("incomplete rank samples")
    for row in samples:
        if not isinstance(row, (tuple, list)) or len(row) != iterations:
            raise ValueError("incomplete iteration samples")
        if any(type(v) not in (int, float) or not math.isfinite(v) or v <= 0 for v in row):
            raise ValueError("latency samples must be finite and positive")
    slowest = [max(column) for column in zip(*samples)]
    ranked = sorted(slowest)
    nearest = lambda q: ranked[math.ceil(iterations * q) - 1]
    return slowest, {
        "latency_mean_us": statistics.fmean(slowest),
        "latency_min_us": ranked[0],
        "latency_max_us": ranked[-1],
        "latency_p50_us": nearest(0.50),
        "latency_p95_us": nearest(0.95),
    }


TIMING = {
    "clock": "perf_counter_ns",
    "boundary": "host_call_to_device_output_ready",
    "includes": ["host_api", "allocation_in_api", "notify_for_fresh_dispatch", "completion_wait"],
    "excludes": ["input_generation", "correctness", "pre_iteration_barrier", "sample_gather", "output_release"],
    "rank_aggregation": "max_per_iteration_then_statistics",
    "percentile": "nearest_rank",
    "cache_policy": "reused_inputs_no_explicit_cache_flush",
    "roundtrip": "direct_dispatch_to_matching_handle_combine_no_expert_compute",
    "roundtrip_fp8": "received_fp8_to_bf16_conversion_included",
    "combine": "matching_handle_and_bf16_input_prepared_before_timing",
}


# ---- the measured side --------------------------------------------------------------------------------------------
def make_inputs(w: Workload, torch):
    """The workload's tensors (all source ranks flattened, rank-major), built from the integer formulas in bulk."""
    ranks = torch.cat([torch.full((n,), r, dtype=torch.int64) for r, n in enumerate(w.tokens_per_rank)])
    tokens = torch.cat([torch.arange(n, dtype=torch.int64) for n in w.tokens_per_rank])
    slots = torch.arange(w.topk, dtype=torch.int64)
    ids = (w.seed + ranks[:, None] * 17 + tokens[:, None] * 7 + slots[None, :]) % w.experts
    if w.route == "skew":
        ids = ids % (w.experts // w.world_size)
    elif w.route == "duplicate" and w.topk > 1:
        ids[:, 1] = ids[:, 0]
    elif w.route == "masked":
        ids = torch.where((w.seed + ranks[:, None] + tokens[:, None] + slots[None, :]) % 5 == 0, torch.full_like(ids, -1), ids)
    columns = torch.arange(w.hidden, dtype=torch.int64)
    x = (((w.seed + ranks[:, None] * 13 + tokens[:, None] * 7 + columns[None, :]) % 127 - 63).float() / 16.0).bfloat16()
    weights = ((w.seed + ranks[:, None] * 19 + tokens[:, None] * 7 + slots[None, :] * 3) % 127).float() / 128.0
    return x, ids, weights


def run(preset, torch, ops, iters=None, warmups=None, revision="0" * 40):
    """Measures the named preset (or a ``Workload``) on the current GPU; returns a list with one ``measured`` record."""
    import deepep_amd
    from deepep_amd.utils import per_token_cast_back, per_token_cast_to_fp8

    w = PRESETS[preset] if isinstance(preset, str) else preset
    if iters is not None:
        w = replace(w, iterations=iters)
    if warmups is not None:
        w = replace(w, warmup=warmups)
    w.validate()
    x, ids, weights = make_inputs(w, torch)
    x, ids, weights = x.cuda(), ids.cuda(), weights.cuda()
    fp8 = w.dtype == "fp8"
    payload = per_token_cast_to_fp8(x) if fp8 else x
    total = sum(w.tokens_per_rank)
    buffer = deepep_amd.ElasticBuffer(None, num_max_tokens_per_rank=min(16384, max(w.tokens_per_rank)), hidden=w.hidden,
                                      num_topk=w.topk, rank=0, world_size=w.world_size, explicitly_destroy=True)
    per_rank = w.experts // w.world_size
    try:
        def dispatch(handle=None):
            # (num_qps=2, the high-throughput path's own value, keeps small batches on EP16+ off the low-latency path,
            # which the protocol does not measure)
            return buffer.dispatch(payload, topk_idx=None if handle is not None else ids,
                                   topk_weights=weights if w.with_weights else None, num_experts=w.experts, handle=handle,
                                   num_qps=2)

        def verify():
            recv, _, recv_w, handle, _ = dispatch()
            local = (ids >= 0) & (ids < per_rank)  # rank 0 owns experts [0, E / world)
            order = torch.sort(torch.where(local, ids, torch.full_like(ids, w.experts)).flatten(), stable=True)
            routes = order.indices[: int(local.sum().item())]
            source = payload if not fp8 else payload[0]
            got = recv if not fp8 else recv[0]
            if got.shape[0] != routes.numel() or not torch.equal(got.view(torch.uint8), source[routes // w.topk].view(torch.uint8)):
                raise RuntimeError("dispatch rows differ from the expanded layout of the deterministic inputs")
            if w.with_weights and not torch.equal(recv_w, weights.flatten()[routes]):
                raise RuntimeError("dispatched weights differ")
            rows = per_token_cast_back(*recv) if fp8 else recv
            out, _, _ = buffer.combine(rows, handle)
            want = torch.zeros((total, w.hidden), dtype=torch.float32, device=x.device)
            for slot in range(w.topk):  # slot order, fp32, one rounding
                hit = local[:, slot]
                want[hit] += rows[handle.route_to_row[:, slot][hit].long()].float()
            if not torch.equal(out, want.bfloat16()):
                raise RuntimeError("combine differs from the slot-ordered fp32 sum")
            return handle, rows

        handle, rows = verify()
        if w.dispatch_mode == "cached":
            operation = {"dispatch": lambda: dispatch(handle),
                         "roundtrip": lambda: buffer.combine(_bf16_rows(dispatch(handle)[0], fp8, per_token_cast_back), handle)}[w.operation]
        else:
            def fresh_roundtrip():
                recv, _, _, fresh, _ = dispatch()
                return buffer.combine(_bf16_rows(recv, fp8, per_token_cast_back), fresh)

            operation = {"dispatch": dispatch, "combine": lambda: buffer.combine(rows, handle), "roundtrip": fresh_roundtrip}[w.operation]
        samples = []
        for iteration in range(w.warmup + w.iterations):
            torch.cuda.synchronize()
            start = time.perf_counter_ns()
            result = operation()
            torch.cuda.synchronize()
            elapsed = (time.perf_counter_ns() - start) / 1000.0
            del result
            if iteration >= w.warmup:
                samples.append(elapsed)
        verify()
    finally:
        buffer.destroy()
    slowest, stats = aggregate_samples([samples], 1, w.iterations)
    share = traffic(w, receiver=0)
    stats["bandwidth_gbps"] = share["effective_bytes"] / stats["latency_mean_us"] / 1e3
    stats["bandwidth_statistic"] = "share_effective_bytes_over_mean_latency"
    return [{
        "schema_version": SCHEMA_VERSION,
        "status": "measured",
        "config": w.to_dict(),
        "config_fingerprint": w.fingerprint(),
        "required_capabilities": w.required_capabilities(),
        "timing": dict(TIMING),
        "traffic": traffic(w),
        "measured_share": {"receiver_rank": 0, "of_world_size": w.world_size, "rows": sum(share["rows_per_source_rank"]),
                           "effective_bytes": share["effective_bytes"]},
        "correctness_result": "passed_pre_and_post",
        "revision": revision,
        "measured_at": datetime.now(timezone.utc).isoformat(),
        "metadata": {"backend": "deepep_amd", "device": torch.cuda.get_device_name(0), "software": f"torch {torch.__version__}",
                     "topology": "1 GPU", "variant": "rank 0's receive share on one GPU" if w.world_size > 1 else "single rank"},
        "rank_samples_us": [samples],
        "rank_max_samples_us": slowest,
        "statistics": stats,
    }]


def _bf16_rows(recv, fp8, cast_back):
    return cast_back(*recv) if fp8 else recv
