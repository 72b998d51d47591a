"""The generic benchmark protocol restated in deepep_amd/protocol_bench.py, pinned by the reference's own checks
(tests/test_benchmark.py:314-352): logical bytes against an independent count of the expanded layout's rows, the fixed
values of the deterministic input formulas, rank maxima taken before percentiles, nearest-rank percentiles."""

import itertools
from dataclasses import replace

import numpy as np
import pytest

from deepep_amd import protocol_bench as pb
from oracle import layout as olayout


@pytest.mark.parametrize("route,operation,dtype", itertools.product(["balanced", "skew", "duplicate", "masked"],
                                                                    ["dispatch", "combine", "roundtrip"], ["bf16", "fp8"]))
def test_bytes_match_independent_route_reference(route, operation, dtype):
    w = pb.Workload(route=route, operation=operation, dtype=dtype, world_size=2, tokens_per_rank=(3, 0), topk=4)
    # rows of the expanded layout, counted by the layout oracle over both ranks' experts instead of by traffic()'s loop
    ids = np.array([pb.route_for_token(w, r, t) for r, n in enumerate(w.tokens_per_rank) for t in range(n)], dtype=np.int64)
    rows = sum(olayout.layout(ids, w.experts, rank * 4, 4)["num_rows"] for rank in range(2))
    forward = rows * w.hidden * (1 if dtype == "fp8" else 2)
    backward = rows * w.hidden * 2
    assert pb.traffic(w)["effective_bytes"] == dict(dispatch=forward, combine=backward, roundtrip=forward + backward)[operation]
    share = sum(pb.traffic(w, receiver=r)["effective_bytes"] for r in range(2))
    assert share == pb.traffic(w)["effective_bytes"]


def test_fixed_values_of_the_input_formulas():  # tests/test_benchmark.py:338-344
    w = pb.Workload(world_size=2, tokens_per_rank=(1, 0), topk=2, route="duplicate", hidden=256)
    assert pb.traffic(w)["effective_bytes"] == 1024  # duplicate slots are separate rows in the expanded layout
    assert pb.route_for_token(w, 0, 0) == (0, 0)
    assert pb.hidden_value(w, 0, 0, 0) == -63 / 16
    assert pb.weight_value(w, 1, 0, 0) == 19 / 128
    masked = replace(w, route="masked", topk=4, tokens_per_rank=(4, 0))
    assert pb.route_for_token(masked, 0, 0)[0] == -1 and -1 not in pb.route_for_token(masked, 0, 1)  # (0+0+t+slot) % 5 == 0


def test_rank_max_is_taken_before_percentiles():  # tests/test_benchmark.py:347-352
    maxima, stats = pb.aggregate_samples([[100, 1], [1, 100]], 2, 2)
    assert maxima == [100, 100]
    assert stats["latency_mean_us"] == stats["latency_p50_us"] == 100
    _, stats = pb.aggregate_samples([list(range(1, 21))], 1, 20)
    assert stats["latency_p50_us"] == 10 and stats["latency_p95_us"] == 19
    with pytest.raises(ValueError):
        pb.aggregate_samples([[1.0, float("nan")]], 1, 2)
    with pytest.raises(ValueError):
        pb.aggregate_samples([[1.0]], 1, 2)


def test_bulk_inputs_equal_the_scalar_formulas():
    import torch

    for route in ("balanced", "skew", "duplicate", "masked"):
        w = pb.Workload(route=route, world_size=2, tokens_per_rank=(5, 3), topk=3, experts=8, hidden=128, seed=11)
        x, ids, weights = pb.make_inputs(w, torch)
        at = 0
        for rank, count in enumerate(w.tokens_per_rank):
            for token in range(count):
                assert tuple(ids[at].tolist()) == pb.route_for_token(w, rank, token)
                assert x[at, 5].item() == pb.hidden_value(w, rank, token, 5) and x[at, 127].item() == pb.hidden_value(w, rank, token, 127)
                assert weights[at, 2].item() == np.float32(pb.weight_value(w, rank, token, 2))
                at += 1


def test_workload_limits_and_fingerprint():
    w = pb.PRESETS["smoke"].validate()
    assert len(w.fingerprint()) == 64 and "single_rank" in w.required_capabilities()
    for bad in (dict(operation="scatter"), dict(hidden=0), dict(tokens_per_rank=(1, 2)), dict(dtype="fp8", hidden=192),
                dict(experts=7, world_size=2, tokens_per_rank=(1, 1)), dict(operation="combine", dispatch_mode="cached")):
        with pytest.raises(ValueError):
            replace(w, **bad).validate()
    for name in pb.PRESETS:
        pb.PRESETS[name].validate()
