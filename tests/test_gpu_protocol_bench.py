"""The generic benchmark protocol measured through the library: every preset's operation passes its correctness
check before and after timing and yields a complete version-1 `measured` record."""

import pytest
import torch

from deepep_amd import ops, protocol_bench as pb

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,changes", [
    ("smoke", {}),
    ("smoke", dict(operation="roundtrip", route="masked", dispatch_mode="cached")),
    ("smoke", dict(operation="combine", route="duplicate", dtype="fp8", hidden=256)),
    ("rank_share", dict(tokens_per_rank=(8,) * 64, hidden=512, route="skew")),
])
def test_protocol_records(name, changes):
    from dataclasses import replace

    workload = replace(pb.PRESETS[name], iterations=3, warmup=1, **changes)
    (record,) = pb.run(workload, torch, ops)
    assert record["schema_version"] == 1 and record["status"] == "measured"
    assert record["correctness_result"] == "passed_pre_and_post"
    assert record["config_fingerprint"] == workload.fingerprint()
    assert len(record["rank_samples_us"][0]) == 3 == len(record["rank_max_samples_us"])
    stats = record["statistics"]
    assert stats["latency_min_us"] <= stats["latency_p50_us"] <= stats["latency_max_us"]
    assert record["measured_share"]["effective_bytes"] <= record["traffic"]["effective_bytes"]
    assert stats["bandwidth_gbps"] > 0 or record["measured_share"]["effective_bytes"] == 0
