"""The generic benchmark protocol measured through the library: every preset's operation passes its correctness
check before and after timing and yields a complete version-1 `measured` record."""

import numpy as np
import pytest
import torch

from deepep_amd import ops, protocol_bench as pb
from oracle import combine as ocombine
from oracle import layout as olayout
from oracle import quant as oquant
from tests.gpu_util import bf16_bits, f32_bits, fp8_bits

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


ORACLE_CASES = [
    ("smoke", {}),
    ("smoke", dict(route="masked")),
    ("smoke", dict(route="duplicate")),
    ("smoke", dict(route="skew", world_size=2, tokens_per_rank=(31, 17))),
    ("smoke", dict(dtype="fp8", hidden=256, route="masked")),
    ("smoke", dict(dtype="fp8", hidden=384, route="duplicate", with_weights=False)),
    ("rank_share", dict(tokens_per_rank=(8,) * 64, hidden=512, route="skew")),
    ("rank_share", dict(tokens_per_rank=(5,) * 63 + (0,), hidden=256, route="balanced", dtype="bf16")),
    ("decode", dict(hidden=1024)),
]


@pytest.mark.parametrize("name,changes", ORACLE_CASES)
def test_protocol_workloads_against_the_oracle(name, changes):
    """The protocol's deterministic inputs through ElasticBuffer.dispatch / combine, compared with the CPU oracle (an
    independent check, as the reference pins its benchmark with its own oracle, tests/test_benchmark.py:314-336): rows,
    scales, weights and per-expert counts of rank 0's expert range bit for bit, then the combine of the dispatched rows."""
    from dataclasses import replace

    import deepep_amd
    from deepep_amd.utils import per_token_cast_back, per_token_cast_to_fp8

    w = replace(pb.PRESETS[name], **changes).validate()
    x, ids, weights = pb.make_inputs(w, torch)
    # the bulk tensors are the integer formulas (spot-checked here, fully in the CPU suite)
    assert tuple(ids[0].tolist()) == pb.route_for_token(w, 0, 0)
    per_rank = w.experts // w.world_size
    fp8 = w.dtype == "fp8"
    xd = x.cuda()
    payload = per_token_cast_to_fp8(xd) if fp8 else xd
    buffer = deepep_amd.ElasticBuffer(None, num_max_tokens_per_rank=max(1, max(w.tokens_per_rank)), hidden=w.hidden,
                                      num_topk=w.topk, rank=0, world_size=w.world_size, explicitly_destroy=True)
    try:
        recv, _, recv_w, handle, _ = buffer.dispatch(payload, topk_idx=ids.cuda(), topk_weights=weights.cuda() if w.with_weights else None,
                                                     num_experts=w.experts, num_qps=2)
        want = olayout.layout(ids.numpy(), w.experts, 0, per_rank)
        rows = want["num_rows"]
        assert handle.num_recv_tokens_per_expert_list == want["counts"].tolist()
        np.testing.assert_array_equal(handle.route_to_row.cpu().numpy(), want["route_to_row"])
        if fp8:
            codes, scales = oquant.cast_to_fp8_int(bf16_bits(x))
            assert recv[0].shape[0] == rows
            np.testing.assert_array_equal(fp8_bits(recv[0]), olayout.expand_rows(codes, want["row_to_route"], w.topk))
            np.testing.assert_array_equal(f32_bits(recv[1]), olayout.expand_rows(scales, want["row_to_route"], w.topk).view(np.uint32))
            rows_bf16 = per_token_cast_back(*recv)
            np.testing.assert_array_equal(bf16_bits(rows_bf16), oquant.cast_back(fp8_bits(recv[0]), recv[1].cpu().numpy()))
        else:
            assert recv.shape[0] == rows
            np.testing.assert_array_equal(bf16_bits(recv), olayout.expand_rows(bf16_bits(x), want["row_to_route"], w.topk))
            rows_bf16 = recv
        if w.with_weights:
            np.testing.assert_array_equal(f32_bits(recv_w), olayout.expand_weights(weights.numpy(), want["row_to_route"]).view(np.uint32))
        out, _, _ = buffer.combine(rows_bf16, handle)
        np.testing.assert_array_equal(bf16_bits(out), ocombine.combine(bf16_bits(rows_bf16), want["route_to_row"]))
    finally:
        buffer.destroy()
