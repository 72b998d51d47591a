"""ElasticBuffer.dispatch / combine at seeded random shapes against the CPU oracle, bit for bit: token counts from 1 up,
widths that are no multiple of 128, masked routes (-1), expert ranges inside [0, E), with and without weights,
BF16 payloads, FP8 payloads with their scales and BF16 payloads quantised by the dispatch itself, then a second payload
over the cached routing."""

import numpy as np
import pytest
import torch

from oracle import combine as ocombine
from oracle import layout as olayout
from oracle import quant as oquant
from tests.gpu_util import bf16_bits, f32_bits, fp8_bits

pytestmark = pytest.mark.gpu


def _draw(seed):
    rng = np.random.default_rng(7000 + seed)
    world = int(rng.choice([1, 2, 4, 8]))
    per_rank = int(rng.choice([1, 2, 3, 8, 32]))
    experts = world * per_rank
    rank = int(rng.integers(0, world))
    topk = int(rng.integers(1, min(experts, 8) + 1))
    tokens = int(rng.choice([1, 2, 5, 64, 129, 300, 1000]))
    mode = str(rng.choice(["bf16", "fp8", "fused"]))  # fp8: (codes, scales) in; fused: BF16 in, quantised by the dispatch
    fp8 = mode != "bf16"
    hidden = int(rng.choice([128, 256, 384, 1024, 7168])) if fp8 else int(rng.choice([16, 64, 208, 1008, 4096]))
    masked = float(rng.choice([0.0, 0.2, 0.9]))
    with_weights = bool(rng.integers(0, 2))
    return world, rank, experts, topk, tokens, mode, hidden, masked, with_weights


@pytest.mark.parametrize("seed", range(96))
def test_dispatch_and_combine_at_random_shapes(seed):
    import deepep_amd
    from deepep_amd.utils import per_token_cast_to_fp8

    world, rank, experts, topk, tokens, mode, hidden, masked, with_weights = _draw(seed)
    fp8 = mode != "bf16"
    case = dict(world=world, rank=rank, experts=experts, topk=topk, tokens=tokens, mode=mode, hidden=hidden, masked=masked,
                with_weights=with_weights)
    print(case, flush=True)
    rng = np.random.default_rng(seed)
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int64) if tokens else np.zeros((0, topk), np.int64)
    ids[rng.random(ids.shape) < masked] = -1
    x = torch.from_numpy(rng.normal(size=(tokens, hidden)).astype(np.float32) * 3).bfloat16()
    weights = torch.from_numpy(rng.random((tokens, topk)).astype(np.float32))
    per_rank = experts // world
    xd = x.cuda()
    payload = per_token_cast_to_fp8(xd) if mode == "fp8" else xd
    buffer = deepep_amd.ElasticBuffer(None, num_max_tokens_per_rank=max(1, tokens), hidden=hidden, num_topk=topk, rank=rank,
                                      world_size=world, use_fp8_dispatch=mode == "fused", explicitly_destroy=True)
    try:
        recv, _, recv_w, handle, _ = buffer.dispatch(payload, topk_idx=torch.from_numpy(ids).cuda(),
                                                     topk_weights=weights.cuda() if with_weights else None, num_experts=experts)
        want = olayout.layout(ids, experts, rank * per_rank, per_rank)
        rows = want["num_rows"]
        assert handle.num_recv_tokens_per_expert_list == want["counts"].tolist(), case
        np.testing.assert_array_equal(handle.route_to_row.cpu().numpy(), want["route_to_row"], err_msg=str(case))
        if fp8:
            codes, scales = oquant.cast_to_fp8_int(bf16_bits(x))
            assert recv[0].shape[0] == rows
            np.testing.assert_array_equal(fp8_bits(recv[0]), olayout.expand_rows(codes, want["row_to_route"], topk), err_msg=str(case))
            np.testing.assert_array_equal(f32_bits(recv[1]), olayout.expand_rows(scales, want["row_to_route"], topk).view(np.uint32),
                                          err_msg=str(case))
        else:
            assert recv.shape[0] == rows
            np.testing.assert_array_equal(bf16_bits(recv), olayout.expand_rows(bf16_bits(x), want["row_to_route"], topk), err_msg=str(case))
        if with_weights:
            np.testing.assert_array_equal(f32_bits(recv_w), olayout.expand_weights(weights.numpy(), want["row_to_route"]).view(np.uint32),
                                          err_msg=str(case))
        # a second payload over the cached routing
        x2 = torch.from_numpy(rng.normal(size=(tokens, hidden)).astype(np.float32)).bfloat16()
        payload2 = per_token_cast_to_fp8(x2.cuda()) if mode == "fp8" else x2.cuda()
        again, _, again_w, handle2, _ = buffer.dispatch(payload2, handle=handle, topk_weights=weights.cuda() if with_weights else None)
        assert handle2.num_recv_tokens_per_expert_list == want["counts"].tolist(), case
        if fp8:
            codes2, scales2 = oquant.cast_to_fp8_int(bf16_bits(x2))
            np.testing.assert_array_equal(fp8_bits(again[0]), olayout.expand_rows(codes2, want["row_to_route"], topk), err_msg=str(case))
            np.testing.assert_array_equal(f32_bits(again[1]), olayout.expand_rows(scales2, want["row_to_route"], topk).view(np.uint32),
                                          err_msg=str(case))
        else:
            np.testing.assert_array_equal(bf16_bits(again), olayout.expand_rows(bf16_bits(x2), want["row_to_route"], topk), err_msg=str(case))
        if with_weights:
            np.testing.assert_array_equal(f32_bits(again_w), f32_bits(recv_w), err_msg=str(case))
        # combine rows of its own (expert outputs): unweighted sum in slot order; the dispatched weights come back on
        # the return channel as [T, K], 0 where a route has no row
        y = torch.from_numpy(rng.normal(size=(rows, hidden)).astype(np.float32)).bfloat16()
        out, out_w, _ = buffer.combine(y.cuda(), handle, topk_weights=recv_w if with_weights else None)
        np.testing.assert_array_equal(bf16_bits(out), ocombine.combine(bf16_bits(y), want["route_to_row"]), err_msg=str(case))
        if with_weights:
            local_route = want["route_to_row"] >= 0
            np.testing.assert_array_equal(f32_bits(out_w), np.where(local_route, weights.numpy(), np.float32(0)).view(np.uint32),
                                          err_msg=str(case))
    finally:
        buffer.destroy()
