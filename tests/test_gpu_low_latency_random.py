"""The low-latency dispatch / combine of one rank's share at seeded random shapes against the CPU oracle, bit for bit:
world sizes 16..64, batches below and above the one-launch limit, capacities at and above the batch, BF16 / FP16 / FP8
payloads (FP32 or packed int32 scales), and top-k below and above the number of experts per rank."""

import numpy as np
import pytest
import torch

from oracle import combine as ocombine
from oracle import layout as olayout
from tests.gpu_util import bf16_bits

pytestmark = pytest.mark.gpu


def _draw(seed):
    rng = np.random.default_rng(9000 + seed)
    world = int(rng.choice([16, 32, 64]))
    local = int(rng.choice([1, 2, 4, 16]))
    experts = world * local
    rank = int(rng.integers(0, world))
    topk = int(rng.integers(1, 9))
    per_rank = int(rng.choice([1, 2, 7, 16, 40]))
    capacity = per_rank + int(rng.choice([0, 0, 3, 24]))
    payload = str(rng.choice(["bfloat16", "float16", "fp8_float32", "fp8_int32"]))
    hidden = int(rng.choice([128, 512, 1024, 7168])) if payload.startswith("fp8") else int(rng.choice([8, 136, 1024, 7168]))
    return world, rank, experts, topk, per_rank, capacity, payload, hidden


@pytest.mark.parametrize("seed", range(32))
def test_low_latency_share_at_random_shapes(seed):
    import deepep_amd

    world, rank, experts, topk, per_rank, capacity, payload, hidden = _draw(seed)
    case = dict(world=world, rank=rank, experts=experts, topk=topk, per_rank=per_rank, capacity=capacity, payload=payload, hidden=hidden)
    print(case, flush=True)
    rng = np.random.default_rng(seed)
    tokens, local = world * per_rank, experts // world
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int64)  # no expert twice per token
    weights = rng.random((tokens, topk)).astype(np.float32)
    values = torch.from_numpy((rng.normal(size=(tokens, hidden)) * 2).astype(np.float32))
    fp8 = payload.startswith("fp8")
    if fp8:
        codes = values.to(torch.float8_e4m3fn)
        words = rng.integers(0x30000000, 0x48000000, size=(tokens, hidden // 128), dtype=np.int64).astype(np.int32)
        scales = torch.from_numpy(words) if payload.endswith("int32") else torch.from_numpy(words).view(torch.float32)
        x = (codes.cuda(), scales.cuda())
    else:
        x = values.to(getattr(torch, payload)).cuda()
    capacity_rows = world * capacity * min(topk, local)
    buffer = deepep_amd.ElasticBuffer(None, num_bytes=8 << 30, rank=rank, world_size=world, explicitly_destroy=True)
    try:
        recv, _, recv_w, handle, _ = buffer.dispatch(x, topk_idx=torch.from_numpy(ids).cuda(), topk_weights=torch.from_numpy(weights).cuda(),
                                                     num_experts=experts, num_max_tokens_per_rank=capacity)
        assert handle.is_low_latency and recv_w is None, case
        lay = olayout.layout(ids, experts, rank * local, local)
        rows = lay["num_rows"]
        got = recv[0] if fp8 else recv
        assert tuple(got.shape) == (capacity_rows, hidden) and rows <= capacity_rows, case
        assert int(handle.send_counts[-1].item()) == rows, case
        source = (x[0] if fp8 else x).view(torch.uint8 if fp8 else torch.int16).cpu().numpy()
        np.testing.assert_array_equal(got[:rows].view(torch.uint8 if fp8 else torch.int16).cpu().numpy(),
                                      olayout.expand_rows(source, lay["row_to_route"], topk), err_msg=str(case))
        if fp8:
            assert recv[1].dtype == x[1].dtype, case
            np.testing.assert_array_equal(recv[1][:rows].view(torch.int32).cpu().numpy(),
                                          olayout.expand_rows(words, lay["row_to_route"], topk), err_msg=str(case))
        expert_dtype = torch.float16 if payload == "float16" else torch.bfloat16
        y = torch.full((capacity_rows, hidden), float("nan"), dtype=expert_dtype, device="cuda")  # the capacity tail is never read
        y[:rows] = torch.from_numpy(rng.normal(size=(rows, hidden)).astype(np.float32)).to(expert_dtype).cuda()
        out, out_w, _ = buffer.combine(y, handle)
        assert out_w is None and out.dtype == expert_dtype and tuple(out.shape) == (tokens, hidden), case
        row_w = olayout.expand_weights(weights, lay["row_to_route"])
        if expert_dtype == torch.float16:
            want = ocombine.combine_fp16(y[:rows].cpu().numpy(), lay["route_to_row"], row_w)
            np.testing.assert_array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16), err_msg=str(case))
        else:
            np.testing.assert_array_equal(bf16_bits(out), ocombine.combine(bf16_bits(y[:rows]), lay["route_to_row"], row_w), err_msg=str(case))
        assert not buffer._runtime.notify_failed
    finally:
        buffer.destroy()
