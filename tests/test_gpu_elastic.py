"""GPU: the public ElasticBuffer / expand / aggregate path end to end against the oracle."""

import numpy as np
import pytest
import torch

from oracle import cases
from oracle import combine as ocombine
from oracle import layout as olayout
from oracle import quant as oquant
from tests.gpu_util import bf16_bits, f32_bits, fp8_bits

pytestmark = pytest.mark.gpu


def test_elastic_buffer_c1_roundtrip_and_cached():
    import deepep_amd

    x, idx, w, cfg = cases.make_inputs("C1")
    buffer = deepep_amd.ElasticBuffer(
        None, num_max_tokens_per_rank=128, hidden=1024, num_topk=4, explicitly_destroy=True
    )
    try:
        xd, idxd, wd = x.cuda(), idx.cuda(), w.cuda()
        recv, none, recv_w, handle, event = buffer.dispatch(xd, topk_idx=idxd, topk_weights=wd, num_experts=16, do_expand=True)
        want = olayout.layout(idx.numpy(), 16)
        assert none is None and handle.num_expanded_tokens == want["num_rows"]
        assert handle.num_recv_tokens_per_expert_list == want["counts"].tolist()
        np.testing.assert_array_equal(handle.psum_num_recv_tokens_per_expert.cpu().numpy(), want["psum"])
        np.testing.assert_array_equal(handle.weight_return_meta.cpu().numpy(), want["row_to_route"])
        np.testing.assert_array_equal(bf16_bits(recv), olayout.expand_rows(bf16_bits(x), want["row_to_route"], 4))
        np.testing.assert_array_equal(f32_bits(recv_w), olayout.expand_weights(w.numpy(), want["row_to_route"]).view(np.uint32))
        y = (recv.float() * 0.5 + 1).bfloat16()
        out, out_w, _ = buffer.combine(y, handle, topk_weights=recv_w)
        np.testing.assert_array_equal(bf16_bits(out), ocombine.combine(bf16_bits(y), want["route_to_row"]))
        np.testing.assert_array_equal(out_w.cpu().numpy(), w.numpy())
        # backward of combine = cached dispatch of the gradient with the same handle
        grad = torch.randn_like(xd)
        grad_rows, _, _, same, _ = buffer.dispatch(grad, handle=handle)
        assert same is handle
        np.testing.assert_array_equal(bf16_bits(grad_rows), olayout.expand_rows(bf16_bits(grad), want["row_to_route"], 4))
        # async variant: caller waits on the event
        with torch.cuda.stream(torch.cuda.Stream()):
            pass
        recv2, _, _, _, ev = buffer.dispatch(xd, handle=handle, async_with_compute_stream=True)
        ev.current_stream_wait()
        assert torch.equal(recv2, recv)
        buffer.barrier(with_cpu_sync=True)
    finally:
        buffer.destroy()
    with pytest.raises(RuntimeError, match="destroyed"):
        buffer.dispatch(xd, topk_idx=idxd, num_experts=16)


def test_elastic_buffer_rank_share_fp8_fused():
    # one EP64 rank's share: 384 experts / 64 = 6 local experts; tokens of all sources flattened
    import deepep_amd

    x, idx, w, cfg = cases.make_inputs("C4", tokens=64 * 48)
    buffer = deepep_amd.ElasticBuffer(
        None, num_bytes=4 << 20, use_fp8_dispatch=True, explicitly_destroy=True, rank=5, world_size=64
    )
    try:
        (q, s), _, recv_w, handle, _ = buffer.dispatch(x.cuda(), topk_idx=idx.cuda(), topk_weights=w.cuda(), num_experts=384)
        want = olayout.layout(idx.numpy(), 384, 30, 6)
        assert handle.num_recv_tokens_per_expert_list == want["counts"].tolist()
        q_ref, s_ref = oquant.cast_to_fp8_torch(x)
        np.testing.assert_array_equal(fp8_bits(q), olayout.expand_rows(fp8_bits(q_ref), want["row_to_route"], 8))
        np.testing.assert_array_equal(f32_bits(s), olayout.expand_rows(f32_bits(s_ref), want["row_to_route"], 8))
        y = torch.randn(handle.num_expanded_tokens, 7168, generator=torch.Generator().manual_seed(3)).bfloat16()
        out, _, _ = buffer.combine(y.cuda(), handle)
        np.testing.assert_array_equal(bf16_bits(out), ocombine.combine(bf16_bits(y), want["route_to_row"]))
    finally:
        buffer.destroy()


def test_direct_expand_and_aggregate():
    from deepep_amd import direct

    x, idx, w, cfg = cases.make_inputs("C1")
    idx[5, 1] = -1
    payload, ew, offsets, counts, mapping = direct.expand(x.cuda(), idx.cuda(), w.cuda(), 16)
    want = olayout.layout(idx.numpy(), 16)
    np.testing.assert_array_equal(offsets.cpu().numpy(), want["offsets"])
    np.testing.assert_array_equal(counts.cpu().numpy(), want["counts"])
    np.testing.assert_array_equal(mapping.cpu().numpy(), want["route_to_row"])
    np.testing.assert_array_equal(bf16_bits(payload), olayout.expand_rows(bf16_bits(x), want["row_to_route"], 4))
    values = torch.rand(want["num_rows"]).cuda()
    out, agg_values = direct.aggregate(payload, ew, values, mapping)
    ref = ocombine.combine(bf16_bits(payload), want["route_to_row"], ew.cpu().numpy())
    np.testing.assert_array_equal(bf16_bits(out), ref)
    np.testing.assert_array_equal(agg_values.cpu().numpy(), ocombine.return_weights(values.cpu().numpy(), want["route_to_row"]))
    (q, s), _, _, _, _ = direct.expand(x.cuda(), idx.cuda(), None, 16, quantize_fp8=True)
    q_ref, s_ref = oquant.cast_to_fp8_torch(x)
    np.testing.assert_array_equal(fp8_bits(q), olayout.expand_rows(fp8_bits(q_ref), want["row_to_route"], 4))


def test_utils_cast_roundtrip():
    from deepep_amd.utils import per_token_cast_back, per_token_cast_to_fp8

    x = torch.randn(33, 512, generator=torch.Generator().manual_seed(0)).bfloat16()
    q, s = per_token_cast_to_fp8(x.cuda())
    back = per_token_cast_back(q, s)
    q_ref, s_ref = oquant.cast_to_fp8_torch(x)
    np.testing.assert_array_equal(bf16_bits(back), oquant.cast_back(fp8_bits(q_ref), s_ref.numpy()))


@pytest.mark.parametrize("payload", ["bfloat16", "float16", "fp8_int32_scales", "fp8_float32_scales"])
def test_low_latency_dispatch_combine_rank_share(payload):
    """The reference's low-latency system test (tests/elastic/test_ep_low_latency.py: routes :397-407, payload
    :421-430, scales :433-446, dispatch checks :482-531, stand-in experts :466-479, expected combine :449-463) for
    one EP16 rank's share: capacity layout [C,H], rows bit-exact per expert block, weights taken from the handle."""
    import deepep_amd

    world, rank, per_rank, hidden, experts, topk = 16, 5, 24, 7168, 64, 8
    local = experts // world
    routes = cases.ll_routes(world, per_rank, topk, experts, seed=3)
    idx = torch.tensor([row for source in routes for row in source])
    sources, toks = np.repeat(np.arange(world), per_rank), np.tile(np.arange(per_rank), world)
    values = torch.from_numpy(cases.ll_payload(sources, toks, hidden))
    w = ((torch.arange(topk) + 1) / 32).repeat(world * per_rank, 1).contiguous()
    fp8 = payload.startswith("fp8")
    if fp8:
        bits = cases.ll_fp8_scale_bits(sources, toks, hidden, packed_e8m0="int32" in payload)
        scales = torch.from_numpy(bits) if "int32" in payload else torch.from_numpy(bits).view(torch.float32)
        x = (values.to(torch.float8_e4m3fn).cuda(), scales.cuda())
    else:
        x = values.to(getattr(torch, payload)).cuda()
    entries = cases.ll_expert_entries(routes, experts, world, rank)
    rows = sum(len(v) for v in entries)
    capacity_rows = world * per_rank * min(topk, local)
    buffer = deepep_amd.ElasticBuffer(None, num_bytes=8 << 30, rank=rank, world_size=world, explicitly_destroy=True)
    try:
        recv, none, recv_w, handle, event = buffer.dispatch(x, topk_idx=idx.cuda(), topk_weights=w.cuda(), num_experts=experts)
        assert none is None and recv_w is None and handle.is_low_latency
        got = recv[0] if fp8 else recv
        assert tuple(got.shape) == (capacity_rows, hidden) and handle.num_expanded_tokens == capacity_rows
        assert handle.num_recv_tokens == world * per_rank and handle.num_recv_tokens_per_expert_list == []
        assert handle.psum_num_recv_tokens_per_expert is None and handle.num_unaligned_recv_tokens_per_expert is None
        assert int(handle.send_counts[-1].item()) == rows
        host = got.float().cpu()
        start = 0
        for block in entries:
            src, tok = zip(*block) if block else ((), ())
            want = cases.ll_payload(src, tok, hidden) if block else np.zeros((0, hidden), np.float32)
            np.testing.assert_array_equal(host[start : start + len(block)].numpy(), want)
            if fp8:
                assert recv[1].dtype == x[1].dtype and tuple(recv[1].shape) == (capacity_rows, hidden // 128)
                got_bits = recv[1][start : start + len(block)].cpu().view(torch.int32).numpy()
                np.testing.assert_array_equal(got_bits, cases.ll_fp8_scale_bits(src, tok, hidden, "int32" in payload)) if block else None
            start += len(block)
        # stand-in experts on the valid rows; the capacity tail stays whatever it is
        expert_dtype = torch.float16 if payload == "float16" else torch.bfloat16
        y = torch.zeros((capacity_rows, hidden), dtype=expert_dtype, device="cuda")
        row_expert = np.concatenate([[rank * local + e] * len(block) for e, block in enumerate(entries)]).astype(np.int64)
        mapped = np.stack([cases.ll_expert_map(host[i].numpy(), int(row_expert[i])) for i in range(rows)])
        y[:rows] = torch.from_numpy(mapped).to(expert_dtype).cuda()
        out, out_w, _ = buffer.combine(y, handle)
        assert out_w is None and out.dtype == expert_dtype and tuple(out.shape) == (world * per_rank, hidden)
        lay = olayout.layout(idx.numpy(), experts, rank * local, local)
        slot = lay["row_to_route"] % topk
        row_w = ((slot + 1) / 32).astype(np.float32)
        if expert_dtype == torch.float16:
            want_out = ocombine.combine_fp16(y[:rows].cpu().numpy(), lay["route_to_row"], row_w)
            np.testing.assert_array_equal(out.cpu().numpy().view(np.uint16), want_out.view(np.uint16))
        else:
            want_out = ocombine.combine(bf16_bits(y[:rows]), lay["route_to_row"], row_w)
            np.testing.assert_array_equal(bf16_bits(out), want_out)
    finally:
        buffer.destroy()


def test_low_latency_capacity_above_the_batch():
    """The usual decode set-up: a fixed num_max_tokens_per_rank above the actual batch and at least top-k experts per
    rank, so that the capacity layout C = P*M*K holds more rows than the batch has routes (T*K).  Dispatch returns
    [C,H], combine takes an expert output of C rows."""
    import deepep_amd

    world, rank, per_rank, capacity, hidden, experts, topk = 16, 3, 8, 32, 1024, 256, 8
    local = experts // world
    routes = cases.ll_routes(world, per_rank, topk, experts, seed=9)
    idx = torch.tensor([row for source in routes for row in source])
    sources, toks = np.repeat(np.arange(world), per_rank), np.tile(np.arange(per_rank), world)
    x = torch.from_numpy(cases.ll_payload(sources, toks, hidden)).bfloat16().cuda()
    w = torch.rand(world * per_rank, topk, generator=torch.Generator().manual_seed(2))
    capacity_rows = world * capacity * min(topk, local)
    assert capacity_rows > world * per_rank * topk
    buffer = deepep_amd.ElasticBuffer(None, num_bytes=8 << 30, rank=rank, world_size=world, explicitly_destroy=True)
    try:
        recv, _, _, handle, _ = buffer.dispatch(x, topk_idx=idx.cuda(), topk_weights=w.cuda(), num_experts=experts,
                                                num_max_tokens_per_rank=capacity)
        assert handle.is_low_latency and tuple(recv.shape) == (capacity_rows, hidden)
        lay = olayout.layout(idx.numpy(), experts, rank * local, local)
        rows = lay["num_rows"]
        assert 0 < rows == int(handle.send_counts[-1].item())
        np.testing.assert_array_equal(bf16_bits(recv[:rows]), olayout.expand_rows(bf16_bits(x), lay["row_to_route"], topk))
        y = torch.zeros((capacity_rows, hidden), dtype=torch.bfloat16, device="cuda")
        y[:rows] = (recv[:rows].float() * 0.5 + 1.0).bfloat16()
        y[rows:] = float("nan")  # the capacity tail is never read
        out, _, _ = buffer.combine(y, handle)
        row_w = olayout.expand_weights(w.numpy(), lay["row_to_route"])
        np.testing.assert_array_equal(bf16_bits(out), ocombine.combine(bf16_bits(y[:rows]), lay["route_to_row"], row_w))
        assert not buffer._runtime.notify_failed
    finally:
        buffer.destroy()


def test_elastic_buffer_all_routes_masked():
    """No valid route at all: the payload kernel is queued before the host knows that R = 0; outputs are empty views,
    the handle says zero rows everywhere, and the combine of nothing is a tensor of zeros."""
    import deepep_amd

    tokens, hidden, topk, experts = 300, 1024, 4, 16
    x = torch.randn(tokens, hidden).bfloat16().cuda()
    idx = torch.full((tokens, topk), -1, dtype=torch.int64).cuda()
    w = torch.rand(tokens, topk).cuda()
    for fp8 in (False, True):
        buffer = deepep_amd.ElasticBuffer(None, num_max_tokens_per_rank=tokens, hidden=hidden, num_topk=topk,
                                          use_fp8_dispatch=fp8, explicitly_destroy=True)
        try:
            recv, _, recv_w, handle, _ = buffer.dispatch(x, topk_idx=idx, topk_weights=w, num_experts=experts)
            payload = recv[0] if fp8 else recv
            assert tuple(payload.shape) == (0, hidden) and tuple(recv_w.shape) == (0,)
            assert handle.num_expanded_tokens == 0 and handle.num_recv_tokens_per_expert_list == [0] * experts
            out, out_w, _ = buffer.combine(torch.empty((0, hidden), dtype=torch.bfloat16, device="cuda"), handle, topk_weights=recv_w)
            assert not out.any() and tuple(out.shape) == (tokens, hidden) and not out_w.any()
        finally:
            buffer.destroy()
