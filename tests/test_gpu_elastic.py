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
