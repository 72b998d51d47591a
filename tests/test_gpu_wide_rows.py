"""Rows wider than any model of the reference (hidden 8192 .. 32 768): BF16 dispatch with weights, the fused FP8
quantiser and the weighted combine against the CPU oracle, bit for bit.  Row widths enter the kernels as loop bounds and
strides only; these sizes show that nothing narrower is baked in."""

import numpy as np
import pytest
import torch

from oracle import combine as ocombine
from oracle import layout as olayout
from oracle import quant as oquant
from tests.gpu_util import bf16_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tokens,topk,experts,hidden", [(1000, 8, 64, 8192), (300, 4, 16, 16384), (50, 2, 4, 32768), (700, 32, 256, 9216)])
def test_dispatch_quantise_combine_at_wide_rows(tokens, topk, experts, hidden):
    from deepep_amd import ops

    rng = np.random.default_rng(hidden + tokens)
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int64)
    ids[rng.random(ids.shape) < 0.1] = -1
    x = torch.from_numpy(rng.normal(size=(tokens, hidden)).astype(np.float32)).bfloat16()
    weights = torch.from_numpy(rng.random((tokens, topk)).astype(np.float32))
    want = olayout.layout(ids, experts)
    ws = ops.Workspace(ops.layout_workspace_bytes(tokens, topk, experts))
    try:
        plan = ops.layout(ws, torch.from_numpy(ids).cuda(), experts)
        _, rows = ops.layout_wait(ws)
        assert rows == want["num_rows"]
        out, _, out_weights = ops.dispatch_copy(x.cuda(), None, weights.cuda(), plan["route_to_row"], plan["row_to_route"], rows)
        np.testing.assert_array_equal(bf16_bits(out), olayout.expand_rows(bf16_bits(x), want["row_to_route"], topk))
        row_weights = olayout.expand_weights(weights.numpy(), want["row_to_route"])
        np.testing.assert_array_equal(out_weights.cpu().numpy(), row_weights)
        codes, scales, _ = ops.dispatch_quant_fp8(x.cuda(), None, plan["route_to_row"], plan["row_to_route"], rows)
        want_codes, want_scales = oquant.cast_to_fp8_torch(x)
        np.testing.assert_array_equal(codes.cpu().view(torch.uint8).numpy(),
                                      olayout.expand_rows(want_codes.view(torch.uint8).numpy(), want["row_to_route"], topk))
        np.testing.assert_array_equal(scales.cpu().numpy(), olayout.expand_rows(want_scales.numpy(), want["row_to_route"], topk))
        y = torch.from_numpy(rng.normal(size=(rows, hidden)).astype(np.float32)).bfloat16()
        combined, _ = ops.combine(y.cuda(), plan["route_to_row"], out_weights)
        np.testing.assert_array_equal(bf16_bits(combined), ocombine.combine(bf16_bits(y), want["route_to_row"], row_weights))
    finally:
        ws.destroy()
