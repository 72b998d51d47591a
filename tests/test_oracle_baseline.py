"""The timed torch-CPU baseline computes exactly what the NumPy oracle computes."""

import numpy as np
import torch

from oracle import baseline, cases
from oracle import combine as ocombine
from oracle import layout as olayout
from oracle import quant as oquant


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_baseline_equals_oracle():
    x, idx, w, cfg = cases.make_inputs("C3", tokens=64, hidden=512)
    idx[3, 2] = -1
    counts, psum, r2row, r2route = baseline.layout(idx, cfg["experts"])
    want = olayout.layout(idx.numpy(), cfg["experts"])
    np.testing.assert_array_equal(counts.numpy(), want["counts"])
    np.testing.assert_array_equal(psum.numpy(), want["psum"])
    np.testing.assert_array_equal(r2row.numpy(), want["route_to_row"])
    np.testing.assert_array_equal(r2route.numpy(), want["row_to_route"])
    q, s, ow = baseline.dispatch_fp8(x, w, r2route, cfg["topk"])
    qi, si = oquant.cast_to_fp8_int(_bits(x))
    np.testing.assert_array_equal(q.view(torch.uint8).numpy(), olayout.expand_rows(qi, want["row_to_route"], cfg["topk"]))
    np.testing.assert_array_equal(s.numpy(), olayout.expand_rows(si, want["row_to_route"], cfg["topk"]))
    np.testing.assert_array_equal(ow.numpy(), olayout.expand_weights(w.numpy(), want["row_to_route"]))
    y = torch.randn(want["num_rows"], 512, generator=torch.Generator().manual_seed(2)).bfloat16()
    for weights in (None, ow):
        got = baseline.combine(y, r2row, weights)
        ref = ocombine.combine(_bits(y), want["route_to_row"], None if weights is None else weights.numpy())
        np.testing.assert_array_equal(_bits(got), ref)


def test_megamoe_baseline_matches_numpy_oracle():
    # the timed torch.matmul form against the NumPy oracle (different BLAS, same roundings): all but a few
    # elements identical, those one BF16 / e4m3 step apart
    from oracle import megamoe as mm

    rng = np.random.default_rng(4)
    x = mm.round_bf16(rng.normal(size=(12, 128)))
    w1 = (rng.normal(size=(256, 128)) * 0.1).astype(np.float32)
    w2 = (rng.normal(size=(128, 128)) * 0.1).astype(np.float32)
    got = baseline.megamoe_expert_forward(torch.from_numpy(x), torch.from_numpy(w1), torch.from_numpy(w2)).float().numpy()
    want = mm.expert_forward(x, w1, w2)
    assert mm.relative_frobenius(got, want) < 5e-3
    assert (got == want).mean() > 0.95
