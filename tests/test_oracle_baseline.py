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
