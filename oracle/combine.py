"""Combine oracle: slot-ordered fp32 reduce of a token's expert rows, RNE to BF16.

Pinned by (tests/test_oracle_combine.py):
  * the reference's bounded-integer fixture (tests/elastic/test_combine.py:496-515): payload
    (t+c+src+g)%7-3, expected base*count + sum((e%3-1)+(s%3-1)) — exact in fp32/bf16;
  * the weighted low-latency fixture (tests/elastic/test_ep_low_latency.py:449-479): weights (s+1)/32,
    expert map y = x*((e%4+1)/4) + (e%3-1)/8;
  * the hand case of tests/test_reference.py:61-67 (6, 9, 20 and the weight channel);
  * the same fixture in FP16 for combine_fp16, checked against the test's own torch formula evaluated with torch
    half tensors (what the reference's expected_combine computes);
  * an fp64 sum (1-ulp bound) and order sensitivity: a reversed-slot sum differs on a crafted input,
    so a wrong accumulation order fails.
"""

from __future__ import annotations

import numpy as np

from .quant import bf16_bits_to_f32, f32_to_bf16_bits


def combine_fp16(y_f16, route_to_row, row_weights=None):
    """The same reduce for IEEE half rows (the low-latency path takes BF16 or FP16 expert outputs and returns the
    same dtype, deep_ep/backends/mesh_clos/elastic.py:596-606; expected_combine,
    tests/elastic/test_ep_low_latency.py:449-463): half -> fp32 exactly, separate multiply and add in fp32, slot
    order, one RNE rounding to half (numpy's float32 -> float16 cast).  y: float16 [R, H]; returns float16 [T, H]."""
    y = np.asarray(y_f16, dtype=np.float16)
    r2r = np.asarray(route_to_row, dtype=np.int64)
    acc = np.zeros((r2r.shape[0], y.shape[1]), dtype=np.float32)
    w = None if row_weights is None else np.asarray(row_weights, dtype=np.float32)
    for slot in range(r2r.shape[1]):
        rows = r2r[:, slot]
        valid = rows >= 0
        safe = np.where(valid, rows, 0)
        if y.shape[0] == 0:
            continue
        tmp = y[safe].astype(np.float32)
        if w is not None:
            tmp = (tmp * w[safe][:, None]).astype(np.float32)
        acc = np.where(valid[:, None], (acc + tmp).astype(np.float32), acc)
    return acc.astype(np.float16)


def combine(y_bf16_bits, route_to_row, row_weights=None):
    """out[t] = bf16_rne( sum over slots s in order, skipping -1, of  fp32(y[row]) (* w[row]) ).

    Operation order follows AggregateRange (csrc/direct/kernels/aggregate/aggregate_impl.h:166-226):
    accumulator starts at +0.0f; per valid slot ``tmp = float(y); tmp = tmp * w; acc = acc + tmp``
    (separate multiply and add, never fused); final cast is round-to-nearest-even (CAST_RINT).
    Unweighted (HT) form: tests/utils/reference.py:104-131, tests/elastic/test_combine.py:504-515.
    Weighted (LL / aggregate / MegaMoE unpermute) form: tests/elastic/test_ep_low_latency.py:449-463.
    y: uint16 [R, H]; route_to_row: int32 [T, K]; row_weights: float32 [R] or None.
    """
    y = np.asarray(y_bf16_bits, dtype=np.uint16)
    r2r = np.asarray(route_to_row, dtype=np.int64)
    tokens, topk = r2r.shape
    hidden = y.shape[1]
    acc = np.zeros((tokens, hidden), dtype=np.float32)
    w = None if row_weights is None else np.asarray(row_weights, dtype=np.float32)
    for slot in range(topk):
        rows = r2r[:, slot]
        valid = rows >= 0
        safe = np.where(valid, rows, 0)
        if y.shape[0] == 0:
            continue
        tmp = bf16_bits_to_f32(y[safe])
        if w is not None:
            tmp = (tmp * w[safe][:, None]).astype(np.float32)
        acc = np.where(valid[:, None], (acc + tmp).astype(np.float32), acc)
    return f32_to_bf16_bits(acc)


def combine_fp64(y_bf16_bits, route_to_row, row_weights=None):
    """Order-free fp64 sum used for the 1-BF16-ulp bound (tests/utils/reference.py:134-155 style)."""
    y = bf16_bits_to_f32(np.asarray(y_bf16_bits, dtype=np.uint16)).astype(np.float64)
    r2r = np.asarray(route_to_row, dtype=np.int64)
    acc = np.zeros((r2r.shape[0], y.shape[1]), dtype=np.float64)
    for slot in range(r2r.shape[1]):
        rows = r2r[:, slot]
        valid = rows >= 0
        safe = np.where(valid, rows, 0)
        if y.shape[0] == 0:
            continue
        tmp = y[safe]
        if row_weights is not None:
            tmp = tmp * np.asarray(row_weights, dtype=np.float64)[safe][:, None]
        acc += np.where(valid[:, None], tmp, 0.0)
    return acc


def return_weights(row_values, route_to_row):
    """Weight-return channel: out[t, s] = values[row(t, s)], 0 for slots without a row.

    docs/elastic.md:71, tests/elastic/test_combine.py:525-531, tests/utils/reference.py:124-126,
    AggregateValuesSimtVf (csrc/direct/kernels/aggregate/aggregate_impl.h:60-63).
    """
    r2r = np.asarray(route_to_row, dtype=np.int64)
    values = np.asarray(row_values, dtype=np.float32)
    if values.size == 0:
        return np.zeros(r2r.shape, dtype=np.float32)
    return np.where(r2r >= 0, values[np.where(r2r >= 0, r2r, 0)], np.float32(0)).astype(np.float32)
