"""Pins the combine oracle on the reference's exact-sum fixtures and on order/rounding properties."""

import numpy as np
import pytest

from oracle import cases
from oracle.combine import combine, combine_fp64, return_weights
from oracle.layout import expand_rows, layout
from oracle.quant import bf16_bits_to_f32, f32_to_bf16_bits


def test_reference_hand_case_sums():
    # tests/test_reference.py:61-67: expert output = x * (expert+1); sums 2*(1+2)=6, 3*3=9, 5*(2+2)=20.
    idx = np.asarray([[0, 1], [2, -1], [1, 1]])
    x = np.asarray([[2.0], [3.0], [5.0]], dtype=np.float32)
    lay = layout(idx, 4)
    rows = expand_rows(x, lay["row_to_route"], 2)
    experts = idx.reshape(-1)[lay["row_to_route"]]
    y = f32_to_bf16_bits(rows * (experts[:, None] + 1))
    out = bf16_bits_to_f32(combine(y, lay["route_to_row"]))
    assert out.ravel().tolist() == [6.0, 9.0, 20.0]
    w = np.asarray([[0.25, 0.5], [0.75, 9.0], [0.125, 0.625]], dtype=np.float32)
    values = 0.5 - w.reshape(-1)[lay["row_to_route"]]
    np.testing.assert_array_equal(
        return_weights(values, lay["route_to_row"]), [[0.25, 0.0], [-0.25, 0.0], [0.375, -0.125]]
    )


@pytest.mark.parametrize("generation", [0, 3])
def test_reference_bounded_integer_fixture(generation):
    # tests/elastic/test_combine.py:496-515 with EP=1: expert e at slot s returns x + (e%3-1) + (s%3-1).
    tokens, hidden, experts, topk = 37, 64, 12, 5
    routes = cases.matrix_routes(1, experts, topk, [tokens])[0]
    idx = np.asarray(routes)
    idx[3, :] = -1
    idx[5, 1] = experts + 2  # >= E is invalid too
    lay = layout(idx, experts)
    base = cases.combine_payload_values(0, tokens, generation, hidden)
    route = lay["row_to_route"]
    e, s = idx.reshape(-1)[route], route % topk
    y = f32_to_bf16_bits(expand_rows(base, route, topk) + ((e % 3 - 1) + (s % 3 - 1))[:, None])
    want = cases.combine_expected_values(idx.tolist(), experts, 0, generation, hidden)
    np.testing.assert_array_equal(bf16_bits_to_f32(combine(y, lay["route_to_row"])), want)


def test_reference_weighted_low_latency_fixture():
    # tests/elastic/test_ep_low_latency.py:449-463: y_e = bf16(x*((e%4+1)/4) + (e%3-1)/8), weight (s+1)/32.
    import torch

    tokens, hidden, experts, topk = 19, 128, 16, 4
    idx = np.asarray(cases.matrix_routes(1, experts, topk, [tokens])[0])
    idx[2, 1] = -1
    x, _ = cases.dispatch_payload_values(0, tokens, 1, hidden)
    xt = torch.from_numpy(x).bfloat16().float()
    expected = torch.zeros_like(xt)
    for t in range(tokens):
        for s in range(topk):
            e = int(idx[t, s])
            if e >= 0:
                expected[t] += (xt[t] * ((e % 4 + 1) / 4) + (e % 3 - 1) / 8).bfloat16().float() * ((s + 1) / 32)
    expected = expected.bfloat16().view(torch.int16).numpy().view(np.uint16)
    lay = layout(idx, experts)
    route = lay["row_to_route"]
    e, s = idx.reshape(-1)[route], route % topk
    rows = torch.from_numpy(expand_rows(xt.numpy(), route, topk))
    y = (rows * torch.from_numpy((e % 4 + 1) / 4).float()[:, None] + torch.from_numpy((e % 3 - 1) / 8).float()[:, None])
    y = y.bfloat16().view(torch.int16).numpy().view(np.uint16)
    w_rows = ((s + 1) / 32).astype(np.float32)
    np.testing.assert_array_equal(combine(y, lay["route_to_row"], w_rows), expected)


def test_low_latency_fixture_in_fp16_and_its_input_recipes():
    """combine_fp16 against the reference test's own formula evaluated in torch half (expected_combine,
    tests/elastic/test_ep_low_latency.py:449-463), on that test's routes and payload recipes (:397-430)."""
    import torch

    from oracle.combine import combine_fp16

    world, tokens, hidden, experts, topk = 4, 5, 64, 16, 3
    routes = cases.ll_routes(world, tokens, topk, experts, seed=7)
    assert all(len(set(row)) == topk for rank in routes for row in rank)  # distinct experts per token
    flat = np.asarray([row for rank in routes for row in rank])
    sources, toks = np.repeat(np.arange(world), tokens), np.tile(np.arange(tokens), world)
    x = cases.ll_payload(sources, toks, hidden)
    assert x[7, :4].tolist() == [0, 1, 0, 2] and x[7, 4] == (1 * 3 + 2 * 5 + 4) % 17 - 8  # identity columns + formula
    xt = torch.from_numpy(x).half().float()
    expected = torch.zeros_like(xt)
    for t in range(flat.shape[0]):
        for s in range(topk):
            e = int(flat[t, s])
            expected[t] += (xt[t] * ((e % 4 + 1) / 4) + (e % 3 - 1) / 8).half().float() * ((s + 1) / 32)
    lay = layout(flat, experts)
    route = lay["row_to_route"]
    e, s = flat.reshape(-1)[route], route % topk
    rows = expand_rows(xt.numpy(), route, topk)
    y = np.stack([cases.ll_expert_map(rows[i], int(e[i])) for i in range(len(route))]).astype(np.float16)
    got = combine_fp16(y, lay["route_to_row"], ((s + 1) / 32).astype(np.float32))
    np.testing.assert_array_equal(got.view(np.uint16), expected.half().numpy().view(np.uint16))
    # what each local expert of rank 1 receives, against the layout's rows for that expert range
    entries = cases.ll_expert_entries(routes, experts, world, 1)
    share = layout(flat, experts, 4, 4)
    assert [len(v) for v in entries] == share["counts"].tolist()
    first = share["row_to_route"][: len(entries[0])] // topk
    assert [(int(t) // tokens, int(t) % tokens) for t in first] == entries[0]
    # scale recipes: packed E8M0 ones, or FP32 words with distinct low bits
    assert cases.ll_fp8_scale_bits([1], [2], 256, True).tolist() == [[0x7F7F7F7F] * 2]
    assert cases.ll_fp8_scale_bits([1], [2], 256, False).tolist() == [[0x3F000001 + 65536 + 256, 0x3F000001 + 65536 + 257]]


def test_slot_order_and_unfused_multiply_add_are_observable():
    # 2^24 + 1 - 2^24: slot order (big, one, -big) gives 0, any other order gives 1 -> order is pinned.
    big = np.float32(2.0**24)
    y = f32_to_bf16_bits(np.asarray([[big], [1.0], [-big]], dtype=np.float32))
    r2r = np.asarray([[0, 1, 2]])
    assert bf16_bits_to_f32(combine(y, r2r))[0, 0] == 0.0
    assert bf16_bits_to_f32(combine(y, np.asarray([[0, 2, 1]])))[0, 0] == 1.0
    # a*w + c with a*w inexact: separate rounding differs from a fused multiply-add
    a, w, c = np.float32(1.0 + 2.0**-7), np.float32(1.0 + 2.0**-23), np.float32(-1.0)
    ybits = f32_to_bf16_bits(np.asarray([[a], [c]], dtype=np.float32))
    got = bf16_bits_to_f32(combine(ybits, np.asarray([[0, 1]]), np.asarray([w, 1.0], np.float32)))[0, 0]
    unfused = np.float32(np.float32(a * w) + c)
    assert got == bf16_bits_to_f32(f32_to_bf16_bits(np.asarray([unfused])))[0]


@pytest.mark.parametrize("seed", range(3))
def test_within_one_bf16_ulp_of_fp64(seed):
    rng = np.random.default_rng(seed)
    tokens, topk, experts, hidden = 50, 8, 32, 96
    idx = rng.integers(-1, experts, size=(tokens, topk))
    lay = layout(idx, experts)
    y = f32_to_bf16_bits(rng.normal(size=(lay["num_rows"], hidden)).astype(np.float32))
    w = rng.random(lay["num_rows"]).astype(np.float32)
    for weights in (None, w):
        got = bf16_bits_to_f32(combine(y, lay["route_to_row"], weights)).astype(np.float64)
        exact = combine_fp64(y, lay["route_to_row"], weights)
        ulp = np.exp2(np.floor(np.log2(np.maximum(np.abs(exact), 2.0**-126))) - 7)
        assert (np.abs(got - exact) <= ulp).all()


def test_tokens_without_rows_are_zero():
    y = f32_to_bf16_bits(np.ones((1, 8), np.float32))
    out = combine(y, np.asarray([[-1, -1], [0, -1]]))
    assert not out[0].any() and (bf16_bits_to_f32(out[1]) == 1.0).all()
    assert not combine(np.zeros((0, 8), np.uint16), np.full((3, 2), -1)).any()
