"""GPU parity: HIP layout / dispatch / quantise / combine through the C-ABI vs the CPU oracle.

Bit-exact for layout, indices, payloads, scales and weights; combine bit-exact against the oracle's
slot-ordered fp32 sum (and therefore within 1 BF16 ulp of the fp64 sum, checked in the CPU suite).
"""

import numpy as np
import pytest
import torch

from oracle import cases
from oracle import combine as ocombine
from oracle import layout as olayout
from oracle import quant as oquant
from tests.gpu_util import bf16_bits, bits_to_bf16, f32_bits, fp8_bits, i32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from deepep_amd import ops as module

    return module


@pytest.fixture(scope="module")
def ws(ops):
    workspace = ops.Workspace(64 << 20)
    yield workspace
    workspace.destroy()


def _check_layout(ops, ws, idx_np, experts, begin=0, local=None):
    idx = torch.from_numpy(np.ascontiguousarray(idx_np, dtype=np.int64)).cuda()
    got = ops.layout(ws, idx, experts, begin, local)
    want = olayout.layout(idx_np, experts, begin, local)
    # the host mailbox (no copy, no stream wait) must agree with the device tensors
    host_counts, host_rows = ops.layout_wait(ws, len(want["counts"]))
    assert host_rows == want["num_rows"] and host_counts == [int(c) for c in want["counts"]]
    assert ops.layout_wait(ws) == (None, host_rows)  # asking again returns the same launch's result
    rows = int(got["num_rows"].item())
    assert rows == want["num_rows"]
    for key in ("counts", "psum", "offsets", "route_to_row"):
        np.testing.assert_array_equal(i32(got[key]), want[key], err_msg=key)
    np.testing.assert_array_equal(i32(got["row_to_route"][:rows]), want["row_to_route"])
    return got, want, rows


LAYOUT_SHAPES = [
    # tokens, topk, experts, begin, local
    (1, 1, 1, 0, 1),
    (3, 2, 4, 0, 4),
    (37, 5, 12, 0, 12),
    (128, 4, 16, 0, 16),
    (128, 8, 256, 0, 256),
    (257, 8, 256, 32, 64),
    (1000, 16, 1024, 0, 1024),
    (4096, 8, 256, 0, 256),
    (16384, 8, 384, 0, 6),
    (16384, 8, 384, 378, 6),
    (5000, 6, 7, 2, 3),
    (300, 32, 1024, 0, 1024),  # the largest top-k and expert count the library takes
    (16384, 8, 256, 0, 256),  # chunks too long for the one-launch kernel's registers: always two launches
]


@pytest.mark.parametrize("one_launch", [True, False])
@pytest.mark.parametrize("tokens,topk,experts,begin,local", LAYOUT_SHAPES)
def test_layout_matches_oracle(ops, ws, tokens, topk, experts, begin, local, one_launch):
    """Both forms of the layout (one launch whose workgroups exchange histograms; count and assign launches)."""
    rng = np.random.default_rng(tokens * 31 + topk)
    idx = rng.integers(-1, experts + 1, size=(tokens, topk))  # includes -1 and == E (both invalid)
    ws.tune("layout_one_launch", one_launch)
    try:
        _check_layout(ops, ws, idx, experts, begin, local)
        _check_layout(ops, ws, idx[::-1].copy(), experts, begin, local)  # the next launch on the workspace gets a tag of its own
    finally:
        ws.tune("layout_one_launch", 1)


def test_layout_wait_for_histograms_that_runs_out_is_reported(ops):
    """A workgroup's wait for the others' histograms is bounded: told to wait for one histogram more than the launch
    has workgroups, with a bound of 100 us, every workgroup gives up and the kernel ends normally.  Such a launch assigns
    nothing (a histogram is missing, so any row computed without it could lie anywhere): every route is left without a row, every count is
    zero, and the host gets an error instead of results.  The workspace stays usable: later layouts take two launches."""
    workspace = ops.Workspace(1 << 20)
    try:
        idx = torch.randint(0, 16, (512, 4), device="cuda")
        want = olayout.layout(idx.cpu().numpy(), 16)
        good = ops.layout(workspace, idx, 16)  # leaves valid histograms of this very input behind
        ops.layout_wait(workspace)
        workspace.tune("layout_exchange_extra_rows", 1)
        workspace.tune("layout_exchange_ticks", 10_000)
        lay = ops.layout(workspace, idx, 16)
        with pytest.raises(RuntimeError, match="histograms"):
            ops.layout_wait(workspace)
        torch.cuda.synchronize()
        assert (lay["route_to_row"] == -1).all() and not lay["counts"].any() and not lay["psum"].any()
        assert not lay["offsets"].any() and int(lay["num_rows"].item()) == 0
        workspace.tune("layout_exchange_extra_rows", 0)
        again = ops.layout(workspace, idx, 16)  # two launches now; the earlier failure has been reported already
        _, rows = ops.layout_wait(workspace)
        assert rows == want["num_rows"]
        np.testing.assert_array_equal(again["route_to_row"].cpu().numpy(), want["route_to_row"])
        np.testing.assert_array_equal(good["route_to_row"].cpu().numpy(), want["route_to_row"])
        with pytest.raises(ValueError, match="unknown key"):
            workspace.tune("no_such_switch", 1)
    finally:
        workspace.destroy()


def test_layout_timeout_nobody_waited_for_is_reported_by_the_next_call(ops):
    """A launch that timed out without a host wait (the way the MegaMoE forward uses the layout): the next launch on
    the workspace reports it, once, and the one after that works."""
    workspace = ops.Workspace(1 << 20)
    try:
        idx = torch.randint(0, 16, (512, 4), device="cuda")
        workspace.tune("layout_exchange_extra_rows", 1)
        workspace.tune("layout_exchange_ticks", 10_000)
        ops.layout(workspace, idx, 16)
        torch.cuda.synchronize()
        workspace.tune("layout_exchange_extra_rows", 0)
        with pytest.raises(RuntimeError, match="histograms"):
            ops.layout(workspace, idx, 16)
        lay = ops.layout(workspace, idx, 16)
        _, rows = ops.layout_wait(workspace)
        want = olayout.layout(idx.cpu().numpy(), 16)
        assert rows == want["num_rows"]
        np.testing.assert_array_equal(lay["route_to_row"].cpu().numpy(), want["route_to_row"])
    finally:
        workspace.destroy()


def test_layout_skew_duplicates_and_masks(ops, ws):
    idx = np.zeros((2048, 8), dtype=np.int64)  # every slot hits expert 0: duplicates count separately
    _check_layout(ops, ws, idx, 256)
    idx = np.full((300, 8), -1, dtype=np.int64)  # all masked
    got, _, rows = _check_layout(ops, ws, idx, 256)
    assert rows == 0
    _check_layout(ops, ws, np.zeros((0, 8), dtype=np.int64), 256)  # zero tokens


def test_layout_reference_matrix_routes(ops, ws):
    # deterministic generator of the reference's golden matrix (tests/utils/cases.py:150-157), EP8 case
    routes = cases.matrix_routes(2, 256, 8, [4096, 4095])  # first two source ranks of ep8_token_volume
    idx = np.asarray([row for rank in routes for row in rank], dtype=np.int64)
    for rank in (0, 3):
        _check_layout(ops, ws, idx, 256, rank * 32, 32)


@pytest.mark.parametrize("name,tokens", [("C1", None), ("C2", None), ("C3", 512), ("C4", 2048)])
@pytest.mark.parametrize("with_weights", [True, False])
def test_dispatch_bf16_bit_exact(ops, ws, name, tokens, with_weights):
    x, idx, w, cfg = cases.make_inputs(name, tokens=tokens)
    got, want, rows = _check_layout(ops, ws, idx.numpy(), cfg["experts"], cfg["expert_begin"], cfg["num_local"])
    xd = x.cuda()
    wd = w.cuda() if with_weights else None
    out, out_scales, out_w = ops.dispatch_copy(xd, None, wd, got["route_to_row"], got["row_to_route"], rows)
    assert out_scales is None
    np.testing.assert_array_equal(bf16_bits(out), olayout.expand_rows(bf16_bits(x), want["row_to_route"], cfg["topk"]))
    if with_weights:
        np.testing.assert_array_equal(f32_bits(out_w), olayout.expand_weights(w.numpy(), want["row_to_route"]).view(np.uint32))
    else:
        assert out_w is None


@pytest.mark.parametrize("hidden", [16, 48, 128, 1024, 7168])
def test_dispatch_bf16_widths_and_reference_payload(ops, ws, hidden):
    # reference fixture values: ((src*13 + t*7 + c*3 + g*11) % 127 - 63) / 16 are BF16-exact
    tokens, topk, experts = 70, 6, 24
    values, _ = cases.dispatch_payload_values(2, tokens, 1, max(hidden, 128))
    x = torch.from_numpy(values[:, :hidden].copy()).bfloat16()
    idx = np.asarray(cases.matrix_routes(1, experts, topk, [tokens])[0])
    got, want, rows = _check_layout(ops, ws, idx, experts)
    w = torch.from_numpy(cases.dispatch_weights(2, tokens, topk, 1))
    out, _, out_w = ops.dispatch_copy(x.cuda(), None, w.cuda(), got["route_to_row"], got["row_to_route"], rows)
    np.testing.assert_array_equal(bf16_bits(out), olayout.expand_rows(bf16_bits(x), want["row_to_route"], topk))
    np.testing.assert_array_equal(out_w.cpu().numpy(), olayout.expand_weights(w.numpy(), want["row_to_route"]))


@pytest.mark.parametrize("name,tokens", [("C1", None), ("C3", 300), ("C4", 4096)])
def test_dispatch_fp8_prequantized_copy(ops, ws, name, tokens):
    # reference semantic: FP8 payload + FP32 scales move unchanged (docs/elastic.md:61)
    x, idx, w, cfg = cases.make_inputs(name, tokens=tokens)
    q, s = oquant.cast_to_fp8_torch(x)
    got, want, rows = _check_layout(ops, ws, idx.numpy(), cfg["experts"], cfg["expert_begin"], cfg["num_local"])
    out, out_s, out_w = ops.dispatch_copy(q.cuda(), s.cuda(), w.cuda(), got["route_to_row"], got["row_to_route"], rows)
    np.testing.assert_array_equal(fp8_bits(out), olayout.expand_rows(fp8_bits(q), want["row_to_route"], cfg["topk"]))
    np.testing.assert_array_equal(f32_bits(out_s), olayout.expand_rows(f32_bits(s), want["row_to_route"], cfg["topk"]))
    np.testing.assert_array_equal(f32_bits(out_w), olayout.expand_weights(w.numpy(), want["row_to_route"]).view(np.uint32))


@pytest.mark.parametrize("scale", [1.0, 1e-3, 300.0, 1e-5, 3e4, 2.0**-20])
def test_cast_to_fp8_bit_exact_random(ops, scale):
    gen = torch.Generator().manual_seed(int(scale * 1000) % 97)
    x = (torch.randn(96, 7168, generator=gen) * scale).bfloat16()
    x[0, :128] = 0
    q, s = ops.cast_to_fp8(x.cuda())
    q_ref, s_ref = oquant.cast_to_fp8_torch(x)
    np.testing.assert_array_equal(fp8_bits(q), fp8_bits(q_ref))
    np.testing.assert_array_equal(f32_bits(s), f32_bits(s_ref))


def test_cast_to_fp8_every_bf16_magnitude(ops):
    # every finite positive BF16 pattern as a block maximum with a spread of smaller entries: exercises
    # the reciprocal, the product rounding and every e4m3 code including subnormals.
    mags = np.arange(0x0001, 0x7F80, dtype=np.uint16)
    block = np.zeros((mags.size, 128), dtype=np.uint16)
    block[:, 0] = mags
    for j in range(1, 128):
        block[:, j] = np.maximum(mags.astype(np.int32) - 3 * j - (j % 5) * 128, 0).astype(np.uint16) | (0x8000 if j % 2 else 0)
    q, s = ops.cast_to_fp8(bits_to_bf16(block))
    q_ref, s_ref = oquant.cast_to_fp8_int(block)
    np.testing.assert_array_equal(fp8_bits(q), q_ref)
    np.testing.assert_array_equal(f32_bits(s), s_ref.view(np.uint32))


@pytest.mark.parametrize("tokens,hidden", [(3, 16), (9, 144), (17, 2064), (5, 7168 + 64), (4, 112)])
def test_cast_to_fp8_short_last_block(ops, tokens, hidden):
    """Widths that are not multiples of 128: the last block is quantised as if padded with zeros
    (deep_ep/utils/math.py:52-53), bit for bit against the reference expression on the padded row."""
    gen = torch.Generator().manual_seed(hidden)
    x = (torch.randn(tokens, hidden, generator=gen) * 3).bfloat16()
    x[0, -16:] = 0  # a short block of zeros: amax floor 1e-4
    padded = torch.nn.functional.pad(x, (0, (-hidden) % 128))
    q_ref, s_ref = oquant.cast_to_fp8_torch(padded)
    q, s = ops.cast_to_fp8(x.cuda())
    assert tuple(s.shape) == (tokens, (hidden + 127) // 128)
    np.testing.assert_array_equal(fp8_bits(q), fp8_bits(q_ref)[:, :hidden])
    np.testing.assert_array_equal(f32_bits(s), f32_bits(s_ref))


@pytest.mark.parametrize("tokens,hidden", [(7, 200), (3, 5), (2, 129), (4, 7168 + 33)])
def test_per_token_cast_to_fp8_any_width(tokens, hidden):
    """The public helper takes any width, like the reference's (deep_ep/utils/math.py:44-61 zero-pads to 128)."""
    from deepep_amd.utils import per_token_cast_to_fp8

    x = (torch.randn(tokens, hidden, generator=torch.Generator().manual_seed(hidden)) * 2).bfloat16()
    q_ref, s_ref = oquant.cast_to_fp8_torch(torch.nn.functional.pad(x, (0, (-hidden) % 128)))
    q, s = per_token_cast_to_fp8(x.cuda())
    assert tuple(q.shape) == (tokens, hidden) and q.is_contiguous() and tuple(s.shape) == (tokens, (hidden + 127) // 128)
    np.testing.assert_array_equal(fp8_bits(q), fp8_bits(q_ref)[:, :hidden])
    np.testing.assert_array_equal(f32_bits(s), f32_bits(s_ref))


def _finite_codes(shape, seed):
    codes = np.random.default_rng(seed).integers(0, 256, shape, dtype=np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x7E  # 0x7F / 0xFF are NaN in e4m3fn; checked apart
    return codes


def test_cast_back_every_code_and_scale_bit_exact(ops):
    """The dequantiser (per_token_cast_back, deep_ep/utils/math.py:64-79): every finite e4m3fn code under scales from
    2^-30 to 2^20 and non-powers of two, bit for bit against the oracle; NaN codes stay NaN."""
    scales = np.array([2.0 ** -30, 1e-4 / 448, 0.001, 1 / 3, 1.0, 1.5, 448.0 / 7, 2.0 ** 20], dtype=np.float32)
    codes = np.tile(np.arange(256, dtype=np.uint8), (scales.size, 1))  # row i: all codes, one 256-column row = 2 blocks
    nan = (codes & 0x7F) == 0x7F
    finite = np.where(nan, 0, codes).astype(np.uint8)
    row_scales = np.stack([scales, scales[::-1]], axis=1).copy()  # a different scale for each of the two blocks
    got = ops.cast_back(torch.from_numpy(finite).cuda().view(torch.float8_e4m3fn), torch.from_numpy(row_scales).cuda())
    np.testing.assert_array_equal(bf16_bits(got), oquant.cast_back(finite, row_scales))
    got_nan = ops.cast_back(torch.from_numpy(codes).cuda().view(torch.float8_e4m3fn), torch.from_numpy(row_scales).cuda())
    assert torch.isnan(got_nan.float().cpu()).numpy()[nan].all()
    np.testing.assert_array_equal(bf16_bits(got_nan)[~nan], oquant.cast_back(finite, row_scales)[~nan])


@pytest.mark.parametrize("tokens,hidden", [(1, 128), (33, 7168), (5, 16), (7, 144), (12, 2064)])
def test_cast_back_widths_and_packed_exponent_scales(ops, tokens, hidden):
    """Widths that are not multiples of 128 (short last block, as the reference pads) and the int32 form of the scales
    (four e8m0 exponent bytes each, math.py:74-76), against the same expression evaluated with torch on the host."""
    from deepep_amd.utils import per_token_cast_back

    blocks = (hidden + 127) // 128
    codes = torch.from_numpy(_finite_codes((tokens, hidden), hidden)).view(torch.float8_e4m3fn)
    scales = torch.rand(tokens, blocks, generator=torch.Generator().manual_seed(tokens)) * 4 + 1e-3
    want = per_token_cast_back(codes, scales)  # host tensors: plain torch
    got = per_token_cast_back(codes.cuda(), scales.cuda())  # device tensors: the HIP kernel
    np.testing.assert_array_equal(bf16_bits(got), bf16_bits(want))
    if blocks % 4 == 0:
        exponents = torch.randint(100, 140, (tokens, blocks), generator=torch.Generator().manual_seed(1), dtype=torch.uint8)
        packed = exponents.view(torch.int32)
        want = per_token_cast_back(codes, packed)
        got = per_token_cast_back(codes.cuda(), packed.cuda())
        np.testing.assert_array_equal(bf16_bits(got), bf16_bits(want))
        as_float = torch.pow(2.0, exponents.float() - 127)
        np.testing.assert_array_equal(bf16_bits(got), bf16_bits(per_token_cast_back(codes, as_float)))


def test_cast_back_restores_what_cast_to_fp8_made(ops):
    """Round trip on the device: quantise, dequantise, compare with the oracle's round trip bit for bit and with the input
    to the format's precision (2^-4 relative per element at most, e4m3 has 3 mantissa bits)."""
    x, _, _, _ = cases.make_inputs("C2")
    q, s = ops.cast_to_fp8(x.cuda())
    back = ops.cast_back(q, s)
    q_ref, s_ref = oquant.cast_to_fp8_torch(x)
    np.testing.assert_array_equal(bf16_bits(back), oquant.cast_back(fp8_bits(q_ref), s_ref.numpy()))
    err = (back.float().cpu() - x.float()).abs()
    bound = x.float().abs().view(x.shape[0], -1, 128).amax(-1, keepdim=True).expand(-1, -1, 128).reshape(x.shape) / 16
    assert (err <= bound + 1e-6).all()


@pytest.mark.parametrize("name,tokens", [("C1", None), ("C2", None), ("C3", 700), ("C4", 4096)])
def test_dispatch_quant_fp8_fused_equals_quantize_then_copy(ops, ws, name, tokens):
    x, idx, w, cfg = cases.make_inputs(name, tokens=tokens)
    q_ref, s_ref = oquant.cast_to_fp8_torch(x)
    got, want, rows = _check_layout(ops, ws, idx.numpy(), cfg["experts"], cfg["expert_begin"], cfg["num_local"])
    out, out_s, out_w = ops.dispatch_quant_fp8(x.cuda(), w.cuda(), got["route_to_row"], got["row_to_route"], rows)
    np.testing.assert_array_equal(fp8_bits(out), olayout.expand_rows(fp8_bits(q_ref), want["row_to_route"], cfg["topk"]))
    np.testing.assert_array_equal(f32_bits(out_s), olayout.expand_rows(f32_bits(s_ref), want["row_to_route"], cfg["topk"]))
    np.testing.assert_array_equal(f32_bits(out_w), olayout.expand_weights(w.numpy(), want["row_to_route"]).view(np.uint32))


@pytest.mark.parametrize("name,tokens", [("C1", None), ("C2", None), ("C3", 600), ("C4", 4096)])
@pytest.mark.parametrize("weighted", [False, True])
def test_combine_matches_oracle(ops, ws, name, tokens, weighted):
    x, idx, w, cfg = cases.make_inputs(name, tokens=tokens)
    got, want, rows = _check_layout(ops, ws, idx.numpy(), cfg["experts"], cfg["expert_begin"], cfg["num_local"])
    gen = torch.Generator().manual_seed(5)
    y = torch.randn(rows, cfg["hidden"], generator=gen).bfloat16()
    w_rows = torch.from_numpy(olayout.expand_weights(w.numpy(), want["row_to_route"]))
    ret = torch.rand(rows, generator=gen)
    out, returned = ops.combine(y.cuda(), got["route_to_row"], w_rows.cuda() if weighted else None, ret.cuda())
    ref = ocombine.combine(bf16_bits(y), want["route_to_row"], w_rows.numpy() if weighted else None)
    np.testing.assert_array_equal(bf16_bits(out), ref)
    np.testing.assert_array_equal(f32_bits(returned), ocombine.return_weights(ret.numpy(), want["route_to_row"]).view(np.uint32))


@pytest.mark.parametrize("hidden,topk", [(8, 2), (520, 3), (1096, 8), (7176, 12), (2048, 32)])
def test_combine_dense_ragged_widths_and_long_topk(ops, hidden, topk):
    """Dense routing takes column parts of 64 16-byte vectors, a wave each: widths that end in a short part (or are
    shorter than one part), and more slots than one batch of loads holds, against the oracle."""
    gen = torch.Generator().manual_seed(hidden + topk)
    tokens, experts = 130, 40
    idx = torch.stack([torch.randperm(experts, generator=gen)[:topk] for _ in range(tokens)])
    idx[5, :] = -1
    idx[9, 0] = experts  # invalid id
    want = olayout.layout(idx.numpy(), experts)
    rows = want["num_rows"]
    assert rows >= tokens  # dense: at least a row per token
    y = torch.randn(rows, hidden, generator=gen).bfloat16()
    w_rows = torch.rand(rows, generator=gen)
    r2r = torch.from_numpy(want["route_to_row"]).cuda()
    for weights in (None, w_rows):
        out, _ = ops.combine(y.cuda(), r2r, None if weights is None else weights.cuda())
        ref = ocombine.combine(bf16_bits(y), want["route_to_row"], None if weights is None else weights.numpy())
        np.testing.assert_array_equal(bf16_bits(out), ref)


def test_combine_reference_bounded_integer_fixture(ops, ws):
    # tests/elastic/test_combine.py:496-515: exact sums base*count + sum((e%3-1)+(s%3-1))
    tokens, hidden, experts, topk, generation = 333, 7168, 64, 8, 2
    idx = np.asarray(cases.matrix_routes(1, experts, topk, [tokens])[0])
    idx[7, :] = -1
    got, want, rows = _check_layout(ops, ws, idx, experts)
    base = cases.combine_payload_values(0, tokens, generation, hidden)
    route = want["row_to_route"]
    e, s = idx.reshape(-1)[route], route % topk
    y = torch.from_numpy(olayout.expand_rows(base, route, topk) + ((e % 3 - 1) + (s % 3 - 1))[:, None].astype(np.float32)).bfloat16()
    out, _ = ops.combine(y.cuda(), got["route_to_row"])
    expected = cases.combine_expected_values(idx.tolist(), experts, 0, generation, hidden)
    np.testing.assert_array_equal(out.float().cpu().numpy(), expected)


def test_combine_order_and_unfused_arithmetic(ops):
    big = 2.0**24
    y = torch.tensor([[big] * 8, [1.0] * 8, [-big] * 8]).bfloat16().cuda()
    r2r = torch.tensor([[0, 1, 2], [0, 2, 1]], dtype=torch.int32).cuda()
    out, _ = ops.combine(y, r2r)
    assert out.float().cpu()[:, 0].tolist() == [0.0, 1.0]
    a, w, c = np.float32(1.0 + 2.0**-7), np.float32(1.0 + 2.0**-23), np.float32(-1.0)
    y = torch.tensor([[float(a)] * 8, [float(c)] * 8]).bfloat16().cuda()
    out, _ = ops.combine(y, torch.tensor([[0, 1]], dtype=torch.int32).cuda(), torch.tensor([float(w), 1.0]).cuda())
    unfused = np.float32(np.float32(a * w) + c)
    assert out.float().cpu()[0, 0].item() == torch.tensor(float(unfused)).bfloat16().float().item()


def test_roundtrip_identity_multiplicity(ops, ws):
    # dispatch then unweighted combine of the untouched rows gives x * (number of valid slots), exactly
    # when x is small-integer valued (tests/test_reference.py:88-97).
    tokens, hidden, experts, topk = 500, 256, 32, 8
    rng = np.random.default_rng(1)
    idx = rng.integers(-1, experts, size=(tokens, topk))
    x = torch.from_numpy(rng.integers(-8, 9, size=(tokens, hidden)).astype(np.float32)).bfloat16()
    got, want, rows = _check_layout(ops, ws, idx, experts)
    out, _, _ = ops.dispatch_copy(x.cuda(), None, None, got["route_to_row"], got["row_to_route"], rows)
    back, _ = ops.combine(out, got["route_to_row"])
    count = (idx >= 0).sum(axis=1, keepdims=True).astype(np.float32)
    np.testing.assert_array_equal(back.float().cpu().numpy(), x.float().numpy() * count)


def test_full_size_prefill_properties(ops, ws):
    # the prefill shape at full size (T=4096, H=7168, E=256, K=8, Zipf): checks that do not need the oracle to
    # materialise 470 MB: row checksums of the FP8 payload against the token checksums, and the combine
    # of the dispatched BF16 rows against count * x on integer-valued input.
    x, idx, w, cfg = cases.make_inputs("C3")
    got, want, rows = _check_layout(ops, ws, idx.numpy(), cfg["experts"])
    assert rows == 4096 * 8
    xd = x.cuda()
    q, s = ops.cast_to_fp8(xd)
    out, out_s, out_w = ops.dispatch_quant_fp8(xd, w.cuda(), got["route_to_row"], got["row_to_route"], rows)
    token_of_row = (got["row_to_route"][:rows] // cfg["topk"]).long()
    assert torch.equal(out.view(torch.uint8), q.view(torch.uint8)[token_of_row])
    assert torch.equal(out_s.view(torch.int32), s.view(torch.int32)[token_of_row])
    assert torch.equal(out_w.view(torch.int32), w.cuda().view(-1).view(torch.int32)[got["row_to_route"][:rows].long()])
    xi = torch.randint(-8, 9, x.shape, generator=torch.Generator().manual_seed(1)).bfloat16().cuda()
    rows_bf16, _, _ = ops.dispatch_copy(xi, None, None, got["route_to_row"], got["row_to_route"], rows)
    back, _ = ops.combine(rows_bf16, got["route_to_row"])
    assert torch.equal(back.float(), xi.float() * 8)


def test_full_size_rank_share_properties(ops, ws):
    """The EP64 rank share at full size (64 x 256 = 16384 candidate tokens, 6 of 384 experts local, top-8, H=7168; the
    reference runs its payload checks at the configured size, tests/elastic/test_dispatch.py:1670-1908): the sparse-share
    kernels (row-major fused FP8 dispatch, served-only combine) against size-independent properties.  Rows of the
    fused dispatch equal the stand-alone quantiser's rows of their tokens; BF16 rows equal their tokens; the weighted
    combine of integer-valued rows is exact and can be stated per token; the served-only combine gives served tokens
    the full combine's rows and leaves the others untouched."""
    x, idx, w, cfg = cases.make_inputs("C4")
    tokens, hidden, topk = cfg["tokens"], cfg["hidden"], cfg["topk"]
    assert tokens == 16384 and hidden == 7168
    got, want, rows = _check_layout(ops, ws, idx.numpy(), cfg["experts"], cfg["expert_begin"], cfg["num_local"])
    assert 1500 < rows < 2600 and rows <= tokens  # sparse share: the row-major kernels run
    xd, wd = x.cuda(), w.cuda()
    route = got["row_to_route"][:rows].long()
    token_of_row = route // topk
    q, s = ops.cast_to_fp8(xd)
    out, out_s, out_w = ops.dispatch_quant_fp8(xd, wd, got["route_to_row"], got["row_to_route"], rows)
    assert torch.equal(out.view(torch.uint8), q.view(torch.uint8)[token_of_row])
    assert torch.equal(out_s.view(torch.int32), s.view(torch.int32)[token_of_row])
    assert torch.equal(out_w.view(torch.int32), wd.view(-1).view(torch.int32)[route])
    # the pre-quantised copy and the BF16 copy move the same rows
    cq, cs, _ = ops.dispatch_copy(q, s, None, got["route_to_row"], got["row_to_route"], rows)
    assert torch.equal(cq.view(torch.uint8), out.view(torch.uint8)) and torch.equal(cs.view(torch.int32), out_s.view(torch.int32))
    xi = torch.randint(-8, 9, x.shape, generator=torch.Generator().manual_seed(2)).bfloat16().cuda()
    rows_bf16, _, _ = ops.dispatch_copy(xi, None, None, got["route_to_row"], got["row_to_route"], rows)
    assert torch.equal(rows_bf16.view(torch.int16), xi.view(torch.int16)[token_of_row])
    # weights k / 4 and |x| <= 8: every product and partial sum is exact, so the combine is x * (sum of the weights of
    # the token's local slots) whatever the order
    slot_w = ((torch.arange(rows) % 4 + 1).float() / 4).cuda()
    local = got["route_to_row"] >= 0
    weight_sum = torch.zeros(tokens, device="cuda")
    weight_sum.index_add_(0, token_of_row, slot_w)
    full, _ = ops.combine(rows_bf16, got["route_to_row"], slot_w)
    assert torch.equal(full.float(), xi.float() * weight_sum[:, None])
    served = local.any(dim=1)
    assert 0 < int(served.sum()) < tokens
    sentinel = torch.full((tokens, hidden), 7.0, dtype=torch.bfloat16, device="cuda")
    part, _ = ops.combine(rows_bf16, got["route_to_row"], slot_w, out=sentinel.clone(), served_only=True)
    assert torch.equal(part[served].view(torch.int16), full[served].view(torch.int16))
    assert torch.equal(part[~served], sentinel[~served]) and not full[~served].any()
    # N(0,1) rows: no closed form, but the two combines must still agree on the served tokens, unweighted too
    y = torch.randn(rows, hidden, generator=torch.Generator().manual_seed(3)).bfloat16().cuda()
    for row_w in (None, out_w):
        full, _ = ops.combine(y, got["route_to_row"], row_w)
        part, _ = ops.combine(y, got["route_to_row"], row_w, out=sentinel.clone(), served_only=True)
        assert torch.equal(part[served].view(torch.int16), full[served].view(torch.int16))
        assert torch.equal(part[~served], sentinel[~served])


def test_argument_errors(ops, ws):
    idx = torch.zeros((4, 2), dtype=torch.int64).cuda()
    with pytest.raises(ValueError):
        ops.layout(ws, idx, 4, 3, 2)  # local range past E
    with pytest.raises(ValueError):
        ops.layout(ws, idx.int(), 4)  # wrong dtype
    lay = ops.layout(ws, idx, 4)
    x = torch.zeros((4, 24), dtype=torch.bfloat16).cuda()
    with pytest.raises(ValueError):
        ops.dispatch_copy(x[:, :20].contiguous(), None, None, lay["route_to_row"], lay["row_to_route"], 8)  # 40-byte rows
    with pytest.raises(ValueError):
        ops.dispatch_quant_fp8(x, None, lay["route_to_row"], lay["row_to_route"], 8)  # H % 128
    with pytest.raises(ValueError):
        ops.combine(torch.zeros((8, 12), dtype=torch.bfloat16).cuda(), lay["route_to_row"])  # H % 8


def test_dispatch_moves_packed_int32_scales_and_fp16_payload(ops, ws):
    # low-latency formats pass through unchanged: FP16 payload rows and int32 words of four packed E8M0 bytes
    rng = np.random.default_rng(3)
    tokens, topk, experts, hidden = 64, 4, 16, 512
    idx_np = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)])
    lay = ops.layout(ws, torch.from_numpy(idx_np).cuda(), experts)
    _, rows = ops.layout_wait(ws)
    want = olayout.layout(idx_np, experts)
    x = torch.from_numpy(rng.normal(size=(tokens, hidden)).astype(np.float16)).cuda()
    packed = torch.from_numpy(rng.integers(-2**31, 2**31 - 1, size=(tokens, hidden // 128), dtype=np.int64).astype(np.int32)).cuda()
    out, out_scales, _ = ops.dispatch_copy(x, packed, None, lay["route_to_row"], lay["row_to_route"], rows)
    token_of_row = want["row_to_route"] // topk
    assert out.dtype == torch.float16 and out_scales.dtype == torch.int32
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint16), x.cpu().numpy().view(np.uint16)[token_of_row])
    np.testing.assert_array_equal(out_scales.cpu().numpy(), packed.cpu().numpy()[token_of_row])


@pytest.mark.parametrize("name,tokens", [("C1", None), ("C2", None), ("C3", 700), ("C4", 2048)])
def test_dispatch_before_the_host_knows_the_row_count(ops, ws, name, tokens):
    """num_rows=None: layout and payload kernels queued back to back into outputs of T*K rows; the first R rows
    equal those of a dispatch sized after the read-back, for the BF16 copy and the fused FP8 path, in dense and
    rank-share routing alike."""
    x, idx, w, cfg = cases.make_inputs(name, tokens=tokens)
    xd, wd = x.cuda(), w.cuda()
    lay = ops.layout(ws, idx.cuda(), cfg["experts"], cfg["expert_begin"], cfg["num_local"])
    early = ops.dispatch_copy(xd, None, wd, lay["route_to_row"], lay["row_to_route"], None)
    early_q = ops.dispatch_quant_fp8(xd, wd, lay["route_to_row"], lay["row_to_route"], None)
    _, rows = ops.layout_wait(ws)
    assert early[0].shape[0] == early_q[0].shape[0] == idx.numel() and early[1] is None
    late = ops.dispatch_copy(xd, None, wd, lay["route_to_row"], lay["row_to_route"], rows)
    late_q = ops.dispatch_quant_fp8(xd, wd, lay["route_to_row"], lay["row_to_route"], rows)
    want = olayout.layout(idx.numpy(), cfg["experts"], cfg["expert_begin"], cfg["num_local"])
    assert rows == want["num_rows"]
    np.testing.assert_array_equal(bf16_bits(early[0][:rows]), olayout.expand_rows(bf16_bits(x), want["row_to_route"], cfg["topk"]))
    np.testing.assert_array_equal(bf16_bits(early[0][:rows]), bf16_bits(late[0]))
    np.testing.assert_array_equal(f32_bits(early[2][:rows]), f32_bits(late[2]))
    np.testing.assert_array_equal(fp8_bits(early_q[0][:rows]), fp8_bits(late_q[0]))
    np.testing.assert_array_equal(f32_bits(early_q[1][:rows]), f32_bits(late_q[1]))
    np.testing.assert_array_equal(f32_bits(early_q[2][:rows]), f32_bits(late_q[2]))


@pytest.mark.parametrize("weighted", [False, True])
def test_combine_fp16_matches_oracle(ops, ws, weighted):
    """IEEE half rows and output (low-latency expert outputs may be FP16): bit-exact against the half oracle,
    including values that round differently in half and BF16 and a sum that overflows half to infinity."""
    x, idx, w, cfg = cases.make_inputs("C2")
    got, want, rows = _check_layout(ops, ws, idx.numpy(), cfg["experts"])
    gen = torch.Generator().manual_seed(9)
    y = (torch.randn(rows, cfg["hidden"], generator=gen) * 3).half()
    y[0, :8] = 60000.0  # several of these in one token overflow the half range
    w_rows = torch.from_numpy(olayout.expand_weights(w.numpy(), want["row_to_route"]))
    out, _ = ops.combine(y.cuda(), got["route_to_row"], w_rows.cuda() if weighted else None)
    assert out.dtype == torch.float16
    ref = ocombine.combine_fp16(y.numpy(), want["route_to_row"], w_rows.numpy() if weighted else None)
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint16), ref.view(np.uint16))


def test_random_shapes_end_to_end(ops, ws):
    """Forty seeded shapes off the beaten path (token counts that are not multiples of the 64-route step, top-k that
    does not divide it, expert counts that are not powers of two, receive shares, masked and repeated experts):
    layout, BF16 dispatch with weights, fused FP8 dispatch and weighted combine, each bit-exact against the oracle."""
    rng = np.random.default_rng(2024)
    for case in range(40):
        topk = int(rng.integers(1, 17))
        experts = int(rng.integers(topk, 600))
        tokens = int(rng.integers(1, 2500))
        hidden = int(rng.choice([128, 256, 384, 1024, 2048]))
        if case % 3 == 0:  # a receive share: a contiguous range of local experts
            local = int(rng.integers(1, experts + 1))
            begin = int(rng.integers(0, experts - local + 1))
        else:
            begin, local = 0, experts
        idx = rng.integers(-1, experts + 1, size=(tokens, topk))  # -1 and E are both "no expert"; repeats allowed
        label = f"case {case}: T={tokens} K={topk} E={experts} begin={begin} L={local} H={hidden}"
        got, want, rows = _check_layout(ops, ws, idx, experts, begin, local)
        gen = torch.Generator().manual_seed(case)
        x = torch.randn(tokens, hidden, generator=gen).bfloat16()
        w = torch.rand(tokens, topk, generator=gen)
        out, _, out_w = ops.dispatch_copy(x.cuda(), None, w.cuda(), got["route_to_row"], got["row_to_route"], rows)
        np.testing.assert_array_equal(bf16_bits(out), olayout.expand_rows(bf16_bits(x), want["row_to_route"], topk), err_msg=label)
        w_rows = olayout.expand_weights(w.numpy(), want["row_to_route"])
        np.testing.assert_array_equal(f32_bits(out_w), w_rows.view(np.uint32), err_msg=label)
        q_ref, s_ref = oquant.cast_to_fp8_torch(x)
        q, s, _ = ops.dispatch_quant_fp8(x.cuda(), None, got["route_to_row"], got["row_to_route"], None)  # R not passed
        np.testing.assert_array_equal(fp8_bits(q[:rows]), olayout.expand_rows(fp8_bits(q_ref), want["row_to_route"], topk), err_msg=label)
        np.testing.assert_array_equal(f32_bits(s[:rows]), olayout.expand_rows(f32_bits(s_ref), want["row_to_route"], topk), err_msg=label)
        y = torch.randn(rows, hidden, generator=gen).bfloat16()
        combined, _ = ops.combine(y.cuda(), got["route_to_row"], torch.from_numpy(w_rows).cuda())
        np.testing.assert_array_equal(bf16_bits(combined), ocombine.combine(bf16_bits(y), want["route_to_row"], w_rows), err_msg=label)


SMALL_SHAPES = [
    # tokens, topk, experts, begin, local, hidden
    (128, 8, 256, 0, 256, 7168),   # the decode shape
    (128, 8, 256, 64, 32, 1024),   # a rank's share: most routes elsewhere
    (1, 1, 4, 0, 4, 128),
    (37, 6, 48, 8, 24, 384),
    (64, 32, 1024, 0, 1024, 256),  # the largest top-k and expert count, 2048 routes
    (256, 8, 16, 0, 16, 512),      # few experts: long runs per expert
]


@pytest.mark.parametrize("tokens,topk,experts,begin,local,hidden", SMALL_SHAPES)
@pytest.mark.parametrize("mode", ["bf16", "fp8_copy", "fp8_quant", "fp16"])
def test_layout_and_dispatch_in_one_launch(ops, ws, tokens, topk, experts, begin, local, hidden, mode):
    """Small batches: layout and payload from one kernel, every workgroup working out its own token's rows.  All
    layout outputs, the host mailbox and the dispatched payload / scales / weights against the oracle, bit for bit."""
    rng = np.random.default_rng(tokens * 7 + topk + hidden)
    idx_np = rng.integers(-1, experts + 1, size=(tokens, topk))  # includes -1 and == E, and repeated experts
    idx = torch.from_numpy(idx_np).cuda()
    x = torch.from_numpy(rng.normal(size=(tokens, hidden)).astype(np.float32)).bfloat16()
    w = torch.from_numpy(rng.random((tokens, topk)).astype(np.float32))
    want = olayout.layout(idx_np, experts, begin, local)
    rows = want["num_rows"]
    scales = None
    if mode == "fp8_copy":
        q, s = oquant.cast_to_fp8_torch(x) if hidden % 128 == 0 else (x.to(torch.float8_e4m3fn), torch.rand(tokens, 3))
        payload, scales = q.cuda(), s.cuda()
    elif mode == "fp16":
        payload = x.to(torch.float16).cuda()
    else:
        payload = x.cuda()
    if mode == "fp8_quant" and hidden % 128:
        pytest.skip("the fused quantiser needs a width that is a multiple of 128")
    lay, out, out_scales, out_w = ops.layout_dispatch_small(ws, idx, payload, scales, w.cuda(), experts, begin, local,
                                                            quantize=mode == "fp8_quant")
    counts, got_rows = ops.layout_wait(ws, local)
    assert got_rows == rows == int(lay["num_rows"].item()) and counts == [int(c) for c in want["counts"]]
    np.testing.assert_array_equal(i32(lay["counts"]), want["counts"])
    np.testing.assert_array_equal(i32(lay["psum"]), want["psum"])
    np.testing.assert_array_equal(i32(lay["offsets"]), want["offsets"])
    np.testing.assert_array_equal(i32(lay["route_to_row"]), want["route_to_row"])
    np.testing.assert_array_equal(i32(lay["row_to_route"])[:rows], want["row_to_route"])
    assert out.shape[0] == tokens * topk
    if mode == "fp8_quant":
        q_ref, s_ref = oquant.cast_to_fp8_torch(x)
        np.testing.assert_array_equal(fp8_bits(out[:rows]), olayout.expand_rows(q_ref.view(torch.uint8).numpy(), want["row_to_route"], topk))
        np.testing.assert_array_equal(f32_bits(out_scales[:rows]), olayout.expand_rows(s_ref.numpy().view(np.uint32), want["row_to_route"], topk))
    else:
        source = payload.cpu().view(torch.uint8 if payload.element_size() == 1 else torch.int16).numpy()
        got = out[:rows].cpu().view(torch.uint8 if payload.element_size() == 1 else torch.int16).numpy()
        np.testing.assert_array_equal(got, olayout.expand_rows(source, want["row_to_route"], topk))
        if scales is not None:
            np.testing.assert_array_equal(f32_bits(out_scales[:rows]), olayout.expand_rows(f32_bits(scales), want["row_to_route"], topk))
    np.testing.assert_array_equal(f32_bits(out_w[:rows]), olayout.expand_weights(w.numpy(), want["row_to_route"]).view(np.uint32))


def test_layout_dispatch_small_limits(ops, ws):
    idx = torch.zeros((300, 8), dtype=torch.int64, device="cuda")  # 2400 routes
    x = torch.zeros((300, 128), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="routes"):
        ops.layout_dispatch_small(ws, idx, x, None, None, 16)


def test_decode_step_in_hip_graph(ops):
    """A decode step (routing layout + BF16 dispatch in one launch, then the weighted combine) has no host
    synchronisation, so a serving loop can capture it once and replay it with new tokens and routes in the same
    buffers.  Every replay is checked against the eager result of the same inputs and against the oracle."""
    tokens, hidden, topk, experts = 96, 2048, 8, 64
    dev = "cuda"
    workspace = ops.Workspace(1 << 20)
    x = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)
    idx = torch.empty((tokens, topk), dtype=torch.int64, device=dev)
    w = torch.empty((tokens, topk), dtype=torch.float32, device=dev)
    result = {}

    def inputs(seed):
        gen = torch.Generator().manual_seed(seed)
        ids = torch.stack([torch.randperm(experts, generator=gen)[:topk] for _ in range(tokens)])
        ids[seed % tokens, 0] = -1  # a masked route
        return torch.randn(tokens, hidden, generator=gen).bfloat16(), ids, torch.rand(tokens, topk, generator=gen)

    def load(problem):
        x.copy_(problem[0]); idx.copy_(problem[1]); w.copy_(problem[2])

    def step():
        lay, rows, _, row_w = ops.layout_dispatch_small(workspace, idx, x, None, w, experts)
        result["out"] = ops.combine(rows, lay["route_to_row"], row_w)[0]
        result["counts"] = lay["counts"]

    problems = [inputs(seed) for seed in (21, 22, 23)]
    try:
        eager = []
        for problem in problems:
            load(problem)
            step()
            torch.cuda.synchronize()
            eager.append((result["out"].clone(), result["counts"].clone()))
            want = olayout.layout(problem[1].numpy(), experts)
            want_rows = olayout.expand_rows(bf16_bits(problem[0]), want["row_to_route"], topk)
            want_w = olayout.expand_weights(problem[2].numpy(), want["row_to_route"])
            want_out = ocombine.combine(want_rows, want["route_to_row"], want_w)
            np.testing.assert_array_equal(bf16_bits(eager[-1][0]), want_out)
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()  # warm-up on the capture stream
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            step()
        for turn in range(2):
            for problem, (want_out, want_counts) in zip(problems, eager):
                load(problem)
                result["out"].zero_()
                torch.cuda.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(result["counts"], want_counts)
                assert torch.equal(result["out"].view(torch.int16), want_out.view(torch.int16)), f"replay {turn} differs from eager"
    finally:
        torch.cuda.synchronize()
        workspace.destroy()


@pytest.mark.parametrize("weighted", [False, True])
def test_combine_served_only_leaves_unserved_tokens_untouched(ops, ws, weighted):
    """One rank's share: tokens without a local route keep what the output held (the reference produces nothing for them
    on this rank), tokens with one get exactly what the zero-filling combine gives them."""
    x, idx, w, cfg = cases.make_inputs("C4", tokens=3000)
    got, want, rows = _check_layout(ops, ws, idx.numpy(), cfg["experts"], cfg["expert_begin"], cfg["num_local"])
    gen = torch.Generator().manual_seed(9)
    y = torch.randn(rows, cfg["hidden"], generator=gen).bfloat16().cuda()
    row_w = torch.rand(rows, generator=gen).cuda() if weighted else None
    back = torch.rand(rows, generator=gen).cuda()
    full, full_back = ops.combine(y, got["route_to_row"], row_w, back)
    sentinel = torch.full((idx.shape[0], cfg["hidden"]), 7.0, dtype=torch.bfloat16, device="cuda")
    part, part_back = ops.combine(y, got["route_to_row"], row_w, back, out=sentinel.clone(), served_only=True)
    served = torch.from_numpy((want["route_to_row"] >= 0).any(axis=1)).cuda()
    assert 0 < int(served.sum()) < idx.shape[0]
    assert torch.equal(part[served].view(torch.int16), full[served].view(torch.int16))
    assert torch.equal(part[~served], sentinel[~served]) and not full[~served].any()
    assert torch.equal(part_back, full_back)
    with pytest.raises(ValueError, match="served_only"):
        ops.combine(y, got["route_to_row"], row_w, served_only=True)


@pytest.mark.parametrize("topk", [1, 6, 32])
def test_combine_served_only_any_topk(ops, topk):
    """The served-only reduce deals 256 // top-k tokens to a workgroup: top-k values that do not divide 256, a ragged last
    workgroup and tokens with several rows give what the zero-filling combine gives on the served tokens."""
    gen = torch.Generator().manual_seed(100 + topk)
    tokens, hidden = 1003, 1024
    routes = tokens * topk
    rows = max(routes // 12, 8)
    route_to_row = torch.full((routes,), -1, dtype=torch.int32)
    route_to_row[torch.randperm(routes, generator=gen)[:rows]] = torch.randperm(rows, generator=gen).int()
    route_to_row = route_to_row.view(tokens, topk).cuda()
    y = torch.randn(rows, hidden, generator=gen).bfloat16().cuda()
    row_w = torch.rand(rows, generator=gen).cuda()
    back = torch.rand(rows, generator=gen).cuda()
    full, full_back = ops.combine(y, route_to_row, row_w, back)
    sentinel = torch.full((tokens, hidden), -3.0, dtype=torch.bfloat16, device="cuda")
    part, part_back = ops.combine(y, route_to_row, row_w, back, out=sentinel.clone(), served_only=True)
    served = (route_to_row >= 0).any(dim=1)
    assert 0 < int(served.sum()) < tokens
    assert torch.equal(part[served].view(torch.int16), full[served].view(torch.int16))
    assert torch.equal(part[~served], sentinel[~served])
    assert torch.equal(part_back, full_back)


def test_share_without_rows_takes_scales_and_weights(ops, ws):
    """A rank none of whose experts is routed to: the outputs are empty tensors (null pointers at the C boundary), with
    scales and weights present on the input side; both dispatch entry points return empty outputs instead of rejecting the
    call."""
    tokens, topk, hidden = 5, 2, 256
    idx = torch.zeros((tokens, topk), dtype=torch.int64, device="cuda")  # every route to expert 0
    lay = ops.layout(ws, idx, 4, 2, 2)  # this rank holds experts 2 and 3
    _, rows = ops.layout_wait(ws)
    assert rows == 0
    x = torch.randn(tokens, hidden, device="cuda").bfloat16()
    weights = torch.rand(tokens, topk, device="cuda")
    codes, scales = ops.cast_to_fp8(x)
    out, out_scales, out_weights = ops.dispatch_copy(codes, scales, weights, lay["route_to_row"], lay["row_to_route"], 0)
    assert out.shape == (0, hidden) and out_scales.shape == (0, hidden // 128) and out_weights.shape == (0,)
    out, out_scales, out_weights = ops.dispatch_quant_fp8(x, weights, lay["route_to_row"], lay["row_to_route"], 0)
    assert out.shape == (0, hidden) and out_scales.shape == (0, hidden // 128) and out_weights.shape == (0,)
    combined, returned = ops.combine(torch.empty((0, hidden), dtype=torch.bfloat16, device="cuda"), lay["route_to_row"],
                                     return_values=torch.empty((0,), device="cuda"))
    assert not combined.any() and not returned.any()


def test_quantiser_on_infinities_and_nans(ops, ws):
    """Blocks that hold inf or NaN through the stand-alone quantiser, the fused dispatch (both grids) and the one-launch
    decode path: codes and scales bit for bit those of the reference expression (a NaN poisons its whole block: NaN scale,
    code 0x7F throughout; an infinite amax gives an infinite scale)."""
    import warnings

    from tests.gpu_util import non_finite_blocks

    x = non_finite_blocks()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)
        want_codes, want_scales = oquant.cast_to_fp8_int(bf16_bits(x))
    codes, scales = ops.cast_to_fp8(x.cuda())
    np.testing.assert_array_equal(fp8_bits(codes), want_codes)
    np.testing.assert_array_equal(f32_bits(scales), want_scales.view(np.uint32))
    tokens, topk, experts = x.shape[0], 2, 4
    idx = torch.stack([torch.arange(tokens) % experts, (torch.arange(tokens) + 1) % experts], dim=1).cuda()
    lay = ops.layout(ws, idx, experts)
    _, rows = ops.layout_wait(ws)
    want = olayout.layout(idx.cpu().numpy(), experts)
    for known in (rows, None):  # row-major grid (R known) and token-major grid (R not known yet)
        out, out_scales, _ = ops.dispatch_quant_fp8(x.cuda(), None, lay["route_to_row"], lay["row_to_route"], known)
        np.testing.assert_array_equal(fp8_bits(out[:rows]), olayout.expand_rows(want_codes, want["row_to_route"], topk))
        np.testing.assert_array_equal(f32_bits(out_scales[:rows]), olayout.expand_rows(want_scales, want["row_to_route"], topk).view(np.uint32))
    plan, out, out_scales, _ = ops.layout_dispatch_small(ws, idx, x.cuda(), None, None, experts, quantize=True)
    np.testing.assert_array_equal(fp8_bits(out[:rows]), olayout.expand_rows(want_codes, want["row_to_route"], topk))
    np.testing.assert_array_equal(f32_bits(out_scales[:rows]), olayout.expand_rows(want_scales, want["row_to_route"], topk).view(np.uint32))


def _same_but_for_nan_encoding(got_bits, want_bits):
    """Equal bit for bit, except that where both are NaN the sign and payload may differ (x86 and the GPU give the
    NaN produced by inf - inf, 0 * inf or a NaN operand different signs)."""
    got_nan, want_nan = (got_bits & 0x7FFF) > 0x7F80, (want_bits & 0x7FFF) > 0x7F80
    np.testing.assert_array_equal(got_nan, want_nan)
    np.testing.assert_array_equal(np.where(got_nan, 0, got_bits), np.where(want_nan, 0, want_bits))


def test_combine_and_cast_back_on_infinities_and_nans(ops):
    """Rows that hold +-inf, NaN, -0, the largest finite values and values that vanish in BF16, weights that are inf, 0,
    NaN, negative or huge: sums that overflow, inf - inf and 0 * inf all come out as in the oracle's fp32 arithmetic."""
    import warnings

    rng = np.random.default_rng(0)
    tokens, topk, experts, hidden = 64, 4, 8, 256
    idx = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int64)
    lay = olayout.layout(idx, experts)
    rows = lay["num_rows"]
    y = torch.from_numpy(rng.normal(size=(rows, hidden)).astype(np.float32)).bfloat16()
    special = [float("inf"), float("-inf"), float("nan"), -float("nan"), 3.3895e38, -3.3895e38, 0.0, -0.0, 1e-40]
    for i in range(0, rows, 3):
        y[i, rng.integers(0, hidden, size=6)] = torch.tensor([special[j] for j in rng.integers(0, len(special), size=6)]).bfloat16()
    w = rng.random(rows).astype(np.float32)
    w[::5], w[1::7], w[2::11], w[3::13], w[4::17] = np.inf, 0, np.nan, -1, 3e38
    route_to_row = torch.from_numpy(lay["route_to_row"]).cuda()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)
        for weights in (None, w):
            out, _ = ops.combine(y.cuda(), route_to_row, None if weights is None else torch.from_numpy(weights).cuda())
            _same_but_for_nan_encoding(bf16_bits(out), ocombine.combine(bf16_bits(y), lay["route_to_row"], weights))
        codes = rng.integers(0, 256, size=(8, 256), dtype=np.uint8)
        scales = rng.random((8, 2)).astype(np.float32)
        scales[0, 0], scales[1, 1], scales[2, 0], scales[3, 1], scales[4, 0], scales[5, 0] = np.inf, np.nan, 0, -1, 3e38, 1e-42
        got = ops.cast_back(torch.from_numpy(codes).cuda().view(torch.float8_e4m3fn), torch.from_numpy(scales).cuda())
        _same_but_for_nan_encoding(bf16_bits(got), oquant.cast_back(codes, scales))
