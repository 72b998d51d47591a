"""GPU parity of the W4A8 path: MX quantiser bit-exact; fused forward within 2e-2 relative Frobenius error
of the fp32 dequantised oracle (oracle/megamoe.py, restating the reference's NumPy oracle)."""

import numpy as np
import pytest
import torch

from oracle import megamoe as mm
from tests.gpu_util import bf16_bits, fp8_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from deepep_amd import ops as module

    return module


@pytest.mark.parametrize("scale", [1.0, 1e-3, 500.0, 1e-30, 1e30])
def test_mx_quant_bit_exact(ops, scale):
    gen = torch.Generator().manual_seed(3)
    x = (torch.randn(77, 1024, generator=gen) * scale).bfloat16()
    x[0, :32] = 0
    x[1, :32] = 448.0
    x[2, 5] = 3.0e38
    codes, scales = ops.mx_quant(x.cuda())
    ref_codes, ref_scales = mm.mx_quantize(x.float().numpy())
    np.testing.assert_array_equal(scales.cpu().numpy(), ref_scales)
    np.testing.assert_array_equal(fp8_bits(codes), ref_codes)


@pytest.mark.parametrize("rows,hidden", [(1, 32), (3, 96), (5, 4096), (129, 160), (64, 7168), (2, 8192 + 32)])
@pytest.mark.parametrize("scale_offset", [0, 1, 4])
def test_mx_quant_ragged_sizes_and_unaligned_scales(ops, rows, hidden, scale_offset):
    """Sizes that end inside a workgroup's 4096 values, and scale pointers off the 16-byte grid (the kernel then
    stores byte by byte), called through the C-ABI with caller-owned buffers."""
    import ctypes

    from deepep_amd import _lib

    gen = torch.Generator().manual_seed(rows * 131 + hidden)
    x = (torch.randn(rows, hidden, generator=gen) * 3.0).bfloat16().cuda()
    codes = torch.zeros(rows * hidden, dtype=torch.uint8, device="cuda")
    store = torch.full((rows * (hidden // 32) + 32,), 0xEE, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    status = _lib.load().dpep_mx_quant(ctypes.c_void_p(x.data_ptr()), rows, hidden, ctypes.c_void_p(codes.data_ptr()),
                                       ctypes.c_void_p(store.data_ptr() + scale_offset), ctypes.c_void_p(stream))
    _lib.check(status, "mx_quant")
    ref_codes, ref_scales = mm.mx_quantize(x.float().cpu().numpy())
    got = store.cpu().numpy()
    n = rows * (hidden // 32)
    np.testing.assert_array_equal(got[scale_offset:scale_offset + n].reshape(rows, -1), ref_scales)
    assert (got[:scale_offset] == 0xEE).all() and (got[scale_offset + n:] == 0xEE).all()  # nothing written outside
    np.testing.assert_array_equal(codes.cpu().numpy().reshape(rows, hidden), ref_codes)


def test_mx_quant_reference_anchors(ops):
    # experiments/megamoe/tests/test_reference.py:37-45
    x = torch.full((2, 64), 0.5)
    x[:, 32:] = 4.0
    codes, scales = ops.mx_quant(x.bfloat16().cuda())
    assert scales.cpu().tolist() == [[118, 121], [118, 121]]
    np.testing.assert_array_equal(mm.mx_dequantize(fp8_bits(codes), scales.cpu().numpy()), x.numpy())
    codes, scales = ops.mx_quant(torch.zeros(1, 32, dtype=torch.bfloat16).cuda())
    assert not fp8_bits(codes).any() and not scales.cpu().numpy().any()


def _make_problem(tokens, hidden, inter, experts, begin, local, topk, seed=0):
    rng = np.random.default_rng(seed)
    x = (rng.normal(size=(tokens, hidden))).astype(np.float32)
    x_codes, x_scales = mm.mx_quantize(x)
    w1 = (rng.normal(size=(local, 2 * inter, hidden)) * 0.02).astype(np.float32)
    w2 = (rng.normal(size=(local, hidden, inter)) * 0.02).astype(np.float32)
    p1, s1 = mm.quantize_weight_mxfp4(w1)
    p2, s2 = mm.quantize_weight_mxfp4(w2)
    idx = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    weights = rng.random((tokens, topk)).astype(np.float32)
    weights /= weights.sum(axis=1, keepdims=True)
    return x_codes, x_scales, (p1, s1), (p2, s2), idx, weights


def _oracle(x_codes, x_scales, l1, l2, idx, weights, begin):
    xq = mm.mx_dequantize(x_codes, x_scales)
    d1 = mm.unpack_weight(*l1)
    d2 = mm.unpack_weight(*l2)
    return mm.round_bf16(mm.local_reference(xq, idx, weights, d1, d2, begin))


def _run(ops, x_codes, x_scales, l1, l2, idx, weights, experts, begin, local, tile_rows=0, column_waves=1):
    tokens, hidden = x_codes.shape
    inter = l2[0].shape[2] * 2
    dev = "cuda"
    w1, s1 = ops.megamoe_prepare_weights(torch.from_numpy(l1[0]).to(dev), torch.from_numpy(l1[1]).reshape(local, 2 * inter, -1).to(dev), True)
    w2, s2 = ops.megamoe_prepare_weights(torch.from_numpy(l2[0]).to(dev), torch.from_numpy(l2[1]).reshape(local, hidden, -1).to(dev), False)
    ws = ops.Workspace(ops.megamoe_workspace_bytes(tokens, idx.shape[1], hidden, inter, local))
    ws.tune("gemm_tile_rows", tile_rows)
    ws.tune("gemm_column_waves", column_waves)
    y = torch.full((tokens, hidden), float("nan"), dtype=torch.bfloat16, device=dev)
    counts = torch.empty((local,), dtype=torch.int32, device=dev)
    ops.megamoe_forward(
        ws, torch.from_numpy(x_codes).to(dev).view(torch.float8_e4m3fn), torch.from_numpy(x_scales).to(dev),
        torch.from_numpy(idx).to(dev), torch.from_numpy(weights).to(dev), w1, s1, w2, s2, experts, begin, local, y, counts,
        intermediate=inter,
    )
    torch.cuda.synchronize()
    out = y.float().cpu().numpy(), counts.cpu().numpy()
    ws.destroy()
    return out


@pytest.mark.parametrize(
    "tokens,hidden,inter,experts,begin,local,topk",
    [
        (64, 512, 512, 4, 0, 4, 2),      # every expert local, tiny
        (300, 512, 512, 8, 2, 3, 4),     # ragged rows, local range inside E, partial tiles
        (257, 1024, 512, 6, 0, 6, 6),    # every token hits every expert
        (96, 512, 768, 8, 6, 2, 1),      # some local experts may be empty
        (200, 768, 1280, 4, 0, 4, 3),    # K of both GEMMs not a multiple of 512 (padded last scale span)
        (128, 512, 512, 64, 16, 32, 2),  # many local experts, most with a handful of rows, some empty
        (150, 1088, 384, 8, 0, 8, 2),    # hidden % 64, intermediate % 128 (the reference's granularity): padded to 1280 / 512
        (96, 1024, 256, 4, 0, 4, 2),     # the reference's smallest intermediate size
        (70, 576, 640, 4, 1, 2, 3),      # both padded, partial local range
        (40, 64, 128, 2, 0, 2, 1),       # the smallest sizes the entry point takes
    ],
)
def test_megamoe_forward_matches_oracle(ops, tokens, hidden, inter, experts, begin, local, topk):
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, begin, local, topk)
    got, counts = _run(ops, x_codes, x_scales, l1, l2, idx, weights, experts, begin, local)
    want = _oracle(x_codes, x_scales, l1, l2, idx, weights, begin)
    np.testing.assert_array_equal(counts, np.bincount(idx.ravel(), minlength=experts)[begin : begin + local])
    assert np.isfinite(got).all()
    err = mm.relative_frobenius(got, want)
    assert err <= 2e-2, err
    untouched = ~((idx >= begin) & (idx < begin + local)).any(axis=1)
    assert not got[untouched].any()  # tokens without a local expert receive zeros


@pytest.mark.parametrize("gate_up", [False, True])
@pytest.mark.parametrize("n,k", [(320, 576), (256, 64), (1024, 1088), (512, 384)])
def test_prepare_weights_pads_like_explicit_padding(ops, n, k, gate_up):
    """The prepared form of a raw tensor whose sizes are not what the GEMM works on equals, byte for byte, the prepared
    form of the same tensor padded by hand (zero codes, scale byte 127 = 1.0; gate and up halves padded separately)."""
    if gate_up and n % 256:
        pytest.skip("gate/up needs N = 2I with I % 128 == 0")
    rng = np.random.default_rng(n + k)
    experts = 2
    packed = rng.integers(0, 256, (experts, n, k // 2), dtype=np.uint8)
    scales = rng.integers(100, 140, (experts, n, k // 32), dtype=np.uint8)
    np_, kp, _ = ops.megamoe_prepared_shape(n, k, gate_up)
    assert kp == ops.megamoe_padded_dim(k) and kp % 256 == 0 and kp >= max(k, 512)
    halves = 2 if gate_up else 1
    big_packed = np.zeros((experts, np_, kp // 2), dtype=np.uint8)
    big_scales = np.full((experts, np_, kp // 32), 127, dtype=np.uint8)
    for h in range(halves):
        src = slice(h * n // halves, (h + 1) * n // halves)
        dst = slice(h * np_ // halves, h * np_ // halves + n // halves)
        big_packed[:, dst, : k // 2] = packed[:, src]
        big_scales[:, dst, : k // 32] = scales[:, src]
    got = ops.megamoe_prepare_weights(torch.from_numpy(packed).cuda(), torch.from_numpy(scales).cuda(), gate_up)
    want = ops.megamoe_prepare_weights(torch.from_numpy(big_packed).cuda(), torch.from_numpy(big_scales).cuda(), gate_up)
    assert got[0].shape == want[0].shape == (experts, np_, kp // 2)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


@pytest.mark.parametrize("tile_rows", [64, 128, 192])
@pytest.mark.parametrize(
    "tokens,hidden,inter,experts,begin,local,topk",
    [
        (300, 512, 512, 8, 2, 3, 4),     # k of both GEMMs = 512: four k tiles, fewer than the copies run ahead at 64 / 128 rows
        (200, 768, 1280, 4, 0, 4, 3),    # short last span in both GEMMs
        (512, 512, 1024, 64, 0, 64, 8),  # 64-row tiles: 512 tiles of four k tiles each, two per workgroup, in the first GEMM
        (700, 1024, 512, 2, 0, 2, 1),    # two experts with several row tiles each
    ],
)
def test_megamoe_forward_at_every_tile_height(ops, tokens, hidden, inter, experts, begin, local, topk, tile_rows):
    """Each tile height forced in turn (the launch would pick one): every height has its own ring depth, so each meets
    the short-k corner differently (with k = 512 a tile has four items, fewer than the copies of the 64- and 128-row
    kernels run ahead: the copy cursor then has to let everything land before it reads the next tile's gather
    indices, in the prologue and at every later switch)."""
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, begin, local, topk, seed=tile_rows)
    got, counts = _run(ops, x_codes, x_scales, l1, l2, idx, weights, experts, begin, local, tile_rows=tile_rows)
    want = _oracle(x_codes, x_scales, l1, l2, idx, weights, begin)
    np.testing.assert_array_equal(counts, np.bincount(idx.ravel(), minlength=experts)[begin : begin + local])
    assert np.isfinite(got).all()
    err = mm.relative_frobenius(got, want)
    assert err <= 2e-2, err


@pytest.mark.parametrize("tile_rows", [64, 128, 192])
@pytest.mark.parametrize(
    "tokens,hidden,inter,experts,begin,local,topk",
    [
        (300, 512, 512, 8, 2, 3, 4),     # four k tiles per tile
        (700, 1024, 512, 2, 0, 2, 1),    # several row tiles per expert
        (512, 1536, 1024, 16, 0, 16, 4), # several column tiles, three spans in the first GEMM
    ],
)
def test_both_grouped_gemm_kernels_agree_bit_for_bit(ops, tokens, hidden, inter, experts, begin, local, topk, tile_rows):
    """The kernel whose waves split the tile's columns (weights as the MFMA's first operand, results transposed, epilogue
    from registers) against the 2 x 2 kernel (weights through LDS, epilogue through an LDS staging area): different
    code, the same products summed over k in the same order, so the forward's output has to be the same bits."""
    problem = _make_problem(tokens, hidden, inter, experts, begin, local, topk, seed=100 + tile_rows)
    x_codes, x_scales, l1, l2, idx, weights = problem
    new, _ = _run(ops, x_codes, x_scales, l1, l2, idx, weights, experts, begin, local, tile_rows=tile_rows, column_waves=1)
    old, _ = _run(ops, x_codes, x_scales, l1, l2, idx, weights, experts, begin, local, tile_rows=tile_rows, column_waves=0)
    np.testing.assert_array_equal(new.view(np.uint32), old.view(np.uint32))


@pytest.mark.parametrize("tokens,hidden,inter,tile_rows", [
    (1000, 2304, 1280, 64),   # 320 + 288 tiles of 18 and 10 k tiles on 256 workgroups
    (1700, 1280, 768, 64),    # 10 and 6 k tiles: the shortest tile that still switches without letting the copies land
    (2000, 2304, 1280, 128),
    (3000, 2304, 1280, 192),
])
def test_several_tiles_per_workgroup_where_k_is_no_multiple_of_512(ops, tokens, hidden, inter, tile_rows):
    """K % 512 == 256 takes the 2 x 2 kernel, whose tiles then end with a span of two k tiles instead of four.  A
    workgroup that goes on to another tile copies up to five items ahead, i.e. into the span after the short one, while
    the scales of the span before it are still being read: with two scale slots that copy overwrote them (64-row tiles,
    more tiles than workgroups: wrong rows, differently on every run); the rings have three slots now."""
    experts = 2
    row_tiles = 2 * -(-tokens // tile_rows)  # every token goes to both experts
    assert row_tiles * (2 * inter // 256) > 256 and row_tiles * (hidden // 256) > 256  # more tiles than workgroups, both GEMMs
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, 0, experts, 2, seed=tile_rows)
    want = _oracle(x_codes, x_scales, l1, l2, idx, weights, 0)
    for attempt in range(2):
        got, counts = _run(ops, x_codes, x_scales, l1, l2, idx, weights, experts, 0, experts, tile_rows=tile_rows)
        assert counts.tolist() == [tokens, tokens]
        err = mm.relative_frobenius(got, want)
        assert err <= 2e-2, (attempt, err)
        norms = np.linalg.norm(want, axis=1)
        assert (np.linalg.norm(got - want, axis=1) / norms).max() <= 6e-2


@pytest.mark.parametrize("tokens,hidden,inter,experts,begin,local,topk,shared", [
    (100, 512, 512, 8, 0, 8, 2, 1),     # one shared expert beside 8 routed ones
    (257, 768, 512, 6, 2, 2, 3, 2),     # two shared experts, partial local range, more than one row tile each
])
def test_megamoe_forward_with_shared_experts(ops, tokens, hidden, inter, experts, begin, local, topk, shared):
    # shared experts take every token with weight 1 after the routed experts
    # (experiments/megamoe/python/deep_ep_experimental/megamoe/golden.py:160-173)
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, begin, local, topk, seed=3)
    rng = np.random.default_rng(99)
    sp1, ss1 = mm.quantize_weight_mxfp4((rng.normal(size=(shared, 2 * inter, hidden)) * 0.02).astype(np.float32))
    sp2, ss2 = mm.quantize_weight_mxfp4((rng.normal(size=(shared, hidden, inter)) * 0.02).astype(np.float32))
    dev = "cuda"
    w1, s1 = ops.megamoe_prepare_weights(torch.from_numpy(l1[0]).to(dev), torch.from_numpy(l1[1]).reshape(local, 2 * inter, -1).to(dev), True)
    w2, s2 = ops.megamoe_prepare_weights(torch.from_numpy(l2[0]).to(dev), torch.from_numpy(l2[1]).reshape(local, hidden, -1).to(dev), False)
    sw1, sws1 = ops.megamoe_prepare_weights(torch.from_numpy(sp1).to(dev), torch.from_numpy(ss1).reshape(shared, 2 * inter, -1).to(dev), True)
    sw2, sws2 = ops.megamoe_prepare_weights(torch.from_numpy(sp2).to(dev), torch.from_numpy(ss2).reshape(shared, hidden, -1).to(dev), False)
    ws = ops.Workspace(ops.megamoe_workspace_bytes(tokens, topk, hidden, inter, local, shared))
    y = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)
    counts = torch.empty((local,), dtype=torch.int32, device=dev)
    try:
        ops.megamoe_forward(
            ws, torch.from_numpy(x_codes).to(dev).view(torch.float8_e4m3fn), torch.from_numpy(x_scales).to(dev),
            torch.from_numpy(idx).to(dev), torch.from_numpy(weights).to(dev), w1, s1, w2, s2, experts, begin, local, y,
            counts, shared=(sw1, sws1, sw2, sws2),
        )
        torch.cuda.synchronize()
        got = y.float().cpu().numpy()
    finally:
        ws.destroy()
    xq = mm.mx_dequantize(x_codes, x_scales)
    want = mm.round_bf16(mm.local_reference(xq, idx, weights, mm.unpack_weight(*l1), mm.unpack_weight(*l2), begin,
                                            mm.unpack_weight(sp1, ss1), mm.unpack_weight(sp2, ss2)))
    np.testing.assert_array_equal(counts.cpu().numpy(), np.bincount(idx.ravel(), minlength=experts)[begin : begin + local])
    assert np.isfinite(got).all()
    err = mm.relative_frobenius(got, want)
    assert err <= 2e-2, err
    # the shared part alone must be there for tokens without any local route
    untouched = ~((idx >= begin) & (idx < begin + local)).any(axis=1)
    if untouched.any():
        only_shared = mm.round_bf16(mm.local_reference(xq[untouched], np.full((int(untouched.sum()), topk), -1), weights[untouched],
                                                       mm.unpack_weight(*l1), mm.unpack_weight(*l2), begin,
                                                       mm.unpack_weight(sp1, ss1), mm.unpack_weight(sp2, ss2)))
        assert mm.relative_frobenius(got[untouched], only_shared) <= 2e-2


def test_megamoe_forward_rank_share_shape(ops):
    # one EP rank's share at reduced token count: H=7168, I=2048, 6 local experts of 384, top-8
    tokens, hidden, inter, experts, local, topk = 2048, 7168, 2048, 384, 6, 8
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, 0, local, topk, seed=1)
    got, counts = _run(ops, x_codes, x_scales, l1, l2, idx, weights, experts, 0, local)
    want = _oracle(x_codes, x_scales, l1, l2, idx, weights, 0)
    np.testing.assert_array_equal(counts, np.bincount(idx.ravel(), minlength=experts)[:local])
    err = mm.relative_frobenius(got, want)
    assert err <= 2e-2, err


def test_public_api_workflow():
    # the reference's public workflow (experiments/megamoe/tests/test_public_api.py:193-260) on real kernels
    from deepep_amd import megamoe

    tokens, hidden, inter, experts, topk = 17, 1024, 512, 4, 2
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, 0, experts, topk, seed=5)
    buf = megamoe.SymmBuffer(None, experts, tokens, topk, hidden, inter)
    try:
        assert tuple(buf.x.shape) == (17, 1024) and tuple(buf.x_sf.shape) == (17, 32)
        raw1 = (torch.from_numpy(l1[0]).cuda(), torch.from_numpy(l1[1]).cuda().view(torch.float8_e8m0fnu))
        raw2 = (torch.from_numpy(l2[0]).cuda().view(torch.int8), torch.from_numpy(l2[1]).cuda())
        p1, p2 = megamoe.transform_weights_for_mega_moe(raw1, raw2)
        buf.x.view(torch.uint8).copy_(torch.from_numpy(x_codes))
        buf.x_sf.view(torch.uint8).copy_(torch.from_numpy(x_scales))
        buf.topk_idx.copy_(torch.from_numpy(idx))
        buf.topk_weights.copy_(torch.from_numpy(weights))
        buf.validate_inputs(tokens)
        buf.prepare(tokens)
        first_ws = buf._workspace
        buf.prepare(tokens)
        assert buf._workspace is first_ws and buf.workspace_bytes > 0
        y = torch.empty((tokens, hidden), dtype=torch.bfloat16, device="cuda")
        stats = torch.tensor([7, 11, 0, 1], dtype=torch.int32, device="cuda")
        per_call = np.bincount(idx.ravel(), minlength=experts)
        assert megamoe.fp8_fp4_mega_moe(y, p1, p2, buf, cumulative_local_expert_recv_stats=stats) is None
        assert stats.cpu().tolist() == (np.array([7, 11, 0, 1]) + per_call).tolist()
        megamoe.fp8_fp4_mega_moe(y, p1, p2, buf, cumulative_local_expert_recv_stats=stats)
        assert stats.cpu().tolist() == (np.array([7, 11, 0, 1]) + 2 * per_call).tolist()
        want = _oracle(x_codes, x_scales, l1, l2, idx, weights, 0)
        assert mm.relative_frobenius(y.float().cpu().numpy(), want) <= 2e-2
        # explicit-input API returns (y, counts); BF16 override is quantised internally
        xb = torch.from_numpy(mm.mx_dequantize(x_codes, x_scales)).bfloat16().cuda()
        y2, counts = megamoe.mega_moe(xb, buf.topk_idx[:tokens], buf.topk_weights[:tokens], p1, p2, buf)
        assert counts.cpu().tolist() == per_call.tolist()
        want2 = _oracle(*mm.mx_quantize(xb.float().cpu().numpy()), l1, l2, idx, weights, 0)
        assert mm.relative_frobenius(y2.float().cpu().numpy(), want2) <= 2e-2
        # error contract
        with pytest.raises(ValueError, match="alias"):
            megamoe.mega_moe(xb, buf.topk_idx[:tokens], buf.topk_weights[:tokens], p1, p2, buf, out=xb)
        with pytest.raises(ValueError, match="prepared"):
            megamoe.mega_moe(xb, buf.topk_idx[:tokens], buf.topk_weights[:tokens], raw1, raw2, buf)
        with pytest.raises(RuntimeError, match="DEEPEP_MEGAMOE_TIMER"):
            buf.allocate_timer()
        for bad in (-1, 4, int(idx[0, 1])):
            saved = buf.topk_idx[0, 0].item()
            buf.topk_idx[0, 0] = bad
            with pytest.raises(ValueError, match=r"rank=0.*token=0"):
                buf.validate_inputs(tokens)
            buf.topk_idx[0, 0] = saved
    finally:
        buf.destroy()
    with pytest.raises(RuntimeError, match="destroyed"):
        megamoe.fp8_fp4_mega_moe(y, p1, p2, buf)


def test_public_api_padded_sizes_and_packed_int32_scales():
    """hidden % 64 and intermediate_hidden % 128 as the reference allows them (api.py:93-105), through the public
    classes; the raw E8M0 scales given once as bytes [E,N,K/64,2] and once packed four to an int32 [E,N,K/128]
    (api.py:340-352 accepts both): same prepared bytes, same output."""
    from deepep_amd import megamoe

    tokens, hidden, inter, experts, topk = 50, 1152, 384, 4, 2
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, 0, experts, topk, seed=9)
    buf = megamoe.SymmBuffer(None, experts, tokens, topk, hidden, inter)
    try:
        as_bytes = [(torch.from_numpy(w).cuda(), torch.from_numpy(sc).cuda()) for w, sc in (l1, l2)]
        as_int32 = [(w, sc.reshape(*w.shape[:2], -1).contiguous().view(torch.int32)) for w, sc in as_bytes]
        assert tuple(as_int32[0][1].shape) == (experts, 2 * inter, hidden // 128)
        p1, p2 = megamoe.transform_weights_for_mega_moe(*as_bytes)
        q1, q2 = megamoe.transform_weights_for_mega_moe(*as_int32)
        for a, b in ((p1, q1), (p2, q2)):
            assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        assert tuple(p1[0].shape) == (experts, 1024, 1280 // 2) and tuple(p2[0].shape) == (experts, 1280, 512 // 2)
        buf.x.view(torch.uint8).copy_(torch.from_numpy(x_codes))
        buf.x_sf.view(torch.uint8).copy_(torch.from_numpy(x_scales))
        buf.topk_idx.copy_(torch.from_numpy(idx))
        buf.topk_weights.copy_(torch.from_numpy(weights))
        buf.validate_inputs(tokens)
        y = torch.full((tokens, hidden), float("nan"), dtype=torch.bfloat16, device="cuda")
        megamoe.fp8_fp4_mega_moe(y, q1, q2, buf)
        want = _oracle(x_codes, x_scales, l1, l2, idx, weights, 0)
        got = y.float().cpu().numpy()
        assert np.isfinite(got).all()
        assert mm.relative_frobenius(got, want) <= 2e-2
        # prepared from a narrower raw tensor (I = 256): padded to the same prepared shape, but not this buffer's weights
        narrow, _ = megamoe.transform_weights_for_mega_moe(
            (as_bytes[0][0][:, :512].contiguous(), as_bytes[0][1][:, :512].contiguous()), as_bytes[1])
        assert narrow[0].shape == q1[0].shape
        with pytest.raises(ValueError, match="do not match the buffer"):
            megamoe.fp8_fp4_mega_moe(y, narrow, q2, buf)
    finally:
        buf.destroy()


def test_megamoe_forward_in_hip_graph(ops):
    # The forward is five launches and no host synchronisation, so it can be captured once and replayed
    # with new inputs in the same buffers; every replay is checked against the eager result.
    tokens, hidden, inter, experts, local, topk = 192, 512, 512, 8, 8, 2
    dev = "cuda"
    problems = [_make_problem(tokens, hidden, inter, experts, 0, local, topk, seed=s) for s in (11, 12, 13)]
    _, _, l1, l2, _, _ = problems[0]
    w1, s1 = ops.megamoe_prepare_weights(torch.from_numpy(l1[0]).to(dev), torch.from_numpy(l1[1]).reshape(local, 2 * inter, -1).to(dev), True)
    w2, s2 = ops.megamoe_prepare_weights(torch.from_numpy(l2[0]).to(dev), torch.from_numpy(l2[1]).reshape(local, hidden, -1).to(dev), False)
    ws = ops.Workspace(ops.megamoe_workspace_bytes(tokens, topk, hidden, inter, local))
    x_codes = torch.empty((tokens, hidden), dtype=torch.uint8, device=dev)
    x_scales = torch.empty((tokens, hidden // 32), dtype=torch.uint8, device=dev)
    idx = torch.empty((tokens, topk), dtype=torch.int32, device=dev)
    weights = torch.empty((tokens, topk), dtype=torch.float32, device=dev)
    y = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)
    counts = torch.empty((local,), dtype=torch.int32, device=dev)

    def load(problem):
        codes, scales, _, _, ids, wts = problem
        x_codes.copy_(torch.from_numpy(codes)); x_scales.copy_(torch.from_numpy(scales))
        idx.copy_(torch.from_numpy(ids)); weights.copy_(torch.from_numpy(wts))

    def forward():
        ops.megamoe_forward(ws, x_codes.view(torch.float8_e4m3fn), x_scales, idx, weights, w1, s1, w2, s2, experts, 0, local, y, counts)

    try:
        eager = []
        for problem in problems:
            load(problem)
            forward()
            torch.cuda.synchronize()
            eager.append((y.clone(), counts.clone()))
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            forward()  # warm-up on the capture stream
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            forward()
        for turn in range(2):
            for problem, (want_y, want_counts) in zip(problems, eager):
                load(problem)
                y.zero_()
                torch.cuda.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(counts, want_counts)
                assert torch.equal(y.view(torch.int16), want_y.view(torch.int16)), f"replay {turn} differs from eager"
    finally:
        torch.cuda.synchronize()
        ws.destroy()


def test_megamoe_forward_in_hip_graph_keeps_its_fillers(ops):
    """A rank's share (most tokens unserved, fewer tiles than workgroups) captured once and replayed: on every replay the
    idle workgroups of the first GEMM must again zero rows of unserved tokens (their stop signal is a device-side
    counter, not a value fixed at capture), and every replay must equal the eager forward bit for bit."""
    tokens, hidden, inter, experts, begin, local, topk = 1536, 512, 512, 64, 8, 2, 4
    dev = "cuda"
    problems = [_make_problem(tokens, hidden, inter, experts, begin, local, topk, seed=s) for s in (21, 22, 23)]
    _, _, l1, l2, _, _ = problems[0]
    w1, s1 = ops.megamoe_prepare_weights(torch.from_numpy(l1[0]).to(dev), torch.from_numpy(l1[1]).reshape(local, 2 * inter, -1).to(dev), True)
    w2, s2 = ops.megamoe_prepare_weights(torch.from_numpy(l2[0]).to(dev), torch.from_numpy(l2[1]).reshape(local, hidden, -1).to(dev), False)
    ws = ops.Workspace(ops.megamoe_workspace_bytes(tokens, topk, hidden, inter, local))
    x_codes = torch.empty((tokens, hidden), dtype=torch.uint8, device=dev)
    x_scales = torch.empty((tokens, hidden // 32), dtype=torch.uint8, device=dev)
    idx = torch.empty((tokens, topk), dtype=torch.int32, device=dev)
    weights = torch.empty((tokens, topk), dtype=torch.float32, device=dev)
    y = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)
    counts = torch.empty((local,), dtype=torch.int32, device=dev)

    def load(problem):
        codes, scales, _, _, ids, wts = problem
        x_codes.copy_(torch.from_numpy(codes)); x_scales.copy_(torch.from_numpy(scales))
        idx.copy_(torch.from_numpy(ids)); weights.copy_(torch.from_numpy(wts))

    def forward():
        ops.megamoe_forward(ws, x_codes.view(torch.float8_e4m3fn), x_scales, idx, weights, w1, s1, w2, s2, experts, begin, local, y, counts)

    def report():
        return ops.megamoe_fill_report(ws, tokens, topk, hidden, inter, local)

    try:
        eager = []
        for problem in problems:
            load(problem)
            y.fill_(float("nan"))
            forward()
            torch.cuda.synchronize()
            fillers, filled = report()
            assert fillers > 0 and filled > 0, (fillers, filled)
            eager.append((y.clone(), counts.clone()))
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            forward()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            forward()
        for turn in range(2):
            for problem, (want_y, want_counts) in zip(problems, eager):
                load(problem)
                y.fill_(float("nan"))
                torch.cuda.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                fillers, filled = report()
                assert fillers > 0 and filled > 0, f"replay {turn}: {fillers} fillers looked at {filled} tokens"
                assert torch.equal(counts, want_counts)
                assert torch.equal(y.view(torch.int16), want_y.view(torch.int16)), f"replay {turn} differs from eager"
    finally:
        torch.cuda.synchronize()
        ws.destroy()


def test_public_api_shared_experts():
    # SymmBuffer(num_shared_experts=S) + transform_weights_for_mega_moe(..., shared=True) + shared_l*_weights
    from deepep_amd import megamoe

    tokens, hidden, inter, experts, topk, shared = 33, 1024, 512, 4, 2, 1
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, 0, experts, topk, seed=8)
    rng = np.random.default_rng(5)
    sp1, ss1 = mm.quantize_weight_mxfp4((rng.normal(size=(shared, 2 * inter, hidden)) * 0.02).astype(np.float32))
    sp2, ss2 = mm.quantize_weight_mxfp4((rng.normal(size=(shared, hidden, inter)) * 0.02).astype(np.float32))
    buf = megamoe.SymmBuffer(None, experts, tokens, topk, hidden, inter, num_shared_experts=shared)
    try:
        p1, p2 = megamoe.transform_weights_for_mega_moe(
            (torch.from_numpy(l1[0]).cuda(), torch.from_numpy(l1[1]).cuda()), (torch.from_numpy(l2[0]).cuda(), torch.from_numpy(l2[1]).cuda()))
        q1, q2 = megamoe.transform_weights_for_mega_moe(
            (torch.from_numpy(sp1).cuda(), torch.from_numpy(ss1).cuda()), (torch.from_numpy(sp2).cuda(), torch.from_numpy(ss2).cuda()),
            shared=True)
        x = (torch.from_numpy(x_codes).cuda().view(torch.float8_e4m3fn), torch.from_numpy(x_scales).cuda())
        ids, wts = torch.from_numpy(idx).cuda(), torch.from_numpy(weights).cuda()
        with pytest.raises(ValueError, match="Shared expert count"):
            megamoe.mega_moe(x, ids, wts, p1, p2, buf)
        with pytest.raises(ValueError, match="both shared"):
            megamoe.mega_moe(x, ids, wts, p1, p2, buf, shared_l1_weights=q1)
        y, counts = megamoe.mega_moe(x, ids, wts, p1, p2, buf, shared_l1_weights=q1, shared_l2_weights=q2)
        assert counts.cpu().tolist() == np.bincount(idx.ravel(), minlength=experts).tolist()
        xq = mm.mx_dequantize(x_codes, x_scales)
        want = mm.round_bf16(mm.local_reference(xq, idx, weights, mm.unpack_weight(*l1), mm.unpack_weight(*l2), 0,
                                                mm.unpack_weight(sp1, ss1), mm.unpack_weight(sp2, ss2)))
        assert mm.relative_frobenius(y.float().cpu().numpy(), want) <= 2e-2
    finally:
        buf.destroy()


def test_rows_of_unserved_tokens_are_zeroed_whoever_writes_them(ops):
    """In a rank's share most tokens reach no local expert; their rows of y must come out as zeros.  Workgroups of the
    first GEMM that get no tile write those zeros while the others compute, and the weighted reduce writes what they
    did not get to: the result may not depend on who wrote a row, on what y held before, or on what the previous call
    on the workspace left behind (a call whose first GEMM fills, then one with more tiles than workgroups, which does
    not, then the first again)."""
    dev = "cuda"
    shapes = [  # tokens, hidden, inter, experts, begin, local, topk
        (1536, 512, 512, 64, 8, 2, 4),      # 2 experts x few tiles: nearly every workgroup fills
        (6144, 512, 2048, 16, 0, 16, 8),    # every expert local: about 1500 tiles, nobody fills, no token unserved
        (1536, 512, 512, 64, 8, 2, 4),
    ]
    workspace = ops.Workspace(max(ops.megamoe_workspace_bytes(t, k, h, i, l) for t, h, i, _, _, l, k in shapes))
    try:
        for call, (tokens, hidden, inter, experts, begin, local, topk) in enumerate(shapes):
            x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, begin, local, topk, seed=call % 2)
            w1, s1 = ops.megamoe_prepare_weights(torch.from_numpy(l1[0]).to(dev), torch.from_numpy(l1[1]).reshape(local, 2 * inter, -1).to(dev), True)
            w2, s2 = ops.megamoe_prepare_weights(torch.from_numpy(l2[0]).to(dev), torch.from_numpy(l2[1]).reshape(local, hidden, -1).to(dev), False)
            y = torch.full((tokens, hidden), float("nan"), dtype=torch.bfloat16, device=dev)
            counts = torch.empty((local,), dtype=torch.int32, device=dev)
            ops.megamoe_forward(
                workspace, torch.from_numpy(x_codes).to(dev).view(torch.float8_e4m3fn), torch.from_numpy(x_scales).to(dev),
                torch.from_numpy(idx).to(dev), torch.from_numpy(weights).to(dev), w1, s1, w2, s2, experts, begin, local, y, counts,
            )
            torch.cuda.synchronize()
            got = y.float().cpu().numpy()
            served = ((idx >= begin) & (idx < begin + local)).any(axis=1)
            assert served.sum() < tokens or local == experts
            assert not np.isnan(got).any()
            assert not got[~served].any()  # exact zeros, every element
            want = _oracle(x_codes, x_scales, l1, l2, idx, weights, begin)
            err = np.linalg.norm(got - want) / np.linalg.norm(want)
            assert err < 2e-2, err
    finally:
        workspace.destroy()


def test_full_size_share_against_its_served_tokens_alone(ops):
    """The benchmark share at full size (16384 candidate tokens, 6 of 384 experts, top-8, H=7168, I=2048), too big
    for the CPU oracle: every token's output depends on that token alone, so the forward over all tokens must
    reproduce, bit for bit, a forward over the served tokens only (which runs with other tile heights, no zero
    rows and the dense reduce), rows of unserved tokens must be exact zeros, and the counts must be a bincount."""
    dev = "cuda"
    tokens, hidden, inter, experts, local, topk = 16384, 7168, 2048, 384, 6, 8
    gen = torch.Generator(device="cpu").manual_seed(5)
    idx = torch.stack([torch.randperm(experts, generator=gen)[:topk] for _ in range(tokens)]).to(torch.int32)
    weights = torch.rand(tokens, topk, generator=gen)
    x = (torch.randn(tokens, hidden, generator=gen) * 0.5).bfloat16().to(dev)
    x_codes, x_scales = ops.mx_quant(x)
    raw1 = torch.randint(0, 256, (local, 2 * inter, hidden // 2), dtype=torch.uint8, generator=gen).to(dev)
    raw2 = torch.randint(0, 256, (local, hidden, inter // 2), dtype=torch.uint8, generator=gen).to(dev)
    sc1 = torch.randint(116, 120, (local, 2 * inter, hidden // 32), dtype=torch.uint8, generator=gen).to(dev)
    sc2 = torch.randint(116, 120, (local, hidden, inter // 32), dtype=torch.uint8, generator=gen).to(dev)
    w1, s1 = ops.megamoe_prepare_weights(raw1, sc1, True)
    w2, s2 = ops.megamoe_prepare_weights(raw2, sc2, False)

    def forward(keep):
        n = int(keep.sum())
        workspace = ops.Workspace(ops.megamoe_workspace_bytes(n, topk, hidden, inter, local))
        y = torch.full((n, hidden), float("nan"), dtype=torch.bfloat16, device=dev)
        counts = torch.empty((local,), dtype=torch.int32, device=dev)
        keep_dev = keep.to(dev)
        ops.megamoe_forward(workspace, x_codes[keep_dev].contiguous(), x_scales[keep_dev].contiguous(), idx[keep].contiguous().to(dev),
                            weights[keep].contiguous().to(dev), w1, s1, w2, s2, experts, 0, local, y, counts)
        torch.cuda.synchronize()
        workspace.destroy()
        return y, counts.cpu()

    served = (idx < local).any(dim=1)
    everyone = torch.ones(tokens, dtype=torch.bool)
    y_all, counts_all = forward(everyone)
    y_served, counts_served = forward(served)
    assert 1500 < int(served.sum()) < 2500
    assert counts_all.tolist() == counts_served.tolist() == torch.bincount(idx.flatten().long(), minlength=experts)[:local].tolist()
    assert not torch.isnan(y_all.float()).any() and not y_all[~served.to(dev)].any()
    assert torch.equal(y_all[served.to(dev)].view(torch.int16), y_served.view(torch.int16))
    assert y_served.float().abs().max() > 0


def test_megamoe_forward_without_any_local_route(ops):
    """Every token routed to experts of other ranks, and the opposite corner, one local expert taking nothing while
    its neighbour takes everything: zero output and zero counts in the first case (the GEMM launches have no tile
    at all), parity with the oracle in the second."""
    dev = "cuda"
    tokens, hidden, inter, experts, begin, local, topk = 200, 512, 512, 16, 4, 2, 2
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, begin, local, topk, seed=3)
    elsewhere = idx.copy()
    elsewhere[(elsewhere >= begin) & (elsewhere < begin + local)] = 0  # expert 0 belongs to another rank
    got, counts = _run(ops, x_codes, x_scales, l1, l2, elsewhere, weights, experts, begin, local)
    assert not got.any() and counts.tolist() == [0, 0]
    one_sided = idx.copy()
    one_sided[one_sided == begin] = begin + 1  # may repeat an expert within a token: give those slots to expert 0
    for t in range(tokens):
        if (one_sided[t] == begin + 1).sum() > 1:
            one_sided[t, 1] = 0
    got, counts = _run(ops, x_codes, x_scales, l1, l2, one_sided, weights, experts, begin, local)
    assert counts[0] == 0 and counts[1] == (one_sided == begin + 1).sum() > 0
    want = _oracle(x_codes, x_scales, l1, l2, one_sided, weights, begin)
    assert mm.relative_frobenius(got, want) <= 2e-2


def test_forward_is_reproducible_whoever_zeroes_which_row(ops):
    """How far the first GEMM's idle workgroups get with the zero rows before they are told to stop changes from run
    to run; the output may not: fifty forwards over the same share, y poisoned before each, all bit-identical."""
    dev = "cuda"
    tokens, hidden, inter, experts, local, topk = 8192, 2048, 1024, 256, 4, 8
    gen = torch.Generator(device="cpu").manual_seed(11)
    idx = torch.stack([torch.randperm(experts, generator=gen)[:topk] for _ in range(tokens)]).to(torch.int32).to(dev)
    weights = torch.rand(tokens, topk, generator=gen).to(dev)
    x_codes, x_scales = ops.mx_quant((torch.randn(tokens, hidden, generator=gen) * 0.5).bfloat16().to(dev))
    w1, s1 = ops.megamoe_prepare_weights(torch.randint(0, 256, (local, 2 * inter, hidden // 2), dtype=torch.uint8, generator=gen).to(dev),
                                         torch.full((local, 2 * inter, hidden // 32), 118, dtype=torch.uint8, device=dev), True)
    w2, s2 = ops.megamoe_prepare_weights(torch.randint(0, 256, (local, hidden, inter // 2), dtype=torch.uint8, generator=gen).to(dev),
                                         torch.full((local, hidden, inter // 32), 118, dtype=torch.uint8, device=dev), False)
    workspace = ops.Workspace(ops.megamoe_workspace_bytes(tokens, topk, hidden, inter, local))
    y = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)
    counts = torch.empty((local,), dtype=torch.int32, device=dev)
    served = (idx < local).any(dim=1)
    first = None
    try:
        for _ in range(50):
            y.fill_(float("nan"))
            ops.megamoe_forward(workspace, x_codes, x_scales, idx, weights, w1, s1, w2, s2, experts, 0, local, y, counts)
            torch.cuda.synchronize()
            if first is None:
                first = y.clone()
                assert not torch.isnan(first.float()).any() and not first[~served].any() and first[served].any()
            else:
                assert torch.equal(y.view(torch.int16), first.view(torch.int16))
    finally:
        workspace.destroy()


def test_forward_served_only_leaves_unserved_rows_untouched(ops):
    """One rank's share with `megamoe_served_only`: rows of y whose token no local expert serves keep what they held
    (other ranks produce them in an EP job), served rows are bit for bit those of the zero-filling forward."""
    tokens, hidden, inter, experts, begin, local, topk = 900, 512, 512, 64, 8, 4, 2
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, begin, local, topk, seed=4)
    dev = "cuda"
    w1, s1 = ops.megamoe_prepare_weights(torch.from_numpy(l1[0]).to(dev), torch.from_numpy(l1[1]).reshape(local, 2 * inter, -1).to(dev), True)
    w2, s2 = ops.megamoe_prepare_weights(torch.from_numpy(l2[0]).to(dev), torch.from_numpy(l2[1]).reshape(local, hidden, -1).to(dev), False)
    ws = ops.Workspace(ops.megamoe_workspace_bytes(tokens, topk, hidden, inter, local))
    counts = torch.empty((local,), dtype=torch.int32, device=dev)
    args = (torch.from_numpy(x_codes).to(dev).view(torch.float8_e4m3fn), torch.from_numpy(x_scales).to(dev),
            torch.from_numpy(idx).to(dev), torch.from_numpy(weights).to(dev), w1, s1, w2, s2, experts, begin, local)
    try:
        full = torch.full((tokens, hidden), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.megamoe_forward(ws, *args, full, counts)
        ws.tune("megamoe_served_only", 1)
        part = torch.full((tokens, hidden), 5.0, dtype=torch.bfloat16, device=dev)
        ops.megamoe_forward(ws, *args, part, counts)
        torch.cuda.synchronize()
        served = torch.from_numpy(((idx >= begin) & (idx < begin + local)).any(axis=1)).to(dev)
        assert 0 < int(served.sum()) < tokens
        assert torch.equal(part[served].view(torch.int16), full[served].view(torch.int16))
        assert (part[~served] == 5.0).all() and not full[~served].any()
    finally:
        ws.destroy()


def test_readme_example_runs_as_written(monkeypatch):
    """The reference README's MegaMoE example (README.md:237-281) with its own imports and call sequence, one shared expert
    included; only the device name and the sizes differ."""
    import deepep_amd

    deepep_amd.install_as_deep_ep()
    from deep_ep_experimental.megamoe import StoreGroup, SymmBuffer, fp8_fp4_mega_moe, transform_weights_for_mega_moe

    monkeypatch.setenv("RANK", "0")
    monkeypatch.setenv("WORLD_SIZE", "1")
    monkeypatch.setenv("LOCAL_WORLD_SIZE", "1")
    tokens, hidden, inter, experts, topk = 40, 1024, 512, 8, 2
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, 0, experts, topk, seed=31)
    rng = np.random.default_rng(32)
    sp1, ss1 = mm.quantize_weight_mxfp4((rng.normal(size=(1, 2 * inter, hidden)) * 0.02).astype(np.float32))
    sp2, ss2 = mm.quantize_weight_mxfp4((rng.normal(size=(1, hidden, inter)) * 0.02).astype(np.float32))
    as_pair = lambda w, sc: (torch.from_numpy(w).cuda(), torch.from_numpy(sc).cuda())  # noqa: E731
    l1_weights, l2_weights, shared_l1_weights, shared_l2_weights = as_pair(*l1), as_pair(*l2), as_pair(sp1, ss1), as_pair(sp2, ss2)
    x_fp8 = torch.from_numpy(x_codes).cuda().view(torch.float8_e4m3fn)
    x_sf = torch.from_numpy(x_scales).cuda().view(torch.float8_e8m0fnu)
    topk_idx, topk_weights = torch.from_numpy(idx).cuda(), torch.from_numpy(weights).cuda()

    group = StoreGroup.from_env()
    try:
        buffer = SymmBuffer(
            group, num_experts=experts, num_max_tokens_per_rank=64,
            num_topk=topk, hidden=hidden, intermediate_hidden=inter,
            num_shared_experts=1, mma_type="fp8xfp4",
            ranks_per_node=int(__import__("os").environ["LOCAL_WORLD_SIZE"]),
        )
        w1, w2 = transform_weights_for_mega_moe(l1_weights, l2_weights)
        shared_w1, shared_w2 = transform_weights_for_mega_moe(shared_l1_weights, shared_l2_weights, shared=True)
        num_tokens = x_fp8.shape[0]
        buffer.x[:num_tokens].copy_(x_fp8)
        buffer.x_sf[:num_tokens].copy_(x_sf)
        buffer.topk_idx[:num_tokens].copy_(topk_idx)
        buffer.topk_weights[:num_tokens].copy_(topk_weights)
        buffer.validate_inputs(num_tokens)
        buffer.prepare(num_tokens)
        y = torch.empty((num_tokens, hidden), dtype=torch.bfloat16, device="cuda")
        assert fp8_fp4_mega_moe(y, w1, w2, buffer, shared_l1_weights=shared_w1, shared_l2_weights=shared_w2) is None
        torch.cuda.synchronize()
        group.barrier("before SHMEM teardown")
        buffer.destroy()
        group.close()
    except BaseException as error:
        group.abort(f"MegaMoE: {type(error).__name__}: {error}")
        raise
    xq = mm.mx_dequantize(x_codes, x_scales)
    want = mm.round_bf16(mm.local_reference(xq, idx, weights, mm.unpack_weight(*l1), mm.unpack_weight(*l2), 0,
                                            mm.unpack_weight(sp1, ss1), mm.unpack_weight(sp2, ss2)))
    assert mm.relative_frobenius(y.float().cpu().numpy(), want) <= 2e-2
