"""The dispatch entry points at seeded random shapes against the CPU oracle, bit for bit, at the level of the C-ABI
wrappers: expand-permute of BF16 / FP16 / FP8 rows with FP32 or packed-int32 scales and weights, with the row count known
(row-major grid for sparse shares, token-major otherwise) or not yet known to the host; the fused quantising dispatch in
both grids; the stand-alone quantiser and dequantiser at widths with a short last block."""

import warnings

import numpy as np
import pytest
import torch

from oracle import layout as olayout
from oracle import quant as oquant
from tests.gpu_util import bf16_bits, f32_bits, fp8_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ws():
    from deepep_amd import ops

    workspace = ops.Workspace(64 << 20)
    yield workspace
    workspace.destroy()


def _draw(seed):
    rng = np.random.default_rng(13000 + seed)
    experts = int(rng.choice([1, 4, 64, 256, 384]))
    local = int(min(experts, rng.choice([1, 2, 6, 64, 256])))
    begin = int(rng.integers(0, experts - local + 1))
    topk = int(min(experts, rng.choice([1, 2, 8, 9])))
    tokens = int(rng.choice([1, 5, 64, 257, 4096, 16384]))
    payload = str(rng.choice(["bf16", "fp16", "fp8_f32", "fp8_i32", "quant"]))
    hidden = int(rng.choice([128, 384, 1024, 7168])) if payload != "bf16" and payload != "fp16" else int(rng.choice([8, 72, 1024, 7168]))
    while tokens * topk * hidden > 48_000_000:
        tokens //= 2
    with_weights = bool(rng.integers(0, 2))
    rows_known = bool(rng.integers(0, 2))
    return experts, begin, local, topk, tokens, payload, hidden, with_weights, rows_known


@pytest.mark.parametrize("seed", range(96))
def test_dispatch_forms_at_random_shapes(ws, seed):
    from deepep_amd import ops

    experts, begin, local, topk, tokens, payload, hidden, with_weights, rows_known = _draw(seed)
    case = dict(experts=experts, begin=begin, local=local, topk=topk, tokens=tokens, payload=payload, hidden=hidden,
                with_weights=with_weights, rows_known=rows_known)
    print(case, flush=True)
    rng = np.random.default_rng(seed)
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int64)
    ids[rng.random(ids.shape) < 0.1] = -1
    want = olayout.layout(ids, experts, begin, local)
    rows = want["num_rows"]
    lay = ops.layout(ws, torch.from_numpy(ids).cuda(), experts, begin, local)
    _, host_rows = ops.layout_wait(ws, local)
    assert host_rows == rows, case
    weights = torch.from_numpy(rng.random((tokens, topk)).astype(np.float32)) if with_weights else None
    x = torch.from_numpy(rng.normal(size=(tokens, hidden)).astype(np.float32) * 3).bfloat16()
    known = rows if rows_known else None
    w_dev = None if weights is None else weights.cuda()
    if payload == "quant":
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", RuntimeWarning)
            codes, scales = oquant.cast_to_fp8_int(bf16_bits(x))
        out, out_scales, out_w = ops.dispatch_quant_fp8(x.cuda(), w_dev, lay["route_to_row"], lay["row_to_route"], known)
        np.testing.assert_array_equal(fp8_bits(out[:rows]), olayout.expand_rows(codes, want["row_to_route"], topk), err_msg=str(case))
        np.testing.assert_array_equal(f32_bits(out_scales[:rows]), olayout.expand_rows(scales, want["row_to_route"], topk).view(np.uint32),
                                      err_msg=str(case))
    else:
        scales = None
        if payload == "bf16":
            source = x
        elif payload == "fp16":
            source = x.to(torch.float16)
        else:
            source = x.to(torch.float8_e4m3fn)
            words = rng.integers(0x30000000, 0x48000000, size=(tokens, hidden // 128), dtype=np.int64).astype(np.int32)
            scales = torch.from_numpy(words) if payload == "fp8_i32" else torch.from_numpy(words).view(torch.float32)
        out, out_scales, out_w = ops.dispatch_copy(source.cuda(), None if scales is None else scales.cuda(), w_dev, lay["route_to_row"],
                                                   lay["row_to_route"], known)
        raw = source.view(torch.uint8).numpy() if source.element_size() == 1 else source.view(torch.int16).numpy()
        got = out[:rows].view(torch.uint8 if source.element_size() == 1 else torch.int16).cpu().numpy()
        np.testing.assert_array_equal(got, olayout.expand_rows(raw, want["row_to_route"], topk), err_msg=str(case))
        if scales is not None:
            assert out_scales.dtype == scales.dtype
            np.testing.assert_array_equal(out_scales[:rows].view(torch.int32).cpu().numpy(),
                                          olayout.expand_rows(words, want["row_to_route"], topk), err_msg=str(case))
    if with_weights:
        np.testing.assert_array_equal(f32_bits(out_w[:rows]), olayout.expand_weights(weights.numpy(), want["row_to_route"]).view(np.uint32),
                                      err_msg=str(case))


@pytest.mark.parametrize("seed", range(32))
def test_quantiser_and_dequantiser_at_random_widths(seed):
    from deepep_amd import ops

    rng = np.random.default_rng(15000 + seed)
    tokens = int(rng.choice([1, 3, 64, 1000, 5000]))
    hidden = int(rng.choice([16, 48, 128, 144, 1008, 1024, 7168, 7184]))
    scale = float(rng.choice([1e-6, 1e-3, 1.0, 300.0, 1e5]))
    x = torch.from_numpy((rng.normal(size=(tokens, hidden)) * scale).astype(np.float32)).bfloat16()
    x[rng.random((tokens, hidden)) < 0.05] = 0
    padded = -(-hidden // 128) * 128
    bits = np.zeros((tokens, padded), dtype=np.uint16)
    bits[:, :hidden] = bf16_bits(x)
    want_codes, want_scales = oquant.cast_to_fp8_int(bits)
    codes, scales = ops.cast_to_fp8(x.cuda())
    np.testing.assert_array_equal(fp8_bits(codes), want_codes[:, :hidden])
    np.testing.assert_array_equal(f32_bits(scales), want_scales.view(np.uint32))
    back = ops.cast_back(codes, scales)
    full = np.zeros((tokens, padded), dtype=np.uint8)
    full[:, :hidden] = fp8_bits(codes)
    np.testing.assert_array_equal(bf16_bits(back), oquant.cast_back(full, want_scales)[:, :hidden])
