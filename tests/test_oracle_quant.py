"""Pins the per-128 FP8 quantizer oracle: torch-library form == integer form, plus reference anchors."""

import numpy as np
import pytest
import torch

from oracle import quant


def _bits(t):
    return t.view(torch.int16).numpy().view(np.uint16)


def test_all_finite_codes_roundtrip_and_midpoints():
    codes = np.concatenate((np.arange(127), np.arange(128, 255))).astype(np.uint8)
    np.testing.assert_array_equal(quant.e4m3fn_encode_rne(quant.e4m3fn_decode(codes)), codes)
    # torch's own decode agrees with ours on every finite code
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    np.testing.assert_array_equal(quant.e4m3fn_decode(codes), ref)
    pos = quant.e4m3fn_decode(np.arange(127, dtype=np.uint8)).astype(np.float64)
    mid = ((pos[:-1] + pos[1:]) / 2).astype(np.float32)
    expected = np.arange(126)
    expected += expected % 2
    np.testing.assert_array_equal(quant.e4m3fn_encode_rne(mid), expected)


def test_reference_rounding_anchors():
    # tests/test_precision.py:76-82
    one = np.asarray([1.00390625, 1.0078125], dtype=np.float32)
    np.testing.assert_array_equal(quant.bf16_bits_to_f32(quant.f32_to_bf16_bits(one)), [1.0, 1.0078125])
    sat = quant.e4m3fn_decode(quant.e4m3fn_encode_rne(np.asarray([500.0, -500.0, 2.0**-9], np.float32), saturate=True))
    np.testing.assert_array_equal(sat, [448.0, -448.0, 2.0**-9])
    # torch cast semantics (no saturation): 500 -> NaN code, 464 (tie) -> 448
    raw = quant.e4m3fn_encode_rne(np.asarray([500.0, 464.0, 463.9, 464.1], np.float32))
    ref = torch.tensor([500.0, 464.0, 463.9, 464.1]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    np.testing.assert_array_equal(raw, ref)


def test_per128_anchor_block_restores_exactly():
    # tests/test_precision.py:84-89: second block (224, 448, 0...) restores exactly.
    row = np.zeros((1, 256), dtype=np.float32)
    row[0, :128] = 1.0
    row[0, 128], row[0, 129] = 224.0, 448.0
    bits = quant.f32_to_bf16_bits(row)
    codes, scales = quant.cast_to_fp8_int(bits)
    back = quant.bf16_bits_to_f32(quant.cast_back(codes, scales))
    assert back[0, 128] == 224.0 and back[0, 129] == 448.0
    assert abs(back[0, 0] - 1.0) <= 0.02
    assert scales[0, 1] == np.float32(1.0)


def test_amax_floor():
    bits = quant.f32_to_bf16_bits(np.full((1, 128), 1e-6, np.float32))
    codes, scales = quant.cast_to_fp8_int(bits)
    assert scales[0, 0] == np.float32(np.float32(1e-4) / np.float32(448.0))
    zero, zs = quant.cast_to_fp8_int(np.zeros((1, 128), np.uint16))
    assert not zero.any() and zs[0, 0] == scales[0, 0]


@pytest.mark.parametrize("seed,scale", [(0, 1.0), (1, 1e-3), (2, 300.0), (3, 1e-5), (4, 3e4), (5, 2.0**-20)])
def test_integer_form_matches_torch_form(seed, scale):
    gen = torch.Generator().manual_seed(seed)
    x = (torch.randn(64, 512, generator=gen) * scale).bfloat16()
    x[0, :128] = 0
    x[1, 5] = 7.5 * scale
    q_t, s_t = quant.cast_to_fp8_torch(x)
    q_i, s_i = quant.cast_to_fp8_int(_bits(x))
    np.testing.assert_array_equal(q_t.view(torch.uint8).numpy(), q_i)
    np.testing.assert_array_equal(s_t.numpy().view(np.uint32), s_i.view(np.uint32))


def test_integer_form_matches_torch_on_every_bf16_magnitude():
    # every finite positive bf16 pattern as the block maximum, with a spread of smaller entries
    mags = np.arange(0x0001, 0x7F80, 7, dtype=np.uint16)
    block = np.zeros((mags.size, 128), dtype=np.uint16)
    block[:, 0] = mags
    for j in range(1, 128):
        block[:, j] = np.maximum(mags.astype(np.int32) - 3 * j - (j % 5) * 128, 0).astype(np.uint16) | (0x8000 if j % 2 else 0)
    x = torch.from_numpy(block.view(np.int16)).view(torch.bfloat16)
    q_t, s_t = quant.cast_to_fp8_torch(x)
    q_i, s_i = quant.cast_to_fp8_int(block)
    np.testing.assert_array_equal(q_t.view(torch.uint8).numpy(), q_i)
    np.testing.assert_array_equal(s_t.numpy().view(np.uint32), s_i.view(np.uint32))


def test_integer_form_matches_torch_on_non_finite_blocks():
    """Infinities and NaNs: torch's amax() and clamp() both propagate NaN, so a block that holds one gets a NaN scale and
    the code 0x7F throughout; an infinite amax gives scale inf, zeros for the finite values and NaN for inf * 0."""
    import warnings

    from tests.gpu_util import non_finite_blocks

    x = non_finite_blocks()
    q_t, s_t = quant.cast_to_fp8_torch(x)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)
        q_i, s_i = quant.cast_to_fp8_int(_bits(x))
    np.testing.assert_array_equal(q_t.view(torch.uint8).numpy(), q_i)
    np.testing.assert_array_equal(s_t.numpy().view(np.uint32), s_i.view(np.uint32))
    assert (q_i[3, :128] == 0x7F).all() and (q_i[10, :128] == 0x7F).all() and (q_i[13, 128:] == 0x7F).all()
    assert np.isnan(s_i[3, 0]) and not np.isnan(s_i[3, 1]) and np.isinf(s_i[1, 0])
