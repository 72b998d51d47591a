"""Per-128-element FP8 e4m3fn block quantizer oracle (and its inverse).

Two independent restatements of per_token_cast_to_fp8 (deep_ep/utils/math.py:45-61; duplicate
tests/clos/common.py:50-58; scalar emulation tests/utils/precision.py:115-128):

  * ``cast_to_fp8_torch``  — the reference's expression evaluated with torch CPU as a library
    (abs / amax / clamp / fp32 multiply / .to(float8_e4m3fn));
  * ``cast_to_fp8_int``    — NumPy fp32 arithmetic plus an integer round-to-nearest-even encoder
    that shares no code with torch's cast.

Pinned by (tests/test_oracle_quant.py): the two agree bit-for-bit on random, tiny, huge and
clamped blocks; the reference's anchors quantize_e4m3fn(+-500)=+-448 (saturating scalar emulation),
2^-9 -> 2^-9, bf16 tie 1.00390625 -> 1.0 (tests/test_precision.py:76-82); the per-128 anchor
[1.0]*128+[224,448] whose second block restores exactly (224, 448) (tests/test_precision.py:84-89);
the amax floor 1e-4; all 254 finite codes round-trip through decode/encode.
"""

from __future__ import annotations

import numpy as np

E4M3_MAX = 448.0


def bf16_bits_to_f32(bits):
    """Widen BF16 bit patterns (uint16) to float32 exactly."""
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(values):
    """Round float32 to BF16 bit patterns, ties to even (finite inputs).

    Same rounding as quantize_bfloat16 (tests/utils/precision.py:72-80) and bf16()
    (experiments/megamoe/python/deep_ep_experimental/megamoe/reference.py:17-20).
    """
    values = np.ascontiguousarray(values, dtype=np.float32)
    bits = values.view(np.uint32)
    rounded = bits + np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1))
    return (rounded >> np.uint32(16)).astype(np.uint16)


def e4m3fn_decode(codes):
    """Decode e4m3fn bytes to float32 (0x7F / 0xFF decode to NaN) — tests/utils/precision.py:83-95."""
    codes = np.asarray(codes, dtype=np.uint8)
    mag = (codes & 0x7F).astype(np.int32)
    exponent, mantissa = mag >> 3, mag & 7
    value = np.where(
        exponent == 0,
        mantissa * 2.0**-9,
        (1.0 + mantissa / 8.0) * np.exp2((exponent - 7).astype(np.float64)),
    )
    value = np.where(mag == 0x7F, np.nan, value)
    return (np.where(codes & 0x80, -value, value)).astype(np.float32)


def e4m3fn_encode_rne(values, saturate=False):
    """float32 -> e4m3fn byte, round-to-nearest-even, integer arithmetic only.

    ``saturate=False`` mirrors torch's ``.to(float8_e4m3fn)``: a magnitude that rounds above 448
    becomes the NaN code 0x7F.  ``saturate=True`` clamps the magnitude to 448 first, like
    quantize_e4m3fn (tests/utils/precision.py:100-112) and fp8_encode
    (experiments/megamoe/.../reference.py:31-41).
    """
    values = np.ascontiguousarray(values, dtype=np.float32)
    bits = values.view(np.uint32)
    sign = ((bits >> np.uint32(24)) & np.uint32(0x80)).astype(np.uint8)
    mag = bits & np.uint32(0x7FFFFFFF)
    if saturate:
        mag = np.minimum(mag, np.float32(E4M3_MAX).view(np.uint32))
    # Normal e4m3 range starts at 2^-6 (fp32 biased exponent 121).
    normal = mag >= np.uint32(121 << 23)
    rounded = mag + np.uint32(0x7FFFF) + ((mag >> np.uint32(20)) & np.uint32(1))
    code_normal = (rounded >> np.uint32(20)).astype(np.int64) - ((127 - 7) << 3)
    # Subnormal: multiples of 2^-9; |v|*512 is exact in fp32 and rint() is ties-to-even.
    code_sub = np.rint(mag.view(np.float32).astype(np.float64) * 512.0).astype(np.int64)
    code = np.where(normal, code_normal, code_sub)
    code = np.where(code > 0x7E, 0x7F, code)
    return code.astype(np.uint8) | sign


def cast_to_fp8_int(x_bf16_bits):
    """per_token_cast_to_fp8 with NumPy fp32 + the integer encoder.  x: uint16 [T, H], H % 128 == 0.

    amax = max|x| per 128 columns in fp32, clamped below at fp32(1e-4);
    inv = fp32(fp32(1/amax) * 448): the reference writes ``448.0 / amax`` and torch evaluates a
    scalar divided by a tensor as ``amax.reciprocal() * 448.0`` — two roundings, not one division;
    q = rne_e4m3fn(fp32(x) * inv) (bf16 x fp32 promotes to an fp32 multiply);
    scale = amax / fp32(448) (a true fp32 division).
    """
    bits = np.asarray(x_bf16_bits, dtype=np.uint16)
    tokens, hidden = bits.shape
    if hidden % 128:
        raise ValueError("hidden must be a multiple of 128")
    x = bf16_bits_to_f32(bits).reshape(tokens, hidden // 128, 128)
    amax = np.maximum(np.abs(x).max(axis=2), np.float32(1e-4)).astype(np.float32)
    inv = ((np.float32(1.0) / amax).astype(np.float32) * np.float32(E4M3_MAX)).astype(np.float32)
    prod = (x * inv[:, :, None]).astype(np.float32)
    codes = e4m3fn_encode_rne(prod).reshape(tokens, hidden)
    scales = (amax / np.float32(E4M3_MAX)).astype(np.float32)
    return codes, scales


def cast_to_fp8_torch(x):
    """The reference expression itself on a torch CPU BF16 tensor (deep_ep/utils/math.py:45-61)."""
    import torch

    tokens, hidden = x.shape
    if hidden % 128:
        raise ValueError("hidden must be a multiple of 128")
    view = x.view(tokens, -1, 128)
    amax = view.abs().float().amax(dim=2).view(tokens, -1).clamp(1e-4)
    q = (view * (448.0 / amax.unsqueeze(2))).to(torch.float8_e4m3fn)
    return q.view(tokens, hidden).contiguous(), (amax / 448.0).view(tokens, -1)


def cast_back(codes, scales):
    """per_token_cast_back (deep_ep/utils/math.py:64-79): bf16_rne(fp32(q) * scale) as uint16 bits."""
    codes = np.asarray(codes, dtype=np.uint8)
    tokens, hidden = codes.shape
    x = e4m3fn_decode(codes).reshape(tokens, hidden // 128, 128)
    prod = (x * np.asarray(scales, dtype=np.float32)[:, :, None]).astype(np.float32)
    return f32_to_bf16_bits(prod.reshape(tokens, hidden))
