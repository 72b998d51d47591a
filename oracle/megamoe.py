"""MegaMoE (W4A8) numeric oracle: MXFP8 per-32 quantizer, MXFP4 weight decode, expert FFN,
post-GMM2 route weighting.

Restates experiments/megamoe/python/deep_ep_experimental/megamoe/reference.py in integer/bit
arithmetic where the reference uses log2/searchsorted, so that the two are independent.

Pinned by (tests/test_oracle_megamoe.py), all vectors held by
experiments/megamoe/tests/test_reference.py:
  * all 254 finite FP8 codes round-trip, midpoints go to the even code, +-1000 saturate to
    126/254 (:22-34);
  * block scales 0.5 -> 118, 4.0 -> 121, zeros -> scale 0 and codes 0, exact restore (:37-45);
  * FP4 nibble order (low nibble = even k) and per-32 scale order (:48-54);
  * bf16 ties-to-even bit patterns (:73-76);
  * decomposition over expert subsets and the single-expert special case (:57-71);
  * route weight applied after GMM2 does not commute with quantization (:79-88);
  * the FFN itself reduces to a library matmul on dequantized fp32 operands;
  * ``swiglu``: closed forms (gate 0, sigmoid(ln 3) = 3/4, saturation, the clip at 80, operand roles) and
    torch's silu; ``expert_forward``: a hand-sized case whose every step is exact, written out in the
    test, and the same chain spelled with torch library routines (reference.py:84-89).
``quantize_weight_mxfp4`` is the build's own OCP-MX weight quantizer: the reference never quantizes weights
(reference.py:72-81 samples packed nibbles directly), so it holds no vector for it.  It is pinned to the OCP MX
v1.0 rule instead: a brute-force nearest-e2m1 search with explicit ties-to-even over block exponents, grid
values and midpoints.  It only builds test and benchmark inputs.

Test infrastructure: only tests/, the driver's smoke check and the benchmark's CPU-baseline leg use this module.
"""

from __future__ import annotations

import numpy as np

from .quant import e4m3fn_decode, e4m3fn_encode_rne, f32_to_bf16_bits, bf16_bits_to_f32

# OCP e2m1 value table indexed by nibble (reference.py:12).
E2M1 = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6, -0.0, -0.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float32)


def round_bf16(x):
    """float32 -> nearest BF16 value (ties to even), returned as float32 (reference.py:17-20)."""
    return bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(x, dtype=np.float32)))


def mx_quantize(x):
    """MXFP8 activation quantizer, block 32 along the last axis (reference.py:44-54).

    x is rounded to BF16 first.  Shared exponent = floor(log2(max(amax, 2^-119))) - 8, floored at
    -127; since amax is a finite fp32 at least 2^-119 its floor(log2) is the biased exponent
    field minus 127, so the e8m0 byte is simply ``biased_exponent(amax) - 8``.  Elements are
    x / 2^exp rounded to e4m3fn (nearest even, magnitude clamped to 448).
    Returns (codes uint8 [..., K], scales uint8 [..., K/32]).
    """
    x = round_bf16(x)
    if x.shape[-1] % 32:
        raise ValueError("last dimension must be a multiple of 32")
    if not np.isfinite(x).all():
        raise ValueError("finite inputs required")
    blocks = x.reshape(*x.shape[:-1], x.shape[-1] // 32, 32)
    amax = np.maximum(np.abs(blocks).max(axis=-1), np.float32(2.0**-119)).astype(np.float32)
    biased = (amax.view(np.uint32) >> np.uint32(23)).astype(np.int32)
    byte = np.maximum(biased - 8, 0)
    # Divide by 2^(byte-127): split the power so neither factor leaves the fp32 normal range.
    shift = 127 - byte
    half = shift // 2
    scaled = blocks * np.exp2(half).astype(np.float32)[..., None]
    scaled = scaled * np.exp2(shift - half).astype(np.float32)[..., None]
    codes = e4m3fn_encode_rne(scaled.astype(np.float32), saturate=True).reshape(x.shape)
    return codes, byte.astype(np.uint8)


def mx_dequantize(codes, scales):
    """fp32(code) * 2^(scale-127) per 32 elements (reference.py:57-59)."""
    codes = np.asarray(codes, dtype=np.uint8)
    values = e4m3fn_decode(codes)
    factor = np.exp2(np.asarray(scales, dtype=np.int32) - 127).astype(np.float32)
    return (values.reshape(*codes.shape[:-1], -1, 32) * factor[..., None]).reshape(codes.shape)


def unpack_weight(packed, scales):
    """MXFP4 weights -> dense float32 (reference.py:62-69).

    packed uint8 [..., N, K/2]: low nibble is element 2j, high nibble element 2j+1.
    scales e8m0 uint8 [..., N, K/64, 2] (or [..., N, K/32]): one power of two per 32 elements of K.
    """
    packed = np.asarray(packed, dtype=np.uint8)
    dense = np.empty(packed.shape[:-1] + (packed.shape[-1] * 2,), dtype=np.float32)
    dense[..., 0::2] = E2M1[packed & 0x0F]
    dense[..., 1::2] = E2M1[packed >> 4]
    groups = dense.shape[-1] // 32
    factor = np.exp2(np.asarray(scales, dtype=np.int32).reshape(*dense.shape[:-1], groups) - 127)
    return (dense.reshape(*dense.shape[:-1], groups, 32) * factor.astype(np.float32)[..., None]).reshape(dense.shape)


def quantize_weight_mxfp4(w):
    """Dense float32 [..., N, K] -> (packed uint8 [..., N, K/2], e8m0 uint8 [..., N, K/64, 2]).

    OCP MX v1.0 recipe: shared exponent = floor(log2(amax)) - 2 (e2m1 emax), elements rounded to
    e2m1 nearest-even with saturation at 6.  The build's own helper (the reference holds no weight quantizer);
    pinned to that rule by brute force in tests/test_oracle_megamoe.py.
    """
    w = np.asarray(w, dtype=np.float32)
    k = w.shape[-1]
    if k % 64:
        raise ValueError("K must be a multiple of 64")
    blocks = w.reshape(*w.shape[:-1], k // 32, 32)
    amax = np.abs(blocks).max(axis=-1)
    biased = (np.maximum(amax, np.float32(2.0**-125)).astype(np.float32).view(np.uint32) >> np.uint32(23)).astype(np.int32)
    byte = np.clip(biased - 2, 0, 254)
    scaled = blocks * np.exp2(127.0 - byte).astype(np.float32)[..., None]
    mag = np.minimum(np.abs(scaled), np.float32(6.0))
    # nearest e2m1 magnitude, ties to the even code: count the rounding boundaries passed
    # (0.25 -> 0, 0.75 -> 1.0, 1.25 -> 1.0, 1.75 -> 2.0, 2.5 -> 2.0, 3.5 -> 4.0, 5.0 -> 4.0).
    code = (mag > 0.25).astype(np.uint8)
    code += mag >= 0.75
    code += mag > 1.25
    code += mag >= 1.75
    code += mag > 2.5
    code += mag >= 3.5
    code += mag > 5.0
    nibble = code | (np.signbit(scaled).astype(np.uint8) << 3)
    nibble = nibble.reshape(*w.shape[:-1], k)
    packed = (nibble[..., 0::2] | (nibble[..., 1::2] << 4)).astype(np.uint8)
    return packed, byte.astype(np.uint8).reshape(*w.shape[:-1], k // 64, 2)


def swiglu(first):
    """bf16( gate / (1 + exp(clip(-gate, -80, 80))) * up ) with first = [gate | up] (reference.py:86-87)."""
    gate, up = np.split(np.asarray(first, dtype=np.float32), 2, axis=-1)
    return round_bf16(gate / (1 + np.exp(np.clip(-gate, -80, 80))) * up)


def expert_forward(x, w1, w2):
    """One expert on dense fp32 operands (reference.py:84-89).

    first = bf16(x @ w1^T); act = swiglu(first); qa = dequant(mx_quantize(act)); out = bf16(qa @ w2^T).
    x is already dequantized fp32 [m, H]; w1 [2I, H] (gate rows then up rows); w2 [H, I].
    """
    first = round_bf16(np.asarray(x, dtype=np.float32) @ np.asarray(w1, dtype=np.float32).T)
    act = swiglu(first)
    qa = mx_dequantize(*mx_quantize(act))
    return round_bf16(qa @ np.asarray(w2, dtype=np.float32).T)


def local_reference(x, indices, weights, l1, l2, first_expert=0, shared_l1=None, shared_l2=None):
    """fp32 sum over local experts (expert order) of expert_forward(x[token]) * w[token, slot]
    (reference.py:92-100); the caller rounds to BF16 at the end (golden.py:121-201).
    Shared experts follow the routed ones: every token, no route weight (golden.py:160-173)."""
    x = np.asarray(x, dtype=np.float32)
    indices = np.asarray(indices)
    result = np.zeros_like(x, dtype=np.float32)
    for local in range(len(l1)):
        token, slot = np.nonzero(indices == first_expert + local)
        if token.size:
            out = expert_forward(x[token], l1[local], l2[local])
            np.add.at(result, token, out * np.asarray(weights, dtype=np.float32)[token, slot, None])
    if shared_l1 is not None:
        for expert in range(len(shared_l1)):
            result += expert_forward(x, shared_l1[expert], shared_l2[expert])
    return result


def relative_frobenius(actual, expected):
    """||actual - expected||_F / ||expected||_F in fp64 (same quantity as relative_rmse,
    reference.py:103-114)."""
    a = np.asarray(actual, dtype=np.float64)
    e = np.asarray(expected, dtype=np.float64)
    return float(np.linalg.norm(a - e) / max(np.linalg.norm(e), 1e-30))
