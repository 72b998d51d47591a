"""Pins the MegaMoE oracle on the vectors held by experiments/megamoe/tests/test_reference.py."""

import numpy as np

from oracle import megamoe as mm
from oracle.quant import e4m3fn_decode, e4m3fn_encode_rne, f32_to_bf16_bits


def test_fp8_codes_midpoints_saturation():  # :22-34
    codes = np.concatenate((np.arange(127), np.arange(128, 255))).astype(np.uint8)
    np.testing.assert_array_equal(e4m3fn_encode_rne(e4m3fn_decode(codes), saturate=True), codes)
    np.testing.assert_array_equal(e4m3fn_encode_rne(np.asarray([1000, -1000], np.float32), saturate=True), [126, 254])
    # closed form of the positive table: c<8 -> c*2^-9 else (1+(c%8)/8)*2^(c//8-7)
    c = np.arange(127)
    table = np.where(c < 8, c * 2.0**-9, (1 + (c % 8) / 8) * np.exp2(c // 8 - 7)).astype(np.float32)
    np.testing.assert_array_equal(e4m3fn_decode(c.astype(np.uint8)), table)


def test_quant_block_scale_and_zero():  # :37-45
    x = np.full((2, 64), 0.5, dtype=np.float32)
    x[:, 32:] = 4.0
    codes, scale = mm.mx_quantize(x)
    np.testing.assert_array_equal(scale, [[118, 121], [118, 121]])
    np.testing.assert_array_equal(mm.mx_dequantize(codes, scale), x)
    codes, scale = mm.mx_quantize(np.zeros((1, 32), np.float32))
    assert not codes.any() and not scale.any()


def test_mx_quantize_matches_float_log2_form():
    # the reference's floating form: exp = max(floor(log2(max(amax, 2^-119))) - 8, -127)
    rng = np.random.default_rng(3)
    x = (rng.normal(size=(64, 256)) * np.exp2(rng.integers(-40, 30, size=(64, 1)))).astype(np.float32)
    x[0, :32] = 448.0
    x[1, :32] = 2.0**-130
    codes, scale = mm.mx_quantize(x)
    xb = mm.round_bf16(x).reshape(64, 8, 32)
    amax = np.abs(xb).max(-1)
    exponent = np.maximum(np.floor(np.log2(np.maximum(amax, 2.0**-119))) - 8, -127)
    np.testing.assert_array_equal(scale, (exponent + 127).astype(np.uint8))
    want = e4m3fn_encode_rne((xb / np.exp2(exponent).astype(np.float32)[..., None]).reshape(64, 256), saturate=True)
    np.testing.assert_array_equal(codes, want)


def test_fp4_nibble_and_scale_order():  # :48-54
    packed = np.tile(np.arange(16, dtype=np.uint8) | (np.arange(16, dtype=np.uint8)[::-1] << 4), 2).reshape(1, 1, 32)
    scales = np.array([[[[127, 128]]]], dtype=np.uint8)
    result = mm.unpack_weight(packed, scales)[0, 0]
    np.testing.assert_array_equal(result[:32:2], mm.E2M1)
    np.testing.assert_array_equal(result[1:32:2], mm.E2M1[::-1])
    np.testing.assert_array_equal(result[32:], result[:32] * 2)


def test_bf16_ties_to_even():  # :73-76
    values = np.array([0x3F808000, 0x3F818000], np.uint32).view(np.float32)
    np.testing.assert_array_equal(f32_to_bf16_bits(values), [0x3F80, 0x3F82])


def test_decomposition_and_single_expert():  # :57-71
    rng = np.random.default_rng(7)
    x = rng.normal(size=(3, 32)).astype(np.float32) * 0.1
    w1 = rng.normal(size=(4, 64, 32)).astype(np.float32) * 0.1
    w2 = rng.normal(size=(4, 32, 32)).astype(np.float32) * 0.1
    ids = np.array([[0, 2], [2, 0], [0, 0]])
    weights = np.array([[0.2, 0.8], [0.7, 0.3], [0.5, 0.5]], np.float32)
    full = mm.local_reference(x, ids, weights, w1, w2, 0)
    split = mm.local_reference(x, ids, weights, w1[:2], w2[:2], 0) + mm.local_reference(x, ids, weights, w1[2:], w2[2:], 2)
    np.testing.assert_allclose(full, split, atol=1e-8)
    np.testing.assert_allclose(full[2:3], mm.expert_forward(x[2:3], w1[0], w2[0]))


def test_shared_experts_are_dense_unweighted_terms():
    # golden.py:160-173: a shared expert takes every token, no route weight, after the routed experts; so the
    # result equals the routed part plus a one-expert "route everything with weight 1" problem per shared expert
    rng = np.random.default_rng(11)
    x = rng.normal(size=(5, 32)).astype(np.float32) * 0.1
    w1 = rng.normal(size=(3, 64, 32)).astype(np.float32) * 0.1
    w2 = rng.normal(size=(3, 32, 32)).astype(np.float32) * 0.1
    s1 = rng.normal(size=(2, 64, 32)).astype(np.float32) * 0.1
    s2 = rng.normal(size=(2, 32, 32)).astype(np.float32) * 0.1
    ids = rng.integers(0, 3, size=(5, 1))
    weights = rng.random((5, 1)).astype(np.float32)
    routed = mm.local_reference(x, ids, weights, w1, w2, 0)
    full = mm.local_reference(x, ids, weights, w1, w2, 0, s1, s2)
    dense = sum(mm.local_reference(x, np.zeros((5, 1), int), np.ones((5, 1), np.float32), s1[e : e + 1], s2[e : e + 1], 0)
                for e in range(2))
    np.testing.assert_allclose(full, routed + dense, atol=1e-7)
    assert np.abs(dense).max() > 0


def test_route_weight_does_not_commute_with_quantization():  # :79-88
    rng = np.random.default_rng(31)
    act = rng.normal(size=(8, 64)).astype(np.float32)
    w2 = rng.normal(size=(32, 64)).astype(np.float32)
    weight = np.array([0.1, -0.37, 0.8, 0.003, 0.19, 0, 0.47, 1], np.float32)[:, None]
    current = mm.round_bf16(mm.mx_dequantize(*mm.mx_quantize(act)) @ w2.T) * weight
    before = mm.round_bf16(mm.mx_dequantize(*mm.mx_quantize(act * weight)) @ w2.T)
    assert mm.relative_frobenius(current, before) > 1e-3
    np.testing.assert_array_equal(current[5], 0)


def test_own_mxfp4_weight_quantizer_is_consistent():
    # self-consistency (the rounding rule itself is pinned by the brute-force test below): exactly representable
    # weights survive, and the error on Gaussian weights stays inside the e2m1 step bound.
    rng = np.random.default_rng(0)
    exact = (mm.E2M1[rng.integers(0, 16, size=(2, 8, 64))] * np.float32(2.0**-7)).astype(np.float32)
    exact[..., 0] = 6 * 2.0**-7
    exact[..., 32] = -6 * 2.0**-7
    packed, scales = mm.quantize_weight_mxfp4(exact)
    np.testing.assert_array_equal(mm.unpack_weight(packed, scales), exact)
    w = (rng.normal(size=(2, 16, 128)) * 0.02).astype(np.float32)
    back = mm.unpack_weight(*mm.quantize_weight_mxfp4(w))
    assert mm.relative_frobenius(back, w) < 0.2


# ---- swiglu / expert_forward / quantize_weight_mxfp4 pinned independently of the oracle's own formulas -----------
def _torch_bf16(values):
    import torch

    return torch.from_numpy(np.ascontiguousarray(values, dtype=np.float32)).bfloat16().float().numpy()


def test_swiglu_closed_forms_and_operand_roles():
    # reference.py:85-87: first = [gate | up]; act = bf16(gate / (1 + exp(clip(-gate, +-80))) * up).
    # Numbers written out here (fp64 arithmetic, torch's BF16 cast), not taken from the oracle.
    ln3 = float(np.log(3.0))
    gate = np.array([0.0, ln3, ln3, 30.0, -30.0, -100.0, 2.0, -2.0], np.float32)
    up = np.array([5.0, 1.0, -2.0, 0.5, 0.5, 1.0, 3.0, 3.0], np.float32)
    want = np.array([
        0.0,                                  # gate 0 -> 0 whatever up is
        0.75 * ln3,                           # sigmoid(ln 3) = 3/4
        -1.5 * ln3,
        15.0,                                 # large gate: silu(gate) = gate
        -30.0 / (1.0 + np.exp(30.0)) * 0.5,   # large negative gate: tiny, negative, not zero
        -100.0 / (1.0 + np.exp(80.0)),        # the clip: exp(100) would overflow fp32 and give -0
        2.0 / (1.0 + np.exp(-2.0)) * 3.0,
        -2.0 / (1.0 + np.exp(2.0)) * 3.0,
    ])
    got = mm.swiglu(np.concatenate([gate, up])[None, :])[0]
    expected = _torch_bf16(want)
    # the fp32 exp differs from fp64 by at most an ulp before the BF16 rounding: allow one BF16 step (2^-8 relative)
    np.testing.assert_allclose(got, expected, rtol=2.0**-8, atol=0)
    np.testing.assert_array_equal(got[[0, 3]], [0.0, 15.0])
    assert got[5] != 0.0 and abs(got[5] + 100.0 / (1.0 + np.exp(80.0))) < 1e-35  # a missing clip gives -0
    # a gate/up swap, a missing sigmoid or gelu instead of silu all fail here:
    swapped = mm.swiglu(np.concatenate([up, gate])[None, :])[0]
    assert not np.allclose(swapped[[1, 2, 6]], expected[[1, 2, 6]], rtol=2.0**-6)


def test_swiglu_matches_torch_silu():
    import torch

    rng = np.random.default_rng(5)
    first = _torch_bf16(rng.normal(size=(64, 256)) * 4.0)
    gate, up = torch.from_numpy(first[:, :128]), torch.from_numpy(first[:, 128:])
    want = (torch.nn.functional.silu(gate) * up).bfloat16().float().numpy()
    got = mm.swiglu(first)
    # x * sigmoid(x) and x / (1 + exp(-x)) round differently in fp32 now and then: at most one BF16 step apart
    np.testing.assert_allclose(got, want, rtol=2.0**-7, atol=1e-30)
    assert (got == want).mean() > 0.97


def test_expert_forward_hand_case():
    # reference.py:84-89 on numbers chosen so that every step is exact and can be written down:
    # for gate >= 32, 1 + exp(-gate) == 1 in fp32, so silu(gate) == gate; products are small integers.
    hidden, inter = 32, 32
    x = np.zeros((1, hidden), np.float32)
    x[0, 0], x[0, 1] = 1.0, 2.0
    w1 = np.zeros((2 * inter, hidden), np.float32)   # rows [0, I) gate, rows [I, 2I) up
    gates = [32.0, 64.0, 32.0, 0.0, 32.0]
    ups = [0.5, -0.25, 1.5, 1.0, 0.515625]            # up_j = 2 * ups[j] (x[1] = 2)
    for j, (g, u) in enumerate(zip(gates, ups)):
        w1[j, 0] = g
        w1[inter + j, 1] = u
    # act = gate * up = [32, -32, 96, 0, 33]; block amax 96 -> exponent floor(log2 96) - 8 = -2, scale 1/4:
    # codes 128, -128, 384 exact; 33 / 0.25 = 132 lies between e4m3 128 and 144 -> 128 -> dequantised 32.
    act = np.array([32.0, -32.0, 96.0, 0.0, 33.0])
    np.testing.assert_array_equal(mm.swiglu((x @ w1.T))[0, :5], act)
    qa = np.array([32.0, -32.0, 96.0, 0.0, 32.0])
    w2 = np.zeros((hidden, inter), np.float32)
    w2[0, :2] = [1.0, 0.5]            # 32 - 16
    w2[1, 2] = 0.25                   # 24
    w2[2, :3] = [1.0, 1.0, 1.0]       # 96
    w2[3, 4] = 1.0                    # 32 (33 if the requantisation were skipped)
    w2[4, 3] = 7.0                    # 0
    w2[5, :5] = [2.0, 0.0, -1.0, 3.0, 0.5]  # 64 - 96 + 16 = -16
    want = np.zeros(hidden, np.float32)
    want[:6] = [16.0, 24.0, 96.0, 32.0, 0.0, -16.0]
    np.testing.assert_array_equal(want[:6], (qa[None, :] @ w2[:6, :5].T)[0])
    np.testing.assert_array_equal(mm.expert_forward(x, w1, w2)[0], want)
    # gate rows and up rows exchanged: silu(1) * 32 etc. - a different answer
    w1_swapped = np.concatenate([w1[inter:], w1[:inter]])
    assert not np.array_equal(mm.expert_forward(x, w1_swapped, w2)[0], want)


def test_expert_forward_matches_torch_chain():
    # the same chain spelled with torch library routines (matmul, F.silu, BF16 casts) on asymmetric random data;
    # the MXFP8 step uses mx_quantize / mx_dequantize, which the vectors above pin.
    import torch

    rng = np.random.default_rng(17)
    x = _torch_bf16(rng.normal(size=(6, 64)))
    w1 = (rng.normal(size=(128, 64)) * 0.2).astype(np.float32)
    w1[64:] *= 3.0  # up rows differ in scale from gate rows
    w2 = (rng.normal(size=(64, 64)) * 0.2).astype(np.float32)
    first = (torch.from_numpy(x) @ torch.from_numpy(w1).T).bfloat16().float()
    act = (torch.nn.functional.silu(first[:, :64]) * first[:, 64:]).bfloat16().float().numpy()
    qa = mm.mx_dequantize(*mm.mx_quantize(act))
    want = (torch.from_numpy(qa) @ torch.from_numpy(w2).T).bfloat16().float().numpy()
    got = mm.expert_forward(x, w1, w2)
    assert mm.relative_frobenius(got, want) < 2e-3  # BF16 / e4m3 steps of a few elements whose silu rounds the other way
    swapped = mm.expert_forward(x, np.concatenate([w1[64:], w1[:64]]), w2)
    assert mm.relative_frobenius(swapped, want) > 0.1


def _nearest_e2m1_ties_even(magnitude):
    """Brute force: the e2m1 code (0..7) nearest to magnitude; of two equally near, the even code."""
    grid = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
    best, best_distance = 0, None
    for code, value in enumerate(grid):
        distance = abs(float(magnitude) - value)
        if best_distance is None or distance < best_distance or (distance == best_distance and code % 2 == 0 and best % 2 == 1):
            best, best_distance = code, distance
    return best


def test_mxfp4_weight_quantizer_against_brute_force():
    # OCP MX v1.0: shared exponent = floor(log2(amax)) - 2 (e2m1 emax); elements to the nearest e2m1 value,
    # ties to the even code, saturating at 6.  Block exponents across the byte's range, every grid value, every
    # midpoint and a hair either side of each.
    grid = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    mids = [(a + b) / 2 for a, b in zip(grid[:-1], grid[1:])]
    probes = sorted(set(grid + mids + [m * (1 - 2.0**-20) for m in mids] + [m * (1 + 2.0**-20) for m in mids] + [5.5, 7.0, 7.9]))
    assert len(probes) > 30
    rows = [probes[i : i + 30] for i in range(0, len(probes), 30)]
    checked = 0
    for exponent in list(range(-120, 121, 7)) + [-125, -1, 0, 1, 124]:
        unit = 2.0**exponent  # value of an element code 1.0: amax lies in [4, 8) units
        for top in (4.0, 5.0, 6.0, 7.9):
            for chunk in rows:
                magnitudes = np.array([top, top] + chunk + [0.0] * (30 - len(chunk)))
                signs = np.where(np.arange(32) % 3 == 1, -1.0, 1.0)
                block = np.zeros(64, np.float32)  # second block of the row: zeros -> byte 0, codes 0
                block[:32] = (magnitudes * signs * unit).astype(np.float32)
                packed, scales = mm.quantize_weight_mxfp4(block[None, :])
                np.testing.assert_array_equal(scales.reshape(-1), [exponent + 127, 0])
                nibbles = np.stack([packed[0] & 15, packed[0] >> 4], -1).reshape(-1)
                assert not nibbles[32:].any()
                for k in range(32):
                    scaled = abs(float(block[k])) / unit
                    want = _nearest_e2m1_ties_even(min(scaled, 6.0)) | (8 if np.signbit(block[k]) else 0)
                    assert nibbles[k] == want, (exponent, top, k, block[k], nibbles[k], want)
                    checked += 1
    assert checked > 8000
    # the second block of a row has its own exponent, stored next to the first: [N, K/64, 2]
    row = np.zeros(64, np.float32)
    row[:32], row[32:] = 6.0, 0.75
    packed, scales = mm.quantize_weight_mxfp4(row[None, :])
    np.testing.assert_array_equal(scales.reshape(-1), [127, 124])
    np.testing.assert_array_equal(mm.unpack_weight(packed, scales)[0], row)
