"""W4A8 forward at seeded random shapes: sizes, expert ranges, top-k and tile heights drawn so that the grouped GEMM meets
column-tile counts that are no multiple of its panel width, experts without rows, single-row experts, tiles in several
rounds and both padded and unpadded K.  Each case is compared with the fp32 oracle and, where both grouped GEMM kernels
take the shape, the two kernels with each other bit for bit."""

import numpy as np
import pytest

from oracle import megamoe as mm
from tests.test_gpu_megamoe import _make_problem, _oracle, _run

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from deepep_amd import ops as module

    return module


def _draw(seed):
    rng = np.random.default_rng(1000 + seed)
    experts = int(rng.choice([2, 3, 6, 8, 16, 32, 48]))
    local = int(rng.integers(1, experts + 1))
    begin = int(rng.integers(0, experts - local + 1))
    topk = int(rng.integers(1, min(experts, 6) + 1))
    tokens = int(rng.choice([1, 7, 65, 130, 257, 400, 640]))
    hidden = int(rng.choice([64, 448, 512, 1024, 1536, 2304]))
    inter = int(rng.choice([128, 384, 512, 1024, 1280]))
    tile_rows = int(rng.choice([0, 64, 128, 192]))
    while local > 1 and local * 2 * inter * hidden > 60_000_000:  # keeps the oracle's fp32 weights to a few hundred MB
        local //= 2
    return tokens, hidden, inter, experts, begin, local, topk, tile_rows


@pytest.mark.parametrize("seed", range(48))
def test_forward_at_random_shapes(ops, seed):
    tokens, hidden, inter, experts, begin, local, topk, tile_rows = _draw(seed)
    case = dict(tokens=tokens, hidden=hidden, inter=inter, experts=experts, begin=begin, local=local, topk=topk, tile_rows=tile_rows)
    print(case, flush=True)
    x_codes, x_scales, l1, l2, idx, weights = _make_problem(tokens, hidden, inter, experts, begin, local, topk, seed=seed)
    got, counts = _run(ops, x_codes, x_scales, l1, l2, idx, weights, experts, begin, local, tile_rows=tile_rows)
    want = _oracle(x_codes, x_scales, l1, l2, idx, weights, begin)
    np.testing.assert_array_equal(counts, np.bincount(idx.ravel(), minlength=experts)[begin : begin + local], err_msg=str(case))
    assert np.isfinite(got).all(), case
    served = ((idx >= begin) & (idx < begin + local)).any(axis=1)
    assert not got[~served].any(), case
    if served.any():
        err = mm.relative_frobenius(got[served], want[served])
        assert err <= 2e-2, (err, case)
        # no single token may carry the error either (a wrong row hides in the norm of a large matrix)
        norms = np.linalg.norm(want[served], axis=1)
        per_token = np.linalg.norm(got[served] - want[served], axis=1) / np.maximum(norms, 1e-6 * norms.max() + 1e-30)
        assert per_token.max() <= 6e-2, (per_token.max(), case)
    other, _ = _run(ops, x_codes, x_scales, l1, l2, idx, weights, experts, begin, local, tile_rows=tile_rows, column_waves=0)
    np.testing.assert_array_equal(got.view(np.uint32), other.view(np.uint32), err_msg=str(case))
