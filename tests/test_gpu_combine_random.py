"""Every form of the combine at seeded random shapes against the CPU oracle, bit for bit: dense and sparse maps (which pick
different kernels and grids), BF16 and FP16 rows, no weights or a weight per row, the weight-return channel, rows that
the caller's tensor does not hold (treated as absent), and the form that leaves unserved tokens untouched."""

import numpy as np
import pytest
import torch

from oracle import combine as ocombine
from tests.gpu_util import bf16_bits, f32_bits

pytestmark = pytest.mark.gpu


def _draw(seed):
    rng = np.random.default_rng(11000 + seed)
    tokens = int(rng.choice([1, 2, 63, 64, 65, 500, 4096, 20000]))
    topk = int(rng.choice([1, 2, 4, 8, 9, 32]))
    hidden = int(rng.choice([8, 16, 72, 512, 520, 1024, 7168]))
    while tokens * hidden > 24_000_000:
        tokens //= 2
    density = float(rng.choice([0.0, 0.01, 0.1, 0.5, 1.0]))
    half = bool(rng.integers(0, 4) == 0)
    weighted = bool(rng.integers(0, 2))
    returned = bool(rng.integers(0, 2))
    served_only = bool(rng.integers(0, 3) == 0) and not half
    short_by = int(rng.choice([0, 0, 1, 7]))  # rows of the map that the caller's tensor does not hold
    return tokens, topk, hidden, density, half, weighted, returned, served_only, short_by


@pytest.mark.parametrize("seed", range(96))
def test_combine_forms_at_random_shapes(seed):
    from deepep_amd import ops

    tokens, topk, hidden, density, half, weighted, returned, served_only, short_by = _draw(seed)
    case = dict(tokens=tokens, topk=topk, hidden=hidden, density=density, half=half, weighted=weighted, returned=returned,
                served_only=served_only, short_by=short_by)
    print(case, flush=True)
    rng = np.random.default_rng(seed)
    valid = rng.random((tokens, topk)) < density
    rows_in_map = int(valid.sum())
    # a permutation of the rows over the valid routes (any one-to-one map is a legal route_to_row)
    route_to_row = np.full((tokens, topk), -1, dtype=np.int32)
    route_to_row[valid] = rng.permutation(rows_in_map).astype(np.int32)
    rows = max(0, rows_in_map - short_by)
    held = np.where(route_to_row >= rows, -1, route_to_row)  # what the oracle sees: rows past the tensor are absent
    dtype = torch.float16 if half else torch.bfloat16
    y = torch.from_numpy(rng.normal(size=(rows, hidden)).astype(np.float32) * 2).to(dtype)
    weights = rng.random(rows).astype(np.float32) * 2 - 0.5 if weighted else None
    values = rng.random(rows).astype(np.float32) if returned else None
    sentinel = 5.0
    out = torch.full((tokens, hidden), sentinel, dtype=dtype, device="cuda")
    got, got_values = ops.combine(y.cuda(), torch.from_numpy(route_to_row).cuda(),
                                  None if weights is None else torch.from_numpy(weights).cuda(),
                                  None if values is None else torch.from_numpy(values).cuda(), out=out, served_only=served_only)
    assert got.data_ptr() == out.data_ptr()
    if half:
        want = ocombine.combine_fp16(y.numpy(), held, weights)
        got_bits, want_bits = got.cpu().numpy().view(np.uint16), want.view(np.uint16)
    else:
        want_bits = ocombine.combine(bf16_bits(y), held, weights)
        got_bits = bf16_bits(got)
    served = (held >= 0).any(axis=1)
    np.testing.assert_array_equal(got_bits[served], want_bits[served], err_msg=str(case))
    if served_only:
        assert (got[torch.from_numpy(~served).cuda()] == sentinel).all(), case
    else:
        assert not got_bits[~served].any(), case
    if returned:
        np.testing.assert_array_equal(f32_bits(got_values), ocombine.return_weights(values, held).view(np.uint32), err_msg=str(case))
