"""The routing layout at seeded random shapes, every form of it against the CPU oracle bit for bit: the one-launch kernel,
the count + assign launches, the entry point that allocates nothing, and (up to 2048 routes) the kernel that lays out
and dispatches a small batch in one launch.  Draws reach the interface's corners: top-k 32, 1024 local experts, a single
token, expert ranges at either end of [0, E), skewed routing (most routes to a few experts) and masked routes."""

import numpy as np
import pytest
import torch

from deepep_amd import _lib
from oracle import layout as olayout
from tests.gpu_util import bf16_bits, i32
from tests.test_zz_no_alloc import _layout_static

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


def _draw(seed):
    rng = np.random.default_rng(5000 + seed)
    experts = int(rng.choice([1, 2, 7, 64, 256, 384, 1024, 4096]))
    local = int(min(experts, rng.choice([1, 2, 6, 32, 256, 1024])))
    begin = int(rng.choice([0, experts - local, rng.integers(0, experts - local + 1)]))
    topk = int(rng.choice([1, 2, 8, 9, 32]))
    tokens = int(rng.choice([1, 3, 64, 255, 256, 1000, 4096, 20000]))
    skew = bool(rng.integers(0, 2))
    masked = float(rng.choice([0.0, 0.1, 0.95]))
    return experts, begin, local, topk, tokens, skew, masked


def _compare(got, want, case):
    rows = want["num_rows"]
    assert int(got["num_rows"].item()) == rows, case
    for key in ("counts", "psum", "offsets", "route_to_row"):
        np.testing.assert_array_equal(i32(got[key]), want[key], err_msg=f"{key} {case}")
    np.testing.assert_array_equal(i32(got["row_to_route"][:rows]), want["row_to_route"], err_msg=str(case))


@pytest.mark.parametrize("seed", range(64))
def test_layout_forms_at_random_shapes(ops, ws, seed):
    experts, begin, local, topk, tokens, skew, masked = _draw(seed)
    case = dict(experts=experts, begin=begin, local=local, topk=topk, tokens=tokens, skew=skew, masked=masked)
    print(case, flush=True)
    rng = np.random.default_rng(seed)
    if skew:  # Zipf-like: most routes to the first few experts of a random order
        order = rng.permutation(experts)
        ids = order[np.minimum(rng.zipf(1.3, size=(tokens, topk)) - 1, experts - 1)]
    else:
        ids = rng.integers(0, experts, size=(tokens, topk))
    ids = ids.astype(np.int64)
    ids[rng.random(ids.shape) < masked] = -1
    ids[rng.random(ids.shape) < 0.01] = experts  # out of range: no row either
    want = olayout.layout(ids, experts, begin, local)
    idx = torch.from_numpy(ids).cuda()
    try:
        for one_launch in (1, 0):
            ws.tune("layout_one_launch", one_launch)
            got = ops.layout(ws, idx, experts, begin, local)
            host_counts, host_rows = ops.layout_wait(ws, local)
            assert host_rows == want["num_rows"] and host_counts == want["counts"].tolist(), case
            _compare(got, want, case)
    finally:
        ws.tune("layout_one_launch", 1)
    _compare(_layout_static(_lib.load(), idx, experts, begin, local), want, case)
    if tokens * topk <= ops.SMALL_BATCH_ROUTES:
        x = torch.from_numpy(rng.normal(size=(tokens, 64)).astype(np.float32)).bfloat16()
        plan, out, _, _ = ops.layout_dispatch_small(ws, idx, x.cuda(), None, None, experts, begin, local)
        _, host_rows = ops.layout_wait(ws, local)
        assert host_rows == want["num_rows"], case
        _compare(plan, want, case)
        np.testing.assert_array_equal(bf16_bits(out[:host_rows]), olayout.expand_rows(bf16_bits(x), want["row_to_route"], topk), err_msg=str(case))


@pytest.mark.parametrize(
    "experts,begin,local,tokens,topk",
    [
        (16384, 16256, 128, 4096, 32),  # the reference's largest expert count, the last rank's range, top-k 32
        (16384, 0, 1024, 20000, 8),     # the most local experts the layout takes
        (65536, 65000, 536, 3000, 9),   # expert numbers beyond 16 bits
        (16384, 8000, 1, 65536, 8),     # a single local expert at the largest batch: one long run of rows
    ],
)
def test_layout_at_the_largest_expert_counts(ops, ws, experts, begin, local, tokens, topk):
    rng = np.random.default_rng(experts + tokens)
    ids = rng.integers(-1, experts, size=(tokens, topk)).astype(np.int64)
    mine = rng.random((tokens, topk)) < 0.4  # (uniform routing alone would leave the local range almost empty)
    ids[mine] = rng.integers(begin, begin + local, size=int(mine.sum()))
    want = olayout.layout(ids, experts, begin, local)
    assert want["num_rows"] > tokens
    idx = torch.from_numpy(ids).cuda()
    case = dict(experts=experts, begin=begin, local=local, tokens=tokens, topk=topk)
    try:
        for one_launch in (1, 0):
            ws.tune("layout_one_launch", one_launch)
            _compare(ops.layout(ws, idx, experts, begin, local), want, case)
    finally:
        ws.tune("layout_one_launch", 1)
    _compare(_layout_static(_lib.load(), idx, experts, begin, local), want, case)
