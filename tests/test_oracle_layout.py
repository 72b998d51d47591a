"""Pins the layout oracle against reference-held vectors, brute force and invariants."""

import hashlib
import json
import os

import numpy as np
import pytest

from oracle import cases
from oracle.layout import expand_rows, expand_weights, layout, layout_bruteforce

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "reference_layout_digests.json")


def _flatten(routes):
    """Concatenate per-source route tables: global token = (source, token) in source-major order."""
    rows = [row for rank in routes for row in rank]
    topk = len(rows[0]) if rows else 0
    return np.asarray(rows, dtype=np.int64).reshape(len(rows), topk)


def test_reference_hand_case():
    # tests/test_reference.py:22-58: 2 ranks, 4 experts; counts ((1,3),(1,0)); rank-0 expanded rows.
    routes = (((0, 1), (2, -1)), ((1, 1),))
    idx = _flatten(routes)
    per_rank = [layout(idx, 4, begin, 2) for begin in (0, 2)]
    assert [tuple(p["counts"].tolist()) for p in per_rank] == [(1, 3), (1, 0)]
    # (expert, source, token, slot) of rank 0 = flat routes 0, 1, 4, 5 (source 1 token 0 is global token 2).
    assert per_rank[0]["row_to_route"].tolist() == [0, 1, 4, 5]
    weights = np.asarray([[0.25, 0.5], [0.75, 9.0], [0.125, 0.625]], dtype=np.float32)
    assert expand_weights(weights, per_rank[0]["row_to_route"]).tolist() == [0.25, 0.5, 0.125, 0.625]
    x = np.asarray([[2], [3], [5]])
    assert expand_rows(x, per_rank[0]["row_to_route"], 2).ravel().tolist() == [2, 2, 5, 5]
    assert per_rank[1]["route_to_row"].tolist() == [[-1, -1], [0, -1], [-1, -1]]


def test_hand_computed_rank_rows():
    # tests/elastic/test_dispatch.py:1951-1958: two ranks x one token, EP2, E=4 -> rank_rows [2, 2].
    idx = _flatten((((0, 2),), ((1, 3),)))
    assert [layout(idx, 4, b, 2)["num_rows"] for b in (0, 2)] == [2, 2]
    # duplicates produce one row per slot
    assert layout(np.asarray([[1, 1]]), 4)["counts"].tolist() == [0, 2, 0, 0]


def _digest(value):
    return hashlib.sha256(json.dumps(value, ensure_ascii=True, separators=(",", ":")).encode("ascii")).hexdigest()


@pytest.mark.parametrize("case", json.load(open(GOLDEN))["cases"], ids=lambda c: c["name"])
def test_golden_manifest_digests(case):
    cfg = case["config"]
    world, experts, topk = cfg["world_size"], cfg["experts"], cfg["topk"]
    routes = cases.matrix_routes(world, experts, topk, cfg["tokens_per_rank"])
    idx = _flatten(routes)
    assert int((idx >= 0).sum()) == case["valid_route_slots"]
    local = experts // world
    per_rank = [layout(idx, experts, rank * local, local) for rank in range(world)]
    assert [p["num_rows"] for p in per_rank] == case["expanded_rows"]
    assert _digest([p["counts"].tolist() for p in per_rank]) == case["expert_counts_sha256"]


@pytest.mark.parametrize("seed", range(6))
def test_matches_bruteforce_and_invariants(seed):
    rng = np.random.default_rng(seed)
    tokens, topk, experts = int(rng.integers(0, 40)), int(rng.integers(1, 9)), int(rng.integers(1, 20))
    begin = int(rng.integers(0, experts))
    local = int(rng.integers(1, experts - begin + 1))
    idx = rng.integers(-2, experts + 2, size=(tokens, topk))
    fast, slow = layout(idx, experts, begin, local), layout_bruteforce(idx, experts, begin, local)
    for key in ("counts", "psum", "offsets", "route_to_row", "row_to_route"):
        np.testing.assert_array_equal(fast[key], slow[key], err_msg=key)
    r2r, r2t = fast["route_to_row"].reshape(-1), fast["row_to_route"]
    valid = (idx.reshape(-1) >= begin) & (idx.reshape(-1) < begin + local) & (idx.reshape(-1) < experts)
    assert fast["num_rows"] == int(valid.sum()) == int(fast["counts"].sum())
    assert (fast["psum"][-1] if local else 0) == fast["num_rows"]
    np.testing.assert_array_equal(np.sort(r2r[valid]), np.arange(fast["num_rows"]))
    assert (r2r[~valid] == -1).all()
    np.testing.assert_array_equal(r2r[r2t], np.arange(fast["num_rows"]))
    for e in range(local):
        seg = r2t[fast["offsets"][e] : fast["offsets"][e + 1]]
        assert (np.diff(seg) > 0).all()
        assert (idx.reshape(-1)[seg] == begin + e).all()


def test_empty_and_all_masked():
    out = layout(np.zeros((0, 4), dtype=np.int64), 8)
    assert out["num_rows"] == 0 and out["counts"].tolist() == [0] * 8
    out = layout(np.full((5, 2), -1), 4)
    assert out["num_rows"] == 0 and (out["route_to_row"] == -1).all()
