"""Routing layout oracle: validity, per-expert counts, prefix sums, stable permutation.

Pinned by (tests/test_oracle_layout.py):
  * the reference's hand case (tests/test_reference.py:22-58): counts ((1,3),(1,0)) and the
    expanded row tuples of rank 0;
  * the golden manifest digests valid_route_slots / expanded_rows / expert_counts_sha256
    (tests/golden/deepep_reference_v2.json) over the restated deterministic generator;
  * brute force: ``layout`` (vectorised stable sort) == ``layout_bruteforce`` (scalar loops in the
    reference's own row order) on random small inputs;
  * invariants: rows are a permutation of the valid routes, row_to_route strictly increasing
    inside an expert, psum[-1] == R.
"""

from __future__ import annotations

import numpy as np


def layout(topk_idx, num_experts, expert_begin=0, num_local=None):
    """Stable counting sort of the T*K routes by local expert.

    Follows: validity ``0 <= e < E`` (csrc/kernels/notify/notify.cpp:58, tests/utils/reference.py:45);
    a route belongs to this rank when ``expert_begin <= e < expert_begin + L``
    (tests/elastic/test_dispatch.py:538-548); counts are per *slot*, duplicates count separately
    (tests/utils/reference.py:46-47); row order is (local expert, source, token, slot)
    (tests/utils/reference.py:70) which for one flattened source stream is (expert, flat route id);
    ``psum`` is the inclusive int32 cumsum (deep_ep/backends/mesh_clos/elastic.py:1475);
    ``offsets`` is the exclusive form with a leading 0 (tests/clos/common.py:254-255);
    ``route_to_row`` is recv_to_expanded_idx with -1 for routes that produce no row
    (tests/clos/common.py:257-279); ``row_to_route`` is weight_return_meta = (src*T+t)*K+s
    (tests/elastic/test_dispatch.py:402-405).
    """
    idx = np.asarray(topk_idx)
    if idx.ndim != 2:
        raise ValueError("topk_idx must be [T, K]")
    num_local = num_experts - expert_begin if num_local is None else num_local
    flat = idx.reshape(-1).astype(np.int64)
    valid = (flat >= 0) & (flat < num_experts) & (flat >= expert_begin) & (flat < expert_begin + num_local)
    routes = np.nonzero(valid)[0]
    local = flat[routes] - expert_begin
    order = np.argsort(local, kind="stable")
    row_to_route = routes[order].astype(np.int32)
    counts = np.bincount(local, minlength=num_local).astype(np.int32)
    psum = np.cumsum(counts, dtype=np.int32)
    offsets = np.zeros(num_local + 1, dtype=np.int32)
    offsets[1:] = psum
    route_to_row = np.full(flat.shape, -1, dtype=np.int32)
    route_to_row[row_to_route] = np.arange(row_to_route.size, dtype=np.int32)
    return dict(
        counts=counts,
        psum=psum,
        offsets=offsets,
        route_to_row=route_to_row.reshape(idx.shape),
        row_to_route=row_to_route,
        num_rows=int(row_to_route.size),
    )


def layout_bruteforce(topk_idx, num_experts, expert_begin=0, num_local=None):
    """Scalar restatement in the reference's own loop order (small inputs only).

    Buckets exactly like ``expert_rows`` (tests/elastic/test_dispatch.py:538-548) and assigns
    rows through per-expert tails like ``_expand_reference`` (tests/clos/common.py:248-287).
    """
    idx = [[int(v) for v in row] for row in np.asarray(topk_idx).tolist()]
    num_local = num_experts - expert_begin if num_local is None else num_local
    topk = len(idx[0]) if idx else 0
    buckets = [[] for _ in range(num_local)]
    for token, row in enumerate(idx):
        for slot, selected in enumerate(row):
            if 0 <= selected < num_experts and expert_begin <= selected < expert_begin + num_local:
                buckets[selected - expert_begin].append(token * topk + slot)
    counts = [len(b) for b in buckets]
    offsets = [0]
    for c in counts:
        offsets.append(offsets[-1] + c)
    tails = offsets[:-1].copy()
    route_to_row = [[-1] * topk for _ in idx]
    row_to_route = [0] * offsets[-1]
    for token, row in enumerate(idx):
        for slot, selected in enumerate(row):
            local = selected - expert_begin
            if 0 <= selected < num_experts and 0 <= local < num_local:
                route_to_row[token][slot] = tails[local]
                row_to_route[tails[local]] = token * topk + slot
                tails[local] += 1
    return dict(
        counts=np.asarray(counts, dtype=np.int32),
        psum=np.asarray(offsets[1:], dtype=np.int32),
        offsets=np.asarray(offsets, dtype=np.int32),
        route_to_row=np.asarray(route_to_row, dtype=np.int32).reshape(len(idx), topk),
        row_to_route=np.asarray(row_to_route, dtype=np.int32),
        num_rows=offsets[-1],
    )


def expand_rows(x, row_to_route, topk):
    """Expand-permute payload: ``out[row] = x[token(row)]`` byte copy.

    Follows expected_payload (tests/elastic/test_dispatch.py:1391-1416) and the scatter in
    _expand_reference (tests/clos/common.py:276-279).  ``x`` is any [T, ...] array (payload bytes,
    scale rows).  Pure index gather: nothing to pin beyond ``layout``.
    """
    x = np.asarray(x)
    return x[np.asarray(row_to_route, dtype=np.int64) // topk]


def expand_weights(topk_weights, row_to_route):
    """``out_weights[row] = topk_weights[t, s]`` fp32 bit copy (tests/clos/common.py:279)."""
    return np.asarray(topk_weights, dtype=np.float32).reshape(-1)[np.asarray(row_to_route, dtype=np.int64)]
