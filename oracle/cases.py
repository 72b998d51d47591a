"""Deterministic inputs: the reference's fixture formulas and the benchmark configurations.

No arithmetic of the hot path lives here; these are input recipes restated from the reference's
tests so that fixtures can be regenerated without the reference checkout.
"""

from __future__ import annotations

import numpy as np


def matrix_routes(world_size, experts, topk, tokens_per_rank):
    """Route table of make_matrix_case (tests/utils/cases.py:150-157):
    expert = (rank*11 + token*7 + slot*13) % E, masked (-1) when (rank*5 + token*3 + slot + 1) % 97 == 0."""
    routes = []
    for rank in range(world_size):
        rank_routes = []
        for token in range(tokens_per_rank[rank]):
            row = []
            for slot in range(topk):
                expert = (rank * 11 + token * 7 + slot * 13) % experts
                if (rank * 5 + token * 3 + slot + 1) % 97 == 0:
                    expert = -1
                row.append(expert)
            rank_routes.append(tuple(row))
        routes.append(tuple(rank_routes))
    return tuple(routes)


def dispatch_payload_values(source, tokens, generation, width):
    """BF16/FP8-exact payload of tests/elastic/test_dispatch.py:1372-1382 as float32, plus scales."""
    rows = np.arange(tokens, dtype=np.int64)[:, None]
    cols = np.arange(width, dtype=np.int64)[None, :]
    hidden = (((source * 13 + rows * 7 + cols * 3 + generation * 11) % 127) - 63).astype(np.float32) / 16
    scales = (((source + rows + np.arange(width // 128)[None, :] + generation) % 7) + 1).astype(np.float32) / 8
    return hidden, scales


def dispatch_weights(source, tokens, topk, generation):
    """tests/elastic/test_dispatch.py:1385-1388."""
    ids = np.arange(tokens * topk, dtype=np.int64).reshape(tokens, topk)
    return (((ids + source * 3 + generation) % 31) + 1).astype(np.float32) / 32


def combine_payload_values(source, tokens, generation, hidden):
    """Bounded-integer BF16 payload of tests/elastic/test_combine.py:496-501 as float32."""
    t = np.arange(tokens, dtype=np.int64)[:, None]
    c = np.arange(hidden, dtype=np.int64)[None, :]
    return (((t + c + source + generation) % 7) - 3).astype(np.float32)


def combine_expected_values(routes, experts, source, generation, hidden):
    """tests/elastic/test_combine.py:504-515: base*count + sum((e%3-1)+(s%3-1)) over valid slots."""
    base = combine_payload_values(source, len(routes), generation, hidden)
    selected = np.asarray(routes, dtype=np.int64)
    valid = (selected >= 0) & (selected < experts)
    slots = np.arange(selected.shape[1])[None, :]
    count = valid.sum(axis=1, keepdims=True)
    bias = (((selected % 3) - 1 + (slots % 3) - 1) * valid).sum(axis=1, keepdims=True)
    return (base * count + bias).astype(np.float32)


# ----------------------------------------------------------------------------------------------
# Benchmark configurations (seeded torch CPU generator, then handed to the device).
# ----------------------------------------------------------------------------------------------

CONFIGS = {
    "C1": dict(tokens=128, hidden=1024, experts=16, topk=4, routing="uniform"),
    "C2": dict(tokens=128, hidden=7168, experts=256, topk=8, routing="uniform"),
    "C3": dict(tokens=4096, hidden=7168, experts=256, topk=8, routing="zipf"),
    "C4": dict(tokens=64 * 256, hidden=7168, experts=384, topk=8, routing="uniform", expert_begin=0, num_local=6),
}


def ll_routes(world_size, tokens, topk, experts, seed):
    """Routes of the low-latency system test (make_routes, tests/elastic/test_ep_low_latency.py:397-407): per
    source rank and token, `topk` distinct experts drawn with random.Random(seed).sample."""
    import random

    rng = random.Random(seed)
    return [[rng.sample(range(experts), topk) for _ in range(tokens)] for _ in range(world_size)]


def ll_payload(sources, tokens, hidden):
    """Payload rows of the same test (payload, :421-430): ((src*3 + tok*5 + col) % 17) - 8, with the first four
    columns replaced by src//16, src%16, tok//16, tok%16 (small integers, exact in BF16, FP16 and FP8)."""
    sources, tokens = np.asarray(sources, dtype=np.int64), np.asarray(tokens, dtype=np.int64)
    values = ((sources[:, None] * 3 + tokens[:, None] * 5 + np.arange(hidden)[None, :]) % 17 - 8).astype(np.float32)
    values[:, 0], values[:, 1] = sources // 16, sources % 16
    values[:, 2], values[:, 3] = tokens // 16, tokens % 16
    return values


def ll_fp8_scale_bits(sources, tokens, hidden, packed_e8m0):
    """Scale words of the same test (fp8_scales, :433-446), as int32 bit patterns [n, ceil(H/128)]: 0x7F7F7F7F
    (four packed E8M0 ones) or FP32 values with bits 0x3F000001 + src*65536 + tok*128 + group."""
    groups = (hidden + 127) // 128
    sources, tokens = np.asarray(sources, dtype=np.int64), np.asarray(tokens, dtype=np.int64)
    if packed_e8m0:
        return np.full((len(sources), groups), 0x7F7F7F7F, dtype=np.int32)
    return (0x3F000001 + sources[:, None] * 65536 + tokens[:, None] * 128 + np.arange(groups)[None, :]).astype(np.int32)


def ll_expert_entries(routes, experts, world_size, rank):
    """(source, token) pairs each local expert of `rank` receives, in source-major order (expert_entries, :410-418)."""
    local = experts // world_size
    entries = [[] for _ in range(local)]
    for source, rows in enumerate(routes):
        for token, selected in enumerate(rows):
            for expert in selected:
                if rank * local <= expert < (rank + 1) * local:
                    entries[expert - rank * local].append((source, token))
    return entries


def ll_expert_map(values_f32, expert):
    """What the test's stand-in expert computes before rounding to its output dtype (prepare_experts, :466-479):
    x * ((e % 4 + 1) / 4) + (e % 3 - 1) / 8, in fp32."""
    return (values_f32 * np.float32((expert % 4 + 1) / 4) + np.float32((expert % 3 - 1) / 8)).astype(np.float32)


def make_inputs(name, seed=0, tokens=None, hidden=None):
    """x ~ N(0,1) BF16 [T,H]; distinct top-k ids (uniform, or Zipf(1.2) popularity sampled without
    replacement); weights = softmax of N(0,1) logits, fp32.  Returns torch CPU tensors."""
    import torch

    cfg = dict(CONFIGS[name])
    if tokens is not None:
        cfg["tokens"] = tokens
    if hidden is not None:
        cfg["hidden"] = hidden
    gen = torch.Generator().manual_seed(seed)
    t, h, e, k = cfg["tokens"], cfg["hidden"], cfg["experts"], cfg["topk"]
    x = torch.randn(t, h, generator=gen).bfloat16()
    if cfg["routing"] == "zipf":
        p = (torch.arange(e, dtype=torch.float64) + 1) ** -1.2
    else:
        p = torch.ones(e, dtype=torch.float64)
    topk_idx = torch.multinomial((p / p.sum()).expand(t, e), k, replacement=False, generator=gen).to(torch.int64)
    topk_weights = torch.softmax(torch.randn(t, k, generator=gen), dim=-1).float()
    cfg.setdefault("expert_begin", 0)
    cfg.setdefault("num_local", e)
    return x, topk_idx, topk_weights, cfg
