"""The reference CPU path (torch CPU, all host threads) used as the timed ``cpu_baseline``.

Same arithmetic as the NumPy oracle, written with the torch CPU routines the reference's own CPU
path uses (tests/clos/common.py:110-118,248-309, deep_ep/utils/math.py:45-61): bincount + stable
argsort layout, index_select expand, per_token_cast_to_fp8, slot-ordered fp32 combine.
Checked against the NumPy oracle in tests/test_oracle_baseline.py.
"""

from __future__ import annotations

import torch


def layout(topk_idx, num_experts, expert_begin=0, num_local=None):
    num_local = num_experts - expert_begin if num_local is None else num_local
    flat = topk_idx.reshape(-1)
    local = flat - expert_begin
    valid = (flat >= 0) & (flat < num_experts) & (local >= 0) & (local < num_local)
    routes = valid.nonzero(as_tuple=True)[0]
    keys = local[routes]
    order = torch.argsort(keys, stable=True)
    row_to_route = routes[order].to(torch.int32)
    counts = torch.bincount(keys, minlength=num_local).to(torch.int32)
    route_to_row = torch.full_like(flat, -1, dtype=torch.int32)
    route_to_row[row_to_route.long()] = torch.arange(row_to_route.numel(), dtype=torch.int32)
    return counts, counts.cumsum(0, dtype=torch.int32), route_to_row.view(topk_idx.shape), row_to_route


def cast_to_fp8(x):
    tokens, hidden = x.shape
    view = x.view(tokens, -1, 128)
    amax = view.abs().float().amax(dim=2).view(tokens, -1).clamp(1e-4)
    q = (view * (448.0 / amax.unsqueeze(2))).to(torch.float8_e4m3fn)
    return q.view(tokens, hidden), (amax / 448.0).view(tokens, -1)


def dispatch_fp8(x, topk_weights, row_to_route, topk):
    q, s = cast_to_fp8(x)
    token = (row_to_route // topk).long()
    out_w = None if topk_weights is None else topk_weights.reshape(-1).index_select(0, row_to_route.long())
    return q.view(torch.uint8).index_select(0, token).view(torch.float8_e4m3fn), s.index_select(0, token), out_w


def dispatch_bf16(x, topk_weights, row_to_route, topk):
    token = (row_to_route // topk).long()
    out_w = None if topk_weights is None else topk_weights.reshape(-1).index_select(0, row_to_route.long())
    return x.index_select(0, token), out_w


def combine(y, route_to_row, row_weights=None):
    tokens, topk = route_to_row.shape
    acc = torch.zeros((tokens, y.shape[1]), dtype=torch.float32)
    for slot in range(topk):
        rows = route_to_row[:, slot].long()
        valid = rows >= 0
        safe = rows.clamp(min=0)
        tmp = y.index_select(0, safe).float()
        if row_weights is not None:
            tmp = tmp * row_weights.index_select(0, safe)[:, None]
        acc = torch.where(valid[:, None], acc + tmp, acc)
    return acc.bfloat16()


def megamoe_expert_forward(x, w1, w2):
    """One expert of the W4A8 FFN the way the reference's CPU oracle evaluates it (experiments/megamoe/python/
    deep_ep_experimental/megamoe/reference.py:84-89) on dense fp32 operands, with torch.matmul for the two
    contractions: first = bf16(x @ w1^T); act = bf16(silu(gate) * up); qa = dequant(mx_quant(act));
    out = bf16(qa @ w2^T).  x [m,H], w1 [2I,H] (gate rows then up rows), w2 [H,I]; returns BF16 [m,H].
    The roundings, SwiGLU and the MXFP8 step are the NumPy oracle's."""
    from . import megamoe

    first = torch.matmul(x, w1.T).bfloat16().float()
    act = megamoe.swiglu(first.numpy())
    qa = torch.from_numpy(megamoe.mx_dequantize(*megamoe.mx_quantize(act)))
    return torch.matmul(qa, w2.T).bfloat16()
