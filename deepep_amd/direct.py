"""Single-rank ``expand`` / ``aggregate`` with the argument meaning of the reference's direct
backend (torch.classes.AscendDeepEP.BufferRuntime.expand / .aggregate,
csrc/direct/bindings/torch_classes.cpp:26-168, csrc/direct/runtime/buffer_runtime.h:133-150;
Python callers deep_ep/backends/direct/buffer.py:753,875).

``expand`` is the expert-major expand-permute with its forward map; ``aggregate`` is the weighted
(or unweighted) per-token fp32 reduce that the low-latency combine and the MegaMoE unpermute also use.
"""

from __future__ import annotations

from typing import Optional, Tuple, Union

import torch

from . import ops

_workspaces = {}


def _workspace(device: torch.device) -> ops.Workspace:
    key = (device.type, device.index)
    ws = _workspaces.get(key)
    if ws is None or ws.closed:
        ws = _workspaces[key] = ops.Workspace(1 << 20, device)
    return ws


def expand(
    x: Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]],
    topk_idx: torch.Tensor,
    topk_weights: Optional[torch.Tensor],
    num_experts: int,
    expert_alignment: int = 1,
    quantize_fp8: bool = False,
):
    """Return (expanded_x | (expanded_x, expanded_x_scales), expanded_topk_weights, expert_offsets[L+1],
    actual_expert_counts[L], recv_to_expanded_idx[N,K]).

    ``topk_idx`` holds local expert ids in [0, num_experts) or -1 (tests/clos/common.py:248-287).
    Reads the row count back to the host once, like the reference's expand host wrapper.
    """
    if expert_alignment != 1:
        raise NotImplementedError("expand supports expert_alignment=1")
    hidden, scales = x if isinstance(x, tuple) else (x, None)
    workspace = _workspace(hidden.device)
    plan = ops.layout(workspace, topk_idx, num_experts)
    _, rows = ops.layout_wait(workspace)
    if quantize_fp8:
        if scales is not None:
            raise ValueError("quantize_fp8 expects a BF16 tensor, not an (fp8, scales) pair")
        out, out_scales, out_w = ops.dispatch_quant_fp8(hidden, topk_weights, plan["route_to_row"], plan["row_to_route"], rows)
    else:
        out, out_scales, out_w = ops.dispatch_copy(hidden, scales, topk_weights, plan["route_to_row"], plan["row_to_route"], rows)
    payload = (out, out_scales) if out_scales is not None else out
    return payload, out_w, plan["offsets"], plan["counts"], plan["route_to_row"]


def aggregate(
    x: torch.Tensor,
    topk_weights: Optional[torch.Tensor],
    expanded_values: Optional[torch.Tensor],
    recv_to_expanded_idx: torch.Tensor,
):
    """Return (aggregated_x[N,H], aggregated_values[N,K] | None).

    acc = 0; for each slot with a row, in slot order: tmp = float(x[row]); tmp *= topk_weights[row]
    (when given); acc += tmp; result = bf16(acc)  (csrc/direct/kernels/aggregate/aggregate_impl.h:166-226).
    """
    return ops.combine(x, recv_to_expanded_idx, topk_weights, expanded_values)
