"""Host-side routing preflight of the MegaMoE path, outside the timed path
(experiments/megamoe/python/deep_ep_experimental/megamoe/validation.py:10-22).

Unlike ``dispatch()``, MegaMoE accepts neither -1 masking nor repeated experts inside one token, so every token
contributes exactly top-k rows.  Messages carry ``rank=R: token=T`` like the reference's collective report.
"""

import math


def _token_fault(ids, probs, num_experts, num_topk):
    """What is wrong with one token's routing, or None."""
    if len(ids) != num_topk or len(probs) != num_topk:
        return f"routing width must equal top-k={num_topk}"
    for expert in ids:
        if type(expert) is not int or expert < 0 or expert >= num_experts:
            return f"expert IDs must be in [0,{num_experts}); -1 masking is unsupported"
    if len(frozenset(ids)) < num_topk:
        return "duplicate expert IDs are unsupported"
    if not all(math.isfinite(value) for value in probs):
        return "route weights must be finite"
    return None


def check_routing(indices, weights, num_experts, num_topk, rank=0):
    """Validates CPU lists taken from the actual input tensors; raises ValueError naming the first bad token."""
    if len(indices) != len(weights):
        raise ValueError(f"rank={rank}: routing IDs and weights have different BS")
    for token in range(len(indices)):
        fault = _token_fault(indices[token], weights[token], num_experts, num_topk)
        if fault is not None:
            raise ValueError(f"rank={rank}: token={token}: {fault}")
