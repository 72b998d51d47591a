"""Host-side routing preflight, outside the timed path
(experiments/megamoe/python/deep_ep_experimental/megamoe/validation.py:10-22)."""

import math


def check_routing(indices, weights, num_experts, num_topk, rank=0):
    """Validate CPU lists taken from the actual input tensors.

    Unlike dispatch(), MegaMoE accepts neither -1 masking nor repeated experts inside one token, so
    every token contributes exactly top-k rows.  Messages carry ``rank=R: token=T`` like the
    reference's collective report."""
    if len(indices) != len(weights):
        raise ValueError(f"rank={rank}: routing IDs and weights have different BS")
    for token, (ids, probs) in enumerate(zip(indices, weights)):
        where = f"rank={rank}: token={token}"
        if len(ids) != num_topk or len(probs) != num_topk:
            raise ValueError(f"{where}: routing width must equal top-k={num_topk}")
        if any(type(expert) is not int or not 0 <= expert < num_experts for expert in ids):
            raise ValueError(f"{where}: expert IDs must be in [0,{num_experts}); -1 masking is unsupported")
        if len(set(ids)) != num_topk:
            raise ValueError(f"{where}: duplicate expert IDs are unsupported")
        if any(not math.isfinite(value) for value in probs):
            raise ValueError(f"{where}: route weights must be finite")
