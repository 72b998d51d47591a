"""The forward / backward recipe of a training step as the reference's README gives it (README.md:164-221): forward is
dispatch -> experts (which apply the received weights once) -> combine; backward is a cached dispatch of the output gradient
with the forward's handle, the experts' backward, and a combine of the input gradients that carries the weight gradients
on its return channel.  Experts here are one linear layer each; outputs and gradients are compared with a dense fp32
torch model of the same layer differentiated by autograd (tolerances of BF16 interfaces).  Run once with synchronous calls
(whose returned event has nothing left to wait for: the reference releases it before returning,
deep_ep/backends/mesh_clos/elastic.py:1001-1003, so the recipe's waits apply to the asynchronous form) and once with
asynchronous ones, waited for as in the recipe."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("asynchronous", [False, True])
@pytest.mark.parametrize("world,rank", [(1, 0), (2, 1)])
def test_training_step_matches_autograd(world, rank, asynchronous):
    import deepep_amd

    tokens, hidden, experts, topk = 96, 256, 8, 3
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(tokens, hidden, generator=gen).bfloat16()
    idx = torch.stack([torch.randperm(experts, generator=gen)[:topk] for _ in range(tokens)])
    idx[torch.rand(idx.shape, generator=gen) < 0.1] = -1
    topk_weights = torch.rand(tokens, topk, generator=gen)
    expert_w = torch.randn(experts, hidden, hidden, generator=gen) / hidden**0.5
    grad_out = torch.randn(tokens, hidden, generator=gen).bfloat16()
    per_rank = experts // world
    local = range(rank * per_rank, (rank + 1) * per_rank)

    # ---- dense fp32 model of this rank's share, differentiated by autograd --------------------------------------
    xr, wr = x.float().requires_grad_(True), topk_weights.clone().requires_grad_(True)
    out_ref = torch.zeros(tokens, hidden)
    for e in local:
        for s in range(topk):
            chosen = idx[:, s] == e
            out_ref = out_ref + chosen[:, None] * wr[:, s : s + 1] * (xr @ expert_w[e])
    (out_ref * grad_out.float()).sum().backward()

    # ---- the recipe ----------------------------------------------------------------------------------------------
    def wait(event):
        if asynchronous:
            event.current_stream_wait()
        else:
            assert event.event is None

    mode = dict(async_with_compute_stream=asynchronous)
    buffer = deepep_amd.ElasticBuffer(None, num_max_tokens_per_rank=tokens, hidden=hidden, num_topk=topk, rank=rank,
                                      world_size=world, explicitly_destroy=True)
    try:
        recv_x, _, recv_weights, handle, event = buffer.dispatch(
            x.cuda(), topk_idx=idx.cuda(), topk_weights=topk_weights.cuda(), num_experts=experts, do_expand=True, **mode)
        wait(event)
        counts = handle.num_recv_tokens_per_expert_list
        row_expert = torch.repeat_interleave(torch.arange(rank * per_rank, (rank + 1) * per_rank), torch.tensor(counts)).cuda()
        weights_of_rows = expert_w.cuda()[row_expert]  # [R, H, H]
        # local_experts_forward: the layer, then the received weight once; BF16 out, rows in received order
        hidden_out = torch.bmm(recv_x.float()[:, None, :], weights_of_rows)[:, 0, :]
        expert_out = (hidden_out * recv_weights[:, None]).bfloat16()
        out, _, event = buffer.combine(expert_out, handle, **mode)
        wait(event)
        # backward
        grad_expert_out, _, _, _, event = buffer.dispatch(grad_out.cuda(), handle=handle, **mode)
        wait(event)
        g = grad_expert_out.float()
        grad_recv_x = torch.bmm((g * recv_weights[:, None])[:, None, :], weights_of_rows.transpose(1, 2))[:, 0, :].bfloat16()
        grad_recv_weights = (g * hidden_out).sum(dim=1)
        grad_x, grad_topk_weights, event = buffer.combine(grad_recv_x, handle, topk_weights=grad_recv_weights.contiguous(), **mode)
        wait(event)
        torch.cuda.synchronize()
    finally:
        buffer.destroy()

    def close(got, want, what):
        got, want = got.float().cpu(), want.float()
        err = (got - want).norm() / want.norm().clamp_min(1e-12)
        assert err <= 1e-2, (what, float(err))

    close(out, out_ref.detach(), "out")
    close(grad_x, xr.grad, "grad_x")
    close(grad_topk_weights, wr.grad, "grad_topk_weights")
    served = (idx >= rank * per_rank) & (idx < (rank + 1) * per_rank)
    assert not grad_topk_weights.cpu()[~served].any()  # routes without a local row get no weight gradient
