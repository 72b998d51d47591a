"""Host orchestration of ElasticBuffer on CPU with a fake native module backed by the oracle —
the counterpart of the reference's fake-native tests (tests/elastic/test_dispatch.py:592-945):
return tuples, handle fields, cached dispatch, version pinning and the error contract."""

import threading
from collections import Counter
from contextlib import nullcontext
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from deepep_amd import elastic, event
from oracle import combine as ocombine
from oracle import layout as olayout
from oracle import quant as oquant


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


class FakeNative:
    """Same call surface as deepep_amd.ops, computed by the CPU oracle."""

    def __init__(self, calls):
        self.calls = calls
        self.fail_next = None

    def layout_workspace_bytes(self, tokens, topk, local):
        return 65536

    def layout(self, ws, topk_idx, num_experts, expert_begin=0, num_local=None):
        self.calls["layout"] += 1
        out = olayout.layout(topk_idx.numpy(), num_experts, expert_begin, num_local)
        local = len(out["counts"])
        meta = torch.from_numpy(np.concatenate([out["counts"], out["psum"], out["offsets"], [out["num_rows"]]]).astype(np.int32))
        full = np.zeros(topk_idx.numel(), dtype=np.int32)
        full[: out["num_rows"]] = out["row_to_route"]
        self.last_layout = ([int(c) for c in out["counts"]], int(out["num_rows"]))
        return dict(counts=meta[:local], psum=meta[local : 2 * local], offsets=meta[2 * local : 3 * local + 1],
                    num_rows=meta[3 * local + 1 :], meta=meta, route_to_row=torch.from_numpy(out["route_to_row"]),
                    row_to_route=torch.from_numpy(full))

    def layout_wait(self, ws, num_local=None, timeout_s=100.0):
        counts, rows = self.last_layout
        return (counts if num_local is not None else None), rows

    def dispatch_copy(self, x, scales, w, route_to_row, row_to_route, rows, capacity_rows=None):
        if self.fail_next:
            raise RuntimeError(self.fail_next)
        self.calls["dispatch_copy"] += 1
        # rows=None: R not known to the caller yet; outputs hold T*K rows (or more), the tail is left as filler
        pad = 0 if rows is not None else max(route_to_row.numel(), capacity_rows or 0) - self.last_layout[1]
        self.calls["dispatch_at_capacity"] += rows is None
        rows = self.last_layout[1] if rows is None else rows
        route = row_to_route[:rows].long()
        token = route // route_to_row.shape[1]

        def padded(t):
            return None if t is None else torch.cat([t, torch.full((pad,) + t.shape[1:], 77).to(t.dtype)])

        out = x.view(torch.uint8 if x.element_size() == 1 else torch.int16)[token]
        return (padded(out).view(x.dtype), padded(None if scales is None else scales[token]),
                padded(None if w is None else w.reshape(-1)[route]))

    SMALL_BATCH_ROUTES = 2048

    def layout_dispatch_small(self, ws, topk_idx, x, scales, w, num_experts, expert_begin=0, num_local=None, quantize=False,
                              capacity_rows=None):
        """One launch for both in the library; here the two oracle steps in a row."""
        self.calls["layout_dispatch_small"] += 1
        plan = self.layout(ws, topk_idx, num_experts, expert_begin, num_local)
        if self.fail_next:
            raise RuntimeError(self.fail_next)
        if quantize:
            moved = self.dispatch_quant_fp8(x, w, plan["route_to_row"], plan["row_to_route"], None)
        else:
            moved = self.dispatch_copy(x, scales, w, plan["route_to_row"], plan["row_to_route"], None, capacity_rows=capacity_rows)
        return (plan, *moved)

    def dispatch_quant_fp8(self, x, w, route_to_row, row_to_route, rows):
        self.calls["dispatch_quant_fp8"] += 1
        q, s = oquant.cast_to_fp8_torch(x)
        return self.dispatch_copy(q, s, w, route_to_row, row_to_route, rows)

    def combine(self, y, route_to_row, row_weights=None, return_values=None):
        self.calls["combine"] += 1
        if y.dtype == torch.float16:
            out = ocombine.combine_fp16(y.numpy(), route_to_row.numpy(), None if row_weights is None else row_weights.numpy())
            return torch.from_numpy(out), None
        out = ocombine.combine(_bits(y), route_to_row.numpy(), None if row_weights is None else row_weights.numpy())
        returned = None
        if return_values is not None:
            returned = torch.from_numpy(ocombine.return_weights(return_values.numpy(), route_to_row.numpy()))
        return torch.from_numpy(out.view(np.int16)).view(torch.bfloat16), returned


@pytest.fixture
def host(monkeypatch):
    calls = Counter()
    stream = SimpleNamespace(synchronize=lambda: calls.update(["sync"]))
    gpu = SimpleNamespace(
        stream=lambda _: nullcontext(),
        current_device=lambda: 0,
        current_stream=lambda _: stream,
        Event=lambda: SimpleNamespace(record=lambda _: None, wait=lambda _: calls.update(["event_wait"])),
    )
    monkeypatch.setattr(event, "gpu_api", lambda: gpu)
    monkeypatch.setattr(elastic, "gpu_api", lambda: gpu)

    def make(world=1, rank=0, hidden=0, topk=0, bound=0, fp8=False, num_bytes=1 << 30):
        native = FakeNative(calls)
        buffer = elastic.ElasticBuffer.__new__(elastic.ElasticBuffer)
        buffer.hidden, buffer.num_topk, buffer.num_max_tokens_per_rank = hidden, topk, bound
        buffer.use_fp8_dispatch = fp8
        buffer._handle_token = object()
        buffer._runtime = SimpleNamespace(
            native=native, device=0, torch_device=torch.device("cpu"), rank=rank, world_size=world, combine_only=False,
            capacity=num_bytes, notify_lock=threading.RLock(), notify_failed=False, notify_inflight=None,
            workspace=object(), stream=stream, closed=False, ensure_alive=lambda: None, close=lambda: None,
        )
        return buffer, native

    return make, calls


def _inputs(tokens=6, hidden=128, experts=8, topk=2, seed=0):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(tokens, hidden, generator=gen).bfloat16()
    idx = torch.stack([torch.randperm(experts, generator=gen)[:topk] for _ in range(tokens)]).to(torch.int64)
    w = torch.rand(tokens, topk, generator=gen)
    return x, idx, w


def test_fresh_dispatch_combine_and_cached_dispatch(host):
    make, calls = host
    buffer, _ = make()
    x, idx, w = _inputs()
    idx[1, 0] = -1
    recv, none, recv_w, handle, ev = buffer.dispatch(x, topk_idx=idx, topk_weights=w, num_experts=8)
    want = olayout.layout(idx.numpy(), 8)
    assert none is None and isinstance(ev, event.EventOverlap)
    assert handle.num_expanded_tokens == want["num_rows"] == recv.shape[0]
    # every expert is local: the payload was queued before the host knew R, into outputs of T*K rows, then narrowed
    assert calls["dispatch_at_capacity"] == 1 and want["num_rows"] < idx.numel()
    assert recv.untyped_storage().nbytes() == idx.numel() * 128 * 2 and recv.is_contiguous()
    assert handle.num_recv_tokens_per_expert_list == want["counts"].tolist()
    assert handle.psum_num_recv_tokens_per_expert.tolist() == want["psum"].tolist()
    assert handle.num_unaligned_recv_tokens_per_expert.tolist() == want["counts"].tolist()
    assert handle.weight_return_meta.tolist() == want["row_to_route"].tolist()
    assert (handle.do_expand, handle.expert_alignment, handle.metadata_version, handle.is_low_latency) == (True, 1, 7, False)
    assert (handle.num_tokens, handle.num_topk, handle.hidden, handle.rank, handle.world_size) == (6, 2, 128, 0, 1)
    assert handle.num_recv_tokens is None and handle.num_sms == handle.num_compute_units == 32
    assert handle.topk_idx.data_ptr() != idx.data_ptr()  # do_handle_copy=True clones the routing
    np.testing.assert_array_equal(_bits(recv), olayout.expand_rows(_bits(x), want["row_to_route"], 2))
    np.testing.assert_array_equal(recv_w.numpy(), olayout.expand_weights(w.numpy(), want["row_to_route"]))
    # combine: unweighted sum + weight return channel [T,K]
    out, out_w, ev2 = buffer.combine(recv, handle, topk_weights=recv_w)
    assert out.shape == x.shape and out_w.shape == (6, 2)
    np.testing.assert_array_equal(out_w.numpy(), np.where(idx.numpy() >= 0, w.numpy(), 0))
    out_only, none_w, _ = buffer.combine(recv, handle)
    assert none_w is None and torch.equal(out_only, out)
    # cached dispatch: same handle object, no new layout
    layouts = calls["layout"]
    recv2, _, _, again, _ = buffer.dispatch(x * 2, handle=handle)
    assert again is handle and calls["layout"] == layouts
    assert torch.equal(recv2, recv * 2)


def test_rank_share_selects_local_experts(host):
    make, calls = host
    buffer, _ = make(world=4, rank=2)
    x, idx, w = _inputs(tokens=16, experts=8, topk=3)
    recv, _, recv_w, handle, _ = buffer.dispatch(x, topk_idx=idx, topk_weights=w, num_experts=8)
    want = olayout.layout(idx.numpy(), 8, 4, 2)
    assert handle.num_recv_tokens_per_expert_list == want["counts"].tolist()
    assert handle.weight_return_meta.tolist() == want["row_to_route"].tolist()
    assert recv.shape[0] == want["num_rows"]
    # a quarter of the experts is local: outputs are sized after the host has read R
    assert calls["dispatch_at_capacity"] == 0 and recv.untyped_storage().nbytes() == want["num_rows"] * 128 * 2


def test_fp8_tuple_and_fused_quant(host):
    make, calls = host
    x, idx, w = _inputs(hidden=256)
    q, s = oquant.cast_to_fp8_torch(x)
    buffer, _ = make()
    (rq, rs), _, _, handle, _ = buffer.dispatch((q, s), topk_idx=idx, num_experts=8)
    assert rq.dtype == torch.float8_e4m3fn and rs.shape == (handle.num_expanded_tokens, 2) and handle.num_sms == 64
    fused, _ = make(fp8=True)
    (fq, fs), _, _, _, _ = fused.dispatch(x, topk_idx=idx, num_experts=8)
    assert torch.equal(fq.view(torch.uint8), rq.view(torch.uint8)) and torch.equal(fs, rs)
    assert calls["dispatch_quant_fp8"] == 1
    with pytest.raises(ValueError, match="scales"):
        buffer.dispatch((q, s[:, :1].contiguous()), topk_idx=idx, num_experts=8)


def test_error_contract_and_no_poisoning(host):
    make, _ = host
    buffer, native = make()
    x, idx, w = _inputs()
    with pytest.raises(NotImplementedError, match="Fresh notify"):
        buffer.dispatch(x, topk_idx=idx, num_experts=8, do_cpu_sync=False)
    with pytest.raises(TypeError, match="do_cpu_sync"):
        buffer.dispatch(x, topk_idx=idx, num_experts=8, do_cpu_sync=1)
    with pytest.raises(NotImplementedError, match="expanded"):
        buffer.dispatch(x, topk_idx=idx, num_experts=8, do_expand=False)
    with pytest.raises(NotImplementedError, match="expert_alignment"):
        buffer.dispatch(x, topk_idx=idx, num_experts=8, expert_alignment=128)
    with pytest.raises(ValueError, match="topk_idx"):
        buffer.dispatch(x, topk_idx=idx.int(), num_experts=8)
    for width in (15, 17, 7169, 7296):
        with pytest.raises(ValueError, match="hidden"):
            buffer.dispatch(torch.zeros(6, width, dtype=torch.bfloat16), topk_idx=idx, num_experts=8)
    for width in (16, 48, 7168):
        buffer.dispatch(torch.zeros(6, width, dtype=torch.bfloat16), topk_idx=idx, num_experts=8)
    with torch.inference_mode():
        frozen = idx.clone()
    with pytest.raises(ValueError, match="do_handle_copy=True"):
        buffer.dispatch(x, topk_idx=frozen, num_experts=8, do_handle_copy=False)
    configured, _ = make(hidden=256)
    with pytest.raises(ValueError, match="buffer configuration"):
        configured.dispatch(x, topk_idx=idx, num_experts=8)
    assert buffer._runtime.notify_failed is False  # validation failures do not poison the runtime
    recv, _, _, handle, _ = buffer.dispatch(x, topk_idx=idx, num_experts=8)
    with pytest.raises(ValueError, match="omit topk_idx"):
        buffer.dispatch(x, topk_idx=idx, handle=handle)
    with pytest.raises(ValueError, match="original hidden"):
        buffer.dispatch(torch.zeros(6, 64, dtype=torch.bfloat16), handle=handle)
    with pytest.raises(ValueError, match="original token count"):
        buffer.dispatch(torch.zeros(5, 128, dtype=torch.bfloat16), handle=handle)
    with pytest.raises(ValueError, match="matching the handle"):
        buffer.combine(recv[:-1].contiguous(), handle)
    with pytest.raises(ValueError, match="matching the handle"):
        buffer.combine(torch.zeros(recv.shape[0], 64, dtype=torch.bfloat16), handle)
    other, _ = make()
    with pytest.raises(ValueError, match="this buffer"):
        other.combine(recv, handle)
    with pytest.raises(NotImplementedError, match="bias"):
        buffer.combine(recv, handle, bias=recv)
    handle.route_to_row.add_(0)  # in-place edit bumps the version counter
    with pytest.raises(ValueError, match="Cached routing was modified"):
        buffer.combine(recv, handle)
    with pytest.raises(ValueError, match="Cached routing was modified"):
        buffer.dispatch(x, handle=handle)
    assert buffer._runtime.notify_failed is False
    # a launch failure does poison the runtime
    native.fail_next = "boom"
    with pytest.raises(RuntimeError, match="boom"):
        buffer.dispatch(x, topk_idx=idx, num_experts=8)
    assert buffer._runtime.notify_failed is True
    with pytest.raises(RuntimeError, match="previous communication launch failed"):
        buffer.dispatch(x, topk_idx=idx, num_experts=8)


def test_keyword_aliases(host):
    make, _ = host
    buffer, _ = make()
    x, idx, w = _inputs()
    _, _, _, handle, _ = buffer.dispatch(x, topk_idx=idx, num_experts=8, num_compute_units=32)
    with pytest.raises(TypeError, match="conflicting"):
        buffer.dispatch(x, topk_idx=idx, num_experts=8, num_compute_units=32, num_sms=0)
    with pytest.raises(ValueError, match="num_compute_units"):
        buffer.dispatch(x, topk_idx=idx, num_experts=8, num_sms=7)
    handle.num_sms = 5
    assert handle.num_compute_units == 5


def test_constructor_gates():
    with pytest.raises(NotImplementedError, match="explicitly_destroy"):
        elastic.ElasticBuffer(num_bytes=1 << 21)
    with pytest.raises(NotImplementedError, match="default options"):
        elastic.ElasticBuffer(num_bytes=1 << 21, deterministic=True, explicitly_destroy=True)
    with pytest.raises(ValueError, match="hidden"):
        elastic.ElasticBuffer(num_bytes=1 << 21, hidden=100, explicitly_destroy=True)
    with pytest.raises(ValueError, match="world_size|Runtime supports"):
        elastic.ElasticBuffer(num_bytes=1 << 21, explicitly_destroy=True, rank=0, world_size=3)
    with pytest.raises(NotImplementedError, match="Pass num_bytes"):
        elastic.ElasticBuffer(explicitly_destroy=True)
    assert elastic.ElasticBuffer.get_buffer_size_hint(None, 4096, 7168, 8) >= 2 << 20


def test_low_latency_path_selection_and_contract(host):
    """Small batches on EP16+ with route weights and default options take the low-latency path
    (deep_ep/backends/mesh_clos/elastic.py:710-746): capacity layout, weights kept in the handle, FP16 accepted."""
    from oracle import cases

    make, calls = host
    world, rank, per_rank, hidden, experts, topk = 16, 3, 4, 64, 32, 3
    routes = cases.ll_routes(world, per_rank, topk, experts, seed=11)
    idx = torch.tensor([row for source in routes for row in source])
    sources, toks = np.repeat(np.arange(world), per_rank), np.tile(np.arange(per_rank), world)
    w = ((torch.arange(topk) + 1) / 32).repeat(world * per_rank, 1).contiguous()
    entries = cases.ll_expert_entries(routes, experts, world, rank)
    rows = sum(len(v) for v in entries)
    capacity_rows = world * per_rank * min(topk, experts // world)
    for dtype in (torch.bfloat16, torch.float16):
        buffer, _ = make(world=world, rank=rank, num_bytes=8 << 30)
        x = torch.from_numpy(cases.ll_payload(sources, toks, hidden)).to(dtype)
        recv, none, recv_w, handle, ev = buffer.dispatch(x, topk_idx=idx, topk_weights=w, num_experts=experts)
        assert none is None and recv_w is None and handle.is_low_latency and calls["dispatch_at_capacity"] >= 1
        assert recv.shape == (capacity_rows, hidden) and recv.dtype == dtype
        assert handle.num_expanded_tokens == capacity_rows and handle.num_recv_tokens == world * per_rank
        assert handle.num_recv_tokens_per_expert_list == [] and handle.psum_num_recv_tokens_per_expert is None
        assert handle.num_unaligned_recv_tokens_per_expert is None and handle.expert_recv_counts is None
        assert int(handle.send_counts[-1]) == rows and handle.send_counts.shape == (experts,)
        start = 0
        for block in entries:  # expert-major blocks, (source, token) order inside (tests/elastic/test_ep_low_latency.py:518-531)
            got = recv[start : start + len(block)].float()
            ids = [(int(r[0]) * 16 + int(r[1]), int(r[2]) * 16 + int(r[3])) for r in got]
            assert ids == block
            start += len(block)
        # combine: weights from the handle, output in the experts' dtype, (out, None, event)
        y = recv.clone()
        y[rows:] = 0  # the capacity tail is not input: make it harmless for the CPU stand-in
        out, out_w, _ = buffer.combine(y, handle)
        assert out_w is None and out.dtype == dtype and out.shape == x.shape
        local = experts // world
        expected = torch.zeros(x.shape)
        for t in range(idx.shape[0]):
            for s in range(topk):
                if rank * local <= int(idx[t, s]) < (rank + 1) * local:
                    expected[t] += x[t].float() * ((s + 1) / 32)
        assert torch.equal(out, expected.to(dtype))
        with pytest.raises(NotImplementedError, match="weights from the handle"):
            buffer.combine(y, handle, topk_weights=torch.ones(capacity_rows))
        with pytest.raises(NotImplementedError, match="default scheduling"):
            buffer.combine(y, handle, num_sms=64)
        with pytest.raises(ValueError, match="matching its handle"):
            buffer.combine(y[:-1].contiguous(), handle)
        with pytest.raises(NotImplementedError, match="Cached dispatch is not supported for LL"):
            buffer.dispatch(x, handle=handle)
    # exactly 8 GiB or an error, never a silent switch to the other path (docs/elastic.md:28)
    small, _ = make(world=world, rank=rank)
    with pytest.raises(ValueError, match="exactly 8 GiB"):
        small.dispatch(x.bfloat16(), topk_idx=idx, topk_weights=w, num_experts=experts)
    # without route weights, with more than 256 tokens per rank, or below EP16 the call is a high-throughput one
    recv, _, recv_w, handle, _ = small.dispatch(x.bfloat16(), topk_idx=idx, num_experts=experts)
    assert not handle.is_low_latency and recv.shape[0] == rows
    ep8, _ = make(world=8, rank=1, num_bytes=8 << 30)
    idx8 = idx[: 8 * per_rank].contiguous()
    _, _, _, handle, _ = ep8.dispatch(x[: 8 * per_rank].bfloat16().contiguous(), topk_idx=idx8, topk_weights=w[: 8 * per_rank].contiguous(), num_experts=experts)
    assert not handle.is_low_latency
