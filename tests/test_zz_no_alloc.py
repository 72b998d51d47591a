"""dpep_layout_static, the layout entry point that allocates nothing (its scratch is a device array inside the
library), called through the C-ABI and checked against dpep_layout and against the CPU oracle on the same inputs: two
calls in a row on the one GPU's shared scratch, the second with a smaller input, every output compared bit for bit.
That it allocates nothing is checked twice: the device's free memory does not move across calls whose outputs exist
already, and the call can be captured into a HIP graph (where an allocation is an error) and replayed on new routes."""

import ctypes

import numpy as np
import pytest
import torch

from deepep_amd import _lib, ops
from oracle import layout as olayout

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _outputs(tokens, topk, local, dev):
    return dict(
        counts=torch.full((local,), -5, dtype=torch.int32, device=dev),
        psum=torch.full((local,), -5, dtype=torch.int32, device=dev),
        offsets=torch.full((local + 1,), -5, dtype=torch.int32, device=dev),
        route_to_row=torch.full((tokens, topk), -5, dtype=torch.int32, device=dev),
        row_to_route=torch.full((tokens * topk,), -5, dtype=torch.int32, device=dev),
        num_rows=torch.full((1,), -5, dtype=torch.int32, device=dev),
    )


def _layout_static(lib, idx, experts, begin, local, out=None):
    tokens, topk = idx.shape
    dev = idx.device
    if out is None:
        out = _outputs(tokens, topk, local, dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    status = lib.dpep_layout_static(_ptr(idx), tokens, topk, experts, begin, local, _ptr(out["counts"]), _ptr(out["psum"]),
                                    _ptr(out["offsets"]), _ptr(out["route_to_row"]), _ptr(out["row_to_route"]),
                                    _ptr(out["num_rows"]), stream)
    _lib.check(status, "layout_static")
    return out


def test_layout_static_matches_layout_on_two_calls_in_a_row():
    lib = _lib.load()
    torch.cuda.set_device(0)
    workspace = ops.Workspace(1 << 20)
    try:
        gen = torch.Generator().manual_seed(7)
        # (tokens, top-k, experts, first local, local): a large input, then a smaller one over the same scratch
        for tokens, topk, experts, begin, local in ((4096, 8, 256, 0, 256), (300, 6, 48, 8, 24), (0, 4, 16, 0, 16)):
            idx = torch.randint(-1, experts + 1, (tokens, topk), generator=gen).cuda()  # -1 and == E: no row
            got = _layout_static(lib, idx, experts, begin, local)
            want = ops.layout(workspace, idx, experts, begin, local)
            torch.cuda.synchronize()
            rows = int(want["num_rows"].item())
            assert int(got["num_rows"].item()) == rows
            for name in ("counts", "psum", "offsets", "route_to_row"):
                np.testing.assert_array_equal(got[name].cpu().numpy(), want[name].cpu().numpy(), err_msg=name)
            np.testing.assert_array_equal(got["row_to_route"][:rows].cpu().numpy(), want["row_to_route"][:rows].cpu().numpy())
            assert tokens == 0 or rows > 0
            _assert_equals_oracle(got, idx, experts, begin, local)
    finally:
        workspace.destroy()


def _assert_equals_oracle(got, idx, experts, begin, local):
    oracle = olayout.layout(idx.cpu().numpy(), experts, begin, local)
    rows = oracle["num_rows"]
    assert int(got["num_rows"].item()) == rows
    for name in ("counts", "psum", "offsets", "route_to_row"):
        np.testing.assert_array_equal(got[name].cpu().numpy(), oracle[name], err_msg=name)
    np.testing.assert_array_equal(got["row_to_route"][:rows].cpu().numpy(), oracle["row_to_route"])


def test_layout_static_allocates_nothing():
    """No workspace exists in this test.  (1) With the outputs allocated beforehand the device's free memory is the same
    before and after static calls, the process's first included when this test runs alone.  (2) The call is captured
    into a HIP graph, where any allocation by the library would fail the capture, and replayed three times on new routes
    in the same buffers; every replay is compared with the CPU oracle."""
    lib = _lib.load()
    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    tokens, topk, experts, begin, local = 1024, 8, 64, 16, 32
    gen = torch.Generator().manual_seed(11)
    idx = torch.randint(-1, experts + 1, (tokens, topk), generator=gen).to(dev)
    out = _outputs(tokens, topk, local, dev)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    for _ in range(3):
        _layout_static(lib, idx, experts, begin, local, out)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    _assert_equals_oracle(out, idx, experts, begin, local)

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        _layout_static(lib, idx, experts, begin, local, out)
    for replay in range(3):
        idx.copy_(torch.randint(-1, experts + 1, (tokens, topk), generator=gen))
        for tensor in out.values():
            tensor.fill_(-5)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _assert_equals_oracle(out, idx, experts, begin, local)


def test_layout_static_rejects_what_it_cannot_hold():
    lib = _lib.load()
    torch.cuda.set_device(0)
    idx = torch.zeros((4, 2), dtype=torch.int64, device="cuda")
    small = torch.zeros((2048,), dtype=torch.int32, device="cuda")
    args = (_ptr(small),) * 6 + (None,)
    assert lib.dpep_layout_static(_ptr(idx), 4, 2, 2048, 0, 1025, *args) == -1
    assert "at most 1024 local experts" in lib.dpep_last_error().decode()
    assert lib.dpep_layout_static(_ptr(idx), 4, 33, 16, 0, 16, *args) == -1
    assert lib.dpep_layout_static(_ptr(idx), 1 << 30, 8, 16, 0, 16, *args) == -1
    assert "T*K" in lib.dpep_last_error().decode()
