"""The C-ABI rejects bad arguments before it touches the GPU, so these run without one: every entry
point returns DPEP_EINVAL (-1) with a message, never crashes, never launches."""

import ctypes

import pytest

from deepep_amd import _lib


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def _message(lib):
    return lib.dpep_last_error().decode()


def test_null_workspace_and_ranges(lib):
    fake = ctypes.c_void_p(0)
    rows = ctypes.c_int32()
    assert lib.dpep_workspace_create(0, ctypes.byref(fake)) == -1 and "bytes" in _message(lib)
    assert lib.dpep_workspace_destroy(None) == -1 and "not a live workspace" in _message(lib)
    assert lib.dpep_layout(None, None, 4, 2, 8, 0, 8, None, None, None, None, None, None, None) == -1
    assert "not a live workspace" in _message(lib)
    assert lib.dpep_layout_wait(None, None, 0, ctypes.byref(rows), 1000) == -1
    assert lib.dpep_layout_workspace_bytes(-1, 2, 8) == 0
    assert lib.dpep_megamoe_workspace_bytes(0, 2, 512, 512, 4, 0) == 0
    assert lib.dpep_megamoe_workspace_bytes(16, 2, 512, 512, 4, -1) == 0
    assert [lib.dpep_megamoe_padded_dim(d) for d in (0, 64, 256, 512, 576, 768, 1088, 7168)] == [0, 512, 512, 512, 768, 768, 1280, 7168]
    shape = [ctypes.c_int() for _ in range(3)]
    refs = [ctypes.byref(v) for v in shape]
    assert lib.dpep_megamoe_prepared_shape(256, 768, 0, *refs) == 0
    assert [v.value for v in shape] == [512, 768, 32]  # two spans of k = 512, the last padded
    assert lib.dpep_megamoe_prepared_shape(2 * 384, 1088, 1, *refs) == 0
    assert [v.value for v in shape] == [1024, 1280, 48]  # gate and up halves padded to 512 each
    assert lib.dpep_megamoe_prepared_shape(4096, 7168, 1, *refs) == 0 and [v.value for v in shape] == [4096, 7168, 224]
    assert lib.dpep_megamoe_prepared_shape(100, 512, 0, *refs) == -1 and "N=100" in _message(lib)
    assert lib.dpep_megamoe_prepared_shape(384, 512, 1, *refs) == -1 and "N=384" in _message(lib)  # I = 192
    assert lib.dpep_megamoe_prepared_shape(256, 96, 0, *refs) == -1 and "K=96" in _message(lib)


def test_payload_entry_points_check_arguments_first(lib):
    # (bad top-k, bad row count, unaligned rows) are reported before any pointer is followed
    assert lib.dpep_combine(None, None, None, 4, 0, 0, 128, None, None, None, None) == -1 and "K=0" in _message(lib)
    assert lib.dpep_combine(None, None, None, 4, 2, -3, 128, None, None, None, None) == -1 and "num_rows" in _message(lib)
    # more rows than routes is fine (a capacity layout); the call then fails on the buffers it was not given
    assert lib.dpep_combine(None, None, None, 4, 2, 9, 128, None, None, None, None) == -1 and "NULL" in _message(lib)
    assert lib.dpep_combine(None, None, None, 4, 2, 4, 12, None, None, None, None) == -1 and "hidden" in _message(lib)
    assert lib.dpep_combine(None, None, None, 0, 2, 0, 128, None, None, None, None) == 0  # nothing to do
    assert lib.dpep_dispatch_copy(None, None, None, None, None, 4, 33, 4, 256, 0, None, None, None, None) == -1
    assert lib.dpep_dispatch_quant_fp8(None, None, None, None, 4, 2, 0, 100, None, None, None, None) == -1
    assert "multiple of 128" in _message(lib)
    assert lib.dpep_cast_to_fp8(None, -1, 128, None, None, None) == -1
    assert lib.dpep_mx_quant(None, 4, 48, None, None, None) == -1
    assert lib.dpep_megamoe_prepare_weights(None, None, 0, 256, 512, 0, None, None, None) == -1
    assert lib.dpep_megamoe_prepare_weights(None, None, 1, 100, 512, 0, None, None, None) == -1 and "N=100" in _message(lib)
    assert lib.dpep_megamoe_forward(None, *([None] * 12), 0, 4, 512, 512, 2, 8, 0, 8, None, None, None) == -1


def test_status_to_exception_mapping(lib):
    lib.dpep_workspace_destroy(None)
    with pytest.raises(ValueError, match="workspace_destroy"):
        _lib.check(-1, "workspace_destroy")
    with pytest.raises(RuntimeError):
        _lib.check(-2, "anything")
    _lib.check(0, "ok")
