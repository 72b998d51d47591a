"""Tensor-level entry points over the C-ABI (the counterpart of ``deep_ep._C`` in the reference,
csrc/bindings/module.cpp:17-95).

Like the reference's ``pointer()`` helper (csrc/ops/dispatch.cpp:36-49) every tensor is re-validated
here — device, dtype, contiguity, exact shape — before its address crosses the boundary.  Outputs
are allocated by the caller's framework (torch), never by the native side.  All calls enqueue on
torch's current stream and return without synchronising.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device) -> ctypes.c_void_p:
    """torch's current stream on ``device`` as a raw hipStream_t."""
    if _raw_stream is not None and device.index is not None:
        return ctypes.c_void_p(_raw_stream(device.index))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class _on_device:
    """``torch.cuda.device(dev)`` that costs nothing when ``dev`` is already current (the usual case)."""

    __slots__ = ("guard",)

    def __init__(self, device):
        self.guard = None if device.index == torch.cuda.current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


def _require(name, t, dtype, shape=None, device=None):
    if not isinstance(t, torch.Tensor):
        raise ValueError(f"{name} must be a tensor")
    if t.device.type != "cuda":
        raise ValueError(f"{name} must live on the GPU (got {t.device})")
    if device is not None and t.device != device:
        raise ValueError(f"{name} is on {t.device}, expected {device}")
    if t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype} (got {t.dtype})")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)} (got {tuple(t.shape)})")
    return t


class Workspace:
    """Owner of the native HBM workspace."""

    def __init__(self, num_bytes: int, device: Optional[torch.device] = None):
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        self._lib = _lib.load()
        handle = ctypes.c_void_p()
        with torch.cuda.device(self.device):
            _lib.check(self._lib.dpep_workspace_create(int(num_bytes), ctypes.byref(handle)), "workspace_create")
        self._handle = handle
        self.num_bytes = int(num_bytes)

    @property
    def handle(self):
        if self._handle is None:
            raise RuntimeError("workspace was destroyed")
        return self._handle

    @property
    def closed(self) -> bool:
        return self._handle is None

    def tune(self, key: str, value: int) -> None:
        """Test and diagnosis switches of the native workspace (``dpep_workspace_tune``)."""
        _lib.check(self._lib.dpep_workspace_tune(self.handle, key.encode(), int(value)), "workspace_tune")

    def destroy(self) -> None:
        if self._handle is not None:
            handle, self._handle = self._handle, None
            with torch.cuda.device(self.device):
                torch.cuda.synchronize(self.device)
                _lib.check(self._lib.dpep_workspace_destroy(handle), "workspace_destroy")


STORE_POLICIES = {"through": 0, "streaming": 1, "cached": 2}


def dispatch_store_policy(policy: Optional[str] = None) -> str:
    """Set (or, with no argument, read) how the dispatch kernels store their payload rows: ``"streaming"`` (default),
    ``"through"`` or ``"cached"``.  Process-wide.  Returns the policy that was in force before the call."""
    if policy is not None and policy not in STORE_POLICIES:
        raise ValueError(f"dispatch_store_policy: {policy!r} is not one of {sorted(STORE_POLICIES)}")
    code = _lib.load().dpep_dispatch_store_policy(3 if policy is None else STORE_POLICIES[policy])
    _lib.check(min(code, 0), "dispatch_store_policy")
    return {v: k for k, v in STORE_POLICIES.items()}[code]


def layout_workspace_bytes(num_tokens: int, num_topk: int, num_local: int) -> int:
    return int(_lib.load().dpep_layout_workspace_bytes(num_tokens, num_topk, num_local))


def layout(ws: Workspace, topk_idx: torch.Tensor, num_experts: int, expert_begin: int = 0, num_local: Optional[int] = None):
    """Routing layout on the device.  Returns device tensors; no host synchronisation.

    dict(counts[L], psum[L], offsets[L+1], route_to_row[T,K], row_to_route[T*K] (first R valid), num_rows[1]).
    """
    lib = _lib.load()
    _require("topk_idx", topk_idx, torch.int64, device=ws.device)
    if topk_idx.ndim != 2:
        raise ValueError("topk_idx must be [T, K]")
    tokens, topk = topk_idx.shape
    num_local = num_experts - expert_begin if num_local is None else num_local
    dev = topk_idx.device
    meta = torch.empty(3 * num_local + 2, dtype=torch.int32, device=dev)
    counts, psum = meta[:num_local], meta[num_local : 2 * num_local]
    offsets, num_rows = meta[2 * num_local : 3 * num_local + 1], meta[3 * num_local + 1 :]
    route_to_row = torch.empty((tokens, topk), dtype=torch.int32, device=dev)
    row_to_route = torch.empty((tokens * topk,), dtype=torch.int32, device=dev)
    with _on_device(dev):
        status = lib.dpep_layout(
            ws.handle, _ptr(topk_idx), tokens, topk, num_experts, expert_begin, num_local, _ptr(counts), _ptr(psum),
            _ptr(offsets), _ptr(route_to_row), _ptr(row_to_route), _ptr(num_rows), _stream(dev),
        )
    _lib.check(status, "layout")
    return dict(counts=counts, psum=psum, offsets=offsets, route_to_row=route_to_row, row_to_route=row_to_route,
                num_rows=num_rows, meta=meta)


def layout_wait(ws: Workspace, num_local: Optional[int] = None, timeout_s: float = 100.0):
    """The one host synchronisation of a fresh dispatch: waits for the most recent ``layout`` on ``ws`` and
    returns ``(counts, num_rows)`` as Python ints (``counts`` is None unless ``num_local`` is given).  The layout
    kernel writes these words into pinned host memory; nothing is copied and no stream is synchronised."""
    lib = _lib.load()
    rows = ctypes.c_int32()
    counts = None
    buf = None
    if num_local is not None:
        buf = (ctypes.c_int32 * num_local)()
    status = lib.dpep_layout_wait(ws.handle, buf, 0 if num_local is None else num_local, ctypes.byref(rows),
                                  int(timeout_s * 1e6))
    _lib.check(status, "layout_wait")
    if buf is not None:
        counts = list(buf)
    return counts, int(rows.value)


def dispatch_copy(x, scales, topk_weights, route_to_row, row_to_route, num_rows: Optional[int],
                  capacity_rows: Optional[int] = None):
    """out[row] = x[token(row)] (+ scale rows, + per-row weights).  x is BF16 [T,H] or FP8 [T,H].

    ``num_rows=None``: R is not known on the host yet (no ``layout_wait``): the outputs are allocated with T*K rows,
    (at least ``capacity_rows``, if given), of which the first R are written; the caller narrows them."""
    lib = _lib.load()
    if not isinstance(x, torch.Tensor) or x.dtype not in (torch.bfloat16, torch.float8_e4m3fn, torch.float16):
        raise ValueError("x must be a BF16, FP16 or FP8 E4M3FN tensor")
    _require("x", x, x.dtype)
    if x.ndim != 2:
        raise ValueError("x must be [T, H]")
    dev = x.device
    tokens, hidden = x.shape
    _require("route_to_row", route_to_row, torch.int32, device=dev)
    topk = route_to_row.shape[1]
    _require("route_to_row", route_to_row, torch.int32, (tokens, topk), dev)
    _require("row_to_route", row_to_route, torch.int32, device=dev)
    row_bytes = hidden * x.element_size()
    if row_bytes % 16:
        raise ValueError("hidden row size must be a multiple of 16 bytes")
    num_rows, known_rows = (max(tokens * topk, capacity_rows or 0), -1) if num_rows is None else (num_rows, num_rows)
    scale_cols = 0
    out_scales = None
    if scales is not None:
        # FP32 scales, or int32 words holding four packed E8M0 bytes (the low-latency scale format,
        # docs/elastic.md:97): either way 4-byte words that are moved bit for bit
        if not isinstance(scales, torch.Tensor) or scales.dtype not in (torch.float32, torch.int32):
            raise ValueError("scales must be FP32 or packed int32")
        _require("scales", scales, scales.dtype, device=dev)
        if scales.ndim != 2 or scales.shape[0] != tokens:
            raise ValueError("scales must be [T, C]")
        scale_cols = scales.shape[1]
        out_scales = torch.empty((num_rows, scale_cols), dtype=scales.dtype, device=dev)
    out_weights = None
    if topk_weights is not None:
        _require("topk_weights", topk_weights, torch.float32, (tokens, topk), dev)
        out_weights = torch.empty((num_rows,), dtype=torch.float32, device=dev)
    out = torch.empty((num_rows, hidden), dtype=x.dtype, device=dev)
    with _on_device(dev):
        status = lib.dpep_dispatch_copy(
            _ptr(x), _ptr(scales), _ptr(topk_weights), _ptr(route_to_row), _ptr(row_to_route), tokens, topk, known_rows,
            row_bytes, scale_cols, _ptr(out), _ptr(out_scales), _ptr(out_weights), _stream(dev),
        )
    _lib.check(status, "dispatch_copy")
    return out, out_scales, out_weights


SMALL_BATCH_ROUTES = 2048  # T*K up to which layout and dispatch share one launch (dpep_layout_dispatch_small)


def layout_dispatch_small(ws: Workspace, topk_idx, x, scales, topk_weights, num_experts: int, expert_begin: int = 0,
                          num_local: Optional[int] = None, quantize: bool = False, capacity_rows: Optional[int] = None):
    """Routing layout and payload dispatch of a small batch in one launch (``1 <= T*K <= SMALL_BATCH_ROUTES``).

    Returns ``(layout, out, out_scales, out_weights)``: ``layout`` as from ``layout()`` (``layout_wait`` works on it),
    the payload outputs as from ``dispatch_copy`` / ``dispatch_quant_fp8`` with ``num_rows=None``: allocated with T*K rows
    (at least ``capacity_rows``), of which the first R are written."""
    lib = _lib.load()
    _require("topk_idx", topk_idx, torch.int64, device=ws.device)
    if topk_idx.ndim != 2:
        raise ValueError("topk_idx must be [T, K]")
    tokens, topk = topk_idx.shape
    if not 1 <= tokens * topk <= SMALL_BATCH_ROUTES:
        raise ValueError(f"layout_dispatch_small takes 1..{SMALL_BATCH_ROUTES} routes")
    dev = topk_idx.device
    allowed = (torch.bfloat16,) if quantize else (torch.bfloat16, torch.float8_e4m3fn, torch.float16)
    if not isinstance(x, torch.Tensor) or x.dtype not in allowed:
        raise ValueError("x must be BF16 (quantize) or a BF16, FP16 or FP8 E4M3FN tensor")
    _require("x", x, x.dtype, device=dev)
    if x.ndim != 2 or x.shape[0] != tokens:
        raise ValueError("x must be [T, H]")
    hidden = x.shape[1]
    row_bytes = hidden * x.element_size()
    if quantize and hidden % 128:
        raise ValueError("hidden must be a multiple of 128 for FP8 dispatch")
    if row_bytes % 16:
        raise ValueError("hidden row size must be a multiple of 16 bytes")
    num_local = num_experts - expert_begin if num_local is None else num_local
    rows = max(tokens * topk, capacity_rows or 0)
    meta = torch.empty(3 * num_local + 2, dtype=torch.int32, device=dev)
    counts, psum = meta[:num_local], meta[num_local : 2 * num_local]
    offsets, num_rows = meta[2 * num_local : 3 * num_local + 1], meta[3 * num_local + 1 :]
    route_to_row = torch.empty((tokens, topk), dtype=torch.int32, device=dev)
    row_to_route = torch.empty((tokens * topk,), dtype=torch.int32, device=dev)
    scale_cols = 0
    out_scales = None
    if quantize:
        if scales is not None:
            raise ValueError("the fused quantiser takes no input scales")
        out = torch.empty((rows, hidden), dtype=torch.float8_e4m3fn, device=dev)
        out_scales = torch.empty((rows, hidden // 128), dtype=torch.float32, device=dev)
    else:
        out = torch.empty((rows, hidden), dtype=x.dtype, device=dev)
        if scales is not None:
            if not isinstance(scales, torch.Tensor) or scales.dtype not in (torch.float32, torch.int32):
                raise ValueError("scales must be FP32 or packed int32")
            _require("scales", scales, scales.dtype, device=dev)
            if scales.ndim != 2 or scales.shape[0] != tokens:
                raise ValueError("scales must be [T, C]")
            scale_cols = scales.shape[1]
            out_scales = torch.empty((rows, scale_cols), dtype=scales.dtype, device=dev)
    out_weights = None
    if topk_weights is not None:
        _require("topk_weights", topk_weights, torch.float32, (tokens, topk), dev)
        out_weights = torch.empty((rows,), dtype=torch.float32, device=dev)
    with _on_device(dev):
        status = lib.dpep_layout_dispatch_small(
            ws.handle, _ptr(topk_idx), _ptr(x), _ptr(scales), _ptr(topk_weights), tokens, topk, num_experts, expert_begin,
            num_local, row_bytes, scale_cols, int(bool(quantize)), _ptr(counts), _ptr(psum), _ptr(offsets), _ptr(route_to_row),
            _ptr(row_to_route), _ptr(num_rows), _ptr(out), _ptr(out_scales), _ptr(out_weights), _stream(dev),
        )
    _lib.check(status, "layout_dispatch_small")
    layout_out = dict(counts=counts, psum=psum, offsets=offsets, route_to_row=route_to_row, row_to_route=row_to_route,
                      num_rows=num_rows, meta=meta)
    return layout_out, out, out_scales, out_weights


def dispatch_quant_fp8(x, topk_weights, route_to_row, row_to_route, num_rows: Optional[int]):
    """Fused per-128 FP8 quantisation + expand-permute of BF16 x [T,H]; ``num_rows=None`` as in ``dispatch_copy``."""
    lib = _lib.load()
    _require("x", x, torch.bfloat16)
    if x.ndim != 2:
        raise ValueError("x must be [T, H]")
    dev = x.device
    tokens, hidden = x.shape
    if hidden % 128:
        raise ValueError("hidden must be a multiple of 128 for FP8 dispatch")
    _require("route_to_row", route_to_row, torch.int32, device=dev)
    topk = route_to_row.shape[1]
    _require("route_to_row", route_to_row, torch.int32, (tokens, topk), dev)
    _require("row_to_route", row_to_route, torch.int32, device=dev)
    num_rows, known_rows = (tokens * topk, -1) if num_rows is None else (num_rows, num_rows)
    out_weights = None
    if topk_weights is not None:
        _require("topk_weights", topk_weights, torch.float32, (tokens, topk), dev)
        out_weights = torch.empty((num_rows,), dtype=torch.float32, device=dev)
    out = torch.empty((num_rows, hidden), dtype=torch.float8_e4m3fn, device=dev)
    out_scales = torch.empty((num_rows, hidden // 128), dtype=torch.float32, device=dev)
    with _on_device(dev):
        status = lib.dpep_dispatch_quant_fp8(
            _ptr(x), _ptr(topk_weights), _ptr(route_to_row), _ptr(row_to_route), tokens, topk, known_rows, hidden,
            _ptr(out), _ptr(out_scales), _ptr(out_weights), _stream(dev),
        )
    _lib.check(status, "dispatch_quant_fp8")
    return out, out_scales, out_weights


def cast_to_fp8(x):
    """per_token_cast_to_fp8 on the device: BF16 [T,H] -> (FP8 [T,H], FP32 [T,ceil(H/128)]); a short last block is
    quantised as if padded with zeros, as the reference does."""
    lib = _lib.load()
    _require("x", x, torch.bfloat16)
    if x.ndim != 2 or x.shape[1] % 16 or x.shape[1] == 0:
        raise ValueError("x must be [T, H] with H a positive multiple of 16")
    tokens, hidden = x.shape
    out = torch.empty((tokens, hidden), dtype=torch.float8_e4m3fn, device=x.device)
    scales = torch.empty((tokens, (hidden + 127) // 128), dtype=torch.float32, device=x.device)
    with _on_device(x.device):
        status = lib.dpep_cast_to_fp8(_ptr(x), tokens, hidden, _ptr(out), _ptr(scales), _stream(x.device))
    _lib.check(status, "cast_to_fp8")
    return out, scales


def cast_back(codes, scales):
    """per_token_cast_back on the device: (FP8 e4m3fn [T,H], scales) -> BF16 [T,H], bf16(fp32(code) * scale) per block of
    128 columns.  scales: FP32 [T, ceil(H/128)], or int32 [T, ceil(H/128)/4] holding four e8m0 exponent bytes each."""
    lib = _lib.load()
    _require("codes", codes, torch.float8_e4m3fn)
    if codes.ndim != 2 or codes.shape[1] % 16 or codes.shape[1] == 0:
        raise ValueError("codes must be [T, H] with H a positive multiple of 16")
    tokens, hidden = codes.shape
    blocks = (hidden + 127) // 128
    if scales.dtype == torch.int32:
        if blocks % 4:
            raise ValueError("int32 scales hold four blocks each: ceil(H/128) must be a multiple of 4")
        _require("scales", scales, torch.int32, (tokens, blocks // 4), codes.device)
    else:
        _require("scales", scales, torch.float32, (tokens, blocks), codes.device)
    out = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=codes.device)
    with _on_device(codes.device):
        status = lib.dpep_cast_back(_ptr(codes), _ptr(scales), int(scales.dtype == torch.int32), tokens, hidden, _ptr(out),
                                    _stream(codes.device))
    _lib.check(status, "cast_back")
    return out


def combine(y, route_to_row, row_weights=None, return_values=None, out=None, served_only=False):
    """out[t] = round( sum_s fp32(y[row(t,s)]) (* row_weights[row]) ) in y's dtype (BF16 or FP16); optional
    weight-return channel.  ``served_only`` (BF16, needs ``out``): tokens without any row keep what ``out`` held instead
    of being zero-filled (one rank's share of an EP job produces nothing for the tokens it does not serve)."""
    lib = _lib.load()
    if not isinstance(y, torch.Tensor) or y.dtype not in (torch.bfloat16, torch.float16):
        raise ValueError("y must be a BF16 or FP16 tensor")
    _require("y", y, y.dtype)
    if y.ndim != 2:
        raise ValueError("y must be [R, H]")
    dev = y.device
    rows, hidden = y.shape
    if hidden % 8:
        raise ValueError("hidden must be a multiple of 8")
    _require("route_to_row", route_to_row, torch.int32, device=dev)
    if route_to_row.ndim != 2:
        raise ValueError("route_to_row must be [T, K]")
    tokens, topk = route_to_row.shape
    if row_weights is not None:
        _require("row_weights", row_weights, torch.float32, (rows,), dev)
    returned = None
    if return_values is not None:
        _require("return_values", return_values, torch.float32, (rows,), dev)
        returned = torch.empty((tokens, topk), dtype=torch.float32, device=dev)
    if out is None:
        if served_only:
            raise ValueError("served_only needs the caller's out (rows of unserved tokens are left as they are)")
        out = torch.empty((tokens, hidden), dtype=y.dtype, device=dev)
    else:
        _require("out", out, y.dtype, (tokens, hidden), dev)
    entry = lib.dpep_combine if y.dtype == torch.bfloat16 else lib.dpep_combine_fp16
    if served_only:
        if y.dtype != torch.bfloat16:
            raise ValueError("served_only is available for BF16 rows")
        entry = lib.dpep_combine_served
    with _on_device(dev):
        status = entry(
            _ptr(y), _ptr(row_weights), _ptr(route_to_row), tokens, topk, rows, hidden, _ptr(out),
            _ptr(return_values), _ptr(returned), _stream(dev),
        )
    _lib.check(status, "combine")
    return out, returned


# ---------------------------------------------------------------------------------------------
# MegaMoE (W4A8) entry points
# ---------------------------------------------------------------------------------------------
def mx_quant(x):
    """MXFP8 activation quantiser: BF16 [B,H] -> (e4m3 codes [B,H] as float8_e4m3fn, e8m0 bytes [B,H/32] uint8)."""
    lib = _lib.load()
    _require("x", x, torch.bfloat16)
    if x.ndim != 2 or x.shape[1] % 32:
        raise ValueError("x must be [B, H] with H a multiple of 32")
    rows, hidden = x.shape
    codes = torch.empty((rows, hidden), dtype=torch.float8_e4m3fn, device=x.device)
    scales = torch.empty((rows, hidden // 32), dtype=torch.uint8, device=x.device)
    with _on_device(x.device):
        status = lib.dpep_mx_quant(_ptr(x), rows, hidden, _ptr(codes), _ptr(scales), _stream(x.device))
    _lib.check(status, "mx_quant")
    return codes, scales


def megamoe_workspace_bytes(num_tokens, num_topk, hidden, intermediate, num_local, num_shared: int = 0) -> int:
    return int(_lib.load().dpep_megamoe_workspace_bytes(num_tokens, num_topk, hidden, intermediate, num_local, num_shared))


def megamoe_padded_dim(dim: int) -> int:
    """What the grouped GEMM works on for a logical hidden / intermediate size (whole 256-column tiles, at least 512)."""
    return int(_lib.load().dpep_megamoe_padded_dim(int(dim)))


def megamoe_prepared_shape(n: int, k: int, gate_up: bool):
    """(padded N, padded K, scale bytes per column) of the prepared form of a raw [L,N,K/2] weight tensor."""
    import ctypes

    out = [ctypes.c_int(0) for _ in range(3)]
    status = _lib.load().dpep_megamoe_prepared_shape(int(n), int(k), int(bool(gate_up)), *(ctypes.byref(v) for v in out))
    _lib.check(status, "megamoe_prepared_shape")
    return tuple(v.value for v in out)


def megamoe_prepare_weights(w_packed, w_scales, gate_up: bool):
    """Raw packed FP4 uint8 [L,N,K/2] + e8m0 uint8 [L,N,K/32] -> the kernel's streaming order, padded to the sizes the
    GEMM works on (``megamoe_prepared_shape``: zero codes and unit scales behind N and K).

    Returns (packed [L,Np,Kp/2], scales [L,Np,scale_cols])."""
    lib = _lib.load()
    _require("w_packed", w_packed, torch.uint8)
    if w_packed.ndim != 3:
        raise ValueError("w_packed must be [L, N, K/2]")
    experts, n, half_k = w_packed.shape
    k = half_k * 2
    _require("w_scales", w_scales.reshape(experts, n, -1), torch.uint8, (experts, n, k // 32), w_packed.device)
    np_, kp, scale_cols = megamoe_prepared_shape(n, k, gate_up)
    out_w = torch.empty((experts, np_, kp // 2), dtype=torch.uint8, device=w_packed.device)
    out_s = torch.empty((experts, np_, scale_cols), dtype=torch.uint8, device=w_packed.device)
    with _on_device(w_packed.device):
        status = lib.dpep_megamoe_prepare_weights(
            _ptr(w_packed), _ptr(w_scales), experts, n, k, int(bool(gate_up)), _ptr(out_w), _ptr(out_s),
            _stream(w_packed.device),
        )
    _lib.check(status, "megamoe_prepare_weights")
    return out_w, out_s


def megamoe_fill_report(ws, num_tokens, num_topk, hidden, intermediate, num_local, num_shared: int = 0):
    """(filler waves, tokens they looked at) of the most recent forward on ``ws``; waits for the current stream."""
    fillers, filled = ctypes.c_int32(0), ctypes.c_int64(0)
    device = ws.device
    status = _lib.load().dpep_megamoe_fill_report(ws.handle, num_tokens, num_topk, hidden, intermediate, num_local, num_shared,
                                                  ctypes.byref(fillers), ctypes.byref(filled), _stream(device))
    _lib.check(status, "megamoe_fill_report")
    return fillers.value, filled.value


def megamoe_forward(ws, x_codes, x_scales, topk_idx, topk_weights, w1, s1, w2, s2, num_experts, expert_begin,
                    num_local, y, expert_token_nums, shared=None, intermediate=None):
    """Fused W4A8 forward of one rank's local experts; writes y [B,H] BF16 and expert_token_nums [L] int32.

    ``intermediate`` = the experts' logical intermediate size; by default what the prepared ``w1`` holds (right unless
    the weights were padded).  ``shared`` = (w1, s1, w2, s2) prepared weights of S shared experts, which every token
    passes through."""
    lib = _lib.load()
    dev = ws.device
    _require("x_codes", x_codes, torch.float8_e4m3fn, device=dev)
    tokens, hidden = x_codes.shape
    _require("x_scales", x_scales, torch.uint8, (tokens, hidden // 32), dev)
    _require("topk_idx", topk_idx, torch.int32, device=dev)
    topk = topk_idx.shape[1]
    _require("topk_idx", topk_idx, torch.int32, (tokens, topk), dev)
    _require("topk_weights", topk_weights, torch.float32, (tokens, topk), dev)
    _require("w1", w1, torch.uint8, device=dev)
    if w1.ndim != 3 or w1.shape[0] != num_local or w1.shape[1] % 2:
        raise ValueError("w1 must be prepared [L, 2I, H/2]")
    if intermediate is None:
        intermediate = w1.shape[1] // 2
    if hidden % 64 or intermediate % 128 or hidden < 64 or intermediate < 128:
        raise ValueError("hidden must be a positive multiple of 64, intermediate of 128")
    n1, k1, cols1 = megamoe_prepared_shape(2 * intermediate, hidden, True)
    n2, k2, cols2 = megamoe_prepared_shape(hidden, intermediate, False)
    _require("w1", w1, torch.uint8, (num_local, n1, k1 // 2), dev)
    _require("s1", s1, torch.uint8, (num_local, n1, cols1), dev)
    _require("w2", w2, torch.uint8, (num_local, n2, k2 // 2), dev)
    _require("s2", s2, torch.uint8, (num_local, n2, cols2), dev)
    _require("y", y, torch.bfloat16, (tokens, hidden), dev)
    _require("expert_token_nums", expert_token_nums, torch.int32, (num_local,), dev)
    num_shared = 0
    sw1 = ss1 = sw2 = ss2 = None
    if shared is not None:
        sw1, ss1, sw2, ss2 = shared
        _require("shared w1", sw1, torch.uint8, device=dev)
        num_shared = sw1.shape[0]
        _require("shared w1", sw1, torch.uint8, (num_shared, n1, k1 // 2), dev)
        _require("shared s1", ss1, torch.uint8, (num_shared, n1, cols1), dev)
        _require("shared w2", sw2, torch.uint8, (num_shared, n2, k2 // 2), dev)
        _require("shared s2", ss2, torch.uint8, (num_shared, n2, cols2), dev)
    with _on_device(dev):
        status = lib.dpep_megamoe_forward(
            ws.handle, _ptr(x_codes), _ptr(x_scales), _ptr(topk_idx), _ptr(topk_weights), _ptr(w1), _ptr(s1), _ptr(w2),
            _ptr(s2), _ptr(sw1), _ptr(ss1), _ptr(sw2), _ptr(ss2), num_shared, tokens, hidden, intermediate, topk,
            num_experts, expert_begin, num_local, _ptr(y), _ptr(expert_token_nums), _stream(dev),
        )
    _lib.check(status, "megamoe_forward")
    return y, expert_token_nums
