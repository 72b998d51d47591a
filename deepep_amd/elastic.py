"""``ElasticBuffer`` / ``EPHandle`` with the reference's V2 interface, on one MI355X.

Mirrors deep_ep/backends/mesh_clos/elastic.py (EPHandle :88-173, ElasticBuffer.__init__ :178-269,
dispatch :648-1008, combine :1010-1283, _notify :1285-1531): same argument names, defaults, return
tuples and exception types.  What is different, deliberately:

  * one process, one GPU: ``world_size`` defaults to 1 (the reference rejects < 2).  Passing
    ``rank``/``world_size`` makes the buffer act as ONE rank's share of an EP job: it owns experts
    ``[rank*E/P, (rank+1)*E/P)`` and ``x`` / ``topk_idx`` are the flattened token stream of all source
    ranks, so rows come out in the reference's (local expert, source rank, token, slot) order;
  * the routing metadata is the plain pair route_to_row / row_to_route instead of SHMEM peer
    tables; payload rows are written straight into torch-allocated outputs;
  * ``use_fp8_dispatch=True`` with a BF16 ``x`` quantises per 128 elements inside the dispatch
    kernel and returns ``(fp8, scales)`` (the reference moves pre-quantised tuples only — which this
    class also accepts);
  * a synchronous call (``async_with_compute_stream=False``) is queued on the caller's current stream; only
    asynchronous calls use the communication stream (see ``_Enqueue``).
"""

from __future__ import annotations

import threading
import warnings
from typing import Optional, Tuple, Union

import torch

from .compat import accept_aliases
from .event import EventHandle, EventOverlap, gpu_api

WORLD_SIZES = (1, 2, 4, 8, 16, 32, 64, 128, 256, 512)
MAX_TOKENS = 16384
MAX_HIDDEN = 7168
MAX_TOPK = 16
MAX_EXPERTS = 1024
MIN_WORKSPACE_BYTES = 2 << 20
WORKSPACE_ALLOCATION_CAP = 64 << 20
LOW_LATENCY_WORKSPACE_BYTES = 8 << 30
LOW_LATENCY_WORLD_SIZES = (16, 32, 64, 128, 256)
LOW_LATENCY_MAX_TOKENS = 256
# Routing tensors whose (data_ptr, version) are pinned at dispatch and re-checked by every later
# cached dispatch and combine.
_ROUTING = ("topk_idx", "route_to_row", "weight_return_meta", "expert_totals", "psum_num_recv_tokens_per_expert")


def _enforce(*rules):
    """Runs argument rules in order: each is ``(holds, exception type, message)``, where ``holds`` is a bool or a
    callable evaluated only when the earlier rules have passed.  The first rule that does not hold raises."""
    for holds, error, message in rules:
        if not (holds() if callable(holds) else holds):
            raise error(message)


def _is_bool(value):
    return type(value) is bool


def _int_among(value, allowed):
    return type(value) is int and value in allowed


def _integer(name, value, lower, upper):
    if type(value) is not int or not lower <= value <= upper:
        raise ValueError(f"{name} must be an integer in [{lower}, {upper}]")


def _validate_hidden(hidden, fp8=False):
    _integer("hidden", hidden, 1, MAX_HIDDEN)
    alignment = 128 if fp8 else 16
    if hidden % alignment:
        raise ValueError(f"hidden must be a multiple of {alignment}")


def _load_native():
    from . import ops

    ops._lib.load()  # raises if libdeepep_amd.so is not built: there is no fallback path
    return ops


class EPHandle:
    """Routing plan produced by a fresh dispatch; reused by cached dispatch and by combine."""

    @accept_aliases(num_compute_units="num_sms")
    def __init__(
        self,
        do_expand: bool,
        num_experts: int,
        expert_alignment: int,
        num_max_tokens_per_rank: int,
        num_sms: int,
        topk_idx: torch.Tensor,
        num_recv_tokens: int,
        num_expanded_tokens: int,
        num_recv_tokens_per_expert_list: list,
        psum_num_recv_tokens_per_scaleup_rank: torch.Tensor,
        psum_num_recv_tokens_per_expert: torch.Tensor,
        num_unaligned_recv_tokens_per_expert: torch.Tensor,
        recv_src_metadata: torch.Tensor,
        dst_buffer_slot_idx: torch.Tensor,
        token_metadata_at_forward: Optional[torch.Tensor],
        channel_linked_list: Optional[torch.Tensor],
        is_low_latency: bool = False,
    ):
        self.do_expand = do_expand
        self.num_experts = num_experts
        self.expert_alignment = expert_alignment
        self.num_max_tokens_per_rank = num_max_tokens_per_rank
        self.num_compute_units = num_sms
        self.topk_idx = topk_idx
        self.num_recv_tokens = num_recv_tokens
        self.num_expanded_tokens = num_expanded_tokens
        self.num_recv_tokens_per_expert_list = num_recv_tokens_per_expert_list
        self.psum_num_recv_tokens_per_scaleup_rank = psum_num_recv_tokens_per_scaleup_rank
        self.psum_num_recv_tokens_per_expert = psum_num_recv_tokens_per_expert
        self.num_unaligned_recv_tokens_per_expert = num_unaligned_recv_tokens_per_expert
        self.recv_src_metadata = recv_src_metadata
        self.dst_buffer_slot_idx = dst_buffer_slot_idx
        self.token_metadata_at_forward = token_metadata_at_forward
        self.channel_linked_list = channel_linked_list
        self.is_low_latency = is_low_latency
        # Single-GPU routing metadata.
        self.route_to_row = None          # int32 [T,K]: row of each route, -1 without a row
        self.weight_return_meta = None    # int32 [R]: flat route id (src*T+t)*K+s of each row
        self.expert_totals = None         # int32 [L]: rows per local expert
        self.expert_offsets = None        # int32 [L+1]: exclusive prefix
        self.source_weights = None        # fp32 [R]: saved route weights (low-latency style handles)
        self.send_counts = None           # int32 [E]: low-latency handles; its last entry is R
        self.expert_recv_counts = None
        self.rank = None
        self.world_size = None
        self.num_tokens = None
        self.num_topk = None
        self.hidden = None
        self.metadata_only = True
        self.metadata_version = 7
        self._buffer_token = None
        self._routing_versions = {}

    @property
    def num_sms(self):
        return self.num_compute_units

    @num_sms.setter
    def num_sms(self, value):
        self.num_compute_units = value


class _Enqueue:
    """Where one call's kernels go, and what the caller gets to wait on.

    The reference always launches on its communication stream and, unless ``async_with_compute_stream`` is set, makes
    the caller's stream wait for it before the call returns (deep_ep/backends/mesh_clos/elastic.py:905-1003).  On one GPU
    that round trip through a second stream buys nothing for a synchronous call, and its events and stream switches cost
    more host time than a decode step's kernels take; so a synchronous call is queued on the caller's own current stream
    (nothing to wait for afterwards, no tensor crosses a stream) and only an asynchronous one goes to the communication
    stream, behind an event on the caller's stream, and hands back an event that keeps its tensors alive.
    One buffer's calls share its workspace: a call queued on another stream than the previous one waits for that stream.
    """

    def __init__(self, runtime, previous_event=None, asynchronous=False):
        self.runtime, self.previous_event, self.asynchronous = runtime, previous_event, asynchronous
        self._scope = None

    def __enter__(self):
        runtime, api = self.runtime, gpu_api()
        if self.previous_event is not None:
            self.previous_event.current_stream_wait()
        if self.asynchronous:
            producer = EventHandle()
            self._scope = api.stream(runtime.stream)
            self._scope.__enter__()
            producer.current_stream_wait()
            target = runtime.stream
        else:
            target = api.current_stream(runtime.device)
        last = getattr(runtime, "last_stream", None)
        if last is not None and last != target:
            target.wait_stream(last)
        runtime.last_stream = target
        return self

    def event(self, retained):
        """What the call returns as its event; asynchronous calls record it on the communication stream (call inside
        the ``with`` block)."""
        if self.asynchronous:
            return EventOverlap._holding(EventHandle(), retained)
        return EventOverlap()

    def __exit__(self, *exc):
        if self._scope is not None:
            self._scope.__exit__(*exc)
        return False


class _Runtime:
    """Process-local owner of the HBM workspace and the communication stream (the single-GPU
    counterpart of deep_ep/_runtime.py:67-308 without SHMEM bootstrap)."""

    def __init__(self, native, num_bytes, rank, world_size, combine_only):
        self.native = native
        self.device = gpu_api().current_device()
        self.torch_device = torch.device("cuda", self.device)
        self.rank, self.world_size = rank, world_size
        self.combine_only = combine_only
        self.capacity = num_bytes
        self.notify_lock = threading.RLock()
        self.notify_failed = False
        self.notify_inflight = None
        # `capacity` is what the caller asked for (the low-latency path insists on exactly 8 GiB, as the reference
        # does); the HBM actually taken is bounded by what the single-GPU kernels use, the layout scratch.
        self.workspace = native.Workspace(min(num_bytes, WORKSPACE_ALLOCATION_CAP), self.torch_device)
        self.stream = gpu_api().Stream(device=self.torch_device)
        self.last_stream = None  # the stream the buffer's most recent kernels were queued on
        self.closed = False

    def ensure_alive(self):
        if self.closed:
            raise RuntimeError("ElasticBuffer was destroyed")

    def close(self):
        if not self.closed:
            self.stream.synchronize()
            if self.last_stream is not None:
                self.last_stream.synchronize()
            self.workspace.destroy()
            self.closed = True
            self.notify_inflight = None


def _resolve_world(group, rank, world_size):
    if group is not None:
        if rank is not None or world_size is not None:
            raise ValueError("Pass either group or rank/world_size, not both")
        import torch.distributed as dist

        if not isinstance(group, dist.ProcessGroup):
            raise TypeError("group must be an initialized torch.distributed ProcessGroup")
        if dist.get_world_size(group) != 1:
            raise NotImplementedError(
                "This build runs one rank per process on one GPU without inter-GPU transport: "
                "use a single-rank group, or rank=/world_size= to compute one rank's share"
            )
        return 0, 1
    if world_size is None and rank is None:
        return 0, 1
    _integer("world_size", world_size, 1, 512)
    if world_size not in WORLD_SIZES:
        raise ValueError("Runtime supports EP1/2/4/8/16/32/64/128/256/512")
    _integer("rank", rank, 0, world_size - 1)
    return rank, world_size


class ElasticBuffer:
    """Dispatch / combine for one EP rank on one GPU; see the module docstring for the deviations."""

    @accept_aliases(num_device_timeout_secs="num_gpu_timeout_secs")
    def __init__(
        self,
        group=None,
        num_bytes: Optional[int] = None,
        num_cpu_bytes: int = 0,
        num_max_tokens_per_rank: int = 0,
        hidden: int = 0,
        num_topk: int = 0,
        use_fp8_dispatch: bool = False,
        deterministic: bool = False,
        allow_hybrid_mode: bool = True,
        allow_multiple_reduction: bool = True,
        prefer_overlap_with_compute: bool = True,
        sl_idx: int = 3,
        num_allocated_qps: int = 0,
        num_cpu_timeout_secs: int = 300,
        num_gpu_timeout_secs: int = 100,
        explicitly_destroy: bool = False,
        *,
        rank: Optional[int] = None,
        world_size: Optional[int] = None,
        bootstrap: str = "default",
        combine_only: bool = False,
        use_1g_huge_pages: bool = True,
        debug_collectives: bool = False,
        machine_type: str = "auto",
        rootinfo_path: Optional[str] = None,
    ):
        native = _load_native()
        defaults_only = (
            num_cpu_bytes == 0 and deterministic is False and allow_hybrid_mode is True and allow_multiple_reduction is True
            and prefer_overlap_with_compute is True and sl_idx == 3 and _int_among(num_allocated_qps, (0, 6))
            and num_gpu_timeout_secs == 100
        )
        _enforce(
            (defaults_only, NotImplementedError, "ElasticBuffer supports default options and num_allocated_qps=0/6"),
            (_is_bool(use_fp8_dispatch), TypeError, "use_fp8_dispatch must be bool"),
            (explicitly_destroy is True, NotImplementedError, "Runtime currently requires explicitly_destroy=True"),
            (_is_bool(combine_only) and _is_bool(debug_collectives), TypeError, "combine_only and debug_collectives must be bool"),
        )
        _integer("num_max_tokens_per_rank", num_max_tokens_per_rank, 0, MAX_TOKENS)
        _integer("num_topk", num_topk, 0, MAX_TOPK)
        _integer("hidden", hidden, 0, MAX_HIDDEN)
        if hidden:
            _validate_hidden(hidden, use_fp8_dispatch)
        resolved_rank, resolved_world = _resolve_world(group, rank, world_size)
        if num_bytes is None:
            if not num_max_tokens_per_rank or not num_topk or not hidden:
                raise NotImplementedError("Pass num_bytes or provide token/topk bounds and hidden")
            num_bytes = self.get_buffer_size_hint(
                group, num_max_tokens_per_rank, hidden, num_topk, use_fp8_dispatch, world_size=world_size
            )
        _integer("num_bytes", num_bytes, MIN_WORKSPACE_BYTES, (1 << 63) - 1)
        self.num_max_tokens_per_rank = num_max_tokens_per_rank
        self.hidden = hidden
        self.num_topk = num_topk
        self.use_fp8_dispatch = use_fp8_dispatch
        self.machine_type = "mi355x"
        self._handle_token = object()
        self._runtime = _Runtime(native, num_bytes, resolved_rank, resolved_world, combine_only)

    def __del__(self):
        runtime = getattr(self, "_runtime", None)
        if runtime is not None and not runtime.closed:
            warnings.warn("ElasticBuffer was not destroyed explicitly; call destroy()", ResourceWarning)

    def _live_runtime(self) -> _Runtime:
        runtime = getattr(self, "_runtime", None)
        if runtime is None:
            raise RuntimeError("ElasticBuffer is not initialised")
        return runtime

    def destroy(self) -> None:
        """Release the workspace; repeating a successful destroy is safe."""
        self._live_runtime().close()

    @staticmethod
    def get_buffer_size_hint(
        group,
        num_max_tokens_per_rank: int,
        hidden: int,
        num_topk: int = 0,
        use_fp8_dispatch: bool = False,
        allow_hybrid_mode: bool = True,
        allow_multiple_reduction: bool = True,
        *,
        world_size: Optional[int] = None,
        machine_type: str = "auto",
        rootinfo_path: Optional[str] = None,
    ) -> int:
        """Workspace bytes for the given bounds.

        Payload rows go straight into the returned tensors, so the workspace only holds the layout
        scratch; the hint is that scratch rounded up to the 2 MiB minimum.
        """
        native = _load_native()
        _validate_hidden(hidden, use_fp8_dispatch)
        if allow_hybrid_mode is not True or allow_multiple_reduction is not True:
            raise NotImplementedError("Dispatch sizing supports only default algorithm options")
        _integer("num_max_tokens_per_rank", num_max_tokens_per_rank, 1, MAX_TOKENS)
        _integer("num_topk", num_topk, 0, MAX_TOPK)
        world = 1 if world_size is None else world_size
        if world not in WORLD_SIZES:
            raise ValueError("Runtime supports EP1/2/4/8/16/32/64/128/256/512")
        scratch = native.layout_workspace_bytes(world * num_max_tokens_per_rank, max(num_topk, 1), MAX_EXPERTS)
        return max(MIN_WORKSPACE_BYTES, (scratch + (2 << 20) - 1) // (2 << 20) * (2 << 20))

    def barrier(self, use_comm_stream: bool = True, with_cpu_sync: bool = False, sequential: bool = True) -> None:
        """Host-synchronous barrier: with one rank it drains the streams the buffer's kernels were queued on."""
        if type(use_comm_stream) is not bool or with_cpu_sync is not True or sequential is not True:
            raise NotImplementedError("Only the host-synchronous sequential barrier is implemented")
        runtime = self._live_runtime()
        runtime.ensure_alive()
        runtime.stream.synchronize()
        if getattr(runtime, "last_stream", None) is not None:
            runtime.last_stream.synchronize()

    @staticmethod
    def capture() -> EventHandle:
        """Record an event on the current stream."""
        return EventHandle()

    def get_comm_stream(self) -> torch.cuda.Stream:
        runtime = self._live_runtime()
        runtime.ensure_alive()
        return runtime.stream

    def get_physical_domain_size(self) -> Tuple[int, int]:
        raise NotImplementedError("ElasticBuffer.get_physical_domain_size is declared but not implemented")

    def get_logical_domain_size(self) -> Tuple[int, int]:
        raise NotImplementedError("ElasticBuffer.get_logical_domain_size is declared but not implemented")

    @accept_aliases(
        scaleout_gbs="rdma_gbs",
        scaleup_gbs="nvlink_gbs",
        compute_read_gbs="sm_read_gbs",
        compute_write_gbs="sm_write_gbs",
        compute_unit_read_gbs="sm_read_gbs",
        compute_unit_write_gbs="sm_write_gbs",
    )
    def get_theoretical_num_sms(
        self,
        num_experts: int,
        num_topk: int,
        num_scaleout_topk: int = 0,
        rdma_gbs: float = 0,
        nvlink_gbs: float = 0,
        sm_read_gbs: float = 200,
        sm_write_gbs: float = 50,
    ) -> int:
        raise NotImplementedError("ElasticBuffer.get_theoretical_num_sms is declared but not implemented")

    get_theoretical_num_compute_units = get_theoretical_num_sms

    @accept_aliases(num_compute_units="num_sms")
    def get_theoretical_num_qps(self, num_sms: int) -> int:
        raise NotImplementedError("ElasticBuffer.get_theoretical_num_qps is declared but not implemented")

    # ------------------------------------------------------------------------------------------
    def _check_tensor(self, value, dtype, shape=None):
        runtime = self._runtime
        return (
            isinstance(value, torch.Tensor)
            and value.dtype == dtype
            and value.device == runtime.torch_device
            and value.is_contiguous()
            and not value.requires_grad
            and (shape is None or tuple(value.shape) == tuple(shape))
        )

    def _check_versions(self, handle):
        for name, version in handle._routing_versions.items():
            tensor = getattr(handle, name)
            if torch.is_inference(tensor) or (tensor.data_ptr(), tensor._version) != version:
                raise ValueError(f"Cached routing was modified: {name}")

    @accept_aliases(num_compute_units="num_sms", use_aligned_col_major_sf="use_tma_aligned_col_major_sf")
    def dispatch(
        self,
        x: Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]],
        topk_idx: Optional[torch.Tensor] = None,
        topk_weights: Optional[torch.Tensor] = None,
        cumulative_local_expert_recv_stats: Optional[torch.Tensor] = None,
        num_experts: Optional[int] = None,
        num_max_tokens_per_rank: Optional[int] = None,
        expert_alignment: Optional[int] = None,
        num_sms: int = 0,
        num_qps: int = 0,
        previous_event: Optional[EventHandle] = None,
        previous_event_before_epilogue: Optional[EventHandle] = None,
        async_with_compute_stream: bool = False,
        allocate_on_comm_stream: bool = False,
        handle: Optional[EPHandle] = None,
        do_handle_copy: bool = True,
        do_cpu_sync: Optional[bool] = None,
        do_expand: Optional[bool] = None,
        do_zero_padding: bool = False,
        use_tma_aligned_col_major_sf: bool = False,
    ):
        """Return ``(expanded_x | (expanded_x, scales), None, expanded_weights | None, handle, event)``.

        Rows are ordered (local expert, source rank, token, top-k slot); one row per valid slot;
        ids < 0 or >= num_experts produce no row; weights are moved, never applied.
        A fresh call computes the layout and reads the per-expert counts back to the host (one
        synchronisation); ``handle=`` reuses a previous plan with a new payload.
        """
        runtime = self._live_runtime()
        runtime.ensure_alive()
        native = runtime.native
        if runtime.combine_only:
            raise ValueError("Dispatch requires combine_only=False when constructing ElasticBuffer")
        if isinstance(handle, EPHandle) and handle.is_low_latency:
            raise NotImplementedError("Cached dispatch is not supported for LL handles")
        if handle is None:
            # Path selection as in the reference (elastic.py:710-746): small batches on EP16+ with weights and
            # default options prefer the low-latency path, decided from host metadata only.
            options = dict(
                do_handle_copy=do_handle_copy, do_cpu_sync=do_cpu_sync, do_expand=do_expand, expert_alignment=expert_alignment,
                num_sms=num_sms, num_qps=num_qps, cumulative_local_expert_recv_stats=cumulative_local_expert_recv_stats,
                previous_event=previous_event, previous_event_before_epilogue=previous_event_before_epilogue,
                async_with_compute_stream=async_with_compute_stream, allocate_on_comm_stream=allocate_on_comm_stream,
                do_zero_padding=do_zero_padding, use_tma_aligned_col_major_sf=use_tma_aligned_col_major_sf,
            )
            chosen = self._choose_low_latency(x, topk_idx, topk_weights, num_experts, num_max_tokens_per_rank, options)
            if chosen is not None:
                capacity, plan = chosen
                if runtime.capacity != LOW_LATENCY_WORKSPACE_BYTES:
                    raise ValueError(
                        "LL dispatch requires Buffer(num_bytes=8589934592), exactly 8 GiB; "
                        f"got {runtime.capacity} bytes for EP{runtime.world_size}"
                    )
                return self._dispatch_low_latency(x, topk_idx, topk_weights, num_experts, capacity, do_handle_copy, plan)
        with runtime.notify_lock:
            if runtime.notify_failed:
                raise RuntimeError("A previous communication launch failed; restart the distributed job")
            fp8_input = isinstance(x, tuple)
            hidden, scales = x if fp8_input and len(x) == 2 else (x, None)
            fuse_quant = self.use_fp8_dispatch and not fp8_input
            fp8 = fp8_input or fuse_quant
            extras_unused = (
                cumulative_local_expert_recv_stats is None and previous_event_before_epilogue is None
                and not allocate_on_comm_stream and not do_zero_padding and not use_tma_aligned_col_major_sf
            )
            _enforce(
                # options
                *((_is_bool(value), TypeError, f"{name} must be bool") for name, value in (
                    ("async_with_compute_stream", async_with_compute_stream),
                    ("allocate_on_comm_stream", allocate_on_comm_stream),
                    ("do_handle_copy", do_handle_copy),
                    ("do_zero_padding", do_zero_padding),
                    ("use_aligned_col_major_sf", use_tma_aligned_col_major_sf),
                )),
                (do_expand is None or do_expand is True, NotImplementedError, "Dispatch supports only the expanded expert layout"),
                (do_cpu_sync is None or _is_bool(do_cpu_sync), TypeError, "do_cpu_sync must be bool or None"),
                (handle is not None or do_cpu_sync is not False, NotImplementedError, "Fresh notify requires do_cpu_sync=None/True"),
                (expert_alignment is None or _int_among(expert_alignment, (1,)), NotImplementedError,
                 "Dispatch supports expert_alignment=1"),
                (extras_unused, NotImplementedError,
                 "Stats, epilogue events, padding and alternate allocation/scale layouts are unavailable"),
                (previous_event is None or (isinstance(previous_event, EventHandle) and previous_event._gpu_index == runtime.device),
                 ValueError, "previous_event must belong to the buffer GPU"),
                # payload
                (not fp8_input or len(x) == 2, ValueError, "FP8 input must be (hidden, scales)"),
                (lambda: self._check_tensor(hidden, torch.float8_e4m3fn if fp8_input else torch.bfloat16) and hidden.ndim == 2,
                 ValueError, "x must be contiguous BF16, or (FP8 E4M3FN, FP32 scales), on the buffer GPU without grad"),
            )
            tokens, width = hidden.shape
            _validate_hidden(width, fp8)
            _enforce(
                (not self.hidden or width == self.hidden, ValueError, "hidden differs from buffer configuration"),
                (lambda: not fp8_input or self._check_tensor(scales, torch.float32, (tokens, width // 128)), ValueError,
                 "FP8 scales must be contiguous FP32 [T,H/128] on the buffer GPU without grad"),
                (_int_among(num_sms, (0, 64 if fp8 else 32)), ValueError, "num_compute_units must be 0/32 for BF16 or 0/64 for FP8"),
                (_int_among(num_qps, (0, 2)), ValueError, "Primary dispatch uses two QPs per peer; num_qps=0/2"),
            )
            world = runtime.world_size
            if handle is not None:
                from_here = (
                    isinstance(handle, EPHandle) and handle._buffer_token is self._handle_token
                    and not handle.metadata_only and handle.metadata_version == 7
                )
                _enforce(
                    (from_here, ValueError, "Cached handle must come from this buffer's successful payload dispatch"),
                    (topk_idx is None, ValueError, "Cached dispatch inherits routing; omit topk_idx"),
                    (lambda: num_experts is None or num_experts == handle.num_experts, ValueError,
                     "num_experts differs from cached routing"),
                )
                self._check_versions(handle)
                num_experts, topk = handle.num_experts, handle.num_topk
                _enforce(
                    (tokens == handle.num_tokens, ValueError, "Cached dispatch requires the original token count"),
                    (width == handle.hidden, ValueError, "Cached dispatch requires the original hidden size"),
                )
            else:
                _enforce(
                    (lambda: self._check_tensor(topk_idx, torch.int64) and topk_idx.ndim == 2 and topk_idx.shape[0] == tokens,
                     ValueError, "topk_idx must be contiguous int64 [T,K] on the buffer GPU"),
                    (lambda: do_handle_copy or not torch.is_inference(topk_idx), ValueError,
                     "Inference routing tensors require do_handle_copy=True"),
                )
                topk = topk_idx.shape[1]
            _integer("tokens", tokens, 1, MAX_TOKENS * world)
            _integer("topk", topk, 1, MAX_TOPK)
            _integer("experts", num_experts, world, MAX_EXPERTS)
            bound = self.num_max_tokens_per_rank
            per_rank = -(-tokens // world)
            capacity = (bound or per_rank) if num_max_tokens_per_rank is None else num_max_tokens_per_rank
            _enforce((num_experts % world == 0, ValueError, "num_experts must be divisible by EP"))
            _integer("num_max_tokens_per_rank", capacity, per_rank, MAX_TOKENS)
            _enforce(
                (not bound or capacity <= bound, ValueError, "Input/capacity exceeds the buffer token bound"),
                (not self.num_topk or self.num_topk == topk, ValueError, "topk differs from buffer configuration"),
                (lambda: topk_weights is None or self._check_tensor(topk_weights, torch.float32, (tokens, topk)), ValueError,
                 "topk_weights must be contiguous FP32 [T,K] on the buffer GPU without grad"),
            )

            # ---- launch -----------------------------------------------------------------------
            try:
                with _Enqueue(runtime, previous_event, async_with_compute_stream) as queue:

                    def payload(rows):
                        if fuse_quant:
                            return native.dispatch_quant_fp8(hidden, topk_weights, route_to_row, row_to_route, rows)
                        return native.dispatch_copy(hidden, scales, topk_weights, route_to_row, row_to_route, rows)

                    if handle is None:
                        # Where most routes stay on this rank, outputs allocated for all T*K routes cost little, and
                        # the payload kernel can be queued right behind the layout: the host reads R while both
                        # run and narrows the outputs, instead of leaving the GPU idle between the two.  A small
                        # batch (a decode step) goes further: layout and payload are one launch.
                        early = 2 * (num_experts // world) >= num_experts
                        if early and 1 <= tokens * topk <= native.SMALL_BATCH_ROUTES:
                            local = num_experts // world
                            with torch.inference_mode(False), torch.no_grad():
                                indices = topk_idx.clone() if do_handle_copy else topk_idx
                                plan, *full = native.layout_dispatch_small(
                                    runtime.workspace, indices, hidden, scales, topk_weights, num_experts, runtime.rank * local,
                                    local, quantize=fuse_quant)
                            route_to_row, row_to_route = plan["route_to_row"], plan["row_to_route"]
                        else:
                            plan, indices = self._notify_launch(topk_idx, num_experts, do_handle_copy)
                            route_to_row, row_to_route = plan["route_to_row"], plan["row_to_route"]
                            full = payload(None) if early else None
                        handle = self._notify_finish(hidden, plan, indices, num_experts, capacity)
                        rows = handle.num_expanded_tokens
                        if early:
                            out, out_scales, out_weights = (None if t is None else t[:rows] for t in full)
                        else:
                            out, out_scales, out_weights = payload(rows)
                    else:
                        route_to_row, row_to_route = handle.route_to_row, handle._row_to_route_full
                        out, out_scales, out_weights = payload(handle.num_expanded_tokens)
                    retained = (hidden, scales, topk_weights, out, out_scales, out_weights, handle.topk_idx) + tuple(
                        getattr(handle, name) for name in _ROUTING
                    )
                    handle.metadata_only = False
                    handle.num_compute_units = 64 if fp8 else 32
                    handle._routing_versions = {
                        name: (getattr(handle, name).data_ptr(), getattr(handle, name)._version) for name in _ROUTING
                    }
                    event = queue.event(retained)
                runtime.notify_inflight = None
                return (out, out_scales) if fp8 else out, None, out_weights, handle, event
            except Exception:
                runtime.notify_failed = True
                raise

    # What each option of a fresh dispatch must be for the call to be eligible for the low-latency path
    # (deep_ep/backends/mesh_clos/elastic.py:710-746 decides the same from host metadata alone): a type the value must
    # have exactly (None: not checked), and the values accepted.
    _LOW_LATENCY_OPTIONS = {
        "do_handle_copy": (bool, (True, False)),
        "do_cpu_sync": (None, (None, True, False)),
        "do_expand": (None, (None, True)),
        "expert_alignment": (None, (None, 1)),
        "num_sms": (int, (0,)),
        "num_qps": (int, (0,)),
        "cumulative_local_expert_recv_stats": (None, (None,)),
        "previous_event": (None, (None,)),
        "previous_event_before_epilogue": (None, (None,)),
        "async_with_compute_stream": (None, (False,)),
        "allocate_on_comm_stream": (None, (False,)),
        "do_zero_padding": (None, (False,)),
        "use_tma_aligned_col_major_sf": (None, (False,)),
    }

    def _choose_low_latency(self, x, topk_idx, topk_weights, num_experts, num_max_tokens_per_rank, options):
        """(capacity, plan) when a fresh dispatch takes the low-latency path, else None."""
        payload = x[0] if isinstance(x, tuple) and len(x) == 2 else x
        if not isinstance(payload, torch.Tensor) or payload.ndim != 2:
            return None
        declared = self.num_max_tokens_per_rank
        if num_max_tokens_per_rank is not None:
            capacity = num_max_tokens_per_rank
        else:
            capacity = declared or -(-payload.shape[0] // self._live_runtime().world_size)
        if type(capacity) is not int or (declared and capacity > declared):
            return None
        for name, (exact_type, accepted) in self._LOW_LATENCY_OPTIONS.items():
            value = options[name]
            # identity or exact-type equality: 0 == False and 1 == True must not pass for each other
            if exact_type is not None and type(value) is not exact_type:
                return None
            if not any(value is good or (type(value) is type(good) and value == good) for good in accepted):
                return None
        plan = self._low_latency_plan(x, topk_idx, topk_weights, num_experts, capacity)
        return None if plan is None else (capacity, plan)

    def _low_latency_plan(self, x, topk_idx, topk_weights, num_experts, capacity):
        """Host-metadata check that selects the low-latency path (elastic.py:401-450); never reads routes.
        Returns the capacity layout's row count, or None when the call is not a low-latency one."""
        runtime = self._runtime
        hidden, scales = x if isinstance(x, tuple) and len(x) == 2 else (x, None)
        if not isinstance(hidden, torch.Tensor) or hidden.ndim != 2:
            return None
        tokens, width = hidden.shape
        per_rank = -(-tokens // runtime.world_size)
        if (
            type(capacity) is not int
            or not 0 < per_rank <= capacity <= LOW_LATENCY_MAX_TOKENS
            or runtime.world_size not in LOW_LATENCY_WORLD_SIZES
            or topk_weights is None
        ):
            return None
        if hidden.dtype not in (torch.bfloat16, torch.float16, torch.float8_e4m3fn):
            return None
        if self.use_fp8_dispatch and hidden.dtype != torch.float8_e4m3fn:
            return None  # quantising inside the dispatch kernel is a high-throughput feature of this build
        if not isinstance(topk_idx, torch.Tensor) or topk_idx.ndim != 2:
            return None
        topk = topk_idx.shape[1]
        if type(num_experts) is not int or num_experts < runtime.world_size or num_experts % runtime.world_size:
            return None
        if (self.hidden and width != self.hidden) or (self.num_topk and topk != self.num_topk):
            return None
        if width <= 0 or (width * hidden.element_size()) % 16 or not 1 <= topk <= 32 or num_experts > MAX_EXPERTS:
            return None
        if hidden.dtype == torch.float8_e4m3fn:
            if (
                not isinstance(scales, torch.Tensor)
                or scales.dtype not in (torch.int32, torch.float32)
                or tuple(scales.shape) != (tokens, (width + 127) // 128)
            ):
                return None
        elif scales is not None:
            return None
        for value, dtype, shape in (
            (hidden, hidden.dtype, (tokens, width)),
            (topk_idx, torch.int64, (tokens, topk)),
            (topk_weights, torch.float32, (tokens, topk)),
        ):
            if not self._check_tensor(value, dtype, shape):
                return None
        if scales is not None and not self._check_tensor(scales, scales.dtype):
            return None
        return {"capacity_rows": runtime.world_size * capacity * min(topk, num_experts // runtime.world_size)}

    def _dispatch_low_latency(self, x, topk_idx, topk_weights, num_experts, capacity, do_handle_copy, plan):
        """Low-latency dispatch (elastic.py:453-564; docs/elastic.md:85-125) for one rank's share: the capacity
        layout ``[C,H]`` with ``C = P*M*min(K, E/P)``, whose first R rows are the valid ones (expert-major), no host
        synchronisation, payload and scales moved bit for bit (BF16, FP16, or FP8 with FP32 / packed-E8M0 int32
        scales), and the route weights kept in the handle for the combine instead of being returned."""
        runtime = self._runtime
        native = runtime.native
        hidden, scales = x if isinstance(x, tuple) else (x, None)
        tokens, width = hidden.shape
        topk = topk_idx.shape[1]
        world = runtime.world_size
        local = num_experts // world
        begin = runtime.rank * local
        rows = plan["capacity_rows"]
        with runtime.notify_lock:
            if runtime.notify_failed:
                raise RuntimeError("A previous communication launch failed; restart the distributed job")
            try:
                with _Enqueue(runtime) as queue:
                    # The payload kernel does not depend on R.  Batches of up to SMALL_BATCH_ROUTES routes (every
                    # low-latency batch with the usual top-k) take one launch for layout and payload; larger ones
                    # queue the payload kernel right behind the layout.  (Experts repeated within a token are
                    # outside the low-latency contract; their surplus rows fall beyond C and are dropped from the
                    # returned view, never written out of bounds.)
                    with torch.inference_mode(False), torch.no_grad():
                        indices = topk_idx.clone() if do_handle_copy else topk_idx
                        if tokens * topk <= native.SMALL_BATCH_ROUTES:
                            layout, *moved = native.layout_dispatch_small(
                                runtime.workspace, indices, hidden, scales, topk_weights, num_experts, begin, local,
                                capacity_rows=rows)
                        else:
                            layout = native.layout(runtime.workspace, indices, num_experts, begin, local)
                            moved = native.dispatch_copy(
                                hidden, scales, topk_weights, layout["route_to_row"], layout["row_to_route"], None,
                                capacity_rows=rows)
                    out, out_scales, row_weights = (None if t is None else t[:rows] for t in moved)
                    # send_counts[e]: rows of experts 0..e on this rank (inclusive), so that its last entry is R
                    send_counts = torch.zeros((num_experts,), dtype=torch.int32, device=hidden.device)
                    send_counts[begin : begin + local] = layout["psum"]
                    send_counts[begin + local :] = layout["num_rows"]
                    handle = EPHandle(
                        True, num_experts, 1, capacity, 0, indices, world * capacity, rows, [], None, None, None, None,
                        None, None, None, is_low_latency=True,
                    )
                    handle.route_to_row = layout["route_to_row"]
                    handle.source_weights = row_weights
                    handle.send_counts = send_counts
                    handle.expert_recv_counts = None
                    handle.metadata_only = False
                    handle._buffer_token = self._handle_token
                    handle.rank, handle.world_size = runtime.rank, world
                    handle.num_tokens, handle.num_topk, handle.hidden = tokens, topk, width
                    retained = (hidden, scales, topk_weights, indices, out, out_scales, row_weights, send_counts,
                                layout["route_to_row"], layout["row_to_route"], layout["meta"])
                    event = queue.event(retained)
                runtime.notify_inflight = None
                return (out, out_scales) if scales is not None else out, None, None, handle, event
            except Exception:
                runtime.notify_failed = True
                raise

    def _combine_low_latency(self, x, handle, topk_weights, bias, num_sms, num_qps, previous_event,
                             previous_event_before_epilogue, async_with_compute_stream, allocate_on_comm_stream):
        """Low-latency combine (elastic.py:566-646): weights come from the handle, output has x's dtype."""
        runtime = self._runtime
        if handle._buffer_token is not self._handle_token or handle.metadata_only:
            raise ValueError("LL handle must come from this buffer's payload dispatch")
        if topk_weights is not None or bias is not None:
            raise NotImplementedError("LL combine takes its weights from the handle and does not support bias")
        if (
            type(num_sms) is not int
            or num_sms != 0
            or type(num_qps) is not int
            or num_qps != 0
            or previous_event is not None
            or previous_event_before_epilogue is not None
            or async_with_compute_stream is not False
            or allocate_on_comm_stream is not False
        ):
            raise NotImplementedError("LL combine supports default scheduling and stream options only")
        if not (
            isinstance(x, torch.Tensor)
            and x.dtype in (torch.bfloat16, torch.float16)
            and self._check_tensor(x, x.dtype, (handle.num_expanded_tokens, handle.hidden))
        ):
            raise ValueError("LL combine requires contiguous BF16/FP16 expert output matching its handle")
        with runtime.notify_lock:
            if runtime.notify_failed:
                raise RuntimeError("A previous communication launch failed; restart the distributed job")
            try:
                with _Enqueue(runtime) as queue:
                    output, _ = runtime.native.combine(x, handle.route_to_row, handle.source_weights, None)
                    event = queue.event((x, output, handle.route_to_row, handle.source_weights, handle.topk_idx))
                runtime.notify_inflight = None
                return output, None, event
            except Exception:
                runtime.notify_failed = True
                raise

    def _notify_launch(self, topk_idx, num_experts, do_handle_copy):
        """Queues the routing layout; returns its device outputs and the routing tensor it read."""
        runtime = self._runtime
        local = num_experts // runtime.world_size
        # Persistent routing keeps version counters even when the caller runs in inference mode.
        with torch.inference_mode(False), torch.no_grad():
            indices = topk_idx.clone() if do_handle_copy else topk_idx
            plan = runtime.native.layout(runtime.workspace, indices, num_experts, runtime.rank * local, local)
        return plan, indices

    def _notify_finish(self, hidden, plan, indices, num_experts, capacity) -> EPHandle:
        """The one host read-back (counts, R) that sizes the outputs, and the handle built from it."""
        runtime = self._runtime
        tokens, width = hidden.shape
        topk = indices.shape[1]
        local = num_experts // runtime.world_size
        # The single host synchronisation: the kernel reports counts and R through pinned host memory.
        counts, rows = runtime.native.layout_wait(runtime.workspace, local, 100.0)  # num_gpu_timeout_secs
        handle = EPHandle(
            True, num_experts, 1, capacity, 64, indices, None, rows, counts, None, plan["psum"], plan["counts"], None,
            None, None, None,
        )
        handle.route_to_row = plan["route_to_row"]
        handle._row_to_route_full = plan["row_to_route"]
        with torch.inference_mode(False), torch.no_grad():
            handle.weight_return_meta = plan["row_to_route"][:rows]
        handle.expert_totals = plan["counts"]
        handle.expert_offsets = plan["offsets"]
        handle.rank, handle.world_size = runtime.rank, runtime.world_size
        handle.num_tokens, handle.num_topk, handle.hidden = tokens, topk, width
        handle._buffer_token = self._handle_token
        return handle

    @accept_aliases(num_compute_units="num_sms")
    def combine(
        self,
        x: torch.Tensor,
        handle: EPHandle,
        topk_weights: Optional[torch.Tensor] = None,
        bias=None,
        num_sms: int = 0,
        num_qps: int = 0,
        previous_event: EventHandle = None,
        previous_event_before_epilogue: Optional[EventHandle] = None,
        async_with_compute_stream: bool = False,
        allocate_on_comm_stream: bool = False,
    ):
        """Return ``(out[T,H] bf16, out_weights[T,K] | None, event)``.

        High-throughput handles: unweighted fp32 sum of each token's expert rows in slot order, one
        rounding to BF16; ``topk_weights[R]`` travel on the separate return channel and come back as
        ``[T,K]`` with 0 in slots without a row.  Low-latency style handles (``is_low_latency``):
        the saved ``handle.source_weights`` multiply each row before the sum.
        """
        runtime = self._live_runtime()
        runtime.ensure_alive()
        native = runtime.native
        if isinstance(handle, EPHandle) and handle.is_low_latency and handle.send_counts is not None:
            return self._combine_low_latency(
                x, handle, topk_weights, bias, num_sms, num_qps, previous_event, previous_event_before_epilogue,
                async_with_compute_stream, allocate_on_comm_stream,
            )
        with runtime.notify_lock:
            if runtime.notify_failed:
                raise RuntimeError("A previous communication launch failed; restart the distributed job")
            from_here = (
                isinstance(handle, EPHandle) and handle._buffer_token is self._handle_token
                and not handle.metadata_only and handle.metadata_version == 7
            )
            _enforce(
                (_is_bool(async_with_compute_stream) and _is_bool(allocate_on_comm_stream), TypeError, "Stream options must be bool"),
                (bias is None, NotImplementedError, "Combine currently supports bias=None"),
                (previous_event_before_epilogue is None and not allocate_on_comm_stream, NotImplementedError,
                 "Epilogue events and allocate_on_comm_stream are unavailable"),
                (_int_among(num_sms, (0, 64)), ValueError, "Combine uses 64 compute units; num_compute_units=0/64"),
                (_int_among(num_qps, (0, 2)), ValueError, "Combine uses two QPs per cross sender; num_qps=0/2"),
                (previous_event is None or (isinstance(previous_event, EventHandle) and previous_event._gpu_index == runtime.device),
                 ValueError, "previous_event must belong to the buffer GPU"),
                (from_here, ValueError, "Combine needs this buffer's successful expanded payload dispatch handle"),
                (lambda: handle.do_expand and handle.expert_alignment == 1, ValueError, "Combine supports expanded layout without padding"),
                (lambda: handle.rank == runtime.rank and handle.world_size == runtime.world_size, ValueError,
                 "Handle topology differs from the buffer"),
            )
            self._check_versions(handle)
            rows = handle.num_expanded_tokens
            weighted = handle.is_low_latency
            _enforce(
                (lambda: self._check_tensor(x, torch.bfloat16, (rows, handle.hidden)), ValueError,
                 "x must be contiguous BF16 [num_expanded_tokens,H] matching the handle on the buffer GPU without grad"),
                (lambda: topk_weights is None or self._check_tensor(topk_weights, torch.float32, (rows,)), ValueError,
                 "topk_weights must be contiguous FP32 [num_expanded_tokens] on the buffer GPU without grad"),
                (not weighted or handle.source_weights is not None, ValueError, "Low-latency handle carries no saved route weights"),
            )
            try:
                with _Enqueue(runtime, previous_event, async_with_compute_stream) as queue:
                    output, output_weights = native.combine(
                        x, handle.route_to_row, handle.source_weights if weighted else None, topk_weights
                    )
                    event = queue.event((x, topk_weights, output, output_weights, handle.topk_idx) + tuple(
                        getattr(handle, name) for name in _ROUTING
                    ))
                runtime.notify_inflight = None
                return output, output_weights, event
            except Exception:
                runtime.notify_failed = True
                raise
