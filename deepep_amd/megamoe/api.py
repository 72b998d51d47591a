"""Inference-only MegaMoE API on one MI355X.

Signatures follow experiments/megamoe/python/deep_ep_experimental/megamoe/api.py (SymmBuffer :63-279,
transform_weights_for_mega_moe :311-379, mega_moe :382-413, fp8_fp4_mega_moe :520-567).  Deviations:

  * one process, one GPU.  ``group`` may be ``None`` / ``LocalGroup()`` (every expert is local) or
    ``LocalGroup(rank, world_size)``: the buffer then computes ONE rank's share of an EP job — it owns
    ``num_experts / world_size`` experts and its inputs hold the flattened tokens of all source ranks
    (capacity ``world_size * num_max_tokens_per_rank`` rows).  The reference needs 2..128 real ranks;
  * prepared weights are this library's fragment order (``dpep_megamoe_prepare_weights``), not Ascend NZ;
  * FP8xFP8 weights are not built.  hidden (multiples of 64) and intermediate_hidden (multiples of 128, from 256)
    have the reference's limits; sizes that are not multiples of 256, and 256 itself, run padded to the next
    one (at least 512): the weights when they are prepared, the input rows by a copy inside the forward;
  * shared experts run as extra experts that take every token (weight 1, added after the routed ones).
"""

from __future__ import annotations

import threading
import warnings

import torch

from .. import ops
from .validation import check_routing

SMALL_BATCH_MAX_TOKENS = 256
API_PROTOCOL = 4


def _integer(name, value, lower, upper):
    if type(value) is not int or not lower <= value <= upper:
        raise ValueError(f"{name} must be an integer in [{lower}, {upper}]")


class LocalGroup:
    """Single-process stand-in for the reference's StoreGroup (deep_ep/_store.py:16-60): an identity
    (rank, world_size) without any transport."""

    def __init__(self, rank: int = 0, world_size: int = 1):
        _integer("world_size", world_size, 1, 128)
        _integer("rank", rank, 0, world_size - 1)
        self._rank, self._size = rank, world_size

    def size(self) -> int:
        return self._size

    def rank(self) -> int:
        return self._rank


class StoreGroup(LocalGroup):
    """The name the reference's examples construct their group with (deep_ep/_store.py:16-60, ``StoreGroup.from_env()``).
    Here it is the identity alone: rank and size come from the launcher's environment, no store is contacted, and the
    calls that coordinate processes answer for this process (one process per GPU, no transport between them)."""

    @classmethod
    def from_env(cls, timeout=300):
        import os

        _integer("timeout", timeout, 1, 86400)
        return cls(int(os.environ.get("RANK", "0")), int(os.environ.get("WORLD_SIZE", "1")))

    def barrier(self, stage=""):
        return None

    def all_gather(self, value, stage):
        if self._size != 1:
            raise NotImplementedError("This build has no transport between processes: all_gather needs a single-rank group")
        return [value]

    def abort(self, error):
        return None

    def close(self):
        return None


def _pair(value, name):
    if not isinstance(value, tuple) or len(value) != 2:
        raise TypeError(f"{name} must be (quantized_data, E8M0_scales)")
    return value


class _PreparedPair(tuple):
    """(weights, scales) in the kernel's streaming order; immutable after preparation."""

    def __new__(cls, weight, scale, gate_up, logical):
        value = super().__new__(cls, (weight, scale))
        value.gate_up = gate_up
        value.logical = tuple(logical)  # (experts, N, K) of the raw tensor; the prepared one may be padded
        value._versions = (weight._version, scale._version)
        return value

    def checked(self):
        if (self[0]._version, self[1]._version) != self._versions:
            raise ValueError("Prepared weights/scales were modified in-place; transform raw ND weights again")
        return self[0], self[1]


class SymmBuffer:
    """Owner of the workspace and the input tensors of one rank.  One in-flight call per buffer."""

    def __init__(
        self,
        group,
        num_experts: int,
        num_max_tokens_per_rank: int,
        num_topk: int,
        hidden: int,
        intermediate_hidden: int,
        num_shared_experts: int = 0,
        mma_type: str = "fp8xfp4",
        activation: str = "swiglu",
        *,
        ranks_per_node: int = 0,
        timeout: int = 120,
    ):
        if group is None:
            group = LocalGroup()
        if not isinstance(group, LocalGroup):
            raise TypeError("Pass a LocalGroup (this build has no multi-process transport)")
        size = group.size()
        _integer("num_experts", num_experts, 1, 16384)
        _integer("num_max_tokens_per_rank", num_max_tokens_per_rank, 1, 65536)
        _integer("num_topk", num_topk, 1, min(32, num_experts))
        _integer("hidden", hidden, 1024, 8192)
        _integer("intermediate_hidden", intermediate_hidden, 256, 4096)
        _integer("num_shared_experts", num_shared_experts, 0, 8)
        _integer("ranks_per_node", ranks_per_node, 0, size)
        _integer("timeout", timeout, 1, 300)
        if hidden % 64 or intermediate_hidden % 128:
            raise ValueError("hidden must be divisible by 64; intermediate_hidden by 128")
        if activation != "swiglu" or mma_type not in {"fp8xfp4", "fp8xfp8"}:
            raise ValueError("Only SwiGLU with FP8xFP4/FP8xFP8 is implemented; no BF16xBF16")
        if mma_type != "fp8xfp4":
            raise NotImplementedError("This build implements FP8xFP4 (W4A8) weights only")
        if num_topk + num_shared_experts > 32:
            raise ValueError("num_topk + num_shared_experts must not exceed 32 in this build")
        if num_experts % size or num_experts // size > 128:
            raise ValueError("Experts must divide EP, with at most 128 local experts")
        if ranks_per_node and size % ranks_per_node:
            raise ValueError("ranks_per_node must divide EP (contiguous node-major ranks)")
        self._lock = threading.Lock()
        self._device = torch.device("cuda", torch.cuda.current_device())
        self.group, self.num_experts = group, num_experts
        self.num_max_tokens_per_rank, self.num_topk = num_max_tokens_per_rank, num_topk
        self.hidden, self.intermediate_hidden = hidden, intermediate_hidden
        self.num_shared_experts, self.mma_type = num_shared_experts, mma_type
        self.ranks_per_node = ranks_per_node
        self.num_local_experts = num_experts // size
        self.capacity_tokens = size * num_max_tokens_per_rank
        self.x = self.x_sf = self.topk_idx = self.topk_weights = None
        self._workspace = None
        self._plan_bs = None
        self._closed = False
        self._last_stream = None  # the stream the most recent call was queued on
        self.allocate_inputs()

    # -- lifetime ----------------------------------------------------------------------------------
    def _ensure_alive(self):
        if self._closed:
            raise RuntimeError("SymmBuffer was destroyed")

    def allocate_inputs(self):
        """Idempotent: the constructor already allocated x, x_sf, topk_idx, topk_weights."""
        self._ensure_alive()
        if self.x is not None:
            return self
        rows = self.capacity_tokens
        self.x = torch.empty((rows, self.hidden), dtype=torch.float8_e4m3fn, device=self._device)
        self.x_sf = torch.empty((rows, self.hidden // 32), dtype=torch.float8_e8m0fnu, device=self._device)
        self.topk_idx = torch.empty((rows, self.num_topk), dtype=torch.int32, device=self._device)
        self.topk_weights = torch.empty((rows, self.num_topk), dtype=torch.float32, device=self._device)
        return self

    def _prepare(self, bs):
        _integer("BS", bs, 1, self.capacity_tokens)
        if self._plan_bs == bs:
            return
        # keep only the current BS's worst-case workspace
        if self._workspace is not None:
            self._workspace.destroy()
            self._workspace = None
        need = ops.megamoe_workspace_bytes(bs, self.num_topk, self.hidden, self.intermediate_hidden, self.num_local_experts,
                                           self.num_shared_experts)
        self._workspace = ops.Workspace(need, self._device)
        self._plan_bs = bs

    def prepare(self, bs: int) -> "SymmBuffer":
        """Build or reuse the plan (workspace) of one batch size, outside the timed path."""
        with self._lock:
            self._ensure_alive()
            self._prepare(bs)
        return self

    @property
    def workspace_bytes(self) -> int:
        return self._workspace.num_bytes if self._workspace is not None else 0

    @property
    def symmetric_buffer_bytes(self) -> int:
        return 0  # no symmetric heap on one GPU

    @property
    def timer_enabled(self) -> bool:
        return False

    def allocate_timer(self):
        self._ensure_alive()
        raise RuntimeError("W4A8 timer requires DEEPEP_MEGAMOE_TIMER=ON (device timers are not built; use rocprofv3)")

    def validate_inputs(self, bs: int, *, x=None) -> None:
        """Synchronising routing scan; run after filling the inputs, outside timing."""
        self._ensure_alive()
        _integer("BS", bs, 1, self.capacity_tokens)
        for name, tensor, dtype, shape in (
            ("topk_idx", self.topk_idx, torch.int32, (self.capacity_tokens, self.num_topk)),
            ("topk_weights", self.topk_weights, torch.float32, (self.capacity_tokens, self.num_topk)),
        ):
            if tensor.device != self._device or tensor.dtype != dtype or tuple(tensor.shape) != shape:
                raise ValueError(f"{name} must retain its buffer dtype/device/shape")
        if x is not None and (x.dtype != torch.bfloat16 or x.device != self._device or tuple(x.shape) != (bs, self.hidden)):
            raise ValueError("x override must be BF16 [BS,H] on the buffer device")
        check_routing(
            self.topk_idx[:bs].cpu().tolist(), self.topk_weights[:bs].cpu().tolist(), self.num_experts, self.num_topk,
            self.group.rank(),
        )

    def destroy(self):
        with self._lock:
            if self._closed:
                return
            if self._last_stream is not None:
                self._last_stream.synchronize()
            if self._workspace is not None:
                self._workspace.destroy()
            self._workspace = self._plan_bs = None
            self.x = self.x_sf = self.topk_idx = self.topk_weights = None
            self._closed = True

    def __del__(self):
        if not getattr(self, "_closed", True):
            warnings.warn("SymmBuffer was not destroyed explicitly; call destroy()", ResourceWarning)


def transform_weights_for_mega_moe(l1_weights, l2_weights, activation: str = "swiglu", *, shared: bool = False):
    """Re-lay raw packed weights once, without quantising again.

    Raw inputs: packed FP4 int8/uint8 ``[E, N, K/2]`` (low nibble = even k; GMM1 rows are gate then up)
    and E8M0 scales ``[E, N, K/64, 2]`` (uint8 / float8_e8m0fnu) or packed int32 ``[E, N, K/128]``.
    Returns ``((w1, s1), (w2, s2))`` in the kernel's order; keep the pairs intact and unmodified.
    """
    if activation != "swiglu":
        raise NotImplementedError("Only SwiGLU is supported")
    # shared=True: the weights of shared experts; this build lays them out exactly like routed ones.
    prepared = []
    for name, value, gate_up in (("l1_weights", l1_weights, True), ("l2_weights", l2_weights, False)):
        weight, scale = _pair(value, name)
        if isinstance(value, _PreparedPair):
            raise ValueError(f"{name}: prepare from raw ND weights, not already prepared weights")
        if not weight.is_cuda or scale.device != weight.device:
            raise ValueError("Move weights and scales to the same GPU before preparing")
        if weight.ndim != 3:
            raise ValueError(f"{name}: weights must be packed [E,N,K/2]")
        if weight.dtype == torch.int8:
            weight = weight.view(torch.uint8)  # reinterpret the FP4 bit patterns
        if weight.dtype != torch.uint8:
            raise TypeError("Weights must be packed FP4 int8/uint8")
        k = weight.shape[-1] * 2
        if k % 64:
            raise ValueError(f"{name}: K must be divisible by 64")
        expected = (*weight.shape[:2], k // 64, 2)
        if scale.dtype == torch.int32 and tuple(scale.shape) == (*weight.shape[:2], k // 128) and k % 128 == 0:
            scale = scale.contiguous().view(torch.uint8).reshape(expected)
        if scale.dtype == torch.float8_e8m0fnu:
            scale = scale.view(torch.uint8)
        if scale.dtype != torch.uint8 or tuple(scale.shape) != expected:
            raise ValueError(f"{name}: expected E8M0 scales {expected} or raw packed int32 [E,N,K/128]")
        if gate_up and weight.shape[1] % 256:
            raise ValueError("Routed FP4 GMM1 requires gate/up widths divisible by 128")
        with torch.inference_mode(False):
            out_w, out_s = ops.megamoe_prepare_weights(
                weight.contiguous(), scale.contiguous().reshape(*weight.shape[:2], k // 32), gate_up
            )
        prepared.append(_PreparedPair(out_w, out_s, gate_up, (weight.shape[0], weight.shape[1], k)))
    return tuple(prepared)


def _overlaps(a, b):
    a0, a1 = a.data_ptr(), a.data_ptr() + a.numel() * a.element_size()
    b0, b1 = b.data_ptr(), b.data_ptr() + b.numel() * b.element_size()
    return a0 < b1 and b0 < a1


def _run(x, topk_idx, topk_weights, l1_weights, l2_weights, sym_buffer, *, shared_l1_weights=None,
         shared_l2_weights=None, out=None, timer=None, cumulative_stats=None):
    if not isinstance(sym_buffer, SymmBuffer):
        raise TypeError("sym_buffer must be this installation's MegaMoE SymmBuffer")
    data, scales = _pair(x, "x") if isinstance(x, tuple) else (x, None)
    if (shared_l1_weights is None) != (shared_l2_weights is None):
        raise ValueError("Supply both shared weight pairs, or neither")
    if timer is not None:
        raise RuntimeError("W4A8 timer requires DEEPEP_MEGAMOE_TIMER=ON (device timers are not built; use rocprofv3)")
    b = sym_buffer
    b._ensure_alive()
    if not isinstance(l1_weights, _PreparedPair) or not isinstance(l2_weights, _PreparedPair):
        raise ValueError(
            "MegaMoE requires prepared weights; call transform_weights_for_mega_moe on raw ND weights "
            "and keep its returned pairs intact"
        )
    if not l1_weights.gate_up or l2_weights.gate_up:
        raise ValueError("l1_weights / l2_weights are swapped")
    w1, s1 = l1_weights.checked()
    w2, s2 = l2_weights.checked()
    shared = None
    if shared_l1_weights is not None:
        if not isinstance(shared_l1_weights, _PreparedPair) or not isinstance(shared_l2_weights, _PreparedPair):
            raise ValueError("Shared weights must come from transform_weights_for_mega_moe(..., shared=True)")
        if not shared_l1_weights.gate_up or shared_l2_weights.gate_up:
            raise ValueError("shared_l1_weights / shared_l2_weights are swapped")
        shared = (*shared_l1_weights.checked(), *shared_l2_weights.checked())
    if (shared[0].shape[0] if shared is not None else 0) != sym_buffer.num_shared_experts:
        raise ValueError("Shared expert count does not match the buffer configuration")
    if data.ndim != 2 or not 0 < data.shape[0] <= b.capacity_tokens or data.shape[1] != b.hidden:
        raise ValueError("x must be nonempty [BS,H] within the buffer capacity")
    if data.device != b._device:
        raise ValueError("x must be on the buffer's creating device")
    bs = data.shape[0]
    if (l1_weights.logical != (b.num_local_experts, b.intermediate_hidden * 2, b.hidden)
            or l2_weights.logical != (b.num_local_experts, b.hidden, b.intermediate_hidden)
            or tuple(topk_idx.shape) != (bs, b.num_topk)):
        raise ValueError("Weight/routing shapes do not match the buffer configuration")
    if topk_idx.dtype != torch.int32:
        raise TypeError("topk_idx must be int32; convert explicitly before timing")
    if scales is None and data.dtype != torch.bfloat16:
        raise TypeError("x must be BF16, or an (FP8 E4M3, E8M0) pair")
    if scales is not None and (data.dtype != torch.float8_e4m3fn or scales.dtype not in (torch.float8_e8m0fnu, torch.uint8)):
        raise TypeError("x pair must be (FP8 E4M3 [BS,H], E8M0 [BS,H/32])")
    tensors = [t for t in (data, scales, topk_idx, topk_weights, w1, s1, w2, s2, *(shared or ())) if t is not None]
    if any(t.requires_grad for t in tensors) or (out is not None and out.requires_grad):
        raise NotImplementedError("MegaMoE is inference-only")
    if out is not None:
        if out.dtype != torch.bfloat16 or tuple(out.shape) != (bs, b.hidden) or out.device != b._device or not out.is_contiguous():
            raise ValueError("out must be contiguous BF16 [BS,H] on the buffer device")
        for tensor in tensors:
            if out.data_ptr() == tensor.data_ptr():
                raise ValueError("out must not alias any input storage")
            if _overlaps(out, tensor):
                raise ValueError("out must not overlap any input storage")
    if cumulative_stats is not None:
        stats = cumulative_stats
        if (stats.dtype != torch.int32 or tuple(stats.shape) != (b.num_local_experts,) or stats.device != b._device
                or not stats.is_contiguous()):
            raise ValueError("Cumulative stats must be contiguous local-expert int32 on the buffer device")
        for tensor in tensors + ([out] if out is not None else []):
            if _overlaps(stats, tensor):
                raise ValueError("Cumulative stats must not alias inputs, output or timer")
    with b._lock:
        b._ensure_alive()
        # The call is queued on the caller's current stream (every call is synchronous with it: the reference makes the
        # caller wait for its own stream before it returns).  Calls of one owner share its workspace, so a call that
        # arrives on another stream than the previous one waits for that stream first.
        caller = torch.cuda.current_stream(b._device)
        if b._last_stream is not None and b._last_stream != caller:
            caller.wait_stream(b._last_stream)
        b._last_stream = caller
        b._prepare(bs)
        if scales is None:
            data, scales = ops.mx_quant(data.contiguous())  # BF16 override: quantised here, not a BF16 GEMM
        if scales.dtype != torch.uint8:
            scales = scales.view(torch.uint8)
        y = out if out is not None else torch.empty((bs, b.hidden), dtype=torch.bfloat16, device=b._device)
        counts = torch.empty((b.num_local_experts,), dtype=torch.int32, device=b._device)
        ops.megamoe_forward(
            b._workspace, data.contiguous(), scales.contiguous(), topk_idx.contiguous(), topk_weights.contiguous(),
            w1, s1, w2, s2, b.num_experts, b.group.rank() * b.num_local_experts, b.num_local_experts, y, counts,
            shared=shared, intermediate=b.intermediate_hidden,
        )
        if cumulative_stats is not None:
            cumulative_stats.add_(counts)
        return y, counts


def mega_moe(x, topk_idx, topk_weights, l1_weights, l2_weights, sym_buffer, *, shared_l1_weights=None,
             shared_l2_weights=None, out=None, timer=None):
    """Explicit-input convenience API.  x: BF16 [B,H], or (FP8 E4M3 [B,H], E8M0 [B,H/32]).
    Returns (y BF16 [B,H], per-call local expert counts int32 [L])."""
    return _run(x, topk_idx, topk_weights, l1_weights, l2_weights, sym_buffer, shared_l1_weights=shared_l1_weights,
                shared_l2_weights=shared_l2_weights, out=out, timer=timer)


def fp8_fp4_mega_moe(y, l1_weights, l2_weights, sym_buffer, shared_l1_weights=None, shared_l2_weights=None,
                     cumulative_local_expert_recv_stats=None, recipe=(1, 1, 32), activation="swiglu",
                     activation_clamp=None, fast_math=True, *, x=None, timer=None) -> None:
    """Write BF16 y in place and return None; add the per-call counts to the stats tensor if given.

    Inputs are the buffer's own x / x_sf / topk_idx / topk_weights (first y.shape[0] rows); ``x=`` is an
    optional BF16 [BS,H] override that is MX-quantised internally.  Route weights are applied after GMM2.
    """
    fixed = {"recipe": (recipe, (1, 1, 32)), "activation": (activation, "swiglu"), "activation_clamp": (activation_clamp, None)}
    if fast_math is not True or any(given != only for given, only in fixed.values()):
        raise NotImplementedError("Supports recipe=(1,1,32), SwiGLU, no clamp, default math only")
    if not isinstance(sym_buffer, SymmBuffer):
        raise TypeError("sym_buffer must be this installation's MegaMoE SymmBuffer")
    sym_buffer._ensure_alive()
    if not (y.ndim == 2 and y.dtype == torch.bfloat16):
        raise ValueError("y must be BF16 [BS,H]")
    batch = y.shape[0]
    if x is None:
        # the buffer's own staging tensors, as many rows as y has
        activations = (sym_buffer.x[:batch], sym_buffer.x_sf[:batch])
    elif x.dtype == torch.bfloat16 and tuple(x.shape) == (batch, sym_buffer.hidden):
        activations = x
    else:
        raise ValueError("x override must be BF16 [BS,H]; omit x for buffered FP8 input")
    shared = dict(shared_l1_weights=shared_l1_weights, shared_l2_weights=shared_l2_weights)
    _run(activations, sym_buffer.topk_idx[:batch], sym_buffer.topk_weights[:batch], l1_weights, l2_weights, sym_buffer,
         out=y, timer=timer, cumulative_stats=cumulative_local_expert_recv_stats, **shared)
