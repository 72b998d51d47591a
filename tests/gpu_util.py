"""Helpers shared by the GPU parity tests (torch <-> numpy bit views)."""

import numpy as np
import torch


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def fp8_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


def f32_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().numpy().view(np.uint32)


def bits_to_bf16(bits: np.ndarray, device="cuda") -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16).to(device)


def i32(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().numpy()


def non_finite_blocks() -> torch.Tensor:
    """BF16 [16, 256] (two 128-column blocks per row) whose blocks hold, besides ordinary values: +inf, -inf, a NaN, a
    negative NaN, a whole block of NaN, inf and NaN together, the largest finite magnitudes, only zeros, -0 and values
    below the amax floor."""
    rng = np.random.default_rng(0)
    x = torch.from_numpy(rng.normal(size=(16, 256)).astype(np.float32)).bfloat16()
    x[1, 3] = float("inf")
    x[2, 130] = float("-inf")
    x[3, 7] = float("nan")
    x[4, :128] = 0
    x[5, :] = 0
    x[6, 5] = 1e38
    x[7, 9] = -3.3895e38
    x[8, :] = 1e-40
    x[9, 0] = -0.0
    x[10, :128] = float("nan")
    x[11, 1] = float("inf")
    x[11, 2] = float("nan")
    x[12, 4] = -float("nan")
    x[13, 255] = float("nan")
    return x
