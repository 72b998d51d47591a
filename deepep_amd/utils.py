"""Tensor helpers with the reference's names (deep_ep/utils/math.py:45-79)."""

from __future__ import annotations

from typing import Tuple

import torch

from . import ops


def per_token_cast_to_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantise each group of 128 values to E4M3 with FP32 scales, on the GPU (HIP kernel).

    Bit-identical to the reference's torch expression on CPU.  ``x`` is a BF16 [T, H] GPU tensor of any width: a last
    block shorter than 128 is quantised as if padded with zeros, as in the reference (the kernel takes widths that
    are multiples of 16; other widths are padded to the next one here and the codes cut back to H)."""
    if x.dim() != 2:
        raise AssertionError("x must be a 2D tensor")
    hidden = x.shape[1]
    if hidden % 16 == 0 or hidden == 0:
        return ops.cast_to_fp8(x)
    codes, scales = ops.cast_to_fp8(torch.nn.functional.pad(x, (0, 16 - hidden % 16)))
    return codes[:, :hidden].contiguous(), scales


def per_token_cast_back(x_fp8: torch.Tensor, x_scales: torch.Tensor) -> torch.Tensor:
    """bf16(fp32(q) * scale) per block of 128 columns (deep_ep/utils/math.py:64-79); an int32 scale holds the e8m0
    exponent bytes of four consecutive blocks.  Device tensors go through the HIP kernel (``dpep_cast_back``); host
    tensors are evaluated with torch, as the reference does on any device."""
    if x_fp8.numel() == 0:
        return x_fp8.to(torch.bfloat16)
    if x_fp8.dim() != 2:
        raise AssertionError("x_fp8 must be a 2D tensor")
    tokens, hidden = x_fp8.shape
    blocks = (hidden + 127) // 128
    if x_fp8.is_cuda and hidden % 16 == 0 and (x_scales.dtype != torch.int or blocks % 4 == 0):
        from . import ops

        scales = x_scales.contiguous()
        scales = scales.view(tokens, -1) if scales.dtype == torch.int else scales.to(torch.float32).view(tokens, blocks)
        return ops.cast_back(x_fp8.contiguous(), scales)
    if x_scales.dtype == torch.int:
        x_scales = (x_scales.view(dtype=torch.uint8).to(torch.int) << 23).view(dtype=torch.float)
    padded = torch.nn.functional.pad(x_fp8.to(torch.float32), (0, blocks * 128 - hidden))
    values = padded.view(tokens, blocks, 128)
    return (values * x_scales.view(tokens, -1, 1)).view(tokens, blocks * 128).to(torch.bfloat16)[:, :hidden].contiguous()
