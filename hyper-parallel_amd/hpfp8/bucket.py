"""FP8 form of the flat gradient bucket.

The reference packs gradients into one flat contiguous buffer, casts it to `reduce_dtype`, reduces
it, casts it back and multiplies by `grad_scale` (hyper_parallel/core/hsdp/hsdp_grad_buffer.py:95-108
and :116-135).  An E4M3 bucket needs a side buffer of scales, so it cannot be expressed as that
single dtype cast; these two functions are the cast-in and cast-back for it.
"""
from __future__ import annotations

import torch

from . import ops


def quantize_bucket(flat: torch.Tensor):
    """flat bf16 [numel] (numel % 128 == 0) -> (codes e4m3 [numel], scale_inv fp32 [numel/128])."""
    if flat.dim() != 1:
        raise ValueError("the bucket must be 1-D")
    if flat.numel() % ops.BLOCK:
        raise ValueError(f"bucket numel {flat.numel()} is not a multiple of {ops.BLOCK}")
    q, scale_inv = ops.quantize_1x128(flat.view(-1, ops.BLOCK))
    return q.view(-1), scale_inv.view(-1)


def dequantize_bucket(codes: torch.Tensor, scale_inv: torch.Tensor, grad_scale: float = 1.0) -> torch.Tensor:
    """Inverse of quantize_bucket: bf16 [numel]; `grad_scale` is applied after the cast back, on the
    bf16 values, as the reference does."""
    if codes.dim() != 1 or codes.numel() % ops.BLOCK:
        raise ValueError("codes must be 1-D with numel a multiple of 128")
    return ops.dequantize_1x128(codes.view(-1, ops.BLOCK), scale_inv.view(-1, 1), grad_scale).view(-1)
