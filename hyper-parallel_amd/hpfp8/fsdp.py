"""FP8 all-gather of sharded weights: the two hooks of the FSDP extension protocol.

hyper_parallel's torch fully_shard looks for `fsdp_pre_all_gather` / `fsdp_post_all_gather` on the
sharded inner tensor (hyper_parallel/platform/torch/fully_shard/param.py:299-310) and carries their
metadata in `ExtensionsData` (hyper_parallel/core/fully_shard/hsdp_utils.py:127-146); it ships no
implementation of them.  With the two functions below a rank quantizes its weight shard once,
the collective moves 1 byte per element plus the block scales instead of 2 bytes, and the gathered
codes are used by `fp8_linear(..., weight_fp8=...)` as they are -- no second quantization.

Shards are slices of dim 0 (FSDP's sharding).  A shard must hold whole 128x128 blocks: its row
count is a multiple of 128.
"""
from __future__ import annotations

from typing import Any, Sequence, Tuple

import torch

from . import ops
from .linear import Fp8Weight


def fsdp_pre_all_gather(weight_shard: torch.Tensor, pow2: bool = False) -> Tuple[Tuple[torch.Tensor, torch.Tensor], Any]:
    """bf16 shard [N/S, K] -> ((codes as uint8 [N/S, K], scale_inv fp32 [N/S/128, K/128]), metadata).

    The two tensors are the all-gather inputs (uint8 rather than float8 so that any collective
    backend accepts them); metadata carries what the post hook needs to rebuild the shapes."""
    if weight_shard.dim() != 2:
        raise ValueError("weight shard must be 2-D")
    codes, scale_inv = ops.quantize_128x128(weight_shard.contiguous(), pow2=pow2)
    return (codes.view(torch.uint8), scale_inv), {"k": weight_shard.shape[1], "pow2": bool(pow2)}


def fsdp_post_all_gather(all_gather_outputs: Sequence[torch.Tensor], metadata: Any, *,
                         with_transpose: bool = True) -> Fp8Weight:
    """Gathered buffers (dim-0 concatenation of every rank's codes and of every rank's scales, flat or
    2-D) -> the unsharded weight's FP8 form.  The transposed codes for dgrad are a byte transpose of the
    gathered codes (128x128 blocks are symmetric)."""
    codes_u8, scale_inv = all_gather_outputs
    k = int(metadata["k"])
    codes = codes_u8.reshape(-1, k).view(ops.FP8)
    scale_inv = scale_inv.reshape(-1, k // ops.BLOCK)
    if codes.shape[0] != scale_inv.shape[0] * ops.BLOCK:
        raise ValueError("gathered codes and scales do not belong together")
    codes_t = ops.transpose_codes(codes) if with_transpose else None
    return Fp8Weight(codes, scale_inv, codes_t, bool(metadata.get("pow2", False)))
