"""FP8 all-gather of sharded weights: the two hooks of the FSDP extension protocol.

hyper_parallel's torch fully_shard looks for `fsdp_pre_all_gather` / `fsdp_post_all_gather` on the
sharded inner tensor (hyper_parallel/platform/torch/fully_shard/param.py:299-310) and carries their
metadata in `ExtensionsData` (hyper_parallel/core/fully_shard/hsdp_utils.py:127-146); it ships no
implementation of them.  With the two functions below a rank quantizes its weight shard once,
the collective moves 1 byte per element plus the block scales instead of 2 bytes, and the gathered
codes are used by `fp8_linear(..., weight_fp8=...)` as they are -- no second quantization.

Shards are slices of dim 0 (FSDP's sharding).  A shard must hold whole 128x128 blocks: its row
count is a multiple of 128.

`Fp8ShardedWeight` is the tensor type that carries the two hooks as METHODS, which is what the reference
probes for (`hasattr(inner_tensor, "fsdp_pre_all_gather")`): wrap a sharded bf16 weight in it and the
extension is detected.  The method signatures are those of the protocol the reference's ExtensionsData
was written for (torch FSDP2's all-gather extensions): `fsdp_pre_all_gather(mesh, outer_size, outer_stride,
module, mp_policy) -> (all_gather_inputs, metadata)` and `fsdp_post_all_gather(all_gather_outputs, metadata,
param_dtype, *, out=None) -> (unsharded_tensor, inner_tensors)`, or None when `out` is given.
"""
from __future__ import annotations

from typing import Any, Optional, Sequence, Tuple

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


class Fp8GatheredWeight(torch.Tensor):
    """The unsharded weight as the post-all-gather hook returns it: a tensor whose elements are the gathered E4M3
    codes [N, K] (a view of the all-gather output, no copy) and which carries the block scales and, made on first
    use, the transposed codes for dgrad.  `fp8_linear(x, w_bf16, weight_fp8=gathered.as_fp8_weight())` consumes it
    without quantizing anything again."""

    @staticmethod
    def __new__(cls, codes: torch.Tensor, scale_inv: torch.Tensor, pow2: bool = False):
        t = torch.Tensor._make_subclass(cls, codes, False)
        t.scale_inv = scale_inv
        t.pow2 = bool(pow2)
        t._codes_t = None
        return t

    __torch_function__ = torch._C._disabled_torch_function_impl     # ops on it see a plain float8 tensor

    def as_fp8_weight(self, with_transpose: bool = True) -> Fp8Weight:
        codes = self.as_subclass(torch.Tensor)
        if with_transpose and self._codes_t is None:
            self._codes_t = ops.transpose_codes(codes)
        return Fp8Weight(codes, self.scale_inv, self._codes_t if with_transpose else None, self.pow2)

    def refresh(self) -> None:
        """The all-gather wrote new codes into the buffer this tensor views: drop what was derived from the old ones."""
        self._codes_t = None


class Fp8ShardedWeight(torch.Tensor):
    """A rank's bf16 weight shard [N/S, K] that all-gathers as E4M3 codes plus 128x128 block scales.

    It is an ordinary bf16 tensor for every operator (optimizers, state dicts, arithmetic) and in addition has the
    two methods the reference's fully_shard looks for on the sharded inner tensor
    (hyper_parallel/platform/torch/fully_shard/param.py:299-310); their metadata travels in the reference's
    `ExtensionsData.all_gather_metadata` (hyper_parallel/core/fully_shard/hsdp_utils.py:127-146)."""

    @staticmethod
    def __new__(cls, shard: torch.Tensor, pow2: bool = False):
        if shard.dim() != 2 or shard.dtype != torch.bfloat16:
            raise TypeError("the shard must be a 2-D bfloat16 tensor")
        if shard.shape[0] % ops.BLOCK or shard.shape[1] % ops.BLOCK:
            raise ValueError("a shard must hold whole 128x128 blocks: both of its dims must be multiples of 128")
        t = torch.Tensor._make_subclass(cls, shard, shard.requires_grad)
        t.pow2 = bool(pow2)
        return t

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        """Every operator sees and returns plain tensors, except `detach`, which keeps the type (and the recipe
        flag): that is what lets an instance be wrapped in `torch.nn.Parameter`."""
        with torch._C.DisableTorchFunctionSubclass():
            out = func(*args, **(kwargs or {}))
        if func is torch.Tensor.detach and isinstance(out, torch.Tensor) and isinstance(args[0], cls):
            out = out.as_subclass(cls)
            out.pow2 = args[0].pow2
        return out

    def fsdp_pre_all_gather(self, mesh=None, outer_size=None, outer_stride=None, module=None, mp_policy=None):
        """-> ((codes uint8 [N/S, K], scale_inv fp32 [N/S/128, K/128]), metadata): the all-gather inputs (1 byte per
        element plus the scales instead of 2 bytes).  The positional arguments are the protocol's and are not needed
        here: the shard's own shape says everything."""
        return fsdp_pre_all_gather(self.as_subclass(torch.Tensor), pow2=self.pow2)

    def fsdp_post_all_gather(self, all_gather_outputs: Sequence[torch.Tensor], metadata: Any,
                             param_dtype: Optional[torch.dtype] = None, *, out: Optional[torch.Tensor] = None):
        """-> (Fp8GatheredWeight, the all-gather outputs it views).  With `out` (the tensor a previous call returned,
        whose storage the collective has just refilled) nothing is rebuilt: its derived transposed codes are
        dropped and None is returned, as the protocol asks."""
        if out is not None:
            if not isinstance(out, Fp8GatheredWeight):
                raise TypeError("out must be the Fp8GatheredWeight a previous call returned")
            out.refresh()
            return None
        f8 = fsdp_post_all_gather(all_gather_outputs, metadata, with_transpose=False)
        return Fp8GatheredWeight(f8.codes, f8.scale_inv, f8.pow2), tuple(all_gather_outputs)
