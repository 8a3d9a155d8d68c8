"""The reference's mixed-precision record and dtype-cast hook, extended to an FP8 target.

`MixedPrecisionPolicy` (hyper_parallel/platform/torch/fully_shard/utils.py:8-24) names the dtypes of
parameters, gradient reduction and outputs; `TorchPlatform.cast_fp_tensor(dtype, x)`
(hyper_parallel/platform/torch/platform.py:587-597) is the single cast every one of those sites goes
through.  An E4M3 target cannot be expressed by that hook as it stands (a cast needs a scale, and the
result is a pair), so this module restates both with the same names and field meanings plus what FP8
needs: `cast_fp_tensor(torch.float8_e4m3fn, x)` returns an `Fp8Tensor` (codes + scale_inv), every
other dtype behaves as in the reference.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import NamedTuple, Optional

import torch

from . import ops
from .linear import RECIPES


class Fp8Tensor(NamedTuple):
    """A tensor cast to E4M3 with one scale: value ~= codes.float() * scale_inv."""
    codes: torch.Tensor          # float8_e4m3fn, the source's shape
    scale_inv: torch.Tensor      # 0-dim float32

    def dequantize(self, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        """The cast back (`.to(origin_dtype)` of hyper_parallel/core/hsdp/hsdp_grad_hook.py:32-40): decode * scale_inv
        rounded once to bf16, or in fp32; any other dtype is a cast of the fp32 result."""
        if dtype in (torch.bfloat16, torch.float32):
            return ops.dequantize_per_tensor(self.codes, self.scale_inv, dtype)
        return ops.dequantize_per_tensor(self.codes, self.scale_inv, torch.float32).to(dtype)


@dataclass
class Fp8MixedPrecisionPolicy:
    """The reference's MixedPrecisionPolicy fields, with the same defaults and meanings, plus:

    fp8_recipe: recipe of the linear layers' matmuls ("blockwise", "per_tensor", "blockwise_pow2"), or None
        to leave them in `param_dtype`.
    fp8_reduce_bucket: quantize the flat gradient bucket to E4M3 in 1x128 groups around the reduction
        (`hpfp8.Fp8GradBucket`) instead of casting it to `reduce_dtype`.
    """
    param_dtype: Optional[torch.dtype] = None
    reduce_dtype: Optional[torch.dtype] = None
    output_dtype: Optional[torch.dtype] = None
    cast_forward_inputs: bool = True
    apply_grad_on_fp32_main_grad: bool = False
    fp8_recipe: Optional[str] = "blockwise"
    fp8_reduce_bucket: bool = False

    def __post_init__(self):
        if self.fp8_recipe is not None and self.fp8_recipe not in RECIPES:
            raise ValueError(f"fp8_recipe must be one of {RECIPES} or None, got {self.fp8_recipe!r}")
        for name in ("param_dtype", "reduce_dtype", "output_dtype"):
            v = getattr(self, name)
            if v is not None and not isinstance(v, torch.dtype):
                raise ValueError(f"{name} must be a torch.dtype or None")     # as core/hsdp/api.py:151-154 checks

    def linear_kwargs(self) -> dict:
        """Keyword arguments for `fp8_linear` / `Fp8Linear` that realise this policy."""
        if self.fp8_recipe is None:
            raise ValueError("this policy leaves the linear layers in param_dtype")
        return {"recipe": self.fp8_recipe,
                "apply_grad_on_fp32_main_grad": self.apply_grad_on_fp32_main_grad and self.fp8_recipe != "per_tensor"}


def cast_fp_tensor(dtype: torch.dtype, x):
    """`TorchPlatform.cast_fp_tensor` with an FP8 target: non-tensors, non-floating tensors and tensors that
    already have `dtype` pass through; `torch.float8_e4m3fn` gives an `Fp8Tensor` (per-tensor amax, scale
    448/amax, the cast of cfg 1); any other dtype is `x.to(dtype)`."""
    if not isinstance(x, torch.Tensor) or not torch.is_floating_point(x) or x.dtype == dtype:
        return x
    if dtype == ops.FP8:
        src = x if x.dtype == torch.bfloat16 else x.to(torch.bfloat16)
        q, _, scale_inv = ops.quantize_per_tensor(src.contiguous())
        return Fp8Tensor(q, scale_inv)
    return x.to(dtype)


# `TorchPlatform.tensor_type_cast`'s name -> dtype table (hyper_parallel/platform/torch/platform.py:195-206) with the
# two names this path adds
_TYPE_NAMES = {"float32": torch.float32, "float16": torch.float16, "int64": torch.int64, "int32": torch.int32,
               "bfloat16": torch.bfloat16, "float8_e4m3fn": ops.FP8}


def tensor_type_cast(input_data: torch.Tensor, cast_type: str):
    """`TorchPlatform.tensor_type_cast` (hyper_parallel/platform/torch/platform.py:195-206) with "float8_e4m3fn"
    among its names: that name gives an `Fp8Tensor` through `cast_fp_tensor`, the others are `.to(dtype)`; an
    unknown name raises the reference's ValueError."""
    if cast_type not in _TYPE_NAMES:
        raise ValueError(f"Unknown cast type: {cast_type}. Supported types: {list(_TYPE_NAMES.keys())}")
    dtype = _TYPE_NAMES[cast_type]
    return cast_fp_tensor(dtype, input_data) if dtype == ops.FP8 else input_data.to(dtype)
