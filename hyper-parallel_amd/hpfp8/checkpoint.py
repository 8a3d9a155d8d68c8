"""FP8 weights on disk, in the `weight` / `weight_scale_inv` convention of DeepSeek-V3 checkpoints.

A linear's weight is stored as two safetensors entries: `<name>.weight` (float8_e4m3fn [N, K]) and
`<name>.weight_scale_inv` (float32 [N/128, K/128]) with `w ~= weight.float() * weight_scale_inv`
expanded over 128x128 blocks -- exactly the (codes, scale_inv) pair of `quantize_weight`.  The
reference stores tensors in safetensors files as well
(hyper_parallel/core/checkpoint/filesystem_storage.py:166-205) but has no FP8 entries; a state dict
made here can be handed to it, or written directly with `save_fp8_checkpoint`.
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from . import ops
from .linear import Fp8Linear, Fp8Weight, quantize_weight

SCALE_SUFFIX = "_scale_inv"


def fp8_state_dict(module: torch.nn.Module) -> Dict[str, torch.Tensor]:
    """The module's state dict with every Fp8Linear weight replaced by its codes plus a
    `<name>.weight_scale_inv` entry; everything else (biases, other layers) unchanged."""
    out = dict(module.state_dict())
    for name, sub in module.named_modules():
        if isinstance(sub, Fp8Linear) and sub.recipe != "per_tensor":
            key = f"{name}.weight" if name else "weight"
            wf = quantize_weight(sub.weight.detach(), with_transpose=False, pow2=sub.recipe == "blockwise_pow2")
            out[key] = wf.codes
            out[key + SCALE_SUFFIX] = wf.scale_inv
    return out


def save_fp8_checkpoint(state: Mapping[str, torch.Tensor], path: str) -> None:
    from safetensors.torch import save_file
    save_file({k: v.detach().contiguous().cpu() for k, v in state.items()}, path)


def load_fp8_checkpoint(path: str, device="cuda") -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file
    return {k: v.to(device) for k, v in load_file(path).items()}


def load_into(module: torch.nn.Module, state: Mapping[str, torch.Tensor]) -> None:
    """Load a state dict that may hold FP8 weights.  An Fp8Linear whose weight comes as codes gets the
    dequantized bf16 values as its parameter and the stored codes as its cached FP8 form, so its
    forward uses the checkpoint's codes as they are (no quantization of a dequantized copy)."""
    plain = {}
    fp8 = {}
    for k, v in state.items():
        if k.endswith(SCALE_SUFFIX):
            continue
        if v.dtype == ops.FP8:
            scale_inv = state.get(k + SCALE_SUFFIX)
            if scale_inv is None:
                raise KeyError(f"{k} is float8 but {k + SCALE_SUFFIX} is missing")
            fp8[k] = (v, scale_inv)
            plain[k] = ops.dequantize_128x128(v.cuda(), scale_inv.cuda().float())
        else:
            plain[k] = v
    module.load_state_dict(plain)
    for name, sub in module.named_modules():
        key = f"{name}.weight" if name else "weight"
        if isinstance(sub, Fp8Linear) and key in fp8 and sub.recipe != "per_tensor":
            codes, scale_inv = fp8[key]
            codes = codes.to(sub.weight.device).contiguous()
            scale_inv = scale_inv.to(sub.weight.device).float().contiguous()
            pow2 = sub.recipe == "blockwise_pow2"
            if pow2 and bool((scale_inv.view(torch.int32) & 0x007FFFFF).any()):
                continue        # plain fp32 scales: this module quantizes the dequantized weight itself
            sub._cache.put(0, sub.weight, Fp8Weight(codes, scale_inv, ops.transpose_codes(codes), pow2))
