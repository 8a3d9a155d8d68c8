"""FP8 form of the flat gradient bucket.

The reference packs gradients into one flat contiguous buffer, casts it to `reduce_dtype`, reduces
it, casts it back and multiplies by `grad_scale` (hyper_parallel/core/hsdp/hsdp_grad_buffer.py:95-108
and :116-135).  An E4M3 bucket needs a side buffer of scales, so it cannot be expressed as that
single dtype cast.  `quantize_bucket` / `dequantize_bucket` are the cast-in and cast-back for an
already packed bucket; `Fp8GradBucket` mirrors the reference's buffer object and fuses the packing
of many gradients with the quantization (and the dequantization with the unpacking).
"""
from __future__ import annotations

import ctypes
from typing import List, Sequence

import torch

from . import _lib, ops


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


class Fp8GradBucket:
    """Index bookkeeping, pack and unpack of HSDPGradBuffer for an E4M3 bucket.

    `numels[e]` is the number of elements parameter e owns in one row of the bucket, i.e. the size of
    one of the `shard_size` chunks of its gradient (`hsdp_param.param.numel()` in
    hsdp_grad_buffer.py:72-80).  Unlike the reference's dense index (each start = previous end),
    starts are rounded up to multiples of 128 so that no 1x128 scaling group straddles two
    parameters; the gaps are padding (zero codes).
    """

    def __init__(self, numels: Sequence[int], shard_size: int = 1, grad_scale: float = 1.0):
        if shard_size < 1:
            raise ValueError("shard_size must be >= 1")
        if any(int(n) <= 0 for n in numels):
            raise ValueError("every parameter needs at least one element per shard")
        self.numels = [int(n) for n in numels]
        self.shard_size = int(shard_size)
        self.grad_scale = float(grad_scale)
        self.offsets: List[int] = []
        end = 0
        for n in self.numels:                       # _init_grad_buffer_index, with 128-aligned starts
            self.offsets.append(end)
            end = -(-(end + n) // ops.BLOCK) * ops.BLOCK
        self.row_elems = end
        k = len(self.numels)
        self._numels_c = (ctypes.c_int64 * max(k, 1))(*self.numels)
        self._offsets_c = (ctypes.c_int64 * max(k, 1))(*self.offsets)

    def _ptr_table(self, tensors, per_tensor_elems):
        if len(tensors) != len(self.numels):
            raise ValueError(f"expected {len(self.numels)} tensors, got {len(tensors)}")
        ptrs = (ctypes.c_void_p * max(len(tensors), 1))()
        for e, (t, n) in enumerate(zip(tensors, per_tensor_elems)):
            if not t.is_cuda or t.device.index != torch.cuda.current_device() or t.dtype != torch.bfloat16 or not t.is_contiguous():
                raise TypeError(f"gradient {e} must be a contiguous bfloat16 tensor on the current GPU")
            if t.numel() != n:
                raise ValueError(f"gradient {e} has {t.numel()} elements, expected {n}")
            ptrs[e] = t.data_ptr()
        return ptrs

    def pack(self, grads: Sequence[torch.Tensor]):
        """_copy_grad_to_unsharded_buffer + cast: gradients (each shard_size * numels[e] elements) ->
        (codes [shard_size, row_elems] e4m3, scale_inv [shard_size, row_elems / 128] fp32)."""
        ptrs = self._ptr_table(grads, [n * self.shard_size for n in self.numels])    # (checks: all on the current GPU)
        dev = torch.device("cuda", torch.cuda.current_device())
        q = torch.empty((self.shard_size, self.row_elems), dtype=ops.FP8, device=dev)
        scale_inv = torch.empty((self.shard_size, self.row_elems // ops.BLOCK), dtype=torch.float32, device=dev)
        _lib.call("hpfp8_bucket_pack_quantize_bf16", ptrs, self._numels_c, self._offsets_c, len(self.numels),
                  self.shard_size, self.row_elems, q.data_ptr(), None, scale_inv.data_ptr(),
                  torch.cuda.current_stream().cuda_stream)
        return q, scale_inv

    def unpack(self, codes_row: torch.Tensor, scale_inv_row: torch.Tensor, outs: Sequence[torch.Tensor]):
        """_set_grad_data: one reduced row (codes [row_elems], scale_inv [row_elems / 128]) -> outs[e]
        (bf16, numels[e] elements each), times grad_scale after the cast back."""
        if codes_row.numel() != self.row_elems or scale_inv_row.numel() != self.row_elems // ops.BLOCK:
            raise ValueError("row does not have this bucket's size")
        if codes_row.dtype != ops.FP8 or scale_inv_row.dtype != torch.float32 or \
                not codes_row.is_contiguous() or not scale_inv_row.is_contiguous():
            raise TypeError("codes must be contiguous float8_e4m3fn and scale_inv contiguous float32")
        ops._check_device(codes_row, "codes_row")            # a row reduced on the host must be copied back first
        ops._check_device(scale_inv_row, "scale_inv_row")
        ptrs = self._ptr_table(outs, self.numels)
        _lib.call("hpfp8_bucket_unpack_dequantize_bf16", ptrs, self._numels_c, self._offsets_c, len(self.numels),
                  self.row_elems, codes_row.data_ptr(), scale_inv_row.data_ptr(), ctypes.c_float(self.grad_scale),
                  torch.cuda.current_stream().cuda_stream)
        return list(outs)
