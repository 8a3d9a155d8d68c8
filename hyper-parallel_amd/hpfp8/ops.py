"""Tensor-level wrappers over the C ABI: quantizers, dequantizers and scaled GEMMs.

All functions take and return torch tensors that live on the GPU; they only check arguments,
allocate outputs with torch and pass raw pointers plus the current HIP stream to libhpfp8.so.
Weight tensors are [out_features, in_features] and the contraction runs over the last dim of both
GEMM operands, the operand roles of the reference's linear operator
(hyper_parallel/core/shard/ops/parallel_matmul.py:377-381).
"""
from __future__ import annotations

from typing import Optional, Tuple

import ctypes

import torch

from . import _lib

BLOCK = 128
FP8 = torch.float8_e4m3fn


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _check_device(x: torch.Tensor, name: str) -> None:
    """Kernels are launched on the current device and its current stream: a tensor that lives on another
    GPU must be used under ``torch.cuda.device(x.device)``."""
    if not x.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got device {x.device}); this path has no CPU fallback")
    if x.device.index != torch.cuda.current_device():
        raise ValueError(f"{name} lives on {x.device} but the current device is cuda:{torch.cuda.current_device()}; "
                         f"call under torch.cuda.device({name}.device)")


def _check_bf16(x: torch.Tensor, name: str, contiguous: bool = True) -> torch.Tensor:
    if not isinstance(x, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    _check_device(x, name)
    if x.dtype != torch.bfloat16:
        raise TypeError(f"{name} must be bfloat16, got {x.dtype}")
    if not contiguous:
        return x
    return x if x.is_contiguous() else x.contiguous()


def _check_fp8(x: torch.Tensor, name: str) -> torch.Tensor:
    _check_device(x, name)
    if x.dtype not in (FP8, torch.uint8):
        raise TypeError(f"{name} must be float8_e4m3fn (or uint8 codes), got {x.dtype}")
    if not x.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return x


def _check_codes_2d(x: torch.Tensor, name: str) -> torch.Tensor:
    """A GEMM operand: 2-D codes with unit inner stride; the row stride may exceed the row length."""
    _check_device(x, name)
    if x.dtype not in (FP8, torch.uint8):
        raise TypeError(f"{name} must be float8_e4m3fn (or uint8 codes), got {x.dtype}")
    if x.dim() != 2 or (x.shape[1] > 1 and x.stride(1) != 1) or (x.shape[0] > 1 and x.stride(0) % 16):
        raise ValueError(f"{name} must be 2-D with unit inner stride and a row stride that is a multiple of 16")
    return x


def _ld(x: torch.Tensor) -> int:
    return x.stride(0) if x.shape[0] > 1 else max(x.shape[1], 16)


def _padded_ld(n: int) -> int:
    """Row stride for a transposed code tensor with n columns: an odd multiple of 128 bytes, so that
    consecutive rows do not all fall on the same HBM channel (n itself is a multiple of 128)."""
    return n if (n // BLOCK) % 2 == 1 else n + BLOCK


def _empty_codes_t(rows: int, cols: int, device) -> torch.Tensor:
    ld = _padded_ld(cols)
    return torch.empty((rows, ld), dtype=FP8, device=device)[:, :cols]


def _check_offs(offs: torch.Tensor) -> torch.Tensor:
    if not isinstance(offs, torch.Tensor) or offs.dtype != torch.int32 or offs.dim() != 1 or not offs.is_contiguous():
        raise TypeError("offs must be a contiguous 1-D int32 GPU tensor")
    _check_device(offs, "offs")
    return offs


def _check_f32(x: torch.Tensor, name: str) -> torch.Tensor:
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dtype != torch.float32:
        raise TypeError(f"{name} must be a float32 GPU tensor")
    _check_device(x, name)
    return x


# ------------------------------------------------------------------------------------------------
# quantizers
# ------------------------------------------------------------------------------------------------
def amax(x: torch.Tensor) -> torch.Tensor:
    """max |x| as a 0-dim fp32 tensor."""
    x = _check_bf16(x, "x")
    out = torch.empty((), dtype=torch.float32, device=x.device)
    _lib.call("hpfp8_amax_bf16", _ptr(x), x.numel(), _ptr(out), _stream())
    return out


# 512 bytes per (device, stream) that hpfp8_quantize_per_tensor_sync_bf16's grid synchronises through: zero when
# created, and left zero by every call, so calls on one stream can share them
_SYNC_WORDS = {}
_ONE_PASS_MAX = 1 << 22


def _sync_words(device: torch.device) -> Optional[torch.Tensor]:
    """The 512-byte block through which the one-launch per-tensor quantizer's grid agrees on the maximum, one per
    (device, stream).  Sharing rule: the block must be zero at launch (the kernel leaves it zero) and two launches
    must never use it at once.  Eager calls on one stream are ordered by the stream, so they may share it.  A
    captured graph is different: it would bake the block's address in, and a replay on another stream could then run
    beside an eager call (or another graph) that uses the same block -- both would write the same slots and the
    maximum would be silently wrong.  So nothing that is being captured gets the block: under capture the
    two-launch form runs, whose only scratch is the caller-visible amax word allocated per call."""
    if torch.cuda.is_current_stream_capturing():
        return None
    key = (device.index if device.index is not None else torch.cuda.current_device(), _stream())
    t = _SYNC_WORDS.get(key)
    if t is None:
        t = _SYNC_WORDS[key] = torch.zeros(128, dtype=torch.int32, device=device)
    return t


def quantize_per_tensor(x: torch.Tensor, amax_in: Optional[torch.Tensor] = None
                        ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """One scale for the whole tensor: returns (codes like x, scale, scale_inv).

    scale = 448 / max(amax, 1e-12) and scale_inv = max(amax, 1e-12) / 448 are 0-dim fp32 tensors.
    With ``amax_in`` (0-dim fp32 GPU tensor) the reduction is skipped and that value is used.
    """
    x = _check_bf16(x, "x")
    q = torch.empty(x.shape, dtype=FP8, device=x.device)
    scale = torch.empty((), dtype=torch.float32, device=x.device)
    scale_inv = torch.empty((), dtype=torch.float32, device=x.device)
    if amax_in is None:
        sync = _sync_words(x.device) if 0 < x.numel() <= _ONE_PASS_MAX else None
        if sync is not None:      # one launch: amax and cast in one pass over x
            _lib.call("hpfp8_quantize_per_tensor_sync_bf16", _ptr(x), x.numel(), _ptr(q), None, _ptr(scale), _ptr(scale_inv),
                      _ptr(sync), _stream())
            return q, scale, scale_inv
        am = torch.empty((), dtype=torch.float32, device=x.device)
        _lib.call("hpfp8_quantize_per_tensor_bf16", _ptr(x), x.numel(), _ptr(q), _ptr(am), _ptr(scale),
                  _ptr(scale_inv), _stream())
    else:
        am = _check_f32(amax_in, "amax_in")
        _lib.call("hpfp8_cast_per_tensor_bf16", _ptr(x), x.numel(), _ptr(am), _ptr(q), _ptr(scale),
                  _ptr(scale_inv), _stream())
    return q, scale, scale_inv


def quantize_1x128(x: torch.Tensor, want_scale: bool = False, kmajor: bool = False, pow2: bool = False):
    """x[..., C] -> (codes, scale_inv[..., C/128]) (plus scale when ``want_scale``).

    With ``kmajor`` the scales are STORED k-block-major ([C/128, rows] in memory) and returned as the
    transposed view, so they index exactly like the row-major result but the GEMM reads them with
    unit stride across rows.  Values are identical in both layouts.

    ``pow2`` (k-block-major layout only; also on the other blockwise quantizers): scale_inv rounded up
    to a power of two, the optional recipe whose GEMMs are ``gemm_blockwise(..., pow2_scales=True)``.
    """
    x = _check_bf16(x, "x")
    if x.dim() < 1:
        raise ValueError("x must have at least one dimension")
    cols = x.shape[-1]
    if cols % BLOCK:
        raise ValueError(f"last dim {cols} is not a multiple of {BLOCK}")
    rows = x.numel() // cols if cols else 0
    q = torch.empty(x.shape, dtype=FP8, device=x.device)
    sshape = x.shape[:-1] + (cols // BLOCK,)
    if pow2 and not kmajor:
        raise ValueError("pow2 scales are written in the k-block-major layout only (kmajor=True)")
    if kmajor:
        store = (cols // BLOCK, rows)
        scale_inv = torch.empty(store, dtype=torch.float32, device=x.device)
        scale = torch.empty(store, dtype=torch.float32, device=x.device) if want_scale else None
        _lib.call("hpfp8_quantize_1x128_kmajor_pow2_bf16" if pow2 else "hpfp8_quantize_1x128_kmajor_bf16", _ptr(x), rows,
                  cols, _ptr(q), _ptr(scale), _ptr(scale_inv), _stream())
        scale_inv = scale_inv.t()
        scale = scale.t() if want_scale else None
        if x.dim() != 2:
            scale_inv = scale_inv.reshape(sshape)
            scale = scale.reshape(sshape) if want_scale else None
    else:
        scale_inv = torch.empty(sshape, dtype=torch.float32, device=x.device)
        scale = torch.empty(sshape, dtype=torch.float32, device=x.device) if want_scale else None
        _lib.call("hpfp8_quantize_1x128_bf16", _ptr(x), rows, cols, _ptr(q), _ptr(scale), _ptr(scale_inv), _stream())
    return (q, scale, scale_inv) if want_scale else (q, scale_inv)


def quantize_128x128(w: torch.Tensor, with_transpose: bool = False, want_scale: bool = False, pow2: bool = False):
    """w[R, C] -> (codes[R, C], scale_inv[R/128, C/128]) (+ codes_t[C, R]) (+ scale)."""
    w = _check_bf16(w, "w")
    if w.dim() != 2:
        raise ValueError("w must be 2-D")
    r, c = w.shape
    if r % BLOCK or c % BLOCK:
        raise ValueError(f"shape {tuple(w.shape)} is not a multiple of {BLOCK} in both dims")
    q = torch.empty((r, c), dtype=FP8, device=w.device)
    qt = _empty_codes_t(c, r, w.device) if with_transpose else None     # row stride padded, see _padded_ld
    scale_inv = torch.empty((r // BLOCK, c // BLOCK), dtype=torch.float32, device=w.device)
    scale = torch.empty_like(scale_inv) if want_scale else None
    _lib.call("hpfp8_quantize_128x128_pow2_bf16" if pow2 else "hpfp8_quantize_128x128_bf16", _ptr(w), r, c, _ptr(q),
              _ptr(qt), _ld(qt) if with_transpose else 0, _ptr(scale), _ptr(scale_inv), _stream())
    out = (q, scale_inv)
    if with_transpose:
        out += (qt,)
    if want_scale:
        out += (scale,)
    return out


def swiglu_quantize_1x128(h: torch.Tensor, kmajor: bool = True, want_act: bool = False, pow2: bool = False,
                          fast: bool = False):
    """h[M, 2I] bf16 (gate | up halves; any row stride that is a multiple of 8) ->
    (codes[M, I], scale_inv[M, I/128]) of act = silu(gate) * up, plus act itself (bf16) if asked for.

    ``fast``: silu from the hardware's exponential and reciprocal approximations instead of the exactly
    specified sequence (about twice as fast; the rounded silu may differ by one bf16 unit in the last place, act by
    two, in about one element per ten thousand; codes and scales are the exact quantization of that act)."""
    h = _check_bf16(h, "h", contiguous=False)
    if h.dim() != 2 or h.shape[1] % (2 * BLOCK):
        raise ValueError("h must be 2-D with a width that is a multiple of 256")
    if h.stride(1) != 1 or h.stride(0) % 8 or h.data_ptr() % 16:
        h = h.contiguous()
    m, inter = h.shape[0], h.shape[1] // 2
    q = torch.empty((m, inter), dtype=FP8, device=h.device)
    s_inv = torch.empty((inter // BLOCK, m) if kmajor else (m, inter // BLOCK), dtype=torch.float32, device=h.device)
    act = torch.empty((m, inter), dtype=torch.bfloat16, device=h.device) if want_act else None
    ld_h = h.stride(0) if m > 1 else 2 * inter
    if fast:
        _lib.call("hpfp8_swiglu_quantize_1x128_fast_bf16", _ptr(h), m, inter, ld_h, int(kmajor), int(pow2),
                  _ptr(q), None, _ptr(s_inv), _ptr(act), _stream())
    else:
        _lib.call("hpfp8_swiglu_quantize_1x128_pow2_bf16" if pow2 else "hpfp8_swiglu_quantize_1x128_bf16", _ptr(h), m,
                  inter, ld_h, int(kmajor), _ptr(q), None, _ptr(s_inv), _ptr(act), _stream())
    if kmajor:
        s_inv = s_inv.t()
    return (q, s_inv, act) if want_act else (q, s_inv)


def swiglu_quantize_1x128_and_128x1_t(h: torch.Tensor, fast: bool = False):
    """Both quantized forms of act = silu(gate) * up from one read of h[M, 2I] = gate | up:
    (codes[M, I], scale_inv[M, I/128], codes_t[I, M], scale_inv_t[I, M/128]), k-block-major scales, bit-identical to
    ``swiglu_quantize_1x128(h, fast=fast)`` and to ``quantize_128x1_t`` of its activation.  M and I multiples of 128."""
    h = _check_bf16(h, "h", contiguous=False)
    if h.dim() != 2 or h.shape[1] % (2 * BLOCK) or h.shape[0] % BLOCK:
        raise ValueError("h must be [M, 2I] with M and I multiples of 128")
    if h.stride(1) != 1 or h.stride(0) % 8 or h.data_ptr() % 16:
        h = h.contiguous()
    m, inter = h.shape[0], h.shape[1] // 2
    q = torch.empty((m, inter), dtype=FP8, device=h.device)
    qt = _empty_codes_t(inter, m, h.device)
    s_inv = torch.empty((inter // BLOCK, m), dtype=torch.float32, device=h.device)
    st_inv = torch.empty((m // BLOCK, inter), dtype=torch.float32, device=h.device)
    _lib.call("hpfp8_swiglu_quantize_1x128_and_128x1_t_bf16", _ptr(h), m, inter, h.stride(0) if m > 1 else 2 * inter,
              int(fast), _ptr(q), None, _ptr(s_inv), _ptr(qt), _ld(qt), None, _ptr(st_inv), _stream())
    return q, s_inv.t(), qt, st_inv.t()


def swiglu_backward(h: torch.Tensor, dact: torch.Tensor) -> torch.Tensor:
    """Gradient of act = silu(gate) * up with respect to h = [gate | up]: h[M, 2I], dact[M, I] -> dh[M, 2I], bf16."""
    h = _check_bf16(h, "h", contiguous=False)
    dact = _check_bf16(dact, "dact")
    if h.dim() != 2 or h.shape[1] % 16 or dact.shape != (h.shape[0], h.shape[1] // 2):
        raise ValueError("h must be [M, 2I] with I a multiple of 8 and dact [M, I]")
    if h.stride(1) != 1 or h.stride(0) % 8 or h.data_ptr() % 16:
        h = h.contiguous()
    m, inter = dact.shape
    dh = torch.empty((m, 2 * inter), dtype=torch.bfloat16, device=h.device)
    _lib.call("hpfp8_swiglu_backward_bf16", _ptr(h), m, inter, h.stride(0) if m > 1 else 2 * inter, _ptr(dact), _ptr(dh),
              2 * inter, _stream())
    return dh


def swiglu_backward_quantize_1x128_and_128x1_t(h: torch.Tensor, dact: torch.Tensor):
    """`swiglu_backward` fused with both quantized forms of its result dh = [d gate | d up] ([M, 2I]; never written in
    bf16): (codes[M, 2I], scale_inv[M, 2I/128], codes_t[2I, M], scale_inv_t[2I, M/128]), k-block-major scales,
    bit-identical to ``quantize_1x128_and_128x1_t(swiglu_backward(h, dact))``.  M and I multiples of 128."""
    h = _check_bf16(h, "h", contiguous=False)
    dact = _check_bf16(dact, "dact")
    if h.dim() != 2 or h.shape[1] % (2 * BLOCK) or h.shape[0] % BLOCK or dact.shape != (h.shape[0], h.shape[1] // 2):
        raise ValueError("h must be [M, 2I] with M and I multiples of 128 and dact [M, I]")
    if h.stride(1) != 1 or h.stride(0) % 8 or h.data_ptr() % 16:
        h = h.contiguous()
    m, inter = dact.shape
    q = torch.empty((m, 2 * inter), dtype=FP8, device=h.device)
    qt = _empty_codes_t(2 * inter, m, h.device)
    s_inv = torch.empty((2 * inter // BLOCK, m), dtype=torch.float32, device=h.device)
    st_inv = torch.empty((m // BLOCK, 2 * inter), dtype=torch.float32, device=h.device)
    _lib.call("hpfp8_swiglu_backward_quantize_1x128_and_128x1_t_bf16", _ptr(h), m, inter, h.stride(0) if m > 1 else 2 * inter,
              _ptr(dact), _ptr(q), None, _ptr(s_inv), _ptr(qt), _ld(qt), None, _ptr(st_inv), _stream())
    return q, s_inv.t(), qt, st_inv.t()


def transpose_codes(q: torch.Tensor) -> torch.Tensor:
    """codes[R, C] -> codes_t[C, R] (byte transpose; R, C multiples of 128).  With 128x128 scaling blocks
    the transposed codes of a weight are its dgrad operand, scales reused with swapped strides."""
    q = _check_codes_2d(q, "q")
    r, c = q.shape
    if r % BLOCK or c % BLOCK:
        raise ValueError(f"shape {tuple(q.shape)} is not a multiple of {BLOCK} in both dims")
    qt = _empty_codes_t(c, r, q.device)
    _lib.call("hpfp8_transpose_codes", _ptr(q), r, c, _ld(q), _ptr(qt), _ld(qt), _stream())
    return qt


def quantize_128x1_t(x: torch.Tensor, want_scale: bool = False, kmajor: bool = False, pow2: bool = False):
    """Transposed re-quantization for wgrad from the bf16 source.

    x[M, K] -> (codes_t[K, M], scale_inv_t[K, M/128]); one scale per 128 consecutive rows of a column.
    With ``kmajor`` the scales are stored [M/128, K] in memory and returned as the transposed view.
    """
    x = _check_bf16(x, "x")
    if x.dim() != 2:
        raise ValueError("x must be 2-D")
    m, k = x.shape
    if m % BLOCK or k % BLOCK:
        raise ValueError(f"shape {tuple(x.shape)} is not a multiple of {BLOCK} in both dims")
    qt = _empty_codes_t(k, m, x.device)                                  # row stride padded, see _padded_ld
    sshape = (m // BLOCK, k) if kmajor else (k, m // BLOCK)
    scale_inv = torch.empty(sshape, dtype=torch.float32, device=x.device)
    scale = torch.empty_like(scale_inv) if want_scale else None
    if pow2 and not kmajor:
        raise ValueError("pow2 scales are written in the block-major layout only (kmajor=True)")
    name = "hpfp8_quantize_128x1_t_kmajor_bf16" if kmajor else "hpfp8_quantize_128x1_t_bf16"
    if pow2:
        name = "hpfp8_quantize_128x1_t_kmajor_pow2_bf16"
    _lib.call(name, _ptr(x), m, k, _ptr(qt), _ld(qt), _ptr(scale), _ptr(scale_inv), _stream())
    if kmajor:
        scale_inv = scale_inv.t()
        scale = scale.t() if want_scale else None
    return (qt, scale, scale_inv) if want_scale else (qt, scale_inv)


def quantize_128x1_t_rows(x: torch.Tensor):
    """`quantize_128x1_t(..., kmajor=True)` of x[M, K] for any M > 0: the last group of a ragged M is filled up with
    zero rows.  Only those last rows are copied for the padding; the whole groups are quantized where they lie.
    Returns (codes_t[K, Mp], scale_inv_t[K, Mp/128]) with Mp = M rounded up to a multiple of 128."""
    x = _check_bf16(x, "x")
    if x.dim() != 2 or x.shape[1] % BLOCK or x.shape[0] == 0:
        raise ValueError("x must be [M, K] with M > 0 and K a multiple of 128")
    m, k = x.shape
    main = m // BLOCK * BLOCK
    mp = main + (BLOCK if m > main else 0)
    qt = _empty_codes_t(k, mp, x.device)
    scale_inv = torch.empty((mp // BLOCK, k), dtype=torch.float32, device=x.device)
    if main:
        _lib.call("hpfp8_quantize_128x1_t_kmajor_bf16", _ptr(x), main, k, _ptr(qt), qt.stride(0), None, _ptr(scale_inv),
                  _stream())
    if m > main:
        tail = torch.zeros((BLOCK, k), dtype=torch.bfloat16, device=x.device)
        tail[:m - main] = x[main:]
        _lib.call("hpfp8_quantize_128x1_t_kmajor_bf16", _ptr(tail), BLOCK, k, qt.data_ptr() + main, qt.stride(0), None,
                  scale_inv.data_ptr() + main // BLOCK * k * 4, _stream())
    return qt, scale_inv.t()


def quantize_1x128_and_128x1_t(x: torch.Tensor, kmajor: bool = True, pow2: bool = False, column_sum: bool = False):
    """Both operand forms of x[M, K] from one read of it.

    Returns (codes[M, K], scale_inv[M, K/128], codes_t[K, M], scale_inv_t[K, M/128]), bit-identical to
    ``quantize_1x128(x, kmajor=kmajor)`` and ``quantize_128x1_t(x, kmajor=kmajor)``.  M and K multiples of 128.
    With ``column_sum`` (k-block-major scales only) a fifth result: the bf16 sum of x over its rows [K], from the
    same read -- a bias gradient when x is grad_out -- with the bits of `column_sum(x)`.
    """
    x = _check_bf16(x, "x")
    if x.dim() != 2:
        raise ValueError("x must be 2-D")
    m, k = x.shape
    if m % BLOCK or k % BLOCK:
        raise ValueError(f"shape {tuple(x.shape)} is not a multiple of {BLOCK} in both dims")
    if column_sum and not kmajor:
        raise ValueError("column_sum comes with the k-block-major scale layout only (kmajor=True)")
    q = torch.empty((m, k), dtype=FP8, device=x.device)
    qt = _empty_codes_t(k, m, x.device)
    s_inv = torch.empty((k // BLOCK, m) if kmajor else (m, k // BLOCK), dtype=torch.float32, device=x.device)
    st_inv = torch.empty((m // BLOCK, k) if kmajor else (k, m // BLOCK), dtype=torch.float32, device=x.device)
    if column_sum:
        part = torch.empty((m // BLOCK, k), dtype=torch.float32, device=x.device)
        _lib.call("hpfp8_quantize_128x1_t_colsum_bf16", _ptr(x), m, k, _ptr(q), None, _ptr(s_inv), _ptr(qt), _ld(qt), None,
                  _ptr(st_inv), int(pow2), _ptr(part), _stream())
        total = torch.empty((k,), dtype=torch.bfloat16, device=x.device)
        _lib.call("hpfp8_column_sum_finish", _ptr(part), m // BLOCK, k, _ptr(total), None, _stream())
        return q, s_inv.t(), qt, st_inv.t(), total
    _lib.call("hpfp8_quantize_1x128_and_128x1_t_pow2_bf16" if pow2 else "hpfp8_quantize_1x128_and_128x1_t_bf16", _ptr(x),
              m, k, int(kmajor), _ptr(q), None, _ptr(s_inv), _ptr(qt), _ld(qt), None, _ptr(st_inv), _stream())
    if kmajor:
        s_inv, st_inv = s_inv.t(), st_inv.t()
    return q, s_inv, qt, st_inv


def column_sum(x: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Sum of x[M, K] (bf16, K a multiple of 128, any M) over its rows, accumulated in fp32 in a fixed order (per
    128-row block, then over the blocks) and returned as bf16 (rounded once) or fp32 [K]: the bias gradient of a
    linear whose grad_out is x.  Same bits as the sum `quantize_1x128_and_128x1_t(..., column_sum=True)` returns."""
    x = _check_bf16(x, "x")
    if x.dim() != 2:
        raise ValueError("x must be 2-D")
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise TypeError("out_dtype must be torch.bfloat16 or torch.float32")
    m, k = x.shape
    if k % BLOCK:
        raise ValueError(f"width {k} is not a multiple of {BLOCK}")
    blocks = (m + BLOCK - 1) // BLOCK
    part = torch.empty((blocks, k), dtype=torch.float32, device=x.device)
    out = torch.empty((k,), dtype=out_dtype, device=x.device)
    bf = out_dtype == torch.bfloat16
    _lib.call("hpfp8_column_sum_bf16", _ptr(x), m, k, _ld(x), _ptr(part), _ptr(out) if bf else None,
              None if bf else _ptr(out), _stream())
    return out


def dequantize_1x128(q: torch.Tensor, scale_inv: torch.Tensor, grad_scale: float = 1.0) -> torch.Tensor:
    """codes[..., C] with scale_inv[..., C/128] -> bf16."""
    q = _check_fp8(q, "q")
    scale_inv = _check_f32(scale_inv, "scale_inv")
    cols = q.shape[-1]
    if cols % BLOCK:
        raise ValueError(f"last dim {cols} is not a multiple of {BLOCK}")
    rows = q.numel() // cols if cols else 0
    if scale_inv.numel() != rows * (cols // BLOCK) or not scale_inv.is_contiguous():
        raise ValueError("scale_inv must be contiguous with one entry per 128 codes")
    out = torch.empty(q.shape, dtype=torch.bfloat16, device=q.device)
    _lib.call("hpfp8_dequantize_1x128_bf16", _ptr(q), _ptr(scale_inv), rows, cols, _ptr(out), float(grad_scale),
              _stream())
    return out


def dequantize_1x128_accumulate(q: torch.Tensor, scale_inv: torch.Tensor, main_grad: torch.Tensor,
                                grad_scale: float = 1.0) -> torch.Tensor:
    """main_grad (fp32, same shape as q, contiguous) += decode(q) * scale_inv * grad_scale, in place."""
    q = _check_fp8(q, "q")
    scale_inv = _check_f32(scale_inv, "scale_inv")
    cols = q.shape[-1]
    if cols % BLOCK:
        raise ValueError(f"last dim {cols} is not a multiple of {BLOCK}")
    rows = q.numel() // cols if cols else 0
    if scale_inv.numel() != rows * (cols // BLOCK) or not scale_inv.is_contiguous() or not q.is_contiguous():
        raise ValueError("q must be contiguous and scale_inv contiguous with one entry per 128 codes")
    _check_f32(main_grad, "main_grad")
    if not main_grad.is_contiguous() or main_grad.numel() != q.numel():
        raise ValueError("main_grad must be a contiguous float32 GPU tensor with as many elements as q")
    _lib.call("hpfp8_dequantize_1x128_accumulate_f32", _ptr(q), _ptr(scale_inv), rows, cols, _ptr(main_grad),
              ctypes.c_float(grad_scale), _stream())
    return main_grad


def dequantize_per_tensor(q: torch.Tensor, scale_inv: torch.Tensor, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """codes (any shape) with one scale_inv (0-dim or 1-element fp32) -> decode * scale_inv as bf16 or fp32: the cast
    back of a tensor that `quantize_per_tensor` cast in."""
    q = _check_fp8(q, "q")
    scale_inv = _check_f32(scale_inv, "scale_inv")
    if scale_inv.numel() != 1:
        raise ValueError("a per-tensor scale has exactly one element")
    out = torch.empty(q.shape, dtype=dtype, device=q.device)
    _lib.call("hpfp8_dequantize_per_tensor", _ptr(q), q.numel(), _ptr(scale_inv), _ptr(out), _out_code(dtype), _stream())
    return out


def dequantize_128x128(q: torch.Tensor, scale_inv: torch.Tensor) -> torch.Tensor:
    q = _check_fp8(q, "q")
    scale_inv = _check_f32(scale_inv, "scale_inv")
    r, c = q.shape
    if r % BLOCK or c % BLOCK:
        raise ValueError(f"shape {tuple(q.shape)} is not a multiple of {BLOCK} in both dims")
    if tuple(scale_inv.shape) != (r // BLOCK, c // BLOCK) or not scale_inv.is_contiguous():
        raise ValueError("scale_inv must be contiguous [R/128, C/128]")
    out = torch.empty((r, c), dtype=torch.bfloat16, device=q.device)
    _lib.call("hpfp8_dequantize_128x128_bf16", _ptr(q), _ptr(scale_inv), r, c, _ptr(out), _stream())
    return out


# ------------------------------------------------------------------------------------------------
# GEMMs
# ------------------------------------------------------------------------------------------------
def _out_code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return _lib.OUT_BF16
    if dtype == torch.float32:
        return _lib.OUT_F32
    raise TypeError(f"out_dtype must be bfloat16 or float32, got {dtype}")


def gemm_blockwise(a: torch.Tensor, sa: torch.Tensor, b: torch.Tensor, sb: torch.Tensor,
                   bias: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.bfloat16,
                   sb_gran: int = 128, out: Optional[torch.Tensor] = None, accumulate: bool = False,
                   pow2_scales: bool = False) -> torch.Tensor:
    """c[M,N] = sum_kb sa[m,kb] * sb[n//sb_gran, kb] * (a[m, kb] . b[n, kb]) (+ bias).

    a[M,K], b[N,K] codes (unit inner stride, any 16-byte-multiple row stride); sa, sb 2-D fp32 views
    (any strides) of scale_inv values.
    """
    a = _check_codes_2d(a, "a")
    b = _check_codes_2d(b, "b")
    sa = _check_f32(sa, "sa")
    sb = _check_f32(sb, "sb")
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise ValueError(f"a {tuple(a.shape)} and b {tuple(b.shape)} must be 2-D with equal last dim")
    m, k = a.shape
    n = b.shape[0]
    if k % BLOCK or n % BLOCK or k == 0:
        raise ValueError(f"K={k} must be a positive multiple of 128 and N={n} a multiple of 128")
    kb = k // BLOCK
    if tuple(sa.shape) != (m, kb):
        raise ValueError(f"sa must be [{m}, {kb}], got {tuple(sa.shape)}")
    want_sb = (n // BLOCK, kb) if sb_gran == 128 else (n, kb)
    if sb_gran not in (1, 128) or tuple(sb.shape) != want_sb:
        raise ValueError(f"sb must be {list(want_sb)} for sb_gran={sb_gran}, got {tuple(sb.shape)}")
    if sb_gran == 1 and (sb.stride(0) != 1 or (kb > 1 and (sb.stride(1) < n or sb.stride(1) % 4)) or sb.data_ptr() % 16):
        sb = sb.t().contiguous().t()        # the kernel wants per-row b scales k-block-major
    if bias is not None:
        bias = _check_bf16(bias, "bias")
        if tuple(bias.shape) != (n,):
            raise ValueError(f"bias must be [{n}]")
    if out is None:
        if accumulate:
            raise ValueError("accumulate needs an existing `out`")
        out = torch.empty((m, n), dtype=out_dtype, device=a.device)
    else:
        _check_device(out, "out")
        if tuple(out.shape) != (m, n) or out.stride(1) != 1:
            raise ValueError("out must be a GPU tensor [M, N] with unit inner stride")
        out_dtype = out.dtype
    if accumulate and out_dtype != torch.float32:
        raise ValueError("accumulate needs a float32 output")
    _lib.call("hpfp8_gemm_blockwise_pow2" if pow2_scales else "hpfp8_gemm_blockwise", _ptr(a), _ld(a), _ptr(sa),
              sa.stride(0), sa.stride(1), _ptr(b), _ld(b), _ptr(sb), sb.stride(0), sb.stride(1), sb_gran, m, n, k, _ptr(bias), _ptr(out),
              out.stride(0) if m > 1 else n, _out_code(out_dtype), int(accumulate), _stream())
    return out


def gemm_blockwise_swiglu_quantize(a: torch.Tensor, sa: torch.Tensor, b: torch.Tensor, sb: torch.Tensor, *,
                                   fast: bool = False, pow2_scales: bool = False, pow2_out: bool = False,
                                   want_scale: bool = False):
    """The gate/up projection with SwiGLU and the 1x128 quantization of its result as the GEMM's epilogue.

    a[M, K] codes with scales sa[M, K/128]; b = codes of W_gate_up [2I, K] (gate rows first) with 128x128 scales
    sb[2I/128, K/128].  Returns (codes[M, I], scale_inv[M, I/128]) of act = silu(gate) * up -- bit for bit what
    `gemm_blockwise` followed by `swiglu_quantize_1x128(kmajor=True)` returns -- without the bf16 gate/up tensor."""
    a = _check_codes_2d(a, "a")
    b = _check_codes_2d(b, "b")
    sa = _check_f32(sa, "sa")
    sb = _check_f32(sb, "sb")
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise ValueError(f"a {tuple(a.shape)} and b {tuple(b.shape)} must be 2-D with equal last dim")
    m, k = a.shape
    n = b.shape[0]
    if k % BLOCK or n % (2 * BLOCK) or k == 0:
        raise ValueError(f"K={k} must be a positive multiple of 128 and the weight's rows {n} a multiple of 256")
    kb, inter = k // BLOCK, n // 2
    if tuple(sa.shape) != (m, kb) or tuple(sb.shape) != (n // BLOCK, kb):
        raise ValueError(f"sa must be [{m}, {kb}] and sb [{n // BLOCK}, {kb}]")
    q = torch.empty((m, inter), dtype=FP8, device=a.device)
    s_inv = torch.empty((inter // BLOCK, m), dtype=torch.float32, device=a.device)
    s = torch.empty_like(s_inv) if want_scale else None
    _lib.call("hpfp8_gemm_blockwise_swiglu_quantize", _ptr(a), _ld(a), _ptr(sa), sa.stride(0), sa.stride(1), _ptr(b),
              _ld(b), _ptr(sb), sb.stride(0), sb.stride(1), m, inter, k, int(fast), int(pow2_scales), int(pow2_out),
              _ptr(q), inter, _ptr(s), _ptr(s_inv), _stream())
    return (q, s_inv.t(), s.t()) if want_scale else (q, s_inv.t())


def gemm_per_tensor(a: torch.Tensor, sa_inv: torch.Tensor, b: torch.Tensor, sb_inv: torch.Tensor,
                    bias: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """c = (a . b^T) * (sa_inv * sb_inv) (+ bias); sa_inv / sb_inv are 0-dim (or 1-element) fp32."""
    a = _check_codes_2d(a, "a")
    b = _check_codes_2d(b, "b")
    sa_inv = _check_f32(sa_inv, "sa_inv")
    sb_inv = _check_f32(sb_inv, "sb_inv")
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise ValueError(f"a {tuple(a.shape)} and b {tuple(b.shape)} must be 2-D with equal last dim")
    if sa_inv.numel() != 1 or sb_inv.numel() != 1:
        raise ValueError("per-tensor scales must have exactly one element")
    m, k = a.shape
    n = b.shape[0]
    if k % BLOCK or n % BLOCK or k == 0:
        raise ValueError(f"K={k} must be a positive multiple of 128 and N={n} a multiple of 128")
    if bias is not None:
        bias = _check_bf16(bias, "bias")
        if tuple(bias.shape) != (n,):
            raise ValueError(f"bias must be [{n}]")
    out = torch.empty((m, n), dtype=out_dtype, device=a.device)
    _lib.call("hpfp8_gemm_per_tensor", _ptr(a), _ld(a), _ptr(sa_inv), _ptr(b), _ld(b), _ptr(sb_inv), m, n, k,
              _ptr(bias), _ptr(out), n, _out_code(out_dtype), _stream())
    return out


def gemm_grouped_blockwise(a: torch.Tensor, sa: torch.Tensor, b: torch.Tensor, sb: torch.Tensor,
                           offs: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                           pow2_scales: bool = False) -> torch.Tensor:
    """MoE grouped GEMM: rows of a[total_m, K] sorted by expert, offs[E] int32 inclusive prefix sums,
    b[E, N, K], sb[E, N/128, K/128], sa[total_m, K/128] -> c[total_m, N].  Rows past offs[-1] are left
    uninitialised (as torch's grouped matmul leaves them)."""
    a = _check_codes_2d(a, "a")
    b = _check_fp8(b, "b")
    sa = _check_f32(sa, "sa")
    sb = _check_f32(sb, "sb")
    if a.dim() != 2 or b.dim() != 3 or a.shape[1] != b.shape[2]:
        raise ValueError(f"a {tuple(a.shape)} must be [total_m, K] and b {tuple(b.shape)} [E, N, K]")
    _check_offs(offs)
    total_m, k = a.shape
    e, n, _ = b.shape
    if offs.numel() != e:
        raise ValueError(f"offs must have {e} entries")
    if k % BLOCK or n % BLOCK or k == 0:
        raise ValueError(f"K={k} must be a positive multiple of 128 and N={n} a multiple of 128")
    kb = k // BLOCK
    if tuple(sa.shape) != (total_m, kb):
        raise ValueError(f"sa must be [{total_m}, {kb}]")
    if tuple(sb.shape) != (e, n // BLOCK, kb) or not sb.is_contiguous():
        raise ValueError(f"sb must be contiguous [{e}, {n // BLOCK}, {kb}]")
    out = torch.empty((total_m, n), dtype=out_dtype, device=a.device)
    _lib.call("hpfp8_gemm_grouped_blockwise_pow2" if pow2_scales else "hpfp8_gemm_grouped_blockwise", _ptr(a), _ld(a), _ptr(sa), sa.stride(0), sa.stride(1), _ptr(b), _ptr(sb),
              _ptr(offs), e, total_m, n, k, _ptr(out), n, _out_code(out_dtype), _stream())
    return out


def gemm_grouped_blockwise_t(a: torch.Tensor, sa: torch.Tensor, b_t: torch.Tensor, sb: torch.Tensor, offs: torch.Tensor,
                             out_dtype: torch.dtype = torch.bfloat16, pow2_scales: bool = False,
                             zero_unrouted: bool = True) -> torch.Tensor:
    """The input gradient of the grouped linear: rows of a[total_m, N] (grad_out codes, 1x128 along N) sorted by
    expert, b_t[K, E * N] the transposed codes of the stacked weight [E * N, K] (what
    ``quantize_128x128(w.view(E * N, K), with_transpose=True)`` or ``transpose_codes`` gives; any row stride),
    sb[E, N/128, K/128] the weight's block scales -> c[total_m, K]: rows of expert e = a_e . W_e.  With
    ``zero_unrouted`` the rows past offs[-1] are set to zero (on the device, no host read of offs)."""
    a = _check_codes_2d(a, "a")
    b_t = _check_codes_2d(b_t, "b_t")
    sa = _check_f32(sa, "sa")
    sb = _check_f32(sb, "sb")
    _check_offs(offs)
    total_m, n = a.shape
    e = offs.numel()
    k = b_t.shape[0]
    if sb.dim() != 3 or e == 0 or b_t.shape[1] != e * n or tuple(sb.shape) != (e, n // BLOCK, k // BLOCK) or not sb.is_contiguous():
        raise ValueError(f"b_t must be [K, E * N] = [{k}, {e * n}] and sb contiguous [E, N/128, K/128]")
    if k % BLOCK or n % BLOCK or n == 0:
        raise ValueError(f"K={k} and N={n} must be multiples of 128, N positive")
    if tuple(sa.shape) != (total_m, n // BLOCK):
        raise ValueError(f"sa must be [{total_m}, {n // BLOCK}]")
    out = torch.empty((total_m, k), dtype=out_dtype, device=a.device)
    # the GEMM behind it: rows of b = K, contraction = N; expert e's operand starts N bytes after its predecessor's
    _lib.call("hpfp8_gemm_grouped_blockwise_strided", _ptr(a), _ld(a), _ptr(sa), sa.stride(0), sa.stride(1), _ptr(b_t), _ld(b_t),
              n, _ptr(sb), sb.stride(0), 1, k // BLOCK, _ptr(offs), e, total_m, k, n, _ptr(out), k, _out_code(out_dtype),
              int(pow2_scales), _stream())
    if zero_unrouted and out_dtype == torch.bfloat16:
        _lib.call("hpfp8_grouped_zero_unrouted_rows_bf16", _ptr(out), k, _ptr(offs), e, total_m, k, _stream())
    elif zero_unrouted:
        raise ValueError("zero_unrouted is implemented for bfloat16 output")
    return out


def grouped_padded_rows(experts: int, total_m: int) -> int:
    """Columns of the padded token axis the grouped wgrad operands live on: (total_m // 128 + experts) * 128."""
    return (total_m // BLOCK + experts) * BLOCK


def grouped_layout(offs: torch.Tensor, total_m: int) -> torch.Tensor:
    """The device-side table (int32) that places every expert's 128-token blocks on the padded token axis, made
    from offs[E] (inclusive prefix sums of rows per expert) without a host read: per expert {first row, rows, first
    padded block, blocks}, the experts ordered by block count, the number of blocks in use, each block's owner."""
    _check_offs(offs)
    e = offs.numel()
    words = 5 * e + 1 + (total_m // BLOCK + e)
    layout = torch.empty((words,), dtype=torch.int32, device=offs.device)
    _lib.call("hpfp8_grouped_layout", _ptr(offs), e, total_m, _ptr(layout), _stream())
    return layout


def quantize_128x1_t_grouped(x: torch.Tensor, layout: torch.Tensor, experts: int, with_1x128: bool = False):
    """The wgrad operand of x[total_m, K] (rows sorted by expert) for the grouped weight gradient: transposed 128x1
    codes on the padded token axis of ``layout`` -- (codes_t[K, P], scale_inv_t[K, P/128]) with P =
    ``grouped_padded_rows``, every expert's groups counted from its own first row, its last group filled up with
    zero codes; blocks beyond those in use are left uninitialised.  With ``with_1x128`` also the 1x128 form of the
    same read, (codes[total_m, K], scale_inv[total_m, K/128]) first; rows that belong to no expert stay
    uninitialised there."""
    x = _check_bf16(x, "x")
    if x.dim() != 2 or x.shape[1] % BLOCK:
        raise ValueError("x must be [total_m, K] with K a multiple of 128")
    _check_device(layout, "layout")
    total_m, k = x.shape
    if layout.dtype != torch.int32 or layout.numel() != 5 * experts + 1 + (total_m // BLOCK + experts) or not layout.is_contiguous():
        raise ValueError("layout does not belong to this expert count and row count")
    p = grouped_padded_rows(experts, total_m)
    qt = _empty_codes_t(k, p, x.device)
    st_inv = torch.empty((p // BLOCK, k), dtype=torch.float32, device=x.device)
    q = s_inv = None
    if with_1x128:
        q = torch.empty((total_m, k), dtype=FP8, device=x.device)
        s_inv = torch.empty((k // BLOCK, total_m), dtype=torch.float32, device=x.device)
    _lib.call("hpfp8_quantize_128x1_t_grouped_bf16", _ptr(x), total_m, k, _ptr(layout), experts, _ptr(qt), _ld(qt),
              _ptr(st_inv), _ptr(q), _ptr(s_inv), _stream())
    if with_1x128:
        return q, s_inv.t(), qt, st_inv.t()
    return qt, st_inv.t()


def gemm_grouped_wgrad(got: torch.Tensor, sgot: torch.Tensor, xt: torch.Tensor, sxt: torch.Tensor, layout: torch.Tensor,
                       experts: int, total_m: int, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """dW[E, N, K]: dW[e] = grad_out_e^T . x_e over expert e's own tokens.  got[N, P] / xt[K, P] and their scales
    [N, P/128] / [K, P/128] are what ``quantize_128x1_t_grouped`` returns for grad_out and x with the same layout."""
    got = _check_codes_2d(got, "got")
    xt = _check_codes_2d(xt, "xt")
    sgot = _check_f32(sgot, "sgot")
    sxt = _check_f32(sxt, "sxt")
    _check_device(layout, "layout")
    p = grouped_padded_rows(experts, total_m)
    n, k = got.shape[0], xt.shape[0]
    if got.shape[1] != p or xt.shape[1] != p or n % BLOCK or k % BLOCK:
        raise ValueError(f"operands must be [N, {p}] and [K, {p}] with N and K multiples of 128")
    for name, s_, rows in (("sgot", sgot, n), ("sxt", sxt, k)):
        if tuple(s_.shape) != (rows, p // BLOCK) or s_.stride(0) != 1 or (p > BLOCK and s_.stride(1) != rows):
            raise ValueError(f"{name} must be the block-major [{rows}, {p // BLOCK}] scales the grouped quantizer returns")
    if layout.dtype != torch.int32 or layout.numel() != 5 * experts + 1 + (total_m // BLOCK + experts):
        raise ValueError("layout does not belong to this expert count and row count")
    out = torch.empty((experts, n, k), dtype=out_dtype, device=got.device)
    _lib.call("hpfp8_gemm_grouped_wgrad", _ptr(got), _ld(got), _ptr(sgot), _ptr(xt), _ld(xt), _ptr(sxt), _ptr(layout),
              experts, total_m, n, k, _ptr(out), _out_code(out_dtype), _stream())
    return out
