"""CPU oracle for the FP8 mixed-precision linear path.  TEST INFRASTRUCTURE ONLY.

Nothing that ships may import this module: only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py use it, and only as the checker.

What it restates
----------------
The reference checkout (mindspore-ai/hyper-parallel) holds no FP8 arithmetic, so there is no
reference quantizer or scaled GEMM to follow line by line.  The oracle therefore restates

  * the numeric recipe the benchmark configuration text fixes ("amax->scale=448/amax, cast,
    GEMM with fp32 accumulation, bf16 out"; "1x128 activation scales", "128x128 block scales",
    "128x1 transposed requant", "1x128 group scales to E4M3 + fp32 scales"), and
  * the calling conventions of the reference call sites the FP8 path slots into:
      - linear operand roles, weight [out, in], contraction over the last dim of both:
        hyper_parallel/core/shard/ops/parallel_matmul.py:377-381
      - flat gradient bucket, cast -> (reduce) -> cast back -> * grad_scale:
        hyper_parallel/core/hsdp/hsdp_grad_buffer.py:95-108 and :116-135

Numeric conventions (all fp32, IEEE, round-to-nearest-even, denormals kept):
  amax      = max(|x|) with x promoted bf16 -> fp32 (exact, order free)
  amax_c    = max(amax, 1e-12f)
  scale     = 448.0f / amax_c          (quantize multiplier, one correctly rounded division)
  scale_inv = amax_c / 448.0f          (dequantize / GEMM-epilogue multiplier, one division)
  code      = e4m3fn_rne( clamp(float(x) * scale, -448, 448) )
  dequant   = bf16_rne( decode(code) * scale_inv )
  gemm      = sum over 128-wide k-blocks, ascending, of
              (sum_k decode(a)*decode(b)) * (sa_inv * sb_inv); bias added in fp32; one final
              rounding to bf16.
Non-finite inputs follow from the same formulas under IEEE rules, with amax and clamp keeping NaN as
torch's eager amax / clamp do: a NaN in a scaling group makes the group's scale, scale_inv and all of
its codes NaN; +-Inf makes scale 0 and scale_inv Inf, the group's finite elements +-0 and the
infinite ones NaN.  Either way the dequantized group (and every GEMM output row or column it feeds)
is NaN throughout, so an overflow check downstream sees it.  Which of the two NaN codes (0x7F, 0xFF)
a cast writes is not specified.

How each function is pinned (tests/test_oracle_pins.py)
-------------------------------------------------------
  e4m3_decode / e4m3_encode : closed form of the OCP 8-bit format (1-4-3, bias 7, max 448,
      NaN = S.1111.111, subnormals k*2^-9) checked against torch's float8_e4m3fn cast for all
      256 codes, all 65536 bf16 bit patterns, every rounding midpoint and its fp32
      neighbours, and a hand-written known-answer table.
  amax, scales              : brute force on tiny inputs; special cases amax = 0 and
      amax < 448/FLT_MAX; NaN / Inf groups against the recipe written with torch's eager operators.
  quantize_*                : each blocked variant equals the per-tensor quantizer applied to
      every block separately (pure-Python loops on small shapes); the transposed variant
      equals quantize_1x128(x.T); the C restatement (fp8_oracle.c) is a second independent
      implementation compared bit for bit.
  scales_from_amax(pow2)    : closed form (a power of two, >= amax/448 and < 2 amax/448, times its
      reciprocal exactly 1, no product beyond 448); the quantizers with it are the ordinary ones
      with that scale (scalar loop with torch's cast); the C restatement derives the same scales from
      frexpf / ldexpf.
  exp_spec, swiglu          : numpy's exp and torch's eager F.silu(gate) * up within their rounding; the C
      restatement (nearbyintf, ldexpf, scalar loop) bit for bit.
  gemm_*                    : torch._scaled_mm on CPU for per-tensor scales (library routine);
      exact integer-valued inputs with unit scales reduce to an exact integer matmul; the
      grouped variant equals a loop of dense calls; float64 dequant matmul bounds the rest.
  dequantize_1x128_accumulate, dequantize_per_tensor_f32 : torch's float8 decode and a scalar loop in torch's fp32
      arithmetic; the association of the two multiplications is pinned by a case where the other one differs.
  swiglu_backward           : torch's float64 autograd of the same graph and closed-form points; its docstring
      states the tolerance contract the device kernel is held to (it uses hardware approximations).
  grouped_layout, quantize_128x1_t_grouped, gemm_grouped_wgrad : hand-computed block tables for ragged, empty and
      malformed offsets; every expert's piece equals quantize_1x128 of that expert's zero-padded rows transposed;
      the weight gradient equals the float64 product of the dequantized per-expert operands and is unchanged by
      the zero padding.
  column_sum                : exact integer column sums on integer-valued inputs (any order of additions is exact
      there, so a dropped or doubled row or a wrong column shows); float64 sums within the fp32 error bound of a
      sum of that many terms; and hand-derived answers on inputs built so that a different order of the fp32
      additions rounds differently (2^24 followed by ones), which pins the order stated in its docstring.
No function here is "parity unpinned" in the mathematical sense; what IS unpinned is parity
with the reference, because the reference has no FP8 code to compare with.
"""
from __future__ import annotations

import numpy as np

FP8_MAX = np.float32(448.0)
AMAX_EPS = np.float32(1e-12)
BLOCK = 128

__all__ = [
    "FP8_MAX", "AMAX_EPS", "BLOCK",
    "bf16_bits_to_f32", "f32_to_bf16_bits", "e4m3_decode", "e4m3_encode",
    "amax", "scales_from_amax", "quantize_per_tensor", "quantize_1x128",
    "quantize_128x128", "quantize_128x1_t", "dequantize_per_tensor", "dequantize_1x128",
    "dequantize_128x128", "quantize_bucket", "dequantize_bucket",
    "gemm_per_tensor", "gemm_blockwise", "gemm_rowwise_both", "gemm_grouped_blockwise",
    "gemm_dequant_f64", "dequantize_per_tensor_f32", "swiglu_backward",
    "grouped_layout", "quantize_128x1_t_grouped", "gemm_grouped_wgrad", "column_sum",
]


# --------------------------------------------------------------------------------------
# bf16 <-> fp32 (bit level).  Tensors travel as uint16 bit patterns so numpy can hold them.
# --------------------------------------------------------------------------------------
def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    """bf16 bit patterns (uint16) -> fp32 values; exact (bf16 is the top half of fp32)."""
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns, round-to-nearest-even; NaN stays NaN (quiet bit forced)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    rounded = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    is_nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    nan_bits = (u >> np.uint32(16)) | np.uint32(0x0040)
    return np.where(is_nan, nan_bits, rounded).astype(np.uint16)


# --------------------------------------------------------------------------------------
# E4M3FN: sign(1) exponent(4, bias 7) mantissa(3).  No Inf.  0x7F / 0xFF are NaN.
# --------------------------------------------------------------------------------------
def e4m3_decode(codes: np.ndarray) -> np.ndarray:
    """uint8 E4M3FN codes -> fp32 values (exact)."""
    c = np.ascontiguousarray(codes, dtype=np.uint8).astype(np.int32)
    sign = np.where(c & 0x80, np.float32(-1.0), np.float32(1.0))
    e = (c >> 3) & 0xF
    m = c & 0x7
    normal = np.ldexp((8 + m).astype(np.float32), e - 10)      # (1 + m/8) * 2^(e-7)
    subnormal = np.ldexp(m.astype(np.float32), -9)               # m * 2^-9
    mag = np.where(e == 0, subnormal, normal).astype(np.float32)
    out = (sign * mag).astype(np.float32)
    out = np.where((c & 0x7F) == 0x7F, np.float32(np.nan), out)
    return out.astype(np.float32)


def e4m3_encode(x: np.ndarray) -> np.ndarray:
    """fp32 -> E4M3FN code, round-to-nearest-even, NOT saturating.

    |x| that rounds above 448 (i.e. |x| >= 464) and NaN give the NaN code 0x7F | sign, the
    behaviour of torch's float8_e4m3fn cast.  Callers clamp to +-448 first.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    sign = ((u >> np.uint32(24)) & np.uint32(0x80)).astype(np.uint32)
    a = u & np.uint32(0x7FFFFFFF)
    # normal target range |x| >= 2^-6: drop 20 mantissa bits with RNE, rebias 127 -> 7
    lsb = (a >> np.uint32(20)) & np.uint32(1)
    r = (a + np.uint32(0x7FFFF) + lsb) >> np.uint32(20)
    normal_code = r.astype(np.int64) - ((127 - 7) << 3)
    # subnormal target range |x| < 2^-6: code = rne(|x| * 2^9); 8 lands on the first normal
    small = a < np.uint32(0x3C800000)                                   # |x| < 2^-6
    mag = np.where(small, a, np.uint32(0)).view(np.float32).astype(np.float64)
    sub_code = np.rint(mag * 512.0).astype(np.int64)
    code = np.where(small, sub_code, normal_code)
    overflow = (code > 0x7E) | (a > np.uint32(0x7F800000)) | (a == np.uint32(0x7F800000))
    code = np.where(overflow, 0x7F, code).astype(np.uint32)
    return (code | sign).astype(np.uint8)


# --------------------------------------------------------------------------------------
# amax / scales
# --------------------------------------------------------------------------------------
def amax(x_f32: np.ndarray, axis=None, keepdims=False) -> np.ndarray:
    """max |x| in fp32."""
    return np.max(np.abs(np.asarray(x_f32, dtype=np.float32)), axis=axis,
                  keepdims=keepdims).astype(np.float32)


def scales_from_amax(am: np.ndarray, pow2: bool = False):
    """amax -> (scale, scale_inv), two independent correctly rounded fp32 divisions.

    pow2 (an optional recipe beyond the stated one, whose scales are plain fp32): scale_inv is rounded
    up to the next power of two -- its fp32 exponent field is then its E8M0 code, the form gfx950's
    block-scaled matrix instruction applies by itself -- and scale is its exact reciprocal."""
    am = np.asarray(am, dtype=np.float32)
    amc = np.maximum(am, AMAX_EPS).astype(np.float32)
    with np.errstate(over="ignore"):
        scale = (FP8_MAX / amc).astype(np.float32)
        scale_inv = (amc / FP8_MAX).astype(np.float32)
    if pow2:
        u = np.ascontiguousarray(scale_inv).view(np.uint32)
        up = (u & np.uint32(0xFF800000)) + np.uint32(0x00800000)
        scale_inv = np.where(((u & np.uint32(0x007FFFFF)) != 0) & (u < np.uint32(0x7F800000)), up, u).astype(np.uint32).view(np.float32).reshape(scale_inv.shape)
        with np.errstate(divide="ignore"):
            scale = (np.float32(1.0) / scale_inv).astype(np.float32)
    return scale, scale_inv


def _cast(x_f32: np.ndarray, scale: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore", invalid="ignore"):   # beyond fp32 range: +-Inf, clamped next; Inf * 0 and NaN stay NaN
        y = (np.asarray(x_f32, dtype=np.float32) * np.asarray(scale, dtype=np.float32)).astype(np.float32)
    y = np.clip(y, -FP8_MAX, FP8_MAX).astype(np.float32)
    return e4m3_encode(y)


# --------------------------------------------------------------------------------------
# quantizers.  x_bits are bf16 bit patterns (uint16) unless stated otherwise.
# --------------------------------------------------------------------------------------
def quantize_per_tensor(x_bits: np.ndarray):
    """One scale for the whole tensor.  Returns (codes u8 like x, scale f32[()], scale_inv)."""
    x = bf16_bits_to_f32(x_bits)
    am = amax(x) if x.size else np.float32(0.0)
    scale, scale_inv = scales_from_amax(am)
    return _cast(x, scale).reshape(x.shape), scale, scale_inv


def quantize_1x128(x_bits: np.ndarray, pow2: bool = False):
    """Row-wise groups of 128 along the last (contraction) dim.

    x[R, C], C % 128 == 0 -> codes[R, C], scale[R, C/128], scale_inv[R, C/128].
    """
    x = bf16_bits_to_f32(x_bits)
    r, c = x.shape
    if c % BLOCK:
        raise ValueError(f"last dim {c} is not a multiple of {BLOCK}")
    g = x.reshape(r, c // BLOCK, BLOCK)
    am = amax(g, axis=2) if g.size else np.zeros((r, c // BLOCK), np.float32)
    scale, scale_inv = scales_from_amax(am, pow2)
    codes = _cast(g, scale[:, :, None]).reshape(r, c)
    return codes, scale, scale_inv


def quantize_128x128(w_bits: np.ndarray, pow2: bool = False):
    """128x128 blocks.  w[R, C] (both % 128 == 0) -> codes[R, C], scale/scale_inv[R/128, C/128]."""
    w = bf16_bits_to_f32(w_bits)
    r, c = w.shape
    if r % BLOCK or c % BLOCK:
        raise ValueError(f"shape {w.shape} is not a multiple of {BLOCK} in both dims")
    g = w.reshape(r // BLOCK, BLOCK, c // BLOCK, BLOCK)
    am = amax(g, axis=(1, 3)) if g.size else np.zeros((r // BLOCK, c // BLOCK), np.float32)
    scale, scale_inv = scales_from_amax(am, pow2)
    codes = _cast(g, scale[:, None, :, None]).reshape(r, c)
    return codes, scale, scale_inv


def quantize_128x1_t(x_bits: np.ndarray, pow2: bool = False):
    """Transposed re-quantization for wgrad, always from the bf16 source.

    x[M, K] (M % 128 == 0) -> codes_t[K, M], scale_t/scale_inv_t[K, M/128], where each scale
    covers 128 consecutive rows of one column of x.
    """
    x = bf16_bits_to_f32(x_bits)
    m, k = x.shape
    if m % BLOCK:
        raise ValueError(f"row count {m} is not a multiple of {BLOCK}")
    g = x.reshape(m // BLOCK, BLOCK, k)
    am = amax(g, axis=1) if g.size else np.zeros((m // BLOCK, k), np.float32)   # [M/128, K]
    scale, scale_inv = scales_from_amax(am, pow2)
    codes = _cast(g, scale[:, None, :]).reshape(m, k)
    return (np.ascontiguousarray(codes.T), np.ascontiguousarray(scale.T),
            np.ascontiguousarray(scale_inv.T))


def _to_bf16_bits_product(vals_f32: np.ndarray, mult: np.ndarray) -> np.ndarray:
    with np.errstate(invalid="ignore"):                 # 0 * Inf of a group that held an Inf stays NaN
        return f32_to_bf16_bits((vals_f32 * np.asarray(mult, np.float32)).astype(np.float32))


def dequantize_per_tensor(codes: np.ndarray, scale_inv) -> np.ndarray:
    """codes * scale_inv -> bf16 bit patterns."""
    return _to_bf16_bits_product(e4m3_decode(codes), np.float32(scale_inv)).reshape(codes.shape)


def dequantize_per_tensor_f32(codes: np.ndarray, scale_inv) -> np.ndarray:
    """decode(codes) * scale_inv as fp32 values (one multiplication, no second rounding): the cast back of the
    per-parameter cast hook (hyper_parallel/core/hsdp/hsdp_grad_hook.py:32-40) when the original dtype is fp32."""
    with np.errstate(invalid="ignore"):
        return (e4m3_decode(codes) * np.float32(scale_inv)).astype(np.float32).reshape(np.shape(codes))


def dequantize_1x128(codes: np.ndarray, scale_inv: np.ndarray) -> np.ndarray:
    r, c = codes.shape
    v = e4m3_decode(codes).reshape(r, c // BLOCK, BLOCK)
    return _to_bf16_bits_product(v, scale_inv[:, :, None]).reshape(r, c)


def dequantize_128x128(codes: np.ndarray, scale_inv: np.ndarray) -> np.ndarray:
    r, c = codes.shape
    v = e4m3_decode(codes).reshape(r // BLOCK, BLOCK, c // BLOCK, BLOCK)
    return _to_bf16_bits_product(v, scale_inv[:, None, :, None]).reshape(r, c)


def quantize_bucket(flat_bits: np.ndarray):
    """Flat gradient bucket (1-D, numel % 128 == 0) -> codes[numel], scale_inv[numel/128].

    Same arithmetic as quantize_1x128 on view(-1, 128); the flat contiguous layout is the one
    the reference packs gradients into (hyper_parallel/core/hsdp/hsdp_grad_buffer.py:95-108).
    """
    flat_bits = np.asarray(flat_bits)
    if flat_bits.ndim != 1 or flat_bits.size % BLOCK:
        raise ValueError("bucket must be 1-D with numel a multiple of 128")
    codes, scale, scale_inv = quantize_1x128(flat_bits.reshape(-1, BLOCK))
    return codes.reshape(-1), scale.reshape(-1), scale_inv.reshape(-1)


def dequantize_bucket(codes: np.ndarray, scale_inv: np.ndarray, grad_scale: float = 1.0) -> np.ndarray:
    """Bucket back to bf16 bits; then `* grad_scale` in bf16 as the reference's cast-back site
    does (hsdp_grad_buffer.py:121-125: buffer.to(dtype) first, then buffer * grad_scale)."""
    bits = dequantize_1x128(codes.reshape(-1, BLOCK), scale_inv.reshape(-1, 1)).reshape(-1)
    if grad_scale != 1.0:
        v = (bf16_bits_to_f32(bits) * np.float32(grad_scale)).astype(np.float32)
        bits = f32_to_bf16_bits(v)
    return bits


def exp_spec(t: np.ndarray) -> np.ndarray:
    """The exponential the SwiGLU kernel defines, operation by operation in IEEE fp32 (no fused
    multiply-add): clamp to [-86, 89], k = rint(t * log2 e), r = t - k * ln2 in two steps, degree-6
    Taylor polynomial in Horner form, times 2^(k-1), times 2 (+inf beyond the largest float).  Not taken
    from the reference (which has no such kernel); pinned against numpy's exp in the tests."""
    f = np.float32
    t = np.minimum(np.maximum(np.asarray(t, f), f(-86.0)), f(89.0))
    k = np.rint(t * f(1.44269504))
    r = t - k * f(0.693359375)
    r = r - k * f(-2.12194440e-4)
    p = np.full_like(r, f(1.0) / f(720.0))
    for c in (f(1.0) / f(120.0), f(1.0) / f(24.0), f(1.0) / f(6.0), f(0.5), f(1.0), f(1.0)):
        p = p * r + c
    half = ((k.astype(np.int32) + 126).astype(np.uint32) << np.uint32(23)).view(f)
    with np.errstate(over="ignore"):
        return ((p * half).astype(f) * f(2.0)).astype(f)


def swiglu(h_bits: np.ndarray) -> np.ndarray:
    """bf16 bits of act = bf16(bf16(silu(gate)) * up) for h = [gate | up] (bf16 bits, [M, 2I]): the
    eager bf16 graph F.silu(gate) * up with its two roundings, silu(g) = g / (1 + exp(-g)) in fp32."""
    h_bits = np.asarray(h_bits, dtype=np.uint16)
    inter = h_bits.shape[-1] // 2
    g = bf16_bits_to_f32(h_bits[..., :inter])
    u = bf16_bits_to_f32(h_bits[..., inter:])
    s = (g / (np.float32(1.0) + exp_spec(-g))).astype(np.float32)
    s = bf16_bits_to_f32(f32_to_bf16_bits(s))
    return f32_to_bf16_bits((s * u).astype(np.float32))


def swiglu_quantize_1x128(h_bits: np.ndarray, pow2: bool = False):
    """(codes, scale, scale_inv, act bits) of the SwiGLU result quantized in 1x128 groups."""
    act = swiglu(h_bits)
    codes, scale, scale_inv = quantize_1x128(act, pow2)
    return codes, scale, scale_inv, act


def swiglu_backward(h_bits: np.ndarray, dact_bits: np.ndarray) -> np.ndarray:
    """bf16 bits of d gate | d up for act = bf16(silu(gate)) * up, h = [gate | up] ([M, 2I] bf16 bits), dact [M, I]:
        sig    = 1 / (1 + exp(-g))                     (fp32)
        silu   = g * sig                               (fp32)
        d up   = bf16( dact * bf16(silu) )             (the rounded silu is what forward multiplied up with)
        d gate = bf16( (dact * up) * (sig + silu * (1 - sig)) )
    every operation a separate fp32 rounding, in this order -- the order of the device kernel.

    TOLERANCE CONTRACT.  The device kernel takes sig from the hardware's base-2 exponential and reciprocal
    approximations (each within one unit in the last place of fp32), which no CPU reproduces bit for bit; here sig
    is the correctly rounded fp32 value of the exact sigmoid.  The two therefore agree to a few fp32 units in the last
    place before the final bf16 rounding: a device result is either the same bf16 value, or one bf16 step away
    where the fp32 value sits next to a rounding boundary (d up: two steps where the bf16 rounding of silu itself
    was such a near-tie), or -- for d gate near gate = -1.278, where sig + silu (1 - sig) passes through zero and its
    terms cancel -- within 1e-3 * |dact * up| absolutely.  tests/test_gpu_linear.py holds the kernel to exactly
    this, with the fraction of differing elements bounded."""
    f = np.float32
    h_bits = np.asarray(h_bits, dtype=np.uint16)
    inter = h_bits.shape[-1] // 2
    g = bf16_bits_to_f32(h_bits[..., :inter])
    u = bf16_bits_to_f32(h_bits[..., inter:])
    d = bf16_bits_to_f32(np.asarray(dact_bits, dtype=np.uint16))
    with np.errstate(over="ignore"):
        sig = (1.0 / (1.0 + np.exp(-g.astype(np.float64)))).astype(f)
    silu = (g * sig).astype(f)
    silu_b = bf16_bits_to_f32(f32_to_bf16_bits(silu))
    du = (d * silu_b).astype(f)
    one_minus = (f(1.0) - sig).astype(f)
    deriv = (sig + (silu * one_minus).astype(f)).astype(f)
    dg = ((d * u).astype(f) * deriv).astype(f)
    return np.concatenate([f32_to_bf16_bits(dg), f32_to_bf16_bits(du)], axis=-1)


def dequantize_1x128_accumulate(codes: np.ndarray, scale_inv: np.ndarray, main_grad: np.ndarray,
                                grad_scale: float = 1.0) -> np.ndarray:
    """main_grad + (decode(codes) * scale_inv) * grad_scale in fp32, operation by operation: the
    `main_grad += reduced_grad` of hyper_parallel/platform/torch/fully_shard/param.py:160-167 with the
    reduced gradient held as E4M3 codes and 1x128 scales."""
    f = np.float32
    v = e4m3_decode(codes).astype(f).reshape(-1, BLOCK)
    v = (v * np.asarray(scale_inv, f).reshape(-1, 1)).astype(f)
    v = (v * f(grad_scale)).astype(f)
    return (np.asarray(main_grad, f).reshape(-1, BLOCK) + v).astype(f).reshape(np.shape(main_grad))


def bucket_offsets(numels):
    """Start of every parameter in a bucket row and the row length: the running index of
    hyper_parallel/core/hsdp/hsdp_grad_buffer.py:72-80, with every start rounded up to a multiple
    of 128 (so that no scaling group straddles two parameters)."""
    offsets, end = [], 0
    for n in numels:
        offsets.append(end)
        end = -(-(end + int(n)) // BLOCK) * BLOCK
    return offsets, end


def pack_bucket(grad_bits, numels, shard_size: int = 1) -> np.ndarray:
    """bf16 bit patterns of the packed bucket [shard_size, row_elems]: row s holds chunk s of every
    gradient at that parameter's offset (`buffer[:, start:end] = grad.view(shard_size, -1)`,
    hsdp_grad_buffer.py:95-108); padding is zero."""
    offsets, row = bucket_offsets(numels)
    out = np.zeros((shard_size, row), dtype=np.uint16)
    for g, n, o in zip(grad_bits, numels, offsets):
        g = np.asarray(g, dtype=np.uint16).reshape(-1)
        if g.size != shard_size * n:
            raise ValueError("gradient size does not match shard_size * numel")
        out[:, o:o + n] = g.reshape(shard_size, n)
    return out


def unpack_bucket(row_bits: np.ndarray, numels):
    """Pieces of one (reduced) bucket row, one per parameter (`buffer[:, start:end]`,
    hsdp_grad_buffer.py:126-135)."""
    offsets, row = bucket_offsets(numels)
    row_bits = np.asarray(row_bits).reshape(-1)
    if row_bits.size != row:
        raise ValueError("row has the wrong length")
    return [row_bits[o:o + n].copy() for n, o in zip(numels, offsets)]


# --------------------------------------------------------------------------------------
# GEMMs.  All return fp32 [M, N] before the final rounding plus the bf16 bit patterns.
# a: codes [M, K]; b: codes [N, K]  (weight layout [out, in], contraction on the last dim of
# both, hyper_parallel/core/shard/ops/parallel_matmul.py:377-381).
# --------------------------------------------------------------------------------------
def _finish(acc_f32: np.ndarray, bias_f32):
    if bias_f32 is not None:
        acc_f32 = (acc_f32 + np.asarray(bias_f32, np.float32)[None, :]).astype(np.float32)
    return acc_f32, f32_to_bf16_bits(acc_f32)


def gemm_per_tensor(a, sa_inv, b, sb_inv, bias_f32=None):
    """y = (A . B^T) * (sa_inv * sb_inv); fp32 accumulation over the whole K."""
    av, bv = e4m3_decode(a), e4m3_decode(b)
    acc = (av @ bv.T).astype(np.float32)
    s = np.float32(np.float32(sa_inv) * np.float32(sb_inv))
    return _finish((acc * s).astype(np.float32), bias_f32)


def gemm_blockwise(a, sa_inv, b, sb_inv, bias_f32=None):
    """a[M,K] with sa_inv[M,K/128]; b[N,K] with sb_inv[N/128,K/128]."""
    m, k = a.shape
    n = b.shape[0]
    av, bv = e4m3_decode(a), e4m3_decode(b)
    acc = np.zeros((m, n), np.float32)
    sb_rows = np.repeat(sb_inv, BLOCK, axis=0)                      # [N, K/128]
    for kb in range(k // BLOCK):
        sl = slice(kb * BLOCK, (kb + 1) * BLOCK)
        part = (av[:, sl] @ bv[:, sl].T).astype(np.float32)
        s = (sa_inv[:, kb].astype(np.float32)[:, None] * sb_rows[:, kb].astype(np.float32)[None, :])
        acc = (acc + part * s.astype(np.float32)).astype(np.float32)
    return _finish(acc, bias_f32)


def gemm_rowwise_both(a, sa_inv, b, sb_inv, bias_f32=None):
    """wgrad form: a[M,K] with sa_inv[M,K/128] and b[N,K] with sb_inv[N,K/128] (both 1x128)."""
    m, k = a.shape
    n = b.shape[0]
    av, bv = e4m3_decode(a), e4m3_decode(b)
    acc = np.zeros((m, n), np.float32)
    for kb in range(k // BLOCK):
        sl = slice(kb * BLOCK, (kb + 1) * BLOCK)
        part = (av[:, sl] @ bv[:, sl].T).astype(np.float32)
        s = sa_inv[:, kb].astype(np.float32)[:, None] * sb_inv[:, kb].astype(np.float32)[None, :]
        acc = (acc + part * s.astype(np.float32)).astype(np.float32)
    return _finish(acc, bias_f32)


def gemm_grouped_blockwise(a, sa_inv, b, sb_inv, offs):
    """MoE grouped form.  a[sumM, K] rows sorted by expert; b[E, N, K]; sb_inv[E, N/128, K/128];
    offs[E] inclusive prefix sums of per-expert row counts (a count may be 0)."""
    e_cnt, n, _ = b.shape
    out = np.zeros((a.shape[0], n), np.float32)
    start = 0
    for e in range(e_cnt):
        end = int(offs[e])
        if end > start:
            out[start:end], _ = gemm_blockwise(a[start:end], sa_inv[start:end], b[e], sb_inv[e])
        start = end
    return out, f32_to_bf16_bits(out)


def grouped_layout(offs, total_m: int):
    """Where every expert's 128-token blocks lie on the padded token axis of the grouped weight gradient:
    ([(first row, rows, first block, blocks) per expert], blocks in use).  offs are inclusive prefix sums of rows per
    expert, read clamped to [previous end, total_m] as the grouped GEMM reads them; an expert owns
    max(1, ceil(rows / 128)) blocks (an empty expert one block of zeros, which adds nothing to any sum).  The axis is
    allocated with (total_m // 128 + E) blocks, which always suffices."""
    table, prev, blk = [], 0, 0
    for off in np.asarray(offs).reshape(-1):
        end = min(max(int(off), prev), int(total_m))
        rows = end - prev
        nb = -(-rows // BLOCK) if rows > 0 else 1
        table.append((prev, rows, blk, nb))
        blk += nb
        prev = end
    return table, blk


def quantize_128x1_t_grouped(x_bits: np.ndarray, offs):
    """The wgrad operand of the MoE grouped linear: x[total_m, K] (rows sorted by expert) -> codes_t[K, P],
    scale_t / scale_inv_t[K, P/128] on the padded token axis (P = (total_m // 128 + E) * 128): expert e's rows,
    filled up with zero rows to whole blocks of 128, quantized like `quantize_128x1_t`, at that expert's blocks.
    Blocks no expert owns are returned as zeros (the device leaves them untouched)."""
    x_bits = np.asarray(x_bits, dtype=np.uint16)
    total_m, k = x_bits.shape
    table, _ = grouped_layout(offs, total_m)
    p = (total_m // BLOCK + len(table)) * BLOCK
    codes_t = np.zeros((k, p), np.uint8)
    scale_t = np.zeros((k, p // BLOCK), np.float32)
    scale_inv_t = np.zeros((k, p // BLOCK), np.float32)
    for start, rows, b0, nb in table:
        padded = np.zeros((nb * BLOCK, k), np.uint16)
        padded[:rows] = x_bits[start:start + rows]
        c, s_, si = quantize_128x1_t(padded)
        codes_t[:, b0 * BLOCK:(b0 + nb) * BLOCK] = c
        scale_t[:, b0:b0 + nb] = s_
        scale_inv_t[:, b0:b0 + nb] = si
    return codes_t, scale_t, scale_inv_t


def gemm_grouped_wgrad(got, sgot_inv, xt, sxt_inv, offs, total_m: int):
    """dW[E, N, K]: dW[e] = go_e^T . x_e, the contraction over expert e's own blocks of the padded token axis;
    got[N, P], xt[K, P] codes with scales [N, P/128], [K, P/128] (`quantize_128x1_t_grouped` of grad_out and x).
    Per expert this is `gemm_rowwise_both` on that expert's columns.  Returns (fp32, bf16 bits)."""
    table, _ = grouped_layout(offs, total_m)
    n, k = got.shape[0], xt.shape[0]
    out = np.zeros((len(table), n, k), np.float32)
    for e, (_, _, b0, nb) in enumerate(table):
        cols = slice(b0 * BLOCK, (b0 + nb) * BLOCK)
        out[e], _ = gemm_rowwise_both(got[:, cols], sgot_inv[:, b0:b0 + nb], xt[:, cols], sxt_inv[:, b0:b0 + nb])
    return out, f32_to_bf16_bits(out)


def column_sum(x_bits: np.ndarray):
    """Bias gradient of a linear whose grad_out is x[m, k] (bf16 bit patterns; k a multiple of 128): the sum over the
    rows, in fp32, in the order the device kernels add (the backward of the aten::linear the reference dispatches at
    hyper_parallel/core/shard/_op_dispatch.py:277-283 sums grad_out over the tokens in an order torch does not
    specify; this build fixes one so that the result is reproducible):
      * rows are taken in blocks of 128 (rows past m count as +0);
      * inside a block, 16 "row quads" rq = 0..15 each add their 8 rows onto +0 in the order 4rq, 4rq+1, 4rq+2,
        4rq+3, 64+4rq, ..., 64+4rq+3;
      * the quads combine four at a time: (q0 + q1) + (q2 + q3) for rq = 4w .. 4w+3, w = 0..3, and the four results
        as ((w0 + w1) + w2) + w3: the block's partial sum;
      * the partial sums are added onto +0 in block order; the total is rounded once to bf16.
    Returns (partial fp32 [ceil(m/128), k], total fp32 [k], total as bf16 bit patterns [k])."""
    f = np.float32
    x = bf16_bits_to_f32(np.asarray(x_bits))
    m, k = x.shape
    mb = (m + BLOCK - 1) // BLOCK
    xp = np.zeros((mb * BLOCK, k), dtype=f)
    xp[:m] = x
    xt = xp.reshape(mb, 2, 16, 4, k)                    # tile row = half * 64 + 4 * rq + j
    quad = np.zeros((mb, 16, k), dtype=f)
    for half in range(2):
        for j in range(4):
            quad = (quad + xt[:, half, :, j, :]).astype(f)
    quad = quad.reshape(mb, 4, 4, k)                    # [block, w, quad within w, column]
    wsum = ((quad[:, :, 0] + quad[:, :, 1]).astype(f) + (quad[:, :, 2] + quad[:, :, 3]).astype(f)).astype(f)
    part = (((wsum[:, 0] + wsum[:, 1]).astype(f) + wsum[:, 2]).astype(f) + wsum[:, 3]).astype(f)
    total = np.zeros((k,), dtype=f)
    for b in range(mb):
        total = (total + part[b]).astype(f)
    return part, total, f32_to_bf16_bits(total)


def gemm_dequant_f64(a, sa_rows_inv, b, sb_rows_inv):
    """Dequantize-then-matmul in float64: the acceptance criterion's right-hand side.

    sa_rows_inv[M, K/128] and sb_rows_inv[N, K/128] are per-row expansions of whatever block
    geometry was used (np.repeat a 128x128 grid along axis 0, broadcast a scalar, ...).
    """
    av = e4m3_decode(a).astype(np.float64) * np.repeat(np.asarray(sa_rows_inv, np.float64), BLOCK, axis=1)
    bv = e4m3_decode(b).astype(np.float64) * np.repeat(np.asarray(sb_rows_inv, np.float64), BLOCK, axis=1)
    return av @ bv.T
