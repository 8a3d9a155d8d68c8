"""GPU parity of the gate/up GEMM whose epilogue is SwiGLU + the 1x128 quantization of the down projection's
input (hpfp8_gemm_blockwise_swiglu_quantize), through the C ABI.

The epilogue is specified as the composition of two operations that have their own parity tests: the blockwise
GEMM with bf16 output and the SwiGLU quantizer on that bf16 tensor.  So the fused call is held bit for bit to
(a) those two calls in a row on the GPU and (b), in the exactly specified form, the CPU oracle's
swiglu_quantize_1x128 applied to the bf16 gate/up tensor the GEMM wrote."""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
import _util as U

pytestmark = pytest.mark.gpu


def _operands(m, inter, k, seed, gpu, pow2=False, kmajor=True):
    import hpfp8
    x = U.randn_bf16((m, k), seed, 1.0, 0.001, 50.0).to(gpu)
    w = U.randn_bf16((2 * inter, k), seed + 1, 0.05).to(gpu)
    xq, sx = hpfp8.quantize_1x128(x, kmajor=kmajor, pow2=pow2)
    wq, sw = hpfp8.quantize_128x128(w, pow2=pow2)
    return xq, sx, wq, sw


def _same(a, b):
    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("fast", [False, True])
@pytest.mark.parametrize("shape", [(256, 128, 128), (64, 256, 256), (300, 384, 512), (1000, 640, 384), (1, 128, 256),
                                   (513, 1152, 1024)])
def test_epilogue_equals_gemm_then_swiglu_quantizer(gpu, shape, fast):
    """Codes, scale_inv and scale of the fused call equal, bit for bit, the bf16 GEMM followed by the SwiGLU
    quantizer; in the exact form they also equal the oracle's SwiGLU quantization of the GEMM's bf16 output.
    Shapes cover a single tile, ragged row counts (the last row tile's rows past M are dropped), several
    scaling groups per row and both layouts of the activation scales."""
    import hpfp8
    m, inter, k = shape
    for kmajor in (True, False):
        xq, sx, wq, sw = _operands(m, inter, k, 11 + m, gpu, kmajor=kmajor)
        h = hpfp8.gemm_blockwise(xq, sx, wq, sw)
        q1, si1 = hpfp8.swiglu_quantize_1x128(h, kmajor=True, fast=fast)
        q, si, s = hpfp8.gemm_blockwise_swiglu_quantize(xq, sx, wq, sw, fast=fast, want_scale=True)
        assert q.shape == (m, inter) and si.shape == (m, inter // 128) and (si.stride(0) == 1 or m == 1)
        assert _same(q, q1), f"codes differ in {int((q.view(torch.uint8) != q1.view(torch.uint8)).sum())} places"
        assert torch.equal(si.contiguous().view(torch.int32), si1.contiguous().view(torch.int32))
        if not fast:
            rq, rs, rsi, _ = O.swiglu_quantize_1x128(U.bits(h))
            assert np.array_equal(U.codes(q), rq)
            assert np.array_equal(U.f32_bits(U.f32(si)), U.f32_bits(rsi))
            assert np.array_equal(U.f32_bits(U.f32(s)), U.f32_bits(rs))


def test_epilogue_with_power_of_two_scales(gpu):
    """The optional recipe: operand scales that are powers of two (applied by the matrix instruction) and / or
    power-of-two scales for the activation -- each combination equals its two unfused calls."""
    import hpfp8
    m, inter, k = 384, 256, 512
    for pow2_in in (False, True):
        xq, sx, wq, sw = _operands(m, inter, k, 5, gpu, pow2=pow2_in)
        h = hpfp8.gemm_blockwise(xq, sx, wq, sw, pow2_scales=pow2_in)
        for pow2_out in (False, True):
            for fast in (False, True):
                q1, si1 = hpfp8.swiglu_quantize_1x128(h, kmajor=True, pow2=pow2_out, fast=fast)
                q, si = hpfp8.gemm_blockwise_swiglu_quantize(xq, sx, wq, sw, fast=fast, pow2_scales=pow2_in,
                                                             pow2_out=pow2_out)
                assert _same(q, q1) and torch.equal(si.contiguous(), si1.contiguous())


def test_epilogue_extreme_gate_values(gpu):
    """Gate values far outside the exponential's range (saturating silu to 0 or to the identity), zeros and a
    non-finite activation group: same codes and scales as the unfused calls, NaN in the same places."""
    import hpfp8
    m, inter, k = 256, 256, 128
    x = torch.zeros((m, k), dtype=torch.bfloat16)
    x[:, 0] = 1.0
    w = U.randn_bf16((2 * inter, k), 3, 0.01)
    w[:inter, 0] = torch.linspace(-300.0, 300.0, inter).to(torch.bfloat16)      # gate = that ramp (plus noise * 0)
    w[inter:, 0] = 2.0
    x[7, 0] = float("inf")                                                        # one row of non-finite outputs
    xq, sx = hpfp8.quantize_1x128(x.to(gpu), kmajor=True)
    wq, sw = hpfp8.quantize_128x128(w.to(gpu))
    h = hpfp8.gemm_blockwise(xq, sx, wq, sw)
    for fast in (False, True):
        q1, si1 = hpfp8.swiglu_quantize_1x128(h, kmajor=True, fast=fast)
        q, si = hpfp8.gemm_blockwise_swiglu_quantize(xq, sx, wq, sw, fast=fast)
        assert np.array_equal(U.canon_nan_codes(U.codes(q)), U.canon_nan_codes(U.codes(q1)))
        assert U.same_f32_or_nan(U.f32(si), U.f32(si1))


def test_epilogue_at_full_size(gpu):
    """BASELINE configuration 2's gate/up projection (4096 x 36864 x 7168, activation 4096 x 18432): fused
    call against the two unfused calls, whole outputs, both forms; and the inference MLP block built on it
    against the same block built from the unfused calls."""
    import hpfp8
    m, inter, k = 4096, 18432, 7168
    xq, sx, wq, sw = _operands(m, inter, k, 21, gpu)
    h = hpfp8.gemm_blockwise(xq, sx, wq, sw)
    for fast in (False, True):
        q1, si1 = hpfp8.swiglu_quantize_1x128(h, kmajor=True, fast=fast)
        q, si = hpfp8.gemm_blockwise_swiglu_quantize(xq, sx, wq, sw, fast=fast)
        assert _same(q, q1) and torch.equal(si.contiguous(), si1.contiguous())
    del h
    x = U.randn_bf16((m, k), 22, 1.0).to(gpu)
    gu = hpfp8.Fp8Weight(wq, sw, None, False)
    dn = hpfp8.quantize_weight(U.randn_bf16((k, inter), 23, 0.02).to(gpu), with_transpose=False)
    y = hpfp8.fp8_swiglu_mlp(x, gu, dn, fast=True)
    xq2, sx2 = hpfp8.quantize_1x128(x, kmajor=True)
    h2 = hpfp8.gemm_blockwise(xq2, sx2, gu.codes, gu.scale_inv)
    aq, sa = hpfp8.swiglu_quantize_1x128(h2, kmajor=True, fast=True)
    y2 = hpfp8.gemm_blockwise(aq, sa, dn.codes, dn.scale_inv)
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))


def test_epilogue_argument_checks(gpu):
    import hpfp8
    xq, sx, wq, sw = _operands(128, 128, 128, 1, gpu)
    with pytest.raises(ValueError):
        hpfp8.gemm_blockwise_swiglu_quantize(xq, sx, wq[:128], sw[:1])          # 128 weight rows: no gate/up pair
    with pytest.raises((ValueError, TypeError)):
        hpfp8.gemm_blockwise_swiglu_quantize(xq.cpu(), sx, wq, sw)
    with pytest.raises(ValueError):
        hpfp8.gemm_blockwise_swiglu_quantize(xq, sx[:, :0], wq, sw)
