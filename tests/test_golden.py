"""The oracle (both implementations) against the committed golden fixtures."""
import os

import numpy as np
import pytest

from oracle import fp8_oracle as O
from oracle import c_oracle as C
import _util as U

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_path_golden.npz"))


@pytest.mark.parametrize("impl", [O, C], ids=["python", "c"])
def test_quantizers_match_golden(impl):
    xb = G["x_bits"]
    q, s, si = impl.quantize_per_tensor(xb)
    assert np.array_equal(q, G["pt_codes"]) and np.float32(s) == G["pt_scale"] and np.float32(si) == G["pt_scale_inv"]
    for name, key in (("quantize_1x128", "g1x128"), ("quantize_128x128", "b128"), ("quantize_128x1_t", "t128x1")):
        q, s, si = getattr(impl, name)(xb)
        assert np.array_equal(q, G[key + "_codes"]), name
        assert np.array_equal(U.f32_bits(s), U.f32_bits(G[key + "_scale"])), name
        assert np.array_equal(U.f32_bits(si), U.f32_bits(G[key + "_scale_inv"])), name
    assert np.array_equal(impl.dequantize_1x128(G["g1x128_codes"], G["g1x128_scale_inv"]), G["g1x128_dequant_bits"])


def test_gemm_matches_golden():
    aq, _, asi = O.quantize_1x128(G["gemm_a_bits"])
    wq, _, wsi = O.quantize_128x128(G["gemm_w_bits"])
    bias = O.bf16_bits_to_f32(G["gemm_bias_bits"])
    y, yb = O.gemm_blockwise(aq, asi, wq, wsi, bias)
    assert np.allclose(y, G["gemm_y_f32"], rtol=1e-6, atol=1e-7)
    assert (yb != G["gemm_y_bits"]).mean() < 1e-3          # BLAS summation order may flip a last bf16 bit
    yc, _ = C.gemm_blockwise(aq, asi, wq, wsi, bias_f32=bias)
    assert np.allclose(yc, G["gemm_y_f32"], rtol=1e-5, atol=1e-6)
    wq1, _, wsi1 = O.quantize_1x128(G["gemm_w_bits"])
    y2, _ = O.gemm_rowwise_both(aq, asi, wq1, wsi1)
    assert np.allclose(y2, G["gemm_rows_y_f32"], rtol=1e-6, atol=1e-7)


def test_bucket_matches_golden():
    c, s, si = O.quantize_bucket(G["bucket_bits"])
    assert np.array_equal(c, G["bucket_codes"]) and np.array_equal(U.f32_bits(si), U.f32_bits(G["bucket_scale_inv"]))
    assert np.array_equal(O.dequantize_bucket(c, si, grad_scale=0.125), G["bucket_back_bits"])


def test_power_of_two_recipe_matches_golden():
    """The optional recipe's fixture: same input tensor, scale_inv rounded up to powers of two."""
    P = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_pow2_golden.npz"))
    xb = G["x_bits"]
    for name, key in (("quantize_1x128", "g1x128"), ("quantize_128x128", "b128"), ("quantize_128x1_t", "t128x1")):
        q, s, si = getattr(O, name)(xb, pow2=True)
        assert np.array_equal(q, P[key + "_codes"]), name
        assert np.array_equal(U.f32_bits(s), U.f32_bits(P[key + "_scale"])), name
        assert np.array_equal(U.f32_bits(si), U.f32_bits(P[key + "_scale_inv"])), name
        assert not (U.f32_bits(si) & 0x007FFFFF).any()
        assert (P[key + "_codes"] != G[key + "_codes"]).any()          # a different quantization, not a copy
    aq, _, asi = O.quantize_1x128(G["gemm_a_bits"], pow2=True)
    wq, _, wsi = O.quantize_128x128(G["gemm_w_bits"], pow2=True)
    y, _ = O.gemm_blockwise(aq, asi, wq, wsi, O.bf16_bits_to_f32(G["gemm_bias_bits"]))
    assert np.allclose(y, P["gemm_y_f32"], rtol=1e-6, atol=1e-7)
    assert np.linalg.norm(y - G["gemm_y_f32"]) / np.linalg.norm(G["gemm_y_f32"]) < 0.05
