"""Writes the golden fixtures in this directory from the oracle (oracle/fp8_oracle.py).

The reference checkout holds no FP8 code and no golden vectors for this path, so nothing here is
derived from running the reference; the fixtures freeze the oracle's conventions (so that it cannot
drift unnoticed) on small seeded inputs that include the corner cases: zero groups, groups below
the 1e-12 clamp, bf16 subnormals, +-448 ties, signed zeros.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import fp8_oracle as O  # noqa: E402
import _util as U  # noqa: E402


def main():
    out = {}
    # --- quantizers on a 256 x 384 tensor with outliers and special rows spliced in
    x = U.randn_bf16((256, 384), seed=1234, outlier_frac=0.001, outlier_mul=50.0)
    sp = U.special_bf16_rows(128)
    x[: sp.shape[0], :128] = sp
    x[128:128 + sp.shape[0], 256:384] = sp
    xb = U.bits(x)
    out["x_bits"] = xb
    q, s, si = O.quantize_per_tensor(xb)
    out["pt_codes"], out["pt_scale"], out["pt_scale_inv"] = q, np.float32(s), np.float32(si)
    q, s, si = O.quantize_1x128(xb)
    out["g1x128_codes"], out["g1x128_scale"], out["g1x128_scale_inv"] = q, s, si
    out["g1x128_dequant_bits"] = O.dequantize_1x128(q, si)
    q, s, si = O.quantize_128x128(xb)
    out["b128_codes"], out["b128_scale"], out["b128_scale_inv"] = q, s, si
    q, s, si = O.quantize_128x1_t(xb)
    out["t128x1_codes"], out["t128x1_scale"], out["t128x1_scale_inv"] = q, s, si

    # --- a small blockwise GEMM (M=64, N=128, K=256) with bias, and its wgrad-form sibling
    a = U.randn_bf16((64, 256), seed=77)
    w = U.randn_bf16((128, 256), seed=78, std=0.02)
    bias = U.randn_bf16((128,), seed=79, std=0.1)
    aq, _, asi = O.quantize_1x128(U.bits(a))
    wq, _, wsi = O.quantize_128x128(U.bits(w))
    y, yb = O.gemm_blockwise(aq, asi, wq, wsi, O.bf16_bits_to_f32(U.bits(bias)))
    out["gemm_a_bits"], out["gemm_w_bits"], out["gemm_bias_bits"] = U.bits(a), U.bits(w), U.bits(bias)
    out["gemm_y_f32"], out["gemm_y_bits"] = y, yb
    wq1, _, wsi1 = O.quantize_1x128(U.bits(w))
    y2, y2b = O.gemm_rowwise_both(aq, asi, wq1, wsi1)
    out["gemm_rows_y_f32"] = y2

    # --- bucket round trip with grad_scale
    g = U.randn_bf16((4096,), seed=5, std=1e-4, outlier_frac=1e-3, outlier_mul=1e3)
    c, s, si = O.quantize_bucket(U.bits(g))
    out["bucket_bits"], out["bucket_codes"], out["bucket_scale_inv"] = U.bits(g), c, si
    out["bucket_back_bits"] = O.dequantize_bucket(c, si, grad_scale=0.125)
    np.savez_compressed(os.path.join(HERE, "fp8_path_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "fp8_path_golden.npz"), {k: v.shape for k, v in out.items() if hasattr(v, "shape")})

    # --- the optional recipe with power-of-two scales, on the same tensor (input: x_bits of the file above)
    p2 = {}
    q, s, si = O.quantize_1x128(xb, pow2=True)
    p2["g1x128_codes"], p2["g1x128_scale"], p2["g1x128_scale_inv"] = q, s, si
    q, s, si = O.quantize_128x128(xb, pow2=True)
    p2["b128_codes"], p2["b128_scale"], p2["b128_scale_inv"] = q, s, si
    q, s, si = O.quantize_128x1_t(xb, pow2=True)
    p2["t128x1_codes"], p2["t128x1_scale"], p2["t128x1_scale_inv"] = q, s, si
    aq, _, asi = O.quantize_1x128(U.bits(a), pow2=True)
    wq, _, wsi = O.quantize_128x128(U.bits(w), pow2=True)
    p2["gemm_y_f32"], _ = O.gemm_blockwise(aq, asi, wq, wsi, O.bf16_bits_to_f32(U.bits(bias)))
    np.savez_compressed(os.path.join(HERE, "fp8_pow2_golden.npz"), **p2)
    print("wrote", os.path.join(HERE, "fp8_pow2_golden.npz"), {k: v.shape for k, v in p2.items()})


if __name__ == "__main__":
    torch.manual_seed(0)
    main()
