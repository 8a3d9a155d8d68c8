"""Pins the CPU oracle to facts it did not author: torch's float8_e4m3fn cast, the closed form of
the OCP E4M3FN format, brute force on small inputs, algebraic identities and a second, independently
written C implementation.  Every function of oracle/fp8_oracle.py is covered by at least one check
that a plausible slip (dropped term, wrong index, transposed operand, wrong rounding) would fail."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from oracle import c_oracle as C
import _util as U

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "e4m3_known_answers.json")))


def torch_encode(x_f32: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(x_f32, np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


# ---------------------------------------------------------------- E4M3 format
def test_decode_all_256_codes_against_torch_and_c():
    codes = np.arange(256, dtype=np.uint8)
    t = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).float().numpy()
    d = O.e4m3_decode(codes)
    c = C.e4m3_decode(codes)
    nan = np.isnan(t)
    assert nan.sum() == 2 and nan[0x7F] and nan[0xFF]
    assert np.array_equal(np.isnan(d), nan) and np.array_equal(np.isnan(c), nan)
    assert np.array_equal(d[~nan].view(np.uint32), t[~nan].view(np.uint32))
    assert np.array_equal(c[~nan].view(np.uint32), t[~nan].view(np.uint32))


def test_decode_known_answers():
    for code, val in KAT["decode"].items():
        got = O.e4m3_decode(np.array([int(code)], np.uint8))[0]
        assert got == np.float32(val) and np.signbit(got) == np.signbit(np.float32(val)), (code, got, val)


def test_encode_known_answers():
    for val, code in KAT["encode"]:
        assert O.e4m3_encode(np.array([val], np.float32))[0] == code, (val, code)
        assert C.e4m3_encode(np.array([val], np.float32))[0] == code, (val, code)


def test_encode_roundtrips_every_code():
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], np.uint8)
    assert np.array_equal(O.e4m3_encode(O.e4m3_decode(codes)), codes)


def test_encode_all_bf16_patterns_against_torch():
    b = np.arange(65536, dtype=np.uint16)
    x = O.bf16_bits_to_f32(b)
    assert np.array_equal(O.e4m3_encode(x), torch_encode(x))


def test_encode_midpoints_and_neighbours_against_torch_and_c():
    codes = np.arange(0, 0x7F, dtype=np.uint8)
    v = O.e4m3_decode(codes).astype(np.float64)
    mids = ((v[:-1] + v[1:]) / 2).astype(np.float32)          # exact in fp32
    pts = [mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
           np.array([448.0, 463.99997, 464.0, 480.0, 1e30, np.inf, np.nan, 0.0, 2.0 ** -10, 2.0 ** -11], np.float32)]
    x = np.concatenate(pts).astype(np.float32)
    x = np.concatenate([x, -x])
    ref = torch_encode(x)
    assert np.array_equal(O.e4m3_encode(x), ref)
    finite = np.isfinite(x)
    assert np.array_equal(C.e4m3_encode(x[finite]), ref[finite])
    # ties go to the even mantissa: the midpoint between codes c and c+1 lands on the even one
    got = O.e4m3_encode(mids)
    want = np.where(codes[:-1] % 2 == 0, codes[:-1], codes[1:])
    assert np.array_equal(got, want)


def test_encode_random_fp32_against_torch():
    rng = np.random.default_rng(7)
    u = rng.integers(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    x = u.view(np.float32)
    assert np.array_equal(O.e4m3_encode(x), torch_encode(x))
    sub = x[:20000]
    sub = sub[np.isfinite(sub)]
    assert np.array_equal(C.e4m3_encode(sub), torch_encode(sub))


# ---------------------------------------------------------------- bf16 conversion
def test_bf16_conversions_against_torch():
    rng = np.random.default_rng(3)
    x = rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 200000).astype(np.float32)
    x = np.concatenate([x, np.array([0.0, -0.0, np.inf, -np.inf, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8], np.float32)])
    want = U.bits(torch.from_numpy(x).to(torch.bfloat16))
    assert np.array_equal(O.f32_to_bf16_bits(x), want)
    assert np.array_equal(O.bf16_bits_to_f32(want).view(np.uint32), want.astype(np.uint32) << 16)


# ---------------------------------------------------------------- amax / scales
def test_scales_closed_form_and_special_cases():
    am = np.array([0.0, 1e-13, 1e-12, 2e-12, 1.0, 448.0, 3.0, 1.2e-38, 3.3895e38], np.float32)
    s, si = O.scales_from_amax(am)
    for a, sv, siv in zip(am, s, si):
        amc = max(np.float32(a), np.float32(1e-12))
        assert sv == np.float32(np.float32(448.0) / amc) and siv == np.float32(amc / np.float32(448.0))
    assert s[0] == s[1] == s[2] == np.float32(448.0) / np.float32(1e-12)   # eps clamp
    assert np.isfinite(s).all() and np.isfinite(si).all() and (si > 0).all()
    assert s[5] == 1.0 and si[5] == 1.0
    # the two multipliers are separate divisions, not reciprocals of each other
    assert si[6] == np.float32(np.float32(3.0) / np.float32(448.0))
    a = np.float32(3.0) / np.float32(7.0)
    s7, si7 = O.scales_from_amax(a)
    assert si7 == np.float32(a / np.float32(448.0)) and si7 != np.float32(np.float32(1.0) / s7)


def test_pow2_scales_closed_form():
    """The optional power-of-two recipe: scale_inv is the smallest power of two that is not below
    amax_c / 448 (as the fp32 quotient), scale is its exact reciprocal, and no value of the group can
    come out beyond 448.  Checked with exact arithmetic (math.frexp / Fraction), not with the bit trick."""
    import math
    from fractions import Fraction
    rng = np.random.default_rng(5)
    am = np.concatenate([
        np.array([0.0, 1e-13, 1e-12, 1.0, 448.0, 450.0, 446.0, 224.0, 896.0, 1.2e-38, 3.3895e38], np.float32),
        (448.0 * 2.0 ** rng.integers(-40, 41, size=40)).astype(np.float32),            # exact powers of two times 448
        np.exp(rng.uniform(-60, 60, size=2000)).astype(np.float32),
    ])
    am = U.from_bits(U.bits(torch.from_numpy(am).to(torch.bfloat16))).float().numpy()   # amax of bf16 data is a bf16 value
    s, si = O.scales_from_amax(am, pow2=True)
    _, q = O.scales_from_amax(am)
    for a, sv, siv, qv in zip(am, s, si, q):
        mant, _ = math.frexp(float(siv))
        assert mant == 0.5                                      # a power of two
        assert Fraction(float(siv)) >= Fraction(float(qv)) and Fraction(float(siv)) < 2 * Fraction(float(qv))
        assert Fraction(float(sv)) * Fraction(float(siv)) == 1
        assert Fraction(float(a)) * Fraction(float(sv)) <= 448  # exact product: the clamp never acts
    assert si[4] == 1.0 and si[5] == 2.0 and si[6] == 1.0 and si[7] == 0.5 and si[8] == 2.0
    assert si[0] == si[1] == si[2] == np.float32(2.0 ** -48)    # eps clamp: 1e-12 / 448 = 2.23e-15 -> 2^-48


def test_pow2_quantizers_are_the_ordinary_ones_with_that_scale():
    x = U.randn_bf16((128, 256), seed=23, outlier_frac=0.01, outlier_mul=50.0)
    x[:6, :128] = U.special_bf16_rows(128)[:6]
    xb = U.bits(x)
    xf = x.float().numpy()
    q, s, si = O.quantize_1x128(xb, pow2=True)
    for r in (0, 1, 2, 3, 4, 5, 77, 127):
        for g in range(2):
            blk = xf[r, g * 128:(g + 1) * 128]
            sv, siv = O.scales_from_amax(np.max(np.abs(blk)), pow2=True)
            want = torch_encode(np.clip(blk * sv, -448.0, 448.0).astype(np.float32))
            assert np.array_equal(q[r, g * 128:(g + 1) * 128], want) and s[r, g] == sv and si[r, g] == siv
    qw, sw, siw = O.quantize_128x128(xb, pow2=True)
    for g in range(2):
        blk = xf[:, g * 128:(g + 1) * 128]
        sv, siv = O.scales_from_amax(np.max(np.abs(blk)), pow2=True)
        assert np.array_equal(qw[:, g * 128:(g + 1) * 128], torch_encode(np.clip(blk * sv, -448.0, 448.0).astype(np.float32)))
        assert sw[0, g] == sv and siw[0, g] == siv
    qt, st, sit = O.quantize_128x1_t(xb, pow2=True)
    q2, s2, si2 = O.quantize_1x128(U.bits(x.t().contiguous()), pow2=True)
    assert np.array_equal(qt, q2) and np.array_equal(st, s2) and np.array_equal(sit, si2)


def test_amax_brute_force():
    x = U.randn_bf16((7, 33), seed=11)
    xf = x.float().numpy()
    best = 0.0
    for v in xf.reshape(-1):
        best = max(best, abs(float(v)))
    assert O.amax(xf) == np.float32(best)


# ---------------------------------------------------------------- quantizers
def _scalar_quantize_block(vals_f32):
    """Straight-line Python restatement used only on tiny blocks."""
    am = np.float32(0.0)
    for v in vals_f32:
        am = max(am, np.float32(abs(v)))
    amc = max(am, np.float32(1e-12))
    scale = np.float32(np.float32(448.0) / amc)
    scale_inv = np.float32(amc / np.float32(448.0))
    out = []
    for v in vals_f32:
        y = np.float32(np.float32(v) * scale)
        y = min(max(y, np.float32(-448.0)), np.float32(448.0))
        out.append(int(torch.tensor([y], dtype=torch.float32).to(torch.float8_e4m3fn).view(torch.uint8)[0]))
    return np.array(out, np.uint8), scale, scale_inv


def test_quantize_1x128_equals_blockwise_loop_with_torch_cast():
    x = U.randn_bf16((6, 256), seed=21, outlier_frac=0.01, outlier_mul=50.0)
    x[:, :128] = U.special_bf16_rows(128)[:6]
    xb = U.bits(x)
    q, s, si = O.quantize_1x128(xb)
    xf = x.float().numpy()
    for r in range(6):
        for gidx in range(2):
            qq, ss, ssi = _scalar_quantize_block(xf[r, gidx * 128:(gidx + 1) * 128])
            assert np.array_equal(q[r, gidx * 128:(gidx + 1) * 128], qq)
            assert s[r, gidx] == ss and si[r, gidx] == ssi


def test_special_rows_behave_as_documented():
    sp = U.special_bf16_rows(128)
    q, s, si = O.quantize_1x128(U.bits(sp))
    assert (q[0] == 0).all() and s[0, 0] == np.float32(448.0) / np.float32(1e-12)       # zero group
    assert q[3, 0] == 0xFE and q[3, -1] == 0x7E                                            # +-448 hit exactly
    assert q[4, 0] == 0x7E and q[4, 1] == 0xFE and q[4, 2] == 88 and q[4, 3] == 90        # scale 1: 17->16, 19->20
    assert q[6, 0] == 0x80 and q[6, 2] == 0x80 | O.e4m3_encode(np.float32([2.0 ** -10 * 448]))[0]
    assert not ((q & 0x7F) == 0x7F).any()                                                   # never NaN codes
    assert (q[9] == 0).sum() == 0 and s[9, 0] == np.float32(448.0) / np.float32(1e-12)    # below the clamp


def test_block_variants_reduce_to_per_tensor_on_each_block():
    x = U.randn_bf16((256, 256), seed=31, outlier_frac=0.002, outlier_mul=50.0)
    xb = U.bits(x)
    q, s, si = O.quantize_128x128(xb)
    for br in range(2):
        for bc in range(2):
            blk = np.ascontiguousarray(xb[br * 128:(br + 1) * 128, bc * 128:(bc + 1) * 128])
            qq, ss, ssi = O.quantize_per_tensor(blk)
            assert np.array_equal(q[br * 128:(br + 1) * 128, bc * 128:(bc + 1) * 128], qq)
            assert s[br, bc] == ss and si[br, bc] == ssi
    q1, s1, si1 = O.quantize_1x128(xb)
    for r in (0, 5, 255):
        qq, ss, ssi = O.quantize_per_tensor(np.ascontiguousarray(xb[r, 128:256]))
        assert np.array_equal(q1[r, 128:256], qq) and s1[r, 1] == ss and si1[r, 1] == ssi


def test_transposed_requant_is_rowwise_quantize_of_the_transpose():
    x = U.randn_bf16((256, 384), seed=41, outlier_frac=0.002, outlier_mul=50.0)
    xb = U.bits(x)
    qt, st, sit = O.quantize_128x1_t(xb)
    q, s, si = O.quantize_1x128(np.ascontiguousarray(xb.T))
    assert np.array_equal(qt, q) and np.array_equal(st, s) and np.array_equal(sit, si)


def test_bucket_is_1x128_on_the_flat_view_and_roundtrip_bound():
    g = U.randn_bf16((128 * 40,), seed=51, std=1e-4, outlier_frac=1e-3, outlier_mul=1e3)
    gb = U.bits(g)
    c, s, si = O.quantize_bucket(gb)
    q, s2, si2 = O.quantize_1x128(gb.reshape(-1, 128))
    assert np.array_equal(c, q.reshape(-1)) and np.array_equal(si, si2.reshape(-1))
    back = O.bf16_bits_to_f32(O.dequantize_bucket(c, si)).reshape(-1, 128)
    orig = O.bf16_bits_to_f32(gb).reshape(-1, 128)
    am = np.abs(orig).max(axis=1, keepdims=True)
    # half an E4M3 step in the top binade is amax/28; the bf16 rounding of the result adds at most
    # 2^-9 of the magnitude (<= amax/512)
    assert (np.abs(back - orig) <= am / 28 + am / 256 + 1e-30).all()
    # grad_scale is applied after the cast back, on bf16 values, with its own rounding
    scaled = O.dequantize_bucket(c, si, grad_scale=0.3)
    want = O.f32_to_bf16_bits((O.bf16_bits_to_f32(O.dequantize_bucket(c, si)) * np.float32(0.3)).astype(np.float32))
    assert np.array_equal(scaled, want)


def test_dequantize_matches_definition():
    x = U.randn_bf16((128, 256), seed=61)
    q, s, si = O.quantize_128x128(U.bits(x))
    d = O.bf16_bits_to_f32(O.dequantize_128x128(q, si))
    want = torch.from_numpy(O.e4m3_decode(q) * np.repeat(np.repeat(si, 128, 0), 128, 1)).to(torch.bfloat16).float().numpy()
    assert np.array_equal(d, want)
    qp, sp, sip = O.quantize_per_tensor(U.bits(x))
    dp = O.bf16_bits_to_f32(O.dequantize_per_tensor(qp, sip))
    wantp = torch.from_numpy(O.e4m3_decode(qp) * sip).to(torch.bfloat16).float().numpy()
    assert np.array_equal(dp, wantp)


# ---------------------------------------------------------------- C restatement, bit for bit
@pytest.mark.parametrize("name", ["quantize_1x128", "quantize_128x128", "quantize_128x1_t"])
def test_c_restatement_bit_exact(name):
    x = U.randn_bf16((256, 384), seed=71, outlier_frac=0.001, outlier_mul=50.0)
    x[:10, :128] = U.special_bf16_rows(128)
    xb = U.bits(x)
    a = getattr(O, name)(xb)
    b = getattr(C, name)(xb)
    assert np.array_equal(a[0], b[0])
    assert np.array_equal(U.f32_bits(a[1]), U.f32_bits(b[1])) and np.array_equal(U.f32_bits(a[2]), U.f32_bits(b[2]))


def test_c_per_tensor_and_dequant_bit_exact():
    x = U.randn_bf16((64, 256), seed=72)
    xb = U.bits(x)
    a, b = O.quantize_per_tensor(xb), C.quantize_per_tensor(xb)
    assert np.array_equal(a[0], b[0]) and a[1] == b[1] and a[2] == b[2]
    q, s, si = O.quantize_1x128(xb)
    assert np.array_equal(O.dequantize_1x128(q, si), C.dequantize_1x128(q, si))


# ---------------------------------------------------------------- non-finite inputs
def _torch_eager_quantize_groups(x: torch.Tensor):
    """The recipe spelled with torch's eager operators on [G, 128] groups: amax and clamp keep NaN."""
    xf = x.float()
    amc = xf.abs().amax(dim=1, keepdim=True).clamp(min=1e-12)
    scale = torch.tensor(448.0) / amc
    scale_inv = amc / torch.tensor(448.0)
    q = (xf * scale).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    return q.numpy(), scale.numpy().reshape(-1), scale_inv.numpy().reshape(-1)


def test_non_finite_inputs_follow_ieee_like_torch_eager_and_c():
    """NaN in a group: scale, scale_inv and every code of the group are NaN.  +-Inf: scale 0, scale_inv
    Inf, finite elements become +-0 and the infinite ones NaN.  Groups beside them are untouched."""
    x = U.nonfinite_bf16(256, 512)
    xb = U.bits(x)
    q, s, si = O.quantize_1x128(xb)
    tq, ts, tsi = _torch_eager_quantize_groups(x.reshape(-1, 128))
    assert np.array_equal(U.canon_nan_codes(q).reshape(-1, 128), U.canon_nan_codes(tq))
    assert U.same_f32_or_nan(s, ts) and U.same_f32_or_nan(si, tsi)
    assert np.isnan(s[0, 0]) and np.isnan(si[0, 0]) and ((q[0, :128] & 0x7F) == 0x7F).all()
    assert s[1, 1] == 0 and np.isposinf(si[1, 1]) and (q[1, 128 + 77] & 0x7F) == 0x7F
    assert ((np.delete(q[1, 128:256], 77) & 0x7F) == 0).all()
    assert np.isnan(s[2, 2]) and np.isnan(s[131, 3]) and np.isposinf(si[130, 0])
    clean = np.isfinite(si)
    assert clean.sum() == si.size - 5 and not ((q.reshape(256, 4, 128)[clean] & 0x7F) == 0x7F).any()
    # the other quantizers and the C restatement
    for name in ("quantize_1x128", "quantize_128x128", "quantize_128x1_t"):
        a, b = getattr(O, name)(xb), getattr(C, name)(xb)
        assert np.array_equal(U.canon_nan_codes(a[0]), U.canon_nan_codes(b[0])), name
        assert U.same_f32_or_nan(a[1], b[1]) and U.same_f32_or_nan(a[2], b[2]), name
    qw, sw, siw = O.quantize_128x128(xb)
    assert np.isnan(siw[0, 0]) and np.isnan(siw[0, 2]) and np.isposinf(siw[0, 1]) and np.isposinf(siw[1, 0]) and np.isnan(siw[1, 3])
    assert np.isfinite(siw).sum() == 3
    qt, st, sit = O.quantize_128x1_t(xb)
    q2, s2, si2 = O.quantize_1x128(np.ascontiguousarray(xb.T))
    assert np.array_equal(qt, q2) and U.same_f32_or_nan(sit, si2)
    a, b = O.quantize_per_tensor(xb), C.quantize_per_tensor(xb)
    assert np.isnan(a[1]) and np.isnan(b[1]) and ((a[0] & 0x7F) == 0x7F).all() and ((b[0] & 0x7F) == 0x7F).all()
    # dequantized, every affected group is NaN throughout: an overflow check on the result sees it
    d = O.bf16_bits_to_f32(O.dequantize_1x128(q, si)).reshape(256, 4, 128)
    assert np.isnan(d[~clean]).all() and np.isfinite(d[clean]).all()


# ---------------------------------------------------------------- GEMMs
def test_gemm_per_tensor_against_torch_scaled_mm():
    x = U.randn_bf16((64, 256), seed=81)
    w = U.randn_bf16((128, 256), seed=82, std=0.02)
    xq, _, sxi = O.quantize_per_tensor(U.bits(x))
    wq, _, swi = O.quantize_per_tensor(U.bits(w))
    y, yb = O.gemm_per_tensor(xq, sxi, wq, swi)
    a = torch.from_numpy(xq).view(torch.float8_e4m3fn)
    b = torch.from_numpy(wq).view(torch.float8_e4m3fn)
    try:
        ref = torch._scaled_mm(a, b.t(), scale_a=torch.tensor(float(sxi)), scale_b=torch.tensor(float(swi)),
                               out_dtype=torch.float32)
    except Exception as e:  # pragma: no cover - depends on the CPU build of torch
        pytest.skip(f"torch._scaled_mm unavailable on this CPU build: {e}")
    rel = np.linalg.norm(y - ref.numpy()) / np.linalg.norm(ref.numpy())
    assert rel < 1e-5, rel


def test_gemm_exact_on_integer_inputs_with_unit_scales():
    """Small integers are exact in E4M3 and their dot products are exact in fp32: the oracle GEMMs
    must then equal the int64 matmul exactly.  Catches transposed operands and wrong block indexing."""
    rng = np.random.default_rng(5)
    ai = rng.integers(-8, 9, size=(48, 384)).astype(np.float32)
    bi = rng.integers(-8, 9, size=(256, 384)).astype(np.float32)
    a, b = O.e4m3_encode(ai), O.e4m3_encode(bi)
    assert np.array_equal(O.e4m3_decode(a), ai)
    want = ai.astype(np.int64) @ bi.astype(np.int64).T
    ones_a = np.ones((48, 3), np.float32)
    y, _ = O.gemm_blockwise(a, ones_a, b, np.ones((2, 3), np.float32))
    assert np.array_equal(y.astype(np.int64), want)
    y, _ = O.gemm_rowwise_both(a, ones_a, b, np.ones((256, 3), np.float32))
    assert np.array_equal(y.astype(np.int64), want)
    y, _ = O.gemm_per_tensor(a, 1.0, b, 1.0)
    assert np.array_equal(y.astype(np.int64), want)
    yc, _ = C.gemm_blockwise(a, ones_a, b, np.ones((2, 3), np.float32))
    assert np.array_equal(yc.astype(np.int64), want)
    # distinct power-of-two scales per block stay exact and expose any mix-up of scale indices
    sa = (2.0 ** rng.integers(-3, 4, size=(48, 3))).astype(np.float32)
    sb = (2.0 ** rng.integers(-3, 4, size=(2, 3))).astype(np.float32)
    want2 = np.zeros((48, 256))
    for kb in range(3):
        part = ai[:, kb * 128:(kb + 1) * 128].astype(np.float64) @ bi[:, kb * 128:(kb + 1) * 128].astype(np.float64).T
        want2 += part * sa[:, kb][:, None] * np.repeat(sb[:, kb], 128)[None, :]
    y, _ = O.gemm_blockwise(a, sa, b, sb)
    assert np.array_equal(y.astype(np.float64), want2)
    yc, _ = C.gemm_blockwise(a, sa, b, sb)
    assert np.array_equal(yc.astype(np.float64), want2)


def test_gemm_blockwise_against_float64_dequant_matmul_and_bias():
    x = U.randn_bf16((96, 384), seed=91, outlier_frac=0.002, outlier_mul=50.0)
    w = U.randn_bf16((256, 384), seed=92, std=0.02)
    bias = U.randn_bf16((256,), seed=93, std=0.1).float().numpy()
    xq, _, sxi = O.quantize_1x128(U.bits(x))
    wq, _, swi = O.quantize_128x128(U.bits(w))
    ref = O.gemm_dequant_f64(xq, sxi, wq, np.repeat(swi, 128, axis=0))
    y, yb = O.gemm_blockwise(xq, sxi, wq, swi)
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 1e-6
    yb_f = O.bf16_bits_to_f32(yb)
    assert np.linalg.norm(yb_f - ref) / np.linalg.norm(ref) < 3e-3      # one bf16 rounding
    y2, _ = O.gemm_blockwise(xq, sxi, wq, swi, bias)
    assert np.allclose(y2 - y, bias[None, :], rtol=0, atol=1e-5)
    yc, _ = C.gemm_blockwise(xq, sxi, wq, swi, bias_f32=bias)
    assert np.linalg.norm(yc - y2) / np.linalg.norm(y2) < 1e-6
    # and the quantization error itself is small against the unquantized product
    exact = x.double().numpy() @ w.double().numpy().T
    assert np.linalg.norm(ref - exact) / np.linalg.norm(exact) < 0.05


def test_gemm_rowwise_both_against_float64():
    a = U.randn_bf16((128, 256), seed=94)
    b = U.randn_bf16((256, 256), seed=95)
    aq, _, asi = O.quantize_1x128(U.bits(a))
    bq, _, bsi = O.quantize_1x128(U.bits(b))
    ref = O.gemm_dequant_f64(aq, asi, bq, bsi)
    y, _ = O.gemm_rowwise_both(aq, asi, bq, bsi)
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 1e-6
    yc, _ = C.gemm_blockwise(aq, asi, bq, bsi, sb_per_row=True)
    assert np.linalg.norm(yc - ref) / np.linalg.norm(ref) < 1e-6


def test_grouped_equals_loop_of_dense_with_empty_experts():
    counts = [5, 0, 130, 0, 1]
    offs = np.cumsum(counts).astype(np.int32)
    total = int(offs[-1])
    x = U.randn_bf16((total, 256), seed=96)
    w = U.randn_bf16((5 * 128, 256), seed=97, std=0.02)
    xq, _, sxi = O.quantize_1x128(U.bits(x))
    wq, _, swi = O.quantize_128x128(U.bits(w))
    wq3, swi3 = wq.reshape(5, 128, 256), swi.reshape(5, 1, 2)
    y, _ = O.gemm_grouped_blockwise(xq, sxi, wq3, swi3, offs)
    start = 0
    for e, cnt in enumerate(counts):
        if cnt:
            ye, _ = O.gemm_blockwise(xq[start:start + cnt], sxi[start:start + cnt], wq3[e], swi3[e])
            assert np.array_equal(y[start:start + cnt], ye)
        start += cnt


def test_bucket_packing_against_an_element_loop():
    """pack_bucket / unpack_bucket restate slicing assignments; pinned by the index arithmetic written
    out element by element on a small case, by the zero padding, and by unpack(pack(x)) == x."""
    rng = np.random.default_rng(9)
    numels, S = [130, 128, 5, 300], 3
    grads = [rng.integers(1, 65535, size=S * n).astype(np.uint16) for n in numels]
    offsets, row = O.bucket_offsets(numels)
    assert offsets == [0, 256, 384, 512] and row == 896
    packed = O.pack_bucket(grads, numels, S)
    want = np.zeros((S, row), dtype=np.uint16)
    for e, n in enumerate(numels):
        for s_ in range(S):
            for i in range(n):
                want[s_, offsets[e] + i] = grads[e][s_ * n + i]
    assert np.array_equal(packed, want)
    covered = np.zeros(row, dtype=bool)
    for e, n in enumerate(numels):
        covered[offsets[e]:offsets[e] + n] = True
    assert not packed[:, ~covered].any()
    for s_ in range(S):
        pieces = O.unpack_bucket(packed[s_], numels)
        for e, n in enumerate(numels):
            assert np.array_equal(pieces[e], grads[e][s_ * n:(s_ + 1) * n])


def test_swiglu_restatement_against_numpy_and_torch():
    """exp_spec within a few fp32 ulp of numpy's exp over its whole clamped range; swiglu equal to
    torch's eager bf16 graph F.silu(gate) * up except where a last-place difference of the fp32
    sigmoid crosses a bf16 rounding boundary (then one bf16 ulp)."""
    import torch
    import torch.nn.functional as F
    t = np.concatenate([np.linspace(-86, 88.7, 200001), np.random.default_rng(0).normal(0, 3, 100000)]).astype(np.float32)
    got = O.exp_spec(t).astype(np.float64)
    want = np.exp(t.astype(np.float64))
    assert np.max(np.abs(got - want) / want) < 4e-7
    assert O.exp_spec(np.float32([0.0]))[0] == 1.0 and O.exp_spec(np.float32([-1000.0]))[0] == O.exp_spec(np.float32([-86.0]))[0] \
        and np.isinf(O.exp_spec(np.float32([89.0, 1000.0]))).all()
    g = torch.randn(64, 512, generator=torch.Generator().manual_seed(1)) * 3
    g[0, :8] = torch.tensor([0.0, -0.0, 50.0, -50.0, 1e-3, -1e-3, 200.0, -200.0])
    u = torch.randn(64, 512, generator=torch.Generator().manual_seed(2))
    h = torch.cat([g, u], dim=1).to(torch.bfloat16)
    ref = (F.silu(h[:, :512]) * h[:, 512:])
    mine = O.swiglu(h.view(torch.int16).numpy().view(np.uint16))
    ref_bits = ref.view(torch.int16).numpy().view(np.uint16)
    diff = np.abs(mine.astype(np.int32) - ref_bits.astype(np.int32))
    same_sign_zero = (mine & 0x7FFF) + (ref_bits & 0x7FFF) == 0
    assert ((diff <= 1) | same_sign_zero).all() and (diff != 0).mean() < 2e-3


def test_c_restatement_of_pow2_scales_and_swiglu_bit_exact():
    """Second implementations written differently (frexpf / ldexpf / nearbyintf and scalar loops against
    exponent-field arithmetic and array operations): power-of-two scales, the specified exponential, and
    the SwiGLU activation agree bit for bit."""
    rng = np.random.default_rng(0)
    am = np.concatenate([np.float32(2.0) ** rng.integers(-60, 60, 300) * rng.uniform(0.5, 2, 300).astype(np.float32),
                         np.float32([0, 1e-13, 1e-12, 448, 224, 448 * 2.0 ** -20, 3.39e38, np.inf, np.nan,
                                     447.99997, 448.00003])]).astype(np.float32)
    s, si = O.scales_from_amax(am, pow2=True)
    cs, csi = C.scales_pow2(am)
    assert U.same_f32_or_nan(s, cs) and U.same_f32_or_nan(si, csi)
    t = np.concatenate([rng.uniform(-100, 100, 20000), rng.normal(0, 3, 20000),
                        [0, -0.0, 88.5, -88.5, 89, -86, 88.72284, 1e-30, np.inf, -np.inf]]).astype(np.float32)
    with np.errstate(all="ignore"):
        a, b = O.exp_spec(t), C.exp_spec(t)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    h = U.randn_bf16((64, 512), 5, 2.0, 0.01, 30.0)
    h[0, :6] = torch.tensor([0.0, -0.0, 88.5, -88.5, -200.0, 200.0], dtype=torch.bfloat16)
    assert np.array_equal(O.swiglu(U.bits(h)), C.swiglu(U.bits(h)))


def test_dequantize_accumulate_against_torch_casts_and_a_scalar_loop():
    """`dequantize_1x128_accumulate`: with a zero main gradient and grad_scale 1 it is torch's float8 decode times
    the group's scale_inv, exactly; in general it equals a scalar loop over elements written with torch's fp32
    arithmetic (decode, times scale_inv, times grad_scale, plus main_grad: four roundings in that order); a
    different association ((scale_inv * grad_scale) first) gives other bits on this data, so the order is pinned."""
    rng = np.random.default_rng(11)
    rows, cols = 6, 256
    codes = rng.integers(0, 256, (rows, cols)).astype(np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x3C                                  # (no NaN codes: compared as numbers)
    si = (rng.uniform(0.3, 3.0, (rows, cols // 128)) * 2.0 ** rng.integers(-12, 3, (rows, cols // 128))).astype(np.float32)
    dec = torch.from_numpy(codes).view(torch.float8_e4m3fn).float()      # torch's decode, not the oracle's
    zero = np.zeros((rows, cols), np.float32)
    got0 = O.dequantize_1x128_accumulate(codes, si, zero, 1.0)
    want0 = (dec * torch.from_numpy(np.repeat(si, 128, axis=1))).numpy() + np.float32(0.0)   # (+0 + -0 = +0)
    assert np.array_equal(got0.view(np.uint32), want0.view(np.uint32))
    main = (rng.normal(0, 1e-2, (rows, cols))).astype(np.float32)
    gs = 0.3
    got = O.dequantize_1x128_accumulate(codes, si, main, gs)
    want = np.empty_like(main)
    tgs = torch.tensor(gs, dtype=torch.float32)
    for r in range(rows):
        for c in range(cols):
            v = dec[r, c] * torch.tensor(si[r, c // 128])                 # fp32 scalar arithmetic, one rounding each
            v = v * tgs
            want[r, c] = float(torch.tensor(main[r, c]) + v)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    other = (main + dec.numpy() * (np.repeat(si, 128, axis=1) * np.float32(gs)).astype(np.float32)).astype(np.float32)
    assert not np.array_equal(other.view(np.uint32), want.view(np.uint32))
    # shape of main_grad is kept, 1-D buckets included
    flat = O.dequantize_1x128_accumulate(codes.reshape(-1), si.reshape(-1), main.reshape(-1), gs)
    assert flat.shape == (rows * cols,) and np.array_equal(flat.reshape(rows, cols).view(np.uint32), want.view(np.uint32))


def test_dequantize_per_tensor_f32_is_torch_decode_times_scale():
    codes = np.arange(256, dtype=np.uint8)
    codes = codes[(codes & 0x7F) != 0x7F]
    dec = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).float().numpy()
    for si in (np.float32(1.0), np.float32(0.0123), np.float32(3.1e-9)):
        got = O.dequantize_per_tensor_f32(codes, si)
        assert np.array_equal(got.view(np.uint32), (dec * si).astype(np.float32).view(np.uint32))
        assert np.array_equal(O.dequantize_per_tensor(codes, si), O.f32_to_bf16_bits(got))


def test_swiglu_backward_against_float64_autograd():
    """`swiglu_backward` against torch's float64 autograd of act = bf16(silu(gate)) * up (d up) and of
    silu(gate) * up (d gate): within bf16 rounding of the exact derivative, and exactly zero / exactly the factor
    at the closed-form points gate = 0 (silu' = 1/2) and large |gate| (silu' -> 1 or 0)."""
    m, inter = 48, 256
    h = U.randn_bf16((m, 2 * inter), 21, 2.0, 0.002, 15.0)
    h[0, :4] = torch.tensor([0.0, -0.0, 40.0, -40.0], dtype=torch.bfloat16)
    da = U.randn_bf16((m, inter), 22, 1e-2)
    da[0, :4] = torch.tensor([0.5, 0.5, 0.25, 0.25], dtype=torch.bfloat16)
    h[0, inter:inter + 4] = torch.tensor([2.0, 2.0, 4.0, 4.0], dtype=torch.bfloat16)
    dh = U.from_bits(O.swiglu_backward(U.bits(h), U.bits(da)))
    g = h[:, :inter].double().requires_grad_(True)
    u = h[:, inter:].double()
    (torch.nn.functional.silu(g) * u * da.double()).sum().backward()
    dg_ref = g.grad
    silu_b = torch.nn.functional.silu(h[:, :inter].double()).to(torch.bfloat16).double()
    du_ref = da.double() * silu_b
    for got, want in ((dh[:, :inter], dg_ref), (dh[:, inter:], du_ref)):
        err = (got.double() - want).abs()
        # half a bf16 step of the result, plus a few fp32 steps of the factor for the cancelling region of silu'
        assert bool((err <= want.abs() * 2.0 ** -8 + (da.double() * u).abs() * 1e-6 + 1e-40).all())
    # closed-form points: silu'(0) = 1/2 -> d gate = dact * up / 2 = 0.5; silu'(40) = 1 -> 1.0; silu'(-40) = 0 (to fp32)
    assert [float(v) for v in dh[0, :3]] == [0.5, 0.5, 1.0] and abs(float(dh[0, 3])) < 1e-14
    # d up at those points: dact * bf16(silu): silu(0) = 0, silu(40) = 40, silu(-40) = -0 (to bf16)
    assert [float(v) for v in dh[0, inter:inter + 3]] == [0.0, 0.0, 10.0] and abs(float(dh[0, inter + 3])) < 1e-14


def test_grouped_layout_and_grouped_transposed_quantizer():
    """The padded token axis of the grouped weight gradient: block tables worked out by hand (ragged counts, empty
    experts, a malformed offset table read clamped), and every expert's piece of the grouped transposed quantizer
    equal to the row-wise 1x128 quantizer applied to that expert's zero-padded rows, transposed."""
    table, used = O.grouped_layout([130, 130, 430, 500], 512)
    assert table == [(0, 130, 0, 2), (130, 0, 2, 1), (130, 300, 3, 3), (430, 70, 6, 1)] and used == 7
    table, used = O.grouped_layout([128, 100, 9999], 300)                 # decreasing, then beyond the row count
    assert table == [(0, 128, 0, 1), (128, 0, 1, 1), (128, 172, 2, 2)] and used == 4
    assert O.grouped_layout([0, 0], 0) == ([(0, 0, 0, 1), (0, 0, 1, 1)], 2)
    for offs, total in (([130, 130, 430, 500], 512), ([0, 7, 7, 263], 263)):
        x = U.randn_bf16((total, 256), 77, 1.0, 0.002, 40.0)
        xb = U.bits(x)
        qt, st, sit = O.quantize_128x1_t_grouped(xb, offs)
        e_cnt = len(offs)
        assert qt.shape == (256, (total // 128 + e_cnt) * 128) and sit.shape == (256, total // 128 + e_cnt)
        table, used = O.grouped_layout(offs, total)
        assert used <= total // 128 + e_cnt
        for start, rows, b0, nb in table:
            padded = np.zeros((nb * 128, 256), np.uint16)
            padded[:rows] = xb[start:start + rows]
            c, s_, si = O.quantize_1x128(np.ascontiguousarray(padded.T))   # [K, nb * 128] with scales [K, nb]
            assert np.array_equal(qt[:, b0 * 128:(b0 + nb) * 128], c)
            assert np.array_equal(st[:, b0:b0 + nb].view(np.uint32), s_.view(np.uint32))
            assert np.array_equal(sit[:, b0:b0 + nb].view(np.uint32), si.view(np.uint32))
            assert not qt[:, b0 * 128 + rows:(b0 + nb) * 128].any()       # the fill is zero codes
        assert not qt[:, used * 128:].any()


def test_grouped_wgrad_against_float64_per_expert():
    """`gemm_grouped_wgrad`: every expert's weight gradient equals the float64 product of that expert's dequantized
    operands (so the zero fill adds nothing and no expert sees another's rows), an empty expert gets exact zeros,
    and moving an expert's rows elsewhere in the batch does not change its result."""
    offs, total, n, k = [130, 130, 430, 500], 512, 128, 256
    go = U.randn_bf16((total, n), 81, 1e-2)
    x = U.randn_bf16((total, k), 82, 1.0)
    got, _, sgot = O.quantize_128x1_t_grouped(U.bits(go), offs)
    xt, _, sxt = O.quantize_128x1_t_grouped(U.bits(x), offs)
    dw, dw_bits = O.gemm_grouped_wgrad(got, sgot, xt, sxt, offs, total)
    assert dw.shape == (4, n, k) and not dw[1].any()
    table, _ = O.grouped_layout(offs, total)
    for e, (start, rows, b0, nb) in enumerate(table):
        cols = slice(b0 * 128, (b0 + nb) * 128)
        ref = O.gemm_dequant_f64(got[:, cols], sgot[:, b0:b0 + nb], xt[:, cols], sxt[:, b0:b0 + nb])
        assert np.linalg.norm(dw[e] - ref) <= 1e-6 * max(np.linalg.norm(ref), 1e-30)
        if rows:
            exact = go[start:start + rows].double().numpy().T @ x[start:start + rows].double().numpy()
            assert np.linalg.norm(dw[e] - exact) / np.linalg.norm(exact) < 0.06
    assert np.array_equal(dw_bits, O.f32_to_bf16_bits(dw))
    # expert 2's 300 rows placed first in another batch: same gradient for it, bit for bit
    perm = np.r_[130:430, 0:130, 430:512]
    got2, _, sgot2 = O.quantize_128x1_t_grouped(U.bits(go)[perm], [300, 430, 430, 500])
    xt2, _, sxt2 = O.quantize_128x1_t_grouped(U.bits(x)[perm], [300, 430, 430, 500])
    dw2, _ = O.gemm_grouped_wgrad(got2, sgot2, xt2, sxt2, [300, 430, 430, 500], total)
    assert np.array_equal(dw2[0].view(np.uint32), dw[2].view(np.uint32)) and np.array_equal(dw2[1].view(np.uint32), dw[0].view(np.uint32))


def test_block_quantizer_against_an_independent_implementation_of_the_same_convention():
    """A third implementation that none of this build's authors wrote: the 128x128 block quantizer that the
    `transformers` package ships for DeepSeek-V3-style FP8 checkpoints (transformers/integrations/finegrained_fp8.py,
    `Fp8Quantize._quantize_one`: scale = 448 / max|block|, clamp, cast, store 1 / scale as weight_scale_inv).  On
    blocks that are not all zero it must produce the oracle's codes bit for bit (same multiplier, same rounding); its
    stored inverse is 1 / (448 / amax) where the oracle divides amax / 448, so the two inverses agree to one unit in
    the last place and are equal in most blocks; and its power-of-two format ("ue8m0": the inverse rounded up to a
    power of two, the multiplier its reciprocal) gives the codes and scales of the oracle's pow2 recipe."""
    fg = pytest.importorskip("transformers.integrations.finegrained_fp8")
    if not hasattr(fg, "Fp8Quantize") or not hasattr(fg.Fp8Quantize, "_quantize_one"):
        pytest.skip("this transformers version has no Fp8Quantize._quantize_one")
    import types
    w = U.randn_bf16((384, 512), 77, 0.02, 0.002, 25.0)
    w[128:256, 0:128] *= 1e-3                                    # a block of small values
    w[0, 0] = 0.75                                               # a block whose maximum is a power of two times 1.5

    def theirs(fmt):
        cfg = types.SimpleNamespace(weight_block_size=(128, 128), scale_fmt=fmt)
        stub = types.SimpleNamespace(hf_quantizer=types.SimpleNamespace(quantization_config=cfg))
        stub._resolve_block_size = lambda value: (128, 128)
        out = fg.Fp8Quantize._quantize_one(stub, "layer.weight", w)
        return out["layer.weight"].view(torch.uint8).numpy(), out["layer.weight_scale_inv"].to(torch.float32).numpy()

    q, _, si = O.quantize_128x128(U.bits(w))
    tq, tsi = theirs("float")
    assert np.array_equal(tq, q), f"{int((tq != q).sum())} codes differ"
    ulps = np.abs(tsi.view(np.int32).astype(np.int64) - si.view(np.int32).astype(np.int64))
    assert ulps.max() <= 1 and (ulps == 0).mean() >= 0.5
    try:
        tq2, tsi2 = theirs("ue8m0")
    except Exception as e:                                       # (a torch build without the E8M0 dtype)
        pytest.skip(f"power-of-two format not available: {e}")
    q2, _, si2 = O.quantize_128x128(U.bits(w), pow2=True)
    assert np.array_equal(tsi2, si2) and np.array_equal(tq2, q2)


# ---- column_sum (bias gradient): facts the oracle did not author ------------------------------------------------

def test_column_sum_is_exact_on_integers_and_bounded_against_float64():
    rng = np.random.default_rng(7)
    for m, k in ((1, 128), (127, 128), (128, 256), (300, 128), (513, 384)):
        ints = rng.integers(-64, 65, size=(m, k)).astype(np.float32)           # bf16-exact, sums far below 2^24
        bits = O.f32_to_bf16_bits(ints)
        part, total, tb = O.column_sum(bits)
        assert part.shape == ((m + 127) // 128, k) and part.dtype == np.float32
        assert np.array_equal(total, ints.sum(axis=0, dtype=np.int64).astype(np.float32))
        want_part = np.stack([ints[b * 128:(b + 1) * 128].sum(axis=0, dtype=np.int64) for b in range(part.shape[0])])
        assert np.array_equal(part, want_part.astype(np.float32))
        assert np.array_equal(tb, O.f32_to_bf16_bits(total))
    # real data: within the error bound of an fp32 sum of m terms, n u sum|x| with u = 2^-24
    x = O.f32_to_bf16_bits((rng.standard_normal((1000, 256)) * 1e-3).astype(np.float32))
    xf = O.bf16_bits_to_f32(x).astype(np.float64)
    _, total, _ = O.column_sum(x)
    assert np.all(np.abs(total - xf.sum(axis=0)) <= 1000 * 2.0 ** -24 * np.abs(xf).sum(axis=0))


def test_column_sum_order_is_the_stated_one():
    """2^24 + 1 rounds back to 2^24 in fp32 (ties to even) while 1 + 1 = 2 survives being added to 2^24: where the
    ones sit relative to the big value tells the orders of addition apart.  Answers derived by hand from the
    order in the docstring, for one column each."""
    big = np.float32(2.0 ** 24)

    def total_of(rows):
        col = np.zeros((256, 128), dtype=np.float32)
        for r, v in rows.items():
            col[r, 0] = v
        return float(O.column_sum(O.f32_to_bf16_bits(col))[1][0])

    # same row quad (rq = 0: rows 0, 1, 2, 3, 64, ...), added one after the other onto 2^24: every 1 is lost
    assert total_of({0: big, 1: 1.0, 2: 1.0, 3: 1.0, 64: 1.0}) == 2.0 ** 24
    # the ones in the neighbouring quad (rq = 1: rows 4..7): they first make 3, which survives (2^24 + 3 -> 2^24 + 4)
    assert total_of({0: big, 4: 1.0, 5: 1.0, 6: 1.0}) == 2.0 ** 24 + 4
    # one 1 each in quads 1, 2, 3 of the same group of four: q0 + q1 loses the first, q2 + q3 = 2 survives
    assert total_of({0: big, 4: 1.0, 8: 1.0, 12: 1.0}) == 2.0 ** 24 + 2
    # one 1 each in three other groups of four (rows 16, 32, 48): ((w0 + w1) + w2) + w3 loses every one of them
    assert total_of({0: big, 16: 1.0, 32: 1.0, 48: 1.0}) == 2.0 ** 24
    # the second block is added as a whole: its three ones make 3 first
    assert total_of({0: big, 128: 1.0, 129: 1.0, 130: 1.0}) == 2.0 ** 24 + 4
    # a purely sequential sum over the rows would have returned 2^24 in every case above
