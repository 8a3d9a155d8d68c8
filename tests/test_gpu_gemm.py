"""GPU parity of the scaled FP8 GEMMs through the C ABI.

Acceptance (stated by the benchmark definition): relative Frobenius error <= 1e-2 against
dequantize-then-fp32-matmul.  The kernels are in fact held to much tighter bounds here:
fp32 output within 1e-4 of a float64 dequantized matmul (the matrix cores sum the 128 products of
one instruction with less than fp32 precision: about 1.4e-5 relative was measured on gfx950), bf16
output within one bf16 rounding, and exact equality on integer-valued inputs with power-of-two
scales, where no rounding occurs at all."""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from oracle import c_oracle as C
import _util as U

pytestmark = pytest.mark.gpu
TOL_SPEC = 1e-2          # the stated tolerance
TOL_F32 = 1e-4           # fp32 output vs float64 reference
TOL_BF16 = 3e-3          # bf16 output: one rounding (2^-9 relative per element)


@pytest.fixture(autouse=True, params=["large tiles only", "default rule"])
def gemm_kernel_choice(request):
    """Most shapes here have few tiles, which the library would hand to its small-tile kernel: every test of this
    module runs once with that kernel switched off (so the 256 x 256-tile kernel sees the small, ragged and edge
    cases too) and once under the default rule."""
    from hpfp8 import _lib
    lib = _lib.load()
    lib.hpfp8_debug_set_small_gemm(1 if request.param == "large tiles only" else 0)
    yield
    lib.hpfp8_debug_set_small_gemm(0)


def rel(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300)


def fp8(codes, dev):
    return torch.from_numpy(np.ascontiguousarray(codes)).to(dev).view(torch.float8_e4m3fn)


def f32t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dev)


def dequant_f64(q, s_rows, dev):
    """codes [R, K] and per-row scales [R, K/128] -> float64 values, with torch on the GPU."""
    lut = torch.from_numpy(O.e4m3_decode(np.arange(256, dtype=np.uint8)).astype(np.float64)).to(dev)
    lut = torch.nan_to_num(lut)
    return lut[q.view(torch.uint8).long()] * s_rows.double().repeat_interleave(128, dim=1)


def ref_f64_torch(aq, sa_rows, bq, sb_rows, dev):
    """float64 dequantized matmul on the GPU with torch (independent of the kernels under test)."""
    return dequant_f64(aq, sa_rows, dev) @ dequant_f64(bq, sb_rows, dev).t()


def check_whole_output_f64(c, aq, sa_rows, bq, sb_rows_of, dev, tol, chunk=2048, bf16_out=False):
    """Every element of c[M, N] against the float64 dequantized matmul, computed `chunk` columns at a time
    (sb_rows_of(n0, n1) gives the per-row scales [n1 - n0, K/128] of b's rows n0..n1): the relative Frobenius
    error over the whole matrix, and -- bf16 output -- every element within one rounding of the exact value."""
    a = dequant_f64(aq, sa_rows, dev)
    amax_a = a.abs().view(a.shape[0], -1, 128).amax(dim=2)            # [M, K/128]
    num = den = 0.0
    n = bq.shape[0]
    for n0 in range(0, n, chunk):
        n1 = min(n0 + chunk, n)
        b = dequant_f64(bq[n0:n1], sb_rows_of(n0, n1), dev)
        ref = a @ b.t()
        got = c[:, n0:n1].double()
        d = got - ref
        num += float((d * d).sum())
        den += float((ref * ref).sum())
        if bf16_out:
            # one bf16 rounding (2^-9 relative; 2^-8 allowed) plus the matrix cores' own summation error: the 128
            # products of one instruction are summed in a fixed-point window about 13 bits below the largest of
            # them (test_matrix_core_summation_window), so a k-block adds up to 2^-11 of its largest product
            bound = ref.abs() * 2.0 ** -8 + 2.0 ** -10 * (amax_a @ b.abs().view(b.shape[0], -1, 128).amax(dim=2).t())
            over = d.abs() - bound
            if bool((over > 0).any()):
                i = int(over.argmax())
                r_, c_ = i // over.shape[1], i % over.shape[1]
                raise AssertionError(f"columns {n0}..{n1}: element ({r_}, {n0 + c_}) got {float(got[r_, c_])!r} ref "
                                     f"{float(ref[r_, c_])!r} bound {float(bound[r_, c_])!r} violations {int((over > 0).sum())}")
        del ref, got, d, b
    err = (num / max(den, 1e-300)) ** 0.5
    assert err < tol, err
    return err


def test_exact_on_integer_inputs(gpu):
    """Integer-valued operands and power-of-two scales make every product and sum exact in fp32, so
    the kernel must reproduce the integer matmul exactly whatever its summation order.  Distinct
    values everywhere expose any wrong tile, row, k-chunk or scale index."""
    import hpfp8
    rng = np.random.default_rng(5)
    M, N, K = 320, 384, 512          # M is not a multiple of the 256-row tile; N spans a partial tile
    ai = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
    bi = rng.integers(-8, 9, size=(N, K)).astype(np.float32)
    a, b = O.e4m3_encode(ai), O.e4m3_encode(bi)
    sa = (2.0 ** rng.integers(-3, 4, size=(M, K // 128))).astype(np.float32)
    sb = (2.0 ** rng.integers(-3, 4, size=(N // 128, K // 128))).astype(np.float32)
    want, _ = O.gemm_blockwise(a, sa, b, sb)
    got = hpfp8.gemm_blockwise(fp8(a, gpu), f32t(sa, gpu), fp8(b, gpu), f32t(sb, gpu), out_dtype=torch.float32)
    assert np.array_equal(U.f32(got), want)
    # per-row scales on both sides (wgrad form)
    sbr = (2.0 ** rng.integers(-3, 4, size=(N, K // 128))).astype(np.float32)
    want, _ = O.gemm_rowwise_both(a, sa, b, sbr)
    got = hpfp8.gemm_blockwise(fp8(a, gpu), f32t(sa, gpu), fp8(b, gpu), f32t(sbr, gpu), sb_gran=1,
                               out_dtype=torch.float32)
    assert np.array_equal(U.f32(got), want)
    # per tensor
    want, _ = O.gemm_per_tensor(a, 0.5, b, 0.25)
    got = hpfp8.gemm_per_tensor(fp8(a, gpu), f32t([0.5], gpu), fp8(b, gpu), f32t([0.25], gpu), out_dtype=torch.float32)
    assert np.array_equal(U.f32(got), want)
    # bf16 output of exactly representable values is exact too
    small = hpfp8.gemm_blockwise(fp8(a[:, :128], gpu), f32t(np.ones((M, 1)), gpu), fp8(b[:, :128], gpu),
                                 f32t(np.ones((N // 128, 1)) / 64, gpu))
    w, _ = O.gemm_blockwise(a[:, :128], np.ones((M, 1), np.float32), b[:, :128], np.ones((N // 128, 1), np.float32) / 64)
    assert np.array_equal(U.f32(small), O.bf16_bits_to_f32(O.f32_to_bf16_bits(w)))


def test_matrix_core_summation_window(gpu):
    """What the FP8 matrix instruction does with the 128 products of one k-block, shown on a case where exact and
    inexact can be told apart: one product `big` and 127 products `big * 2^-j`, all exactly representable.  While
    every product lies within 2^-11 of the largest the sum is exact (as on the integer-valued tests); smaller
    products are partly lost -- the instruction adds in a fixed-point window about 13 bits below its largest
    product, not in fp32 -- and the loss stays below 2^-11 of that product.  This is why fp32 outputs are compared
    with float64 references at 1e-4 and not at fp32's own 1e-6; it is 1000 times inside the stated 1e-2."""
    import hpfp8
    ones = torch.ones((128, 128), dtype=torch.float32).to(torch.float8_e4m3fn).to(gpu)
    one = torch.ones((1, 1), device=gpu)
    seen_inexact = False
    for big in (448.0, 256.0):
        for j in range(0, 18):
            small = big * 2.0 ** -j
            a = torch.full((256, 128), small, dtype=torch.float32)
            a[:, 0] = big
            aq = a.to(torch.float8_e4m3fn)
            if float(aq[0, 1].float()) != small:          # not an E4M3 value any more
                continue
            c = hpfp8.gemm_blockwise(aq.to(gpu), torch.ones((256, 1), device=gpu), ones, one, out_dtype=torch.float32)
            got, exact = float(c[0, 0]), big + 127 * small   # (exact in fp32: at most 16 significant bits)
            assert bool((c == c[0, 0]).all())
            if j <= 11:
                assert got == exact, (big, j, got, exact)
            else:
                assert abs(got - exact) <= big * 2.0 ** -11, (big, j, got, exact)
                seen_inexact = seen_inexact or got != exact
    assert seen_inexact, "the matrix cores summed products 2^-12 and less of the largest exactly: tolerances can be tightened"


def test_non_finite_groups_make_their_output_rows_nan_and_no_others(gpu):
    """Activations with NaN / +-Inf planted in rows 0, 1, 2, 130 and 131: exactly those rows of the
    output are NaN, in every scale mode, and all other rows are what they are without the planted values
    (a NaN group must not leak into rows that share its tile, its wave or its scale loads)."""
    import hpfp8
    x = U.nonfinite_bf16(256, 512)
    w = U.randn_bf16((384, 512), 31, 0.02)
    bad_rows = np.zeros(256, bool)
    bad_rows[[0, 1, 2, 130, 131]] = True
    xg, wg = x.to(gpu), w.to(gpu)
    xc = x.clone()
    xc[bad_rows] = 1.0
    xcg = xc.to(gpu)
    for pow2 in (False, True):
        xq, sx = hpfp8.quantize_1x128(xg, kmajor=True, pow2=pow2)
        cq, sc = hpfp8.quantize_1x128(xcg, kmajor=True, pow2=pow2)
        wq, sw = hpfp8.quantize_128x128(wg, pow2=pow2)
        w1, sw1 = hpfp8.quantize_1x128(wg, kmajor=True, pow2=pow2)
        for out_dtype in (torch.bfloat16, torch.float32):
            for kw, bq, sb in (({}, wq, sw), ({"sb_gran": 1}, w1, sw1)):
                y = hpfp8.gemm_blockwise(xq, sx, bq, sb, out_dtype=out_dtype, pow2_scales=pow2, **kw)
                yc = hpfp8.gemm_blockwise(cq, sc, bq, sb, out_dtype=out_dtype, pow2_scales=pow2, **kw)
                nan = torch.isnan(y).cpu().numpy()
                assert nan[bad_rows].all() and not nan[~bad_rows].any(), (pow2, out_dtype, kw)
                assert torch.equal(y[~torch.from_numpy(bad_rows).to(gpu)], yc[~torch.from_numpy(bad_rows).to(gpu)])
        # the planted values on the other operand: columns of the output (x as the b operand, row scales)
        y = hpfp8.gemm_blockwise(w1, sw1, xq, sx, sb_gran=1, out_dtype=torch.float32, pow2_scales=pow2)
        nan = torch.isnan(y).cpu().numpy()
        assert nan[:, bad_rows].all() and not nan[:, ~bad_rows].any()
        # accumulate: NaN rows stay NaN, the others add up as usual
        acc = torch.ones((256, 384), dtype=torch.float32, device=gpu)
        hpfp8.gemm_blockwise(xq, sx, w1, sw1, sb_gran=1, out=acc, accumulate=True, pow2_scales=pow2)
        nan = torch.isnan(acc).cpu().numpy()
        assert nan[bad_rows].all() and not nan[~bad_rows].any()
    # against the oracle, codes and scales as the oracle makes them
    rq, _, rsi = O.quantize_1x128(U.bits(x))
    rw, _, rswi = O.quantize_128x128(U.bits(w))
    want, _ = O.gemm_blockwise(rq, rsi, rw, rswi)
    assert np.array_equal(np.isnan(want).all(axis=1), bad_rows) and not np.isnan(want[~bad_rows]).any()
    xq, sx = hpfp8.quantize_1x128(xg, kmajor=True)
    wq, sw = hpfp8.quantize_128x128(wg)
    got = U.f32(hpfp8.gemm_blockwise(xq, sx, wq, sw, out_dtype=torch.float32))
    assert rel(got[~bad_rows], want[~bad_rows]) < TOL_F32
    # per tensor: one NaN anywhere makes the scale, and with it every output, NaN
    xq, _, sxi = hpfp8.quantize_per_tensor(xg)
    wq, _, swi = hpfp8.quantize_per_tensor(wg)
    assert bool(torch.isnan(hpfp8.gemm_per_tensor(xq, sxi, wq, swi)).all())


def test_golden_gemm(gpu):
    import os
    import hpfp8
    G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_path_golden.npz"))
    a = U.from_bits(G["gemm_a_bits"], gpu)
    w = U.from_bits(G["gemm_w_bits"], gpu)
    bias = U.from_bits(G["gemm_bias_bits"], gpu)
    aq, asi = hpfp8.quantize_1x128(a)
    wq, wsi = hpfp8.quantize_128x128(w)
    y32 = hpfp8.gemm_blockwise(aq, asi, wq, wsi, bias=bias, out_dtype=torch.float32)
    assert rel(U.f32(y32), G["gemm_y_f32"]) < TOL_F32
    y = hpfp8.gemm_blockwise(aq, asi, wq, wsi, bias=bias)
    assert rel(U.f32(y), G["gemm_y_f32"]) < TOL_BF16
    diff = np.abs(U.bits(y).astype(np.int32) - G["gemm_y_bits"].astype(np.int32))
    assert (diff != 0).mean() < 3e-2    # only rounding flips from summation precision
    wq1, wsi1 = hpfp8.quantize_1x128(w)
    y2 = hpfp8.gemm_blockwise(aq, asi, wq1, wsi1, sb_gran=1, out_dtype=torch.float32)
    assert rel(U.f32(y2), G["gemm_rows_y_f32"]) < TOL_F32


def test_cfg1_per_tensor_linear(gpu):
    """Config 1 at full size: x[2048,1024] ~ N(0,1), W[1024,1024] ~ N(0,0.02), seed 0."""
    import hpfp8
    g = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn((2048, 1024), generator=g).to(torch.bfloat16)
    w = (torch.randn((1024, 1024), generator=g) * 0.02).to(torch.bfloat16)
    xq, _, sxi = hpfp8.quantize_per_tensor(x.to(gpu))
    wq, _, swi = hpfp8.quantize_per_tensor(w.to(gpu))
    rxq, _, rsxi = O.quantize_per_tensor(U.bits(x))
    rwq, _, rswi = O.quantize_per_tensor(U.bits(w))
    assert np.array_equal(U.codes(xq), rxq) and np.array_equal(U.codes(wq), rwq)
    assert float(sxi) == float(rsxi) and float(swi) == float(rswi)
    want, want_bits = O.gemm_per_tensor(rxq, rsxi, rwq, rswi)
    y32 = hpfp8.gemm_per_tensor(xq, sxi, wq, swi, out_dtype=torch.float32)
    y = hpfp8.gemm_per_tensor(xq, sxi, wq, swi)
    assert rel(U.f32(y32), want) < TOL_F32
    assert rel(U.f32(y), want) < TOL_BF16 < TOL_SPEC
    # the library routine: torch._scaled_mm on the GPU with the same codes and scales
    try:
        lib = torch._scaled_mm(xq, wq.t(), scale_a=sxi.reshape(()), scale_b=swi.reshape(()), out_dtype=torch.bfloat16)
        assert rel(U.f32(y), U.f32(lib)) < TOL_BF16
    except (RuntimeError, NotImplementedError) as e:
        print("torch._scaled_mm not usable here:", e)
    # end to end against the unquantized product: quantization error only
    exact = x.double() @ w.double().t()
    assert rel(U.f32(y), exact.numpy()) < 0.05


def test_output_row_stride_and_many_tiles_per_workgroup(gpu):
    """c may be a column slice of a wider buffer (ldc > N), and the neighbouring columns must stay
    untouched; 1200 tiles on a grid of one workgroup per CU gives every workgroup several tiles."""
    import hpfp8
    M, N, K = 5000, 15360, 256
    x = U.randn_bf16((M, K), 11, 1.0, 0.001, 50.0).to(gpu)
    w = U.randn_bf16((N, K), 12, 0.006).to(gpu)
    xq, sxi = hpfp8.quantize_1x128(x, kmajor=True)
    wq, swi = hpfp8.quantize_128x128(w)
    ref = ref_f64_torch(xq, sxi, wq, swi.repeat_interleave(128, dim=0), gpu)
    for dt, tol in ((torch.float32, TOL_F32), (torch.bfloat16, TOL_BF16)):
        wide = torch.full((M, N + 24), 7.0, dtype=dt, device=gpu)
        out = wide[:, 8:8 + N]
        hpfp8.gemm_blockwise(xq, sxi, wq, swi, out=out)
        assert rel(U.f32(out), ref.cpu().numpy()) < tol
        assert bool((wide[:, :8] == 7.0).all()) and bool((wide[:, 8 + N:] == 7.0).all())
        assert torch.equal(out, hpfp8.gemm_blockwise(xq, sxi, wq, swi, out_dtype=dt))


@pytest.mark.parametrize("M,N,K", [(320, 384, 512), (2500, 7808, 128), (3000, 5248, 256)])
def test_accumulate_onto_fp32_is_exact_on_integer_inputs(gpu, M, N, K):
    """accumulate adds the product onto what c holds.  With integer-valued operands, power-of-two scales
    and an integer-valued c every sum is exact in fp32, so the result must equal old + product whatever
    the order of summation; the larger cases give every workgroup several tiles (also with a single
    k-block per tile), a ragged last row tile, a half-used last column tile and ldc > N, and the
    columns of the wider buffer next to c must stay untouched."""
    import hpfp8
    rng = np.random.default_rng(M + N + K)
    ai = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
    bi = rng.integers(-8, 9, size=(N, K)).astype(np.float32)
    a, b = O.e4m3_encode(ai), O.e4m3_encode(bi)
    sa = (2.0 ** rng.integers(-3, 4, size=(M, K // 128))).astype(np.float32)
    sb = (2.0 ** rng.integers(-3, 4, size=(N // 128, K // 128))).astype(np.float32)
    sbr = (2.0 ** rng.integers(-3, 4, size=(N, K // 128))).astype(np.float32)
    old = rng.integers(-1000, 1001, size=(M, N)).astype(np.float32)
    aq, bq = fp8(a, gpu), fp8(b, gpu)
    for gran, sb_np in ((128, sb), (1, sbr)):
        prod = hpfp8.gemm_blockwise(aq, f32t(sa, gpu), bq, f32t(sb_np, gpu), sb_gran=gran, out_dtype=torch.float32)
        if M * N * K <= 64 * 1024 * 1024:
            want, _ = (O.gemm_blockwise if gran == 128 else O.gemm_rowwise_both)(a, sa, b, sb_np)
            assert np.array_equal(U.f32(prod), want)
        wide = torch.full((M, N + 12), 7.0, dtype=torch.float32, device=gpu)
        c = wide[:, 4:4 + N]
        c.copy_(torch.from_numpy(old))
        hpfp8.gemm_blockwise(aq, f32t(sa, gpu), bq, f32t(sb_np, gpu), sb_gran=gran, out=c, accumulate=True)
        assert torch.equal(c, torch.from_numpy(old).to(gpu) + prod)
        hpfp8.gemm_blockwise(aq, f32t(sa, gpu), bq, f32t(sb_np, gpu), sb_gran=gran, out=c, accumulate=True)
        assert torch.equal(c, torch.from_numpy(old).to(gpu) + 2 * prod)
        assert bool((wide[:, :4] == 7.0).all()) and bool((wide[:, 4 + N:] == 7.0).all())


@pytest.mark.parametrize("M,N,K,seed", [(256, 256, 128, 1), (512, 1024, 7168, 2), (1000, 384, 1024, 3),
                                         (8, 128, 256, 4), (4096, 512, 2048, 5)])
def test_blockwise_forward_shapes(gpu, M, N, K, seed):
    import hpfp8
    x = U.randn_bf16((M, K), seed, 1.0, 0.001, 50.0).to(gpu)
    w = U.randn_bf16((N, K), seed + 100, 0.006).to(gpu)
    bias = U.randn_bf16((N,), seed + 200, 0.05).to(gpu)
    xq, sxi = hpfp8.quantize_1x128(x)
    wq, swi = hpfp8.quantize_128x128(w)
    ref = ref_f64_torch(xq, sxi, wq, swi.repeat_interleave(128, dim=0), gpu)
    y32 = hpfp8.gemm_blockwise(xq, sxi, wq, swi, out_dtype=torch.float32)
    assert rel(U.f32(y32), ref.cpu().numpy()) < TOL_F32
    yb = hpfp8.gemm_blockwise(xq, sxi, wq, swi, bias=bias)
    refb = ref + bias.double()[None, :]
    assert rel(U.f32(yb), refb.cpu().numpy()) < TOL_BF16 < TOL_SPEC
    if M * N * K <= 512 * 1024 * 1024:
        want, _ = O.gemm_blockwise(U.codes(xq), U.f32(sxi), U.codes(wq), U.f32(swi))
        assert rel(U.f32(y32), want) < TOL_F32
    # k-major scale storage gives the same result bit for bit
    xq2, sxk = hpfp8.quantize_1x128(x, kmajor=True)
    assert torch.equal(hpfp8.gemm_blockwise(xq2, sxk, wq, swi, out_dtype=torch.float32), y32)
    # accumulate into an fp32 buffer
    acc = torch.full((M, N), 1.5, dtype=torch.float32, device=gpu)
    hpfp8.gemm_blockwise(xq, sxi, wq, swi, out=acc, accumulate=True)
    assert rel(U.f32(acc), (ref + 1.5).cpu().numpy()) < TOL_F32


@pytest.mark.parametrize("M,N,K", [(320, 384, 512), (2500, 7808, 128), (3000, 5248, 256)])
def test_power_of_two_scales_through_the_matrix_instruction(gpu, M, N, K):
    """hpfp8_gemm_blockwise_pow2 hands the scales to the matrix instruction as E8M0 block scales.  On
    integer-valued operands with power-of-two scales every sum is exact, so both forms (128x128 and
    per-row b scales) must equal the integer matmul and the kernel that scales with FMAs; only the
    exponent of a scale may matter (mantissa bits set on purpose change nothing)."""
    import hpfp8
    rng = np.random.default_rng(M + N)
    ai = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
    bi = rng.integers(-8, 9, size=(N, K)).astype(np.float32)
    a, b = O.e4m3_encode(ai), O.e4m3_encode(bi)
    sa = (2.0 ** rng.integers(-3, 4, size=(M, K // 128))).astype(np.float32)
    sb = (2.0 ** rng.integers(-3, 4, size=(N // 128, K // 128))).astype(np.float32)
    sbr = (2.0 ** rng.integers(-3, 4, size=(N, K // 128))).astype(np.float32)
    aq, bq = fp8(a, gpu), fp8(b, gpu)
    bias = U.randn_bf16((N,), 9, 4.0).to(gpu)
    for gran, sb_np in ((128, sb), (1, sbr)):
        plain = hpfp8.gemm_blockwise(aq, f32t(sa, gpu), bq, f32t(sb_np, gpu), sb_gran=gran, out_dtype=torch.float32)
        got = hpfp8.gemm_blockwise(aq, f32t(sa, gpu), bq, f32t(sb_np, gpu), sb_gran=gran, out_dtype=torch.float32,
                                   pow2_scales=True)
        assert torch.equal(got, plain)
        if M * N * K <= 64 * 1024 * 1024:
            want, _ = (O.gemm_blockwise if gran == 128 else O.gemm_rowwise_both)(a, sa, b, sb_np)
            assert np.array_equal(U.f32(got), want)
        noisy_a = f32t(sa * np.float32(1.5), gpu)          # same exponents, other mantissas
        assert torch.equal(hpfp8.gemm_blockwise(aq, noisy_a, bq, f32t(sb_np, gpu), sb_gran=gran, out_dtype=torch.float32,
                                                pow2_scales=True), plain)
        old = torch.from_numpy(rng.integers(-1000, 1001, size=(M, N)).astype(np.float32)).to(gpu)
        c = old.clone()
        hpfp8.gemm_blockwise(aq, f32t(sa, gpu), bq, f32t(sb_np, gpu), sb_gran=gran, out=c, accumulate=True, pow2_scales=True)
        assert torch.equal(c, old + plain)
        wide = torch.full((M, N + 16), 7.0, dtype=torch.bfloat16, device=gpu)
        out = wide[:, 8:8 + N]
        hpfp8.gemm_blockwise(aq, f32t(sa, gpu), bq, f32t(sb_np, gpu), sb_gran=gran, bias=bias, out=out, pow2_scales=True)
        assert torch.equal(out, hpfp8.gemm_blockwise(aq, f32t(sa, gpu), bq, f32t(sb_np, gpu), sb_gran=gran, bias=bias))
        assert bool((wide[:, :8] == 7.0).all()) and bool((wide[:, 8 + N:] == 7.0).all())


def test_power_of_two_recipe_on_real_data(gpu):
    """Quantized with power-of-two scales, the hardware-scaled GEMM agrees with a float64 dequantized
    matmul like the FMA-scaled one does (forward / dgrad form and wgrad form)."""
    import hpfp8
    M, N, K = 1024, 1536, 2048
    x = U.randn_bf16((M, K), 81, 1.0, 0.001, 50.0).to(gpu)
    w = U.randn_bf16((N, K), 82, 0.006).to(gpu)
    xq, sx = hpfp8.quantize_1x128(x, kmajor=True, pow2=True)
    wq, sw = hpfp8.quantize_128x128(w, pow2=True)
    ref = ref_f64_torch(xq, sx, wq, sw.repeat_interleave(128, dim=0), gpu)
    y32 = hpfp8.gemm_blockwise(xq, sx, wq, sw, out_dtype=torch.float32, pow2_scales=True)
    assert rel(U.f32(y32), ref.cpu().numpy()) < TOL_F32
    assert rel(U.f32(hpfp8.gemm_blockwise(xq, sx, wq, sw, pow2_scales=True)), ref.cpu().numpy()) < TOL_BF16
    assert rel(U.f32(y32), (x.double() @ w.double().t()).cpu().numpy()) < 0.06       # against the unquantized product
    xt, sxt = hpfp8.quantize_128x1_t(x, kmajor=True, pow2=True)       # [K, M]
    g = U.randn_bf16((M, N), 83, 1e-3).to(gpu)
    gt, sgt = hpfp8.quantize_128x1_t(g, kmajor=True, pow2=True)       # [N, M]
    refw = ref_f64_torch(gt, sgt, xt, sxt, gpu)
    dw = hpfp8.gemm_blockwise(gt, sgt, xt, sxt, sb_gran=1, out_dtype=torch.float32, pow2_scales=True)
    assert rel(U.f32(dw), refw.cpu().numpy()) < TOL_F32


def test_repeated_launches_give_identical_bits(gpu):
    """The kernels synchronise their LDS buffers by hand (counted waits and one barrier per k-block); a
    missing wait would show as launches of the same problem that differ now and then.  Every form,
    several tiles per workgroup, 40 launches each."""
    import hpfp8
    T, A, B = 512, 2560, 7808
    ga = U.randn_bf16((T, A), 61, 1e-3).to(gpu)
    gb = U.randn_bf16((T, B), 62).to(gpu)
    at, sat = hpfp8.quantize_128x1_t(ga, kmajor=True)
    bt, sbt = hpfp8.quantize_128x1_t(gb, kmajor=True)
    aq, sa = hpfp8.quantize_1x128(ga.t().contiguous(), kmajor=True)
    bq, sb = hpfp8.quantize_128x128(gb.t().contiguous())
    one = torch.ones(1, device=gpu)
    old = torch.from_numpy(np.random.default_rng(0).standard_normal((A, B)).astype(np.float32)).to(gpu)
    acc = torch.empty_like(old)

    def accumulate():
        acc.copy_(old)
        return hpfp8.gemm_blockwise(at, sat, bt, sbt, sb_gran=1, out=acc, accumulate=True)

    forms = {
        "row scales": lambda: hpfp8.gemm_blockwise(at, sat, bt, sbt, sb_gran=1),
        "row scales, fp32": lambda: hpfp8.gemm_blockwise(at, sat, bt, sbt, sb_gran=1, out_dtype=torch.float32),
        "row scales, accumulate": accumulate,
        "block scales": lambda: hpfp8.gemm_blockwise(aq, sa, bq, sb),
        "per tensor": lambda: hpfp8.gemm_per_tensor(aq, one, bq, one),
    }
    for name, fn in forms.items():
        first = fn().clone()
        for _ in range(40):
            assert torch.equal(fn(), first), name


def test_cfg2_dense_mlp_forward_whole_output_and_quantizers(gpu):
    """Config 2: x[4096,7168] with 0.1% x50 outliers, W[36864,7168] ~ N(0,0.006), at full size.  Both quantizers'
    complete outputs equal the C restatement byte for byte (codes) and bit for bit (scales); the whole 4096 x 36864
    output is compared with the float64 dequantized matmul; plus linearity in the scales (doubling every activation
    scale doubles the output exactly)."""
    import hpfp8
    M, N, K = 4096, 36864, 7168
    g = torch.Generator(device=gpu).manual_seed(0)
    x = torch.randn((M, K), generator=g, device=gpu)
    idx = torch.randperm(M * K, generator=g, device=gpu)[: round(0.001 * M * K)]
    x.view(-1)[idx] *= 50
    x = x.to(torch.bfloat16)
    w = (torch.randn((N, K), generator=g, device=gpu) * 0.006).to(torch.bfloat16)
    xq, sxi = hpfp8.quantize_1x128(x, kmajor=True)
    wq, swi = hpfp8.quantize_128x128(w)
    cq, _, csi = C.quantize_1x128(U.bits(x))
    assert np.array_equal(U.codes(xq), cq) and np.array_equal(U.f32_bits(U.f32(sxi)), U.f32_bits(csi))
    cq, _, csi = C.quantize_128x128(U.bits(w))
    assert np.array_equal(U.codes(wq), cq) and np.array_equal(U.f32_bits(U.f32(swi)), U.f32_bits(csi))
    del cq, csi
    y = hpfp8.gemm_blockwise(xq, sxi, wq, swi)
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    err = check_whole_output_f64(y, xq, sxi, wq, lambda n0, n1: swi[n0 // 128:n1 // 128].repeat_interleave(128, dim=0),
                                 gpu, TOL_BF16, bf16_out=True)
    assert err < TOL_SPEC
    y2 = hpfp8.gemm_blockwise(xq, sxi * 2, wq, swi)
    assert torch.equal(y2.float(), y.float() * 2)
    # against the unquantized bf16 product on a slice
    exact = x.double() @ w[:256].double().t()
    assert rel(U.f32(y[:, :256]), exact.cpu().numpy()) < 0.05


def test_cfg3_backward_whole_outputs_and_transposed_quantizers(gpu):
    """Config 3 (o_proj backward) at its full size, M = 4096 tokens, W[7168, 16384]: dgrad = go . W and wgrad =
    go^T . x (a contraction of 32 k-blocks over the tokens) with the 128x1 transposed requantization of both
    operands.  The transposed quantizers' complete outputs (and the fused 1x128 + 128x1^T form) equal the C
    restatement bit for bit; both GEMM outputs are compared whole with the float64 dequantized matmul."""
    import hpfp8
    M, N, K = 4096, 7168, 16384
    x = U.randn_bf16((M, K), 30).to(gpu)
    go = U.laplace_bf16((M, N), 31, 1e-3).to(gpu)
    w = U.randn_bf16((N, K), 32, 0.006).to(gpu)
    wq, swi, wqt = hpfp8.quantize_128x128(w, with_transpose=True)
    assert torch.equal(wqt.view(torch.uint8), wq.view(torch.uint8).t())
    goq, sgo, got, sgot = hpfp8.quantize_1x128_and_128x1_t(go, kmajor=True)
    xt, sxt = hpfp8.quantize_128x1_t(x, kmajor=True)
    for src, qt_, st_ in ((go, got, sgot), (x, xt, sxt)):
        cq, _, csi = C.quantize_128x1_t(U.bits(src))
        assert np.array_equal(U.codes(qt_), cq) and np.array_equal(U.f32_bits(U.f32(st_)), U.f32_bits(csi))
    cq, _, csi = C.quantize_1x128(U.bits(go))
    assert np.array_equal(U.codes(goq), cq) and np.array_equal(U.f32_bits(U.f32(sgo)), U.f32_bits(csi))
    del cq, csi
    dx = hpfp8.gemm_blockwise(goq, sgo, wqt, swi.t(), out_dtype=torch.float32)
    assert dx.shape == (M, K)
    swt = swi.t()
    check_whole_output_f64(dx, goq, sgo, wqt, lambda n0, n1: swt[n0 // 128:n1 // 128].repeat_interleave(128, dim=0),
                           gpu, TOL_F32)
    dx16 = hpfp8.gemm_blockwise(goq, sgo, wqt, swi.t())
    assert rel(U.f32(dx16[:512]), U.f32(dx[:512])) < TOL_BF16
    del dx, dx16
    dw = hpfp8.gemm_blockwise(got, sgot, xt, sxt, sb_gran=1, out_dtype=torch.float32)
    assert dw.shape == (N, K)
    check_whole_output_f64(dw, got, sgot, xt, lambda n0, n1: sxt[n0:n1], gpu, TOL_F32)
    exact = go.double().t()[:384] @ x.double()[:, :640]
    assert rel(U.f32(dw[:384, :640]), exact.cpu().numpy()) < 0.06


def _zipf_counts(total, experts, seed, zeros=2):
    g = torch.Generator(device="cpu").manual_seed(seed)
    perm = torch.randperm(experts, generator=g)
    p = (torch.arange(1, experts + 1, dtype=torch.float64) ** -1.1)[perm]
    p = p / p.sum()
    counts = torch.multinomial(p, total, replacement=True, generator=g).bincount(minlength=experts)
    order = torch.argsort(p)
    for z in order[:zeros]:
        counts[order[-1]] += counts[z]
        counts[z] = 0
    return counts


@pytest.mark.parametrize("experts,total,N,K,seed", [(5, 700, 256, 384, 1), (32, 8192, 512, 1024, 2), (3, 0, 128, 128, 3)])
def test_grouped_against_loop_of_dense(gpu, experts, total, N, K, seed):
    import hpfp8
    counts = _zipf_counts(total, experts, seed) if total else torch.zeros(experts, dtype=torch.int64)
    assert int(counts.sum()) == total
    offs = counts.cumsum(0).to(torch.int32).to(gpu)
    x = U.randn_bf16((max(total, 1), K), seed + 10)[:total].to(gpu)
    w = U.randn_bf16((experts * N, K), seed + 20, 0.006).to(gpu)
    xq, sxi = hpfp8.quantize_1x128(x)
    wq, swi = hpfp8.quantize_128x128(w)
    wq3, swi3 = wq.view(experts, N, K), swi.view(experts, N // 128, K // 128)
    y = hpfp8.gemm_grouped_blockwise(xq, sxi, wq3, swi3, offs, out_dtype=torch.float32)
    assert y.shape == (total, N)
    start = 0
    for e in range(experts):
        cnt = int(counts[e])
        if cnt:
            dense = hpfp8.gemm_blockwise(xq[start:start + cnt], sxi[start:start + cnt], wq3[e], swi3[e],
                                         out_dtype=torch.float32)
            assert torch.equal(y[start:start + cnt], dense), f"expert {e}"
            if e % 7 == 0:
                ref = ref_f64_torch(xq[start:start + cnt], sxi[start:start + cnt], wq3[e],
                                    swi3[e].repeat_interleave(128, dim=0), gpu)
                assert rel(U.f32(dense), ref.cpu().numpy()) < TOL_F32
        start += cnt
    # the same with power-of-two scales handed to the matrix instruction: grouped == loop of dense
    xq, sxi = hpfp8.quantize_1x128(x, kmajor=True, pow2=True)
    wq, swi = hpfp8.quantize_128x128(w, pow2=True)
    wq3, swi3 = wq.view(experts, N, K), swi.view(experts, N // 128, K // 128)
    y = hpfp8.gemm_grouped_blockwise(xq, sxi, wq3, swi3, offs, out_dtype=torch.float32, pow2_scales=True)
    start = 0
    for e in range(experts):
        cnt = int(counts[e])
        if cnt:
            dense = hpfp8.gemm_blockwise(xq[start:start + cnt], sxi[start:start + cnt], wq3[e], swi3[e],
                                         out_dtype=torch.float32, pow2_scales=True)
            assert torch.equal(y[start:start + cnt], dense), f"expert {e} (power-of-two scales)"
        start += cnt


def test_grouped_leaves_rows_past_the_last_offset_alone(gpu):
    import hpfp8
    K, N = 256, 128
    x = U.randn_bf16((300, K), 40).to(gpu)
    w = U.randn_bf16((2 * N, K), 41, 0.01).to(gpu)
    xq, sxi = hpfp8.quantize_1x128(x)
    wq, swi = hpfp8.quantize_128x128(w)
    offs = torch.tensor([100, 260], dtype=torch.int32, device=gpu)
    from hpfp8 import _lib, ops
    out = torch.full((300, N), 7.0, dtype=torch.float32, device=gpu)
    _lib.call("hpfp8_gemm_grouped_blockwise", xq.data_ptr(), K, sxi.data_ptr(), sxi.stride(0), sxi.stride(1),
              wq.data_ptr(), swi.data_ptr(), offs.data_ptr(), 2, 300, N, K, out.data_ptr(), N, _lib.OUT_F32,
              ops._stream())
    assert bool((out[260:] == 7.0).all()) and not bool((out[:260] == 7.0).any())


def test_grouped_clamps_a_malformed_offset_table(gpu):
    """Offsets that decrease or run past the row count are read as clamped (an expert's end is at least
    the previous end and at most total_m): the result is that of the clamped table and no row outside
    a or c is touched."""
    import hpfp8
    from hpfp8 import _lib, ops
    K, N, total = 256, 256, 700
    x = U.randn_bf16((total, K), 50).to(gpu)
    w = U.randn_bf16((4 * N, K), 51, 0.01).to(gpu)
    xq, sxi = hpfp8.quantize_1x128(x)
    wq, swi = hpfp8.quantize_128x128(w)
    bad = torch.tensor([300, 200, 650, 900], dtype=torch.int32, device=gpu)      # clamps to 300, 300, 650, 700
    good = torch.tensor([300, 300, 650, 700], dtype=torch.int32, device=gpu)
    outs = []
    for offs in (bad, good):
        out = torch.full((total + 8, N), 7.0, dtype=torch.float32, device=gpu)
        _lib.call("hpfp8_gemm_grouped_blockwise", xq.data_ptr(), K, sxi.data_ptr(), sxi.stride(0), sxi.stride(1),
                  wq.data_ptr(), swi.data_ptr(), offs.data_ptr(), 4, total, N, K, out.data_ptr(), N, _lib.OUT_F32,
                  ops._stream())
        outs.append(out)
    assert torch.equal(outs[0], outs[1]) and bool((outs[0][total:] == 7.0).all())
    assert not bool((outs[0][:total] == 7.0).any())


def test_cfg4_moe_grouped_full_size(gpu):
    """The grouped configuration at its real size (32 experts, 16384 tokens routed top-8 with Zipf
    popularity = 131072 rows, fused gate/up [4096, 7168] per expert): every expert's rows equal the
    dense kernel on that expert bit for bit (the grouped form only changes which tile goes where),
    and for every expert that has rows its first row tile and its last (ragged) one agree with the
    dequantize-then-float64 product over all 4096 output columns."""
    import hpfp8
    experts, total, N, K = 32, 131072, 4096, 7168
    counts = _zipf_counts(total, experts, 7)
    assert int(counts.sum()) == total and int((counts == 0).sum()) >= 2
    offs = counts.cumsum(0).to(torch.int32).to(gpu)
    g = torch.Generator(device=gpu).manual_seed(3)
    xq = torch.empty((total, K), dtype=torch.float8_e4m3fn, device=gpu)
    sxi = torch.empty((K // 128, total), dtype=torch.float32, device=gpu).t()
    for r0 in range(0, total, 16384):
        xc = torch.randn((16384, K), generator=g, device=gpu).to(torch.bfloat16)
        q_, s_ = hpfp8.quantize_1x128(xc, kmajor=True)
        xq[r0:r0 + 16384] = q_
        sxi[r0:r0 + 16384] = s_
    wq = torch.empty((experts, N, K), dtype=torch.float8_e4m3fn, device=gpu)
    swi = torch.empty((experts, N // 128, K // 128), dtype=torch.float32, device=gpu)
    for e in range(experts):
        wc = (torch.randn((N, K), generator=g, device=gpu) * 0.006).to(torch.bfloat16)
        wq[e], swi[e] = hpfp8.quantize_128x128(wc)
    del xc, wc
    y = hpfp8.gemm_grouped_blockwise(xq, sxi, wq, swi, offs)
    assert y.shape == (total, N) and y.dtype == torch.bfloat16
    start, checked = 0, 0
    for e in range(experts):
        cnt = int(counts[e])
        if cnt:
            dense = hpfp8.gemm_blockwise(xq[start:start + cnt], sxi[start:start + cnt], wq[e], swi[e])
            assert torch.equal(y[start:start + cnt], dense), f"expert {e}"
            del dense
            wd = dequant_f64(wq[e], swi[e].repeat_interleave(128, dim=0), gpu)
            last0 = start + (cnt - 1) // 256 * 256
            for r0, r1 in {(start, min(start + 256, start + cnt)), (last0, start + cnt)}:
                ref = dequant_f64(xq[r0:r1], sxi[r0:r1], gpu) @ wd.t()
                d = (y[r0:r1].double() - ref).abs()
                assert float(d.norm() / ref.norm()) < TOL_BF16, f"expert {e} rows {r0}..{r1}"
                xa = dequant_f64(xq[r0:r1], sxi[r0:r1], gpu)
                bound = ref.abs() * 2.0 ** -8 + 2.0 ** -10 * (xa.abs().view(r1 - r0, -1, 128).amax(dim=2) @
                                                              wd.abs().view(N, -1, 128).amax(dim=2).t())
                assert bool((d <= bound).all()), f"expert {e} rows {r0}..{r1}"
                checked += 1
            del wd
        start += cnt
    assert checked >= int((counts > 0).sum())


def test_activation_matrix_larger_than_2_gib(gpu):
    """Tiles are addressed relative to their own first row, so the code matrix as a whole may exceed
    what a 32-bit byte offset spans: rows beyond byte 2^31 give the same bits as the same rows
    passed on their own."""
    import hpfp8
    M, N, K = 327680, 256, 7168                      # a is 2.19 GiB
    g = torch.Generator(device=gpu).manual_seed(9)
    a = torch.randint(0, 0x7F, (M, K), generator=g, device=gpu, dtype=torch.uint8)
    a |= torch.randint(0, 2, (M, K), generator=g, device=gpu, dtype=torch.uint8) << 7
    a = a.view(torch.float8_e4m3fn)
    sa = (torch.rand((K // 128, M), generator=g, device=gpu) + 0.5).t()
    w = (torch.randn((N, K), generator=g, device=gpu) * 0.01).to(torch.bfloat16)
    wq, sw = hpfp8.quantize_128x128(w)
    y = hpfp8.gemm_blockwise(a, sa, wq, sw)
    for r0 in (0, 299520, M - 256):                  # 299520 * 7168 is just below 2^31, the tile crosses it
        part = hpfp8.gemm_blockwise(a[r0:r0 + 256], sa[r0:r0 + 256], wq, sw)
        assert torch.equal(y[r0:r0 + 256], part), r0
    ref = ref_f64_torch(a[M - 256:], sa[M - 256:], wq, sw.repeat_interleave(128, dim=0), gpu)
    assert rel(U.f32(y[M - 256:]), ref.cpu().numpy()) < TOL_BF16


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_output_matrix_larger_than_4_gib(gpu, out_dtype):
    """A tile's stores are addressed relative to the tile's first element (32-bit offsets inside the tile,
    64-bit base), so c as a whole may exceed 4 GiB: rows whose byte offset lies beyond 2^32 hold the same
    bits as the same rows computed on their own, and the accumulate form adds onto them in place."""
    import hpfp8
    f32 = out_dtype == torch.float32
    M, N, K = (33024, 36864, 128) if f32 else (65792, 36864, 128)      # c is 4.5 GiB either way
    g = torch.Generator(device=gpu).manual_seed(11)
    a = torch.randint(0, 0x7F, (M, K), generator=g, device=gpu, dtype=torch.uint8).view(torch.float8_e4m3fn)
    sa = (torch.rand((1, M), generator=g, device=gpu) + 0.5).t()
    w = (torch.randn((N, K), generator=g, device=gpu) * 0.01).to(torch.bfloat16)
    wq, sw = hpfp8.quantize_128x128(w)
    y = hpfp8.gemm_blockwise(a, sa, wq, sw, out_dtype=out_dtype)
    assert y.numel() * y.element_size() > (1 << 32)
    first_beyond = (1 << 32) // (N * y.element_size())                 # the row that contains byte 2^32
    for r0 in (0, first_beyond - 128, M - 256, M - 100):
        part = hpfp8.gemm_blockwise(a[r0:r0 + 256], sa[r0:r0 + 256], wq, sw, out_dtype=out_dtype)
        assert torch.equal(y[r0:r0 + 256], part), r0
    ref = ref_f64_torch(a[M - 256:], sa[M - 256:], wq, sw.repeat_interleave(128, dim=0), gpu)
    assert rel(U.f32(y[M - 256:].float()), ref.cpu().numpy()) < (TOL_F32 if f32 else TOL_BF16)
    if f32:
        w1, sw1 = hpfp8.quantize_1x128(w, kmajor=True)
        before = y[M - 256:].clone()
        add = hpfp8.gemm_blockwise(a[M - 256:], sa[M - 256:], w1, sw1, sb_gran=1, out_dtype=torch.float32)
        hpfp8.gemm_blockwise(a, sa, w1, sw1, sb_gran=1, out=y, accumulate=True)
        assert rel(U.f32(y[M - 256:]), U.f32(before + add)) < 1e-6


def test_weight_matrix_larger_than_2_gib(gpu):
    """The b operand beyond 2^31 bytes (dense, and as the stacked weights of a grouped call): columns of c
    that belong to weight rows past that mark equal the same rows passed on their own."""
    import hpfp8
    M, N, K = 256, 327680, 7168                      # b is 2.19 GiB
    g = torch.Generator(device=gpu).manual_seed(12)
    b = torch.randint(0, 0x7F, (N, K), generator=g, device=gpu, dtype=torch.uint8)
    b |= torch.randint(0, 2, (N, K), generator=g, device=gpu, dtype=torch.uint8) << 7
    b = b.view(torch.float8_e4m3fn)
    sb = torch.rand((N // 128, K // 128), generator=g, device=gpu) + 0.5
    x = torch.randn((M, K), generator=g, device=gpu).to(torch.bfloat16)
    xq, sx = hpfp8.quantize_1x128(x, kmajor=True)
    y = hpfp8.gemm_blockwise(xq, sx, b, sb)
    for n0 in (0, 299520, N - 256):                  # 299520 * 7168 is just below 2^31
        part = hpfp8.gemm_blockwise(xq, sx, b[n0:n0 + 256], sb[n0 // 128:n0 // 128 + 2])
        assert torch.equal(y[:, n0:n0 + 256], part), n0
    ref = ref_f64_torch(xq, sx, b[N - 256:], sb[(N - 256) // 128:].repeat_interleave(128, dim=0), gpu)
    assert rel(U.f32(y[:, N - 256:]), ref.cpu().numpy()) < TOL_BF16
    # the same bytes as 80 experts of 4096 rows each: the last expert's weights lie beyond 2^31
    E, Ne = 80, 4096
    offs = torch.zeros(E, dtype=torch.int32, device=gpu)
    offs[-2:] = torch.tensor([100, M], dtype=torch.int32)       # experts 0..77 empty, 78 gets 100 rows, 79 the rest
    yg = hpfp8.gemm_grouped_blockwise(xq, sx, b.view(E, Ne, K), sb.view(E, Ne // 128, K // 128), offs)
    assert torch.equal(yg[:100], hpfp8.gemm_blockwise(xq[:100], sx[:100], b[78 * Ne:79 * Ne], sb[78 * 32:79 * 32]))
    assert torch.equal(yg[100:], hpfp8.gemm_blockwise(xq[100:], sx[100:], b[79 * Ne:], sb[79 * 32:]))


@pytest.fixture
def small_gemm_mode():
    """Sets the kernel-selection hook for one test and restores the default rule afterwards."""
    from hpfp8 import _lib
    lib = _lib.load()
    yield lib.hpfp8_debug_set_small_gemm
    lib.hpfp8_debug_set_small_gemm(0)


@pytest.mark.parametrize("shape", [(2048, 1024, 1024), (1, 128, 128), (130, 384, 256), (64, 2304, 512), (257, 128, 1152),
                                   (1000, 640, 384), (2048, 2304, 256), (4100, 1024, 384)])
def test_small_tile_kernel_equals_the_large_tile_kernel_and_the_oracle(gpu, shape, small_gemm_mode):
    """The small-tile kernel (problems with few tiles: BASELINE configuration 1, decode-sized M) does the same
    arithmetic in the same order as the 256 x 256-tile kernel: identical bits for the block and the per-tensor
    form, fp32 and bf16 output, with and without bias, ragged M; and the fp32 output agrees with the oracle as the
    large kernel's does.  Both of its tile heights are covered: 64 rows where 128 x 128 tiles would be fewer than the
    256 compute units (the first six shapes), 128 rows otherwise (288 and 264 such tiles in the last two)."""
    import hpfp8
    m, n, k = shape
    x = U.randn_bf16((m, k), 40 + m, 1.0, 0.001, 30.0).to(gpu)
    w = U.randn_bf16((n, k), 41 + n, 0.05).to(gpu)
    bias = U.randn_bf16((n,), 42, 0.5).to(gpu)
    xq, sx = hpfp8.quantize_1x128(x)
    wq, sw = hpfp8.quantize_128x128(w)
    xt, _, sxt = hpfp8.quantize_per_tensor(x)
    wt, _, swt = hpfp8.quantize_per_tensor(w)
    out = {}
    for mode in (1, 2):
        small_gemm_mode(mode)
        out[mode] = [hpfp8.gemm_blockwise(xq, sx, wq, sw, out_dtype=torch.float32),
                     hpfp8.gemm_blockwise(xq, sx, wq, sw, bias=bias),
                     hpfp8.gemm_per_tensor(xt, sxt, wt, swt, out_dtype=torch.float32),
                     hpfp8.gemm_per_tensor(xt, sxt, wt, swt, bias=bias)]
    for big, small in zip(out[1], out[2]):
        assert torch.equal(big.view(torch.int32) if big.dtype == torch.float32 else big.view(torch.int16),
                           small.view(torch.int32) if small.dtype == torch.float32 else small.view(torch.int16))
    if m * n * k <= 2048 * 1024 * 1024:
        want, _ = O.gemm_blockwise(U.codes(xq), U.f32(sx), U.codes(wq), U.f32(sw))
        assert rel(U.f32(out[2][0]), want) < TOL_F32
    # a strided a operand and k-block-major scales take the same path
    small_gemm_mode(2)
    xq2, sx2 = hpfp8.quantize_1x128(x, kmajor=True)
    c2 = hpfp8.gemm_blockwise(xq2, sx2, wq, sw, out_dtype=torch.float32)
    assert torch.equal(c2, out[2][0])


def test_small_problems_select_the_small_tile_kernel(gpu, small_gemm_mode):
    """Under the default rule configuration 1 (32 large tiles) runs the small-tile kernel and configuration 2 does
    not; observable through the hook: forcing either kernel gives the same bits, so only timing can tell -- here
    the rule itself is checked through identical results in all three modes on a small and a larger problem."""
    import hpfp8
    for m, n, k in ((2048, 1024, 1024), (1024, 8192, 256)):
        x = U.randn_bf16((m, k), 50, 1.0).to(gpu)
        w = U.randn_bf16((n, k), 51, 0.05).to(gpu)
        xq, sx = hpfp8.quantize_1x128(x, kmajor=True)
        wq, sw = hpfp8.quantize_128x128(w)
        res = []
        for mode in (0, 1, 2):
            small_gemm_mode(mode)
            res.append(hpfp8.gemm_blockwise(xq, sx, wq, sw))
        assert torch.equal(res[0], res[1]) and torch.equal(res[0], res[2])
