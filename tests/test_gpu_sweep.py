"""Seeded random sweeps over shapes, layouts and options of the GEMM and quantizer entry points.

GEMM cases use integer-valued operands and power-of-two scales, so every product and sum is exact in fp32
and the result must equal the float64 dequantized matmul bit for bit whatever the kernel's tiling and
summation order; quantizer cases are compared bit for bit with the C restatement of the oracle.  Each case
prints its parameters first, so a failure (or a fault) names the case."""
import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from oracle import c_oracle as C
import _util as U

pytestmark = pytest.mark.gpu


def _eq_f32(t, ref):
    return np.array_equal(U.f32_bits(U.f32(t)), U.f32_bits(ref))


@pytest.fixture(params=["large tiles only", "default rule"])
def gemm_kernel_choice(request):
    """The sweep's shapes have few tiles: once with the small-tile kernel switched off, once under the default rule."""
    from hpfp8 import _lib
    lib = _lib.load()
    lib.hpfp8_debug_set_small_gemm(1 if request.param == "large tiles only" else 0)
    yield
    lib.hpfp8_debug_set_small_gemm(0)


@pytest.mark.parametrize("seed", [0, 1])
def test_random_gemm_cases_are_exact(gpu, seed, gemm_kernel_choice):
    import hpfp8
    rng = np.random.default_rng(seed)
    lut = torch.nan_to_num(torch.from_numpy(O.e4m3_decode(np.arange(256, dtype=np.uint8)).astype(np.float64)).to(gpu))

    def deq(q):
        return lut[q.view(torch.uint8).long()]

    def enc(a):
        return torch.from_numpy(O.e4m3_encode(a)).to(gpu).view(torch.float8_e4m3fn)

    def pow2s(shape):
        return torch.from_numpy((2.0 ** rng.integers(-3, 4, size=shape)).astype(np.float32)).to(gpu)

    for case in range(60):
        M = int(rng.choice([1, 7, 100, 255, 256, 257, 300, 511, 513, 700, 1030, 2049]))
        N = 128 * int(rng.integers(1, 12))
        K = 128 * int(rng.integers(1, 7))
        mode = str(rng.choice(["block", "row", "tensor", "grouped"]))
        f32 = bool(rng.integers(0, 2))
        bias = bool(rng.integers(0, 2)) and mode != "grouped"
        acc = f32 and mode in ("block", "row") and bool(rng.integers(0, 2))
        hw = mode != "tensor" and bool(rng.integers(0, 2))          # scales applied by the matrix instruction
        pad = int(rng.choice([0, 8, 24]))
        kmajor = bool(rng.integers(0, 2))
        print(f"seed {seed} case {case}: {mode} M={M} N={N} K={K} f32={f32} bias={bias} acc={acc} hw={hw} pad={pad} "
              f"kmajor={kmajor}", flush=True)
        kb = K // 128
        a = enc(rng.integers(-8, 9, size=(M, K)).astype(np.float32))
        sa = pow2s((M, kb))
        if kmajor:
            sa = sa.t().contiguous().t()
        dt = torch.float32 if f32 else torch.bfloat16
        bvec = torch.from_numpy(rng.integers(-64, 65, size=(N,)).astype(np.float32)).to(gpu).to(torch.bfloat16) if bias else None
        wide = torch.full((M, N + pad), 3.0, dtype=dt, device=gpu)
        c = wide[:, 8:8 + N] if pad else wide
        A = deq(a) * sa.double().repeat_interleave(128, dim=1)
        if mode == "grouped":
            E = int(rng.integers(1, 6))
            cuts = np.sort(rng.integers(0, M + 1, size=E - 1)) if E > 1 else np.array([], dtype=np.int64)
            offs = np.concatenate([cuts, [M]]).astype(np.int32)
            b = enc(rng.integers(-8, 9, size=(E * N, K)).astype(np.float32)).view(E, N, K)
            sb = pow2s((E, N // 128, kb))
            got = hpfp8.gemm_grouped_blockwise(a, sa, b, sb, torch.from_numpy(offs).to(gpu), out_dtype=dt, pow2_scales=hw)
            want = torch.zeros(M, N, dtype=torch.float64, device=gpu)
            prev = 0
            for e in range(E):
                B = deq(b[e]) * sb[e].double().repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
                want[prev:offs[e]] = A[prev:offs[e]] @ B.t()
                prev = int(offs[e])
        elif mode == "tensor":
            b = enc(rng.integers(-8, 9, size=(N, K)).astype(np.float32))
            got = hpfp8.gemm_per_tensor(a, torch.tensor([0.5], device=gpu), b, torch.tensor([0.25], device=gpu),
                                        bias=bvec, out_dtype=dt)
            want = (deq(a) @ deq(b).t()) * 0.125
        else:
            b = enc(rng.integers(-8, 9, size=(N, K)).astype(np.float32))
            gran = 128 if mode == "block" else 1
            sb = pow2s((N // gran, kb))
            Bs = deq(b) * sb.double().repeat_interleave(gran, dim=0).repeat_interleave(128, dim=1)
            want = A @ Bs.t()
            if acc:
                old = torch.from_numpy(rng.integers(-500, 501, size=(M, N)).astype(np.float32)).to(gpu)
                c.copy_(old)
                want = want + old.double()
            hpfp8.gemm_blockwise(a, sa, b, sb, bias=bvec, sb_gran=gran, out=c, accumulate=acc, pow2_scales=hw)
            got = c
        if bias:
            want = want + bvec.double()[None, :]
        # integer / dyadic values: exact in fp32; in bf16, one rounding of the exact value
        assert torch.equal(got, want.to(dt)), "result differs"
        if mode in ("block", "row") and pad:
            assert bool((wide[:, :8] == 3.0).all()) and bool((wide[:, 8 + N:] == 3.0).all()), "wrote outside its columns"


@pytest.mark.parametrize("seed", [0])
def test_random_quantizer_cases_are_bit_exact(gpu, seed):
    import hpfp8
    rng = np.random.default_rng(seed)
    for case in range(40):
        rows = int(rng.choice([1, 3, 16, 100, 127, 128, 129, 300, 640]))
        cols = 128 * int(rng.integers(1, 20))
        std = float(rng.choice([1e-6, 1e-3, 0.02, 1.0, 300.0, 1e30]))
        of = float(rng.choice([0.0, 0.001, 0.05]))
        om = float(rng.choice([1.0, 50.0, 1e3]))
        pow2 = bool(rng.integers(0, 2))
        print(f"seed {seed} case {case}: rows={rows} cols={cols} std={std} of={of} om={om} pow2={pow2}", flush=True)
        x = U.randn_bf16((rows, cols), int(rng.integers(0, 1 << 30)), std, of, om)
        if rng.integers(0, 3) == 0:      # a zero group, a negative zero, the smallest subnormal
            xb0 = U.bits(x).copy()
            xb0[rng.integers(0, rows), :128] = 0
            xb0[rng.integers(0, rows), rng.integers(0, cols)] = 0x8000
            xb0[rng.integers(0, rows), rng.integers(0, cols)] = 0x0001
            x = U.from_bits(xb0)
        xb = U.bits(x)
        xg = x.to(gpu)
        q, s, si = hpfp8.quantize_per_tensor(xg)
        rq, rs, rsi = C.quantize_per_tensor(xb)
        assert np.array_equal(U.codes(q), rq) and _eq_f32(s, rs) and _eq_f32(si, rsi), "per tensor"
        ref = O if pow2 else C
        kw = {"pow2": True} if pow2 else {}
        rq1, rs1, rsi1 = ref.quantize_1x128(xb, **kw)
        for km in ((True,) if pow2 else (False, True)):
            q, s, si = hpfp8.quantize_1x128(xg, want_scale=True, kmajor=km, **kw)
            assert np.array_equal(U.codes(q), rq1) and _eq_f32(s, rs1) and _eq_f32(si, rsi1), f"1x128 kmajor={km}"
        assert np.array_equal(U.bits(hpfp8.dequantize_1x128(q, si.contiguous())), C.dequantize_1x128(rq1, rsi1)), "dequantize"
        if rows % 128 == 0:
            q, si, qt, s = hpfp8.quantize_128x128(xg, with_transpose=True, want_scale=True, **kw)
            rq, rs, rsi = ref.quantize_128x128(xb, **kw)
            assert np.array_equal(U.codes(q), rq) and _eq_f32(s, rs) and _eq_f32(si, rsi) and np.array_equal(U.codes(qt), rq.T), "128x128"
            assert np.array_equal(U.codes(hpfp8.transpose_codes(q)), rq.T), "transpose_codes"
            rqt, rst, rsit = ref.quantize_128x1_t(xb, **kw)
            for km in ((True,) if pow2 else (False, True)):
                qt, s, si = hpfp8.quantize_128x1_t(xg, want_scale=True, kmajor=km, **kw)
                assert np.array_equal(U.codes(qt), rqt) and _eq_f32(s, rst) and _eq_f32(si, rsit), f"128x1_t kmajor={km}"
                q1, si1, qt2, sit2 = hpfp8.quantize_1x128_and_128x1_t(xg, kmajor=km, **kw)
                assert np.array_equal(U.codes(q1), rq1) and _eq_f32(si1, rsi1) and np.array_equal(U.codes(qt2), rqt) \
                    and _eq_f32(sit2, rsit), f"both forms kmajor={km}"
        if cols % 256 == 0 and std <= 300.0:
            wq, _, wsi, wact = O.swiglu_quantize_1x128(xb, **kw)
            for km in (False, True):
                q, si, act = hpfp8.swiglu_quantize_1x128(xg, kmajor=km, want_act=True, **kw)
                assert np.array_equal(U.codes(q), wq) and _eq_f32(si, wsi) and np.array_equal(U.bits(act), wact), f"swiglu kmajor={km}"
