"""GPU parity of the quantize / dequantize kernels through the C ABI: codes byte-exact and fp32
scales bit-exact against the CPU oracle on the same seeded inputs and on the golden fixtures."""
import os

import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
from oracle import c_oracle as C
import _util as U

pytestmark = pytest.mark.gpu
G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_path_golden.npz"))


def eq_f32(gpu_t, ref):
    return np.array_equal(U.f32_bits(U.f32(gpu_t)), U.f32_bits(ref))


def test_hardware_cast_all_bf16_patterns(gpu):
    """Every finite bf16 bit pattern through the cast with scale 1 (amax = 448) and with a scale that
    makes results land in the subnormal range: the hardware converter must agree with the oracle."""
    import hpfp8
    b = np.arange(65536, dtype=np.uint16)
    f = O.bf16_bits_to_f32(b)
    keep = np.isfinite(f)
    b = b[keep]
    pad = (-b.size) % 128
    b = np.concatenate([b, np.zeros(pad, np.uint16)])
    x = U.from_bits(b, gpu)
    for amax_val in (448.0, 448.0 * 64, 448.0 * 2 ** 20, 1.0, 2.0 ** -100, 3.0 / 7.0):
        am = torch.tensor(amax_val, dtype=torch.float32, device=gpu)
        q, s, si = hpfp8.quantize_per_tensor(x, amax_in=am)
        scale, scale_inv = O.scales_from_amax(np.float32(amax_val))
        want = O._cast(O.bf16_bits_to_f32(b), scale)
        assert eq_f32(s, scale) and eq_f32(si, scale_inv)
        got = U.codes(q)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, (amax_val, [(hex(b[i]), got[i], want[i]) for i in bad[:8]])


def test_golden_fixtures(gpu):
    import hpfp8
    x = U.from_bits(G["x_bits"], gpu)
    q, s, si = hpfp8.quantize_per_tensor(x)
    assert np.array_equal(U.codes(q), G["pt_codes"]) and eq_f32(s, G["pt_scale"]) and eq_f32(si, G["pt_scale_inv"])
    q, s, si = hpfp8.quantize_1x128(x, want_scale=True)
    assert np.array_equal(U.codes(q), G["g1x128_codes"]) and eq_f32(s, G["g1x128_scale"]) and eq_f32(si, G["g1x128_scale_inv"])
    d = hpfp8.dequantize_1x128(q, si)
    assert np.array_equal(U.bits(d), G["g1x128_dequant_bits"])
    q, si, qt, s = hpfp8.quantize_128x128(x, with_transpose=True, want_scale=True)
    assert np.array_equal(U.codes(q), G["b128_codes"]) and eq_f32(s, G["b128_scale"]) and eq_f32(si, G["b128_scale_inv"])
    assert np.array_equal(U.codes(qt), G["b128_codes"].T)
    qt, s, si = hpfp8.quantize_128x1_t(x, want_scale=True)
    assert np.array_equal(U.codes(qt), G["t128x1_codes"]) and eq_f32(s, G["t128x1_scale"]) and eq_f32(si, G["t128x1_scale_inv"])
    c, si = hpfp8.quantize_bucket(U.from_bits(G["bucket_bits"], gpu))
    assert np.array_equal(U.codes(c), G["bucket_codes"]) and eq_f32(si, G["bucket_scale_inv"])
    back = hpfp8.dequantize_bucket(c, si, grad_scale=0.125)
    assert np.array_equal(U.bits(back), G["bucket_back_bits"])
    P = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_pow2_golden.npz"))
    q, s, si = hpfp8.quantize_1x128(x, want_scale=True, kmajor=True, pow2=True)
    assert np.array_equal(U.codes(q), P["g1x128_codes"]) and eq_f32(s, P["g1x128_scale"]) and eq_f32(si, P["g1x128_scale_inv"])
    q, si, qt, s = hpfp8.quantize_128x128(x, with_transpose=True, want_scale=True, pow2=True)
    assert np.array_equal(U.codes(q), P["b128_codes"]) and eq_f32(s, P["b128_scale"]) and eq_f32(si, P["b128_scale_inv"])
    qt, s, si = hpfp8.quantize_128x1_t(x, want_scale=True, kmajor=True, pow2=True)
    assert np.array_equal(U.codes(qt), P["t128x1_codes"]) and eq_f32(s, P["t128x1_scale"]) and eq_f32(si, P["t128x1_scale_inv"])


@pytest.mark.parametrize("pow2", [False, True])
def test_128x128_two_blocks_per_workgroup(gpu, pow2):
    # from 4096 blocks on, with an even number of block columns and no transposed copy, a workgroup quantizes two
    # neighbouring blocks: same bits as the oracle and as the one-block kernel (which the transposing call uses)
    import hpfp8
    x = U.randn_bf16((16384, 4096), 21, 0.05, 0.002, 300.0)
    xb = U.bits(x)
    xg = x.to(gpu)
    rq, rs, rsi = O.quantize_128x128(xb, pow2=True) if pow2 else C.quantize_128x128(xb)
    q, si, s = hpfp8.quantize_128x128(xg, want_scale=True, pow2=pow2)
    assert np.array_equal(U.codes(q), rq) and eq_f32(s, rs) and eq_f32(si, rsi)
    q1, si1, qt1, s1 = hpfp8.quantize_128x128(xg, with_transpose=True, want_scale=True, pow2=pow2)
    assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(si, si1) and torch.equal(s, s1)


@pytest.mark.parametrize("shape,seed,std,of,om", [
    ((2048, 1024), 0, 1.0, 0.0, 1.0),          # cfg 1 activations
    ((1024, 1024), 1, 0.02, 0.0, 1.0),         # cfg 1 weights
    ((512, 7168), 2, 1.0, 0.001, 50.0),        # cfg 2 activations (row subset)
    ((384, 640), 3, 0.006, 0.0, 1.0),
    ((128, 128), 4, 1e-4, 1e-3, 1e3),
])
def test_seeded_parity_all_quantizers(gpu, shape, seed, std, of, om):
    import hpfp8
    x = U.randn_bf16(shape, seed, std, of, om)
    xb = U.bits(x)
    xg = x.to(gpu)
    # per tensor (amax reduction + cast)
    q, s, si = hpfp8.quantize_per_tensor(xg)
    rq, rs, rsi = C.quantize_per_tensor(xb)
    assert eq_f32(hpfp8.amax(xg), O.amax(O.bf16_bits_to_f32(xb)))
    assert np.array_equal(U.codes(q), rq) and eq_f32(s, rs) and eq_f32(si, rsi)
    # 1x128
    q, s, si = hpfp8.quantize_1x128(xg, want_scale=True)
    rq, rs, rsi = C.quantize_1x128(xb)
    assert np.array_equal(U.codes(q), rq) and eq_f32(s, rs) and eq_f32(si, rsi)
    assert np.array_equal(U.bits(hpfp8.dequantize_1x128(q, si)), C.dequantize_1x128(rq, rsi))
    # 128x128 with transposed copy
    q, si, qt, s = hpfp8.quantize_128x128(xg, with_transpose=True, want_scale=True)
    rq, rs, rsi = C.quantize_128x128(xb)
    assert np.array_equal(U.codes(q), rq) and eq_f32(s, rs) and eq_f32(si, rsi)
    assert np.array_equal(U.codes(qt), rq.T)
    q2, si2 = hpfp8.quantize_128x128(xg)
    assert np.array_equal(U.codes(q2), rq) and eq_f32(si2, rsi)
    assert np.array_equal(U.bits(hpfp8.dequantize_128x128(q, si)), O.dequantize_128x128(rq, rsi))
    # 128x1 transposed
    qt, s, si = hpfp8.quantize_128x1_t(xg, want_scale=True)
    rq, rs, rsi = C.quantize_128x1_t(xb)
    assert np.array_equal(U.codes(qt), rq) and eq_f32(s, rs) and eq_f32(si, rsi)
    # both forms from one read of x: same codes and scales as the two separate quantizers
    rq1, _, rsi1 = C.quantize_1x128(xb)
    for kmajor in (True, False):
        q1, si1, qt2, sit2 = hpfp8.quantize_1x128_and_128x1_t(xg, kmajor=kmajor)
        assert np.array_equal(U.codes(q1), rq1) and eq_f32(si1, rsi1)
        assert np.array_equal(U.codes(qt2), rq) and eq_f32(sit2, rsi)
        if min(si1.shape) > 1 and min(sit2.shape) > 1:      # (strides of a one-column tensor say nothing)
            assert (si1.stride(0) == 1) == kmajor and (sit2.stride(0) == 1) == kmajor


@pytest.mark.parametrize("shape,seed,std,of,om", [
    ((512, 7168), 2, 1.0, 0.001, 50.0),
    ((384, 640), 3, 0.006, 0.0, 1.0),
    ((128, 128), 4, 1e-4, 1e-3, 1e3),
    ((256, 256), 5, 1e30, 0.0, 1.0),
])
def test_power_of_two_scale_quantizers(gpu, shape, seed, std, of, om):
    """The optional recipe with scale_inv rounded up to a power of two: codes and scales of all four
    entry points bit for bit against the oracle."""
    import hpfp8
    x = U.randn_bf16(shape, seed, std, of, om)
    x[0, :128] = 0                                   # an all-zero group
    xb = U.bits(x)
    xg = x.to(gpu)
    q, s, si = hpfp8.quantize_1x128(xg, want_scale=True, kmajor=True, pow2=True)
    rq, rs, rsi = O.quantize_1x128(xb, pow2=True)
    assert np.array_equal(U.codes(q), rq) and eq_f32(s, rs) and eq_f32(si, rsi)
    assert not (U.f32_bits(U.f32(si)) & 0x007FFFFF).any()
    q, si, qt, s = hpfp8.quantize_128x128(xg, with_transpose=True, want_scale=True, pow2=True)
    rqw, rsw, rsiw = O.quantize_128x128(xb, pow2=True)
    assert np.array_equal(U.codes(q), rqw) and eq_f32(s, rsw) and eq_f32(si, rsiw) and np.array_equal(U.codes(qt), rqw.T)
    qt, s, si = hpfp8.quantize_128x1_t(xg, want_scale=True, kmajor=True, pow2=True)
    rqt, rst, rsit = O.quantize_128x1_t(xb, pow2=True)
    assert np.array_equal(U.codes(qt), rqt) and eq_f32(s, rst) and eq_f32(si, rsit)
    q1, si1, qt2, sit2 = hpfp8.quantize_1x128_and_128x1_t(xg, kmajor=True, pow2=True)
    assert np.array_equal(U.codes(q1), rq) and eq_f32(si1, rsi)
    assert np.array_equal(U.codes(qt2), rqt) and eq_f32(sit2, rsit)
    with pytest.raises(ValueError):
        hpfp8.quantize_1x128(xg, pow2=True)          # only the k-block-major layout


@pytest.mark.parametrize("shape", [(512, 7168), (100, 384), (16, 128), (33, 640)])
def test_kmajor_scale_layouts_hold_the_same_values(gpu, shape):
    import hpfp8
    x = U.randn_bf16(shape, 77, 1.0, 0.001, 50.0)
    xg = x.to(gpu)
    q, s, si = hpfp8.quantize_1x128(xg, want_scale=True)
    qk, sk, sik = hpfp8.quantize_1x128(xg, want_scale=True, kmajor=True)
    assert sik.shape == si.shape and sik.stride(0) == 1            # stored [C/128, rows]
    assert torch.equal(q.view(torch.uint8), qk.view(torch.uint8)) and torch.equal(si, sik) and torch.equal(s, sk)
    rq, rs, rsi = C.quantize_1x128(U.bits(x))
    assert np.array_equal(U.codes(qk), rq) and eq_f32(sik, rsi) and eq_f32(sk, rs)
    if shape[0] % 128 == 0:
        qt, st, sit = hpfp8.quantize_128x1_t(xg, want_scale=True)
        qtk, stk, sitk = hpfp8.quantize_128x1_t(xg, want_scale=True, kmajor=True)
        assert sitk.stride(0) == 1 and torch.equal(qt.view(torch.uint8), qtk.view(torch.uint8))
        assert torch.equal(sit, sitk) and torch.equal(st, stk)


def test_laplace_gradients_and_transposed_identity(gpu):
    import hpfp8
    go = U.laplace_bf16((512, 896), seed=9, scale=1e-3)
    gg = go.to(gpu)
    qt, si = hpfp8.quantize_128x1_t(gg)
    q, si2 = hpfp8.quantize_1x128(gg.t().contiguous())
    assert torch.equal(qt.view(torch.uint8), q.view(torch.uint8)) and torch.equal(si, si2)
    rq, rs, rsi = C.quantize_128x1_t(U.bits(go))
    assert np.array_equal(U.codes(qt), rq) and eq_f32(si, rsi)


def test_special_values_and_edge_shapes(gpu):
    import hpfp8
    sp = U.special_bf16_rows(256)
    q, s, si = hpfp8.quantize_1x128(sp.to(gpu), want_scale=True)
    rq, rs, rsi = O.quantize_1x128(U.bits(sp))
    assert np.array_equal(U.codes(q), rq) and eq_f32(s, rs) and eq_f32(si, rsi)
    # empty tensors
    e = torch.empty((0, 128), dtype=torch.bfloat16, device=gpu)
    q, si = hpfp8.quantize_1x128(e)
    assert q.shape == (0, 128) and si.shape == (0, 1)
    assert float(hpfp8.amax(torch.empty((0,), dtype=torch.bfloat16, device=gpu))) == 0.0
    # per-tensor with a ragged tail (numel not a multiple of 8)
    x = U.randn_bf16((1003,), 17)
    q, s, si = hpfp8.quantize_per_tensor(x.to(gpu))
    rq, rs, rsi = O.quantize_per_tensor(U.bits(x))
    assert np.array_equal(U.codes(q), rq) and eq_f32(s, rs) and eq_f32(si, rsi)
    # one group, one row; 3-D input
    x = U.randn_bf16((3, 5, 256), 18)
    q, si = hpfp8.quantize_1x128(x.to(gpu))
    rq, rs, rsi = O.quantize_1x128(U.bits(x).reshape(15, 256))
    assert np.array_equal(U.codes(q).reshape(15, 256), rq) and eq_f32(si.reshape(15, 2), rsi)
    with pytest.raises(ValueError):
        hpfp8.quantize_1x128(torch.zeros((4, 100), dtype=torch.bfloat16, device=gpu))
    with pytest.raises(ValueError):
        hpfp8.quantize_128x1_t(torch.zeros((100, 128), dtype=torch.bfloat16, device=gpu))


def test_non_finite_inputs_every_quantizer(gpu):
    """NaN and +-Inf planted in known groups: scales bit for bit (NaN where the oracle's are NaN), codes
    byte for byte up to the sign of NaN codes, for every quantizer; groups beside the planted ones keep
    ordinary codes; dequantized, the planted groups are NaN throughout."""
    import hpfp8
    x = U.nonfinite_bf16(256, 512)
    xb = U.bits(x)
    xg = x.to(gpu)

    def same(q, rq, scales, rscales):
        assert np.array_equal(U.canon_nan_codes(U.codes(q)), U.canon_nan_codes(rq))
        for a, b in zip(scales, rscales):
            assert U.same_f32_or_nan(U.f32(a), b)

    rq, rs, rsi = O.quantize_1x128(xb)
    for kmajor in (False, True):
        q, s, si = hpfp8.quantize_1x128(xg, want_scale=True, kmajor=kmajor)
        same(q, rq, (s, si), (rs, rsi))
    clean = np.isfinite(rsi)
    assert clean.sum() == rsi.size - 5
    assert not ((U.codes(q).reshape(256, 4, 128)[clean] & 0x7F) == 0x7F).any()
    d = U.f32(hpfp8.dequantize_1x128(q, si.contiguous()).float()).reshape(256, 4, 128)
    assert np.isnan(d[~clean]).all() and np.isfinite(d[clean]).all()
    rqw, rsw, rsiw = O.quantize_128x128(xb)
    q, si, qt, s = hpfp8.quantize_128x128(xg, with_transpose=True, want_scale=True)
    same(q, rqw, (s, si), (rsw, rsiw))
    same(qt, rqw.T, (), ())
    rqt, rst, rsit = O.quantize_128x1_t(xb)
    for kmajor in (False, True):
        qt, s, si = hpfp8.quantize_128x1_t(xg, want_scale=True, kmajor=kmajor)
        same(qt, rqt, (s, si), (rst, rsit))
        q1, si1, qt2, sit2 = hpfp8.quantize_1x128_and_128x1_t(xg, kmajor=kmajor)
        same(q1, rq, (si1,), (rsi,))
        same(qt2, rqt, (sit2,), (rsit,))
    # the power-of-two recipe: the same groups are NaN / Inf
    rq2, rs2, rsi2 = O.quantize_1x128(xb, pow2=True)
    q, s, si = hpfp8.quantize_1x128(xg, want_scale=True, kmajor=True, pow2=True)
    same(q, rq2, (s, si), (rs2, rsi2))
    # per tensor: a NaN anywhere makes every code and both scales NaN; with only an Inf the scale is 0
    q, s, si = hpfp8.quantize_per_tensor(xg)
    rqp, rsp, rsip = O.quantize_per_tensor(xb)
    same(q, rqp, (s, si), (rsp, rsip))
    assert np.isnan(U.f32(s)).all() and ((U.codes(q) & 0x7F) == 0x7F).all()
    xi = xb[1:2].copy()
    q, s, si = hpfp8.quantize_per_tensor(U.from_bits(xi, gpu))
    rqp, rsp, rsip = O.quantize_per_tensor(xi)
    same(q, rqp, (s, si), (rsp, rsip))
    assert float(s) == 0.0 and np.isposinf(U.f32(si)).all()
    # a caller-supplied amax (the clamped cast): NaN elements stay NaN, infinite ones saturate
    am = torch.tensor(3.0, dtype=torch.float32, device=gpu)
    q, s, si = hpfp8.quantize_per_tensor(xg, amax_in=am)
    scale, _ = O.scales_from_amax(np.float32(3.0))
    want = O._cast(O.bf16_bits_to_f32(xb), scale)
    same(q, want, (), ())
    got = U.codes(q)
    assert (got[0, 5] & 0x7F) == 0x7F and got[1, 128 + 77] == 0x7E and got[2, 256 + 1] == 0xFE and ((got & 0x7F) == 0x7F).sum() == 3
    # SwiGLU fused with the quantizer: x as [gate | up], so planted values sit in gates and in ups
    q, si, act = hpfp8.swiglu_quantize_1x128(xg, kmajor=True, want_act=True)
    with np.errstate(all="ignore"):
        rqs, _, rsis, ract = O.swiglu_quantize_1x128(xb)
    same(q, rqs, (si,), (rsis,))
    assert U.same_f32_or_nan(U.f32(act.float()), O.bf16_bits_to_f32(ract))
    assert np.isnan(rsis).sum() + np.isinf(rsis).sum() == 5
    # gradient bucket: quantize, and the fused pack / unpack of the same elements
    flat = xg.reshape(-1)
    c, si = hpfp8.quantize_bucket(flat)
    same(c, rq.reshape(-1), (si,), (rsi,))
    back = hpfp8.dequantize_bucket(c, si, grad_scale=0.5)
    assert np.array_equal(np.isnan(U.f32(back.float())).reshape(256, 4, 128).all(axis=2), ~clean)
    bucket = hpfp8.Fp8GradBucket([flat.numel()], shard_size=1, grad_scale=0.5)
    qb, sib = bucket.pack([flat])
    same(qb, rq.reshape(1, -1), (sib,), (rsi,))
    out = [torch.zeros(flat.numel(), dtype=torch.bfloat16, device=gpu)]
    bucket.unpack(qb[0].contiguous(), sib[0].contiguous(), out)
    assert np.array_equal(np.isnan(U.f32(out[0].float())).reshape(256, 4, 128).all(axis=2), ~clean)
    assert np.array_equal(U.bits(out[0])[np.repeat(clean.reshape(-1), 128)], U.bits(back)[np.repeat(clean.reshape(-1), 128)])


def test_bucket_full_size_properties(gpu):
    """2^29-element bucket (cfg 5): properties that do not need a CPU pass over 1 GiB:
    a strided sample of groups against the oracle, idempotence of quantize(dequantize(.)) on the
    codes, and the per-group error bound."""
    import hpfp8
    n = 1 << 29
    g = torch.Generator(device=gpu).manual_seed(0)
    flat = (torch.randn(n, generator=g, device=gpu, dtype=torch.float32) * 1e-4)
    idx = torch.randint(0, n, (n // 10000,), generator=g, device=gpu)
    flat[idx] *= 1e3
    flat = flat.to(torch.bfloat16)
    codes, si = hpfp8.quantize_bucket(flat)
    assert codes.shape == (n,) and si.shape == (n // 128,)
    # sample of groups vs the oracle
    gsel = torch.arange(0, n // 128, 4099, device=gpu)
    rows = flat.view(-1, 128)[gsel].cpu()
    rq, rs, rsi = O.quantize_1x128(U.bits(rows))
    assert np.array_equal(U.codes(codes.view(-1, 128)[gsel]), rq)
    assert np.array_equal(U.f32_bits(U.f32(si[gsel])), U.f32_bits(rsi.reshape(-1)))
    back = hpfp8.dequantize_bucket(codes, si)
    rback = O.dequantize_1x128(rq, rsi)
    assert np.array_equal(U.bits(back.view(-1, 128)[gsel]), rback)
    # error bound per group: |x - back| <= amax/28 + amax/256
    am = flat.view(-1, 128).float().abs().amax(dim=1, keepdim=True)
    err = (back.view(-1, 128).float() - flat.view(-1, 128).float()).abs()
    assert bool((err <= am / 28 + am / 256 + 1e-30).all())
    del err, am
    # no NaN codes, and every group uses the top of the range (its amax element maps to +-448)
    c8 = codes.view(torch.uint8).view(-1, 128)
    assert not bool(((c8 & 0x7F) == 0x7F).any())
    assert bool((((c8 & 0x7F) == 0x7E).any(dim=1)).all())


@pytest.mark.parametrize("shard_size,grad_scale", [(1, 1.0), (2, 0.125), (4, 0.3)])
def test_fused_bucket_pack_and_unpack(gpu, shard_size, grad_scale):
    """Fp8GradBucket.pack == quantize_1x128 of the oracle's packed rows; unpack == the oracle's cast
    back of one row, sliced.  Sizes cover: multiples of 128, a ragged tail (zero-padded group), a
    parameter smaller than one vector, odd chunk sizes (unaligned chunk starts for shard_size > 1),
    more parameters than one launch carries, and one parameter spanning several workgroups."""
    import hpfp8
    numels = [384 * 256, 1000, 7, 128, 129, 4099, 20000] + [256 + 8 * i for i in range(60)]
    rng = np.random.default_rng(13)
    grads = []
    for e, n in enumerate(numels):
        g = U.randn_bf16((shard_size * n,), 100 + e, 1e-3 * (1 + e % 5), 0.002, 200.0)
        grads.append(g)
    bucket = hpfp8.Fp8GradBucket(numels, shard_size=shard_size, grad_scale=grad_scale)
    offsets, row = O.bucket_offsets(numels)
    assert bucket.offsets == offsets and bucket.row_elems == row
    q, si = bucket.pack([g.to(gpu) for g in grads])
    packed = O.pack_bucket([U.bits(g) for g in grads], numels, shard_size)
    rq, _, rsi = O.quantize_1x128(packed)
    assert np.array_equal(U.codes(q), rq)
    assert np.array_equal(U.f32_bits(U.f32(si)), U.f32_bits(rsi))
    # the reduced row: take row (shard_size - 1) as it is (a real reduction would produce another row of codes)
    r = shard_size - 1
    outs = [torch.full((n,), 7.0, dtype=torch.bfloat16, device=gpu) for n in numels]
    bucket.unpack(q[r].contiguous(), si[r].contiguous(), outs)
    back = O.dequantize_bucket(rq[r], rsi[r], grad_scale)
    for e, piece in enumerate(O.unpack_bucket(back, numels)):
        assert np.array_equal(U.bits(outs[e]), piece), e
    # same values as the unfused path on the packed bf16 row
    flat = torch.from_numpy(packed[r].astype(np.int16)).view(torch.bfloat16).to(gpu)
    c2, s2 = hpfp8.quantize_bucket(flat)
    assert torch.equal(c2.view(torch.uint8), q[r].view(torch.uint8)) and torch.equal(s2, si[r])


def test_bucket_argument_checks(gpu):
    import hpfp8
    b = hpfp8.Fp8GradBucket([256, 100], shard_size=2)
    good = [torch.zeros(512, dtype=torch.bfloat16, device=gpu), torch.zeros(200, dtype=torch.bfloat16, device=gpu)]
    with pytest.raises(ValueError):
        b.pack(good[:1])
    with pytest.raises(ValueError):
        b.pack([good[0], torch.zeros(100, dtype=torch.bfloat16, device=gpu)])
    with pytest.raises(TypeError):
        b.pack([good[0], torch.zeros(200, dtype=torch.float32, device=gpu)])
    q, si = b.pack(good)
    assert q.shape == (2, 384) and si.shape == (2, 3) and not bool(q.view(torch.uint8).any())
    # tensors that do not live on the current GPU never reach a kernel: a row reduced on the host, a host gradient
    outs = [torch.empty(256, dtype=torch.bfloat16, device=gpu), torch.empty(100, dtype=torch.bfloat16, device=gpu)]
    with pytest.raises(ValueError, match="must live on the GPU"):
        b.unpack(q[0].cpu(), si[0], outs)
    with pytest.raises(ValueError, match="must live on the GPU"):
        b.unpack(q[0], si[0].cpu(), outs)
    with pytest.raises(TypeError):
        b.unpack(q[0], si[0], [outs[0].cpu(), outs[1]])
    with pytest.raises(TypeError):
        b.pack([good[0].cpu(), good[1]])
    xq, sx = hpfp8.quantize_1x128(torch.zeros((128, 128), dtype=torch.bfloat16, device=gpu), kmajor=True)
    wq, sw = hpfp8.quantize_128x128(torch.zeros((128, 128), dtype=torch.bfloat16, device=gpu))
    with pytest.raises(ValueError, match="must live on the GPU"):
        hpfp8.gemm_blockwise(xq, sx, wq, sw, out=torch.empty((128, 128), dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="must live on the GPU"):
        hpfp8.gemm_grouped_blockwise(xq, sx, wq.view(1, 128, 128), sw.view(1, 1, 1), torch.tensor([128], dtype=torch.int32))
    with pytest.raises((TypeError, ValueError)):
        hpfp8.dequantize_1x128_accumulate(xq, sx.contiguous(), torch.zeros((128, 128)))


@pytest.mark.parametrize("shape,kmajor", [((256, 768), True), ((100, 256), False), ((512, 36864), True)])
def test_swiglu_fused_with_quantize(gpu, shape, kmajor):
    """act bits, codes and scales of the fused kernel equal the oracle's bit for bit (the exponential is
    defined operation by operation on both sides); act agrees with torch's eager bf16 graph on the GPU
    up to one bf16 ulp where the last place of the sigmoid crosses a rounding boundary; a strided
    input (rows of a wider buffer) gives the same result."""
    import hpfp8
    import torch.nn.functional as F
    m, w2 = shape
    h = U.randn_bf16(shape, 5, 2.0, 0.001, 30.0)
    h[0, :6] = torch.tensor([0.0, -0.0, 88.5, -88.5, -200.0, 200.0], dtype=torch.bfloat16)
    hg = h.to(gpu)
    q, si, act = hpfp8.swiglu_quantize_1x128(hg, kmajor=kmajor, want_act=True)
    rq, _, rsi, ract = O.swiglu_quantize_1x128(U.bits(h))
    assert np.array_equal(U.bits(act), ract)
    assert np.array_equal(U.codes(q), rq) and np.array_equal(U.f32_bits(U.f32(si)), U.f32_bits(rsi))
    assert (si.stride(0) == 1) == kmajor or min(si.shape) == 1
    ref = F.silu(hg[:, :w2 // 2]) * hg[:, w2 // 2:]
    d = (act.view(torch.int16).int() - ref.view(torch.int16).int()).abs()
    both_zero = ((act.view(torch.int16) & 0x7FFF) == 0) & ((ref.view(torch.int16) & 0x7FFF) == 0)
    assert bool(((d <= 1) | both_zero).all()) and float((d != 0).float().mean()) < 2e-3
    wide = torch.zeros((m, w2 + 64), dtype=torch.bfloat16, device=gpu)
    wide[:, :w2] = hg
    q2, si2 = hpfp8.swiglu_quantize_1x128(wide[:, :w2], kmajor=kmajor)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(si2, si)
    # the optional power-of-two scales
    q3, si3 = hpfp8.swiglu_quantize_1x128(hg, kmajor=kmajor, pow2=True)
    rq3, _, rsi3, _ = O.swiglu_quantize_1x128(U.bits(h), pow2=True)
    assert np.array_equal(U.codes(q3), rq3) and np.array_equal(U.f32_bits(U.f32(si3)), U.f32_bits(rsi3))


@pytest.mark.parametrize("pow2", [False, True])
def test_swiglu_fast_form(gpu, pow2):
    """The form with the hardware's exponential and reciprocal: the bf16 silu within one unit in the last
    place of the exactly specified form's, hence act within two (and so against torch's eager graph),
    differing at all in well under 0.1 % of the elements; codes and scales are bit for bit the oracle's 1x128 quantization of the act it wrote;
    special inputs (zeros, 88.5, +-200, NaN, +-Inf) give what the exact form gives, -88.5 a zero."""
    import hpfp8
    import torch.nn.functional as F
    h = U.randn_bf16((512, 7168), 5, 2.0, 0.001, 30.0)
    h[0, :6] = torch.tensor([0.0, -0.0, 88.5, -88.5, -200.0, 200.0], dtype=torch.bfloat16)
    h[1, 0] = float("nan")
    h[2, 1] = float("inf")
    h[3, 2] = float("-inf")
    h[4, 3584 + 7] = float("inf")
    hg = h.to(gpu)
    q, si, act = hpfp8.swiglu_quantize_1x128(hg, kmajor=True, want_act=True, pow2=pow2, fast=True)
    qe, sie, acte = hpfp8.swiglu_quantize_1x128(hg, kmajor=True, want_act=True, pow2=pow2)
    a, e = act.view(torch.int16).int(), acte.view(torch.int16).int()
    nan_a, nan_e = torch.isnan(act), torch.isnan(acte)
    assert torch.equal(nan_a, nan_e) and int(nan_a.sum()) >= 2
    d = (a - e).abs()[~nan_a]
    # (the reciprocal instruction returns 0 where 1 + exp(-g) exceeds 2^126, g < -87.3, where the exact form
    # still gives |silu| ~ 1e-37: both are zero for every purpose, but far apart counted in bf16 steps)
    tiny = ((act.float().abs() < 1e-30) & (acte.float().abs() < 1e-30))[~nan_a]
    # one step in the bf16 rounding of silu (a near-tie decided the other way) can become two in the product
    assert bool(((d <= 2) | tiny).all())
    assert float(((d != 0) & ~tiny).float().mean()) < 1e-3 and float(((d > 1) & ~tiny).float().mean()) < 1e-4
    assert torch.equal(act[0, :3], acte[0, :3]) and torch.equal(act[0, 4:6], acte[0, 4:6]) and float(act[0, 3].abs()) < 1e-30
    ref = F.silu(hg[:, :3584]) * hg[:, 3584:]
    dr = (a - ref.view(torch.int16).int()).abs()[~nan_a]
    assert float((dr > 2).float().mean()) < 1e-5 and float((dr > 1).float().mean()) < 1e-4 and float((dr != 0).float().mean()) < 3e-3
    # the quantizer half stays exact: codes and scales of the act that was written
    with np.errstate(all="ignore"):
        rq, _, rsi = O.quantize_1x128(U.bits(act), pow2=pow2)
    assert np.array_equal(U.canon_nan_codes(U.codes(q)), U.canon_nan_codes(rq)) and U.same_f32_or_nan(U.f32(si), rsi)
    # without act, and with row-major scales: same codes
    q2, si2 = hpfp8.swiglu_quantize_1x128(hg, kmajor=False, pow2=pow2, fast=True)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and U.same_f32_or_nan(U.f32(si2), U.f32(si))


@pytest.mark.parametrize("fast", [False, True])
def test_swiglu_with_both_quantized_forms(gpu, fast):
    """One read of the gate/up output gives the 1x128 codes and the transposed 128x1 codes of the activation:
    bit for bit what the SwiGLU quantizer and the transposing quantizer of its bf16 activation give (and, in
    the exact form, what the oracle gives); a strided source gives the same."""
    import hpfp8
    h = U.randn_bf16((256, 1536), 6, 2.0, 0.001, 30.0)
    h[0, :6] = torch.tensor([0.0, -0.0, 88.5, -88.5, -200.0, 200.0], dtype=torch.bfloat16)
    hg = h.to(gpu)
    q, si, qt, sit = hpfp8.ops.swiglu_quantize_1x128_and_128x1_t(hg, fast=fast)
    q1, si1, act = hpfp8.swiglu_quantize_1x128(hg, kmajor=True, want_act=True, fast=fast)
    qt1, sit1 = hpfp8.quantize_128x1_t(act, kmajor=True)
    assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(si, si1)
    assert torch.equal(qt.view(torch.uint8), qt1.view(torch.uint8)) and torch.equal(sit, sit1)
    assert si.stride(0) == 1 and sit.stride(0) == 1
    if not fast:
        rq, _, rsi, ract = O.swiglu_quantize_1x128(U.bits(h))
        rqt, _, rsit = O.quantize_128x1_t(ract)
        assert np.array_equal(U.codes(q), rq) and eq_f32(si, rsi) and np.array_equal(U.codes(qt), rqt) and eq_f32(sit, rsit)
    wide = torch.zeros((256, 1536 + 64), dtype=torch.bfloat16, device=gpu)
    wide[:, :1536] = hg
    q2, si2, qt2, sit2 = hpfp8.ops.swiglu_quantize_1x128_and_128x1_t(wide[:, :1536], fast=fast)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(qt2.view(torch.uint8), qt.view(torch.uint8))
    assert torch.equal(si2, si) and torch.equal(sit2, sit)
    with pytest.raises(ValueError):
        hpfp8.ops.swiglu_quantize_1x128_and_128x1_t(hg[:100], fast=fast)


@pytest.mark.parametrize("rows", [1, 100, 128, 300, 384])
def test_transposed_quantizer_on_a_ragged_row_count(gpu, rows):
    """Whole groups quantized in place and the last, ragged, group from a zero-filled copy: the bits of the
    transposing quantizer on the zero-padded tensor."""
    import hpfp8
    x = U.randn_bf16((rows, 384), 41, 1.0, 0.01, 30.0).to(gpu)
    big = torch.zeros((640, 384), dtype=torch.bfloat16, device=gpu)
    big[7:7 + rows] = x                                      # (a row slice that starts at an odd row of its buffer)
    qt, sit = hpfp8.ops.quantize_128x1_t_rows(big[7:7 + rows])
    mp = -(-rows // 128) * 128
    xp = torch.zeros((mp, 384), dtype=torch.bfloat16, device=gpu)
    xp[:rows] = x
    wqt, wsit = hpfp8.quantize_128x1_t(xp, kmajor=True)
    assert qt.shape == (384, mp) and torch.equal(qt.view(torch.uint8), wqt.view(torch.uint8)) and torch.equal(sit, wsit)
    assert sit.stride(0) == 1


def test_dequantize_accumulate_into_fp32_main_grad(gpu):
    import hpfp8
    g = U.randn_bf16((300, 640), 71, 1e-3, 0.002, 100.0)
    q, si = hpfp8.quantize_1x128(g.to(gpu))
    main = torch.randn((300, 640), generator=torch.Generator().manual_seed(3)) * 1e-3
    got = hpfp8.dequantize_1x128_accumulate(q, si, main.to(gpu).clone(), grad_scale=0.25)
    want = O.dequantize_1x128_accumulate(U.codes(q), U.f32(si), main.numpy(), 0.25)
    assert np.array_equal(U.f32_bits(U.f32(got)), U.f32_bits(want))
    # twice the same gradient with grad_scale 1 == adding the bf16-free dequantized values twice
    again = hpfp8.dequantize_1x128_accumulate(q, si, got, grad_scale=1.0)
    want2 = O.dequantize_1x128_accumulate(U.codes(q), U.f32(si), want, 1.0)
    assert np.array_equal(U.f32_bits(U.f32(again)), U.f32_bits(want2))


@pytest.mark.parametrize("n", [5, 8, 3007, 2048 * 1024, 4 * 1024 * 1024, 4 * 1024 * 1024 + 8])
def test_per_tensor_one_pass_form_and_its_bounded_wait(gpu, n):
    """Per-tensor quantization on both sides of the size where one pass over x (the grid keeps it in registers and
    agrees on the maximum through the amax word) gives way to two passes: codes, both scales and the amax word equal
    the oracle's bit for bit -- also when every workgroup's wait for the others is cut to nothing from the host, so
    that each computes the maximum alone (the kernel's exit path for a grid that is not resident together)."""
    import hpfp8
    from hpfp8 import _lib
    x = (U.randn_bf16((n,), 100 + n % 7, 1.0, 0.0005, 30.0)).to(gpu)
    rq, rs, rsi = O.quantize_per_tensor(U.bits(x))
    ram = np.float32(np.abs(x.float().cpu().numpy()).max())
    lib = _lib.load()
    try:
        for limit in (1 << 22, 0):
            lib.hpfp8_debug_set_spin_limit(limit)
            for _ in range(2):
                q = torch.empty((n,), dtype=torch.float8_e4m3fn, device=gpu)
                am = torch.full((1,), float("nan"), dtype=torch.float32, device=gpu)      # (garbage in the word before the call)
                sc = torch.empty((2,), dtype=torch.float32, device=gpu)
                _lib.call("hpfp8_quantize_per_tensor_bf16", x.data_ptr(), n, q.data_ptr(), am.data_ptr(), sc.data_ptr(),
                          sc.data_ptr() + 4, torch.cuda.current_stream().cuda_stream)
                torch.cuda.synchronize()
                assert np.array_equal(U.codes(q), rq)
                assert U.f32_bits(U.f32(sc))[0] == U.f32_bits(rs) and U.f32_bits(U.f32(sc))[1] == U.f32_bits(rsi)
                assert U.f32_bits(U.f32(am))[0] == U.f32_bits(ram), "the amax word is not a clean fp32 maximum"
    finally:
        lib.hpfp8_debug_set_spin_limit(1 << 22)
    q2, s2, si2 = hpfp8.quantize_per_tensor(x)
    assert np.array_equal(U.codes(q2), rq) and U.f32_bits(U.f32(si2)) == U.f32_bits(rsi)


def test_per_tensor_single_launch_form_with_self_clearing_sync_words(gpu):
    """hpfp8_quantize_per_tensor_sync_bf16: one launch, the grid synchronising through 16 bytes of the caller's that
    are zero before the first call.  Calls of different sizes in a row on the same words give the oracle's codes,
    scales and amax each time and leave the words zero -- also with every workgroup's wait cut to nothing (each then
    computes the maximum alone and the words are still cleared); the call replays from a captured graph on changing
    data; sizes beyond the one-pass limit and a misaligned pointer are refused."""
    import hpfp8
    from hpfp8 import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    sync = torch.zeros(128, dtype=torch.int32, device=gpu)
    try:
        for limit in (1 << 22, 0):
            lib.hpfp8_debug_set_spin_limit(limit)
            for n in (2048 * 1024, 5, 3007, 4 * 1024 * 1024, 8, 300000):
                x = U.randn_bf16((n,), 200 + n % 11, 1.0 + n % 3, 0.0005, 30.0).to(gpu)
                rq, rs, rsi = O.quantize_per_tensor(U.bits(x))
                q = torch.empty((n,), dtype=torch.float8_e4m3fn, device=gpu)
                out = torch.full((3,), float("nan"), dtype=torch.float32, device=gpu)
                _lib.call("hpfp8_quantize_per_tensor_sync_bf16", x.data_ptr(), n, q.data_ptr(), out.data_ptr(), out.data_ptr() + 4,
                          out.data_ptr() + 8, sync.data_ptr(), st)
                torch.cuda.synchronize()
                assert np.array_equal(U.codes(q), rq), (limit, n)
                o = U.f32_bits(U.f32(out))
                assert o[0] == U.f32_bits(np.float32(np.abs(x.float().cpu().numpy()).max()))
                assert o[1] == U.f32_bits(rs) and o[2] == U.f32_bits(rsi)
                assert int(sync.abs().sum()) == 0, "the sync words were not left zero"
    finally:
        lib.hpfp8_debug_set_spin_limit(1 << 22)
    # the Python wrapper takes this form for small tensors (same bits as the two-launch form)
    x = U.randn_bf16((2048, 1024), 7, 1.0, 0.001, 20.0).to(gpu)
    q1, s1, si1 = hpfp8.quantize_per_tensor(x)
    rq, rs, rsi = O.quantize_per_tensor(U.bits(x))
    assert np.array_equal(U.codes(q1), rq) and U.f32_bits(U.f32(si1)) == U.f32_bits(rsi) and U.f32_bits(U.f32(s1)) == U.f32_bits(rs)
    # graph replay on changing data (no clearing between replays)
    xs = [U.randn_bf16((1024, 512), 300 + i, 1.0 + i).to(gpu) for i in range(4)]
    x_static = xs[0].clone()
    qg = torch.empty((1024, 512), dtype=torch.float8_e4m3fn, device=gpu)
    og = torch.zeros(3, dtype=torch.float32, device=gpu)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _lib.call("hpfp8_quantize_per_tensor_sync_bf16", x_static.data_ptr(), x_static.numel(), qg.data_ptr(), og.data_ptr(),
                  og.data_ptr() + 4, og.data_ptr() + 8, sync.data_ptr(), side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _lib.call("hpfp8_quantize_per_tensor_sync_bf16", x_static.data_ptr(), x_static.numel(), qg.data_ptr(), og.data_ptr(),
                  og.data_ptr() + 4, og.data_ptr() + 8, sync.data_ptr(), torch.cuda.current_stream().cuda_stream)
    for x in xs[1:] + xs[:2]:
        x_static.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        rq, rs, rsi = O.quantize_per_tensor(U.bits(x))
        assert np.array_equal(U.codes(qg), rq) and U.f32_bits(U.f32(og))[2] == U.f32_bits(rsi)
        assert int(sync.abs().sum()) == 0
    # limits
    big = torch.zeros(4 * 1024 * 1024 + 8, dtype=torch.bfloat16, device=gpu)
    qb = torch.empty(big.shape, dtype=torch.float8_e4m3fn, device=gpu)
    assert lib.hpfp8_quantize_per_tensor_sync_bf16(big.data_ptr(), big.numel(), qb.data_ptr(), None, None, og.data_ptr(), sync.data_ptr(), st) == -2
    assert lib.hpfp8_quantize_per_tensor_sync_bf16(big.data_ptr(), 1024, qb.data_ptr(), None, None, og.data_ptr(), sync.data_ptr() + 16, st) == -3
    assert lib.hpfp8_quantize_per_tensor_sync_bf16(big.data_ptr(), 1024, qb.data_ptr(), None, None, og.data_ptr(), None, st) == -1


def test_tensors_beyond_2_31_elements(gpu):
    """4.3 GB of bf16 (2.15e9 elements): element offsets no longer fit 32 bits.  Every quantizer gives, on
    row blocks at the start, across the 2^31-element mark and at the end, the bits it gives for those rows
    passed on their own; the last rows are also checked against the oracle."""
    import hpfp8
    rows, cols = 300032, 7168                        # 2344 x 128 rows
    g = torch.Generator(device=gpu).manual_seed(3)
    x = torch.empty((rows, cols), dtype=torch.bfloat16, device=gpu)
    for r in range(0, rows, 37504):                  # filled in pieces: no 8.6 GB fp32 temporary
        x[r:r + 37504] = torch.randn((37504, cols), generator=g, device=gpu).to(torch.bfloat16)
    assert x.numel() > (1 << 31)
    cross = ((1 << 31) // cols) // 128 * 128         # the 128-row block that contains element 2^31
    blocks = (0, cross, rows - 128)
    u8 = lambda t: t.view(torch.uint8)
    for kmajor in (False, True):
        q, s, si = hpfp8.quantize_1x128(x, want_scale=True, kmajor=kmajor)
        for r0 in blocks:
            pq, ps, psi = hpfp8.quantize_1x128(x[r0:r0 + 128], want_scale=True, kmajor=kmajor)
            assert torch.equal(u8(q[r0:r0 + 128]), u8(pq)) and torch.equal(si[r0:r0 + 128], psi) and torch.equal(s[r0:r0 + 128], ps)
    rq, rs, rsi = O.quantize_1x128(U.bits(x[rows - 128:]))
    assert np.array_equal(U.codes(q[rows - 128:]), rq) and eq_f32(si[rows - 128:], rsi)
    back = hpfp8.dequantize_1x128(q, si.contiguous())
    assert np.array_equal(U.bits(back[rows - 128:]), O.dequantize_1x128(rq, rsi))
    del q, s, si, back
    q, si, qt, s = hpfp8.quantize_128x128(x, with_transpose=True, want_scale=True)
    for r0 in blocks:
        pq, psi, pqt, ps = hpfp8.quantize_128x128(x[r0:r0 + 128], with_transpose=True, want_scale=True)
        assert torch.equal(u8(q[r0:r0 + 128]), u8(pq)) and torch.equal(si[r0 // 128], psi[0]) and torch.equal(s[r0 // 128], ps[0])
        assert torch.equal(u8(qt[:, r0:r0 + 128]), u8(pqt))
    del q, si, qt, s
    for kmajor in (False, True):
        q1, si1, qt, sit = hpfp8.quantize_1x128_and_128x1_t(x, kmajor=kmajor)
        for r0 in blocks:
            p1, psi1, pqt, psit = hpfp8.quantize_1x128_and_128x1_t(x[r0:r0 + 128], kmajor=kmajor)
            assert torch.equal(u8(q1[r0:r0 + 128]), u8(p1)) and torch.equal(si1[r0:r0 + 128], psi1)
            assert torch.equal(u8(qt[:, r0:r0 + 128]), u8(pqt)) and torch.equal(sit[:, r0 // 128], psit[:, 0])
        del q1, si1, qt, sit
    qt, sit = hpfp8.quantize_128x1_t(x, kmajor=True)
    rqt, _, rsit = O.quantize_128x1_t(U.bits(x[rows - 128:]))
    assert np.array_equal(U.codes(qt[:, rows - 128:]), rqt) and eq_f32(sit[:, -1], rsit[:, 0])
    am = hpfp8.amax(x)
    assert float(am) == float(x.view(torch.int16).bitwise_and(0x7FFF).max().view(torch.bfloat16).float())
    del qt, sit
    # the remaining entry points: per-tensor cast, 128x128 dequantize, byte transpose, SwiGLU forms
    q, s, si = hpfp8.quantize_per_tensor(x)
    pq, _, _ = hpfp8.quantize_per_tensor(x[rows - 128:], amax_in=am)
    assert torch.equal(u8(q[rows - 128:]), u8(pq)) and float(si) == float(np.float32(float(am)) / np.float32(448.0))
    del q
    q, si = hpfp8.quantize_128x128(x)
    back = hpfp8.dequantize_128x128(q, si)
    qt = hpfp8.transpose_codes(q)
    for r0 in blocks:
        pq, psi = hpfp8.quantize_128x128(x[r0:r0 + 128])
        assert torch.equal(back[r0:r0 + 128], hpfp8.dequantize_128x128(pq, psi))
        assert torch.equal(u8(qt[:, r0:r0 + 128]), u8(hpfp8.transpose_codes(pq)))
    del q, si, back, qt
    for fast in (False, True):
        q, si, act = hpfp8.swiglu_quantize_1x128(x, kmajor=True, want_act=True, fast=fast)
        for r0 in blocks:
            pq, psi, pact = hpfp8.swiglu_quantize_1x128(x[r0:r0 + 128], kmajor=True, want_act=True, fast=fast)
            assert torch.equal(u8(q[r0:r0 + 128]), u8(pq)) and torch.equal(si[r0:r0 + 128], psi) and torch.equal(act[r0:r0 + 128], pact)
        del q, si
    dh = hpfp8.ops.swiglu_backward(x, act)
    for r0 in blocks:
        assert torch.equal(dh[r0:r0 + 128], hpfp8.ops.swiglu_backward(x[r0:r0 + 128], act[r0:r0 + 128]))


def test_column_sum_bias_gradient_fused_and_standalone(gpu):
    """The bias gradient (fp32 column sums of grad_out in the oracle's stated order, rounded once to bf16): the
    standalone kernel on ragged and whole row counts, and the form fused into the dual quantizer, whose codes and
    scales must stay those of the plain dual quantizer."""
    import hpfp8
    from hpfp8 import ops
    for (m, k), seed in (((1, 128), 1), ((127, 256), 2), ((128, 128), 3), ((300, 384), 4), ((1024, 512), 5)):
        x = U.laplace_bf16((m, k), seed, 1e-3)
        part, total, tb = O.column_sum(U.bits(x))
        got32 = ops.column_sum(x.to(gpu), out_dtype=torch.float32)
        got16 = ops.column_sum(x.to(gpu))
        assert np.array_equal(U.f32_bits(got32.cpu().numpy()), U.f32_bits(total)), (m, k)
        assert np.array_equal(U.bits(got16), tb), (m, k)
    # a strided source (a column slice of a wider matrix)
    wide = U.randn_bf16((256, 512), 6).to(gpu)
    sl = wide[:, 128:384]
    assert torch.equal(ops.column_sum(sl), ops.column_sum(sl.contiguous()))
    # 2^24 and ones: the order of the additions is the stated one (see the oracle's pin of the same cases)
    col = torch.zeros((256, 128), dtype=torch.bfloat16)
    col[0, 0], col[4, 0], col[8, 0], col[12, 0] = 2.0 ** 24, 1.0, 1.0, 1.0
    assert float(ops.column_sum(col.to(gpu), out_dtype=torch.float32)[0]) == 2.0 ** 24 + 2
    for pow2 in (False, True):
        x = U.laplace_bf16((512, 384), 7, 1e-3).to(gpu)
        q, s, qt, st, db = ops.quantize_1x128_and_128x1_t(x, kmajor=True, pow2=pow2, column_sum=True)
        q0, s0, qt0, st0 = ops.quantize_1x128_and_128x1_t(x, kmajor=True, pow2=pow2)
        assert torch.equal(q.view(torch.uint8), q0.view(torch.uint8)) and torch.equal(qt.view(torch.uint8), qt0.view(torch.uint8))
        assert torch.equal(s, s0) and torch.equal(st, st0)
        assert np.array_equal(U.bits(db), O.column_sum(U.bits(x))[2]) and torch.equal(db, ops.column_sum(x))
    with pytest.raises(ValueError):
        ops.quantize_1x128_and_128x1_t(x, kmajor=False, column_sum=True)
    with pytest.raises(ValueError):
        ops.column_sum(torch.zeros((4, 100), dtype=torch.bfloat16, device=gpu))


def test_column_sum_at_full_size_against_float64(gpu):
    """cfg 2's grad_out shape: the fused bias gradient against torch's float64 column sum (within the fp32 bound of a
    4096-term sum) and, on a column block, against the oracle bit for bit."""
    from hpfp8 import ops
    go = (torch.randn((4096, 36864), device=gpu, generator=torch.Generator(device=gpu).manual_seed(9)) * 1e-3).to(torch.bfloat16)
    _, _, _, _, db = ops.quantize_1x128_and_128x1_t(go, kmajor=True, column_sum=True)
    ref = go.double().sum(dim=0)
    bound = 4096 * 2.0 ** -24 * go.double().abs().sum(dim=0) + ref.abs() * 2.0 ** -8      # fp32 sum + one bf16 rounding
    assert bool(((db.double() - ref).abs() <= bound).all())
    sl = go[:, 1280:1536].contiguous()
    assert np.array_equal(U.bits(db[1280:1536]), O.column_sum(U.bits(sl))[2])
