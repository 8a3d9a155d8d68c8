"""GPU parity of the MoE grouped backward through the C ABI: the device-side layout table, the grouped transposed
quantizer (bit for bit against the oracle), the grouped weight-gradient GEMM (against a per-expert loop of the
oracle's `gemm_rowwise_both` and a float64 reference), the input gradient on the stacked weight's transposed codes,
and the whole forward + backward replayed from a captured graph (nothing reads `offs` on the host)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import fp8_oracle as O
import _util as U

pytestmark = pytest.mark.gpu


def rel(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


CASES = [
    ([130, 130, 430, 500], 512),            # ragged counts, an empty expert, rows that belong to no expert
    ([0, 7, 7, 263], 263),                  # leading empty expert, a tiny one, odd total
    ([128, 100, 9999], 300),                # malformed table: read clamped
    ([0, 0, 0], 0),                         # no rows at all
    ([256], 256),
]


@pytest.mark.parametrize("offs,total", CASES)
def test_layout_table_matches_the_oracle(gpu, offs, total):
    from hpfp8 import ops
    e = len(offs)
    layout = ops.grouped_layout(torch.tensor(offs, dtype=torch.int32, device=gpu), total).cpu().numpy()
    table, used = O.grouped_layout(offs, total)
    assert layout[:4 * e].reshape(e, 4).tolist() == [list(t) for t in table]
    assert int(layout[5 * e]) == used
    order = layout[4 * e:5 * e].tolist()
    nbs = [t[3] for t in table]
    assert sorted(order) == list(range(e))
    assert order == sorted(range(e), key=lambda i: (-nbs[i], i))           # longest first, ties by index
    owner = layout[5 * e + 1:].tolist()
    want = []
    for i, t in enumerate(table):
        want += [i] * t[3]
    assert owner == want + [-1] * (total // 128 + e - used)


@pytest.mark.parametrize("offs,total", CASES[:3])
@pytest.mark.parametrize("dual", [False, True])
def test_grouped_transposed_quantizer_bit_exact(gpu, offs, total, dual):
    from hpfp8 import ops
    e, k = len(offs), 384
    x = U.randn_bf16((total, k), 91, 1.0, 0.002, 40.0)
    toffs = torch.tensor(offs, dtype=torch.int32, device=gpu)
    layout = ops.grouped_layout(toffs, total)
    out = ops.quantize_128x1_t_grouped(x.to(gpu), layout, e, with_1x128=dual)
    qt, sit = out[-2:]
    rqt, _, rsit = O.quantize_128x1_t_grouped(U.bits(x), offs)
    table, used = O.grouped_layout(offs, total)
    assert qt.shape == rqt.shape and sit.shape == rsit.shape and sit.stride(0) == 1
    assert np.array_equal(U.codes(qt)[:, :used * 128], rqt[:, :used * 128])
    assert np.array_equal(U.f32_bits(U.f32(sit))[:, :used], U.f32_bits(rsit)[:, :used])
    if dual:
        q, si = out[:2]
        rq, _, rsi = O.quantize_1x128(U.bits(x))
        last = table[-1][0] + table[-1][1]                               # rows beyond belong to no expert
        assert np.array_equal(U.codes(q)[:last], rq[:last])
        assert np.array_equal(U.f32_bits(U.f32(si))[:last], U.f32_bits(rsi)[:last])


@pytest.mark.parametrize("offs,total,n,k", [([130, 130, 430, 500], 512, 256, 384), ([0, 7, 7, 263], 263, 128, 640),
                                            ([300, 300, 300, 1324, 1324, 2000], 2048, 512, 768), ([0, 0, 0], 0, 128, 128)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_grouped_wgrad_against_the_oracle_and_float64(gpu, offs, total, n, k, out_dtype):
    """dW[e] = go_e^T . x_e for every expert from one launch: against the oracle's per-expert `gemm_rowwise_both`
    (fp32 output within the matrix cores' summation error, bf16 output within one rounding), exact zeros for
    experts without rows, and independent of what the unused padded blocks hold."""
    from hpfp8 import ops
    e = len(offs)
    go = U.randn_bf16((total, n), 93, 1e-2, 0.001, 30.0)
    x = U.randn_bf16((total, k), 94, 1.0)
    toffs = torch.tensor(offs, dtype=torch.int32, device=gpu)
    layout = ops.grouped_layout(toffs, total)
    got, sgot = ops.quantize_128x1_t_grouped(go.to(gpu), layout, e)
    xt, sxt = ops.quantize_128x1_t_grouped(x.to(gpu), layout, e)
    table, used = O.grouped_layout(offs, total)
    # poison what no expert owns: the GEMM must not read it
    got.view(torch.uint8)[:, used * 128:] = 0x7F
    xt.view(torch.uint8)[:, used * 128:] = 0x7F
    sgot[:, used:] = float("nan")
    sxt[:, used:] = float("nan")
    dw = ops.gemm_grouped_wgrad(got, sgot, xt, sxt, layout, e, total, out_dtype=out_dtype)
    assert dw.shape == (e, n, k) and dw.dtype == out_dtype
    want, want_bits = O.gemm_grouped_wgrad(U.codes(got), U.f32(sgot), U.codes(xt), U.f32(sxt), offs, total)
    for i, (start, rows, b0, nb) in enumerate(table):
        if rows == 0:
            assert not bool(dw[i].any()), f"expert {i} has no rows"
            continue
        ref = torch.from_numpy(want[i])
        if out_dtype == torch.float32:
            assert rel(dw[i].cpu(), ref) < 1e-4, f"expert {i}"
        else:
            d = (dw[i].cpu().view(torch.int16).int() - torch.from_numpy(want_bits[i].view(np.int16)).int()).abs()
            small = (dw[i].cpu().float() - ref).abs() <= 1e-4 * float(ref.abs().max())
            assert bool(((d <= 1) | small).all()), f"expert {i}"
        exact = go[start:start + rows].double().t() @ x[start:start + rows].double()
        assert rel(dw[i].cpu(), exact) < 0.06


def test_grouped_input_gradient_on_stacked_transposed_codes(gpu):
    """dx_e = go_e . W_e through the strided grouped entry point equals, expert by expert, the dense dgrad GEMM on
    that expert's rows bit for bit; rows of no expert come back as zeros."""
    import hpfp8
    from hpfp8 import ops
    offs, total, n, k = [130, 130, 430, 500], 512, 256, 384
    e = len(offs)
    w = U.randn_bf16((e, n, k), 95, 0.05).to(gpu)
    go = U.randn_bf16((total, n), 96, 1e-2).to(gpu)
    f8 = hpfp8.quantize_grouped_weight(w)
    assert f8.codes_t.shape == (k, e * n)
    goq, sgo = ops.quantize_1x128(go, kmajor=True)
    toffs = torch.tensor(offs, dtype=torch.int32, device=gpu)
    dx = ops.gemm_grouped_blockwise_t(goq, sgo, f8.codes_t, f8.scale_inv, toffs)
    assert dx.shape == (total, k) and not bool(dx[500:].any())
    start = 0
    for i, end in enumerate(offs):
        if end > start:
            wq_i, sw_i, wqt_i = ops.quantize_128x128(w[i], with_transpose=True)
            dense = ops.gemm_blockwise(goq[start:end], sgo[start:end], wqt_i, sw_i.t())
            assert torch.equal(dx[start:end], dense), f"expert {i}"
        start = max(start, end)


def test_grouped_linear_forward_backward_replays_from_a_graph(gpu):
    """Forward and backward of the grouped linear recorded once and replayed with other data AND other rows per
    expert (offs is device data: nothing on the host depends on it): every replay equals the eager call."""
    import hpfp8
    e, n, k, total = 4, 256, 384, 640
    w = U.randn_bf16((e, n, k), 97, 0.05).to(gpu).requires_grad_(True)
    x_s = torch.zeros((total, k), dtype=torch.bfloat16, device=gpu).requires_grad_(True)
    go_s = torch.zeros((total, n), dtype=torch.bfloat16, device=gpu)
    offs_s = torch.zeros((e,), dtype=torch.int32, device=gpu)

    def step():
        x_s.grad = None
        w.grad = None
        y = hpfp8.fp8_grouped_linear(x_s, w, offs_s)
        y.backward(go_s)
        return y.detach(), x_s.grad, w.grad

    datas = []
    for seed, counts in ((1, [130, 0, 300, 70]), (2, [0, 640, 0, 0]), (3, [1, 129, 255, 200])):
        datas.append((U.randn_bf16((total, k), 100 + seed).to(gpu), U.randn_bf16((total, n), 200 + seed, 1e-2).to(gpu),
                      torch.tensor(counts).cumsum(0).to(torch.int32).to(gpu)))
    with torch.no_grad():
        x_s.copy_(datas[0][0]); go_s.copy_(datas[0][1]); offs_s.copy_(datas[0][2])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_g, dx_g, dw_g = step()
    for xd, god, offd in datas[1:] + datas[:1]:
        with torch.no_grad():
            x_s.copy_(xd); go_s.copy_(god); offs_s.copy_(offd)
        graph.replay()
        torch.cuda.synchronize()
        got = (y_g.clone(), dx_g.clone(), dw_g.clone())
        xe = xd.clone().requires_grad_(True)
        we = w.detach().clone().requires_grad_(True)
        ye = hpfp8.fp8_grouped_linear(xe, we, offd)
        ye.backward(god)
        last = int(offd[-1])
        assert torch.equal(got[0][:last], ye.detach()[:last])
        assert torch.equal(got[1], xe.grad) and torch.equal(got[2], we.grad)


def test_cfg4_moe_layer_backward_full_size(gpu):
    """Config 4 at its real size (32 experts, 131072 routed rows with Zipf popularity and two empty experts, weights
    [32, 4096, 7168]): the grouped transposed quantizer against the C oracle on two experts' blocks, the weight
    gradient of every expert against a float64 reference on a block of its output, exact zeros for the empty experts,
    and the input gradient's per-expert first and last rows against float64."""
    import hpfp8
    from hpfp8 import ops
    from oracle import c_oracle as C
    from test_gpu_gemm import _zipf_counts, dequant_f64
    experts, total, N, K = 32, 131072, 4096, 7168
    counts = _zipf_counts(total, experts, 7)
    offs_l = counts.cumsum(0).tolist()
    offs = counts.cumsum(0).to(torch.int32).to(gpu)
    g = torch.Generator(device=gpu).manual_seed(11)
    x = torch.empty((total, K), dtype=torch.bfloat16, device=gpu)
    go = torch.empty((total, N), dtype=torch.bfloat16, device=gpu)
    for r0 in range(0, total, 16384):
        x[r0:r0 + 16384] = torch.randn((16384, K), generator=g, device=gpu).to(torch.bfloat16)
        go[r0:r0 + 16384] = (torch.randn((16384, N), generator=g, device=gpu) * 1e-3).to(torch.bfloat16)
    layout = ops.grouped_layout(offs, total)
    goq, sgo, got, sgot = ops.quantize_128x1_t_grouped(go, layout, experts, with_1x128=True)
    xt, sxt = ops.quantize_128x1_t_grouped(x, layout, experts)
    table, used = O.grouped_layout(offs_l, total)
    # the transposed quantizer on two experts (a large one and the smallest non-empty one) against the C restatement
    nonempty = [i for i, t in enumerate(table) if t[1] > 0]
    small = min(nonempty, key=lambda i: table[i][1])
    for i in (nonempty[0], small):
        start, rows, b0, nb = table[i]
        nb_chk = min(nb, 8)                                   # (the first 1024 tokens of a large expert, and the ragged end)
        for blk0 in {0, nb - nb_chk}:
            r0 = start + blk0 * 128
            r1 = min(r0 + nb_chk * 128, start + rows)
            padded = torch.zeros((nb_chk * 128, K), dtype=torch.bfloat16)
            padded[:r1 - r0] = x[r0:r1].cpu()
            cq, _, csi = C.quantize_128x1_t(U.bits(padded))
            cols = slice((b0 + blk0) * 128, (b0 + blk0 + nb_chk) * 128)
            assert np.array_equal(U.codes(xt[:, cols]), cq), f"expert {i}"
            assert np.array_equal(U.f32_bits(U.f32(sxt[:, b0 + blk0:b0 + blk0 + nb_chk])), U.f32_bits(csi)), f"expert {i}"
    dw = ops.gemm_grouped_wgrad(got, sgot, xt, sxt, layout, experts, total)
    assert dw.shape == (experts, N, K)
    for i, (start, rows, b0, nb) in enumerate(table):
        if rows == 0:
            assert not bool(dw[i].any()), f"expert {i} has no rows"
            continue
        cols = slice(b0 * 128, (b0 + nb) * 128)
        r0, c0 = (i * 256) % (N - 256), (i * 512) % (K - 512)           # a different 256 x 512 block per expert
        ref = (dequant_f64(got[r0:r0 + 256, cols], sgot[r0:r0 + 256, b0:b0 + nb], gpu) @
               dequant_f64(xt[c0:c0 + 512, cols], sxt[c0:c0 + 512, b0:b0 + nb], gpu).t())
        assert rel(dw[i, r0:r0 + 256, c0:c0 + 512], ref) < 3e-3, f"expert {i}"
        exact = go[start:start + rows, r0:r0 + 256].double().t() @ x[start:start + rows, c0:c0 + 512].double()
        assert rel(dw[i, r0:r0 + 256, c0:c0 + 512], exact) < 0.06, f"expert {i}"
    del dw
    w8 = []
    gw = torch.Generator(device=gpu).manual_seed(12)
    wq = torch.empty((experts * N, K), dtype=torch.float8_e4m3fn, device=gpu)
    swi = torch.empty((experts, N // 128, K // 128), dtype=torch.float32, device=gpu)
    for e in range(experts):
        wc = (torch.randn((N, K), generator=gw, device=gpu) * 0.006).to(torch.bfloat16)
        wq[e * N:(e + 1) * N], swi[e] = ops.quantize_128x128(wc)
    wqt = ops.transpose_codes(wq)
    dx = ops.gemm_grouped_blockwise_t(goq, sgo, wqt, swi, offs)
    for i, (start, rows, b0, nb) in enumerate(table):
        if rows == 0:
            continue
        wd = dequant_f64(wqt[:, i * N:(i + 1) * N], swi[i].t().repeat_interleave(128, dim=0), gpu)      # [K, N]
        last0 = start + (rows - 1) // 256 * 256
        for r0, r1 in {(start, min(start + 256, start + rows)), (last0, start + rows)}:
            ref = dequant_f64(goq[r0:r1], sgo[r0:r1], gpu) @ wd.t()
            assert rel(dx[r0:r1], ref) < 3e-3, f"expert {i} rows {r0}..{r1}"
