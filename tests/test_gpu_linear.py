"""fp8_linear / Fp8Linear against torch.nn.functional.linear: same calling convention, same shapes,
forward and gradients within FP8 quantization error; and against the oracle pipeline on small sizes."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import fp8_oracle as O
import _util as U

pytestmark = pytest.mark.gpu


def rel(a, b):
    a = a.detach().double().cpu().numpy()
    b = b.detach().double().cpu().numpy()
    return np.linalg.norm(a - b) / np.linalg.norm(b)


@pytest.mark.parametrize("recipe", ["blockwise", "per_tensor"])
def test_forward_backward_vs_f_linear(gpu, recipe):
    import hpfp8
    x = U.randn_bf16((4, 128, 512), 1).to(gpu).requires_grad_(True)
    w = U.randn_bf16((384, 512), 2, 0.02).to(gpu).requires_grad_(True)
    b = U.randn_bf16((384,), 3, 0.1).to(gpu).requires_grad_(True)
    go = U.randn_bf16((4, 128, 384), 4, 1e-3).to(gpu)
    y = hpfp8.fp8_linear(x, w, b, recipe=recipe)
    assert y.shape == (4, 128, 384) and y.dtype == torch.bfloat16
    y.backward(go)
    gx, gw, gb = x.grad.clone(), w.grad.clone(), b.grad.clone()
    x.grad = w.grad = b.grad = None
    yr = F.linear(x.float(), w.float(), b.float())
    yr.backward(go.float())
    tol = 0.06 if recipe == "blockwise" else 0.08
    assert rel(y, yr) < tol and rel(gx, x.grad) < tol and rel(gw, w.grad) < tol
    assert rel(gb, b.grad) < 1e-2
    assert gx.shape == x.shape and gw.shape == w.shape and gb.shape == b.shape


def test_forward_equals_oracle_pipeline(gpu):
    import hpfp8
    x = U.randn_bf16((256, 384), 11, 1.0, 0.001, 50.0)
    w = U.randn_bf16((256, 384), 12, 0.02)
    bias = U.randn_bf16((256,), 13, 0.1)
    y = hpfp8.fp8_linear(x.to(gpu), w.to(gpu), bias.to(gpu))
    xq, _, sxi = O.quantize_1x128(U.bits(x))
    wq, _, swi = O.quantize_128x128(U.bits(w))
    want, want_bits = O.gemm_blockwise(xq, sxi, wq, swi, bias.float().numpy())
    got = y.float().cpu().numpy()
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 3e-3
    diff = np.abs(U.bits(y).astype(np.int32) - want_bits.astype(np.int32))
    assert (diff != 0).mean() < 3e-2


def test_module_is_a_drop_in_for_nn_linear(gpu):
    import hpfp8
    torch.manual_seed(0)
    lin = torch.nn.Linear(256, 128, bias=True).to(gpu).to(torch.bfloat16)
    mod = hpfp8.Fp8Linear(256, 128, bias=True, device=gpu)
    mod.load_state_dict(lin.state_dict())
    x = U.randn_bf16((128, 256), 21).to(gpu)
    assert rel(mod(x), lin(x)) < 0.06
    opt = torch.optim.SGD(mod.parameters(), lr=0.1)
    loss0 = None
    for _ in range(5):
        opt.zero_grad()
        loss = (mod(x).float() ** 2).mean()
        loss.backward()
        opt.step()
        loss0 = loss0 if loss0 is not None else float(loss)
    assert float(loss) < loss0
    nob = hpfp8.Fp8Linear(256, 128, bias=False, device=gpu)
    assert nob(x).shape == (128, 128)


def test_grouped_linear_forward(gpu):
    import hpfp8
    counts = torch.tensor([130, 0, 300, 82])
    offs = counts.cumsum(0).to(torch.int32).to(gpu)
    x = U.randn_bf16((512, 256), 31).to(gpu)
    w = U.randn_bf16((4, 128, 256), 32, 0.02).to(gpu)
    y = hpfp8.fp8_grouped_linear(x, w, offs)
    start = 0
    for e in range(4):
        c = int(counts[e])
        if c:
            ref = F.linear(x[start:start + c].float(), w[e].float())
            assert rel(y[start:start + c], ref) < 0.06
        start += c
