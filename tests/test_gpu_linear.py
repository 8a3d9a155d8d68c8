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


@pytest.mark.parametrize("recipe", ["blockwise", "per_tensor", "blockwise_pow2"])
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
    # the bias gradient is the oracle's fp32 column sum of grad_out, bit for bit, whichever kernel produced it
    assert np.array_equal(U.bits(gb), O.column_sum(U.bits(go.reshape(-1, 384)))[2])


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
        loss0 = loss0 if loss0 is not None else float(loss.detach())
    assert float(loss.detach()) < loss0
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


def test_prequantized_weight_and_module_cache(gpu):
    """fp8_linear with a weight quantized beforehand gives bit-identical outputs and gradients to the
    call that quantizes it itself; the module's cache is refreshed when the parameter is written."""
    import hpfp8
    x = U.randn_bf16((256, 384), 31).to(gpu).requires_grad_(True)
    w = U.randn_bf16((256, 384), 32, 0.02).to(gpu).requires_grad_(True)
    go = U.randn_bf16((256, 256), 33, 1e-3).to(gpu)
    y0 = hpfp8.fp8_linear(x, w)
    y0.backward(go)
    gx0, gw0 = x.grad.clone(), w.grad.clone()
    x.grad = w.grad = None
    for with_t in (True, False):              # without transposed codes they are made from the codes
        wf = hpfp8.quantize_weight(w.detach(), with_transpose=with_t)
        y1 = hpfp8.fp8_linear(x, w, weight_fp8=wf)
        y1.backward(go)
        assert torch.equal(y1, y0) and torch.equal(x.grad, gx0) and torch.equal(w.grad, gw0)
        x.grad = w.grad = None
    mod = hpfp8.Fp8Linear(384, 256, bias=False, cache_weight=True, device=gpu)
    with torch.no_grad():
        mod.weight.copy_(w)
    a = mod(x.detach())
    key = mod._fp8_key
    assert torch.equal(a, y0.detach()) and torch.equal(mod(x.detach()), a) and mod._fp8_key == key
    with torch.no_grad():
        mod.weight.mul_(2.0)                  # an in-place update, as an optimizer step is
    b = mod(x.detach())
    assert mod._fp8_key != key and torch.equal(b, hpfp8.fp8_linear(x.detach(), mod.weight.detach()))
    # the per-tensor recipe: same bits with the weight quantized beforehand, cached by the module, refused under
    # the other recipe
    y0 = hpfp8.fp8_linear(x, w, recipe="per_tensor")
    y0.backward(go)
    gx0, gw0 = x.grad.clone(), w.grad.clone()
    x.grad = w.grad = None
    wf = hpfp8.quantize_weight(w.detach(), per_tensor=True)
    y1 = hpfp8.fp8_linear(x, w, recipe="per_tensor", weight_fp8=wf)
    y1.backward(go)
    assert torch.equal(y1, y0) and torch.equal(x.grad, gx0) and torch.equal(w.grad, gw0)
    with pytest.raises(ValueError):
        hpfp8.fp8_linear(x, w, weight_fp8=wf)
    with pytest.raises(ValueError):
        hpfp8.fp8_linear(x, w, recipe="per_tensor", weight_fp8=hpfp8.quantize_weight(w.detach()))
    mod = hpfp8.Fp8Linear(384, 256, bias=False, recipe="per_tensor", cache_weight=True, device=gpu)
    with torch.no_grad():
        mod.weight.copy_(w)
    a = mod(x.detach())
    first = mod._fp8
    assert torch.equal(a, y0.detach()) and torch.equal(mod(x.detach()), a) and mod._fp8 is first


def test_weight_gradient_onto_fp32_main_grad(gpu):
    """apply_grad_on_fp32_main_grad: the first backward creates weight.main_grad as the fp32 weight
    gradient, later ones are added onto it by the wgrad GEMM, weight.grad stays empty and the other
    gradients are those of the ordinary call."""
    import hpfp8
    x = U.randn_bf16((512, 384), 51).to(gpu).requires_grad_(True)
    w = U.randn_bf16((256, 384), 52, 0.02).to(gpu).requires_grad_(True)
    go1 = U.randn_bf16((512, 256), 53, 1e-3).to(gpu)
    go2 = U.randn_bf16((512, 256), 54, 2e-3).to(gpu)
    grads = []
    for go in (go1, go2):
        hpfp8.fp8_linear(x, w).backward(go)
        grads.append((x.grad.clone(), w.grad.float().clone()))
        x.grad = w.grad = None
    hpfp8.fp8_linear(x, w, apply_grad_on_fp32_main_grad=True).backward(go1)
    assert w.grad is None and w.main_grad.dtype == torch.float32 and torch.equal(x.grad, grads[0][0])
    first = w.main_grad.clone()
    assert torch.equal(first.to(torch.bfloat16).float(), grads[0][1])      # the same sums before the bf16 rounding
    x.grad = None
    hpfp8.fp8_linear(x, w, apply_grad_on_fp32_main_grad=True).backward(go2)
    assert w.grad is None and torch.equal(x.grad, grads[1][0])
    want = first.double() + grads[1][1].double()
    assert rel(w.main_grad, want) < 3e-3                                   # (grads[1] went through bf16)
    second_alone = w.main_grad.double() - first.double()
    assert rel(second_alone, grads[1][1]) < 5e-3
    mod = hpfp8.Fp8Linear(384, 256, bias=True, apply_grad_on_fp32_main_grad=True, device=gpu)
    mod(x.detach()).backward(go1)
    mod(x.detach()).backward(go1)
    assert mod.weight.grad is None and mod.bias.grad is not None
    ref_mod = hpfp8.Fp8Linear(384, 256, bias=True, device=gpu)
    ref_mod.load_state_dict(mod.state_dict())
    ref_mod(x.detach()).backward(go1)
    assert rel(mod.weight.main_grad, 2 * ref_mod.weight.grad.double()) < 3e-3
    with pytest.raises(ValueError):
        hpfp8.fp8_linear(x, w, recipe="per_tensor", apply_grad_on_fp32_main_grad=True)
    # the power-of-two recipe accumulates the same way
    w.main_grad = None
    hpfp8.fp8_linear(x, w, recipe="blockwise_pow2", apply_grad_on_fp32_main_grad=True).backward(go1)
    once = w.main_grad.clone()
    hpfp8.fp8_linear(x, w, recipe="blockwise_pow2", apply_grad_on_fp32_main_grad=True).backward(go1)
    assert w.grad is None and rel(w.main_grad, 2 * once.double()) < 1e-6 and rel(once, grads[0][1]) < 0.1


@pytest.mark.parametrize("recipe", ["blockwise", "per_tensor", "blockwise_pow2"])
def test_forward_replays_from_a_captured_graph(gpu, recipe):
    """Every entry point only enqueues kernels on the stream it is given (no allocation, no
    synchronisation, no memset), so a forward pass can be captured into a graph; each replay, with
    eager work and synchronisations in between, must give the eager result for the input of the moment."""
    import hpfp8
    w = U.randn_bf16((384, 512), 71, 0.02).to(gpu)
    b = U.randn_bf16((384,), 72, 0.1).to(gpu)
    xs = [U.randn_bf16((256, 512), 73 + i, 1.0 + i).to(gpu) for i in range(4)]
    x_static = xs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        for _ in range(3):
            hpfp8.fp8_linear(x_static, w, b, recipe=recipe)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph), torch.no_grad():
        y_static = hpfp8.fp8_linear(x_static, w, b, recipe=recipe)
    for x in xs[1:] + xs[:2]:
        x_static.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        with torch.no_grad():
            want = hpfp8.fp8_linear(x, w, b, recipe=recipe)
        assert torch.equal(y_static, want)


def test_fp8_all_gather_hooks_rebuild_the_full_weight(gpu):
    """Per-shard quantization + concatenation (what an all-gather of the hook outputs produces) equals
    quantizing the whole weight, transposed codes included; transpose_codes is a byte transpose."""
    import hpfp8
    w = U.randn_bf16((512, 384), 41, 0.02).to(gpu)
    shards = w.chunk(4, dim=0)                # FSDP shards dim 0; 128 rows each
    outs, metas = zip(*(hpfp8.fsdp.fsdp_pre_all_gather(s) for s in shards))
    assert outs[0][0].dtype == torch.uint8 and outs[0][0].shape == (128, 384)
    gathered = (torch.cat([o[0].reshape(-1) for o in outs]), torch.cat([o[1].reshape(-1) for o in outs]))
    wf = hpfp8.fsdp.fsdp_post_all_gather(gathered, metas[0])
    ref = hpfp8.quantize_weight(w, with_transpose=True)
    assert torch.equal(wf.codes.view(torch.uint8), ref.codes.view(torch.uint8))
    assert torch.equal(wf.scale_inv, ref.scale_inv)
    assert torch.equal(wf.codes_t.view(torch.uint8), ref.codes_t.view(torch.uint8))
    assert np.array_equal(U.codes(wf.codes_t), U.codes(wf.codes).T)
    x = U.randn_bf16((128, 384), 42).to(gpu)
    assert torch.equal(hpfp8.fp8_linear(x, w, weight_fp8=wf), hpfp8.fp8_linear(x, w))


def test_fsdp_extension_methods_on_the_sharded_tensor(gpu):
    """The tensor type that carries the all-gather extension as methods: detected the way the reference detects it
    (`hasattr(inner_tensor, ...)`, hyper_parallel/platform/torch/fully_shard/param.py:299-310), an ordinary bf16
    parameter otherwise, and its two hooks -- called as methods with the protocol's argument lists -- rebuild the
    whole weight's FP8 form from the per-shard pieces without a second quantization."""
    import hpfp8
    from hpfp8.fsdp import Fp8ShardedWeight, Fp8GatheredWeight
    w = U.randn_bf16((512, 384), 43, 0.02).to(gpu)
    shards = [torch.nn.Parameter(Fp8ShardedWeight(s.contiguous())) for s in w.chunk(4, dim=0)]
    inner = shards[0]
    assert hasattr(inner, "fsdp_pre_all_gather") and hasattr(inner, "fsdp_post_all_gather")
    assert isinstance(inner, torch.nn.Parameter) and inner.dtype == torch.bfloat16 and inner.requires_grad
    assert type(inner * 2) is torch.Tensor                      # arithmetic sees a plain tensor
    with pytest.raises(ValueError):
        Fp8ShardedWeight(w[:100])
    outs, metas = zip(*(s.fsdp_pre_all_gather(None, s.shape, s.stride(), None, None) for s in shards))
    assert outs[0][0].dtype == torch.uint8 and outs[0][1].dtype == torch.float32
    bufs = (torch.cat([o[0].reshape(-1) for o in outs]), torch.cat([o[1].reshape(-1) for o in outs]))   # the all-gather
    unsharded, inner_tensors = inner.fsdp_post_all_gather(bufs, metas[0], torch.bfloat16)
    assert isinstance(unsharded, Fp8GatheredWeight) and unsharded.shape == (512, 384)
    assert unsharded.data_ptr() == bufs[0].data_ptr() and inner_tensors[0] is bufs[0]      # a view, no copy
    ref = hpfp8.quantize_weight(w, with_transpose=True)
    wf = unsharded.as_fp8_weight()
    assert torch.equal(wf.codes.view(torch.uint8), ref.codes.view(torch.uint8)) and torch.equal(wf.scale_inv, ref.scale_inv)
    assert torch.equal(wf.codes_t.view(torch.uint8), ref.codes_t.view(torch.uint8))
    x = U.randn_bf16((128, 384), 44).to(gpu).requires_grad_(True)
    wp = w.clone().requires_grad_(True)
    y = hpfp8.fp8_linear(x, wp, weight_fp8=wf)
    y.backward(U.randn_bf16((128, 512), 45, 1e-3).to(gpu))
    assert torch.equal(y, hpfp8.fp8_linear(x.detach(), w)) and x.grad is not None and wp.grad is not None
    # a later all-gather refills the same buffers; with out= nothing is rebuilt but what was derived is dropped
    w2 = (w.float() * 1.5).to(torch.bfloat16)
    outs2 = [Fp8ShardedWeight(s.contiguous()).fsdp_pre_all_gather()[0] for s in w2.chunk(4, dim=0)]
    bufs[0].copy_(torch.cat([o[0].reshape(-1) for o in outs2]))
    bufs[1].copy_(torch.cat([o[1].reshape(-1) for o in outs2]))
    assert inner.fsdp_post_all_gather(bufs, metas[0], torch.bfloat16, out=unsharded) is None
    ref2 = hpfp8.quantize_weight(w2, with_transpose=True)
    wf2 = unsharded.as_fp8_weight()
    assert torch.equal(wf2.codes.view(torch.uint8), ref2.codes.view(torch.uint8))
    assert torch.equal(wf2.codes_t.view(torch.uint8), ref2.codes_t.view(torch.uint8)) and torch.equal(wf2.scale_inv, ref2.scale_inv)


def test_weight_cache_contract_and_inference_mode(gpu, monkeypatch):
    """Writes the version counter never sees (`.data`) leave the cache stale until `invalidate_fp8_cache()` (or the
    optimizer hook) drops it; `load_state_dict` drops it by itself.  Under `torch.no_grad()` a Parameter's
    `requires_grad` does not make forward prepare anything for a backward."""
    import hpfp8
    from hpfp8 import ops
    plain = hpfp8.Fp8Linear(384, 256, bias=False, device=gpu)   # the default: no cache, so no write can go unseen
    x = U.randn_bf16((128, 384), 51).to(gpu)
    a = plain(x).detach().clone()
    plain.weight.data.mul_(2.0)
    assert plain._fp8 is None and torch.equal(plain(x).detach(), hpfp8.fp8_linear(x, plain.weight.detach()))
    assert not torch.equal(plain(x).detach(), a)
    mod = hpfp8.Fp8Linear(384, 256, bias=False, cache_weight=True, device=gpu)
    a = mod(x).detach().clone()
    mod.weight.data.mul_(2.0)                                   # _version does not move
    stale = mod(x).detach()
    assert torch.equal(stale, a)
    mod.invalidate_fp8_cache()
    b = mod(x).detach()
    assert not torch.equal(b, a) and torch.equal(b, hpfp8.fp8_linear(x, mod.weight.detach()))
    opt = torch.optim.SGD(mod.parameters(), lr=0.5)
    handle = hpfp8.attach_optimizer(opt, mod)
    mod(x).float().square().mean().backward()
    cached = mod._fp8
    opt.step()
    assert mod._fp8 is None and cached is not None              # the step hook dropped it
    handle.remove()
    c = mod(x).detach().clone()
    sd = {k: v.clone() * 0.5 for k, v in mod.state_dict().items()}
    mod.load_state_dict(sd)
    assert mod._fp8 is None
    assert not torch.equal(mod(x).detach(), c)
    mlp = hpfp8.Fp8SwiGLUMLP(256, 384, cache_weight=True, device=gpu)
    y0 = mlp(U.randn_bf16((128, 256), 52).to(gpu)).detach().clone()
    mlp.down_proj.weight.data.mul_(0.5)
    hpfp8.invalidate_fp8_caches(mlp)
    assert not torch.equal(mlp(U.randn_bf16((128, 256), 52).to(gpu)).detach(), y0)
    # inference: no dual quantization of x, no transposed weight codes
    calls = []
    real_dual, real_w = ops.quantize_1x128_and_128x1_t, ops.quantize_128x128
    monkeypatch.setattr(ops, "quantize_1x128_and_128x1_t", lambda *a_, **k: calls.append("dual") or real_dual(*a_, **k))
    monkeypatch.setattr(ops, "quantize_128x128", lambda *a_, **k: calls.append(("w", k.get("with_transpose", False))) or real_w(*a_, **k))
    w = torch.nn.Parameter(U.randn_bf16((256, 384), 53, 0.02).to(gpu))
    xr = x.clone().requires_grad_(True)
    with torch.no_grad():
        y_inf = hpfp8.fp8_linear(xr, w)
    assert calls == [("w", False)] and not y_inf.requires_grad
    calls.clear()
    y_tr = hpfp8.fp8_linear(xr, w)
    assert calls == ["dual", ("w", True)] and torch.equal(y_tr.detach(), y_inf)


def test_fp8_checkpoint_round_trip(gpu, tmp_path):
    """Weights written as `weight` (float8_e4m3fn) + `weight_scale_inv` (the DeepSeek-V3 convention)
    and read back: the loaded module computes with the stored codes, so its output equals the
    saving module's bit for bit; the stored pair dequantizes to within the block's step."""
    import hpfp8
    from safetensors.torch import load_file
    torch.manual_seed(1)
    model = torch.nn.Sequential(hpfp8.Fp8Linear(256, 384, bias=True, device=gpu),
                                torch.nn.GELU(),
                                hpfp8.Fp8Linear(384, 128, bias=False, device=gpu))
    x = U.randn_bf16((128, 256), 61).to(gpu)
    y = model(x)
    path = str(tmp_path / "model.safetensors")
    hpfp8.checkpoint.save_fp8_checkpoint(hpfp8.checkpoint.fp8_state_dict(model), path)
    raw = load_file(path)
    assert raw["0.weight"].dtype == torch.float8_e4m3fn and raw["0.weight_scale_inv"].shape == (3, 2)
    assert raw["0.bias"].dtype == torch.bfloat16 and "2.weight_scale_inv" in raw
    clone = torch.nn.Sequential(hpfp8.Fp8Linear(256, 384, bias=True, device=gpu),
                                torch.nn.GELU(),
                                hpfp8.Fp8Linear(384, 128, bias=False, device=gpu))
    hpfp8.checkpoint.load_into(clone, hpfp8.checkpoint.load_fp8_checkpoint(path, device=gpu))
    assert torch.equal(clone(x), y)
    w, wd = model[0].weight.detach().float(), clone[0].weight.detach().float()
    amax = w.view(3, 128, 2, 128).abs().amax(dim=(1, 3), keepdim=True)
    assert bool(((w - wd).view(3, 128, 2, 128).abs() <= amax / 28 + amax / 256).all())


def test_policy_record_and_fp8_cast_hook(gpu):
    """The mixed-precision record keeps the reference's fields and defaults; the cast hook behaves like
    the reference's for ordinary dtypes and returns codes + scale for an E4M3 target (the per-tensor
    cast of cfg 1, bit for bit against the oracle)."""
    import hpfp8
    pol = hpfp8.Fp8MixedPrecisionPolicy()
    assert (pol.param_dtype, pol.reduce_dtype, pol.output_dtype) == (None, None, None)
    assert pol.cast_forward_inputs is True and pol.apply_grad_on_fp32_main_grad is False
    assert pol.linear_kwargs() == {"recipe": "blockwise", "apply_grad_on_fp32_main_grad": False}
    with pytest.raises(ValueError):
        hpfp8.Fp8MixedPrecisionPolicy(fp8_recipe="nope")
    with pytest.raises(ValueError):
        hpfp8.Fp8MixedPrecisionPolicy(reduce_dtype="float32")
    x = U.randn_bf16((256, 384), 91).to(gpu)
    assert hpfp8.cast_fp_tensor(torch.bfloat16, x) is x
    assert hpfp8.cast_fp_tensor(torch.float32, x).dtype == torch.float32
    ints = torch.arange(4, device=gpu)
    assert hpfp8.cast_fp_tensor(torch.float8_e4m3fn, ints) is ints and hpfp8.cast_fp_tensor(torch.float32, "s") == "s"
    t = hpfp8.cast_fp_tensor(torch.float8_e4m3fn, x)
    rq, _, rsi = O.quantize_per_tensor(U.bits(x))
    assert np.array_equal(U.codes(t.codes), rq) and np.array_equal(U.f32_bits(U.f32(t.scale_inv)), U.f32_bits(rsi))
    assert rel(t.dequantize(torch.float32), x.float()) < 0.05
    # the cast back is the library's kernel, bit for bit the oracle's decode * scale_inv (bf16: rounded once)
    assert np.array_equal(U.bits(t.dequantize()), O.dequantize_per_tensor(rq, rsi))
    assert np.array_equal(U.f32_bits(U.f32(t.dequantize(torch.float32))), U.f32_bits(O.dequantize_per_tensor_f32(rq, rsi)))
    assert t.dequantize(torch.float16).dtype == torch.float16
    odd = hpfp8.cast_fp_tensor(torch.float8_e4m3fn, x.reshape(-1)[:1000 * 3 + 7].contiguous())       # n % 16 != 0
    oq, _, osi = O.quantize_per_tensor(U.bits(x.reshape(-1)[:3007]))
    assert np.array_equal(U.bits(odd.dequantize()), O.dequantize_per_tensor(oq, osi))
    assert np.array_equal(U.f32_bits(U.f32(odd.dequantize(torch.float32))), U.f32_bits(O.dequantize_per_tensor_f32(oq, osi)))
    # the name-keyed cast of the reference's platform, with the FP8 name added
    t2 = hpfp8.tensor_type_cast(x, "float8_e4m3fn")
    assert torch.equal(t2.codes.view(torch.uint8), t.codes.view(torch.uint8)) and torch.equal(t2.scale_inv, t.scale_inv)
    assert hpfp8.tensor_type_cast(x, "float32").dtype == torch.float32 and hpfp8.tensor_type_cast(ints, "int32").dtype == torch.int32
    with pytest.raises(ValueError, match="Unknown cast type"):
        hpfp8.tensor_type_cast(x, "float8")
    pol = hpfp8.Fp8MixedPrecisionPolicy(apply_grad_on_fp32_main_grad=True, fp8_recipe="blockwise_pow2")
    w = U.randn_bf16((256, 384), 92, 0.02).to(gpu).requires_grad_(True)
    hpfp8.fp8_linear(x, w, **pol.linear_kwargs()).backward(U.randn_bf16((256, 256), 93, 1e-3).to(gpu))
    assert w.grad is None and w.main_grad.dtype == torch.float32


@pytest.mark.parametrize("fast", [False, True])
def test_swiglu_mlp_forward(gpu, fast):
    """The fused MLP forward is the chain of its parts bit for bit (quantize, GEMM, SwiGLU + quantize, GEMM),
    prequantized weights give the same output as bf16 weights, and the result stays within FP8 quantization
    noise of torch's bf16 MLP."""
    import hpfp8
    import torch.nn.functional as F
    g = torch.Generator(device="cpu").manual_seed(4)
    m, k, inter, n = 384, 512, 768, 640
    x = torch.randn((2, m // 2, k), generator=g).to(torch.bfloat16).to(gpu)
    wgu = (torch.randn((2 * inter, k), generator=g) * 0.05).to(torch.bfloat16).to(gpu)
    wd = (torch.randn((n, inter), generator=g) * 0.05).to(torch.bfloat16).to(gpu)
    y = hpfp8.fp8_swiglu_mlp(x, wgu, wd, fast=fast)
    assert y.shape == (2, m // 2, n) and y.dtype == torch.bfloat16 and not y.requires_grad
    # the chain of its parts
    xq, sx = hpfp8.quantize_1x128(x.reshape(m, k), kmajor=True)
    gq, gs = hpfp8.quantize_128x128(wgu)
    dq, ds = hpfp8.quantize_128x128(wd)
    h = hpfp8.gemm_blockwise(xq, sx, gq, gs)
    aq, sa = hpfp8.swiglu_quantize_1x128(h, kmajor=True, fast=fast)
    want = hpfp8.gemm_blockwise(aq, sa, dq, ds)
    assert torch.equal(y.reshape(m, n), want)
    y2 = hpfp8.fp8_swiglu_mlp(x, hpfp8.quantize_weight(wgu, with_transpose=False), hpfp8.quantize_weight(wd, with_transpose=False), fast=fast)
    assert torch.equal(y, y2)
    hr = F.linear(x, wgu)
    ref = F.linear(F.silu(hr[..., :inter]) * hr[..., inter:], wd)
    err = float((y.float() - ref.float()).norm() / ref.float().norm())
    assert err < 0.08, err
    with pytest.raises(ValueError):
        hpfp8.fp8_swiglu_mlp(x, wgu, wd[:, :640])


def test_swiglu_backward_kernel_vs_torch_autograd(gpu):
    """d gate | d up of the kernel against autograd of the same function evaluated in fp32 (results rounded
    to bf16 once on both sides): equal up to bf16 rounding of values that differ in the last bits of fp32;
    a strided h gives the same bits."""
    import hpfp8
    m, inter = 300, 1024
    h = U.randn_bf16((m, 2 * inter), 7, 2.0, 0.001, 20.0).to(gpu)
    h[0, :4] = torch.tensor([0.0, -0.0, 30.0, -30.0], dtype=torch.bfloat16)
    da = U.randn_bf16((m, inter), 8, 1e-2).to(gpu)
    dh = hpfp8.ops.swiglu_backward(h, da)
    assert dh.shape == (m, 2 * inter) and dh.dtype == torch.bfloat16
    g = h[:, :inter].float().requires_grad_(True)
    u = h[:, inter:].float()
    F.silu(g).backward(da.float() * u)                                  # d gate = (d act * up) * silu'(gate), all fp32
    dg_ref = g.grad.to(torch.bfloat16)
    silu_b = F.silu(h[:, :inter].float()).to(torch.bfloat16).float()   # forward multiplied up with the rounded silu
    du_f32 = da.float() * silu_b
    du_ref = du_f32.to(torch.bfloat16)
    # one bf16 step, or -- where silu' passes through zero (gate near -1.28) and its two terms cancel -- an
    # absolute error far below one step of the factor d act * up that it scales
    scale = (da.float() * u).abs()
    for got, want, slack in ((dh[:, :inter], dg_ref, 1e-3 * scale), (dh[:, inter:], du_ref, 0 * scale)):
        d = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs()
        small = (got.float() - want.float()).abs() <= slack + 1e-30
        # (d up: where the bf16 rounding of silu is a near-tie decided the other way, one step there is up to two here)
        assert bool(((d <= 2) | small).all()) and float(((d > 1) & ~small).float().mean()) < 1e-4
        assert float(((d != 0) & ~small).float().mean()) < 0.02
    assert rel(dh[:, :inter], g.grad) < 5e-3 and rel(dh[:, inter:], du_f32) < 5e-3
    # against the oracle's restatement of the same operation order (oracle/fp8_oracle.py swiglu_backward), to the
    # tolerance contract stated there: same bf16 value, or one step (d up: two) where a last-place difference of the
    # hardware's sigmoid crosses a rounding boundary, or inside the cancellation slack of silu'
    want = U.from_bits(O.swiglu_backward(U.bits(h), U.bits(da))).to(gpu)
    for lo, hi, steps, slack in ((0, inter, 1, 1e-3 * scale), (inter, 2 * inter, 2, 0 * scale)):
        got_h, want_h = dh[:, lo:hi], want[:, lo:hi]
        d = (got_h.view(torch.int16).int() - want_h.view(torch.int16).int()).abs()
        small = (got_h.float() - want_h.float()).abs() <= slack + 1e-30
        assert bool(((d <= steps) | small).all())
        assert float(((d != 0) & ~small).float().mean()) < 5e-3
    wide = torch.zeros((m, 2 * inter + 64), dtype=torch.bfloat16, device=gpu)
    wide[:, :2 * inter] = h
    assert torch.equal(hpfp8.ops.swiglu_backward(wide[:, :2 * inter], da), dh)
    with pytest.raises(ValueError):
        hpfp8.ops.swiglu_backward(h, da[:, :512])


def test_swiglu_mlp_training_step_vs_torch(gpu):
    """Forward and the three gradients of the MLP block against torch's fp32 autograd of the same graph, within
    FP8 quantization noise; the forward value equals the inference path's bit for bit."""
    import hpfp8
    g = torch.Generator(device="cpu").manual_seed(5)
    m, k, inter, n = 256, 512, 640, 384
    x = torch.randn((2, m // 2, k), generator=g).to(torch.bfloat16).to(gpu).requires_grad_(True)
    wgu = (torch.randn((2 * inter, k), generator=g) * 0.05).to(torch.bfloat16).to(gpu).requires_grad_(True)
    wd = (torch.randn((n, inter), generator=g) * 0.05).to(torch.bfloat16).to(gpu).requires_grad_(True)
    go = (torch.randn((2, m // 2, n), generator=g) * 1e-2).to(torch.bfloat16).to(gpu)
    y = hpfp8.fp8_swiglu_mlp(x, wgu, wd)
    assert y.requires_grad and y.shape == (2, m // 2, n)
    with torch.no_grad():
        assert torch.equal(y, hpfp8.fp8_swiglu_mlp(x, wgu, wd))
    y.backward(go)
    gx, ggu, gd = x.grad.clone(), wgu.grad.clone(), wd.grad.clone()
    x.grad = wgu.grad = wd.grad = None
    hr = F.linear(x.float(), wgu.float())
    yr = F.linear(F.silu(hr[..., :inter]) * hr[..., inter:], wd.float())
    yr.backward(go.float())
    assert rel(y, yr) < 0.08 and rel(gx, x.grad) < 0.1 and rel(ggu, wgu.grad) < 0.1 and rel(gd, wd.grad) < 0.08
    # weights quantized ahead of the step: same bits
    wgu.grad = wd.grad = None
    x3 = x.detach().clone().requires_grad_(True)
    y3 = hpfp8.fp8_swiglu_mlp(x3, wgu, wd, gate_up_fp8=hpfp8.quantize_weight(wgu), down_fp8=hpfp8.quantize_weight(wd))
    y3.backward(go)
    assert torch.equal(y3, y) and torch.equal(x3.grad, gx) and torch.equal(wgu.grad, ggu) and torch.equal(wd.grad, gd)
    wgu.grad = wd.grad = None
    # only the input needs a gradient (frozen weights)
    x2 = x.detach().clone().requires_grad_(True)
    y2 = hpfp8.fp8_swiglu_mlp(x2, wgu.detach(), wd.detach())
    y2.backward(go)
    assert torch.equal(y2, y) and rel(x2.grad, gx) < 1e-6


def test_swiglu_backward_fused_with_both_quantized_forms(gpu):
    """The gradient of SwiGLU quantized for the gate/up projection's dgrad and wgrad as it is computed: codes and
    scales of both forms equal, bit for bit, the two quantizers applied to the bf16 gradient that the stand-alone
    backward kernel writes (rows of a wider buffer as h give the same); and the MLP block as one autograd node
    (which uses it) returns the same output and the same three gradients, bit for bit, as the chain of
    fp8_linear and the SwiGLU + down-projection node that it replaces."""
    import hpfp8
    from hpfp8 import ops
    from hpfp8.linear import _Fp8SwiGLUDown
    m, inter = 384, 640
    h = U.randn_bf16((m, 2 * inter), 31, 2.0, 0.001, 20.0).to(gpu)
    h[0, :6] = torch.tensor([0.0, -0.0, 88.5, -88.5, -200.0, 200.0], dtype=torch.bfloat16)
    dact = U.randn_bf16((m, inter), 32, 1e-2, 0.001, 50.0).to(gpu)
    dh = ops.swiglu_backward(h, dact)
    q1, s1, qt1, st1 = hpfp8.quantize_1x128_and_128x1_t(dh, kmajor=True)
    q, s, qt, st = ops.swiglu_backward_quantize_1x128_and_128x1_t(h, dact)
    assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(s, s1)
    assert torch.equal(qt.view(torch.uint8), qt1.view(torch.uint8)) and torch.equal(st, st1)
    assert s.stride(0) == 1 and st.stride(0) == 1
    wide = torch.zeros((m, 2 * inter + 64), dtype=torch.bfloat16, device=gpu)
    wide[:, :2 * inter] = h
    q2, s2, qt2, st2 = ops.swiglu_backward_quantize_1x128_and_128x1_t(wide[:, :2 * inter], dact)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(qt2.view(torch.uint8), qt.view(torch.uint8))
    assert torch.equal(s2, s) and torch.equal(st2, st)
    with pytest.raises(ValueError):
        ops.swiglu_backward_quantize_1x128_and_128x1_t(h[:100], dact[:100])
    # the block as one node against the two nodes it replaces
    g = torch.Generator(device="cpu").manual_seed(9)
    k, n = 512, 384
    x = torch.randn((m, k), generator=g).to(torch.bfloat16).to(gpu).requires_grad_(True)
    wgu = (torch.randn((2 * inter, k), generator=g) * 0.05).to(torch.bfloat16).to(gpu).requires_grad_(True)
    wd = (torch.randn((n, inter), generator=g) * 0.05).to(torch.bfloat16).to(gpu).requires_grad_(True)
    go = (torch.randn((m, n), generator=g) * 1e-2).to(torch.bfloat16).to(gpu)
    for fast in (True, False):
        y = hpfp8.fp8_swiglu_mlp(x, wgu, wd, fast=fast)
        assert type(y.grad_fn).__name__.startswith("_Fp8SwiGLUMLPBlock")
        got = torch.autograd.grad(y, (x, wgu, wd), go)
        y0 = _Fp8SwiGLUDown.apply(hpfp8.fp8_linear(x, wgu), wd, fast)
        want = torch.autograd.grad(y0, (x, wgu, wd), go)
        assert torch.equal(y, y0)
        for a, b in zip(got, want):
            assert torch.equal(a, b)
    # an input that needs no gradient: the same weight gradients
    y = hpfp8.fp8_swiglu_mlp(x.detach(), wgu, wd)
    got2 = torch.autograd.grad(y, (wgu, wd), go)
    ref2 = torch.autograd.grad(hpfp8.fp8_swiglu_mlp(x, wgu, wd), (wgu, wd), go)
    assert torch.equal(got2[0], ref2[0]) and torch.equal(got2[1], ref2[1])


def test_mlp_training_step_replays_from_a_captured_graph(gpu):
    """Forward and backward of the MLP block captured into one graph (weights prequantized outside it): every
    replay, with eager work and synchronisations in between, gives the eager step's output and gradients for
    the input of the moment."""
    import hpfp8
    g = torch.Generator(device="cpu").manual_seed(6)
    m, k, inter, n = 256, 512, 640, 384
    wgu = (torch.randn((2 * inter, k), generator=g) * 0.05).to(torch.bfloat16).to(gpu).requires_grad_(True)
    wd = (torch.randn((n, inter), generator=g) * 0.05).to(torch.bfloat16).to(gpu).requires_grad_(True)
    gu8, d8 = hpfp8.quantize_weight(wgu.detach()), hpfp8.quantize_weight(wd.detach())
    xs = [torch.randn((m, k), generator=g).mul(1.0 + i).to(torch.bfloat16).to(gpu) for i in range(4)]
    go = (torch.randn((m, n), generator=g) * 1e-2).to(torch.bfloat16).to(gpu)
    x_static = xs[0].clone().requires_grad_(True)

    def step(x):
        y = hpfp8.fp8_swiglu_mlp(x, wgu, wd, gate_up_fp8=gu8, down_fp8=d8)
        gx, ggu, gd = torch.autograd.grad(y, (x, wgu, wd), go)
        return y, gx, ggu, gd

    if hasattr(torch.autograd.graph, "set_warn_on_accumulate_grad_stream_mismatch"):
        torch.autograd.graph.set_warn_on_accumulate_grad_stream_mismatch(False)    # (leaves made on the default stream, used on a side stream)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step(x_static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step(x_static)
    for x in xs[1:] + xs[:2]:
        with torch.no_grad():
            x_static.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        want = step(x.clone().requires_grad_(True))
        for a, b in zip(outs, want):
            assert torch.equal(a, b)


def test_swiglu_mlp_module_caches_weights_and_trains(gpu):
    """The module equals the functional form on its own parameters, quantizes each weight once until the
    parameter is written, and an SGD step through it lowers a least-squares loss."""
    import hpfp8
    torch.manual_seed(0)
    mlp = hpfp8.Fp8SwiGLUMLP(256, 384, cache_weight=True, device=gpu)
    x = torch.randn((128, 256), device=gpu).to(torch.bfloat16)
    y = mlp(x)
    want = hpfp8.fp8_swiglu_mlp(x, mlp.gate_up_proj.weight, mlp.down_proj.weight)
    assert torch.equal(y, want) and y.requires_grad
    first = mlp._fp8[0]
    mlp(x)
    assert mlp._fp8[0] is first                       # same parameter version: no second quantization
    target = torch.randn((128, 256), device=gpu).to(torch.bfloat16)
    opt = torch.optim.SGD(mlp.parameters(), lr=0.05)
    losses = []
    for _ in range(5):
        opt.zero_grad()
        loss = (mlp(x).float() - target.float()).pow(2).mean()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert mlp._fp8[0] is not first                   # the optimizer wrote the parameter
    assert losses[-1] < losses[0]
    assert set(mlp.state_dict()) == {"gate_up_proj.weight", "down_proj.weight"}


def test_two_threads_on_two_streams(gpu):
    """Calls from two host threads, each on a stream of its own, run concurrently and give the bits of the same
    calls made one after the other on the default stream (no shared state inside the library besides the
    per-thread error text)."""
    import threading
    import hpfp8
    xs = [U.randn_bf16((512, 1024), 90 + i).to(gpu) for i in range(2)]
    ws = [U.randn_bf16((768, 1024), 95 + i, 0.02).to(gpu) for i in range(2)]

    def work(x, w):
        xq, sx = hpfp8.quantize_1x128(x, kmajor=True)
        wq, sw = hpfp8.quantize_128x128(w)
        y = hpfp8.gemm_blockwise(xq, sx, wq, sw)
        h = hpfp8.gemm_blockwise(xq, sx, wq, sw, out_dtype=torch.float32)
        aq, sa = hpfp8.swiglu_quantize_1x128(y, kmajor=True, fast=True)
        return y, h, aq.view(torch.uint8), sa

    want = [work(x, w) for x, w in zip(xs, ws)]
    torch.cuda.synchronize()
    got = [None, None]
    errors = []

    def run(i):
        try:
            stream = torch.cuda.Stream()
            stream.wait_stream(torch.cuda.default_stream())
            with torch.cuda.stream(stream):
                for _ in range(20):
                    got[i] = work(xs[i], ws[i])
                try:
                    hpfp8.quantize_1x128(xs[i][:, :100])          # an error in this thread only
                except ValueError:
                    pass
            stream.synchronize()
        except Exception as e:                                    # pragma: no cover
            errors.append(e)

    threads = [threading.Thread(target=run, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for g_, w_ in zip(got, want):
        for a, b in zip(g_, w_):
            assert torch.equal(a, b)


@pytest.mark.parametrize("recipe", ["blockwise", "per_tensor", "blockwise_pow2"])
def test_empty_batch_and_one_dimensional_input(gpu, recipe):
    """F.linear's behaviour at the edges of the batch: no rows gives no rows, with zero weight and bias gradients;
    a 1-D input gives a 1-D output."""
    import hpfp8
    w = U.randn_bf16((384, 512), 2, 0.02).to(gpu).requires_grad_(True)
    b = U.randn_bf16((384,), 3, 0.1).to(gpu).requires_grad_(True)
    x = torch.empty((0, 512), dtype=torch.bfloat16, device=gpu, requires_grad=True)
    y = hpfp8.fp8_linear(x, w, b, recipe=recipe)
    assert y.shape == (0, 384)
    y.backward(torch.empty_like(y))
    assert x.grad.shape == (0, 512) and not bool(w.grad.any()) and not bool(b.grad.any()) and w.grad.shape == w.shape
    v = U.randn_bf16((512,), 5).to(gpu)
    y1 = hpfp8.fp8_linear(v, w.detach(), b.detach(), recipe=recipe)
    assert y1.shape == (384,) and torch.equal(y1, hpfp8.fp8_linear(v[None], w.detach(), b.detach(), recipe=recipe)[0])
    if recipe == "blockwise":
        x3 = torch.empty((2, 0, 512), dtype=torch.bfloat16, device=gpu, requires_grad=True)
        wgu = U.randn_bf16((512, 512), 6, 0.02).to(gpu).requires_grad_(True)
        wd = U.randn_bf16((384, 256), 7, 0.02).to(gpu).requires_grad_(True)
        y3 = hpfp8.fp8_swiglu_mlp(x3, wgu, wd)
        assert y3.shape == (2, 0, 384)
        y3.backward(torch.empty_like(y3))
        assert x3.grad.shape == x3.shape and not bool(wgu.grad.any()) and not bool(wd.grad.any())


@pytest.mark.parametrize("recipe", ["blockwise", "per_tensor", "blockwise_pow2"])
def test_token_count_that_is_not_a_multiple_of_128(gpu, recipe):
    """Any batch size trains: the weight gradient's groups along the tokens are filled up with zero rows, which
    is exactly the gradient of the batch with those rows appended (bit for bit), and stays within FP8 noise of
    F.linear's."""
    import hpfp8
    x = U.randn_bf16((3, 100, 512), 1).to(gpu).requires_grad_(True)          # 300 tokens
    w = U.randn_bf16((384, 512), 2, 0.02).to(gpu).requires_grad_(True)
    b = U.randn_bf16((384,), 3, 0.1).to(gpu).requires_grad_(True)
    go = U.randn_bf16((3, 100, 384), 4, 1e-3).to(gpu)
    y = hpfp8.fp8_linear(x, w, b, recipe=recipe)
    y.backward(go)
    gx, gw, gb = x.grad.clone(), w.grad.clone(), b.grad.clone()
    x.grad = w.grad = b.grad = None
    yr = F.linear(x.float(), w.float(), b.float())
    yr.backward(go.float())
    tol = 0.06 if recipe == "blockwise" else 0.08
    assert rel(y, yr) < tol and rel(gx, x.grad) < tol and rel(gw, w.grad) < tol and rel(gb, b.grad) < 1e-2
    w.grad = None
    xp = torch.cat([x.detach().reshape(300, 512), torch.zeros((84, 512), dtype=torch.bfloat16, device=gpu)]).requires_grad_(True)
    gop = torch.cat([go.reshape(300, 384), torch.zeros((84, 384), dtype=torch.bfloat16, device=gpu)])
    hpfp8.fp8_linear(xp, w, b, recipe=recipe).backward(gop)
    if recipe != "per_tensor":                                               # (per tensor: the bias row changes no amax either)
        assert torch.equal(w.grad, gw)
    assert rel(w.grad, gw) < 1e-6
    if recipe == "blockwise":
        wgu = U.randn_bf16((512, 512), 6, 0.05).to(gpu).requires_grad_(True)
        wd = U.randn_bf16((384, 256), 7, 0.05).to(gpu).requires_grad_(True)
        x2 = x.detach().clone().requires_grad_(True)
        hpfp8.fp8_swiglu_mlp(x2, wgu, wd).backward(go)
        hr = F.linear(x2.detach().float(), wgu.float())
        yr = F.linear(F.silu(hr[..., :256]) * hr[..., 256:], wd.float())
        gr = torch.autograd.grad(yr, (wgu, wd), go.float())
        assert rel(wgu.grad, gr[0]) < 0.1 and rel(wd.grad, gr[1]) < 0.08 and x2.grad.shape == x2.shape


def test_grouped_linear_backward(gpu):
    """Input and weight gradients of the grouped linear against a loop of F.linear over the experts (fp32
    autograd), experts with no rows and rows that belong to no expert included."""
    import hpfp8
    counts = torch.tensor([130, 0, 300, 70])                    # 500 of 512 rows are routed
    offs = counts.cumsum(0).to(torch.int32).to(gpu)
    x = U.randn_bf16((512, 256), 31).to(gpu).requires_grad_(True)
    w = U.randn_bf16((4, 384, 256), 32, 0.05).to(gpu).requires_grad_(True)
    go = U.randn_bf16((512, 384), 33, 1e-2).to(gpu)
    y = hpfp8.fp8_grouped_linear(x, w, offs)
    y.backward(go)
    gx, gw = x.grad.clone(), w.grad.clone()
    x.grad = w.grad = None
    start = 0
    for e in range(4):
        c = int(counts[e])
        if c:
            F.linear(x[start:start + c].float(), w[e].float()).backward(go[start:start + c].float())
        start += c
    assert rel(gx[:500], x.grad[:500]) < 0.06 and not bool(gx[500:].any())
    assert rel(gw, w.grad) < 0.08 and not bool(gw[1].any())
    for e in (0, 2, 3):
        assert rel(gw[e], w.grad[e]) < 0.08
    # only one of the two gradients
    x1 = x.detach().clone().requires_grad_(True)
    hpfp8.fp8_grouped_linear(x1, w.detach(), offs).backward(go)
    assert torch.equal(x1.grad, gx)
    w1 = w.detach().clone().requires_grad_(True)
    hpfp8.fp8_grouped_linear(x.detach(), w1, offs).backward(go)
    assert torch.equal(w1.grad, gw)


def test_grouped_linear_prequantized_weight_and_inference(gpu):
    """`weight_fp8` for the grouped linear gives the same outputs and gradients bit for bit; under no_grad nothing is
    prepared for a backward."""
    import hpfp8
    counts = torch.tensor([130, 0, 300, 70])
    offs = counts.cumsum(0).to(torch.int32).to(gpu)
    x = U.randn_bf16((512, 256), 31).to(gpu).requires_grad_(True)
    w = U.randn_bf16((4, 384, 256), 32, 0.05).to(gpu).requires_grad_(True)
    go = U.randn_bf16((512, 384), 33, 1e-2).to(gpu)
    y0 = hpfp8.fp8_grouped_linear(x, w, offs)
    y0.backward(go)
    gx, gw = x.grad.clone(), w.grad.clone()
    x.grad = w.grad = None
    for with_t in (True, False):
        f8 = hpfp8.quantize_grouped_weight(w.detach(), with_transpose=with_t)
        y1 = hpfp8.fp8_grouped_linear(x, w, offs, weight_fp8=f8)
        y1.backward(go)
        assert torch.equal(y1[:500], y0[:500]) and torch.equal(x.grad, gx) and torch.equal(w.grad, gw)
        x.grad = w.grad = None
    with torch.no_grad():
        y2 = hpfp8.fp8_grouped_linear(x, w, offs)
    assert torch.equal(y2[:500], y0.detach()[:500]) and not y2.requires_grad
    with pytest.raises(ValueError):
        hpfp8.fp8_grouped_linear(x, w, offs[:3])
