"""FP8 linear with the calling convention of torch.nn.functional.linear.

`fp8_linear(input, weight, bias=None)` is what a model swaps in for `F.linear`: same argument
order, weight [out_features, in_features], contraction over the last dim of both, output
`input.shape[:-1] + (out_features,)` in bf16 -- the operator the reference registers in
hyper_parallel/core/shard/ops/yaml/torch_mm.yaml:6-9 and type-checks in
hyper_parallel/core/shard/ops/parallel_matmul.py:344-404.  Being a plain function on local
tensors it also fits `custom_shard(func, ...)` (hyper_parallel/core/shard/local_func.py:26-128).

Recipes
  "blockwise"  : activations / output gradients 1x128, weights 128x128; wgrad operands are
                 quantized 128x1 (transposed) from the bf16 sources, in the same pass that makes
                 the 1x128 codes where both are needed.
  "per_tensor" : one scale per tensor (amax -> 448/amax); backward also per tensor.
  "blockwise_pow2" : the blockwise groups with every scale_inv rounded up to a power of two (E8M0
                 scales, as DeepSeek-V3.1 trains with).  gfx950's matrix instruction applies such
                 scales itself, so the three GEMMs do no scaling arithmetic and run 10 % (forward,
                 dgrad) to 23 % (wgrad) faster; the price is up to one binade of headroom per group.
                 An extension: the benchmarked recipe is "blockwise" with plain fp32 scales.
"""
from __future__ import annotations

from typing import NamedTuple, Optional

import torch
from torch import nn

from . import ops

RECIPES = ("blockwise", "per_tensor", "blockwise_pow2")


class Fp8Weight(NamedTuple):
    """A weight [N, K] already in its blockwise FP8 form: what `fp8_linear` would otherwise make from
    the bf16 weight on every call."""
    codes: torch.Tensor                 # e4m3 [N, K]
    scale_inv: torch.Tensor             # fp32 [N/128, K/128]
    codes_t: Optional[torch.Tensor]     # e4m3 [K, N] (dgrad operand) or None
    pow2: bool = False                  # scales are powers of two ("blockwise_pow2")

    def __repr__(self) -> str:
        # Shapes and addresses, never element values: the reference's dispatcher makes its layout-cache key from
        # str() of every non-tensor argument (hyper_parallel/core/shard/_op_dispatch.py:205-210, :226-231), and a
        # tuple's default repr would print (and copy to the host) whole device tensors on every call.
        def one(t):
            return "None" if t is None else f"{tuple(t.shape)}@{t.data_ptr():#x}"
        return f"Fp8Weight(codes={one(self.codes)}, scale_inv={one(self.scale_inv)}, codes_t={one(self.codes_t)}, pow2={self.pow2})"


def quantize_weight(weight: torch.Tensor, with_transpose: bool = True, pow2: bool = False,
                    per_tensor: bool = False) -> Fp8Weight:
    """128x128-block quantization of a bf16 weight (and its transposed codes for dgrad); with ``per_tensor`` the
    weight's form under the "per_tensor" recipe instead: codes and one scale_inv (0-dim)."""
    if per_tensor:
        wq, _, sw = ops.quantize_per_tensor(weight)
        return Fp8Weight(wq, sw, None, False)
    if with_transpose:
        wq, sw, wqt = ops.quantize_128x128(weight, with_transpose=True, pow2=pow2)
        return Fp8Weight(wq, sw, wqt, pow2)
    wq, sw = ops.quantize_128x128(weight, pow2=pow2)
    return Fp8Weight(wq, sw, None, pow2)


def _hand_off(func, tensors, args, kwargs, defaults):
    """The `__torch_function__` protocol for a Python-level operator: when any tensor argument is of a subclass that
    overrides `__torch_function__` (the reference's DTensor, hyper_parallel/platform/torch/dtensor.py:50-62), the
    call is given to that hook with THIS function object as `func` -- the reference derives its registry key from
    `func.__name__` (hyper_parallel/platform/torch/platform.py:159-174) and, after layout inference, calls the
    function again on the local tensors (hyper_parallel/core/shard/_op_dispatch.py:277-283), where this returns
    NotImplemented and the kernels run.  Keyword arguments still at their defaults are left out, so that a plain
    call reaches the hook as (input, weight, bias) exactly like `torch.nn.functional.linear` does."""
    if not torch.overrides.has_torch_function(tensors):
        return NotImplemented
    kw = {k: v for k, v in kwargs.items()
          if not (v is defaults[k] or (isinstance(v, (str, bool)) and v == defaults[k]))}
    return torch.overrides.handle_torch_function(func, tensors, *args, **kw)


def _flatten(x: torch.Tensor):
    return x.reshape(-1, x.shape[-1])


def _pad_rows(t: torch.Tensor) -> torch.Tensor:
    """t[M, C] with zero rows appended up to the next multiple of 128: tokens that contribute nothing to a
    weight gradient, so that the 128x1 groups along the tokens are whole (the last one holds fewer real values)."""
    pad = -t.shape[0] % ops.BLOCK
    return torch.nn.functional.pad(t, (0, 0, 0, pad)) if pad else t


def _empty_batch_grads(ctx, go):
    """(dx, dw, db) of a linear whose batch is empty: no token contributes, so the weight and bias gradients are
    zero (an fp32 main gradient is left as it is, or created as zeros)."""
    need_dx, need_dw = ctx.need
    dx = go.new_zeros(ctx.x_shape) if need_dx else None
    dw = None
    if need_dw:
        param = getattr(ctx, "main_grad_of", None)
        if param is None:
            dw = go.new_zeros(ctx.w_shape)
        elif getattr(param, "main_grad", None) is None:
            param.main_grad = torch.zeros(ctx.w_shape, dtype=torch.float32, device=go.device)
    db = go.new_zeros(ctx.w_shape[0]) if ctx.has_bias else None
    return dx, dw, db


class _Fp8LinearBlockwise(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, wq=None, sw=None, wqt=None, on_main_grad=False, pow2=False, grad_mode=True):
        ctx.main_grad_of = weight if on_main_grad else None
        ctx.pow2 = pow2
        x2 = _flatten(x)
        m = x2.shape[0]
        # grad_mode: whether the caller ran with gradients enabled (inside this function they never are).  A
        # Parameter has requires_grad set under torch.no_grad() too; without a backward to come nothing is
        # prepared or kept for it.
        need_dx, need_dw = grad_mode and x.requires_grad, grad_mode and weight.requires_grad
        # With a weight gradient to come and a token count that allows it, x is read once: its 1x128
        # codes for this GEMM and its transposed 128x1 codes for wgrad, which are what is kept for
        # backward (1 byte per element instead of the bf16 source).
        fused = need_dw and m % ops.BLOCK == 0 and m > 0
        if fused:
            xq, sx, xt, sxt = ops.quantize_1x128_and_128x1_t(x2.contiguous(), kmajor=True, pow2=pow2)
        else:
            xq, sx = ops.quantize_1x128(x2, kmajor=True, pow2=pow2)
            xt = sxt = None
        if wq is None:                          # no prequantized form of the weight was passed in
            if need_dx:
                wq, sw, wqt = ops.quantize_128x128(weight, with_transpose=True, pow2=pow2)
            else:
                wq, sw = ops.quantize_128x128(weight, pow2=pow2)
        elif need_dx and wqt is None:
            wqt = ops.transpose_codes(wq)
        y = ops.gemm_blockwise(xq, sx, wq, sw, bias=bias, pow2_scales=pow2)
        ctx.save_for_backward(x2 if (need_dw and not fused) else None, xt, sxt, wqt if need_dx else None, sw)
        ctx.x_shape = x.shape
        ctx.w_shape = weight.shape
        ctx.has_bias = bias is not None
        ctx.need = (need_dx, need_dw)
        return y.reshape(x.shape[:-1] + (weight.shape[0],))

    @staticmethod
    def backward(ctx, grad_out):
        x2, xt, sxt, wqt, sw = ctx.saved_tensors
        need_dx, need_dw = ctx.need
        pow2 = ctx.pow2
        go = _flatten(grad_out)
        if go.dtype != torch.bfloat16:
            go = go.to(torch.bfloat16)
        go = go.contiguous()
        m = go.shape[0]
        if m == 0:
            return _empty_batch_grads(ctx, go) + (None, None, None, None, None, None)
        ragged = m % ops.BLOCK != 0            # wgrad then runs on zero-padded token rows
        dx = dw = db = None
        goq = sgo = got = sgot = None
        if need_dx and need_dw and not ragged:
            if ctx.has_bias:                   # one read of grad_out: both operand forms and the bias gradient
                goq, sgo, got, sgot, db = ops.quantize_1x128_and_128x1_t(go, kmajor=True, pow2=pow2, column_sum=True)
            else:
                goq, sgo, got, sgot = ops.quantize_1x128_and_128x1_t(go, kmajor=True, pow2=pow2)
        else:
            if need_dx:
                goq, sgo = ops.quantize_1x128(go, kmajor=True, pow2=pow2)
            if need_dw:
                got, sgot = ops.quantize_128x1_t(_pad_rows(go), kmajor=True, pow2=pow2)
            if ctx.has_bias:
                db = ops.column_sum(go)
        if need_dx:
            # dx[M,K] = go[M,N] . W[N,K]: contraction over N, b operand = W^T codes [K,N] whose
            # 128x128 scales are W's with the two strides swapped.
            dx = ops.gemm_blockwise(goq, sgo, wqt, sw.t(), pow2_scales=pow2).reshape(ctx.x_shape)
        if need_dw:
            # dW[N,K] = go^T[N,M] . x[M,K]: contraction over tokens, both operands 1x128 along M
            if xt is None:
                xt, sxt = ops.quantize_128x1_t(_pad_rows(x2), kmajor=True, pow2=pow2)
            param = ctx.main_grad_of
            if param is None:
                dw = ops.gemm_blockwise(got, sgot, xt, sxt, sb_gran=1, pow2_scales=pow2)
            elif getattr(param, "main_grad", None) is None:
                # the fp32 main gradient of hyper_parallel/platform/torch/fully_shard/param.py:134-167: the
                # first weight gradient creates it, later ones are added onto it by the GEMM itself, and
                # .grad stays empty
                param.main_grad = ops.gemm_blockwise(got, sgot, xt, sxt, sb_gran=1, out_dtype=torch.float32,
                                                     pow2_scales=pow2)
            else:
                ops.gemm_blockwise(got, sgot, xt, sxt, sb_gran=1, out=param.main_grad, accumulate=True, pow2_scales=pow2)
        return dx, dw, db, None, None, None, None, None, None


class _Fp8LinearPerTensor(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, wq=None, sw=None):
        x2 = _flatten(x)
        xq, _, sx = ops.quantize_per_tensor(x2)
        if wq is None:                          # no prequantized form of the weight was passed in
            wq, _, sw = ops.quantize_per_tensor(weight)
        y = ops.gemm_per_tensor(xq, sx, wq, sw, bias=bias)
        # With one scale per tensor the codes of a transposed tensor are the transposed codes, so backward
        # needs no second quantization of x and W: it keeps the codes (1 byte per element) where their
        # shapes allow the byte transpose, and the bf16 tensors otherwise.
        m = x2.shape[0]
        can_t = m % ops.BLOCK == 0 and m > 0
        ctx.codes_saved = can_t
        if can_t:
            ctx.save_for_backward(xq if weight.requires_grad else None, sx, wq if x.requires_grad else None, sw)
        else:
            ctx.save_for_backward(x2, weight)
        ctx.x_shape = x.shape
        ctx.w_shape = weight.shape
        ctx.has_bias = bias is not None
        ctx.need = (x.requires_grad, weight.requires_grad)
        return y.reshape(x.shape[:-1] + (weight.shape[0],))

    @staticmethod
    def backward(ctx, grad_out):
        need_dx, need_dw = ctx.need
        go = _flatten(grad_out)
        if go.dtype != torch.bfloat16:
            go = go.to(torch.bfloat16)
        go = go.contiguous()
        if go.shape[0] == 0:
            return _empty_batch_grads(ctx, go) + (None, None)
        dx = dw = db = None
        if ctx.codes_saved:
            xq, sx, wq, sw = ctx.saved_tensors
            goq, _, sgo = ops.quantize_per_tensor(go)
            if need_dx:
                dx = ops.gemm_per_tensor(goq, sgo, ops.transpose_codes(wq), sw).reshape(ctx.x_shape)
            if need_dw:
                dw = ops.gemm_per_tensor(ops.transpose_codes(goq), sgo, ops.transpose_codes(xq), sx)
        else:
            x2, weight = ctx.saved_tensors
            if need_dx:
                goq, _, sgo = ops.quantize_per_tensor(go)
                wtq, _, swt = ops.quantize_per_tensor(weight.t().contiguous())
                dx = ops.gemm_per_tensor(goq, sgo, wtq, swt).reshape(ctx.x_shape)
            if need_dw:
                gotq, _, sgot = ops.quantize_per_tensor(_pad_rows(go).t().contiguous())
                xtq, _, sxt = ops.quantize_per_tensor(_pad_rows(x2).t().contiguous())
                dw = ops.gemm_per_tensor(gotq, sgot, xtq, sxt)
        if ctx.has_bias:
            db = ops.column_sum(go)
        return dx, dw, db, None, None


def fp8_linear(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, *,
               recipe: str = "blockwise", weight_fp8: Optional[Fp8Weight] = None,
               apply_grad_on_fp32_main_grad: bool = False) -> torch.Tensor:
    """y = input @ weight.T + bias computed through E4M3 operands with fp32 accumulation.

    input [..., in_features] bf16, weight [out_features, in_features] bf16, bias [out_features] bf16
    or None; returns bf16 [..., out_features].  in_features and out_features must be multiples of
    128 (ragged tails are rejected, not padded); the token count may be anything (for the weight gradient,
    whose scaling groups run along the tokens, a ragged count is filled up with zero rows).

    `weight_fp8` is the weight's FP8 form under the same recipe made earlier -- by `quantize_weight`, or
    from all-gathered FP8 shards (`hpfp8.fsdp`) -- and saves its quantization in this call; `weight`
    is still the tensor that receives the gradient.

    `apply_grad_on_fp32_main_grad` (blockwise recipe; the flag of the reference's mixed-precision
    policy, hyper_parallel/platform/torch/fully_shard/param.py:134-167) sends the weight gradient to
    `weight.main_grad` instead of `weight.grad`: a float32 [out_features, in_features] tensor that the
    first backward creates and every later one adds onto, inside the wgrad GEMM.
    """
    out = _hand_off(fp8_linear, tuple(t for t in (input, weight, bias) if t is not None), (input, weight, bias),
                    dict(recipe=recipe, weight_fp8=weight_fp8, apply_grad_on_fp32_main_grad=apply_grad_on_fp32_main_grad),
                    _FP8_LINEAR_DEFAULTS)
    if out is not NotImplemented:
        return out
    if recipe not in RECIPES:
        raise ValueError(f"recipe must be one of {RECIPES}, got {recipe!r}")
    if weight.dim() != 2:
        raise ValueError("weight must be [out_features, in_features]")
    if input.shape[-1] != weight.shape[1]:
        raise ValueError(f"input last dim {input.shape[-1]} != weight in_features {weight.shape[1]}")
    for name, t in (("input", input), ("weight", weight), ("bias", bias)):
        if t is not None and t.dtype != torch.bfloat16:
            raise TypeError(f"{name} must be bfloat16, got {t.dtype}")
    pow2 = recipe == "blockwise_pow2"
    if apply_grad_on_fp32_main_grad:
        if recipe == "per_tensor":
            raise ValueError("apply_grad_on_fp32_main_grad is only implemented for the blockwise recipes")
        mg = getattr(weight, "main_grad", None)
        if mg is not None and (mg.dtype != torch.float32 or tuple(mg.shape) != tuple(weight.shape) or
                               not mg.is_contiguous()):
            raise ValueError("weight.main_grad must be a contiguous float32 tensor of the weight's shape")
    if weight_fp8 is not None:
        if tuple(weight_fp8.codes.shape) != tuple(weight.shape):
            raise ValueError("weight_fp8 does not have the weight's shape")
        if recipe == "per_tensor":
            if weight_fp8.scale_inv.numel() != 1:
                raise ValueError("weight_fp8 was not quantized with one scale per tensor")
            return _Fp8LinearPerTensor.apply(input, weight, bias, weight_fp8.codes, weight_fp8.scale_inv)
        if weight_fp8.scale_inv.dim() != 2:
            raise ValueError("weight_fp8 was quantized with one scale per tensor")
        if bool(weight_fp8.pow2) != pow2:
            raise ValueError("weight_fp8 was quantized for the other blockwise recipe")
        return _Fp8LinearBlockwise.apply(input, weight, bias, weight_fp8.codes, weight_fp8.scale_inv,
                                         weight_fp8.codes_t, apply_grad_on_fp32_main_grad, pow2, torch.is_grad_enabled())
    if recipe != "per_tensor":
        return _Fp8LinearBlockwise.apply(input, weight, bias, None, None, None, apply_grad_on_fp32_main_grad, pow2,
                                         torch.is_grad_enabled())
    return _Fp8LinearPerTensor.apply(input, weight, bias)


_FP8_LINEAR_DEFAULTS = dict(recipe="blockwise", weight_fp8=None, apply_grad_on_fp32_main_grad=False)


def _init_like_nn_linear(weight: torch.Tensor, bias: Optional[torch.Tensor]) -> None:
    """torch.nn.Linear.reset_parameters, in place on the parameters' own device (no fp32 host copy of the layer)."""
    import math
    with torch.no_grad():
        nn.init.kaiming_uniform_(weight, a=math.sqrt(5))
        if bias is not None:
            bound = 1.0 / math.sqrt(weight.shape[1]) if weight.shape[1] > 0 else 0.0
            nn.init.uniform_(bias, -bound, bound)


class _Fp8WeightCache:
    """FP8 forms of a module's bf16 weights, kept between calls.

    Contract.  An entry is refreshed when the parameter's autograd version counter or its data pointer changes:
    that covers in-place updates under ``torch.no_grad()`` (what torch's optimizers do), ``copy_`` (what
    ``load_state_dict`` does) and a parameter that was replaced.  It does NOT cover writes the version counter never
    sees: through ``param.data``, under ``torch.autograd._unsafe_preserve_version_counter``, or by a collective that
    refills a persistent buffer at the same address (the reference's all-gather into ``_unsharded_param``,
    hyper_parallel/platform/torch/fully_shard/param.py:627-647).  After such a write call
    ``module.invalidate_fp8_cache()`` -- `attach_optimizer` registers that as an optimizer step hook, and the
    modules do it themselves after ``load_state_dict`` -- or construct the module with ``cache_weight=False``."""

    def __init__(self, n: int = 1):
        self._fp8 = [None] * n
        self._key = [None] * n

    def get(self, i: int, w: torch.Tensor, make) -> Fp8Weight:
        key = (w._version, w.data_ptr())
        if self._key[i] != key:
            with torch.no_grad():
                self._fp8[i] = make(w.detach())
            self._key[i] = key
        return self._fp8[i]

    def put(self, i: int, w: torch.Tensor, fp8: Fp8Weight) -> None:
        """Install an FP8 form made elsewhere (stored codes read from a checkpoint) as the cached form of w as it is now."""
        self._fp8[i] = fp8
        self._key[i] = (w._version, w.data_ptr())

    def clear(self) -> None:
        self._fp8 = [None] * len(self._fp8)
        self._key = [None] * len(self._key)


def invalidate_fp8_caches(module: nn.Module) -> None:
    """`invalidate_fp8_cache()` on every submodule that has one."""
    for m in module.modules():
        f = getattr(m, "invalidate_fp8_cache", None)
        if callable(f):
            f()


def attach_optimizer(optimizer: torch.optim.Optimizer, module: nn.Module):
    """Drop the cached FP8 weights of `module` after every `optimizer.step()`, however that step writes the
    parameters.  Returns the hook handle."""
    return optimizer.register_step_post_hook(lambda *_: invalidate_fp8_caches(module))


class Fp8Linear(nn.Module):
    """Drop-in for torch.nn.Linear (bf16 parameters) whose matmuls run through fp8_linear.

    By default the weight is quantized in every call, which is always right.  ``cache_weight=True`` keeps the
    weight's FP8 form between calls (the micro-batches of one optimizer step, inference): an opt-in, because some
    writes to a parameter cannot be seen from here -- see `_Fp8WeightCache` for when the cached form is refreshed by
    itself and when `invalidate_fp8_cache()` must be called."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, *, recipe: str = "blockwise",
                 cache_weight: bool = False, apply_grad_on_fp32_main_grad: bool = False, device=None,
                 dtype=torch.bfloat16):
        super().__init__()
        self.cache_weight = cache_weight
        self.apply_grad_on_fp32_main_grad = apply_grad_on_fp32_main_grad
        self._cache = _Fp8WeightCache(1)
        if recipe not in RECIPES:
            raise ValueError(f"recipe must be one of {RECIPES}, got {recipe!r}")
        if in_features % ops.BLOCK or out_features % ops.BLOCK:
            raise ValueError("in_features and out_features must be multiples of 128")
        self.in_features, self.out_features, self.recipe = in_features, out_features, recipe
        self.weight = nn.Parameter(torch.empty((out_features, in_features), device=device, dtype=dtype))
        self.bias = nn.Parameter(torch.empty(out_features, device=device, dtype=dtype)) if bias else None
        self.reset_parameters()
        self.register_load_state_dict_post_hook(lambda module, _keys: module.invalidate_fp8_cache())

    def reset_parameters(self) -> None:
        _init_like_nn_linear(self.weight, self.bias)
        self.invalidate_fp8_cache()

    def invalidate_fp8_cache(self) -> None:
        """Forget the cached FP8 form of the weight: the next forward quantizes it again."""
        self._cache.clear()

    @property
    def _fp8(self):
        return self._cache._fp8[0]

    @property
    def _fp8_key(self):
        return self._cache._key[0]

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if not self.cache_weight:
            return fp8_linear(input, self.weight, self.bias, recipe=self.recipe,
                              apply_grad_on_fp32_main_grad=self.apply_grad_on_fp32_main_grad)
        # The FP8 form of the weight is kept until the parameter is written again (optimizer step,
        # load_state_dict, ...): micro-batches of one step and inference calls quantize it once.
        f8 = self._cache.get(0, self.weight, lambda w: quantize_weight(
            w, with_transpose=True, pow2=self.recipe == "blockwise_pow2", per_tensor=self.recipe == "per_tensor"))
        return fp8_linear(input, self.weight, self.bias, recipe=self.recipe, weight_fp8=f8,
                          apply_grad_on_fp32_main_grad=self.apply_grad_on_fp32_main_grad)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.bias is not None}, recipe={self.recipe}")


def quantize_grouped_weight(weight: torch.Tensor, with_transpose: bool = True) -> Fp8Weight:
    """The blockwise FP8 form of the experts' stacked weight [E, N, K]: codes [E, N, K], scale_inv [E, N/128, K/128]
    and (for the input gradient) the transposed codes of the stacked matrix, [K, E * N]."""
    if weight.dim() != 3:
        raise ValueError("weight must be [E, N, K]")
    e, n, k = weight.shape
    flat = weight.reshape(e * n, k)
    if with_transpose:
        wq, sw, wqt = ops.quantize_128x128(flat, with_transpose=True)
    else:
        (wq, sw), wqt = ops.quantize_128x128(flat), None
    return Fp8Weight(wq.view(e, n, k), sw.view(e, n // ops.BLOCK, k // ops.BLOCK), wqt, False)


class _Fp8GroupedLinear(torch.autograd.Function):
    """Grouped (MoE) linear with the blockwise recipe: forward, the input gradient and the weight gradient are one
    grouped GEMM each.  Everything that depends on the rows per expert is derived from `offs` on the device (the
    layout table of the padded token axis the wgrad operands live on), so nothing here reads `offs` on the host and
    forward + backward can be captured in a HIP graph."""

    @staticmethod
    def forward(ctx, x, weight, offs, wq=None, sw=None, wqt=None, grad_mode=True):
        e, n, k = weight.shape
        total_m = x.shape[0]
        need_dx, need_dw = grad_mode and x.requires_grad, grad_mode and weight.requires_grad
        layout = xt = sxt = None
        if need_dw:
            # one read of x: its 1x128 codes for this GEMM and its transposed codes, grouped by expert, for wgrad
            layout = ops.grouped_layout(offs, total_m)
            xq, sx, xt, sxt = ops.quantize_128x1_t_grouped(x.contiguous(), layout, e, with_1x128=True)
        else:
            xq, sx = ops.quantize_1x128(x, kmajor=True)
        if wq is None:                          # no prequantized form of the weight was passed in
            f8 = quantize_grouped_weight(weight, with_transpose=need_dx)
            wq, sw, wqt = f8.codes, f8.scale_inv, f8.codes_t
        elif need_dx and wqt is None:
            wqt = ops.transpose_codes(wq.view(e * n, k))
        y = ops.gemm_grouped_blockwise(xq, sx, wq, sw, offs)
        ctx.save_for_backward(xt, sxt, layout, wqt if need_dx else None, sw, offs)
        ctx.w_shape = weight.shape
        ctx.total_m = total_m
        ctx.need = (need_dx, need_dw)
        return y

    @staticmethod
    def backward(ctx, grad_out):
        xt, sxt, layout, wqt, sw, offs = ctx.saved_tensors
        need_dx, need_dw = ctx.need
        e, n, k = ctx.w_shape
        go = grad_out.to(torch.bfloat16).contiguous()
        dx = dw = None
        goq = sgo = got = sgot = None
        if need_dw:                              # one read of grad_out for both of its operand forms
            out = ops.quantize_128x1_t_grouped(go, layout, e, with_1x128=need_dx)
            (goq, sgo, got, sgot) = out if need_dx else (None, None) + out
        elif need_dx:
            goq, sgo = ops.quantize_1x128(go, kmajor=True)
        if need_dx:
            # dx_e = go_e . W_e: the grouped kernel on the stacked weight's transposed codes (128x128 blocks are
            # symmetric, so W's scales serve with their two block strides swapped); rows of no expert are zeroed
            dx = ops.gemm_grouped_blockwise_t(goq, sgo, wqt, sw, offs)
        if need_dw:
            dw = ops.gemm_grouped_wgrad(got, sgot, xt, sxt, layout, e, ctx.total_m)
        return dx, dw, None, None, None, None, None


def fp8_grouped_linear(input: torch.Tensor, weight: torch.Tensor, offs: torch.Tensor, *,
                       weight_fp8: Optional[Fp8Weight] = None) -> torch.Tensor:
    """MoE grouped linear: rows of input[total_m, K] are sorted by expert, offs[E] are the inclusive int32
    prefix sums of rows per expert (a count may be 0), weight[E, N, K] -> bf16 [total_m, N]; rows past offs[-1]
    are left uninitialised, as torch's grouped matmul leaves them (their input gradient is zero).  Differentiable in
    input and weight (blockwise recipe); neither forward nor backward reads offs on the host.  ``weight_fp8`` is the
    weight's FP8 form made earlier by `quantize_grouped_weight` (e.g. once per optimizer step)."""
    out = _hand_off(fp8_grouped_linear, (input, weight, offs), (input, weight, offs), dict(weight_fp8=weight_fp8),
                    dict(weight_fp8=None))
    if out is not NotImplemented:
        return out
    if input.dim() != 2 or weight.dim() != 3 or input.shape[1] != weight.shape[2]:
        raise ValueError("input must be [total_m, K] and weight [E, N, K]")
    if input.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("input and weight must be bfloat16")
    if offs.numel() != weight.shape[0]:
        raise ValueError(f"offs must have {weight.shape[0]} entries")
    if weight_fp8 is not None:
        if tuple(weight_fp8.codes.shape) != tuple(weight.shape) or weight_fp8.scale_inv.dim() != 3 or weight_fp8.pow2:
            raise ValueError("weight_fp8 must be the blockwise form of this weight (quantize_grouped_weight)")
        return _Fp8GroupedLinear.apply(input, weight, offs, weight_fp8.codes, weight_fp8.scale_inv, weight_fp8.codes_t,
                                       torch.is_grad_enabled())
    return _Fp8GroupedLinear.apply(input, weight, offs, None, None, None, torch.is_grad_enabled())


class _Fp8SwiGLUDown(torch.autograd.Function):
    """y = F.linear(silu(gate) * up, w_down) for h = [gate | up] (blockwise recipe): the activation is computed and
    quantized for the GEMM in one pass over h, which also makes the activation's transposed 128x1 codes for wgrad;
    backward quantizes grad_out once for both of its GEMMs and ends with the gradient of SwiGLU itself."""

    @staticmethod
    def forward(ctx, h, weight, fast=True, wq=None, sw=None, wqt=None):
        h2 = _flatten(h)
        m = h2.shape[0]
        # With a weight gradient to come and a token count that allows it, the gate/up output is read once for
        # both forms of the activation: its 1x128 codes for this GEMM and its transposed 128x1 codes, kept for wgrad.
        fused = weight.requires_grad and m % ops.BLOCK == 0 and m > 0
        if fused:
            aq, sa, at, sat = ops.swiglu_quantize_1x128_and_128x1_t(h2, fast=fast)
        else:
            aq, sa = ops.swiglu_quantize_1x128(h2, kmajor=True, fast=fast)
            at = sat = None
        if wq is None:                          # no prequantized form of the weight was passed in
            if h.requires_grad:
                wq, sw, wqt = ops.quantize_128x128(weight, with_transpose=True)
            else:
                wq, sw = ops.quantize_128x128(weight)
        elif h.requires_grad and wqt is None:
            wqt = ops.transpose_codes(wq)
        y = ops.gemm_blockwise(aq, sa, wq, sw)
        ctx.save_for_backward(h2 if h.requires_grad or (weight.requires_grad and not fused) else None, wqt, sw, at, sat)
        ctx.fast = fast
        ctx.h_shape = h.shape
        ctx.x_shape, ctx.w_shape, ctx.has_bias = h.shape, weight.shape, False
        ctx.need = (h.requires_grad, weight.requires_grad)
        return y.reshape(h.shape[:-1] + (weight.shape[0],))

    @staticmethod
    def backward(ctx, grad_out):
        h2, wqt, sw, at, sat = ctx.saved_tensors
        need_dh, need_dw = ctx.need
        go = _flatten(grad_out)
        if go.dtype != torch.bfloat16:
            go = go.to(torch.bfloat16)
        go = go.contiguous()
        m = go.shape[0]
        if m == 0:
            return _empty_batch_grads(ctx, go)[:2] + (None, None, None, None)
        ragged = m % ops.BLOCK != 0            # wgrad then runs on zero-padded token rows
        dh = dw = None
        goq = sgo = got = sgot = None
        if need_dh and need_dw and not ragged:
            goq, sgo, got, sgot = ops.quantize_1x128_and_128x1_t(go, kmajor=True)
        else:
            if need_dh:
                goq, sgo = ops.quantize_1x128(go, kmajor=True)
            if need_dw:
                got, sgot = ops.quantize_128x1_t(_pad_rows(go), kmajor=True)
        if need_dw:
            if at is None:
                # the activation again (bf16 this time), for its 128x1 codes along the tokens
                _, _, act = ops.swiglu_quantize_1x128(h2, kmajor=True, want_act=True, fast=ctx.fast)
                at, sat = ops.quantize_128x1_t(_pad_rows(act), kmajor=True)
                del act
            dw = ops.gemm_blockwise(got, sgot, at, sat, sb_gran=1)
        if need_dh:
            dact = ops.gemm_blockwise(goq, sgo, wqt, sw.t())
            dh = ops.swiglu_backward(h2, dact).reshape(ctx.h_shape)
        return dh, dw, None, None, None, None


class _Fp8SwiGLUMLPBlock(torch.autograd.Function):
    """The whole block y = F.linear(silu(gate) * up, w_down), gate | up = F.linear(x, w_gate_up), as one autograd node
    (blockwise recipe, both weights trained, token count a multiple of 128).  Every bf16 tensor between the GEMMs is
    read once: x, the gate/up output and grad_out each give both of their operand forms in one pass, and in backward
    the gradient of SwiGLU is quantized for the gate/up projection's two GEMMs as it is computed, so d gate | d up is
    never written in bf16."""

    @staticmethod
    def forward(ctx, x, w_gate_up, w_down, fast, gu8, dn8):
        x2 = _flatten(x).contiguous()
        need_dx = x.requires_grad
        xq, sx, xt, sxt = ops.quantize_1x128_and_128x1_t(x2, kmajor=True)

        def forms(w, f8):
            if f8 is None:
                return ops.quantize_128x128(w, with_transpose=True)
            return f8.codes, f8.scale_inv, f8.codes_t if f8.codes_t is not None else ops.transpose_codes(f8.codes)
        gq, gs, gqt = forms(w_gate_up, gu8)
        dq, ds, dqt = forms(w_down, dn8)
        h = ops.gemm_blockwise(xq, sx, gq, gs)
        aq, sa, at, sat = ops.swiglu_quantize_1x128_and_128x1_t(h, fast=fast)
        y = ops.gemm_blockwise(aq, sa, dq, ds)
        ctx.save_for_backward(h, xt, sxt, gqt if need_dx else None, gs, dqt, ds, at, sat)
        ctx.x_shape, ctx.need_dx = x.shape, need_dx
        return y.reshape(x.shape[:-1] + (w_down.shape[0],))

    @staticmethod
    def backward(ctx, grad_out):
        h, xt, sxt, gqt, gs, dqt, ds, at, sat = ctx.saved_tensors
        go = _flatten(grad_out)
        if go.dtype != torch.bfloat16:
            go = go.to(torch.bfloat16)
        goq, sgo, got, sgot = ops.quantize_1x128_and_128x1_t(go.contiguous(), kmajor=True)
        dw_down = ops.gemm_blockwise(got, sgot, at, sat, sb_gran=1)
        dact = ops.gemm_blockwise(goq, sgo, dqt, ds.t())
        dhq, sdh, dht, sdht = ops.swiglu_backward_quantize_1x128_and_128x1_t(h, dact)
        dx = ops.gemm_blockwise(dhq, sdh, gqt, gs.t()).reshape(ctx.x_shape) if ctx.need_dx else None
        dw_gate_up = ops.gemm_blockwise(dht, sdht, xt, sxt, sb_gran=1)
        return dx, dw_gate_up, dw_down, None, None, None


def fp8_swiglu_mlp(input: torch.Tensor, w_gate_up, w_down, *, fast: bool = True,
                   gate_up_fp8: Optional[Fp8Weight] = None, down_fp8: Optional[Fp8Weight] = None) -> torch.Tensor:
    """A SwiGLU MLP block (DeepSeekV3 dense MLP): ``F.linear(F.silu(gate) * up, w_down)`` with
    ``gate | up = F.linear(input, w_gate_up)`` -- in the reference two aten::linear calls dispatched at
    hyper_parallel/core/shard/_op_dispatch.py:277-283 with eager bf16 elementwise ops between them.  Here the
    activation is computed and quantized for the down projection in one pass over the gate/up output, and
    never exists in bf16 in forward.

    w_gate_up [2I, K] (gate rows first) and w_down [N, I]: bf16 tensors, or `Fp8Weight`s (quantized once,
    e.g. by `quantize_weight(w, with_transpose=False)`) for inference.  With bf16 weights and gradients
    enabled the result carries an autograd graph (blockwise recipe); ``gate_up_fp8`` / ``down_fp8`` are then the
    weights' FP8 forms made earlier by `quantize_weight` (e.g. once per optimizer step for all its micro-batches),
    as `fp8_linear`'s ``weight_fp8``.  ``fast`` selects the SwiGLU kernel that uses the hardware exponential and
    reciprocal."""
    out = _hand_off(fp8_swiglu_mlp, tuple(t for t in (input, w_gate_up, w_down) if isinstance(t, torch.Tensor)),
                    (input, w_gate_up, w_down), dict(fast=fast, gate_up_fp8=gate_up_fp8, down_fp8=down_fp8),
                    _FP8_MLP_DEFAULTS)
    if out is not NotImplemented:
        return out
    fp8_weights = isinstance(w_gate_up, Fp8Weight) or isinstance(w_down, Fp8Weight)
    if not fp8_weights and torch.is_grad_enabled() and (input.requires_grad or w_gate_up.requires_grad or w_down.requires_grad):
        if w_gate_up.shape[0] % (2 * ops.BLOCK) or w_down.shape[1] != w_gate_up.shape[0] // 2:
            raise ValueError("w_gate_up must be [2I, K] with I a multiple of 128 and w_down [N, I]")
        for f8 in (gate_up_fp8, down_fp8):
            if f8 is not None and f8.pow2:
                raise ValueError("the training path of fp8_swiglu_mlp uses the blockwise recipe with plain fp32 scales")
        d8 = down_fp8
        if d8 is not None and d8.codes.shape != w_down.shape:
            raise ValueError("down_fp8 does not belong to w_down")
        if gate_up_fp8 is not None and gate_up_fp8.codes.shape != w_gate_up.shape:
            raise ValueError("gate_up_fp8 does not belong to w_gate_up")
        if input.shape[-1] != w_gate_up.shape[1]:
            raise ValueError(f"input last dim {input.shape[-1]} != w_gate_up in_features {w_gate_up.shape[1]}")
        rows = input.numel() // max(input.shape[-1], 1)
        if (w_gate_up.requires_grad and w_down.requires_grad and rows > 0 and rows % ops.BLOCK == 0
                and input.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and w_down.dtype == torch.bfloat16):
            return _Fp8SwiGLUMLPBlock.apply(input, w_gate_up, w_down, fast, gate_up_fp8, d8)
        h = fp8_linear(input, w_gate_up, weight_fp8=gate_up_fp8)
        return _Fp8SwiGLUDown.apply(h, w_down, fast, *((d8.codes, d8.scale_inv, d8.codes_t) if d8 is not None else ()))
    gu = w_gate_up if isinstance(w_gate_up, Fp8Weight) else (gate_up_fp8 or quantize_weight(w_gate_up.detach(), with_transpose=False))
    dn = w_down if isinstance(w_down, Fp8Weight) else (down_fp8 or quantize_weight(w_down.detach(), with_transpose=False))
    inter = gu.codes.shape[0] // 2
    if gu.codes.shape[0] % (2 * ops.BLOCK) or dn.codes.shape[1] != inter:
        raise ValueError("w_gate_up must be [2I, K] with I a multiple of 128 and w_down [N, I]")
    with torch.no_grad():
        x2 = _flatten(input)
        xq, sx = ops.quantize_1x128(x2, kmajor=True, pow2=gu.pow2)
        # SwiGLU and the quantization of the down projection's input are the gate/up GEMM's epilogue: the gate/up
        # output never exists in bf16
        aq, sa = ops.gemm_blockwise_swiglu_quantize(xq, sx, gu.codes, gu.scale_inv, fast=fast, pow2_scales=gu.pow2,
                                                    pow2_out=dn.pow2)
        y = ops.gemm_blockwise(aq, sa, dn.codes, dn.scale_inv, pow2_scales=dn.pow2)
    return y.reshape(input.shape[:-1] + (dn.codes.shape[0],))


_FP8_MLP_DEFAULTS = dict(fast=True, gate_up_fp8=None, down_fp8=None)


class Fp8SwiGLUMLP(nn.Module):
    """A SwiGLU MLP block with bf16 parameters ``gate_up_proj.weight`` [2 * intermediate, hidden] (gate rows
    first) and ``down_proj.weight`` [hidden, intermediate], computed by `fp8_swiglu_mlp`.  With
    ``cache_weight=True`` it keeps, like `Fp8Linear`, the FP8 forms of its weights until a parameter is written
    again, so the micro-batches of one optimizer step and inference calls quantize them once (the same opt-in
    and the same contract: `_Fp8WeightCache`)."""

    def __init__(self, hidden_size: int, intermediate_size: int, *, fast: bool = True, cache_weight: bool = False,
                 device=None, dtype=torch.bfloat16):
        super().__init__()
        if hidden_size % ops.BLOCK or intermediate_size % ops.BLOCK:
            raise ValueError("hidden_size and intermediate_size must be multiples of 128")
        self.hidden_size, self.intermediate_size, self.fast = hidden_size, intermediate_size, fast
        self.cache_weight = cache_weight
        self.gate_up_proj = nn.Linear(hidden_size, 2 * intermediate_size, bias=False, device=device, dtype=dtype)
        self.down_proj = nn.Linear(intermediate_size, hidden_size, bias=False, device=device, dtype=dtype)
        self._cache = _Fp8WeightCache(2)
        self.register_load_state_dict_post_hook(lambda module, _keys: module.invalidate_fp8_cache())

    def invalidate_fp8_cache(self) -> None:
        """Forget the cached FP8 forms of both weights (see `_Fp8WeightCache` for when this is needed)."""
        self._cache.clear()

    @property
    def _fp8(self):
        return self._cache._fp8

    def _weight_fp8(self, i: int, w: torch.Tensor) -> Fp8Weight:
        return self._cache.get(i, w, lambda t: quantize_weight(t, with_transpose=True))

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        wgu, wd = self.gate_up_proj.weight, self.down_proj.weight
        if not self.cache_weight:
            return fp8_swiglu_mlp(input, wgu, wd, fast=self.fast)
        return fp8_swiglu_mlp(input, wgu, wd, fast=self.fast, gate_up_fp8=self._weight_fp8(0, wgu),
                              down_fp8=self._weight_fp8(1, wd))

    def extra_repr(self) -> str:
        return f"hidden_size={self.hidden_size}, intermediate_size={self.intermediate_size}, fast={self.fast}"
