"""Layout rule that lets hyper_parallel dispatch `fp8_linear` on DTensors.

It mirrors the reference's rule for `linear`
(hyper_parallel/core/shard/ops/parallel_matmul.py:342-429): output layout = input's batch dims +
weight's dim 0; a sharded contraction dim marks the output Partial(sum) and pre-divides the bias by
the number of shards.  FP8 adds one constraint the caller must meet: shard boundaries along both
weight dims and along the contraction dim must be multiples of 128, so that no 1x128 group or
128x128 block straddles two ranks (the kernels reject other shapes).

This module imports hyper_parallel and is only loaded by hyper_parallel's own dispatcher; the hpfp8
package never imports it.  The dispatcher finds it either as a top-level module (`distributed_op_file`, with
HYPER_PARALLEL_OPS_PYTHON_PATH naming this directory, which the dispatcher itself puts on sys.path:
hyper_parallel/core/shard/_op_dispatch.py:140-146, :176-186) or as `hpfp8.plugin.parallel_fp8_linear`
(`distributed_op_module`); the sibling module with the rule is imported accordingly.
"""
from hyper_parallel.core.layout import Layout
from hyper_parallel.core.shard.ops.parallel_ops import DistributedOp

if __package__:
    from .layout_rule import BLOCK, bias_divisor, infer_fp8_linear_map
else:
    from layout_rule import BLOCK, bias_divisor, infer_fp8_linear_map


def check_local_shapes(x, w) -> None:
    """The FP8 constraint on what one rank holds: the local contraction dim and the local output dim are whole
    multiples of 128, so that no 1x128 group or 128x128 block straddles two ranks."""
    k, n = int(w.shape[-1]), int(w.shape[0])
    if int(x.shape[-1]) != k:
        raise ValueError(f"fp8_linear: local contraction dims differ: input {int(x.shape[-1])}, weight {k}")
    if k % BLOCK or n % BLOCK:
        raise ValueError(f"fp8_linear: the local weight shard [{n}, {k}] does not hold whole 128x128 blocks; "
                         f"shard boundaries must be multiples of {BLOCK}")


class Fp8LinearDistributedOp(DistributedOp):
    """Distributed implementation for fp8_linear(input, weight, bias)."""

    def infer_layout(self, layouts, extra_args):
        # (input, weight, bias) always arrive positionally; the dispatcher appends one entry per keyword argument
        # (hyper_parallel/core/shard/_op_dispatch.py:224-241), and fp8_linear's keywords (recipe, weight_fp8,
        # apply_grad_on_fp32_main_grad) are not tensors, so their entries carry no layout.
        if len(layouts) < 3:
            raise ValueError(f"fp8_linear layout length is not 3, but {len(layouts)}")
        if any(extra is not None for extra in layouts[3:]):
            raise ValueError("fp8_linear takes three tensors (input, weight, bias); its keyword arguments are not "
                             "distributed tensors")
        x_layout, w_layout, bias_layout = layouts[:3]
        if not x_layout or not w_layout:
            raise ValueError(f"x_layout : {x_layout}, w_layout : {w_layout}")
        if x_layout.mesh_shape != w_layout.mesh_shape:
            raise ValueError("fp8_linear inputs must have same mesh_shape")
        if bias_layout and bias_layout.mesh_shape != x_layout.mesh_shape:
            raise ValueError("fp8_linear bias and x must have same mesh_shape")
        out_map, partial_axes = infer_fp8_linear_map(
            x_layout.alias_tensor_map, w_layout.alias_tensor_map,
            bias_layout.alias_tensor_map if bias_layout else None)
        out = Layout(mesh_shape=x_layout.mesh_shape, alias_name=x_layout.alias_name, rank_list=x_layout.rank_list)
        out = out(*out_map)
        for axis in partial_axes:
            out.set_partial_by_dev_axis(axis, "sum")
        return out

    def get_expand_impl(self, func, output_layout, layouts, extra_args):
        """Always a wrapper (the reference's linear returns None when there is nothing to rescale): the local
        shards are checked against the 128 alignment before the kernels see them, and with a sharded contraction
        the bias is pre-divided so that the all-reduce(sum) of the partial outputs adds it once."""
        x_layout = layouts[0]
        factor = bias_divisor(x_layout.alias_tensor_map, x_layout.mesh_shape, x_layout.alias_name)
        rescale = factor != 1 and bool(layouts[2])

        def expand_impl(x, w, bias=None, **kwargs):
            check_local_shapes(x, w)
            return func(x, w, bias / factor if rescale and bias is not None else bias, **kwargs)

        return expand_impl
