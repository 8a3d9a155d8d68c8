"""Layout rule that lets hyper_parallel dispatch `fp8_linear` on DTensors.

It mirrors the reference's rule for `linear`
(hyper_parallel/core/shard/ops/parallel_matmul.py:342-429): output layout = input's batch dims +
weight's dim 0; a sharded contraction dim marks the output Partial(sum) and pre-divides the bias by
the number of shards.  FP8 adds one constraint the caller must meet: shard boundaries along both
weight dims and along the contraction dim must be multiples of 128, so that no 1x128 group or
128x128 block straddles two ranks (the kernels reject other shapes).

This module imports hyper_parallel and is only loaded by hyper_parallel's own dispatcher; the hpfp8
package never imports it.
"""
import os
import sys

from hyper_parallel.core.layout import Layout
from hyper_parallel.core.shard.ops.parallel_ops import DistributedOp

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from layout_rule import bias_divisor, infer_fp8_linear_map  # noqa: E402  (same directory, loaded by file path)


class Fp8LinearDistributedOp(DistributedOp):
    """Distributed implementation for fp8_linear(input, weight, bias)."""

    def infer_layout(self, layouts, extra_args):
        if len(layouts) != 3:
            raise ValueError(f"fp8_linear layout length is not 3, but {len(layouts)}")
        x_layout, w_layout, bias_layout = layouts
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
        x_layout = layouts[0]
        factor = bias_divisor(x_layout.alias_tensor_map, x_layout.mesh_shape, x_layout.alias_name)
        if factor == 1 or not layouts[2]:
            return None

        def expand_impl(x, w, bias):
            return func(x, w, bias / factor)

        return expand_impl
