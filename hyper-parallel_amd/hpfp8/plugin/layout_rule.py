"""Layout rule of fp8_linear on alias tensor maps, free of any hyper_parallel import.

A tensor's layout is written the way the reference writes it: one entry per tensor dim, each the
name of the mesh axis that shards the dim, a tuple of names, or "None"
(hyper_parallel/core/layout.py:202-234).  This module restates the rule of the reference's
`LinearDistributedOp.infer_layout` / `get_expand_impl`
(hyper_parallel/core/shard/ops/parallel_matmul.py:342-429) on that representation, and adds the
one constraint FP8 brings: every local shard must keep whole 1x128 groups and 128x128 blocks.
`parallel_fp8_linear.Fp8LinearDistributedOp` wraps it in the reference's Layout objects.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

BLOCK = 128


def _axes(entry) -> Tuple[str, ...]:
    if entry == "None":
        return ()
    return tuple(entry) if isinstance(entry, tuple) else (entry,)


def infer_fp8_linear_map(x_map: Sequence, w_map: Sequence, bias_map: Optional[Sequence]):
    """(alias map of the output, mesh axes along which the output is a partial sum).

    Same checks, same order and same messages' meaning as parallel_matmul.py:376-406: the contraction
    dims (last dim of x and of w) must be sharded alike; the output takes x's leading dims and w's
    dim 0; a bias must be sharded like w's dim 0; a sharded contraction makes the output
    Partial(sum) along those axes.
    """
    x_map, w_map = tuple(x_map), tuple(w_map)
    if not x_map or not w_map:
        raise ValueError(f"x_layout : {x_map}, w_layout : {w_map}")
    if x_map[-1] != w_map[-1]:
        raise ValueError(f"Contracting dimensions must have same layout. Got {x_map[-1]} and {w_map[-1]}")
    if bias_map is not None and tuple(bias_map)[0] != w_map[0]:
        raise ValueError(f"Output dimensions must have same sharding. Got weight output dim sharding: {w_map[0]} "
                         f"and bias output dim sharding: {tuple(bias_map)[0]}")
    out_map = x_map[:-1] + (w_map[0],)
    partial_axes = _axes(x_map[-1])
    used = [a for entry in out_map for a in _axes(entry)]
    for a in partial_axes:                      # layout.py:437-438: a partial axis must not also shard a dim
        if a in used:
            raise ValueError("Partial dim must be replicate.")
    return out_map, partial_axes


def bias_divisor(x_map: Sequence, mesh_shape: Sequence[int], alias_name: Sequence[str]) -> int:
    """What the bias is divided by before the local call so that the later all-reduce(sum) adds it once
    (parallel_matmul.py:408-429): the number of devices along the contraction's mesh axes."""
    f = 1
    for a in _axes(tuple(x_map)[-1]):
        f *= int(mesh_shape[list(alias_name).index(a)])
    return f


def alias_to_tensor_map(alias_map: Sequence, alias_name: Sequence[str]):
    """The numeric tensor map of `Layout.to_dict()` (layout.py:205-234): mesh axis i of n maps to
    n - 1 - i, "None" to -1."""
    n = len(alias_name)

    def one(a):
        return -1 if a == "None" else n - 1 - list(alias_name).index(a)

    return tuple(tuple(one(a) for a in e) if isinstance(e, tuple) else one(e) for e in alias_map)


def check_fp8_shard_alignment(global_shape: Sequence[int], alias_map: Sequence, mesh_shape: Sequence[int],
                              alias_name: Sequence[str], dims: Sequence[int]) -> None:
    """Raise unless every listed dim, after sharding, is still a multiple of 128 (so that no scaling
    group or block straddles two ranks)."""
    for d in dims:
        ways = 1
        for a in _axes(tuple(alias_map)[d]):
            ways *= int(mesh_shape[list(alias_name).index(a)])
        size = int(global_shape[d])
        if size % ways or (size // ways) % BLOCK:
            raise ValueError(f"fp8_linear: dim {d} of size {size} sharded {ways} ways leaves local size "
                             f"{size / ways:g}, not a multiple of {BLOCK}")
