"""Stand-ins for the two reference classes the dispatcher plugin derives from and builds, so that the plugin file
can be EXECUTED where hyper_parallel is not installed.  Test infrastructure only.

They restate the interface the plugin touches, nothing more:
  * `Layout` -- hyper_parallel/core/layout.py:142-157 (constructor), :187-242 (calling a layout with alias names
    gives a copy whose `alias_tensor_map` is those names and whose numeric `tensor_map` counts mesh axes from the
    right, "None" = -1, an axis used twice is an error), :244-255 (`to_dict`), :433-441 (`set_partial_by_dev_axis`
    refuses an axis that shards a tensor dim), and the read-only properties `mesh_shape`, `alias_name`, `rank_list`,
    `partial`.
  * `DistributedOp` -- hyper_parallel/core/shard/ops/parallel_ops.py:23-84: constructed with the operator name,
    which registers the instance; `infer_layout` / `get_expand_impl` are what subclasses override.
"""
import copy
import sys
import types

REGISTRY = {}


class Layout:
    def __init__(self, mesh_shape, alias_name, rank_list=None, init_backend=True):
        if len(mesh_shape) != len(alias_name):
            raise ValueError("mesh_shape and alias_name must have the same length")
        self.mesh_shape, self.alias_name = tuple(mesh_shape), tuple(alias_name)
        n = 1
        for s in mesh_shape:
            n *= s
        self.rank_list = tuple(rank_list) if rank_list else tuple(range(n))
        self.partial = [None] * len(mesh_shape)
        self.alias_tensor_map = None
        self.tensor_map = None

    def __call__(self, *alias_tensor_map):
        obj = copy.deepcopy(self)
        used, tmap = [], ()

        def one(a):
            if a == "None":
                return -1
            if a not in obj.alias_name:
                raise ValueError(f"The axis {a} is not found in {obj.alias_name}")
            if a in used:
                raise ValueError(f"The axis {a} has been set more than one in {obj.alias_name}")
            used.append(a)
            return len(obj.alias_name) - 1 - obj.alias_name.index(a)

        for e in alias_tensor_map:
            tmap += (tuple(one(a) for a in e),) if isinstance(e, tuple) else (one(e),)
        obj.alias_tensor_map, obj.tensor_map = tuple(alias_tensor_map), tmap
        return obj

    def to_dict(self):
        return {"mesh_shape": self.mesh_shape, "tensor_map": self.tensor_map, "alias_name": self.alias_name,
                "rank_list": self.rank_list}

    def set_partial_by_dev_axis(self, axis, op):
        flat = [a for e in (self.alias_tensor_map or ()) for a in (e if isinstance(e, tuple) else (e,))]
        if axis in flat:
            raise ValueError("Partial dim must be replicate.")
        self.partial[self.alias_name.index(axis)] = op

    def is_partial(self):
        return any(p is not None for p in self.partial)


class DistributedOp:
    def __init__(self, op_name):
        self.op_name = op_name
        REGISTRY[op_name] = self

    def infer_layout(self, layouts, extra_args):
        return (layouts[0],) if layouts else None

    def get_expand_impl(self, func, output_layout, layouts, extra_args):
        return None


def install():
    """Put the stand-ins where the plugin imports the reference classes from; returns the names to remove again."""
    names = ["hyper_parallel", "hyper_parallel.core", "hyper_parallel.core.layout", "hyper_parallel.core.shard",
             "hyper_parallel.core.shard.ops", "hyper_parallel.core.shard.ops.parallel_ops"]
    if "hyper_parallel" in sys.modules:
        raise RuntimeError("a real hyper_parallel is imported; the stand-in must not shadow it")
    for n in names:
        sys.modules[n] = types.ModuleType(n)
    sys.modules["hyper_parallel.core.layout"].Layout = Layout
    sys.modules["hyper_parallel.core.shard.ops.parallel_ops"].DistributedOp = DistributedOp
    return names


def uninstall(names):
    for n in names:
        sys.modules.pop(n, None)
