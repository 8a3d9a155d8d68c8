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
  * `DTensor` and `Dispatcher` -- the route of one operator call: `DTensorBase.__torch_function__`
    (hyper_parallel/platform/torch/dtensor.py:50-62) hands (func, args, kwargs) to `OpDispatcher.dispatch`
    (hyper_parallel/core/shard/_op_dispatch.py:634-673): name = `func.__name__`
    (hyper_parallel/platform/torch/platform.py:159-174); whitelisted names run on the unwrapped tensors; a name without
    a registered rule raises RuntimeError; otherwise `_with_layout_infer` (:245-298, argument handling :190-243):
    positional tensors with a layout are replaced by their local tensors, everything else goes to `extra_args`, every
    keyword adds one (layout or None) entry, `infer_layout(layouts, extra_args)` gives the output layout,
    `get_expand_impl(func, output_layout, layouts, extra_args)` an optional wrapper, the (wrapper or) function runs on
    the local tensors and the result is wrapped with the output layout.  `layout_infer_ops` /
    `_register_single_distributed_op` (:148-186) are the two members a late registration uses.
"""
import copy
import importlib
import sys
import types

import torch

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


class DTensor(torch.Tensor):
    """A local tensor plus a layout, whose operator calls all go to DISPATCHER (set by the test)."""
    DISPATCHER = None

    @staticmethod
    def __new__(cls, local, layout):
        t = torch.Tensor._make_subclass(cls, local, local.requires_grad)
        t._local_tensor, t._layout = local, layout
        return t

    @property
    def layout(self):
        return self._layout

    def to_local(self):
        return self._local_tensor

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        return cls.DISPATCHER.dispatch(func, args, kwargs or {})


class Dispatcher:
    WHITELIST = ("__get__", "__set__", "dim", "__len__", "__bool__", "__format__", "item", "requires_grad_")

    def __init__(self):
        self.layout_infer_ops = {}
        self.seen = []                                  # operator names in the order they arrived

    def _register_single_distributed_op(self, op_name, config):
        mod = importlib.import_module(config["distributed_op_module"] if "distributed_op_module" in config
                                      else config["distributed_op_file"])
        getattr(mod, config["distributed_op_class"])(op_name)

    def dispatch(self, func, args, kwargs):
        name = func.__name__ if hasattr(func, "__name__") else str(func)
        self.seen.append(name)
        if name in self.WHITELIST:
            with torch._C.DisableTorchFunctionSubclass():
                return func(*[a.to_local() if isinstance(a, DTensor) else a for a in args], **kwargs)
        if name not in self.layout_infer_ops:
            raise RuntimeError(f"Operator {name} dose not contain parallel layout infer func.")
        layouts, extra, local_args, local_kwargs = [], [], [], dict(kwargs)
        for a in args:
            if a is None or not hasattr(a, "_layout"):
                layouts.append(None)
                local_args.append(a)
                if a is not None:
                    extra.append(a)
                    str(a)                              # the reference's cache key prints every such argument
            else:
                layouts.append(a.layout)
                local_args.append(a.to_local())
        for k, v in kwargs.items():
            if v is None or not hasattr(v, "_layout"):
                layouts.append(None)
                if v is not None:
                    extra.append(v)
                    str(v)
            else:
                layouts.append(v.layout)
                local_kwargs[k] = v.to_local()
        op = REGISTRY[name]
        out_layout = op.infer_layout(layouts, extra)
        impl = op.get_expand_impl(func, out_layout, layouts, extra) or func
        return DTensor(impl(*local_args, **local_kwargs), out_layout)


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
