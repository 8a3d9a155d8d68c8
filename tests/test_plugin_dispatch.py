"""The dispatcher plugin file itself, executed: loaded the two ways the reference's dispatcher loads a
user operator (hyper_parallel/core/shard/_op_dispatch.py:153-186: `distributed_op_file` imported as a top-level
module from HYPER_PARALLEL_OPS_PYTHON_PATH, or `distributed_op_module`), registered under the YAML's name, and run
on the reference's own expected layouts (tests/mindspore/ut/parallel_ops_infer/test_parallel_linear.py:31-110) with
stand-ins for the two reference classes it builds on (tests/_hp_standin.py).  No GPU is touched: the local
function the wrapper calls is a recorder."""
import importlib
import os
import sys

import pytest
import yaml

import _hp_standin as HP

PLUGIN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "hyper-parallel_amd", "hpfp8", "plugin")


class _T:
    def __init__(self, *shape):
        self.shape = shape

    def __truediv__(self, f):
        t = _T(*self.shape)
        t.divided_by = f
        return t


@pytest.fixture(params=["file", "module"])
def op(request):
    names = HP.install()
    cfg = yaml.safe_load(open(os.path.join(PLUGIN_DIR, "fp8_linear_ops.yaml")))["fp8_linear"]
    added = None
    try:
        if request.param == "file":
            added = os.path.abspath(PLUGIN_DIR)
            sys.path.insert(0, added)               # what _extend_sys_path does with HYPER_PARALLEL_OPS_PYTHON_PATH
            mod = importlib.import_module(cfg["distributed_op_file"])
        else:
            mod = importlib.import_module("hpfp8.plugin." + cfg["distributed_op_file"])
        inst = getattr(mod, cfg["distributed_op_class"])("fp8_linear")
        assert HP.REGISTRY["fp8_linear"] is inst
        yield inst
    finally:
        HP.uninstall(names)
        for n in (cfg["distributed_op_file"], "layout_rule", "hpfp8.plugin." + cfg["distributed_op_file"]):
            sys.modules.pop(n, None)
        if added:
            sys.path.remove(added)


LAYOUT = HP.Layout((2, 4), ("dp", "mp"), list(range(8)))


def test_infer_layout_on_the_reference_expectations(op):
    out = op.infer_layout((LAYOUT("dp", "None"), LAYOUT("None", "None"), None), ())
    assert out.to_dict()["tensor_map"] == (1, -1) and out.partial == [None, None]
    out = op.infer_layout((LAYOUT("dp", "None"), LAYOUT("mp", "None"), LAYOUT("mp")), ())
    assert out.to_dict()["tensor_map"] == (1, 0)
    out = op.infer_layout((LAYOUT("dp", "mp"), LAYOUT("None", "mp"), None), ())
    assert out.to_dict()["tensor_map"] == (1, -1) and out.partial == [None, "sum"]
    with pytest.raises(ValueError, match="length is not 3"):
        op.infer_layout((LAYOUT("dp", "None"), LAYOUT("None", "None")), ())
    with pytest.raises(ValueError, match="Contracting"):
        op.infer_layout((LAYOUT("dp", "None"), LAYOUT("None", "mp"), None), ())
    with pytest.raises(ValueError, match="same mesh_shape"):
        op.infer_layout((LAYOUT("dp", "None"), HP.Layout((4, 2), ("dp", "mp"))("None", "None"), None), ())


def test_expand_wrapper_checks_alignment_and_rescales_the_bias(op):
    calls = []

    def local_fp8_linear(x, w, bias=None):
        calls.append((x, w, bias))
        return "y"

    # contraction sharded 4 ways, bias present: bias / 4 before the local call, shapes checked
    layouts = (LAYOUT("dp", "mp"), LAYOUT("None", "mp"), LAYOUT("None"))
    out_layout = op.infer_layout((layouts[0], layouts[1], None), ())
    f = op.get_expand_impl(local_fp8_linear, out_layout, layouts, ())
    assert f(_T(2048, 1792), _T(36864, 1792), _T(36864)) == "y"
    assert calls[-1][2].divided_by == 4
    with pytest.raises(ValueError, match="whole 128x128 blocks"):
        f(_T(2048, 288), _T(36864, 288), _T(36864))            # 1152 / 4: a 1x128 group would straddle two ranks
    with pytest.raises(ValueError, match="contraction dims differ"):
        f(_T(2048, 256), _T(36864, 128), None)
    # nothing sharded along the contraction: the bias passes through untouched, the check still runs
    layouts = (LAYOUT("dp", "None"), LAYOUT("mp", "None"), LAYOUT("mp"))
    f = op.get_expand_impl(local_fp8_linear, op.infer_layout(layouts, ()), layouts, ())
    b = _T(9216)
    f(_T(2048, 7168), _T(9216, 7168), b)
    assert calls[-1][2] is b
    with pytest.raises(ValueError, match="whole 128x128 blocks"):
        f(_T(2048, 7168), _T(9216 // 8 - 64, 7168), None)
    assert len(calls) == 2


# ---- the hand-off: does the reference's interception point ever see `fp8_linear`? -------------------------------

class _Recording(__import__("torch").Tensor):
    """A tensor subclass whose `__torch_function__` records what it is handed, like the reference's DTensor hook
    (hyper_parallel/platform/torch/dtensor.py:50-62), and answers with a marker."""
    calls = []

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        cls.calls.append((func, args, kwargs or {}))
        return "handled"


def _rec(*shape):
    import torch
    return torch.zeros(shape, dtype=torch.bfloat16).as_subclass(_Recording)


def test_fp8_linear_offers_itself_to_torch_function():
    import torch
    import hpfp8
    _Recording.calls.clear()
    x, w, b = _rec(4, 256), _rec(128, 256), _rec(128)
    assert hpfp8.fp8_linear(x, w, b) == "handled"
    func, args, kwargs = _Recording.calls[-1]
    # the registry key the reference derives (hyper_parallel/platform/torch/platform.py:159-174)
    assert func is hpfp8.fp8_linear and func.__name__ == "fp8_linear"
    assert len(args) == 3 and args[0] is x and args[1] is w and args[2] is b
    assert kwargs == {}                       # defaults are not passed on: the hook sees F.linear's three arguments
    # no bias: still three positional arguments, the third None (what LinearDistributedOp expects, parallel_matmul.py:361)
    assert hpfp8.fp8_linear(x, w) == "handled"
    assert _Recording.calls[-1][1][2] is None and len(_Recording.calls[-1][1]) == 3
    # keyword arguments that differ from their defaults travel as keywords
    f8 = hpfp8.Fp8Weight(torch.zeros(128, 256), torch.zeros(1, 2), None)
    assert hpfp8.fp8_linear(x, w, None, recipe="per_tensor", weight_fp8=f8, apply_grad_on_fp32_main_grad=True) == "handled"
    assert _Recording.calls[-1][2] == {"recipe": "per_tensor", "weight_fp8": f8, "apply_grad_on_fp32_main_grad": True}
    # one subclass argument is enough (a plain input against a distributed weight)
    assert hpfp8.fp8_linear(torch.zeros(4, 256, dtype=torch.bfloat16), w) == "handled"
    assert len(_Recording.calls) == 4 and all(c[0] is hpfp8.fp8_linear for c in _Recording.calls)


def test_grouped_and_mlp_offer_themselves_too():
    import torch
    import hpfp8
    _Recording.calls.clear()
    offs = torch.zeros(2, dtype=torch.int32)
    assert hpfp8.fp8_grouped_linear(_rec(8, 128), _rec(2, 128, 128), offs) == "handled"
    assert _Recording.calls[-1][0].__name__ == "fp8_grouped_linear" and _Recording.calls[-1][2] == {}
    assert hpfp8.fp8_swiglu_mlp(_rec(8, 128), _rec(256, 128), _rec(128, 128), fast=False) == "handled"
    assert _Recording.calls[-1][0].__name__ == "fp8_swiglu_mlp" and _Recording.calls[-1][2] == {"fast": False}


def test_fp8_weight_prints_no_tensor_values():
    import torch
    import hpfp8
    f8 = hpfp8.Fp8Weight(torch.arange(6.0).reshape(2, 3), torch.ones(1, 1), None, True)
    s = str(f8)
    assert "(2, 3)@0x" in s and "pow2=True" in s and "tensor(" not in s and "codes_t=None" in s


# ---- registration without losing the built-in operators ---------------------------------------------------------

def _fake_package(tmp_path):
    """A directory tree shaped like an installed hyper_parallel: two built-in YAML files where the dispatcher looks."""
    d = tmp_path / "site" / "hyper_parallel" / "core" / "shard" / "ops" / "yaml"
    d.mkdir(parents=True)
    (d / "torch_mm.yaml").write_text("linear:\n  dist_op_name: _linear\n  distributed_op_class: LinearDistributedOp\n"
                                     "  distributed_op_file: parallel_matmul\n")
    (d / "elementwise.yaml").write_text("__default__:\n  distributed_op_file: parallel_elementwise\nadd:\n"
                                        "  dist_op_name: _add\n  distributed_op_class: ElementWiseDistributedOp\n")
    return str(tmp_path / "site" / "hyper_parallel")


def test_merged_yaml_directory_keeps_the_builtin_operators(tmp_path):
    from hpfp8.plugin import install
    pkg = _fake_package(tmp_path)
    env = {"HYPER_PARALLEL_OPS_PYTHON_PATH": "/somewhere/else"}
    d = install.prepare_env(str(tmp_path / "merged"), hyper_parallel_dir=pkg, environ=env)
    assert env["HYPER_PARALLEL_OPS_YAML_DIR"] == d and os.path.isabs(d)
    assert env["HYPER_PARALLEL_OPS_PYTHON_PATH"].split(":") == ["/somewhere/else", install.PLUGIN_DIR]
    # what safe_load_yaml_from_dir (_op_dispatch.py:613-632) would read from that directory
    names = {}
    for f in sorted(os.listdir(d)):
        assert f.endswith(".yaml")
        for k, v in yaml.safe_load(open(os.path.join(d, f))).items():
            assert k not in names
            names[k] = v
    assert {"linear", "add", "fp8_linear"} <= set(names)
    assert names["fp8_linear"]["distributed_op_file"] == "parallel_fp8_linear"
    assert os.path.exists(os.path.join(install.PLUGIN_DIR, names["fp8_linear"]["distributed_op_file"] + ".py"))
    # a built-in file that already defines fp8_linear is an error here, as it would be in the dispatcher
    (tmp_path / "site" / "hyper_parallel" / "core" / "shard" / "ops" / "yaml" / "x.yaml").write_text(
        "fp8_linear:\n  dist_op_name: other\n")
    with pytest.raises(ValueError, match="already defines"):
        install.merged_yaml_dir(str(tmp_path / "merged2"), hyper_parallel_dir=pkg)
    with pytest.raises(FileNotFoundError):
        install.builtin_yaml_dir(str(tmp_path))


def test_register_on_a_live_dispatcher():
    from hpfp8.plugin import install
    names = HP.install()
    try:
        disp = HP.Dispatcher()
        disp.layout_infer_ops["linear"] = {"dist_op_name": "_linear"}
        install.register(disp)
        assert set(disp.layout_infer_ops) == {"linear", "fp8_linear"}          # nothing else was touched
        assert disp.layout_infer_ops["fp8_linear"]["distributed_op_module"] == "hpfp8.plugin.parallel_fp8_linear"
        assert type(HP.REGISTRY["fp8_linear"]).__name__ == "Fp8LinearDistributedOp"
        install.register(disp)                                                  # idempotent
        # an operator that is not registered still fails the reference's way
        HP.DTensor.DISPATCHER = disp
        import torch
        t = HP.DTensor(torch.zeros(2, 2), LAYOUT("None", "None"))
        with pytest.raises(RuntimeError, match="dose not contain parallel layout infer func"):
            torch.add(t, t)
    finally:
        HP.uninstall(names)
        HP.REGISTRY.pop("fp8_linear", None)
        sys.modules.pop("hpfp8.plugin.parallel_fp8_linear", None)
        sys.modules.pop("hpfp8.plugin.layout_rule", None)


def test_keyword_arguments_add_layout_entries_without_layout(op):
    """The dispatcher appends one entry per keyword (None for a non-tensor); the rule reads the first three."""
    out = op.infer_layout([LAYOUT("dp", "mp"), LAYOUT("None", "mp"), None, None, None], ["per_tensor", True])
    assert out.to_dict()["tensor_map"] == (1, -1) and out.partial == [None, "sum"]
    with pytest.raises(ValueError, match="keyword arguments are not distributed"):
        op.infer_layout([LAYOUT("dp", "mp"), LAYOUT("None", "mp"), None, LAYOUT("None")], [])
    seen = {}

    def local(x, w, bias=None, **kw):
        seen.update(kw)
        return "y"
    layouts = [LAYOUT("dp", "None"), LAYOUT("None", "None"), None, None]
    f = op.get_expand_impl(local, op.infer_layout(layouts, ["per_tensor"]), layouts, ["per_tensor"])
    assert f(_T(4, 128), _T(128, 128), None, recipe="per_tensor") == "y" and seen == {"recipe": "per_tensor"}
