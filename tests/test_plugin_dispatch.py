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
