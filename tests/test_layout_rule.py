"""Layout rule of the fp8_linear dispatcher plugin, on the reference's own expectations.

The expected tensor maps and partial lists below are the ones asserted for `LinearDistributedOp` in
the reference's tests/mindspore/ut/parallel_ops_infer/test_parallel_linear.py (mesh (2, 4), axes
("dp", "mp")): data-parallel :31-43, hybrid :46-60, hybrid tensor parallel :63-78, partial with a
sharded contraction :94-110.  Two further cases of that file (:80-92 and :113-128) contradict the
reference's code (parallel_matmul.py:376-381 rejects unequal contraction layouts, and accepts an
unsharded bias next to an unsharded weight dim 0); the rule here follows the code.
"""
import importlib.util
import os

import pytest

_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "hyper-parallel_amd", "hpfp8", "plugin",
                     "layout_rule.py")
_spec = importlib.util.spec_from_file_location("hpfp8_layout_rule", _path)
R = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(R)

MESH, NAMES = (2, 4), ("dp", "mp")


def _partial_list(axes):
    return ["sum" if n in axes else None for n in NAMES]


@pytest.mark.parametrize("x,w,b,want_map,want_partial", [
    (("dp", "None"), ("None", "None"), None, (1, -1), [None, None]),        # data parallel
    (("dp", "None"), ("mp", "None"), ("mp",), (1, 0), [None, None]),        # hybrid dp + mp
    (("dp", "mp"), ("None", "mp"), None, (1, -1), [None, "sum"]),           # sharded contraction -> Partial(sum)
    # not in the reference's file: a 3-D input and tuple entries, same rule (leading dims pass through)
    (("None", "dp", ("mp",)), ("None", ("mp",)), None, (-1, 1, -1), [None, "sum"]),
])
def test_expected_maps_of_the_reference_tests(x, w, b, want_map, want_partial):
    out_map, partial_axes = R.infer_fp8_linear_map(x, w, b)
    assert R.alias_to_tensor_map(out_map, NAMES) == want_map
    assert _partial_list(partial_axes) == want_partial


def test_rejections_follow_the_reference_code():
    with pytest.raises(ValueError, match="Contracting"):
        R.infer_fp8_linear_map(("dp", "None"), ("None", "mp"), None)
    with pytest.raises(ValueError, match="Output dimensions"):
        R.infer_fp8_linear_map(("dp", "None"), ("mp", "None"), ("None",))
    with pytest.raises(ValueError, match="replicate"):           # contraction axis also shards an output dim
        R.infer_fp8_linear_map(("mp", "mp"), ("None", "mp"), None)


def test_bias_divisor_and_alignment():
    assert R.bias_divisor(("dp", "mp"), MESH, NAMES) == 4
    assert R.bias_divisor(("dp", ("dp", "mp")), MESH, NAMES) == 8
    assert R.bias_divisor(("dp", "None"), MESH, NAMES) == 1
    # cfg 2's weight [36864, 7168] split 4 ways along dim 0 keeps whole blocks; 7168 / 8 = 896 = 7 * 128 too
    R.check_fp8_shard_alignment((36864, 7168), ("mp", "None"), MESH, NAMES, dims=(0, 1))
    R.check_fp8_shard_alignment((36864, 7168), ("None", ("dp", "mp")), MESH, NAMES, dims=(0, 1))
    with pytest.raises(ValueError, match="multiple of 128"):
        R.check_fp8_shard_alignment((36864, 1152), ("None", "mp"), MESH, NAMES, dims=(1,))   # 1152 / 4 = 288
