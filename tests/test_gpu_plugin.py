"""The dispatcher-level drop-in end to end on the GPU: a distributed tensor's `__torch_function__` hook receives
`fp8_linear`, the registered rule infers the output layout, its expand wrapper pre-divides the bias and calls the
real `fp8_linear` on this rank's local shards -- the route of hyper_parallel/platform/torch/dtensor.py:50-62 ->
hyper_parallel/core/shard/_op_dispatch.py:634-673, :245-298 -> hyper_parallel/core/shard/ops/parallel_matmul.py:406-429,
driven by the stand-in dispatcher of tests/_hp_standin.py (hyper_parallel itself is not installed here).  The local
result is checked against the oracle's blockwise GEMM on the same local shards with bias / 4."""
import sys

import numpy as np
import pytest
import torch

from oracle import fp8_oracle as O
import _hp_standin as HP
import _util as U

pytestmark = pytest.mark.gpu


@pytest.fixture
def dispatcher():
    from hpfp8.plugin import install
    names = HP.install()
    try:
        disp = HP.Dispatcher()
        install.register(disp)
        HP.DTensor.DISPATCHER = disp
        yield disp
    finally:
        HP.DTensor.DISPATCHER = None
        HP.uninstall(names)
        HP.REGISTRY.pop("fp8_linear", None)
        for n in ("hpfp8.plugin.parallel_fp8_linear", "hpfp8.plugin.layout_rule"):
            sys.modules.pop(n, None)


MESH = HP.Layout((2, 4), ("dp", "mp"), list(range(8)))


def test_contraction_sharded_four_ways_through_the_plugin(gpu, dispatcher):
    import hpfp8
    m, n, k, ways = 256, 384, 2048, 4
    x = U.randn_bf16((m, k), 21, 1.0, 0.001, 50.0)
    w = U.randn_bf16((n, k), 22, 0.02)
    bias = U.randn_bf16((n,), 23, 0.5)
    kl = k // ways
    total = np.zeros((m // 2, n), dtype=np.float64)
    for r in range(ways):                         # mesh coordinate along "mp"; "dp" coordinate 0
        xl = x[: m // 2, r * kl:(r + 1) * kl].contiguous()
        wl = w[:, r * kl:(r + 1) * kl].contiguous()
        xd = HP.DTensor(xl.to(gpu), MESH("dp", "mp"))
        wd = HP.DTensor(wl.to(gpu), MESH("None", "mp"))
        bd = HP.DTensor(bias.to(gpu), MESH("None"))
        dispatcher.seen.clear()
        y = hpfp8.fp8_linear(xd, wd, bd)
        # the hook saw exactly one operator, under the name the YAML registers
        assert dispatcher.seen == ["fp8_linear"]
        assert isinstance(y, HP.DTensor)
        assert y.layout.to_dict()["tensor_map"] == (1, -1) and y.layout.partial == [None, "sum"]
        local = y.to_local()
        assert type(local) is torch.Tensor and local.shape == (m // 2, n) and local.dtype == torch.bfloat16
        # the oracle on the same local shards, bias divided by the number of shards of the contraction; the
        # division is the wrapper's bf16 tensor division (parallel_matmul.py:423: `bias / scaling_factor`)
        xq, _, sxi = O.quantize_1x128(U.bits(xl))
        wq, _, swi = O.quantize_128x128(U.bits(wl))
        b4 = (bias / ways).float().numpy()
        want, want_bits = O.gemm_blockwise(xq, sxi, wq, swi, b4)
        got = local.float().cpu().numpy()
        assert np.linalg.norm(got - want) / np.linalg.norm(want) < 3e-3
        diff = np.abs(U.bits(local).astype(np.int32) - want_bits.astype(np.int32))
        assert (diff != 0).mean() < 3e-2            # the last bf16 bit, where the matrix instruction's sum order shows
        total += got.astype(np.float64)
    # what the all-reduce(sum) of the four partial outputs gives: the full linear, the bias added once
    ref = x[: m // 2].double().numpy() @ w.double().numpy().T + bias.double().numpy()
    assert np.linalg.norm(total - ref) / np.linalg.norm(ref) < 0.05


def test_keywords_and_column_parallel_through_the_plugin(gpu, dispatcher):
    import hpfp8
    m, n, k = 128, 512, 256
    x = U.randn_bf16((m, k), 31)
    w = U.randn_bf16((n, k), 32, 0.02)
    bias = U.randn_bf16((n,), 33, 0.5)
    nl = n // 4
    wl, bl = w[nl:2 * nl].contiguous(), bias[nl:2 * nl].contiguous()
    f8 = hpfp8.quantize_weight(wl.to(gpu), per_tensor=True)
    xd = HP.DTensor(x.to(gpu), MESH("dp", "None"))
    wd = HP.DTensor(wl.to(gpu), MESH("mp", "None"))
    bd = HP.DTensor(bl.to(gpu), MESH("mp"))
    y = hpfp8.fp8_linear(xd, wd, bd, recipe="per_tensor", weight_fp8=f8)
    assert dispatcher.seen[-1] == "fp8_linear" and y.layout.to_dict()["tensor_map"] == (1, 0)
    assert y.layout.partial == [None, None]
    xq, _, sxi = O.quantize_per_tensor(U.bits(x))
    wq, _, swi = O.quantize_per_tensor(U.bits(wl))
    want, _ = O.gemm_per_tensor(xq, sxi, wq, swi, bl.float().numpy())       # nothing sharded along k: bias as it is
    got = y.to_local().float().cpu().numpy()
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 3e-3
    # a shard that would split a 128-wide group is refused before any kernel runs
    with pytest.raises(ValueError, match="whole 128x128 blocks"):
        hpfp8.fp8_linear(HP.DTensor(x[:, :192].contiguous().to(gpu), MESH("dp", "mp")),
                         HP.DTensor(w[:, :192].contiguous().to(gpu), MESH("None", "mp")), None)
    # a distributed weight with a plain local input: the hook still gets the call, and the rule refuses the
    # input without a layout the way the reference's rule does (parallel_matmul.py:368-369)
    with pytest.raises(ValueError, match="x_layout"):
        hpfp8.fp8_linear(x.to(gpu), wd, None)
