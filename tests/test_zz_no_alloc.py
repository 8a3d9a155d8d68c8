"""The entry point that allocates nothing, `hpfp8_quantize_per_tensor_noalloc_bf16`, called through the C ABI with
raw pointers: its codes, scale and scale_inv equal those of `hpfp8_quantize_per_tensor_bf16` (the entry point it
is a variant of, whose amax word the caller supplies) bit for bit -- on two calls in a row that share the library's
device memory, the second with a smaller input and a smaller maximum, so that anything the first call left behind
would show."""
import ctypes

import numpy as np
import pytest
import torch

import _util as U

pytestmark = pytest.mark.gpu


def _both(x):
    from hpfp8 import _lib
    n = x.numel()
    stream = torch.cuda.current_stream().cuda_stream
    out = []
    for noalloc in (False, True):
        q = torch.full((n + 64,), 0x55, dtype=torch.uint8, device=x.device)          # (guard bytes past the end)
        scale = torch.full((2,), -1.0, dtype=torch.float32, device=x.device)
        if noalloc:
            _lib.call("hpfp8_quantize_per_tensor_noalloc_bf16", x.data_ptr(), n, q.data_ptr(), scale.data_ptr(),
                      scale.data_ptr() + 4, stream)
        else:
            amax = torch.empty((1,), dtype=torch.float32, device=x.device)
            _lib.call("hpfp8_quantize_per_tensor_bf16", x.data_ptr(), n, q.data_ptr(), amax.data_ptr(), scale.data_ptr(),
                      scale.data_ptr() + 4, stream)
        torch.cuda.synchronize()
        assert bool((q[n:] == 0x55).all())
        out.append((q[:n].cpu().numpy(), scale.cpu().numpy().view(np.uint32)))
    return out


def test_no_alloc_entry_point_equals_the_allocating_one_twice_in_a_row(gpu):
    from hpfp8 import _lib
    from oracle import fp8_oracle as O
    big = (U.randn_bf16((2048, 1024), 5).float() * 7.0).to(torch.bfloat16).to(gpu)          # cfg 1's activation shape
    small = U.randn_bf16((1000 * 3 + 5,), 6, 0.01).to(gpu)                                  # smaller, and a ragged count
    for x in (big, small):
        (q0, s0), (q1, s1) = _both(x.reshape(-1))
        assert np.array_equal(q0, q1) and np.array_equal(s0, s1)
        rq, rs, rsi = O.quantize_per_tensor(U.bits(x.reshape(-1)))
        assert np.array_equal(q1, rq) and s1[0] == U.f32_bits(rs) and s1[1] == U.f32_bits(rsi)
    # beyond its maximum the entry point refuses, and says so
    lib = _lib.load()
    rc = lib.hpfp8_quantize_per_tensor_noalloc_bf16(big.data_ptr(), 4 * 1024 * 1024 + 8, big.data_ptr(), None, None, None)
    assert rc == -2 and b"exceed the maximum" in lib.hpfp8_last_error()
