"""Benchmark of the FP8 linear hot path on one MI355X.

A step is one blockwise-FP8 forward of the DeepSeekV3 dense-MLP gate/up projection
(x[4096,7168] bf16 with 0.1% x50 outliers, W[36864,7168] bf16 ~ N(0,0.006)):
    quantize x 1x128  ->  quantize W 128x128  ->  scaled FP8 GEMM (fp32 accumulation, bf16 out)
with all inputs resident in HBM when the clock starts and every kernel launched through the C ABI
on preallocated buffers.  One JSON line is printed:

    value      = 2*M*N*K / step time, TFLOP/s (whole step, quantizers included)
    roofline   = the dominant kernel (the GEMM) alone, timed with HIP events on its stream
    quantize   = the HBM-bound kernels alone, GB/s of algorithmic bytes, same timing method
    cpu_baseline = the CPU oracle's C restatement on a bounded sample of the same workload

    other_configs = the kernels of configurations 1, 3, 4 and 5, each with its own roofline fraction

Usage: python bench.py [--gpus 1] [--steps 50] [--warmup 50] [--all] [--headline-only] [--no-cpu-baseline]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "hyper-parallel_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

M, N, K = 4096, 36864, 7168
PEAK_FP8_TFLOPS = 5000.0     # MI355X dense FP8 MFMA
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E
# Bytes per GEMM launch that crossed the L2 <-> memory-fabric boundary come from rocprofv3 --pmc runs (FETCH_SIZE,
# calibrated on a copy of known size, + WRITE_SIZE; and the requests among them destined for the memory controller)
# whose summary is kept in PROFILE together with the sha256 of the kernel source it was measured on; the figure is
# only reported while csrc/gemm.hip is still that source (otherwise `traffic` is null, with a line on stderr, until
# the counters are collected again).
PROFILE = os.path.join(ROOT, "profiles", "bench_cfg2_gemm_blockwise_and_quantizers.md")
GEMM_SOURCE = os.path.join(ROOT, "hyper-parallel_amd", "csrc", "gemm.hip")


def gemm_source_digest(path=GEMM_SOURCE):
    """sha256 of csrc/gemm.hip: the profile summary records the digest of the source its counters were collected on."""
    import hashlib
    with open(path, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()


def gemm_traffic_bytes():
    """({"tcc_ea": bytes per launch across the L2 <-> fabric boundary, "dram_path": bytes of those requests that were
    destined for the memory controller} or None, the reason).  None -- and a loud line on stderr -- when the profile
    summary is absent or was collected on another version of the kernel source: a stale figure is not reported."""
    import re
    try:
        text = open(PROFILE).read()
    except OSError:
        return None, "no profile summary"
    m = re.search(r"traffic_bytes=(\d+)\s+dram_path_bytes=(\d+)\s+gemm_source_sha256=([0-9a-f]{64})", text)
    if not m:
        return None, "profile summary has no traffic line"
    if m.group(3) != gemm_source_digest():
        why = ("profiles/%s was collected on another version of csrc/gemm.hip (its digest %s..., the source's %s...): "
               "collect FETCH_SIZE / WRITE_SIZE again" % (os.path.basename(PROFILE), m.group(3)[:12], gemm_source_digest()[:12]))
        print("bench.py: STALE TRAFFIC FIGURE NOT REPORTED: " + why, file=sys.stderr, flush=True)
        return None, why
    return {"tcc_ea": int(m.group(1)), "dram_path": int(m.group(2))}, "profiles/" + os.path.basename(PROFILE)


def cpu_draw(gen, shape, kind="randn", chunk=1 << 26):
    """fp32 values from the CPU generator `gen`, drawn in row chunks (bounded host memory), as one fp32 CPU tensor."""
    import torch
    fn = torch.randn if kind == "randn" else torch.rand
    rows = shape[0]
    per = max(1, chunk // max(1, int(torch.Size(shape[1:]).numel())))
    parts = [fn((min(per, rows - r),) + tuple(shape[1:]), generator=gen, dtype=torch.float32) for r in range(0, rows, per)]
    return parts[0] if len(parts) == 1 else torch.cat(parts)


def make_inputs(dev):
    """cfg 2's tensors, drawn with torch.Generator('cpu').manual_seed(0) in fp32, in this order -- x = randn(M, K), the
    outlier positions randperm(M * K)[:k], W = randn(N, K) * 0.006 -- then cast to bf16 and copied to the device, so a
    CPU run and a GPU run of the configuration see identical bytes."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(0)
    x = cpu_draw(g, (M, K))
    k = round(0.001 * M * K)
    idx = torch.randperm(M * K, generator=g)[:k]
    x.view(-1)[idx] *= 50.0
    x = x.to(torch.bfloat16)
    w = (cpu_draw(g, (N, K)) * 0.006).to(torch.bfloat16)
    return x.to(dev), w.to(dev)


def event_ms(pairs):
    return [s.elapsed_time(e) for s, e in pairs]


def cpu_baseline(x_bits, w_bits, target_seconds=15.0):
    """The C restatement of the oracle (OpenMP over the host cores) on a bounded sample of the same
    step: quantize all of W (128x128), quantize the first `ms` rows of x (1x128), scaled GEMM of those
    rows against all of W.  The whole-step time is extrapolated linearly in the row count."""
    import numpy as np
    from oracle import c_oracle as C
    threads = C.num_threads()
    t0 = time.perf_counter()
    wq, _, swi = C.quantize_128x128(w_bits)
    t_qw = time.perf_counter() - t0
    xq8, _, sxi8 = C.quantize_1x128(np.ascontiguousarray(x_bits[:8]))
    t0 = time.perf_counter()
    C.gemm_blockwise(xq8, sxi8, wq, swi)
    t8 = max(time.perf_counter() - t0, 1e-6)
    ms = int(min(x_bits.shape[0], max(8, (target_seconds - t_qw) / t8 * 8))) // 8 * 8
    ms = max(ms, 8)
    xs = np.ascontiguousarray(x_bits[:ms])
    t0 = time.perf_counter()
    xq, _, sxi = C.quantize_1x128(xs)
    t_qx = time.perf_counter() - t0
    t0 = time.perf_counter()
    C.gemm_blockwise(xq, sxi, wq, swi)
    t_g = time.perf_counter() - t0
    step_seconds = t_qw + (t_qx + t_g) * (M / ms)
    # beside it, what the reference executes on a CPU today for this layer: aten::linear in bf16
    # (hyper_parallel/core/shard/_op_dispatch.py:283), on as many of the first rows as take about 3 s
    import torch
    import torch.nn.functional as F
    torch.set_num_threads(threads)
    xt = torch.from_numpy(np.ascontiguousarray(x_bits).view(np.int16)).view(torch.bfloat16)
    wt = torch.from_numpy(w_bits.view(np.int16)).view(torch.bfloat16)
    F.linear(xt[:64], wt)
    t0 = time.perf_counter()
    F.linear(xt[:64], wt)
    t64 = max(time.perf_counter() - t0, 1e-6)
    xt = xt[:max(64, min(xt.shape[0], int(3.0 / t64) * 64))]          # about 3 s of work
    t0 = time.perf_counter()
    F.linear(xt, wt)
    t_lin = max(time.perf_counter() - t0, 1e-6)
    return {
        "value": 2.0 * M * N * K / step_seconds / 1e12,
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"quantize W[{N},{K}] ({t_qw:.1f} s) + quantize x[:{ms}] ({t_qx:.2f} s) + scaled GEMM of those "
                  f"{ms} rows against all of W ({t_g:.1f} s), {threads} OpenMP threads; whole step extrapolated "
                  f"linearly in rows to {step_seconds:.0f} s",
        "aten_linear_bf16_on_cpu": {"value": 2.0 * xt.shape[0] * N * K / t_lin / 1e12, "unit": "TFLOP/s", "cores": threads,
                                    "sample": f"F.linear(x[:{xt.shape[0]}], W) in bf16, {t_lin:.2f} s"},
    }


def cpu_baselines_other_configs():
    """The CPU legs of configurations 1, 3, 4 and 5 (host cores of this box, the oracle's C restatement with OpenMP;
    cfg 1 also torch._scaled_mm on CPU): cfg 1 at full size, median of 5; the others on a bounded sample of the same
    distribution with the factor to the full configuration stated; and, for cfg 5, what the reference does at that
    site today: the dtype round trip bf16 -> reduce_dtype -> bf16 of
    hyper_parallel/core/hsdp/hsdp_grad_buffer.py:105-106 and :121-122 (torch on CPU, reduce_dtype = float32)."""
    import numpy as np
    import torch
    from oracle import c_oracle as C
    from oracle import fp8_oracle as O
    threads = C.num_threads()
    torch.set_num_threads(threads)
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
    res = {"cores": threads}

    def median_of(fn, n=5):
        ts = []
        for _ in range(n):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2]

    # cfg 1, full size, the tensors of the GPU run (CPU generator, seed 0)
    g = torch.Generator(device="cpu").manual_seed(0)
    x = cpu_draw(g, (2048, 1024)).to(torch.bfloat16)
    w = (cpu_draw(g, (1024, 1024)) * 0.02).to(torch.bfloat16)
    xb, wb = bits(x), bits(w)
    fl1 = 2.0 * 2048 * 1024 * 1024

    def oracle_step():
        xq, _, sx = C.quantize_per_tensor(xb)
        wq, _, sw = C.quantize_per_tensor(wb)
        return O.gemm_per_tensor(xq, sx, wq, sw)
    t_or = median_of(oracle_step)
    xq, _, sx = C.quantize_per_tensor(xb)
    wq, _, sw = C.quantize_per_tensor(wb)
    F8 = torch.float8_e4m3fn
    xa, wa = torch.from_numpy(xq).view(F8), torch.from_numpy(wq).view(F8)
    sxt, swt = torch.tensor(float(sx)), torch.tensor(float(sw))
    c1 = {"oracle_quantize_x_quantize_w_gemm": {"ms": t_or * 1e3, "TFLOP/s": fl1 / t_or / 1e12, "sample": "full size, median of 5"}}
    try:
        # (torch's CPU routine for float8 operands takes about 10 s for the full 2048 rows: a quarter of them, x 4)
        xa4 = xa[:512]
        t_sm = median_of(lambda: torch._scaled_mm(xa4, wa.t(), scale_a=sxt, scale_b=swt, out_dtype=torch.bfloat16)) * 4
        c1["torch_scaled_mm_gemm_only"] = {"ms": t_sm * 1e3, "TFLOP/s": fl1 / t_sm / 1e12,
                                           "sample": "512 of 2048 rows, median of 5, x 4"}
    except Exception as err:          # (not in every CPU build of torch)
        c1["torch_scaled_mm_gemm_only"] = f"unavailable: {type(err).__name__}"
    xg_, wg_ = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    go_ = torch.ones((2048, 1024), dtype=torch.bfloat16)

    def lin_fwd_bwd():
        torch.nn.functional.linear(xg_, wg_).backward(go_)
        xg_.grad = wg_.grad = None
    t_bf = median_of(lin_fwd_bwd)
    c1["aten_linear_bf16_forward_backward"] = {"ms": t_bf * 1e3, "TFLOP/s": 3 * fl1 / t_bf / 1e12, "sample": "full size, median of 5"}
    res["cfg1_per_tensor"] = c1

    # cfg 3 (M 4096, N 7168, K 16384): dgrad on the first 256 token rows (x 16), wgrad on the first 1024 columns of x (x 16)
    g = torch.Generator(device="cpu").manual_seed(0)
    m, n, k, ms_, ks_ = 4096, 7168, 16384, 256, 1024
    xs = bits(cpu_draw(g, (m, ks_)).to(torch.bfloat16))
    u = cpu_draw(g, (m, n), kind="rand") - 0.5
    go = bits((-(2 ** -0.5) * torch.sign(u) * torch.log1p(-2 * u.abs().clamp(max=0.4999999)) * 1e-3).to(torch.bfloat16))
    wt = bits((cpu_draw(g, (k, n)) * 0.006).to(torch.bfloat16))          # W^T [K, N], drawn directly in that layout
    t0 = time.perf_counter()
    wtq, _, swt_ = C.quantize_128x128(wt)
    t_qw = time.perf_counter() - t0
    t0 = time.perf_counter()
    goq, _, sgo = C.quantize_1x128(np.ascontiguousarray(go[:ms_]))
    C.gemm_blockwise(goq, sgo, wtq, swt_)
    t_d = time.perf_counter() - t0
    t0 = time.perf_counter()
    got, _, sgot = C.quantize_128x1_t(go)
    xt, _, sxt_ = C.quantize_128x1_t(xs)
    t_q = time.perf_counter() - t0
    t0 = time.perf_counter()
    C.gemm_blockwise(got, sgot, xt, sxt_, sb_per_row=True)
    t_w = time.perf_counter() - t0
    fl3 = 2.0 * m * n * k
    res["cfg3_backward"] = {
        "dgrad": {"TFLOP/s": fl3 / (t_d * m / ms_) / 1e12, "sample": f"quantize + GEMM of {ms_} of {m} token rows ({t_d:.1f} s), x {m // ms_}"},
        "wgrad": {"TFLOP/s": fl3 / (t_w * k / ks_) / 1e12, "sample": f"GEMM on {ks_} of {k} columns of x ({t_w:.1f} s), x {k // ks_}"},
        "requant_t_GB/s": (m * n + m * ks_) * 3 / t_q / 1e9,
        "quantize_w_128x128_GB/s": k * n * 3 / t_qw / 1e9,
    }
    del wt, wtq, go, got, xs, xt

    # cfg 4: 512 rows of one expert against that expert's weight [4096, 7168] (131072 rows in all: x 256)
    g = torch.Generator(device="cpu").manual_seed(0)
    we = bits((cpu_draw(g, (4096, 7168)) * 0.006).to(torch.bfloat16))
    xe = bits(cpu_draw(g, (512, 7168)).to(torch.bfloat16))
    weq, _, swe = C.quantize_128x128(we)
    t0 = time.perf_counter()
    xeq, _, sxe = C.quantize_1x128(xe)
    C.gemm_blockwise(xeq, sxe, weq, swe)
    t_e = time.perf_counter() - t0
    res["cfg4_moe_grouped"] = {"forward": {"TFLOP/s": 2.0 * 512 * 4096 * 7168 / t_e / 1e12,
                                           "sample": f"quantize + GEMM of 512 rows of one expert ({t_e:.1f} s), x 256 for the 131072 routed rows"}}
    del we, weq

    # cfg 5: 2^25 of the 2^29 elements (x 16); and the reference's own cast round trip at this site on 2^27 (x 4)
    nel = 1 << 25
    flat = bits((torch.randn(nel, generator=g) * 1e-4).to(torch.bfloat16)).reshape(-1, 128)
    t0 = time.perf_counter()
    cq, _, csi = C.quantize_1x128(flat)
    t_q5 = time.perf_counter() - t0
    t0 = time.perf_counter()
    C.dequantize_1x128(cq, csi)
    t_d5 = time.perf_counter() - t0
    nb5 = nel * 3 + nel // 128 * 4
    big = (torch.randn(1 << 27, generator=g) * 1e-4).to(torch.bfloat16)
    t0 = time.perf_counter()
    back = big.to(torch.float32).to(torch.bfloat16)
    t_rt = time.perf_counter() - t0
    res["cfg5_bucket"] = {
        "quantize_GB/s": nb5 / t_q5 / 1e9, "dequantize_GB/s": nb5 / t_d5 / 1e9,
        "sample": f"2^25 of 2^29 elements (x 16): {t_q5:.2f} s + {t_d5:.2f} s",
        "reference_cast_round_trip_bf16_fp32_bf16": {"GB/s": (1 << 27) * 12 / t_rt / 1e9,
                                                     "sample": f"torch on CPU, 2^27 of 2^29 elements (x 4): {t_rt:.2f} s; 2 + 4 bytes "
                                                               "per element cast in, 4 + 2 cast back"},
    }
    del back, big
    return res


def _time(fn, iters=30, warm=40):
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s0.record()
    for _ in range(iters):
        fn()
    s1.record()
    torch.cuda.synchronize()
    return s0.elapsed_time(s1) / iters


CACHE_BYTES = 256 << 20         # the Infinity Cache between the L2s and HBM


def _n_sets(bytes_per_set):
    """How many copies of a kernel's buffers to rotate through so that a launch finds none of its data in the
    Infinity Cache: the copies together hold more than 2.5 times its size."""
    return max(2, int(2.5 * CACHE_BYTES // max(1, bytes_per_set)) + 1)


def _time_rot(launch, nsets, iters=30, warm=40):
    """Like _time for launch(i), which must use buffer set i % nsets."""
    import torch
    for i in range(warm):
        launch(i % nsets)
    torch.cuda.synchronize()
    s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s0.record()
    for i in range(iters):
        launch(i % nsets)
    s1.record()
    torch.cuda.synchronize()
    return s0.elapsed_time(s1) / iters


def quantizer_rows(src, dev, prefix="", iters=30, warm=40):
    """Every quantizer form of one bf16 source [m, k] through the C ABI on preallocated buffers that rotate beyond the
    Infinity Cache (source copies and outputs alike): {name: {ms, GB/s, frac_hbm}}."""
    import torch
    from hpfp8 import _lib
    from hpfp8.ops import _padded_ld
    m, k = src.shape
    FP8 = torch.float8_e4m3fn
    st = torch.cuda.current_stream().cuda_stream
    ld_t = _padded_ld(m)
    n = _n_sets(m * k * 4)
    xs = [src] + [src.clone() for _ in range(n - 1)]
    q = [torch.empty((m, k), dtype=FP8, device=dev) for _ in range(n)]
    qt = [torch.empty((k, ld_t), dtype=FP8, device=dev) for _ in range(n)]
    s1 = torch.empty((k // 128, m), dtype=torch.float32, device=dev)
    s2 = torch.empty((m // 128, k), dtype=torch.float32, device=dev)
    part = torch.empty((m // 128, k), dtype=torch.float32, device=dev)
    db = torch.empty((k,), dtype=torch.bfloat16, device=dev)
    P = lambda t: t.data_ptr()
    sc = m * k // 128 * 4
    out = {}
    T = lambda fn: _time_rot(fn, n, iters=iters, warm=warm)
    out[prefix + "quantize_1x128"] = _gb(m * k * 3 + sc, T(lambda i: _lib.call(
        "hpfp8_quantize_1x128_kmajor_bf16", P(xs[i]), m, k, P(q[i]), None, P(s1), st)))
    out[prefix + "requant_t"] = _gb(m * k * 3 + sc, T(lambda i: _lib.call(
        "hpfp8_quantize_128x1_t_kmajor_bf16", P(xs[i]), m, k, P(qt[i]), ld_t, None, P(s2), st)))
    out[prefix + "quantize_both_forms"] = _gb(m * k * 4 + 2 * sc, T(lambda i: _lib.call(
        "hpfp8_quantize_1x128_and_128x1_t_bf16", P(xs[i]), m, k, 1, P(q[i]), None, P(s1), P(qt[i]), ld_t, None, P(s2), st)))

    def with_bias(i):
        _lib.call("hpfp8_quantize_128x1_t_colsum_bf16", P(xs[i]), m, k, P(q[i]), None, P(s1), P(qt[i]), ld_t, None, P(s2), 0,
                  P(part), st)
        _lib.call("hpfp8_column_sum_finish", P(part), m // 128, k, P(db), None, st)
    out[prefix + "quantize_both_forms_and_bias_gradient"] = dict(
        _gb(m * k * 4 + 3 * sc, T(with_bias)), note="two launches: the quantizer, then the sum over the 128-row blocks")
    # what the two transposing access patterns allow on this machine: the same loads and stores with nothing between them
    out[prefix + "requant_t_traffic_model"] = _gb(m * k * 3, T(lambda i: _lib.call(
        "hpfp8_debug_transpose_traffic_model", P(xs[i]), m, k, P(qt[i]), ld_t, None, st)))
    out[prefix + "quantize_both_forms_traffic_model"] = _gb(m * k * 4, T(lambda i: _lib.call(
        "hpfp8_debug_transpose_traffic_model", P(xs[i]), m, k, P(qt[i]), ld_t, P(q[i]), st)))
    return out


def _tf(flops, ms):
    return {"ms": ms, "TFLOP/s": flops / ms / 1e9, "frac_mfma": flops / ms / 1e9 / PEAK_FP8_TFLOPS}


def _gb(nbytes, ms):
    return {"ms": ms, "GB/s": nbytes / ms / 1e6, "frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBS}


def zipf_counts(experts, total, seed=0):
    """Rows per expert of configuration 4: multinomial over p_e ~ rank^-1.1 (seeded permutation of the experts), the
    two least popular experts emptied into the most popular one."""
    import torch
    gc = torch.Generator(device="cpu").manual_seed(seed)
    perm = torch.randperm(experts, generator=gc)
    pz = (torch.arange(1, experts + 1, dtype=torch.float64) ** -1.1)[perm]
    pz = pz / pz.sum()
    counts = torch.multinomial(pz, total, replacement=True, generator=gc).bincount(minlength=experts)
    order = torch.argsort(pz)
    for z in order[:2]:
        counts[order[-1]] += counts[z]
        counts[z] = 0
    return counts


def other_configs_compact(dev):
    """The other four benchmark configurations, each kernel with its own roofline fraction (HIP events around
    back-to-back launches after a warm-up): cfg 1 per-tensor quantize + GEMM, cfg 3 backward GEMMs and transposed
    requantizers, cfg 4 MoE grouped GEMMs and the whole grouped layer, cfg 5 bucket quantize / dequantize.  Every
    HBM-bound kernel whose tensors would fit the Infinity Cache runs on buffers that rotate beyond it.  cfg 1 and 3
    are drawn with the CPU generator (seed 0, one generator per configuration, tensors in the order listed in the
    benchmark's description); cfg 4's 2.4e9 and cfg 5's 5.4e8 values are drawn on the GPU (same distributions, seed
    0), where they take a second instead of a minute."""
    import torch
    import hpfp8
    from hpfp8 import ops
    res = {"data_generator": {"cfg1": "cpu seed 0", "cfg2": "cpu seed 0", "cfg3": "cpu seed 0",
                              "cfg4": "gpu seed 0 (deviation: 2.4e9 values)", "cfg5": "gpu seed 0 (deviation: 5.4e8 values)"}}
    g = torch.Generator(device=dev).manual_seed(0)
    # cfg 1: per-tensor linear 2048 x 1024 x 1024 (launch-bound: times include the launches)
    g1 = torch.Generator(device="cpu").manual_seed(0)
    x = cpu_draw(g1, (2048, 1024)).to(torch.bfloat16).to(dev)
    w = (cpu_draw(g1, (1024, 1024)) * 0.02).to(torch.bfloat16).to(dev)
    xq, _, sx = hpfp8.quantize_per_tensor(x)
    wq, _, sw = hpfp8.quantize_per_tensor(w)
    # (timed through the C ABI with outputs allocated beforehand: at this size the Python wrappers' allocations
    # would be most of the time; 64 copies of x and of its codes, 384 MB, so that no launch finds its data in a cache)
    from hpfp8 import _lib
    st = torch.cuda.current_stream().cuda_stream
    n1 = 64
    x1 = [x] + [x.clone() for _ in range(n1 - 1)]
    q1 = [torch.empty((2048, 1024), dtype=torch.uint8, device=dev) for _ in range(n1)]
    xq1 = [xq] + [xq.clone() for _ in range(n1 - 1)]
    w3 = torch.zeros(3, dtype=torch.float32, device=dev)
    c1 = [torch.empty((2048, 1024), dtype=torch.bfloat16, device=dev) for _ in range(n1)]
    pw = w3.data_ptr()
    sync = torch.zeros(128, dtype=torch.int32, device=dev)
    quant = lambda i: _lib.call("hpfp8_quantize_per_tensor_sync_bf16", x1[i].data_ptr(), x.numel(), q1[i].data_ptr(), pw, pw + 4,
                                pw + 8, sync.data_ptr(), st)
    gemm = lambda i: _lib.call("hpfp8_gemm_per_tensor", xq1[i].data_ptr(), 1024, sx.data_ptr(), wq.data_ptr(), 1024, sw.data_ptr(),
                               2048, 1024, 1024, None, c1[i].data_ptr(), 1024, 0, st)
    t_q = _time_rot(quant, n1, iters=200, warm=100)
    t_g = _time_rot(gemm, n1, iters=200, warm=100)
    t_both = _time_rot(lambda i: (quant(i), gemm(i)), n1, iters=200, warm=100)
    res["cfg1_per_tensor"] = {"quantize_x": _gb(x.numel() * 3, t_q), "gemm": _tf(2.0 * 2048 * 1024 * 1024, t_g),
                              "quantize_x_plus_gemm_us": t_both * 1e3,
                              "note": "launch-bound: two launches (one-pass amax + cast, 128 x 128-tile GEMM), times "
                                      "include the launches; buffers rotate over 64 copies"}
    del x, w, xq, wq, q1, c1, x1, xq1
    # cfg 2's layer as an inference MLP block: the gate/up GEMM with SwiGLU + the 1x128 quantizer as its epilogue
    # (no bf16 gate/up tensor), then the down projection
    x = torch.randn((4096, 7168), generator=g, device=dev).to(torch.bfloat16)
    gu = hpfp8.quantize_weight((torch.randn((36864, 7168), generator=g, device=dev) * 0.006).to(torch.bfloat16), with_transpose=False)
    dn = hpfp8.quantize_weight((torch.randn((7168, 18432), generator=g, device=dev) * 0.006).to(torch.bfloat16), with_transpose=False)
    xq, sx = hpfp8.quantize_1x128(x, kmajor=True)
    fl_gu, fl_mlp = 2.0 * 4096 * 36864 * 7168, 2.0 * 4096 * 7168 * (36864 + 18432)
    with torch.no_grad():
        res["cfg2_mlp_inference"] = {
            "gate_up_gemm_with_swiglu_quantize_epilogue": _tf(fl_gu, _time(
                lambda: ops.gemm_blockwise_swiglu_quantize(xq, sx, gu.codes, gu.scale_inv, fast=True), iters=20)),
            "block_forward": _tf(fl_mlp, _time(lambda: hpfp8.fp8_swiglu_mlp(x, gu, dn, fast=True), iters=20)),
        }
    # for orientation, on the same codes: this library's block-scaled kernel beside the vendor library's FP8 GEMMs
    # (one scale per tensor; one scale per row of each operand, its finest scaling here)
    one = torch.ones((), dtype=torch.float32, device=dev)
    orient = {"this_library_blockwise": _tf(fl_gu, _time(lambda: ops.gemm_blockwise(xq, sx, gu.codes, gu.scale_inv), iters=20))}
    try:
        orient["vendor_per_tensor"] = _tf(fl_gu, _time(lambda: torch._scaled_mm(
            xq, gu.codes.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16), iters=20))
        ra, rb = torch.ones((4096, 1), device=dev), torch.ones((1, 36864), device=dev)
        orient["vendor_rowwise"] = _tf(fl_gu, _time(lambda: torch._scaled_mm(
            xq, gu.codes.t(), scale_a=ra, scale_b=rb, out_dtype=torch.bfloat16), iters=20))
    except Exception as err:          # (absent or differently named in another torch build)
        orient["vendor"] = f"unavailable: {type(err).__name__}"
    res["cfg2_gemm_beside_vendor_library"] = orient
    del x, gu, dn, xq, sx
    torch.cuda.empty_cache()
    # cfg 3: o_proj backward, M = 4096 tokens, W[7168, 16384]
    m, n, k = 4096, 7168, 16384
    g3 = torch.Generator(device="cpu").manual_seed(0)
    x = cpu_draw(g3, (m, k)).to(torch.bfloat16).to(dev)
    u = cpu_draw(g3, (m, n), kind="rand") - 0.5
    go = (-(2 ** -0.5) * torch.sign(u) * torch.log1p(-2 * u.abs().clamp(max=0.4999999)) * 1e-3).to(torch.bfloat16).to(dev)
    w = (cpu_draw(g3, (n, k)) * 0.006).to(torch.bfloat16).to(dev)
    del u
    wq, sw, wqt = hpfp8.quantize_128x128(w, with_transpose=True)
    goq, sgo = hpfp8.quantize_1x128(go, kmajor=True)
    got, sgot = hpfp8.quantize_128x1_t(go, kmajor=True)
    xt, sxt = hpfp8.quantize_128x1_t(x, kmajor=True)
    fl = 2.0 * m * n * k
    main_grad = torch.zeros((n, k), dtype=torch.float32, device=dev)
    r3 = {
        "dgrad_gemm": _tf(fl, _time(lambda: hpfp8.gemm_blockwise(goq, sgo, wqt, sw.t()))),
        "wgrad_gemm": _tf(fl, _time(lambda: hpfp8.gemm_blockwise(got, sgot, xt, sxt, sb_gran=1))),
        "wgrad_gemm_into_fp32_main_grad": _tf(fl, _time(
            lambda: hpfp8.gemm_blockwise(got, sgot, xt, sxt, sb_gran=1, out=main_grad, accumulate=True))),
    }
    del main_grad, wq, wqt, goq, got, xt
    torch.cuda.empty_cache()
    r3.update(quantizer_rows(x, dev, "x_"))
    r3.update(quantizer_rows(go, dev, "grad_out_"))
    # the weight with its transposed codes (470 MB per launch: beyond the cache by itself; two sets all the same)
    from hpfp8.ops import _padded_ld
    ldw = _padded_ld(n)
    ws = [w, w.clone()]
    wqs = [torch.empty((n, k), dtype=torch.float8_e4m3fn, device=dev) for _ in range(2)]
    wts = [torch.empty((k, ldw), dtype=torch.float8_e4m3fn, device=dev) for _ in range(2)]
    sws = torch.empty((n // 128, k // 128), dtype=torch.float32, device=dev)
    r3["quantize_w_with_transpose"] = _gb(n * k * 4 + (n // 128) * (k // 128) * 4, _time_rot(lambda i: _lib.call(
        "hpfp8_quantize_128x128_bf16", ws[i].data_ptr(), n, k, wqs[i].data_ptr(), wts[i].data_ptr(), ldw, None, sws.data_ptr(), st), 2))
    r3["note"] = "quantizer rows: source copies and outputs rotate over more than 640 MB (Infinity Cache: 256 MB)"
    res["cfg3_backward"] = r3
    del x, go, w, ws, wqs, wts
    torch.cuda.empty_cache()
    # cfg 4: MoE grouped, 32 experts, 131072 routed rows, Zipf(1.1) counts, two empty experts
    e, n, k, total = 32, 4096, 7168, 131072
    counts = zipf_counts(e, total)
    offs = counts.cumsum(0).to(torch.int32).to(dev)
    xg4 = torch.randn((total, k), generator=g, device=dev).to(torch.bfloat16).requires_grad_(True)
    wg4 = (torch.randn((e, n, k), generator=g, device=dev) * 0.006).to(torch.bfloat16).requires_grad_(True)
    go4 = (torch.randn((total, n), generator=g, device=dev) * 1e-3).to(torch.bfloat16)
    layout = ops.grouped_layout(offs, total)
    xq, sx, xt, sxt = ops.quantize_128x1_t_grouped(xg4.detach(), layout, e, with_1x128=True)
    goq, sgo, got, sgot = ops.quantize_128x1_t_grouped(go4, layout, e, with_1x128=True)
    f8 = hpfp8.quantize_grouped_weight(wg4.detach())
    fl = 2.0 * total * n * k
    r4 = {"rows": total, "experts": e, "min_rows": int(counts.min()), "max_rows": int(counts.max())}
    r4["forward_gemm"] = _tf(fl, _time(lambda: ops.gemm_grouped_blockwise(xq, sx, f8.codes, f8.scale_inv, offs), iters=5, warm=5))
    r4["dgrad_gemm"] = _tf(fl, _time(lambda: ops.gemm_grouped_blockwise_t(goq, sgo, f8.codes_t, f8.scale_inv, offs), iters=5, warm=3))
    r4["wgrad_gemm"] = _tf(fl, _time(lambda: ops.gemm_grouped_wgrad(got, sgot, xt, sxt, layout, e, total), iters=5, warm=3))
    r4["quantize_both_forms_x_grouped"] = _gb(total * k * 4 + 2 * total * (k // 128) * 4, _time(
        lambda: ops.quantize_128x1_t_grouped(xg4.detach(), layout, e, with_1x128=True), iters=5, warm=3))
    del xq, xt, goq, got
    torch.cuda.empty_cache()

    def grouped_train(f8w):
        hpfp8.fp8_grouped_linear(xg4, wg4, offs, weight_fp8=f8w).backward(go4)
        xg4.grad = wg4.grad = None
    r4["layer_forward_backward"] = dict(_tf(3 * fl, _time(lambda: grouped_train(f8), iters=3, warm=3)),
                                        note="weights' FP8 form made once per optimizer step (weight_fp8); quantizers of x "
                                             "and grad_out, grouped forward, dgrad and wgrad GEMMs; no host read of offs")
    r4["layer_forward_backward_weights_quantized_inside"] = _tf(3 * fl, _time(lambda: grouped_train(None), iters=3, warm=2))
    res["cfg4_moe_grouped"] = r4
    del xg4, wg4, go4, f8
    torch.cuda.empty_cache()
    # cfg 5: gradient bucket, 2^29 elements
    nel = 1 << 29
    flat = torch.randn(nel, generator=g, device=dev) * 1e-4
    idx = torch.randint(0, nel, (nel // 10000,), generator=g, device=dev)
    flat[idx] *= 1e3
    flat = flat.to(torch.bfloat16)
    nbytes = nel * 3 + (nel // 128) * 4
    codes, si = hpfp8.quantize_bucket(flat)
    res["cfg5_bucket"] = {"quantize": _gb(nbytes, _time(lambda: hpfp8.quantize_bucket(flat))),
                          "dequantize": _gb(nbytes, _time(lambda: hpfp8.dequantize_bucket(codes, si)))}
    del flat, codes, si
    torch.cuda.empty_cache()
    return res


def cfg3_quantizers_only(dev, iters=8, warm=4):
    """--cfg3-quantizers: nothing but the quantizer rows of configuration 3 (x[4096, 16384] and grad_out[4096, 7168],
    drawn as in the full run, every form, on rotating buffers), with few launches: the command the counter runs of
    profiles/ use, so that their per-kernel rows hold these shapes only."""
    import torch
    m, n, k = 4096, 7168, 16384
    g3 = torch.Generator(device="cpu").manual_seed(0)
    x = cpu_draw(g3, (m, k)).to(torch.bfloat16).to(dev)
    u = cpu_draw(g3, (m, n), kind="rand") - 0.5
    go = (-(2 ** -0.5) * torch.sign(u) * torch.log1p(-2 * u.abs().clamp(max=0.4999999)) * 1e-3).to(torch.bfloat16).to(dev)
    res = quantizer_rows(x, dev, "x_", iters=iters, warm=warm)
    del x
    torch.cuda.empty_cache()
    res.update(quantizer_rows(go, dev, "grad_out_", iters=iters, warm=warm))
    return res


def board_power(fns, launches=1200):
    """Mean board power (W), its cap (W) and the mean shader clock (MHz) while each callable runs `launches` times back
    to back, read from the amdgpu driver's hwmon files of the card; {} when the files are not there."""
    import glob
    import threading
    import torch
    base = "/sys/class/drm/card*/device/hwmon/hwmon*/"
    pw = sorted(glob.glob(base + "power1_input") or glob.glob(base + "power1_average"))[:1]
    fq = sorted(glob.glob(base + "freq1_input"))[:1]
    cap = sorted(glob.glob(base + "power1_cap"))[:1]
    if not pw:
        return {}

    def read(path):
        try:
            return int(open(path).read().strip())
        except (OSError, ValueError):
            return None
    out = {"cap_W": (read(cap[0]) or 0) / 1e6 if cap else None}
    for name, fn in fns.items():
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
        samples, stop = [], threading.Event()

        def sampler():
            while not stop.is_set():
                samples.append((read(pw[0]), read(fq[0]) if fq else None))
                time.sleep(0.02)
        th = threading.Thread(target=sampler)
        th.start()
        s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s0.record()
        for _ in range(launches):
            fn()
        s1.record()
        torch.cuda.synchronize()
        stop.set()
        th.join()
        tail = samples[len(samples) // 4:]                      # (the first quarter: clocks and the sensor's average settling)
        p_ = [a for a, _ in tail if a]
        f_ = [b for _, b in tail if b]
        out[name] = {"ms": s0.elapsed_time(s1) / launches, "board_W": sum(p_) / len(p_) / 1e6 if p_ else None,
                     "sclk_MHz": sum(f_) / len(f_) / 1e6 if f_ else None, "samples": len(tail)}
    return out


def more_measurements(dev):
    """--all: what the layers around the benchmarked kernels cost (the dense-MLP block with its fused SwiGLU, a
    training step of cfg 2's layer), the optional power-of-two recipe, the vendor library's per-tensor GEMM for
    orientation, and the fused bucket pack / unpack."""
    import torch
    import torch.nn.functional as F
    import hpfp8
    res = {}
    g = torch.Generator(device=dev).manual_seed(0)
    tf, gb = _tf, _gb
    # the step after cfg 2 in the MLP: SwiGLU of the gate/up output fused with the 1x128 quantization for the
    # down projection (read 2 x 2 bytes, write 1 byte + scales per activation)
    hgu = torch.randn((4096, 36864), generator=g, device=dev).to(torch.bfloat16)
    res["cfg2_swiglu_quantize"] = gb(4096 * 18432 * 5 + 4096 * (18432 // 128) * 4,
                                     _time(lambda: hpfp8.swiglu_quantize_1x128(hgu, kmajor=True)))
    res["cfg2_swiglu_quantize_fast"] = gb(4096 * 18432 * 5 + 4096 * (18432 // 128) * 4,
                                          _time(lambda: hpfp8.swiglu_quantize_1x128(hgu, kmajor=True, fast=True)))
    res["cfg2_swiglu_quantize_both_forms_fast"] = gb(4096 * 18432 * 6 + 2 * 4096 * (18432 // 128) * 4, _time(
        lambda: hpfp8.ops.swiglu_quantize_1x128_and_128x1_t(hgu, fast=True)))
    # the whole dense-MLP block forward: gate/up linear, SwiGLU, down linear [7168 <- 18432]
    wd_bf16 = (torch.randn((7168, 18432), device=dev) * 0.006).to(torch.bfloat16)
    wgu_bf16 = (torch.randn((36864, 7168), device=dev) * 0.006).to(torch.bfloat16)
    x_mlp = torch.randn((4096, 7168), device=dev).to(torch.bfloat16)
    gu_q, dn_q = hpfp8.quantize_weight(wgu_bf16, with_transpose=False), hpfp8.quantize_weight(wd_bf16, with_transpose=False)

    def torch_mlp():
        h = F.linear(x_mlp, wgu_bf16)
        return F.linear(F.silu(h[:, :18432]) * h[:, 18432:], wd_bf16)
    mlp_flop = 2.0 * 4096 * 7168 * (36864 + 18432)
    t_fp8 = _time(lambda: hpfp8.fp8_swiglu_mlp(x_mlp, gu_q, dn_q, fast=True), iters=20)
    t_bf16 = _time(torch_mlp, iters=20)
    res["cfg2_mlp_block_forward"] = {"fp8_ms": t_fp8, "TFLOP/s": mlp_flop / t_fp8 / 1e9, "torch_bf16_ms": t_bf16,
                                     "note": "weights prequantized; x quantize + 2 GEMMs + fused SwiGLU/quantize (fast form)"}
    # the same block in training: forward + backward (weights quantized inside, as in an optimizer step)
    xg_, wgu_p, wd_p = x_mlp.clone().requires_grad_(True), wgu_bf16.clone().requires_grad_(True), wd_bf16.clone().requires_grad_(True)
    go_mlp = (torch.randn((4096, 7168), device=dev) * 1e-3).to(torch.bfloat16)

    def fp8_train():
        hpfp8.fp8_swiglu_mlp(xg_, wgu_p, wd_p).backward(go_mlp)
        xg_.grad = wgu_p.grad = wd_p.grad = None

    def bf16_train():
        h = F.linear(xg_, wgu_p)
        F.linear(F.silu(h[:, :18432]) * h[:, 18432:], wd_p).backward(go_mlp)
        xg_.grad = wgu_p.grad = wd_p.grad = None
    t_fp8 = _time(fp8_train, iters=10, warm=15)
    t_bf16 = _time(bf16_train, iters=10, warm=15)
    res["cfg2_mlp_block_forward_backward"] = {"fp8_ms": t_fp8, "TFLOP/s": 3 * mlp_flop / t_fp8 / 1e9, "torch_bf16_ms": t_bf16}
    dact = torch.randn((4096, 18432), device=dev).to(torch.bfloat16)
    res["cfg2_swiglu_backward"] = gb(4096 * 18432 * 10, _time(lambda: hpfp8.ops.swiglu_backward(hgu, dact)))
    del wd_bf16, wgu_bf16, x_mlp, gu_q, dn_q, xg_, wgu_p, wd_p, go_mlp, dact, hgu
    # cfg 2 as a training step of the module: forward + backward through fp8_linear (the weight's FP8 form
    # made beforehand, as Fp8Linear's cache does), beside torch's bf16 F.linear on the same tensors
    xt_ = torch.randn((4096, 7168), generator=g, device=dev).to(torch.bfloat16).requires_grad_(True)
    wt_ = (torch.randn((36864, 7168), generator=g, device=dev) * 0.006).to(torch.bfloat16).requires_grad_(True)
    got_ = (torch.randn((4096, 36864), generator=g, device=dev) * 1e-3).to(torch.bfloat16)
    wf_ = hpfp8.quantize_weight(wt_.detach())

    def _step(fn):
        y_ = fn()
        y_.backward(got_)
        xt_.grad = None
        wt_.grad = None

    ms_fp8 = _time(lambda: _step(lambda: hpfp8.fp8_linear(xt_, wt_, weight_fp8=wf_)), iters=20, warm=30)
    ms_bf16 = _time(lambda: _step(lambda: F.linear(xt_, wt_)), iters=20, warm=30)
    res["cfg2_training_step"] = {"fp8_linear_fwd_bwd_ms": ms_fp8, "torch_bf16_linear_fwd_bwd_ms": ms_bf16,
                                 "TFLOP/s": 3 * 2.0 * 4096 * 36864 * 7168 / ms_fp8 / 1e9}
    # the optional recipe with power-of-two scales (not the benchmarked one): the matrix instruction applies the
    # scales itself; same tensors, quantized with that recipe
    wf2_ = hpfp8.quantize_weight(wt_.detach(), pow2=True)
    ms_p2 = _time(lambda: _step(lambda: hpfp8.fp8_linear(xt_, wt_, recipe="blockwise_pow2", weight_fp8=wf2_)), iters=20, warm=30)
    xq2_, sx2_ = hpfp8.quantize_1x128(xt_.detach(), kmajor=True, pow2=True)
    fl2 = 2.0 * 4096 * 36864 * 7168
    res["recipe_blockwise_pow2"] = {
        "cfg2_forward_gemm": tf(fl2, _time(lambda: hpfp8.gemm_blockwise(xq2_, sx2_, wf2_.codes, wf2_.scale_inv, pow2_scales=True))),
        "cfg2_training_step_fwd_bwd_ms": ms_p2,
        "cfg2_training_step_TFLOP/s": 3 * fl2 / ms_p2 / 1e9,
    }
    # for orientation: this library's per-tensor GEMM and the vendor library's (hipBLASLt through
    # torch._scaled_mm, unit scales) on the same codes; neither is the benchmarked recipe
    one_ = torch.ones((), dtype=torch.float32, device=dev)
    orient = {"per_tensor_gemm": tf(fl2, _time(lambda: hpfp8.gemm_per_tensor(xq2_, one_, wf2_.codes, one_)))}
    try:
        orient["vendor_scaled_mm"] = tf(fl2, _time(lambda: torch._scaled_mm(xq2_, wf2_.codes.t(), scale_a=one_, scale_b=one_,
                                                                            out_dtype=torch.bfloat16)))
    except Exception as err:          # (absent or differently named in another torch build)
        orient["vendor_scaled_mm"] = f"unavailable: {type(err).__name__}"
    try:   # the vendor library's finest scaling on this stack: one scale per row of a and per row of b, applied at the end
        ra_, rb_ = torch.ones((4096, 1), device=dev), torch.ones((1, 36864), device=dev)
        orient["vendor_scaled_mm_rowwise"] = tf(fl2, _time(lambda: torch._scaled_mm(xq2_, wf2_.codes.t(), scale_a=ra_, scale_b=rb_,
                                                                                    out_dtype=torch.bfloat16)))
        torch._scaled_mm(xq2_, wf2_.codes.t(), scale_a=sx2_.contiguous(), scale_b=wf2_.scale_inv, out_dtype=torch.bfloat16)
        orient["vendor_blockwise_1x128_128x128"] = "available"
    except Exception as err:
        orient["vendor_blockwise_1x128_128x128"] = f"unavailable: {str(err).splitlines()[0][:80]}"
    res["cfg2_shape_per_tensor_for_orientation"] = orient
    # what the board draws and clocks at while these GEMMs run back to back (the driver's hwmon files, sampled from a
    # host thread every 20 ms during about a second of launches each; absent files leave the entry empty)
    power_fns = {"blockwise_gemm": lambda: hpfp8.gemm_blockwise(xq2_, sx2_, wf2_.codes, wf2_.scale_inv),
                 "per_tensor_gemm": lambda: hpfp8.gemm_per_tensor(xq2_, one_, wf2_.codes, one_)}
    if "vendor_scaled_mm" in orient:
        power_fns["vendor_scaled_mm"] = lambda: torch._scaled_mm(xq2_, wf2_.codes.t(), scale_a=one_, scale_b=one_,
                                                                 out_dtype=torch.bfloat16)
    res["board_power_during_gemms"] = board_power(power_fns)
    del wf2_, xq2_, sx2_, xt_, wt_, got_, wf_
    torch.cuda.empty_cache()
    # cfg 3 under the optional recipe, and its weight gradient added onto an fp32 main gradient
    m, n, k = 4096, 7168, 16384
    x = torch.randn((m, k), generator=g, device=dev).to(torch.bfloat16)
    go = (torch.randn((m, n), generator=g, device=dev) * 1e-3).to(torch.bfloat16)
    w = (torch.randn((n, k), generator=g, device=dev) * 0.006).to(torch.bfloat16)
    fl = 2.0 * m * n * k
    got2, sgot2 = hpfp8.quantize_128x1_t(go, kmajor=True, pow2=True)
    xt2, sxt2 = hpfp8.quantize_128x1_t(x, kmajor=True, pow2=True)
    goq2, sgo2 = hpfp8.quantize_1x128(go, kmajor=True, pow2=True)
    wq2, sw2, wqt2 = hpfp8.quantize_128x128(w, with_transpose=True, pow2=True)
    res["recipe_blockwise_pow2"].update({
        "cfg3_dgrad_gemm": tf(fl, _time(lambda: hpfp8.gemm_blockwise(goq2, sgo2, wqt2, sw2.t(), pow2_scales=True))),
        "cfg3_wgrad_gemm": tf(fl, _time(lambda: hpfp8.gemm_blockwise(got2, sgot2, xt2, sxt2, sb_gran=1, pow2_scales=True))),
    })
    del got2, xt2, goq2, wq2, wqt2
    got, sgot = hpfp8.quantize_128x1_t(go, kmajor=True)
    xt, sxt = hpfp8.quantize_128x1_t(x, kmajor=True)
    main_grad = torch.zeros((n, k), dtype=torch.float32, device=dev)
    res["cfg3_wgrad_gemm_into_fp32_main_grad"] = tf(
        fl, _time(lambda: hpfp8.gemm_blockwise(got, sgot, xt, sxt, sb_gran=1, out=main_grad, accumulate=True)))
    del main_grad, x, go, w, got, xt
    torch.cuda.empty_cache()
    # cfg 4's grouped GEMM under the optional recipe (timing only: the same codes under power-of-two scales)
    e, n, k, total = 32, 4096, 7168, 131072
    offs = zipf_counts(e, total).cumsum(0).to(torch.int32).to(dev)
    xq, sx = hpfp8.quantize_1x128(torch.randn((total, k), generator=g, device=dev).to(torch.bfloat16), kmajor=True)
    wq, sw = hpfp8.quantize_128x128((torch.randn((e * n, k), generator=g, device=dev) * 0.006).to(torch.bfloat16))
    sx2 = torch.exp2(torch.ceil(torch.log2(sx)))
    sw2 = torch.exp2(torch.ceil(torch.log2(sw)))
    ms2 = _time(lambda: hpfp8.gemm_grouped_blockwise(xq, sx2, wq.view(e, n, k), sw2.view(e, n // 128, k // 128), offs,
                                                     pow2_scales=True), iters=5)
    res["recipe_blockwise_pow2"]["cfg4_moe_grouped_gemm"] = tf(2.0 * total * n * k, ms2)
    del xq, sx, wq, sw, sx2, sw2
    torch.cuda.empty_cache()
    # cfg 5's 2^29 elements as 72 separate gradients (64 of 2048x4096 minus 8 of them split into bias-sized
    # pieces): packing fused with the quantization, and the cast back fused with the unpacking
    nel = 1 << 29
    flat = (torch.randn(nel, generator=g, device=dev) * 1e-4).to(torch.bfloat16)
    nbytes = nel * 3 + (nel // 128) * 4
    sizes = [2048 * 4096] * 56 + [7168] * 8 + [2048 * 4096 * 8 - 7168 * 8]
    views, pos = [], 0
    for n_ in sizes:
        views.append(flat[pos:pos + n_])
        pos += n_
    bucket = hpfp8.Fp8GradBucket(sizes, shard_size=1, grad_scale=0.5)
    q2, si2 = bucket.pack(views)
    outs = [torch.empty(n_, dtype=torch.bfloat16, device=dev) for n_ in sizes]
    res["cfg5_bucket_fused"] = {"pack_and_quantize_72_grads": gb(nbytes, _time(lambda: bucket.pack(views))),
                                "dequantize_and_unpack_72_grads": gb(nbytes, _time(lambda: bucket.unpack(q2[0], si2[0], outs)))}
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=50)   # the clock needs ~25 ms of load to leave its idle state
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--all", action="store_true",
                    help="also time the layers around the kernels, the optional recipe and the fused bucket forms "
                         "(adds a 'more' key; the other four configurations are always under 'other_configs')")
    ap.add_argument("--headline-only", action="store_true", help="skip the other configurations")
    ap.add_argument("--cfg3-quantizers", action="store_true",
                    help="run only the quantizer rows of configuration 3 (for counter collection) and print them")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU's share of the path; this build has no multi-GPU leg "
                 "(run with --gpus 1).")

    import torch
    import hpfp8
    from hpfp8 import _lib

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    lib = _lib.load()
    assert lib.hpfp8_check_device() == 0, lib.hpfp8_last_error().decode()
    dev = torch.device("cuda:0")
    if args.cfg3_quantizers:
        print(json.dumps({"cfg3_quantizers": cfg3_quantizers_only(dev)}))
        return
    x, w = make_inputs(dev)

    # preallocated outputs: nothing is allocated inside the timed region
    FP8 = torch.float8_e4m3fn
    xq = torch.empty((M, K), dtype=FP8, device=dev)
    sx = torch.empty((K // 128, M), dtype=torch.float32, device=dev)   # k-block-major: element (m, kb) at [kb, m]
    wq = torch.empty((N, K), dtype=FP8, device=dev)
    sw = torch.empty((N // 128, K // 128), dtype=torch.float32, device=dev)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def q_act():
        _lib.call("hpfp8_quantize_1x128_kmajor_bf16", x.data_ptr(), M, K, xq.data_ptr(), None, sx.data_ptr(), stream)

    def q_wgt():
        _lib.call("hpfp8_quantize_128x128_bf16", w.data_ptr(), N, K, wq.data_ptr(), None, 0, None, sw.data_ptr(), stream)

    def gemm():
        _lib.call("hpfp8_gemm_blockwise", xq.data_ptr(), K, sx.data_ptr(), 1, M, wq.data_ptr(), K, sw.data_ptr(),
                  K // 128, 1, 128, M, N, K, None, y.data_ptr(), N, _lib.OUT_BF16, 0, stream)

    def ev():
        return torch.cuda.Event(enable_timing=True)

    # The chip leaves its idle clocks only after ~20 launches (about 25 ms) of load: with fewer warm-up steps
    # than that asked for, the difference is run first, untimed like the warm-up itself, so that the timed
    # steps measure the steady state whatever --warmup is.
    ramp_steps = max(0, 40 - args.warmup)
    for _ in range(ramp_steps + args.warmup):
        q_act(); q_wgt(); gemm()
    torch.cuda.synchronize()

    marks = []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        e = [ev() for _ in range(4)]
        e[0].record(); q_act()
        e[1].record(); q_wgt()
        e[2].record(); gemm()
        e[3].record()
        marks.append(e)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    ms_step = wall * 1e3 / args.steps
    t_g = sum(event_ms([(e[2], e[3]) for e in marks])) / args.steps

    # HBM-bound kernels alone: back-to-back launches between one event pair; the activation buffers
    # rotate over > 256 MB so that the Infinity Cache cannot serve the reads.
    reps = max(args.steps, 12)
    xs = [x] + [x.clone() for _ in range(5)]
    xqs = [xq] + [torch.empty_like(xq) for _ in range(5)]
    torch.cuda.synchronize()
    s0, s1 = ev(), ev()
    s0.record()
    for i in range(reps):
        _lib.call("hpfp8_quantize_1x128_kmajor_bf16", xs[i % 6].data_ptr(), M, K, xqs[i % 6].data_ptr(), None,
                  sx.data_ptr(), stream)
    s1.record()
    torch.cuda.synchronize()
    t_qa = s0.elapsed_time(s1) / reps
    # (the weight and its codes are 790 MB per launch, beyond the cache by themselves; two sets all the same)
    w2, wq2 = w.clone(), torch.empty_like(wq)
    wsets = ((w, wq), (w2, wq2))
    torch.cuda.synchronize()
    s0, s1 = ev(), ev()
    s0.record()
    for i in range(reps):
        ws_, wqs_ = wsets[i % 2]
        _lib.call("hpfp8_quantize_128x128_bf16", ws_.data_ptr(), N, K, wqs_.data_ptr(), None, 0, None, sw.data_ptr(), stream)
    s1.record()
    torch.cuda.synchronize()
    t_qw = s0.elapsed_time(s1) / reps
    del w2, wq2, wsets
    del xs, xqs
    flops = 2.0 * M * N * K
    bytes_qa = M * K * 3 + M * (K // 128) * 4
    bytes_qw = N * K * 3 + (N // 128) * (K // 128) * 4
    gemm_tflops = flops / (t_g * 1e-3) / 1e12

    # spot check inside the bench: the timed buffers hold the right answer (float64 reference on a slice)
    lut = torch.tensor([float(v) for v in torch.arange(256, dtype=torch.uint8).view(FP8).float().nan_to_num()],
                       dtype=torch.float64, device=dev)
    a64 = lut[xq[:256].view(torch.uint8).long()] * sx.t()[:256].double().repeat_interleave(128, dim=1)
    b64 = lut[wq[:256].view(torch.uint8).long()] * sw[:2].double().repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
    ref = a64 @ b64.t()
    err = float((y[:256, :256].double() - ref).norm() / ref.norm())
    assert err < 1e-2, f"GEMM output is wrong: rel Frobenius error {err}"

    traffic, traffic_source = gemm_traffic_bytes()
    out = {
        "metric": "FP8 linear TFLOP/s & % FP8 MFMA peak; quantize GB/s & % HBM peak (1 GPU)",
        "value": flops / (ms_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "untimed_clock_ramp_steps": ramp_steps,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3 (fp32 accumulate, bf16 out)",
        "data": "synthetic",
        "config": {
            "workload": "DeepSeekV3 dense-MLP blockwise FP8 forward: x[4096,7168] bf16 (0.1% x50 outliers) 1x128 "
                        "scales, W_gate_up[36864,7168] bf16 N(0,0.006) 128x128 scales; step = quantize x + quantize W + "
                        "scaled GEMM, bf16 out",
            "M": M, "N": N, "K": K,
        },
        "roofline": {
            "kernel": "gemm_kernel<block scales> (hpfp8_gemm_blockwise)",
            "bound": "mfma",
            "achieved": gemm_tflops,
            "peak": PEAK_FP8_TFLOPS,
            "unit": "TFLOP/s",
            "frac": gemm_tflops / PEAK_FP8_TFLOPS,
            "traffic": traffic["tcc_ea"] if traffic else None,
            "traffic_dram_path": traffic["dram_path"] if traffic else None,
            "traffic_source": traffic_source,
            "ms": t_g,
        },
        "quantize": {
            "act_1x128": {"GB/s": bytes_qa / (t_qa * 1e-3) / 1e9, "frac_hbm": bytes_qa / (t_qa * 1e-3) / 1e9 / PEAK_HBM_GBS,
                          "ms": t_qa, "bytes": bytes_qa},
            "weight_128x128": {"GB/s": bytes_qw / (t_qw * 1e-3) / 1e9,
                               "frac_hbm": bytes_qw / (t_qw * 1e-3) / 1e9 / PEAK_HBM_GBS, "ms": t_qw, "bytes": bytes_qw},
        },
        "check": {"gemm_rel_frobenius_vs_f64_dequant_matmul": err},
    }
    host_copies = None
    if not args.no_cpu_baseline:
        import numpy as np
        host_copies = (x[:2048].cpu().view(torch.int16).numpy().view(np.uint16),
                       w.cpu().view(torch.int16).numpy().view(np.uint16))
    del x, w, xq, wq, y
    torch.cuda.empty_cache()
    if not args.headline_only:
        out["other_configs"] = other_configs_compact(dev)
    if args.all:
        out["more"] = more_measurements(dev)
    if host_copies is not None:
        out["cpu_baseline"] = cpu_baseline(*host_copies)
        if not args.headline_only:
            out["cpu_baseline"]["other_configs"] = cpu_baselines_other_configs()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
