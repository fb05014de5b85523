#!/usr/bin/env python3
"""Benchmark of the vecops matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME] [--no-cpu]

A "step" is one pass of the hot path over one batch of synthetic operands that are already resident in HBM.  The
default workload is the configuration the headline metric is quoted on (bf16 GEMM, M=N=K=4096, A[M,K] and B[K,N]
row-major, fp32 accumulate, bf16 output); every other benchmark configuration - the fp32 1024^3 product on both
compute strategies, the four irregular batched shapes, the int8 quantised matmul, the weight-only GEMV at M = 1, 4, 16 -
and the prepacked-weights and runtime-quantised forms are measured in the same run and reported under "secondary",
together with the matrix-core yardstick (what the machine sustains on the benchmark's operand values with nothing but
matrix instructions).  Prints ONE JSON line.

Timing: W warm-up launches, then exactly K launches between two device synchronisations give `ms_per_step` and
`value`; `roofline.achieved` is the median over 7 repetitions of max(K, 50) back-to-back launches timed with HIP
events on the stream the launches go to (torch's current stream).
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks (dense)
PEAK_BF16_TFLOPS = 2500.0
PEAK_INT8_TOPS = 5000.0
PEAK_FP32_MATRIX_TFLOPS = 157.3
PEAK_HBM_GBPS = 8000.0
REPETITIONS = 7

# HBM-side bytes per launch recorded with rocprofv3 (FETCH_SIZE and WRITE_SIZE in KiB per dispatch x 1024, FETCH
# scaled by 2.000 and WRITE by 1.000: what the same counters read for a 1 GiB device copy, `--only copy`).  Counters
# cannot be read from inside this process: these are the figures of the named summaries, for exactly these workloads.
# (FETCH_SIZE KiB, WRITE_SIZE KiB, the summary that holds them)
RECORDED_COUNTERS = {
    "bf16": (98503, 32768, "profiles/tile_gemm_bf16_4096.md"),
    "int8": (55098, 88095, "profiles/tile_gemm_wide_i8_dequant_2048x4096x11008.md"),
    "gemv_m1": (29647, 112, "profiles/skinny_w8a16_m1_m4_m16_4096x14336.md"),
    "gemv_m4": (29761, 112, "profiles/skinny_w8a16_m1_m4_m16_4096x14336.md"),
    "gemv_m16": (30145, 448, "profiles/skinny_w8a16_m1_m4_m16_4096x14336.md"),
    "bf16_packed": (98490, 32768, "profiles/tile_gemm_packed16_bf16_4096.md"),
    "bf16_mid_kn_1024x4096x4096": (49256, 8192, "profiles/tile_gemm_deep128_bf16_1024x4096x4096.md"),
    "bf16_mid_nk_1024x4096x4096": (49245, 8192, "profiles/tile_gemm_deep128_bf16_1024x4096x4096.md"),
    "int8_packed": (55095, 88108, "profiles/tile_gemm_wide_i8_dequant_2048x4096x11008.md"),
    "fp32_f32": (12357, 4096, "profiles/tile_gemm_f32_compute_1024.md"),
    "bf16_mid_nk_2048x11008x4096": (109918, 48106, "profiles/tile_gemm_wide_16_bf16_2048x11008x4096.md"),
    "int8_square": (49596, 65536, "profiles/tile_gemm_i8_dequant_4096.md"),
    "batched_3000x3000x17": (5673, 283496, "profiles/tile_gemm_short_k_bf16_batched_8x3000x3000x17.md"),
    "bf16_mid_kn_3000x3000x3000": (54935, 17770, "profiles/tile_gemm_192_bf16_3000x3000x3000.md"),
}
RECORDED_TRAFFIC = {key: (int((fetch * 2.000 + write * 1.000) * 1024), source) for key, (fetch, write, source) in RECORDED_COUNTERS.items()}


def _traffic(key):
    if key not in RECORDED_TRAFFIC:
        return {"traffic": None}
    nbytes, source = RECORDED_TRAFFIC[key]
    return {"traffic": nbytes, "traffic_source": "recorded: " + source}


def _measure(fn, steps, warmup):
    """fn(i) enqueues one launch on torch's current stream.  Returns the wall time per step of exactly `steps`
    launches between two synchronisations, and the median / extremes of HIP-event time per launch over
    REPETITIONS runs of max(steps, 50) launches."""
    import torch
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(i)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    launches = max(steps, 50)
    per_launch = []
    for _ in range(REPETITIONS):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for i in range(launches):
            fn(i)
        stop.record()
        torch.cuda.synchronize()
        per_launch.append(start.elapsed_time(stop) / launches)
    return {"wall_ms": wall_ms, "event_ms": statistics.median(per_launch), "event_ms_min": min(per_launch),
            "event_ms_max": max(per_launch), "launches_per_repetition": launches, "repetitions": REPETITIONS}


def _kernel_label(plan, operands):
    from vecops_amd import capi
    family = capi.FAMILY_NAMES.get(plan.family, str(plan.family))
    loads = "16-byte loads" if plan.vector_a and plan.vector_b else "element loads"
    b = {0: "B K-contiguous", 1: "B as [K,N]", 2: "B strided"}[plan.b_layout]
    split = f", split-K {plan.split_k}" if plan.split_k > 1 else ""
    wide = "tile_gemm_wide_i8_kernel" if operands.startswith("int8") else f"tile_gemm_wide_16_kernel<{operands}>"
    kernel = wide if family == "tile_256x352" else f"tile_gemm_kernel<{operands}>"
    return f"vecops_hip {kernel} family {family}, {loads}, {b}{split}"


def _roofline(bound, achieved, peak, unit, **extra):
    out = {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak}
    out.update(extra)
    return out


def _timing_fields(t):
    return {"event_ms": t["event_ms"], "event_ms_min": t["event_ms_min"], "event_ms_max": t["event_ms_max"],
            "repetitions": t["repetitions"], "launches_per_repetition": t["launches_per_repetition"]}


def _bf16_operands(dev):
    import numpy as np
    import torch
    from vecops_amd import synth
    n = 4096
    a = synth.bf16_round(synth.normal(1, (n, n), 0.02))
    b_kn = synth.bf16_round(synth.normal(2, (n, n), 0.02))
    ta = torch.from_numpy(a.view(np.int16)).to(dev).view(torch.bfloat16)
    tb = torch.from_numpy(b_kn.view(np.int16)).to(dev).view(torch.bfloat16)
    return a, b_kn, ta, tb


def bench_mfma_ceiling(dev, steps, warmup, which="bf16"):
    """The matrix-core yardstick: nothing but independent matrix instructions, one wavefront per SIMD on all compute
    units, on the benchmark's operand values and on zeros - on both instruction shapes the tile kernels use (32x32 and
    16x16).  `value` is the higher of the two on the benchmark's operands, `shape` names it."""
    import torch
    from vecops_amd import capi, synth
    out = torch.empty(256 * 256, dtype=torch.int32, device=dev)
    if which == "bf16":
        _, _, values, _ = _bf16_operands(dev)
        labels, unit, peak = ("v_mfma_f32_32x32x16_bf16", "v_mfma_f32_16x16x32_bf16"), "TFLOP/s", PEAK_BF16_TFLOPS
        what = "normal(0, 0.02) rounded to bf16 (the GEMM's A operand)"
    else:
        values = torch.from_numpy(synth.int8_sym(1, (2048, 4096))).to(dev)
        labels, unit, peak = ("v_mfma_i32_32x32x32_i8", "v_mfma_i32_16x16x64_i8"), "TOP/s", PEAK_INT8_TOPS
        what = "int8 uniform[-127,127] (the quantised matmul's A operand)"
    zeros = torch.zeros_like(values)
    res = {}
    for shape in (0, 1):
        for name, operands in (("benchmark_operands", values), ("zeros", zeros)):
            ops_per_launch = [0]

            def launch(i, operands=operands, shape=shape):
                ops_per_launch[0] = capi.mfma_stream(operands, 256, 512 if shape == 0 else 1024, out, shape=shape)
            t = _measure(launch, max(5, steps // 10), max(2, warmup // 5))
            res[shape, name] = ops_per_launch[0] / (t["event_ms"] * 1e-3) / 1e12
    best = max((0, 1), key=lambda shape: res[shape, "benchmark_operands"])
    return {"metric": f"mfma_ceiling_{which}", "workload": "256 workgroups x 4 wavefronts of nothing but independent matrix "
            f"instructions (sixteen accumulator tiles per wavefront, no memory traffic), operands: {what}; and zeros",
            "value": res[best, "benchmark_operands"], "unit": unit, "shape": labels[best],
            "on_zeros": res[best, "zeros"], "peak": peak,
            "by_shape": {labels[shape]: {"benchmark_operands": res[shape, "benchmark_operands"], "zeros": res[shape, "zeros"]}
                         for shape in (0, 1)},
            "frac_of_peak": res[best, "benchmark_operands"] / peak, "frac_of_peak_on_zeros": res[best, "zeros"] / peak}


def bench_bf16_gemm(dev, steps, warmup):
    import torch
    from vecops_amd import capi
    n = 4096
    a, b_kn, ta, tb = _bf16_operands(dev)
    tb_view = tb.t()                      # [N,K] view with strides (1, N): vecops' way to pass B[K,N]
    c = torch.empty((n, n), dtype=torch.bfloat16, device=dev)
    run = capi.PreparedMatmul(ta, tb_view, c)       # descriptors and plan built once: a step is one call of the C ABI
    plan = run.plan
    t = _measure(lambda i: run(), steps, warmup)
    flops = 2.0 * n * n * n
    tflops = flops / (t["event_ms"] * 1e-3) / 1e12
    return {
        "wall_ms": t["wall_ms"], "value": flops / (t["wall_ms"] * 1e-3) / 1e12,
        "roofline": _roofline("mfma", tflops, PEAK_BF16_TFLOPS, "TFLOP/s", kernel=_kernel_label(plan, "bf16"),
                              algorithmic_flops_per_launch=flops, algorithmic_bytes_per_launch=3 * 2 * n * n,
                              **_traffic("bf16"), **_timing_fields(t)),
        "host": (a, b_kn),
    }


def bench_fp32_gemm(dev, steps, warmup, compute, n=1024):
    """BASELINE configs[0]: fp32 1024^3, A[M,K] and B[K,N] row-major, U[-1,1); multiplied as bf16 (vecops' x86
    behaviour) or in fp32 (its SME_F32F32 atom)."""
    import torch
    from vecops_amd import capi, synth
    a = torch.from_numpy(synth.uniform_pm1(1, (n, n))).to(dev)
    b_kn = torch.from_numpy(synth.uniform_pm1(2, (n, n))).to(dev)
    c = torch.empty((n, n), dtype=torch.float32, device=dev)
    code = capi.COMPUTE_F32 if compute == "f32" else capi.COMPUTE_BF16
    plan = capi.plan_matmul(a, b_kn.t(), c, compute=code)
    ws = torch.empty(max(int(plan.workspace_bytes), 1), dtype=torch.uint8, device=dev)
    run = capi.PreparedMatmul(a, b_kn.t(), c, compute=code, workspace=ws)   # a step is one call of the C ABI
    t = _measure(lambda i: run(), max(steps, 200) if n <= 1024 else steps, warmup)
    flops = 2.0 * n ** 3
    tflops = flops / (t["event_ms"] * 1e-3) / 1e12
    peak = PEAK_FP32_MATRIX_TFLOPS if compute == "f32" else PEAK_BF16_TFLOPS
    label = _kernel_label(plan, "f32" if compute == "f32" else "f32 as bf16")
    family = capi.FAMILY_NAMES.get(plan.family)
    tile = {"tile_64": 64, "tile_128": 128}.get(family, 0)
    if compute == "f32" and tile and (-(-n // tile)) ** 2 * max(int(plan.split_k), 1) <= 256 and n % 32 == 0 and n // 32 // max(int(plan.split_k), 1) >= 8:
        label = label.replace("tile_gemm_kernel<f32>", "tile_gemm_deep_f32_kernel")   # what run_problem launches for such a plan
    return {"metric": f"fp32_gemm_{n}_{compute}_compute_tflops", "workload": f"fp32 GEMM M=N=K={n}, A[M,K] and B[K,N] "
            f"row-major, uniform[-1,1), multiplied in {'fp32' if compute == 'f32' else 'bf16 (rounded on load)'}, fp32 "
            "accumulate and output (BASELINE configs[0])", "value": tflops, "unit": "TFLOP/s",
            "us_per_step": t["wall_ms"] * 1e3, "dtype": "f32" if compute == "f32" else "f32 memory, bf16 compute",
            "roofline": _roofline("mfma", tflops, peak, "TFLOP/s", kernel=label,
                                  algorithmic_flops_per_launch=flops, algorithmic_bytes_per_launch=3 * 4 * n * n,
                                  **(_traffic("fp32_f32") if compute == "f32" and n == 1024 else {"traffic": None}),
                                  **_timing_fields(t))}


def bench_bf16_mid(dev, steps, warmup, m, n, k, b_as_kn):
    """A product of at most one 128 x 128 workgroup per compute unit (default 1024 x 4096 x 4096: a prefill batch of 1024
    tokens against a 4096-wide weight), bf16 in and out: the four-stage 128 x 128 kernel's workload."""
    import numpy as np
    import torch
    from vecops_amd import capi, synth
    a = torch.from_numpy(synth.bf16_round(synth.normal(1, (m, k), 0.02)).view(np.int16)).to(dev).view(torch.bfloat16)
    b = torch.from_numpy(synth.bf16_round(synth.normal(2, (k, n) if b_as_kn else (n, k), 0.02)).view(np.int16)).to(dev).view(torch.bfloat16)
    b = b.t() if b_as_kn else b
    c = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    plan = capi.plan_matmul(a, b, c)
    ws = torch.empty(max(int(plan.workspace_bytes), 1), dtype=torch.uint8, device=dev)
    run = capi.PreparedMatmul(a, b, c, workspace=ws)
    t = _measure(lambda i: run(), steps, warmup)
    flops = 2.0 * m * n * k
    tflops = flops / (t["event_ms"] * 1e-3) / 1e12
    label = _kernel_label(plan, "bf16")
    split = max(int(plan.split_k), 1)
    workgroups = -(-m // 128) * -(-n // 128) * split
    if capi.FAMILY_NAMES.get(plan.family) == "tile_128" and workgroups <= 256 and k % 64 == 0 and k // 64 // split >= 8:
        label = label.replace("tile_gemm_kernel<bf16>", "tile_gemm_deep128_kernel<bf16>")   # what run_problem launches for such a plan
    roof = _roofline("mfma", tflops, PEAK_BF16_TFLOPS, "TFLOP/s", kernel=label, algorithmic_flops_per_launch=flops,
                     algorithmic_bytes_per_launch=2 * (m * k + n * k + m * n),
                     **_traffic(f"bf16_mid_{'kn' if b_as_kn else 'nk'}_{m}x{n}x{k}"), **_timing_fields(t))
    return {"metric": f"bf16_gemm_{m}x{n}x{k}_tflops", "workload": f"bf16 ({m},{n},{k}), A[M,K] and B[{'K,N' if b_as_kn else 'N,K'}], "
            "normal(0,0.02), fp32 accumulate, bf16 output", "value": tflops, "unit": "TFLOP/s",
            "us_per_step": t["wall_ms"] * 1e3, "dtype": "bf16", "roofline": roof}


def bench_batched(dev, steps, warmup, m, n, k):
    """BASELINE configs[2]: batch 8, bf16 operands uniform[-1,1), fp32 accumulate and output."""
    import numpy as np
    import torch
    from vecops_amd import capi, synth
    batch = 8
    a = torch.from_numpy(synth.bf16_round(synth.uniform_pm1(1, (batch, m, k))).view(np.int16)).to(dev).view(torch.bfloat16)
    b = torch.from_numpy(synth.bf16_round(synth.uniform_pm1(2, (batch, n, k))).view(np.int16)).to(dev).view(torch.bfloat16)
    c = torch.empty((batch, m, n), dtype=torch.float32, device=dev)
    plan = capi.plan_matmul(a, b, c)
    ws = torch.empty(max(int(plan.workspace_bytes), 1), dtype=torch.uint8, device=dev)
    run = capi.PreparedMatmul(a, b, c, workspace=ws)   # a step is one call of the C ABI
    t = _measure(lambda i: run(), max(steps, 100), warmup)
    flops = batch * 2.0 * m * n * k
    nbytes = batch * (2 * m * k + 2 * n * k + 4 * m * n)
    tflops = flops / (t["event_ms"] * 1e-3) / 1e12
    gbps = nbytes / (t["event_ms"] * 1e-3) / 1e9
    # the bound is the one that takes longer at the machine's peaks
    mfma_bound = flops / (PEAK_BF16_TFLOPS * 1e12) >= nbytes / (PEAK_HBM_GBPS * 1e9)
    roof = (_roofline("mfma", tflops, PEAK_BF16_TFLOPS, "TFLOP/s") if mfma_bound
            else _roofline("hbm", gbps, PEAK_HBM_GBPS, "GB/s"))
    label = _kernel_label(plan, "bf16")
    if capi.FAMILY_NAMES[plan.family] == "tile_128" and 8 <= k <= 32:
        label = "tile_gemm_short_k_kernel<bf16>"   # what run_problem launches for such a plan
    roof.update(kernel=label, algorithmic_flops_per_launch=flops, algorithmic_bytes_per_launch=nbytes,
                **_traffic(f"batched_{m}x{n}x{k}"), **_timing_fields(t))
    return {"metric": f"bf16_batched_{m}x{n}x{k}_tflops", "workload": f"batch 8 x bf16 ({m},{n},{k}), A[8,M,K] and "
            "B[8,N,K], uniform[-1,1), fp32 accumulate and output (BASELINE configs[2])", "value": tflops,
            "unit": "TFLOP/s", "hbm_gbps": gbps, "us_per_step": t["wall_ms"] * 1e3, "dtype": "bf16", "roofline": roof}


GROUPED_SHAPES = [(777, 1000, 3001), (1, 4097, 129), (255, 63, 8191), (3000, 3000, 17), (1300, 700, 520), (64, 5000, 1030),
                  (2000, 2000, 264), (500, 300, 4100)]


def bench_grouped(dev, steps, warmup):
    """Irregular batches: eight bf16 products of unlike shapes (BASELINE configs[2]'s four among them, unbatched) as one
    vecops_hip_matmul_grouped call, and the same eight as separate vecops_hip_matmul calls."""
    import numpy as np
    import torch
    from vecops_amd import capi, synth
    a_list, b_list, c_list = [], [], []
    for i, (m, n, k) in enumerate(GROUPED_SHAPES):
        a_list.append(torch.from_numpy(synth.bf16_round(synth.uniform_pm1(10 + i, (m, k))).view(np.int16)).to(dev).view(torch.bfloat16))
        b_list.append(torch.from_numpy(synth.bf16_round(synth.uniform_pm1(40 + i, (n, k))).view(np.int16)).to(dev).view(torch.bfloat16))
        c_list.append(torch.empty((m, n), dtype=torch.float32, device=dev))
    ws = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
    # (a call is seven launches - two groups split K - and a separate-calls step ten: at most 100 steps between
    # synchronisations, because with thousands of launches queued the HIP runtime's own bookkeeping stalls the host
    # in the first such loop of a process, 160-200 us per step of wall time where the GPU needs 76)
    count = min(max(steps, 50), 100)
    run = capi.PreparedGrouped(a_list, b_list, c_list, workspace=ws)    # a step is one call of the C ABI
    grouped = _measure(lambda i: run(), count, max(warmup, count))

    def one_by_one(i):
        for a, b, c in zip(a_list, b_list, c_list):
            capi.matmul(a, b, c, workspace=ws)
    looped = _measure(one_by_one, count, max(warmup, count))
    flops = sum(2.0 * m * n * k for m, n, k in GROUPED_SHAPES)
    tflops = flops / (grouped["event_ms"] * 1e-3) / 1e12
    roof = _roofline("mfma", tflops, PEAK_BF16_TFLOPS, "TFLOP/s", kernel="vecops_hip tile_gemm_grouped_kernel<bf16>",
                     algorithmic_flops_per_launch=flops, traffic=None, **_timing_fields(grouped))
    return {"metric": "bf16_grouped_irregular_tflops", "workload": "eight bf16 products of unlike shapes "
            f"{GROUPED_SHAPES}, fp32 out, one vecops_hip_matmul_grouped call", "value": tflops, "unit": "TFLOP/s",
            "us_per_step": grouped["wall_ms"] * 1e3, "separate_calls_event_us": looped["event_ms"] * 1e3,
            "separate_calls_wall_us": looped["wall_ms"] * 1e3, "dtype": "bf16", "roofline": roof}


def bench_int8_dequant(dev, steps, warmup, ceiling=None):
    import torch
    from vecops_amd import capi, synth
    m, k, n = 2048, 4096, 11008
    a = torch.from_numpy(synth.int8_sym(1, (m, k))).to(dev)
    b = torch.from_numpy(synth.int8_sym(2, (n, k))).to(dev)
    rs = torch.from_numpy(synth.scales(3, m)).to(dev)
    cs = torch.from_numpy(synth.scales(4, n)).to(dev)
    c = torch.empty((m, n), dtype=torch.float32, device=dev)
    need = capi.lib().vecops_hip_matmul_i8_dequant_workspace(m, n, k)   # the caller owns the scratch
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    plan = capi.plan_matmul(a, b, torch.empty((m, n), dtype=torch.int32, device=dev))
    t = _measure(lambda i: capi.matmul_i8_dequant(a, b, rs, cs, c, workspace=ws), steps, warmup)
    ops = 2.0 * m * n * k
    tops = ops / (t["event_ms"] * 1e-3) / 1e12
    roof = _roofline("mfma", tops, PEAK_INT8_TOPS, "TOP/s", kernel=_kernel_label(plan, "int8") + ", dequantising epilogue",
                     algorithmic_ops_per_launch=ops, algorithmic_bytes_per_launch=m * k + n * k + 4 * m * n + 4 * (m + n),
                     **_traffic("int8"), **_timing_fields(t))
    if ceiling:
        roof.update(measured_ceiling=ceiling, frac_of_ceiling=tops / ceiling)
    return {"metric": "int8_quantized_matmul_tops", "workload": "int8 2048x4096x11008, per-token x per-channel "
            "dequant fused, fp32 out (BASELINE configs[3])", "value": tops, "unit": "TOP/s", "ms_per_step": t["wall_ms"],
            "dtype": "int8", "roofline": roof}


def bench_int8_square(dev, steps, warmup, ceiling=None):
    """int8 4096^3 with the same fused dequantisation: the extents the headline metric names for both operand classes."""
    import torch
    from vecops_amd import capi, synth
    n = 4096
    a = torch.from_numpy(synth.int8_sym(1, (n, n))).to(dev)
    b = torch.from_numpy(synth.int8_sym(2, (n, n))).to(dev)
    rs = torch.from_numpy(synth.scales(3, n)).to(dev)
    cs = torch.from_numpy(synth.scales(4, n)).to(dev)
    c = torch.empty((n, n), dtype=torch.float32, device=dev)
    ws = torch.empty(max(capi.lib().vecops_hip_matmul_i8_dequant_workspace(n, n, n), 1), dtype=torch.uint8, device=dev)
    plan = capi.plan_matmul(a, b, torch.empty((n, n), dtype=torch.int32, device=dev))
    t = _measure(lambda i: capi.matmul_i8_dequant(a, b, rs, cs, c, workspace=ws), steps, warmup)
    ops = 2.0 * n ** 3
    tops = ops / (t["event_ms"] * 1e-3) / 1e12
    roof = _roofline("mfma", tops, PEAK_INT8_TOPS, "TOP/s", kernel=_kernel_label(plan, "int8") + ", dequantising epilogue",
                     algorithmic_ops_per_launch=ops, algorithmic_bytes_per_launch=2 * n * n + 4 * n * n + 8 * n,
                     **_traffic("int8_square"), **_timing_fields(t))
    if ceiling:
        roof.update(measured_ceiling=ceiling, frac_of_ceiling=tops / ceiling)
    return {"metric": "int8_gemm_4096_tops", "workload": "int8 4096^3, per-token x per-channel dequant fused, fp32 out",
            "value": tops, "unit": "TOP/s", "ms_per_step": t["wall_ms"], "dtype": "int8", "roofline": roof}


def bench_runtime_quant(dev, steps, warmup):
    """fp32 activations quantised per row on the way in (vecops' RuntimePerRowAsymmetricQuantizeTransform), int8
    weights, correction row, per-token x per-channel dequantisation: three launches (quantise, weight row sums,
    the int8 product) timed as one step."""
    import ctypes as C
    import numpy as np
    import torch
    from vecops_amd import capi, synth
    m, k, n, zp = 2048, 4096, 11008, 7
    mult = (np.float32(4.0) * (np.float32(1.0) + synth.uniform_pm1(11, (m,)) * np.float32(0.5))).astype(np.float32)
    a_host = ((synth.uniform_pm1(12, (m, k)) * np.float32(140.0) + np.float32(128 - zp)) / mult[:, None]).astype(np.float32)
    b_host = synth.int8_sym(2, (n, k))
    a, b = torch.from_numpy(a_host).to(dev), torch.from_numpy(b_host).to(dev)
    tm = torch.from_numpy(mult).to(dev)
    rs = torch.from_numpy((np.float32(1.0) / mult).astype(np.float32)).to(dev)
    cs = torch.from_numpy(synth.scales(4, n)).to(dev)
    corr = torch.from_numpy((-zp * b_host.astype(np.int64).sum(axis=1)).astype(np.int32)).to(dev)
    c = torch.empty((m, n), dtype=torch.float32, device=dev)
    oa, ob, oc = capi.operand(a), capi.operand(b), capi.operand(c)
    need = capi.lib().vecops_hip_matmul_runtime_quant_workspace(C.byref(oa), C.byref(ob), C.byref(oc))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    t = _measure(lambda i: capi.matmul_runtime_quant(a, tm, zp, b, rs, cs, c, correction=corr, workspace=ws), steps, warmup)
    ops = 2.0 * m * n * k
    tops = ops / (t["event_ms"] * 1e-3) / 1e12
    # (the product runs on the quantised bytes: the plan of int8 operands of these extents names its kernel)
    plan = capi.plan_matmul(torch.empty((m, k), dtype=torch.int8, device=dev), b, torch.empty((m, n), dtype=torch.int32, device=dev))
    return {"metric": "runtime_quantized_matmul_tops", "workload": "fp32 activations 2048x4096 quantised per row to "
            "uint8 on the way in, int8 weights 11008x4096, correction row, per-token x per-channel dequant, fp32 out",
            "value": tops, "unit": "TOP/s", "ms_per_step": t["wall_ms"], "dtype": "int8",
            "roofline": _roofline("mfma", tops, PEAK_INT8_TOPS, "TOP/s", traffic=None,
                                  kernel="vecops_hip quantize_and_row_sums_kernel + " +
                                         _kernel_label(plan, "int8").replace("vecops_hip ", "") + ", dequantising epilogue",
                                  algorithmic_ops_per_launch=ops,
                                  algorithmic_bytes_per_launch=4 * m * k + n * k + 4 * m * n + 4 * (2 * m + 2 * n),
                                  **_timing_fields(t))}


def bench_bf16_gemm_packed(dev, steps, warmup):
    """The headline shape with B packed once beforehand (vecops' prepacked-weights mode): the packing is
    outside the timed region, as in the reference's own prepacked rows."""
    import torch
    from vecops_amd import capi
    n = 4096
    _, _, ta, tb = _bf16_operands(dev)
    packed = capi.pack_b(tb.t())
    c = torch.empty((n, n), dtype=torch.bfloat16, device=dev)
    family = capi.FAMILY_NAMES.get(capi.plan_matmul_packed_b(ta, packed, c).family)
    t = _measure(lambda i: capi.matmul_packed_b(ta, packed, c), steps, warmup)
    flops = 2.0 * n * n * n
    tflops = flops / (t["event_ms"] * 1e-3) / 1e12
    return {"metric": "bf16_gemm_4096_prepacked_b_tflops", "workload": "bf16 GEMM M=N=K=4096, B prepacked "
            "(vecops_hip_pack_b, not timed), fp32 accumulate, bf16 out", "value": tflops, "unit": "TFLOP/s",
            "ms_per_step": t["wall_ms"], "dtype": "bf16",
            "roofline": _roofline("mfma", tflops, PEAK_BF16_TFLOPS, "TFLOP/s",
                                  kernel=("vecops_hip tile_gemm_packed16_kernel<bf16>" if family == "tile_256"   # (aligned A, whole K tiles)
                                          else "vecops_hip tile_gemm_packed_b_kernel<bf16>") + f" family {family}",
                                  algorithmic_flops_per_launch=flops, algorithmic_bytes_per_launch=3 * 2 * n * n,
                                  **_traffic("bf16_packed"), **_timing_fields(t))}


def bench_int8_dequant_packed(dev, steps, warmup):
    import torch
    from vecops_amd import capi, synth
    m, k, n = 2048, 4096, 11008
    a = torch.from_numpy(synth.int8_sym(1, (m, k))).to(dev)
    packed = capi.pack_b(torch.from_numpy(synth.int8_sym(2, (n, k))).to(dev))
    rs = torch.from_numpy(synth.scales(3, m)).to(dev)
    cs = torch.from_numpy(synth.scales(4, n)).to(dev)
    c = torch.empty((m, n), dtype=torch.float32, device=dev)
    need = capi.lib().vecops_hip_matmul_i8_dequant_workspace(m, n, k)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    family = capi.FAMILY_NAMES.get(capi.plan_matmul_packed_b(a, packed, torch.empty((m, n), dtype=torch.int32, device=dev)).family)
    t = _measure(lambda i: capi.matmul_i8_dequant_packed_b(a, packed, rs, cs, c, workspace=ws), steps, warmup)
    ops = 2.0 * m * n * k
    tops = ops / (t["event_ms"] * 1e-3) / 1e12
    return {"metric": "int8_quantized_matmul_prepacked_b_tops", "workload": "int8 2048x4096x11008, weights prepacked "
            "(not timed), per-token x per-channel dequant fused, fp32 out", "value": tops, "unit": "TOP/s",
            "ms_per_step": t["wall_ms"], "dtype": "int8",
            "roofline": _roofline("mfma", tops, PEAK_INT8_TOPS, "TOP/s",
                                  kernel=("vecops_hip tile_gemm_wide_i8_kernel<packed B>" if family == "tile_256x352"
                                          else "vecops_hip tile_gemm_packed_b_kernel<int8>")
                                  + f" family {family}, dequantising epilogue",
                                  algorithmic_ops_per_launch=ops,
                                  algorithmic_bytes_per_launch=m * k + n * k + 4 * m * n + 4 * (m + n),
                                  **_traffic("int8_packed"), **_timing_fields(t))}


def bench_gemv(dev, steps, warmup, m=1):
    import torch
    from vecops_amd import capi, synth
    k, n, group = 4096, 14336, 128
    copies = 8   # 8 x 58.7 MB of weights: the working set exceeds the 256 MB Infinity Cache
    x = torch.from_numpy(synth.bf16_round(synth.normal(1, (m, k))).view("int16")).to(dev).view(torch.bfloat16)
    w0 = torch.from_numpy(synth.int8_sym(2, (n, k))).to(dev)
    ws = [w0] + [torch.roll(w0, shifts=i, dims=0) for i in range(1, copies)]
    s = torch.from_numpy(synth.scales(3, (n, k // group))).to(dev)
    ss = [s.clone() for _ in range(copies)]
    y = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    t = _measure(lambda i: capi.matmul_w8a16_group(x, ws[i % copies], ss[i % copies], y, group), max(steps, 200), warmup)
    nbytes = n * k + 4 * n * (k // group) + 2 * m * k + 2 * m * n
    gbps = nbytes / (t["event_ms"] * 1e-3) / 1e9
    kernel = ("vecops_hip skinny_w8a16_stream_kernel" if m == 1 else "vecops_hip skinny_w8a16_stream_rows_kernel"
              if m == 2 else "vecops_hip skinny_w8a16_mfma_resident_kernel")
    return {"metric": f"w8a16_gemv_m{m}_hbm_gbps", "workload": f"weight-only int8 GEMV M={m} K=4096 N=14336 group 128, "
            "bf16 activations, bf16 out, weights rotated through 8 buffers (BASELINE configs[4])", "value": gbps,
            "unit": "GB/s", "us_per_step": t["wall_ms"] * 1e3, "dtype": "int8 x bf16 -> f32",
            "roofline": _roofline("hbm", gbps, PEAK_HBM_GBPS, "GB/s", kernel=kernel, algorithmic_bytes_per_launch=nbytes,
                                  **_traffic(f"gemv_m{m}"), **_timing_fields(t))}


def bench_read_ceiling(dev, steps, warmup):
    """The read-only yardstick on the GEMV's bytes: the 58.7 MB of one weight matrix, rotated through the same eight
    buffers, streamed by a kernel that does nothing else.  `value` is the best of a few grid sizes."""
    import torch
    from vecops_amd import capi, synth
    k, n, copies = 4096, 14336, 8
    w0 = torch.from_numpy(synth.int8_sym(2, (n, k))).to(dev)
    ws = [w0] + [torch.roll(w0, shifts=i, dims=0) for i in range(1, copies)]
    out = torch.empty(8192 * 256, dtype=torch.int32, device=dev)
    by_grid = {}
    for workgroups in (512, 1024, 2048, 4096):
        t = _measure(lambda i: capi.read_stream(ws[i % copies], workgroups, out), max(steps, 200), warmup)
        by_grid[workgroups] = {"us": t["event_ms"] * 1e3, "gbps": n * k / (t["event_ms"] * 1e-3) / 1e9}
    best = max(by_grid, key=lambda g: by_grid[g]["gbps"])
    return {"metric": "hbm_read_ceiling_gbps", "workload": f"read-only stream of {n * k} bytes (the GEMV's weights), "
            "rotated through 8 buffers, launched back to back", "value": by_grid[best]["gbps"], "unit": "GB/s",
            "us_per_launch": by_grid[best]["us"], "workgroups": best, "by_workgroups": by_grid, "peak": PEAK_HBM_GBPS,
            "frac_of_peak": by_grid[best]["gbps"] / PEAK_HBM_GBPS}


def bench_tile_families(dev, steps, warmup):
    """The measurement the rule table's tile-quality constants come from: bf16 4096^3 (B as [K,N]) and the int8
    2048 x 4096 x 11008 product, required of every tile family in turn (vecops_hip_matmul_family)."""
    import torch
    from vecops_amd import capi, synth
    families = ["tile_256", "tile_256x128", "tile_128x256", "tile_128", "tile_64"]
    n = 4096
    _, _, ta, tb = _bf16_operands(dev)
    c = torch.empty((n, n), dtype=torch.bfloat16, device=dev)
    m, k, nn = 2048, 4096, 11008
    ai = torch.from_numpy(synth.int8_sym(1, (m, k))).to(dev)
    bi = torch.from_numpy(synth.int8_sym(2, (nn, k))).to(dev)
    ci = torch.empty((m, nn), dtype=torch.int32, device=dev)
    rows = []
    for family in families:
        request = capi.family_request(family, capi.SELECT_REQUIRE)
        t16 = _measure(lambda i: capi.matmul_family(ta, tb.t(), c, request), steps, warmup)
        t8 = _measure(lambda i: capi.matmul_family(ai, bi, ci, request), steps, warmup)
        rows.append({"family": family, "bf16_4096_us": t16["event_ms"] * 1e3, "int8_2048x4096x11008_us": t8["event_ms"] * 1e3})
    base = rows[0]["bf16_4096_us"]
    for r in rows:
        r["bf16_quality_vs_tile_256"] = base / r["bf16_4096_us"]
    return {"metric": "tile_family_calibration", "workload": "bf16 4096^3 (B as [K,N]) and int8 2048x4096x11008 -> int32 on "
            "each required tile family", "unit": "us", "value": base, "families": rows}


RULE_CHECK_SHAPES = [
    # (class, M, N, K): the shapes the rule table's thresholds were set on, and the known holes
    ("bf16", 4096, 4096, 4096), ("bf16", 2048, 2048, 2048), ("bf16", 1536, 4096, 4096), ("bf16", 1024, 4096, 4096),
    ("bf16", 768, 4096, 4096), ("bf16", 512, 4096, 4096), ("bf16", 768, 11008, 4096), ("bf16", 1024, 4096, 11008),
    ("bf16", 768, 3072, 12288), ("bf16", 512, 2048, 16384), ("bf16", 384, 384, 1024), ("bf16", 512, 512, 4096),
    ("bf16", 3000, 3000, 3000), ("bf16", 1536, 11008, 4096),
    ("int8", 2048, 11008, 4096), ("int8", 4096, 4096, 4096), ("int8", 1024, 4096, 4096), ("int8", 768, 3072, 12288),
    ("int8", 512, 1024, 8192),
    # the band of 32 to 256 tiles of 128 x 128 (one workgroup per compute unit at most)
    ("bf16", 640, 4096, 4096), ("bf16", 896, 4096, 4096), ("bf16", 1024, 2048, 8192), ("bf16", 384, 3072, 8192),
    ("bf16", 256, 4096, 4096), ("bf16", 1024, 4096, 6144), ("bf16", 128, 8192, 8192), ("int8", 768, 4096, 4096),
    # B stored [K,N] (the layout of the headline line)
    ("bf16_kn", 1024, 4096, 4096), ("bf16_kn", 512, 4096, 4096), ("bf16_kn", 768, 3072, 12288), ("bf16_kn", 2048, 2048, 2048),
    ("bf16_kn", 256, 4096, 4096),
    # where the 256 x 352 tile's count fits the units (16-bit operands, B [N,K])
    ("bf16", 2048, 11008, 4096), ("bf16", 4096, 11008, 4096), ("bf16", 6144, 6144, 6144), ("bf16", 4096, 4224, 4096),
    ("bf16", 1024, 11008, 4096), ("bf16", 3072, 4096, 4096),
    # where 192 x 192 tiles fit one round (operands whose loads write LDS, B [N,K]) - and where they only nearly do
    ("bf16", 3072, 3072, 4096), ("bf16", 1344, 6144, 4096), ("int8", 3000, 3000, 3008), ("int8", 768, 11008, 4096),
    ("bf16", 2304, 2304, 8192), ("bf16", 1920, 3840, 4096), ("bf16", 2048, 4096, 11008),
    ("bf16_kn", 3000, 3000, 3000), ("bf16_kn", 768, 11008, 4096), ("bf16_kn", 1344, 6144, 4096),
    # one round of bigger tiles by a K split
    ("bf16", 1500, 3000, 8192), ("bf16", 2304, 2304, 16384), ("bf16", 2000, 2600, 6144),
]


def bench_rule_check(dev, steps, warmup):
    """The rule table against what it chooses between: every shape of RULE_CHECK_SHAPES on every tile family with K
    split 1, 2, 3 and 4 ways (vecops_hip_matmul_family, Require), and as the table plans it.  `regret_us` = the
    table's time minus the fastest requested combination's."""
    import numpy as np
    import torch
    from vecops_amd import capi, synth
    families = ["tile_256", "tile_256x352", "tile_192", "tile_256x128", "tile_128x256", "tile_128", "tile_64"]
    steps, warmup = max(10, steps // 10), max(10, warmup // 10)
    ws = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
    rows = []
    for kind, m, n, k in RULE_CHECK_SHAPES:
        if kind in ("bf16", "bf16_kn"):
            a = torch.from_numpy(synth.bf16_round(synth.normal(1, (m, k), 0.02)).view(np.int16)).to(dev).view(torch.bfloat16)
            b = torch.from_numpy(synth.bf16_round(synth.normal(2, (n, k), 0.02)).view(np.int16)).to(dev).view(torch.bfloat16)
            b = b.view(k, n).t() if kind == "bf16_kn" else b    # the same bits read as a [K,N] matrix
            c = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
        else:
            a = torch.from_numpy(synth.int8_sym(1, (m, k))).to(dev)
            b = torch.from_numpy(synth.int8_sym(2, (n, k))).to(dev)
            c = torch.empty((m, n), dtype=torch.int32, device=dev)
        plan = capi.plan_matmul(a, b, c)
        auto = _measure(lambda i: capi.matmul(a, b, c, workspace=ws), steps, warmup)["event_ms"] * 1e3
        tried = {}
        for family in families:
            for split in (1, 2, 3, 4):
                request = capi.family_request(family, capi.SELECT_REQUIRE, split_k=split)
                try:
                    need = capi.plan_matmul_family(a, b, c, request).workspace_bytes
                    if need > ws.numel():
                        continue
                    t = _measure(lambda i: capi.matmul_family(a, b, c, request, workspace=ws), steps, warmup)
                except capi.VecopsHipError:
                    continue   # the family cannot serve this problem
                tried[f"{family}/{split}"] = round(t["event_ms"] * 1e3, 2)
        best = min(tried, key=tried.get)
        pick = capi.FAMILY_NAMES.get(plan.family, str(plan.family)) + f"/{max(plan.split_k, 1)}" + (
            f" (+{plan.peeled_columns} peeled columns)" if plan.peeled_columns else "")
        rows.append({"shape": f"{kind} {m}x{n}x{k}", "pick": pick, "pick_us": round(auto, 2), "best": best,
                     "best_us": tried[best], "regret_us": round(auto - tried[best], 2), "tried_us": tried})
    worst = max(rows, key=lambda r: r["regret_us"])
    return {"metric": "rule_table_regret", "workload": "every shape of RULE_CHECK_SHAPES on every tile family x K split 1..4 "
            "against the rule table's own plan (HIP events)", "unit": "us", "value": worst["regret_us"],
            "worst_shape": worst["shape"], "shapes": rows}


VENDOR_GRID = [(m, n, k) for (n, k) in ((4096, 4096), (11008, 4096), (4096, 11008)) for m in (512, 768, 1024, 1536, 2048, 4096)] + [
    (2048, 2048, 2048), (3000, 3000, 3000), (4096, 4224, 4096), (6144, 6144, 6144), (8192, 8192, 8192), (128, 8192, 8192),
    (256, 4096, 4096), (5000, 5000, 1024), (1000, 1000, 1000)]


def bench_vendor_grid(dev, steps, warmup):
    """This library against the vendor's (hipBLASLt through torch.matmul, torch._int_mm) on a grid of shapes: bf16 -> bf16
    with B stored [N,K] and [K,N], int8 -> int32 with B [N,K]; one process, HIP events, the median of five runs of as
    many launches as fill about 20 ms."""
    import numpy as np
    import torch
    from vecops_amd import capi, synth

    def time_us(fn, hint_us):
        n = max(5, min(200, int(20000 / hint_us)))
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        runs = []
        for _ in range(5):
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(n):
                fn()
            stop.record()
            torch.cuda.synchronize()
            runs.append(start.elapsed_time(stop) / n * 1e3)
        return round(sorted(runs)[2], 1)

    ws = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    rows = []
    for m, n, k in VENDOR_GRID:
        hint = max(10.0, 2.0 * m * n * k / 1.2e9)
        a = torch.from_numpy(synth.bf16_round(synth.normal(1, (m, k), 0.02)).view(np.int16)).to(dev).view(torch.bfloat16)
        b = torch.from_numpy(synth.bf16_round(synth.normal(2, (n, k), 0.02)).view(np.int16)).to(dev).view(torch.bfloat16)
        c = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
        row = {"shape": f"{m}x{n}x{k}"}
        for layout in ("nk", "kn"):
            ours_b = b if layout == "nk" else b.view(k, n).t()      # the same bits read as a [K,N] matrix
            theirs_b = b.t() if layout == "nk" else b.view(k, n)
            plan = capi.plan_matmul(a, ours_b, c)
            run = capi.PreparedMatmul(a, ours_b, c, workspace=ws)
            row[f"bf16_{layout}"] = {"ours_us": time_us(lambda: run(), hint),
                                     "vendor_us": time_us(lambda: torch.matmul(a, theirs_b, out=c), hint),
                                     "plan": capi.FAMILY_NAMES.get(plan.family, str(plan.family)) + f"/{max(plan.split_k, 1)}" +
                                             ("+peel" if plan.peeled_columns else "")}
        ai = torch.from_numpy(synth.int8_sym(1, (m, k))).to(dev)
        bi = torch.from_numpy(synth.int8_sym(2, (n, k))).to(dev)
        ci = torch.empty((m, n), dtype=torch.int32, device=dev)
        plan = capi.plan_matmul(ai, bi, ci)
        run = capi.PreparedMatmul(ai, bi, ci, workspace=ws)
        entry = {"ours_us": time_us(lambda: run(), hint / 2),
                 "plan": capi.FAMILY_NAMES.get(plan.family, str(plan.family)) + f"/{max(plan.split_k, 1)}" +
                         ("+peel" if plan.peeled_columns else "")}
        try:
            entry["vendor_us"] = time_us(lambda: torch._int_mm(ai, bi.t(), out=ci), hint / 2)
        except RuntimeError:
            entry["vendor_us"] = None                               # extents torch._int_mm does not take
        row["int8_nk"] = entry
        rows.append(row)
    ratios = [r[key]["ours_us"] / r[key]["vendor_us"] for r in rows for key in ("bf16_nk", "bf16_kn", "int8_nk") if r[key]["vendor_us"]]
    return {"metric": "time_against_vendor_library", "workload": "VENDOR_GRID: bf16 -> bf16 (B [N,K] and [K,N]) against torch.matmul, "
            "int8 -> int32 against torch._int_mm, microseconds per product", "unit": "ours / vendor, geometric mean",
            "value": float(np.exp(np.mean(np.log(ratios)))), "level_or_ahead": sum(r <= 1.02 for r in ratios), "of": len(ratios),
            "shapes": rows}


def bench_copy(dev, steps, warmup):
    """A plain device-to-device copy of known size: the yardstick the FETCH_SIZE / WRITE_SIZE
    counters of the other workloads are scaled by."""
    import torch
    nbytes = 1 << 30
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    t = _measure(lambda i: dst.copy_(src), steps, warmup)
    return {"metric": "device_copy_gbps", "workload": "torch copy_ of 1 GiB (reads 1 GiB, writes 1 GiB)",
            "bytes_read_per_launch": nbytes, "bytes_written_per_launch": nbytes,
            "value": 2.0 * nbytes / (t["event_ms"] * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": t["wall_ms"]}


def recorded_reference():
    """vecops' own CPU matmul on the headline workload, as timed in the build container by oracle/time_reference.py
    (the vecops tree is not present where the benchmark runs): figures with their provenance, or None."""
    path = os.path.join(ROOT, "baseline", "vecops_cpu_container.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        doc = json.load(f)
    rows = [e for e in doc["entries"] if e["config"].startswith("bf16 4096^3")]
    return {"source": "baseline/vecops_cpu_container.json (oracle/time_reference.py, in the build container)",
            "what": doc["what"], "host": doc["host"],
            "entries": [{"config": e["config"], "lanes": e["lanes"], "value": e["rate"] / 1e3, "unit": "TFLOP/s",
                         "ms": e["ms"]} for e in rows]}


def cpu_baseline(a, b_kn):
    """The bf16 4096^3 workload on the host cores: the real vecops CPU matmul when oracle/_ref runs here (AMX host),
    else the oracle's vectorised all-core port, on a bounded row slab of the same operands.  The reference's own
    figures from the build container ride along either way."""
    import numpy as np
    from oracle.oracle import Oracle, Reference
    n = 4096
    ref = Reference.load()
    budget_s = 12.0
    if ref is not None:
        c = np.zeros((n, n), np.uint16)
        reps, t0 = 0, time.perf_counter()
        while reps == 0 or time.perf_counter() - t0 < budget_s:
            ref.dense_bf16_bf16(a, b_kn, c, b_is_kn=True)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        out = {"value": 2.0 * n ** 3 / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "reference",
               "sample": f"full 4096^3 product x {reps}, vecops ops::matmul<AMX_BF16F32> on one thread, dense tensors, "
                         f"B as the transposed view of [K,N] ({dt * 1e3:.0f} ms each)"}
    else:
        oracle = Oracle()
        b_nk = np.ascontiguousarray(b_kn.T)
        rows = 256
        t0 = time.perf_counter()
        oracle.matmul_bf16_dense(a[:rows], b_nk, out_bf16=True)
        probe = time.perf_counter() - t0
        rows = int(min(n, max(256, 256 * (budget_s / max(probe, 1e-3)))))
        rows -= rows % 256
        reps, t0 = 0, time.perf_counter()
        while reps == 0 or time.perf_counter() - t0 < budget_s:
            oracle.matmul_bf16_dense(a[:rows], b_nk, out_bf16=True)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        out = {"value": 2.0 * rows * n * n / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.threads(), "kind": "port",
               "sample": f"first {rows} of 4096 rows of A against all of B, {reps} times ({dt:.2f} s each), "
                         "oracle C port, OpenMP"}
    recorded = recorded_reference()
    if recorded:
        out["recorded_reference"] = recorded
    return out


ONLY = ["bf16", "int8", "int8_square", "gemv", "copy", "bf16_packed", "int8_packed", "runtime_quant", "mfma_ceiling", "read_ceiling",
        "fp32", "batched", "bf16_mid", "families", "grouped", "rule_check", "vendor_grid"]


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=300,
                    help="untimed launches before the timed ones (after idling the chip takes about 200 launches of "
                         "the headline kernel, 25 ms, to settle at its clock under load)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", choices=ONLY, help="run a single workload (for profiling)")
    ap.add_argument("--gemv-m", type=int, default=1, help="activation rows of the --only gemv workload (1..16)")
    ap.add_argument("--ceiling-dtype", choices=["bf16", "int8"], default="bf16", help="operands of --only mfma_ceiling")
    ap.add_argument("--fp32-compute", choices=["bf16", "f32"], default="bf16", help="compute type of --only fp32")
    ap.add_argument("--fp32-size", type=int, default=1024, help="M = N = K of --only fp32 (1024: BASELINE configs[0])")
    ap.add_argument("--batched-shape", default="777,1000,3001", help="M,N,K of --only batched")
    ap.add_argument("--mid-shape", default="1024,4096,4096", help="M,N,K of --only bf16_mid")
    ap.add_argument("--mid-layout", choices=["kn", "nk"], default="kn", help="how B is stored for --only bf16_mid")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the matmul path is built and measured on a single MI355X "
              "(--gpus must be 1)", file=sys.stderr)
        return 2

    import torch
    from vecops_amd import capi
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    capi.lib()  # fails loudly when the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.synchronize()
    K, W = args.steps, args.warmup

    single = {
        "int8": lambda: bench_int8_dequant(dev, K, W),
        "int8_square": lambda: bench_int8_square(dev, K, W),
        "copy": lambda: bench_copy(dev, K, W),
        "bf16_packed": lambda: bench_bf16_gemm_packed(dev, K, W),
        "int8_packed": lambda: bench_int8_dequant_packed(dev, K, W),
        "runtime_quant": lambda: bench_runtime_quant(dev, K, W),
        "gemv": lambda: bench_gemv(dev, K, W, m=args.gemv_m),
        "mfma_ceiling": lambda: bench_mfma_ceiling(dev, K, W, args.ceiling_dtype),
        "read_ceiling": lambda: bench_read_ceiling(dev, K, W),
        "fp32": lambda: bench_fp32_gemm(dev, K, W, args.fp32_compute, args.fp32_size),
        "batched": lambda: bench_batched(dev, K, W, *[int(v) for v in args.batched_shape.split(",")]),
        "bf16_mid": lambda: bench_bf16_mid(dev, K, W, *[int(v) for v in args.mid_shape.split(",")], args.mid_layout == "kn"),
        "families": lambda: bench_tile_families(dev, K, W),
        "grouped": lambda: bench_grouped(dev, K, W),
        "rule_check": lambda: bench_rule_check(dev, K, W),
        "vendor_grid": lambda: bench_vendor_grid(dev, K, W),
    }
    if args.only in single:
        print(json.dumps(single[args.only]()))
        return 0

    main_res = bench_bf16_gemm(dev, K, W)
    a, b_kn = main_res.pop("host")
    head = {
        "metric": "bf16_gemm_4096_tflops", "value": main_res["value"], "unit": "TFLOP/s", "n_gpus": 1,
        "steps": K, "warmup": W, "ms_per_step": main_res["wall_ms"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "bf16 GEMM M=N=K=4096, A[M,K] and B[K,N] row-major, normal(0,0.02), fp32 accumulate, "
                               "bf16 output (BASELINE configs[1])", "M": 4096, "N": 4096, "K": 4096},
    }
    roofline = main_res["roofline"]
    secondary = None
    if args.only != "bf16":
        ceiling_bf16 = bench_mfma_ceiling(dev, K, W, "bf16")
        ceiling_int8 = bench_mfma_ceiling(dev, K, W, "int8")
        # what the machine sustains on these operand values with nothing but matrix instructions (the better of the
        # two instruction shapes): the practical ceiling - the clocks follow the power the multipliers draw; `frac`
        # stays against the nominal peak
        roofline["measured_ceiling"] = ceiling_bf16["value"]
        roofline["measured_ceiling_shape"] = ceiling_bf16["shape"]
        roofline["frac_of_ceiling"] = roofline["achieved"] / ceiling_bf16["value"]
        int8 = bench_int8_dequant(dev, K, W, ceiling=ceiling_int8["value"])
        int8_square = bench_int8_square(dev, K, W, ceiling=ceiling_int8["value"])
        gemv = {m: bench_gemv(dev, K, W, m=m) for m in (1, 4, 16)}
        read_ceiling = bench_read_ceiling(dev, K, W)
        for r in gemv.values():   # what a kernel that only reads the weights sustains on the same buffers
            r["roofline"]["measured_read_ceiling"] = read_ceiling["value"]
            r["roofline"]["frac_of_read_ceiling"] = r["roofline"]["achieved"] / read_ceiling["value"]
        fp32 = {c: bench_fp32_gemm(dev, K, W, c) for c in ("bf16", "f32")}
        packed16, packed8 = bench_bf16_gemm_packed(dev, K, W), bench_int8_dequant_packed(dev, K, W)
        secondary = [bench_batched(dev, K, W, m, n, k)
                     for (m, n, k) in [(777, 1000, 3001), (1, 4097, 129), (255, 63, 8191), (3000, 3000, 17)]]
        secondary += [bench_bf16_mid(dev, K, W, 1024, 4096, 4096, True), bench_bf16_mid(dev, K, W, 2048, 2048, 2048, False),
                      bench_bf16_mid(dev, K, W, 2048, 11008, 4096, False), bench_bf16_mid(dev, K, W, 3000, 3000, 3000, True)]
        secondary += [bench_runtime_quant(dev, K, W), bench_grouped(dev, K, W), ceiling_bf16, ceiling_int8, read_ceiling, packed16,
                      packed8,
                      fp32["bf16"], fp32["f32"], gemv[16], gemv[4], gemv[1], int8_square, int8]

        def brief(r):
            return {"frac": round(r["roofline"]["frac"], 4), "event_us": round(r["roofline"]["event_ms"] * 1e3, 2),
                    "value": round(r["value"], 1), "unit": r["unit"]}
        # the other components of the headline metric and the remaining benchmark configurations, in short: the full
        # records are in `secondary`
        roofline["also"] = {"int8_cfg4": brief(int8), "int8_4096": brief(int8_square), "int8_cfg4_prepacked": brief(packed8), "gemv_m1": brief(gemv[1]),
                            "gemv_m4": brief(gemv[4]), "gemv_m16": brief(gemv[16]), "fp32_1024_f32_compute": brief(fp32["f32"]),
                            "fp32_1024_bf16_compute": brief(fp32["bf16"]), "bf16_4096_prepacked": brief(packed16),
                            "hbm_read_ceiling_gbps": round(read_ceiling["value"], 1)}
    # (the long list first: a reader who sees only the end of the line sees the headline and its roofline)
    line = {}
    if secondary is not None:
        line["secondary"] = secondary
    if not args.no_cpu and args.only is None:
        line["cpu_baseline"] = cpu_baseline(a, b_kn)
    line.update(head)
    line["roofline"] = roofline
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
