#!/usr/bin/env python3
"""Benchmark of the vecops matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

A "step" is one pass of the hot path over one batch of synthetic operands that are
already resident in HBM.  The default workload is the configuration the headline
metric is quoted on (bf16 GEMM, M=N=K=4096, A[M,K] and B[K,N] row-major, fp32
accumulate, bf16 output); the int8 quantised matmul, the M=1 weight-only GEMV and the
prepacked-weights forms of the two GEMMs are measured in the same run and reported
under "secondary".  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks
PEAK_BF16_TFLOPS = 2500.0
PEAK_INT8_TOPS = 5000.0
PEAK_HBM_GBPS = 8000.0

# HBM-side bytes per launch from the rocprofv3 FETCH_SIZE / WRITE_SIZE passes kept under
# profiles/ (KiB per dispatch x 1024, FETCH scaled by 2.000 and WRITE by 1.000: what the
# same counters read for a 1 GiB device copy, `--only copy`).  Counters cannot be read
# from inside this process, so these are the recorded figures for exactly these workloads.
TRAFFIC_BF16_4096 = int((98479.5 * 2.000 + 32768 * 1.000) * 1024)
TRAFFIC_INT8_DEQUANT = int((95283.3 * 2.000 + 88064 * 1.000) * 1024)
TRAFFIC_GEMV_M1 = int((29647.4 * 2.000 + 112.0 * 1.000) * 1024)
TRAFFIC_BF16_4096_PACKED = int((98468.3 * 2.000 + 32768 * 1.000) * 1024)
TRAFFIC_INT8_DEQUANT_PACKED = int((95160.6 * 2.000 + 88064 * 1.000) * 1024)


def _device_tensors_bf16_gemm(dev):
    import numpy as np
    import torch
    from vecops_amd import synth
    n = 4096
    a = synth.bf16_round(synth.normal(1, (n, n), 0.02))
    b_kn = synth.bf16_round(synth.normal(2, (n, n), 0.02))
    ta = torch.from_numpy(a.view(np.int16)).to(dev).view(torch.bfloat16)
    tb = torch.from_numpy(b_kn.view(np.int16)).to(dev).view(torch.bfloat16)
    return a, b_kn, ta, tb


def _time_launches(fn, steps, warmup):
    """Returns (wall ms per step, HIP-event ms per launch) for `steps` back-to-back launches
    on torch's current stream - the stream the launcher is handed."""
    import torch
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return wall_ms, start.elapsed_time(stop) / steps


def bench_bf16_gemm(dev, steps, warmup):
    import torch
    from vecops_amd import capi
    n = 4096
    a, b_kn, ta, tb = _device_tensors_bf16_gemm(dev)
    tb_view = tb.t()                      # [N,K] view with strides (1, N): vecops' way to pass B[K,N]
    c = torch.empty((n, n), dtype=torch.bfloat16, device=dev)
    wall_ms, ev_ms = _time_launches(lambda i: capi.matmul(ta, tb_view, c), steps, warmup)
    flops = 2.0 * n * n * n
    tflops = flops / (ev_ms * 1e-3) / 1e12
    return {
        "wall_ms": wall_ms, "event_ms": ev_ms, "value": flops / (wall_ms * 1e-3) / 1e12,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_BF16_TFLOPS, "traffic": TRAFFIC_BF16_4096,
                     "kernel": "vecops_hip::tile_gemm_kernel<bf16, 256x256x64, loads into LDS, B as [K,N]>",
                     "algorithmic_flops_per_launch": flops, "algorithmic_bytes_per_launch": 3 * 2 * n * n},
        "host": (a, b_kn),
    }


def bench_int8_dequant(dev, steps, warmup):
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
    wall_ms, ev_ms = _time_launches(lambda i: capi.matmul_i8_dequant(a, b, rs, cs, c, workspace=ws), steps, warmup)
    ops = 2.0 * m * n * k
    tops = ops / (ev_ms * 1e-3) / 1e12
    return {"metric": "int8_quantized_matmul_tops", "workload": "int8 2048x4096x11008, per-token x per-channel "
            "dequant fused, fp32 out", "value": tops, "unit": "TOP/s", "ms_per_step": wall_ms, "dtype": "int8",
            "roofline": {"bound": "mfma", "achieved": tops, "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                         "frac": tops / PEAK_INT8_TOPS, "traffic": TRAFFIC_INT8_DEQUANT,
                         "kernel": "vecops_hip::tile_gemm_kernel<int8, 256x256x128, loads into LDS, dequant epilogue>",
                         "algorithmic_ops_per_launch": ops,
                         "algorithmic_bytes_per_launch": m * k + n * k + 4 * m * n + 4 * (m + n)}}


def bench_runtime_quant(dev, steps, warmup):
    """fp32 activations quantised per row on the way in (vecops' RuntimePerRowAsymmetricQuantizeTransform), int8
    weights, correction row, per-token x per-channel dequantisation: three launches (quantise, weight row sums,
    the int8 product) timed as one step."""
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
    import ctypes as C
    need = capi.lib().vecops_hip_matmul_runtime_quant_workspace(C.byref(oa), C.byref(ob), C.byref(oc))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    wall_ms, ev_ms = _time_launches(
        lambda i: capi.matmul_runtime_quant(a, tm, zp, b, rs, cs, c, correction=corr, workspace=ws), steps, warmup)
    ops = 2.0 * m * n * k
    tops = ops / (ev_ms * 1e-3) / 1e12
    return {"metric": "runtime_quantized_matmul_tops", "workload": "fp32 activations 2048x4096 quantised per row to "
            "uint8 on the way in, int8 weights 11008x4096, correction row, per-token x per-channel dequant, fp32 out",
            "value": tops, "unit": "TOP/s", "ms_per_step": wall_ms, "dtype": "int8",
            "roofline": {"bound": "mfma", "achieved": tops, "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                         "frac": tops / PEAK_INT8_TOPS, "traffic": None,
                         "kernel": "vecops_hip::quantize_rows_kernel + byte_row_sums_kernel + tile_gemm_kernel<int8, "
                                   "256x256x128, loads into LDS, dequant epilogue>",
                         "algorithmic_ops_per_launch": ops,
                         "algorithmic_bytes_per_launch": 4 * m * k + n * k + 4 * m * n + 4 * (2 * m + 2 * n)}}


def bench_bf16_gemm_packed(dev, steps, warmup):
    """The headline shape with B packed once beforehand (vecops' prepacked-weights mode): the packing is
    outside the timed region, as in the reference's own prepacked rows."""
    import torch
    from vecops_amd import capi
    n = 4096
    _, _, ta, tb = _device_tensors_bf16_gemm(dev)
    packed = capi.pack_b(tb.t())
    c = torch.empty((n, n), dtype=torch.bfloat16, device=dev)
    wall_ms, ev_ms = _time_launches(lambda i: capi.matmul_packed_b(ta, packed, c), steps, warmup)
    flops = 2.0 * n * n * n
    tflops = flops / (ev_ms * 1e-3) / 1e12
    return {"metric": "bf16_gemm_4096_prepacked_b_tflops", "workload": "bf16 GEMM M=N=K=4096, B prepacked "
            "(vecops_hip_pack_b, not timed), fp32 accumulate, bf16 out", "value": tflops, "unit": "TFLOP/s",
            "ms_per_step": wall_ms, "dtype": "bf16",
            "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": tflops / PEAK_BF16_TFLOPS, "traffic": TRAFFIC_BF16_4096_PACKED,
                         "kernel": "vecops_hip::tile_gemm_packed_b_kernel<bf16, 256x256x64>",
                         "algorithmic_flops_per_launch": flops, "algorithmic_bytes_per_launch": 3 * 2 * n * n}}


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
    wall_ms, ev_ms = _time_launches(
        lambda i: capi.matmul_i8_dequant_packed_b(a, packed, rs, cs, c, workspace=ws), steps, warmup)
    ops = 2.0 * m * n * k
    tops = ops / (ev_ms * 1e-3) / 1e12
    return {"metric": "int8_quantized_matmul_prepacked_b_tops", "workload": "int8 2048x4096x11008, weights prepacked "
            "(not timed), per-token x per-channel dequant fused, fp32 out", "value": tops, "unit": "TOP/s",
            "ms_per_step": wall_ms, "dtype": "int8",
            "roofline": {"bound": "mfma", "achieved": tops, "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                         "frac": tops / PEAK_INT8_TOPS, "traffic": TRAFFIC_INT8_DEQUANT_PACKED,
                         "kernel": "vecops_hip::tile_gemm_packed_b_kernel<int8, 256x256x128, dequant epilogue>",
                         "algorithmic_ops_per_launch": ops,
                         "algorithmic_bytes_per_launch": m * k + n * k + 4 * m * n + 4 * (m + n)}}


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
    wall_ms, ev_ms = _time_launches(
        lambda i: capi.matmul_w8a16_group(x, ws[i % copies], ss[i % copies], y, group), steps, warmup)
    nbytes = n * k + 4 * n * (k // group) + 2 * m * k + 2 * m * n
    gbps = nbytes / (ev_ms * 1e-3) / 1e9
    return {"metric": f"w8a16_gemv_m{m}_hbm_gbps", "workload": f"weight-only int8 GEMV M={m} K=4096 N=14336 group 128, "
            "bf16 activations, bf16 out, weights rotated through 8 buffers", "value": gbps, "unit": "GB/s",
            "us_per_step": wall_ms * 1e3, "dtype": "int8 x bf16 -> f32",
            "roofline": {"bound": "hbm", "achieved": gbps, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                         "frac": gbps / PEAK_HBM_GBPS, "traffic": TRAFFIC_GEMV_M1 if m == 1 else None,
                         "kernel": "vecops_hip::skinny_w8a16_stream_kernel" if m == 1 else
                                   "vecops_hip::skinny_w8a16_stream_rows_kernel" if m == 2 else
                                   "vecops_hip::skinny_w8a16_mfma_resident_kernel",
                         "algorithmic_bytes_per_launch": nbytes}}


def bench_copy(dev, steps, warmup):
    """A plain device-to-device copy of known size: the yardstick the FETCH_SIZE / WRITE_SIZE
    counters of the other workloads are scaled by."""
    import torch
    nbytes = 1 << 30
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    wall_ms, ev_ms = _time_launches(lambda i: dst.copy_(src), steps, warmup)
    return {"metric": "device_copy_gbps", "workload": "torch copy_ of 1 GiB (reads 1 GiB, writes 1 GiB)",
            "bytes_read_per_launch": nbytes, "bytes_written_per_launch": nbytes,
            "value": 2.0 * nbytes / (ev_ms * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": wall_ms}


def cpu_baseline(a, b_kn):
    """The bf16 4096^3 workload on the host cores: the real vecops CPU matmul when
    oracle/_ref runs here (AMX host), else the oracle's vectorised all-core port, on a
    bounded row slab of the same operands."""
    import numpy as np
    from oracle.oracle import Oracle, Reference
    n = 4096
    b_nk = np.ascontiguousarray(b_kn.T)
    ref = Reference.load()
    budget_s = 12.0
    if ref is not None:
        c = np.zeros((n, n), np.uint16)
        reps, t0 = 0, time.perf_counter()
        while reps == 0 or time.perf_counter() - t0 < budget_s:
            ref.matmul_bf16_bf16(a, b_nk, c)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        return {"value": 2.0 * n ** 3 / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "reference",
                "sample": f"full 4096^3 product x {reps}, vecops ops::matmul<AMX_BF16F32> on one thread "
                          f"({dt * 1e3:.0f} ms each, B pre-transposed to [N,K])"}
    oracle = Oracle()
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
    return {"value": 2.0 * rows * n * n / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.threads(), "kind": "port",
            "sample": f"first {rows} of 4096 rows of A against all of B, {reps} times ({dt:.2f} s each), "
                      "oracle C port, OpenMP"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", choices=["bf16", "int8", "gemv", "copy", "bf16_packed", "int8_packed", "runtime_quant"], help="run a single workload (for profiling)")
    ap.add_argument("--gemv-m", type=int, default=1, help="activation rows of the --only gemv workload (1..16)")
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

    if args.only == "int8":
        print(json.dumps(bench_int8_dequant(dev, args.steps, args.warmup)))
        return 0
    if args.only == "copy":
        print(json.dumps(bench_copy(dev, args.steps, args.warmup)))
        return 0
    if args.only == "bf16_packed":
        print(json.dumps(bench_bf16_gemm_packed(dev, args.steps, args.warmup)))
        return 0
    if args.only == "int8_packed":
        print(json.dumps(bench_int8_dequant_packed(dev, args.steps, args.warmup)))
        return 0
    if args.only == "runtime_quant":
        print(json.dumps(bench_runtime_quant(dev, args.steps, args.warmup)))
        return 0
    if args.only == "gemv":
        print(json.dumps(bench_gemv(dev, args.steps, args.warmup, m=args.gemv_m)))
        return 0

    main_res = bench_bf16_gemm(dev, args.steps, args.warmup)
    a, b_kn = main_res.pop("host")
    line = {
        "metric": "bf16_gemm_4096_tflops", "value": main_res["value"], "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_res["wall_ms"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "bf16 GEMM M=N=K=4096, A[M,K] and B[K,N] row-major, normal(0,0.02), fp32 accumulate, "
                               "bf16 output (BASELINE configs[1])", "M": 4096, "N": 4096, "K": 4096},
        "roofline": main_res["roofline"],
    }
    if args.only != "bf16":
        line["secondary"] = [bench_int8_dequant(dev, args.steps, args.warmup),
                             bench_gemv(dev, max(args.steps, 200), args.warmup, m=1),
                             bench_gemv(dev, max(args.steps, 200), args.warmup, m=4),
                             bench_gemv(dev, max(args.steps, 200), args.warmup, m=16),
                             bench_bf16_gemm_packed(dev, args.steps, args.warmup),
                             bench_int8_dequant_packed(dev, args.steps, args.warmup),
                             bench_runtime_quant(dev, args.steps, args.warmup)]
    if not args.no_cpu and args.only is None:
        line["cpu_baseline"] = cpu_baseline(a, b_kn)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
