#!/usr/bin/env python3
"""Times the real vecops CPU matmul (oracle/_ref, built from the vecops sources by oracle/Makefile) on the five
benchmark configurations, on one lane and on eight lanes, and writes baseline/vecops_cpu_container.json.

    python oracle/time_reference.py

vecops' matmul is single-threaded per call by design; callers shard across lanes (the pattern of
tests/ops/StatefulMatmulTest.cpp:106-151).  Here a lane is a host thread that calls the reference on its own row
slab of A and C (column slab of B and C when M <= 16), with its own workspace and its own online pack of B - what
an application that splits the work itself would get.  The reference only exists where the vecops tree does: the
benchmark on the GPU box prints these recorded figures, with their provenance, beside its own CPU port.
"""
from __future__ import annotations

import json
import os
import platform
import sys
import threading
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
sys.path = [p for p in sys.path if os.path.abspath(p or ".") != HERE]  # `oracle` is the package, not oracle/oracle.py
sys.path.insert(0, ROOT)
from oracle.oracle import Reference  # noqa: E402
from vecops_amd import synth  # noqa: E402

OUT = os.path.join(os.path.dirname(HERE), "baseline", "vecops_cpu_container.json")


def _time(fn, budget_s=4.0, min_reps=2):
    fn()  # first touch, page faults
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < min_reps or (time.perf_counter() < t_end and len(times) < 7):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return float(np.median(times)), len(times)


def _lanes(work, lanes):
    """Runs work(i, lanes) for i < lanes on host threads (the calls release the interpreter lock)."""
    if lanes == 1:
        work(0, 1)
        return
    threads = [threading.Thread(target=work, args=(i, lanes)) for i in range(lanes)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()


def _slab(total, i, lanes):
    step = -(-total // lanes)
    return min(total, i * step), min(total, (i + 1) * step)


def main() -> int:
    ref = Reference.load()
    if ref is None:
        print("oracle/_ref/libvecops_ref.so is not built or this host has no AMX", file=sys.stderr)
        return 2
    entries = []

    def record(config, lanes, seconds, reps, work, unit, note):
        rate = work / seconds / 1e9
        entries.append({"config": config, "lanes": lanes, "ms": seconds * 1e3, "rate": rate, "unit": unit, "reps": reps,
                        "note": note})
        print(f"{config:56s} lanes={lanes}  {seconds * 1e3:9.2f} ms  {rate:9.1f} {unit}", flush=True)

    import ctypes as C
    L = ref.lib
    P, I = C.c_void_p, C.c_int64

    def ptr(x):
        assert x.flags["C_CONTIGUOUS"]
        return P(x.ctypes.data)

    def check(rc):
        if rc != 0:
            raise RuntimeError("reference matmul unavailable")

    for lanes in (1, 8):
        # configs[0]: fp32 1024^3, A[M,K] and B[K,N] row-major, U[-1,1): fp32 memory, bf16 compute, fp32 out
        n = 1024
        a, b_kn = synth.uniform_pm1(1, (n, n)), synth.uniform_pm1(2, (n, n))
        c = np.zeros((n, n), np.float32)

        def w0(i, nl):
            r0, r1 = _slab(n, i, nl)
            check(L.vref_dense_f32_f32(ptr(a[r0:r1]), ptr(b_kn), ptr(c[r0:r1]), I(r1 - r0), I(n), I(n), 1))
        s, reps = _time(lambda: _lanes(w0, lanes))
        record("fp32 1024^3 (fp32 memory, bf16 compute, fp32 out)", lanes, s, reps, 2.0 * n ** 3, "GFLOP/s",
               "ops::matmul<AMX_BF16F32>, dense tensors, B as the transposed view of [K,N]")

        # configs[1]: bf16 4096^3, bf16 out, B[K,N] row-major (BASELINE) and B[N,K]
        n = 4096
        a16 = synth.bf16_round(synth.normal(1, (n, n), 0.02))
        b16 = synth.bf16_round(synth.normal(2, (n, n), 0.02))
        c16 = np.zeros((n, n), np.uint16)
        for kn, label in ((1, "[K,N]"), (0, "[N,K]")):
            def w1(i, nl, kn=kn):
                r0, r1 = _slab(n, i, nl)
                check(L.vref_dense_bf16_bf16(ptr(a16[r0:r1]), ptr(b16), ptr(c16[r0:r1]), I(r1 - r0), I(n), I(n), kn))
            s, reps = _time(lambda: _lanes(w1, lanes), budget_s=6.0)
            record(f"bf16 4096^3 (B as {label}, bf16 out)", lanes, s, reps, 2.0 * n ** 3, "GFLOP/s",
                   "ops::matmul<AMX_BF16F32>, dense tensors")

        # configs[2]: batch 8 of four irregular shapes, bf16 in, fp32 out (lanes split the batch)
        for (m, nn, k) in [(777, 1000, 3001), (1, 4097, 129), (255, 63, 8191), (3000, 3000, 17)]:
            a3 = synth.bf16_round(synth.uniform_pm1(1, (8, m, k)))
            b3 = synth.bf16_round(synth.uniform_pm1(2, (8, nn, k)))
            c3 = np.zeros((8, m, nn), np.float32)

            def w2(i, nl):
                r0, r1 = _slab(8, i, nl)
                if r1 > r0:
                    check(L.vref_dense_bf16_f32_batched(ptr(a3[r0:r1]), ptr(b3[r0:r1]), ptr(c3[r0:r1]), I(r1 - r0), I(m), I(nn), I(k)))
            s, reps = _time(lambda: _lanes(w2, lanes), budget_s=3.0)
            record(f"bf16 batch 8 x ({m},{nn},{k}), fp32 out", lanes, s, reps, 8 * 2.0 * m * nn * k, "GFLOP/s",
                   "rank-3 ops::matmul<AMX_BF16F32>, dense tensors; lanes split the batch")

        # configs[3]: int8 2048 x 4096 x 11008 with per-token x per-channel dequantisation, fp32 out
        m, k, nn = 2048, 4096, 11008
        ai, bi = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (nn, k))
        rs = synth.scales(3, m)
        cs = np.zeros(nn + 64, np.float32)   # the transform's vector load reads past n (matmul/Quantization.h:229-231)
        cs[:nn] = synth.scales(4, nn)
        ci = np.zeros((m, nn), np.float32)

        def w3(i, nl):
            r0, r1 = _slab(m, i, nl)
            check(L.vref_dense_i8_dequant(ptr(ai[r0:r1]), ptr(bi), ptr(rs[r0:r1]), ptr(cs), ptr(ci[r0:r1]), I(r1 - r0), I(nn), I(k)))
        s, reps = _time(lambda: _lanes(w3, lanes), budget_s=5.0)
        record("int8 2048x4096x11008 + dequant, fp32 out", lanes, s, reps, 2.0 * m * nn * k, "GOP/s",
               "ops::matmul<AMX_I8I32<int8,int8>> with RuntimePerRowColumnDequantizeTransform, dense tensors; every lane packs all of B")

        # configs[4] has no vecops counterpart (no weight-only group-scaled matmul): the nearest form it can express,
        # bf16 x bf16 with the weights dequantised to bf16 beforehand
        k, nn = 4096, 14336
        wq = synth.bf16_round((synth.int8_sym(2, (nn, k)).astype(np.float32) * np.float32(0.01)))
        for m in (1, 4, 16):
            x = synth.bf16_round(synth.normal(1, (m, k)))
            outs = [np.zeros((m, _slab(nn, i, lanes)[1] - _slab(nn, i, lanes)[0]), np.uint16) for i in range(lanes)]

            def w4(i, nl):
                r0, r1 = _slab(nn, i, nl)
                check(L.vref_dense_bf16_bf16(ptr(x), ptr(wq[r0:r1]), ptr(outs[i]), I(m), I(r1 - r0), I(k), 0))
            s, reps = _time(lambda: _lanes(w4, lanes), budget_s=2.0)
            record(f"bf16 M={m} x 14336 x 4096 (weights pre-dequantised to bf16)", lanes, s, reps, 2.0 * m * nn * k,
                   "GFLOP/s", "nearest vecops form of the weight-only int8 GEMV, dense tensors; lanes split N")

    cpu = "unknown"
    with open("/proc/cpuinfo") as f:
        for line in f:
            if line.startswith("model name"):
                cpu = line.split(":", 1)[1].strip()
                break
    doc = {"what": "vecops' own CPU matmul (oracle/_ref/libvecops_ref.so, built from the vecops sources with ROCm clang, "
                   "-O2 -march=sapphirerapids) on the build container",
           "host": {"cpu": cpu, "logical_cpus": os.cpu_count(), "machine": platform.machine()},
           "method": "median of 2-7 repetitions after one untimed call; a lane is a host thread with its own slab",
           "entries": entries}
    with open(OUT, "w") as f:
        json.dump(doc, f, indent=1)
    print("wrote", OUT)
    return 0


if __name__ == "__main__":
    sys.exit(main())
