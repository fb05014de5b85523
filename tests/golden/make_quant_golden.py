"""Writes tests/golden/vecops_quant_golden.npz: outputs of the REAL vecops CPU matmul with fp32
activations quantised on the way in by RuntimePerRowAsymmetricQuantizeTransform
(oracle/_ref/libvecops_ref.so, compiled from the vecops sources in the build container; needs AMX)
for the inputs of tests/golden_cases.py: the edge-value table and the fused-rounding discriminator read
back through an identity B, the seeded pipeline cases QUANT_CASES (int32 sums and dequantised fp32), and the
batched cases QUANT_BATCHED_CASES (shared or per-batch activations and weights; dequantised fp32).

    python tests/golden/make_quant_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from golden_cases import (QUANT_BATCHED_CASES, QUANT_CASES, QUANT_EDGE_ZERO_POINTS, make_quant_batched_inputs,  # noqa: E402
                          make_quant_inputs, quant_edge_inputs, quant_fma_inputs)
from oracle.oracle import Reference  # noqa: E402


def main() -> None:
    ref = Reference.load()
    if ref is None:
        raise SystemExit("oracle/_ref/libvecops_ref.so is not built or this host lacks AMX")
    out = {}
    a, eye, mult = quant_edge_inputs()
    for zp in QUANT_EDGE_ZERO_POINTS:
        out[f"edge_zp{zp}"] = ref.matmul_runtime_quant(a, eye, mult, zp, np.zeros(64, np.int32))
    fa, fmult = quant_fma_inputs()
    out["fma_a"], out["fma_multipliers"] = fa, fmult
    out["fma_bytes"] = ref.matmul_runtime_quant(fa, np.ones((1, 1), np.int8), fmult, -15, np.zeros(1, np.int32))
    for case in QUANT_CASES:
        inp = make_quant_inputs(case)
        out[case["name"] + "_i32"] = ref.matmul_runtime_quant(inp["a"], inp["b"], inp["multipliers"], case["zp"],
                                                              inp["correction"])
        out[case["name"] + "_f32"] = ref.matmul_runtime_quant(inp["a"], inp["b"], inp["multipliers"], case["zp"],
                                                              inp["correction"], inp["row_scales"],
                                                              inp["column_scales"])
    for case in QUANT_BATCHED_CASES:
        inp = make_quant_batched_inputs(case)
        out[case["name"] + "_f32"] = ref.matmul_runtime_quant_batched(
            inp["a"], inp["b"], inp["multipliers"], inp["zero_point"], inp["row_scales"], inp["column_scales"],
            inp["correction"], batch=case["batch"])
    for name, value in out.items():
        print(f"{name:28s} -> {value.shape} {value.dtype}")
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vecops_quant_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
