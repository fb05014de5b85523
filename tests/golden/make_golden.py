"""Writes tests/golden/vecops_matmul_golden.npz: outputs of the REAL vecops CPU
matmul (oracle/_ref/libvecops_ref.so, compiled from the vecops sources in the
build container; needs AMX) for seeded inputs.  Inputs are not stored: the cases
below regenerate them from vecops_amd.synth with the seeds listed here, and
tests/golden_cases.py holds the same table for the consumers.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from golden_cases import CASES, make_inputs  # noqa: E402
from oracle.oracle import Reference  # noqa: E402


def main() -> None:
    ref = Reference.load()
    if ref is None:
        raise SystemExit("oracle/_ref/libvecops_ref.so is not built or this host lacks AMX")
    out = {}
    for case in CASES:
        name, kind = case["name"], case["kind"]
        inp = make_inputs(case)
        if kind == "bf16_f32":
            c = np.zeros(inp["c_shape"], np.float32)
            if inp["a"].ndim == 3:
                ref.matmul_bf16_f32_batched(inp["a"], inp["b"], c)
            else:
                ref.matmul_bf16_f32(inp["a"], inp["b"], c, cin=inp.get("cin"))
        elif kind == "bf16_bf16":
            c = np.zeros(inp["c_shape"], np.uint16)
            ref.matmul_bf16_bf16(inp["a"], inp["b"], c)
        elif kind == "f32_f32":
            c = np.zeros(inp["c_shape"], np.float32)
            ref.matmul_f32_f32(inp["a"], inp["b"], c)
        elif kind == "f32_bf16":
            c = np.zeros(inp["c_shape"], np.uint16)
            ref.matmul_f32_bf16(inp["a"], inp["b"], c)
        elif kind == "i8_i32":
            c = np.zeros(inp["c_shape"], np.int32)
            ref.matmul_i8_i32(inp["a"], inp["b"], c, cin=inp.get("cin"))
        elif kind == "u8i8_i32":
            c = np.zeros(inp["c_shape"], np.int32)
            ref.matmul_u8i8_i32(inp["a"], inp["b"], c)
        elif kind == "i8_dequant":
            c = ref.matmul_i8_dequant(inp["a"], inp["b"], inp["row_scales"], inp["column_scales"],
                                      inp.get("correction"))
        else:
            raise ValueError(kind)
        out[name] = c
        print(f"{name:34s} {kind:11s} -> {c.shape} {c.dtype}")
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vecops_matmul_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
