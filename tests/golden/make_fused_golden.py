"""Writes tests/golden/vecops_fused_golden.npz: outputs of the REAL vecops CPU matmul with fused
output transforms (oracle/_ref/libvecops_ref.so, compiled from the vecops sources in the build
container; needs AMX) for the seeded inputs of tests/golden_cases.py::FUSED_CASES.

    python tests/golden/make_fused_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from golden_cases import FUSED_CASES, FUSED_OUT_DTYPES, make_fused_inputs  # noqa: E402
from oracle.oracle import Reference  # noqa: E402


def main() -> None:
    ref = Reference.load()
    if ref is None:
        raise SystemExit("oracle/_ref/libvecops_ref.so is not built or this host lacks AMX")
    out = {}
    for case in FUSED_CASES:
        inp = make_fused_inputs(case)
        lo, hi = case.get("clamp", (0.0, 0.0))
        c = ref.matmul_fused(inp["a"], inp["b"], inp["bias"], FUSED_OUT_DTYPES[case.get("out", "f32")],
                             activation=case.get("act", 0), scale=case.get("scale"), shift=case.get("shift"),
                             column_scales=inp["column_scales"], lo=lo, hi=hi)
        out[case["name"]] = c
        print(f"{case['name']:32s} -> {c.shape} {c.dtype}")
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vecops_fused_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
