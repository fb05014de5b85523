"""The committed golden vectors (outputs of the real vecops CPU matmul, see
tests/golden/make_golden.py) against the oracle (CPU) and against the gfx950
kernels through the C ABI (GPU)."""
import os

import numpy as np
import pytest

from conftest import rel_err
from golden_cases import CASES, GOLDEN_PATH, make_inputs
from oracle import oracle as O
from vecops_amd import synth

GOLDEN = np.load(GOLDEN_PATH)

# fp32 results differ from the reference only by summation order; bound scaled with K.
def fp32_tol(k):
    return 2e-6 * max(1.0, k / 32)


def check(case, got):
    want = GOLDEN[case["name"]]
    kind = case["kind"]
    if kind in ("i8_i32", "u8i8_i32"):
        assert np.array_equal(got, want)                      # bit-exact
    elif kind == "i8_dequant":
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))  # bit-exact
    elif kind in ("bf16_bf16", "f32_bf16"):
        assert rel_err(synth.bf16_to_f32(got), synth.bf16_to_f32(want)) <= 2 ** -7   # one bf16 ulp
        assert (got != want).mean() < 0.02                                           # and rarely even that
    else:
        assert rel_err(got, want) <= fp32_tol(case["k"])


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_oracle_reproduces_golden(oracle, case):
    inp = make_inputs(case)
    kind = case["kind"]
    if kind == "i8_dequant":
        got = oracle.matmul_i8_dequant(inp["a"], inp["b"], inp["row_scales"], inp["column_scales"],
                                       inp.get("correction"))
    else:
        dt = {"bf16_f32": np.float32, "f32_f32": np.float32, "bf16_bf16": np.uint16, "f32_bf16": np.uint16,
              "i8_i32": np.int32, "u8i8_i32": np.int32}[kind]
        got = np.zeros(inp["c_shape"], dt)
        atom = O.ATOM_I8I32 if kind in ("i8_i32", "u8i8_i32") else O.ATOM_BF16F32
        oracle.matmul(inp["a"], inp["b"], got, cin=inp.get("cin"), atom=atom, acc_f64=True)
    check(case, got)


def _to_device(arr, device, bf16):
    """numpy (possibly strided / broadcast) -> torch tensor with the same strides."""
    import torch
    base = arr
    while isinstance(base.base, np.ndarray):
        base = base.base
    flat = np.ascontiguousarray(base).reshape(-1)
    t = torch.from_numpy(flat.view(np.int16) if bf16 else flat).to(device)
    if bf16:
        t = t.view(torch.bfloat16)
    offset = (arr.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // arr.itemsize
    return torch.as_strided(t, arr.shape, [s // arr.itemsize for s in arr.strides], offset)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_gpu_reproduces_golden(device, case):
    import torch
    from vecops_amd import capi
    kind = case["kind"]
    inp = make_inputs(case)
    in_bf16 = kind in ("bf16_f32", "bf16_bf16")
    a = _to_device(inp["a"], device, in_bf16)
    b = _to_device(inp["b"], device, in_bf16)
    if kind == "i8_dequant":
        c = torch.full(inp["c_shape"], float("nan"), dtype=torch.float32, device=device)
        corr = torch.from_numpy(inp["correction"]).to(device) if "correction" in inp else None
        capi.matmul_i8_dequant(a, b, torch.from_numpy(inp["row_scales"]).to(device),
                               torch.from_numpy(inp["column_scales"]).to(device), c, correction=corr)
        torch.cuda.synchronize()
        got = c.cpu().numpy()
    else:
        out_dt = {"bf16_f32": torch.float32, "f32_f32": torch.float32, "bf16_bf16": torch.bfloat16,
                  "f32_bf16": torch.bfloat16, "i8_i32": torch.int32, "u8i8_i32": torch.int32}[kind]
        c = torch.zeros(inp["c_shape"], dtype=out_dt, device=device)
        cin = torch.from_numpy(inp["cin"]).to(device) if "cin" in inp else None
        capi.matmul(a, b, c, c_in=cin)
        torch.cuda.synchronize()
        got = c.view(torch.int16).cpu().numpy().view(np.uint16) if out_dt == torch.bfloat16 else c.cpu().numpy()
    check(case, got)


# --- runtime per-row asymmetric quantisation of fp32 activations -------------------------------------------------

QUANT_GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vecops_quant_golden.npz")


def test_quantize_rows_edge_values_match_the_reference(oracle):
    """Every branch of the fp32 -> uint8 input conversion (truncation toward zero, saturation, NaN, infinities,
    values outside int32) as the real vecops build produced it, read back through an identity B."""
    from golden_cases import QUANT_EDGE_ZERO_POINTS, quant_edge_inputs
    gold = np.load(QUANT_GOLDEN)
    a, eye, mult = quant_edge_inputs()
    for zp in QUANT_EDGE_ZERO_POINTS:
        want = gold[f"edge_zp{zp}"]
        assert want.min() >= 0 and want.max() == 255
        assert np.array_equal(oracle.quantize_rows(a, mult, zp).astype(np.int32), want), zp


def test_quantize_rows_rounds_twice_like_the_reference(oracle):
    """Elements built so that one fused rounding of a * multiplier + zero_point gives byte 0 and two roundings
    give byte 1: the reference gives 1 for every one of them, and so does the oracle."""
    gold = np.load(QUANT_GOLDEN)
    a, mult, want = gold["fma_a"], gold["fma_multipliers"], gold["fma_bytes"]
    fused = np.trunc(a[:, 0].astype(np.float64) * mult.astype(np.float64) - 15.0)
    assert (fused == 0).all() and (want == 1).all()
    assert np.array_equal(oracle.quantize_rows(a, mult, -15).astype(np.int32), want)


def test_runtime_quant_pipeline_matches_the_reference(oracle):
    """quantise -> u8 x s8 sums + correction row -> per-row x per-column dequantisation, against the real build
    (tests/ops/MatmulConversionTestCommon.h:1437-1540): int32 sums and fp32 outputs bit for bit."""
    from golden_cases import QUANT_CASES, make_quant_inputs
    from oracle import oracle as O
    gold = np.load(QUANT_GOLDEN)
    for case in QUANT_CASES:
        inp = make_quant_inputs(case)
        q = oracle.quantize_rows(inp["a"], inp["multipliers"], case["zp"])
        assert q.min() == 0 and q.max() == 255                     # both ends of the byte range saturate
        acc = np.zeros((case["m"], case["n"]), np.int32)
        oracle.matmul(q, inp["b"], acc, cin=np.broadcast_to(inp["correction"], acc.shape), atom=O.ATOM_I8I32,
                      acc_f64=True, c_bf16=False)
        assert np.array_equal(acc, gold[case["name"] + "_i32"]), case["name"]
        out = oracle.fused_outputs(acc, np.float32, row_scales=inp["row_scales"], column_scales=inp["column_scales"])
        assert np.array_equal(out.view(np.uint32), gold[case["name"] + "_f32"].view(np.uint32)), case["name"]


def test_batched_runtime_quant_pipeline_matches_the_reference(oracle):
    """Shared or per-batch activations and weights (tests/ops/MatmulConversionTestCommon.h:1277-1434, on that test's
    own operands and on seeded ones): the oracle's pieces composed batch by batch against the real build, bit for bit."""
    from golden_cases import QUANT_BATCHED_CASES, make_quant_batched_inputs, quant_batched_by_oracle
    gold = np.load(QUANT_GOLDEN)
    for case in QUANT_BATCHED_CASES:
        inp = make_quant_batched_inputs(case)
        out = quant_batched_by_oracle(oracle, inp, case["batch"])
        assert np.array_equal(out.view(np.uint32), gold[case["name"] + "_f32"].view(np.uint32)), case["name"]
    # the reference test's own expectation on its operands: every output an exact small multiple of the scales
    inp = make_quant_batched_inputs(QUANT_BATCHED_CASES[0])
    q = oracle.quantize_rows(inp["a"][0], inp["multipliers"][:5], 7)
    assert np.array_equal(q.astype(np.int64), (np.arange(5 * 65).reshape(5, 65) % 7 - 3) + 7)
