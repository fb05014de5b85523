"""Case table shared by tests/golden/make_golden.py (which ran the real vecops CPU
matmul on these inputs) and the tests that compare the oracle and the GPU kernels
with the stored outputs.  Inputs come from vecops_amd.synth seeds; shapes follow
the reference's own tests (file:line per case)."""
import os

import numpy as np

from vecops_amd import synth

GOLDEN_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vecops_matmul_golden.npz")

CASES = [
    # tests/ops/MatmulTest.cpp:434-452 (microkernel shapes and K tails)
    {"name": "bf16_37x51x79", "kind": "bf16_f32", "m": 37, "n": 51, "k": 79},
    {"name": "bf16_1x128x65", "kind": "bf16_f32", "m": 1, "n": 128, "k": 65},
    {"name": "bf16_512x1x256", "kind": "bf16_f32", "m": 512, "n": 1, "k": 256},
    {"name": "bf16_96x16x67", "kind": "bf16_f32", "m": 96, "n": 16, "k": 67},
    {"name": "bf16_130x270x1000", "kind": "bf16_f32", "m": 130, "n": 270, "k": 1000},
    # BASELINE config 3 shapes scaled to fixture size (ragged M/N/K)
    {"name": "bf16_77x100x301", "kind": "bf16_f32", "m": 77, "n": 100, "k": 301},
    {"name": "bf16_255x63x819", "kind": "bf16_f32", "m": 255, "n": 63, "k": 819},
    {"name": "bf16_300x300x17", "kind": "bf16_f32", "m": 300, "n": 300, "k": 17},
    # bf16 output: RNE of the fp32 accumulator (tests/ops/MatmulConversionTestCommon.h:87-145)
    {"name": "bf16out_64x96x160", "kind": "bf16_bf16", "m": 64, "n": 96, "k": 160},
    # fp32 memory -> bf16 compute (the only fp32 path of the x86 backend)
    {"name": "f32mem_33x65x257", "kind": "f32_f32", "m": 33, "n": 65, "k": 257},
    {"name": "f32mem_bf16out_33x65x257", "kind": "f32_bf16", "m": 33, "n": 65, "k": 257},
    # B handed over as [K,N] row-major (tests/ops/MatmulOrientationTest.cpp:65-70)
    {"name": "bf16_nn_70x90x130", "kind": "bf16_f32", "m": 70, "n": 90, "k": 130, "b_layout": "kn"},
    # A transposed in memory as well
    {"name": "bf16_tn_70x90x130", "kind": "bf16_f32", "m": 70, "n": 90, "k": 130, "a_layout": "km"},
    # inner stride 2, padded rows (tests/ops/MatmulTest.cpp:220-279)
    {"name": "bf16_inner2_19x21x35", "kind": "bf16_f32", "m": 19, "n": 21, "k": 35, "inner": 2},
    # rank 3, broadcast B / broadcast A (tests/ops/MatmulBatchTest.cpp:176-335)
    {"name": "bf16_batch3_sharedB", "kind": "bf16_f32", "m": 19, "n": 21, "k": 35, "batch": 3, "share": "b"},
    {"name": "bf16_batch3_sharedA", "kind": "bf16_f32", "m": 19, "n": 21, "k": 35, "batch": 3, "share": "a"},
    {"name": "bf16_batch4", "kind": "bf16_f32", "m": 40, "n": 33, "k": 72, "batch": 4},
    # explicit C input (ops/Matmul.h:144-146)
    {"name": "bf16_cin_37x51x79", "kind": "bf16_f32", "m": 37, "n": 51, "k": 79, "cin": True},
    # int8 (tests/ops/MatmulTest.cpp:1005-1023)
    {"name": "i8_19x21x69", "kind": "i8_i32", "m": 19, "n": 21, "k": 69},
    {"name": "i8_1x128x65", "kind": "i8_i32", "m": 1, "n": 128, "k": 65},
    {"name": "i8_130x140x515", "kind": "i8_i32", "m": 130, "n": 140, "k": 515},
    {"name": "i8_cin_35x53x257", "kind": "i8_i32", "m": 35, "n": 53, "k": 257, "cin": True},
    {"name": "u8i8_19x21x69", "kind": "u8i8_i32", "m": 19, "n": 21, "k": 69},
    # fused per-row x per-column dequantisation (tests/ops/MatmulConversionTestCommon.h:1437-1540)
    {"name": "deq_67x129x515", "kind": "i8_dequant", "m": 67, "n": 129, "k": 515},
    {"name": "deq_corr_67x129x515", "kind": "i8_dequant", "m": 67, "n": 129, "k": 515, "correction": True},
    {"name": "deq_256x384x1024", "kind": "i8_dequant", "m": 256, "n": 384, "k": 1024},
]


def make_inputs(case: dict) -> dict:
    m, n, k = case["m"], case["n"], case["k"]
    kind = case["kind"]
    batch = case.get("batch")
    out = {}
    if kind in ("bf16_f32", "bf16_bf16"):
        gen = lambda seed, shape: synth.bf16_round(synth.uniform_pm1(seed, shape))  # noqa: E731
    elif kind in ("f32_f32", "f32_bf16"):
        gen = synth.uniform_pm1
    else:
        gen = synth.int8_sym
    inner = case.get("inner", 1)
    if batch:
        share = case.get("share")
        a = gen(1, (m, k)) if share == "a" else gen(1, (batch, m, k))
        b = gen(2, (n, k)) if share == "b" else gen(2, (batch, n, k))
        if share == "a":
            a = np.broadcast_to(a, (batch, m, k))
        if share == "b":
            b = np.broadcast_to(b, (batch, n, k))
        out["c_shape"] = (batch, m, n)
    elif inner > 1:
        a = gen(1, (m, inner * k + 3))[:, 0:inner * k:inner]
        b = gen(2, (n, inner * k + 5))[:, 0:inner * k:inner]
        out["c_shape"] = (m, n)
    else:
        a = gen(1, (m, k))
        b = gen(2, (n, k))
        if kind == "u8i8_i32":
            a = (synth.draws(1, m * k) % np.uint64(256)).astype(np.uint8).reshape(m, k)
        if case.get("a_layout") == "km":
            a = np.ascontiguousarray(a.T).T
        if case.get("b_layout") == "kn":
            b = np.ascontiguousarray(b.T).T
        out["c_shape"] = (m, n)
    out["a"], out["b"] = a, b
    if case.get("cin"):
        if kind == "i8_i32":
            out["cin"] = ((synth.draws(3, m * n) % np.uint64(200001)).astype(np.int64) - 100000).astype(
                np.int32).reshape(m, n)
        else:
            out["cin"] = synth.uniform_pm1(3, (m, n))
    if kind == "i8_dequant":
        out["row_scales"] = synth.scales(3, m)
        out["column_scales"] = synth.scales(4, n)
        if case.get("correction"):
            out["correction"] = ((synth.draws(5, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32)
    return out


# ---- fused output transforms --------------------------------------------------------------------
# Outputs of the real vecops matmul with the output transforms its own tests attach
# (tests/ops/MatmulFusionTest.cpp:29-112; builders in tests/ops/MatmulConversionTestCommon.h).
# Fields: kind bf16 | i8; out f32 | bf16 | u8 | i8; bias = stride-0 C-input row; act 0 none, 1 relu,
# 2 clamp, 3 sigmoid, 4 silu; scale / shift = runtime scalars; colscale = per-column fp32 scales.
FUSED_GOLDEN_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vecops_fused_golden.npz")

FUSED_CASES = [
    # MatmulFusionTest.RuntimePerColumnScaleAndClampAreFused (19, 23, 65)
    {"name": "fz_bf16_scale", "kind": "bf16", "m": 19, "n": 23, "k": 65, "scale": 0.75},
    {"name": "fz_bf16_colscale", "kind": "bf16", "m": 19, "n": 23, "k": 65, "colscale": True},
    {"name": "fz_bf16_bias_clamp", "kind": "bf16", "m": 19, "n": 23, "k": 65, "bias": True, "act": 2,
     "clamp": (-0.25, 0.25)},
    # MatmulFusionTest.MixedBiasNarrowAndActivationsAreFused
    {"name": "fz_bf16_bias_relu_bf16out", "kind": "bf16", "m": 19, "n": 23, "k": 65, "bias": True, "act": 1,
     "out": "bf16"},
    {"name": "fz_bf16_relu", "kind": "bf16", "m": 19, "n": 23, "k": 65, "act": 1},
    {"name": "fz_bf16_sigmoid", "kind": "bf16", "m": 19, "n": 23, "k": 65, "act": 3},
    {"name": "fz_bf16_sigmoid_1x8x129", "kind": "bf16", "m": 1, "n": 8, "k": 129, "act": 3},
    {"name": "fz_bf16_silu_1x8x129", "kind": "bf16", "m": 1, "n": 8, "k": 129, "act": 4},
    {"name": "fz_bf16_bias_silu_1x8x129", "kind": "bf16", "m": 1, "n": 8, "k": 129, "bias": True, "act": 4},
    {"name": "fz_bf16_relu_8x1x129", "kind": "bf16", "m": 8, "n": 1, "k": 129, "act": 1},
    # a shape with whole tiles and edges, every step at once, bf16 out
    {"name": "fz_bf16_all_130x270x200", "kind": "bf16", "m": 130, "n": 270, "k": 200, "bias": True, "colscale": True,
     "scale": 0.375, "shift": -0.125, "act": 4, "out": "bf16"},
    # MatmulFusionTest.IndependentQuantizationAndNativeI8Accumulate: integer bias, per-column scale,
    # requantisation with an output zero point (1, 8, 129)
    {"name": "fz_i8_bias_colscale", "kind": "i8", "m": 1, "n": 8, "k": 129, "bias": True, "colscale": True},
    {"name": "fz_i8_bias_colscale_zp_u8", "kind": "i8", "m": 1, "n": 8, "k": 129, "bias": True, "colscale": True,
     "shift": 7.0, "out": "u8"},
    # bigger and ragged, signed and unsigned byte outputs that saturate on both sides
    {"name": "fz_i8_requant_u8_67x129x515", "kind": "i8", "m": 67, "n": 129, "k": 515, "bias": True, "colscale": True,
     "shift": 128.0, "out": "u8"},
    {"name": "fz_i8_requant_i8_67x129x515", "kind": "i8", "m": 67, "n": 129, "k": 515, "bias": True, "colscale": True,
     "out": "i8"},
    {"name": "fz_i8_scale_relu_67x129x515", "kind": "i8", "m": 67, "n": 129, "k": 515, "scale": -0.001953125, "act": 1},
    {"name": "fz_i8_clamp_35x53x257", "kind": "i8", "m": 35, "n": 53, "k": 257, "colscale": True, "act": 2,
     "clamp": (-20.0, 35.5)},
    {"name": "fz_i8_sigmoid_35x53x257", "kind": "i8", "m": 35, "n": 53, "k": 257, "scale": 0.0001220703125, "act": 3},
    {"name": "fz_i8_silu_256x384x1024", "kind": "i8", "m": 256, "n": 384, "k": 1024, "colscale": True, "act": 4},
    # byte outputs of values outside int32 and of NaN (inf * 0): INT32_MIN before the saturating narrow
    {"name": "fz_i8_huge_u8", "kind": "i8", "m": 5, "n": 40, "k": 64, "scale": 1.0e6, "out": "u8"},
    {"name": "fz_i8_huge_i8", "kind": "i8", "m": 5, "n": 40, "k": 64, "scale": 1.0e6, "out": "i8"},
    {"name": "fz_i8_inf_u8", "kind": "i8", "m": 5, "n": 40, "k": 64, "scale": float("inf"), "out": "u8",
     "zero_rows": True},
    {"name": "fz_i8_inf_i8", "kind": "i8", "m": 5, "n": 40, "k": 64, "scale": float("inf"), "out": "i8",
     "zero_rows": True},
]

FUSED_OUT_DTYPES = {"f32": np.float32, "bf16": np.uint16, "u8": np.uint8, "i8": np.int8}


def make_fused_inputs(case: dict) -> dict:
    """a, b (bf16 bits as uint16, or int8), bias (fp32 / int32 [n] or None), column_scales (fp32 [n] or None)."""
    m, n, k = case["m"], case["n"], case["k"]
    out = {}
    if case["kind"] == "bf16":
        out["a"] = synth.bf16_round(synth.uniform_pm1(11, (m, k)))
        out["b"] = synth.bf16_round(synth.uniform_pm1(12, (n, k)))
        out["bias"] = synth.uniform_pm1(13, (n,)) if case.get("bias") else None
    else:
        out["a"] = synth.int8_sym(11, (m, k))
        out["b"] = synth.int8_sym(12, (n, k))
        if case.get("zero_rows"):
            out["a"][1, :] = 0          # accumulator 0: inf * 0 = NaN
        out["bias"] = (((synth.draws(13, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32)
                       if case.get("bias") else None)
    out["column_scales"] = synth.scales(14, n) if case.get("colscale") else None
    return out


# --- runtime per-row asymmetric quantisation of fp32 activations (matmul/Quantization.h:91-146) ----------
# fp32 values whose quantised bytes show every branch of the conversion: truncation toward zero on both
# sides, saturation at 0 and 255, values outside int32, infinities, NaN, denormals.
QUANT_EDGE_VALUES = [0.0, 0.4, 0.5, 0.99, 1.0, 1.5, 2.5, -0.4, -0.5, -0.99, -1.0, -1.5, -7.0, -7.5, -8.0, -100.0, 247.0,
                     247.5, 248.0, 248.9, 249.0, 300.0, 1e6, 3e9, -3e9, 1e20, -1e20, float("inf"), float("-inf"),
                     float("nan"), -0.0, 2147483520.0, -2147483648.0, 4294967040.0, 1e-40, 254.99, 255.0, 255.5, 256.0,
                     127.5, 128.0]
QUANT_EDGE_MULTIPLIERS = [1.0, 0.5, 3.0]
QUANT_EDGE_ZERO_POINTS = [7, 0, -3]
QUANT_CASES = [
    {"name": "rq_19x21x69", "m": 19, "n": 21, "k": 69, "zp": 7},
    {"name": "rq_67x129x515", "m": 67, "n": 129, "k": 515, "zp": 128},
    {"name": "rq_130x70x1000_zp0", "m": 130, "n": 70, "k": 1000, "zp": 0},
]


# Batched runtime-quantised products (tests/ops/MatmulConversionTestCommon.h:1277-1434): "ref" cases use that test's own
# operand formulas and sizes (tests/ops/MatmulFusionTest.cpp:103-108; it instantiates shared b and shared a - the other two
# combinations are run here on the same formulas), "seeded" cases this repository's generators.
QUANT_BATCHED_CASES = [
    {"name": "rqb_ref_3x5x7x65_a_per_batch_b_shared", "kind": "ref", "batch": 3, "m": 5, "n": 7, "k": 65, "shared_a": False, "shared_b": True},
    {"name": "rqb_ref_3x5x7x65_a_shared_b_per_batch", "kind": "ref", "batch": 3, "m": 5, "n": 7, "k": 65, "shared_a": True, "shared_b": False},
    {"name": "rqb_ref_3x5x7x65_both_per_batch", "kind": "ref", "batch": 3, "m": 5, "n": 7, "k": 65, "shared_a": False, "shared_b": False},
    {"name": "rqb_ref_3x5x7x33_both_shared", "kind": "ref", "batch": 3, "m": 5, "n": 7, "k": 33, "shared_a": True, "shared_b": True},
    {"name": "rqb_4x37x150x300_both_per_batch", "kind": "seeded", "batch": 4, "m": 37, "n": 150, "k": 300, "shared_a": False, "shared_b": False},
    {"name": "rqb_3x130x70x515_a_shared", "kind": "seeded", "batch": 3, "m": 130, "n": 70, "k": 515, "shared_a": True, "shared_b": False},
]


def make_quant_batched_inputs(case):
    """a [batch or 1, M, K] f32, b [batch or 1, N, K] i8, multipliers / row_scales [a's batches * M], correction
    [b's batches * N], column_scales [N], zero_point."""
    import numpy as np
    from vecops_amd import synth
    batch, m, n, k = case["batch"], case["m"], case["n"], case["k"]
    ab, bb = (1 if case["shared_a"] else batch), (1 if case["shared_b"] else batch)
    if case["kind"] == "ref":
        zp = 7
        idx = np.arange(ab * m)
        mult = (4 << (idx % 3)).astype(np.float32)
        rs = (np.float32(1.0) / mult).astype(np.float32)
        flat = np.arange(ab * m * k).reshape(ab * m, k)
        a = ((flat % 7 - 3).astype(np.float32) * rs[:, None]).astype(np.float32).reshape(ab, m, k)
        b = (-3 + (np.arange(bb * n * k) * 5 + 11) % 7).astype(np.int8).reshape(bb, n, k)
        cs = (np.float32(0.03125) + (np.arange(n) % 5).astype(np.float32) * np.float32(0.0078125)).astype(np.float32)
    else:
        zp = 9
        mult = (np.float32(4.0) * (np.float32(1.0) + synth.uniform_pm1(21, (ab * m,)) * np.float32(0.5))).astype(np.float32)
        rs = (np.float32(1.0) / mult).astype(np.float32)
        a = ((synth.uniform_pm1(22, (ab * m, k)) * np.float32(140.0) + np.float32(128 - zp)) / mult[:, None]).astype(np.float32)
        a = a.reshape(ab, m, k)
        b = synth.int8_sym(23, (bb * n, k)).reshape(bb, n, k)
        cs = synth.scales(24, n)
    correction = (-zp * b.astype(np.int64).sum(axis=2)).astype(np.int32).reshape(bb * n)
    return {"a": a, "b": b, "multipliers": mult, "row_scales": rs, "column_scales": cs, "correction": correction,
            "zero_point": zp}


def quant_batched_by_oracle(oracle, inp, batch):
    """The batched pipeline composed from the oracle's pinned pieces, batch by batch: quantise, u8 x s8 sums plus the
    batch's correction row, per-row x per-column dequantisation."""
    import numpy as np
    from oracle import oracle as O
    a, b = inp["a"], inp["b"]
    m, n = a.shape[1], b.shape[1]
    out = np.empty((batch, m, n), np.float32)
    for i in range(batch):
        ia, ib = (0 if a.shape[0] == 1 else i), (0 if b.shape[0] == 1 else i)
        mult, rs = inp["multipliers"][ia * m:(ia + 1) * m], inp["row_scales"][ia * m:(ia + 1) * m]
        q = oracle.quantize_rows(a[ia], mult, inp["zero_point"])
        acc = np.zeros((m, n), np.int32)
        oracle.matmul(q, b[ib], acc, cin=np.broadcast_to(inp["correction"][ib * n:(ib + 1) * n], acc.shape),
                      atom=O.ATOM_I8I32, acc_f64=True, c_bf16=False)
        out[i] = oracle.fused_outputs(acc, np.float32, row_scales=rs, column_scales=inp["column_scales"])
    return out


def quant_edge_inputs():
    """a [3,64] (each row the edge values, zero-padded), identity b [64,64]: the int32 sums are the bytes."""
    import numpy as np
    vals = np.array(QUANT_EDGE_VALUES, dtype=np.float32)
    a = np.zeros((len(QUANT_EDGE_MULTIPLIERS), 64), np.float32)
    a[:, :vals.size] = vals
    return a, np.eye(64, dtype=np.int8), np.array(QUANT_EDGE_MULTIPLIERS, np.float32)


def quant_fma_inputs():
    """Elements whose product a * multiplier rounds up to 16.0 in fp32 while the exact product lies at
    least 2^-23 below it: with zero point -15 two roundings give trunc(16 - 15) = 1, one fused rounding
    trunc(1 - delta) = 0.  Returns (a [1,64], b identity, multipliers [1], zero_point)."""
    import numpy as np
    rng = np.random.default_rng(5)
    found = []
    while len(found) < 64:
        x = rng.uniform(15.5, 16.5, 4096).astype(np.float32)
        mlt = np.float32(rng.uniform(0.97, 1.03))
        for xv in x:
            exact = float(xv) * float(mlt)
            if np.float32(xv) * mlt == np.float32(16.0) and exact < 16.0 - 2.0 ** -22:
                found.append((xv, mlt))
                break
    # one multiplier per row: keep the elements that share the first multiplier, else one row per element
    a = np.array([[f[0] for f in found]], np.float32).T.copy()        # [64,1] -> one element per row
    mult = np.array([f[1] for f in found], np.float32)
    return a, mult


def make_quant_inputs(case):
    import numpy as np
    from vecops_amd import synth
    m, n, k = case["m"], case["n"], case["k"]
    mult = (np.float32(4.0) * (np.float32(1.0) + synth.uniform_pm1(11, (m,)) * np.float32(0.5))).astype(np.float32)
    # activations spread over a little more than the byte range after quantisation, fractions included
    a = ((synth.uniform_pm1(12, (m, k)) * np.float32(140.0) + np.float32(128 - case["zp"])) / mult[:, None]).astype(np.float32)
    b = synth.int8_sym(13, (n, k))
    correction = (-case["zp"] * b.astype(np.int64).sum(axis=1)).astype(np.int32)
    return {"a": a, "b": b, "multipliers": mult, "correction": correction,
            "row_scales": (np.float32(1.0) / mult).astype(np.float32), "column_scales": synth.scales(14, n)}
