"""Fused output transforms (scales, shift, relu / clamp / sigmoid / silu, requantised byte outputs).

CPU: the oracle's restatement (vo_fused_outputs on the oracle's accumulators) against golden vectors written
by the real vecops CPU matmul with the transforms its own tests attach (tests/golden/make_fused_golden.py),
and against that library directly where it is built.
GPU: vecops_hip_matmul_fused against the same golden vectors and against the oracle on shapes that reach
every store path of the kernels (staged fast path, general path, split-K reduction, K = 0).

Tolerances: int8 operands give exact int32 accumulators, so every transform made of multiplies, adds, max and
min and every conversion is compared bit for bit; sigmoid and silu within 8e-4 (the reference tests' own fp32
bound, tests/ops/MatmulConversionTestCommon.h:79-83; the exact exp, the reference's vector exp and the GPU's
hardware exp differ by a few ulp).  bf16 operands: fp32 sums differ by summation order, bound 2e-6 * K/32 as
for the unfused product (16-bit outputs: one bf16 ulp).
"""
import numpy as np
import pytest

from conftest import rel_err
from golden_cases import FUSED_CASES, FUSED_GOLDEN_PATH, FUSED_OUT_DTYPES, make_fused_inputs
from oracle import oracle as O
from vecops_amd import synth

GOLDEN = np.load(FUSED_GOLDEN_PATH)
SMOOTH = (3, 4)  # sigmoid, silu: not bit-comparable


def oracle_fused(oracle, case, inp):
    """Oracle accumulators (C-input row added) through the oracle's output transform."""
    m, n = case["m"], case["n"]
    integer = case["kind"] == "i8"
    acc = np.zeros((m, n), np.int32 if integer else np.float32)
    cin = None
    if inp["bias"] is not None:
        cin = np.broadcast_to(inp["bias"], (m, n))
    oracle.matmul(inp["a"], inp["b"], acc, cin=cin, atom=O.ATOM_I8I32 if integer else O.ATOM_BF16F32, acc_f64=True,
                  c_bf16=False)
    lo, hi = case.get("clamp", (0.0, 0.0))
    return oracle.fused_outputs(acc, FUSED_OUT_DTYPES[case.get("out", "f32")], activation=case.get("act", 0),
                                scale=case.get("scale"), shift=case.get("shift"),
                                column_scales=inp["column_scales"], lo=lo, hi=hi)


def check(case, got, want):
    out = case.get("out", "f32")
    integer = case["kind"] == "i8"
    smooth = case.get("act", 0) in SMOOTH
    assert got.dtype == want.dtype and got.shape == want.shape
    if out in ("u8", "i8"):
        assert np.array_equal(got, want)
    elif integer and not smooth:
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))          # bit-exact, signed zeros included
    elif out == "bf16":
        assert rel_err(synth.bf16_to_f32(got), synth.bf16_to_f32(want)) <= 2 ** -7
    else:
        tol = 8e-4 if smooth else 2e-6 * max(1.0, case["k"] / 32)
        assert rel_err(got, want) <= tol


@pytest.mark.parametrize("case", FUSED_CASES, ids=[c["name"] for c in FUSED_CASES])
def test_oracle_reproduces_fused_golden(oracle, case):
    inp = make_fused_inputs(case)
    with np.errstate(over="ignore", invalid="ignore"):
        got = oracle_fused(oracle, case, inp)
    check(case, got, GOLDEN[case["name"]])


def test_golden_byte_cases_reach_both_rails():
    """The saturating cases really saturate on both sides and the NaN / out-of-range cases hold the
    INT32_MIN outcome (0 for u8, -128 for i8), so a wrong conversion rule cannot pass unnoticed."""
    u8 = GOLDEN["fz_i8_requant_u8_67x129x515"]
    assert (u8 == 0).any() and (u8 == 255).any() and ((u8 > 0) & (u8 < 255)).any()
    i8 = GOLDEN["fz_i8_requant_i8_67x129x515"]
    assert (i8 == -128).any() and (i8 == 127).any()
    assert (GOLDEN["fz_i8_inf_u8"] == 0).all()                      # +inf, -inf and NaN all give 0
    assert (GOLDEN["fz_i8_inf_i8"] == -128).all()
    huge = GOLDEN["fz_i8_huge_u8"]
    assert (huge == 255).any() and (huge == 0).any()


def test_reference_agrees_with_fused_golden(reference):
    """Where the real library is built: regenerating two cases gives the committed bytes."""
    for name in ("fz_i8_requant_u8_67x129x515", "fz_bf16_bias_clamp"):
        case = next(c for c in FUSED_CASES if c["name"] == name)
        inp = make_fused_inputs(case)
        lo, hi = case.get("clamp", (0.0, 0.0))
        got = reference.matmul_fused(inp["a"], inp["b"], inp["bias"], FUSED_OUT_DTYPES[case.get("out", "f32")],
                                     activation=case.get("act", 0), scale=case.get("scale"), shift=case.get("shift"),
                                     column_scales=inp["column_scales"], lo=lo, hi=hi)
        assert np.array_equal(got, GOLDEN[name])


def test_fused_outputs_closed_forms(oracle):
    """The oracle's transform against numpy float32 arithmetic written independently for each step."""
    rng = np.random.default_rng(5)
    acc = rng.integers(-200000, 200000, size=(9, 31)).astype(np.int32)
    cs = rng.uniform(0.001, 0.01, size=31).astype(np.float32)
    rs = rng.uniform(0.5, 2.0, size=9).astype(np.float32)
    f = acc.astype(np.float32)
    want = ((f * rs[:, None]) * cs[None, :]) * np.float32(0.5) + np.float32(3.25)
    got = oracle.fused_outputs(acc, np.float32, row_scales=rs, column_scales=cs, scale=0.5, shift=3.25)
    assert np.array_equal(got, want)
    assert np.array_equal(oracle.fused_outputs(acc, np.float32, activation=1), np.maximum(f, 0))
    assert np.array_equal(oracle.fused_outputs(acc, np.float32, activation=2, lo=-5.0, hi=7.0), np.clip(f, -5, 7))
    x = (f * np.float32(1e-4)).astype(np.float64)
    sig = oracle.fused_outputs(acc, np.float32, scale=1e-4, activation=3)
    assert np.allclose(sig, 1 / (1 + np.exp(-x)), rtol=1e-6, atol=0)
    silu = oracle.fused_outputs(acc, np.float32, scale=1e-4, activation=4)
    assert np.allclose(silu, x / (1 + np.exp(-x)), rtol=1e-6, atol=1e-30)
    # byte outputs: truncation toward zero, both rails, and the INT32_MIN rule
    v = np.array([[-1.9, -0.5, 0.5, 1.9, 254.9, 255.0, 300.0, -129.0, 127.9, 3e9, -3e9, np.inf, -np.inf, np.nan]],
                 np.float32)
    assert oracle.fused_outputs(v, np.uint8).tolist() == [[0, 0, 0, 1, 254, 255, 255, 0, 127, 0, 0, 0, 0, 0]]
    assert oracle.fused_outputs(v, np.int8).tolist() == [[-1, 0, 0, 1, 127, 127, 127, -128, 127, -128, -128, -128,
                                                          -128, -128]]
    # relu and clamp of NaN follow max_ps / min_ps (second operand), -0.0 becomes +0.0 under relu
    z = oracle.fused_outputs(np.array([[np.nan, -0.0]], np.float32), np.float32, activation=1)
    assert z.view(np.uint32).tolist() == [[0, 0]]
    assert oracle.fused_outputs(np.array([[np.nan]], np.float32), np.float32, activation=2, lo=-1.0, hi=2.0)[0, 0] == -1.0


# ---- GPU ------------------------------------------------------------------------------------------

def _dev(arr, device, bf16=False):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(arr).view(np.int16) if bf16 else np.ascontiguousarray(arr)).to(device)
    return t.view(torch.bfloat16) if bf16 else t


def _torch_out(kind, shape, device):
    import torch
    dt = {"f32": torch.float32, "bf16": torch.bfloat16, "u8": torch.uint8, "i8": torch.int8}[kind]
    if kind in ("f32", "bf16"):
        return torch.full(shape, float("nan"), dtype=dt, device=device)
    return torch.full(shape, 77, dtype=dt, device=device)


def _host(c, kind):
    import torch
    if kind == "bf16":
        return c.view(torch.int16).cpu().numpy().view(np.uint16)
    return c.cpu().numpy()


def run_gpu(case, inp, device, c=None, row_scales=None):
    import torch
    from vecops_amd import capi
    bf16 = case["kind"] == "bf16"
    a, b = _dev(inp["a"], device, bf16), _dev(inp["b"], device, bf16)
    m, n = case["m"], case["n"]
    out = case.get("out", "f32")
    if c is None:
        c = _torch_out(out, (m, n), device)
    cin = None
    if inp["bias"] is not None:
        cin = _dev(inp["bias"], device).reshape(1, n).expand(m, n)          # row stride 0
    cs = _dev(inp["column_scales"], device) if inp["column_scales"] is not None else None
    rs = _dev(row_scales, device) if row_scales is not None else None
    ep = capi.epilogue(activation=case.get("act", 0), scale=case.get("scale"), shift=case.get("shift"),
                       row_scales=rs, column_scales=cs, clamp=case.get("clamp", (0.0, 0.0)))
    capi.matmul_fused(a, b, c, ep, c_in=cin)
    torch.cuda.synchronize()
    return _host(c, out)


@pytest.mark.gpu
@pytest.mark.parametrize("case", FUSED_CASES, ids=[c["name"] for c in FUSED_CASES])
def test_gpu_reproduces_fused_golden(device, case):
    got = run_gpu(case, make_fused_inputs(case), device)
    check(case, got, GOLDEN[case["name"]])


# shapes that reach the staged fast path on whole and edge tiles of every tile family, split-K and the 64 tile
GPU_SHAPES = [(256, 512, 256), (300, 260, 192), (2457, 1221, 72), (4187, 900, 72), (1938, 900, 72), (63, 40, 4096)]
GPU_VARIANTS = [
    {"kind": "i8", "bias": True, "colscale": True, "shift": 3.0, "out": "u8"},
    {"kind": "i8", "bias": True, "colscale": True, "out": "i8"},
    {"kind": "i8", "colscale": True, "scale": 0.5, "act": 1},
    {"kind": "i8", "bias": True, "scale": 0.001, "act": 2, "clamp": (-30.0, 41.5)},
    {"kind": "i8", "scale": 1e-4, "act": 4},
    {"kind": "i8"},                                                      # int32 sums leaving as plain floats
    {"kind": "bf16", "bias": True, "act": 1, "out": "bf16"},
    {"kind": "bf16", "bias": True, "colscale": True, "scale": 0.375, "shift": -0.125, "act": 4},
    {"kind": "bf16", "act": 3, "out": "bf16"},
]


@pytest.mark.gpu
@pytest.mark.parametrize("shape", GPU_SHAPES, ids=["x".join(map(str, s)) for s in GPU_SHAPES])
@pytest.mark.parametrize("variant", range(len(GPU_VARIANTS)))
def test_gpu_fused_against_oracle(device, oracle, shape, variant):
    case = dict(GPU_VARIANTS[variant], m=shape[0], n=shape[1], k=shape[2])
    inp = make_fused_inputs(case)
    got = run_gpu(case, inp, device)
    with np.errstate(over="ignore", invalid="ignore"):
        want = oracle_fused(oracle, case, inp)
    check(case, got, want)


@pytest.mark.gpu
def test_gpu_fused_row_and_column_scales_equal_dequant(device):
    """Row and column scales on int32 sums are the dequantisation: same bits as vecops_hip_matmul_i8_dequant,
    rank 2 (the kernels' dequantisation stage) and rank 3 (row scales indexed [batch][M])."""
    import torch
    from vecops_amd import capi
    m, n, k, batch = 130, 270, 520, 3
    a = _dev(synth.int8_sym(1, (batch, m, k)), device)
    b = _dev(synth.int8_sym(2, (batch, n, k)), device)
    rs = _dev(synth.scales(3, (batch, m)), device)
    cs = _dev(synth.scales(4, (n,)), device)
    fused = torch.full((batch, m, n), float("nan"), device=device)
    capi.matmul_fused(a, b, fused, capi.epilogue(row_scales=rs, column_scales=cs))
    for i in range(batch):
        plain = torch.full((m, n), float("nan"), device=device)
        capi.matmul_i8_dequant(a[i], b[i], rs[i], cs, plain)
        assert torch.equal(fused[i].view(torch.int32), plain.view(torch.int32))
        one = torch.full((m, n), float("nan"), device=device)
        capi.matmul_fused(a[i], b[i], one, capi.epilogue(row_scales=rs[i].contiguous(), column_scales=cs))
        assert torch.equal(one.view(torch.int32), plain.view(torch.int32))


@pytest.mark.gpu
def test_gpu_fused_strided_outputs_and_full_c_in(device, oracle):
    """General store path: C with a column stride, an unaligned base, and a full [M,N] C-input."""
    import torch
    from vecops_amd import capi
    m, n, k = 150, 77, 96
    case = {"kind": "i8", "m": m, "n": n, "k": k, "colscale": True, "act": 1, "out": "f32"}
    inp = make_fused_inputs(case)
    cin_host = ((synth.draws(21, m * n) % np.uint64(20001)).astype(np.int64) - 10000).astype(np.int32).reshape(m, n)
    acc = np.zeros((m, n), np.int32)
    oracle.matmul(inp["a"], inp["b"], acc, cin=cin_host, atom=O.ATOM_I8I32, acc_f64=True, c_bf16=False)
    want = oracle.fused_outputs(acc, np.float32, activation=1, column_scales=inp["column_scales"])
    a, b = _dev(inp["a"], device), _dev(inp["b"], device)
    cin = _dev(cin_host, device)
    cs = _dev(inp["column_scales"], device)
    ep = capi.epilogue(activation="relu", column_scales=cs)
    wide = torch.full((m, 2 * n), float("nan"), device=device)
    capi.matmul_fused(a, b, wide[:, ::2], ep, c_in=cin)                       # column stride 2
    assert np.array_equal(wide[:, ::2].cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert torch.isnan(wide[:, 1::2]).all()
    flat = torch.full((m * n + 1,), float("nan"), device=device)
    off = flat[1:].view(m, n)                                                 # 4-byte aligned base only
    capi.matmul_fused(a, b, off, ep, c_in=cin)
    assert np.array_equal(off.cpu().numpy().view(np.uint32), want.view(np.uint32))
    dense = torch.full((m, n), float("nan"), device=device)                   # staged path with a full C-input
    capi.matmul_fused(a, b, dense, ep, c_in=cin)
    assert np.array_equal(dense.cpu().numpy().view(np.uint32), want.view(np.uint32))
    # byte output with an odd row stride: element stores
    case8 = dict(case, out="u8", shift=100.0)
    want8 = oracle.fused_outputs(acc, np.uint8, activation=1, column_scales=inp["column_scales"], shift=100.0)
    buf = torch.full((m, n + 2), 9, dtype=torch.uint8, device=device)
    capi.matmul_fused(a, b, buf[:, :n], capi.epilogue(activation="relu", column_scales=cs, shift=100.0), c_in=cin)
    assert np.array_equal(buf[:, :n].cpu().numpy(), want8)
    assert (buf[:, n:] == 9).all()


@pytest.mark.gpu
def test_gpu_fused_zero_k_and_validation(device):
    import torch
    from vecops_amd import capi
    m, n = 5, 12
    a = torch.zeros((m, 0), dtype=torch.bfloat16, device=device)
    b = torch.zeros((n, 0), dtype=torch.bfloat16, device=device)
    bias = torch.linspace(-2, 2, n, device=device)
    c = torch.full((m, n), float("nan"), device=device)
    capi.matmul_fused(a, b, c, capi.epilogue(activation="relu", shift=0.5), c_in=bias.reshape(1, n).expand(m, n))
    torch.cuda.synchronize()
    assert torch.equal(c, torch.clamp(bias + 0.5, min=0).expand(m, n))         # transform(C_in) for an empty sum
    a8 = torch.zeros((m, 16), dtype=torch.int8, device=device)
    b8 = torch.zeros((n, 16), dtype=torch.int8, device=device)
    with pytest.raises(capi.VecopsHipError) as info:                           # int8 sums cannot leave as bf16
        capi.matmul_fused(a8, b8, torch.zeros((m, n), dtype=torch.bfloat16, device=device), capi.epilogue())
    assert info.value.code == 2
    bad = capi.epilogue()
    bad.activation = 9
    with pytest.raises(capi.VecopsHipError) as info:
        capi.matmul_fused(a8, b8, c, bad)
    assert info.value.code == 1


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(19, 23, 65), (32, 64, 128), (300, 270, 515)], ids=["19x23x65", "32x64x128", "300x270x515"])
def test_gpu_dual_asymmetric_u8(device, oracle, shape):
    """Both operands asymmetric uint8 with zero points 3 and 5: the int32 correction matrix
    -za*sum(b) - zb*sum(a) + k*za*zb comes in as C-input and the sums leave through a fused scale
    (tests/ops/MatmulConversionTestCommon.h:763-866, MatmulFusionTest.DualAsymmetricU8UsesRowAndColumnCorrection)."""
    import torch
    from vecops_amd import capi
    m, n, k = shape
    za, zb = 3, 5
    a = ((synth.draws(31, m * k) % np.uint64(7)).astype(np.int64) + za).astype(np.uint8).reshape(m, k)
    b = ((synth.draws(32, n * k) % np.uint64(7)).astype(np.int64) + zb).astype(np.uint8).reshape(n, k)
    sum_a = a.astype(np.int64).sum(axis=1)
    sum_b = b.astype(np.int64).sum(axis=1)
    corr = (-za * sum_b[None, :] - zb * sum_a[:, None] + k * za * zb).astype(np.int32)
    # closed form: the corrected sum is the product of the zero-point-free values
    exact = (a.astype(np.int64) - za) @ (b.astype(np.int64) - zb).T
    want = exact.astype(np.float32) * np.float32(0.0625)
    acc = np.zeros((m, n), np.int32)
    oracle.matmul(a, b, acc, cin=corr, atom=O.ATOM_I8I32, acc_f64=True, c_bf16=False)
    assert np.array_equal(oracle.fused_outputs(acc, np.float32, scale=0.0625), want)
    c = torch.full((m, n), float("nan"), device=device)
    capi.matmul_fused(_dev(a, device), _dev(b, device), c, capi.epilogue(scale=0.0625), c_in=_dev(corr, device))
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))
