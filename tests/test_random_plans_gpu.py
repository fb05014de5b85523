"""Seeded random products through the rule table's own plans: extents around the tile sizes and the one-workgroup-per-unit
band, both B layouts, padded rows, batches, C inputs, fp32 / bf16 / int32 outputs - bf16 and f16 against float64 sums of the
same operands (the bound is the fp32 accumulation's: 2e-6 * max(1, K / 32) of max(1, |c|), and bf16 outputs within half
a unit of their last place more), int8 exactly.  What the oracle checks case by case elsewhere is here swept: the point is
that no plan the table can make from these ingredients mis-addresses a tile."""
import numpy as np
import pytest

from conftest import rel_err
from test_matmul_gpu import fp32_tol

pytestmark = pytest.mark.gpu


def _extent(rng, choices):
    base = int(rng.choice(choices))
    return max(1, base + int(rng.choice([0, 0, 0, -1, 1, -8, 8, 24, -40, 100])))


def _cases(kind, count, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        m = _extent(rng, [64, 128, 256, 384, 512, 768, 1024, 1536, 2048])
        n = _extent(rng, [64, 128, 256, 512, 1024, 2048, 3072, 4096])
        if rng.random() < 0.6:
            n = (n + 7) // 8 * 8                              # rows of a [K,N] operand stay 16-byte aligned
        k = int(rng.choice([64, 128, 512, 576, 1024, 2048, 4096, 8192])) + int(rng.choice([0, 0, 0, 0, 8, 16, 64, -24]))
        if 2.0 * m * n * k > 2.0 * 2048 * 4096 * 4096:
            k = max(64, k // 4)
        batch = int(rng.choice([1, 1, 1, 2, 3])) if m * n <= 1 << 20 else 1
        out.append(dict(kind=kind, m=m, n=n, k=max(8, k), batch=batch, b_as_kn=bool(rng.random() < 0.5),
                        pad_a=int(rng.choice([0, 0, 8, 64])), pad_b=int(rng.choice([0, 0, 8, 64])),
                        c_in=bool(rng.random() < 0.3), narrow_out=bool(rng.random() < 0.5)))
    return out


CASES = _cases("bf16", 28, 101) + _cases("f16", 8, 202) + _cases("i8", 16, 303)


@pytest.mark.parametrize("case", CASES, ids=lambda c: "{kind}-{batch}x{m}x{n}x{k}-{lay}{cin}{out}-pad{pad_a}.{pad_b}".format(
    lay="kn" if c["b_as_kn"] else "nk", cin="-cin" if c["c_in"] else "", out="-narrow" if c["narrow_out"] else "", **c))
def test_random_product_through_the_rule_table(device, case):
    import torch
    from vecops_amd import capi
    kind, m, n, k, batch = case["kind"], case["m"], case["n"], case["k"], case["batch"]
    gen = torch.Generator(device="cpu").manual_seed(m * 131 + n * 17 + k)
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "i8": torch.int8}[kind]

    def operand(rows, cols, pad):
        """[batch, rows, cols] as a view of rows padded by `pad` elements."""
        if kind == "i8":
            store = torch.randint(-128, 128, (batch, rows, cols + pad), generator=gen, dtype=torch.int8)
        else:
            store = (torch.rand((batch, rows, cols + pad), generator=gen) * 2 - 1).to(dtype)
        return store.to(device)[:, :, :cols]

    a = operand(m, k, case["pad_a"])
    if case["b_as_kn"]:
        b = operand(k, n, case["pad_b"]).transpose(1, 2)          # the [N,K] view of a [K,N] matrix
    else:
        b = operand(n, k, case["pad_b"])
    exact = kind == "i8"
    out_dtype = torch.int32 if exact else (dtype if case["narrow_out"] else torch.float32)
    c_in = None
    if case["c_in"]:
        c_in = (torch.randint(-1000, 1000, (batch, m, n), generator=gen, dtype=torch.int32) if exact
                else (torch.rand((batch, m, n), generator=gen) * 2 - 1).to(out_dtype)).to(device)
    c = torch.full((batch, m, n), -7 if exact else float("nan"), dtype=out_dtype, device=device)
    if batch == 1:
        a, b, c = a[0], b[0], c[0]
        c_in = None if c_in is None else c_in[0]
    capi.matmul(a, b, c, c_in=c_in)
    torch.cuda.synchronize()
    if exact:
        want = torch.matmul(a.double(), b.double().transpose(-1, -2))     # exact: |sums| < 2^53
        if c_in is not None:
            want = want + c_in.double()
        assert torch.equal(c.to(torch.int64), want.to(torch.int64))
        return
    want = torch.matmul(a.double(), b.double().transpose(-1, -2))
    if c_in is not None:
        want = want + c_in.double()
    tol = fp32_tol(k)
    if out_dtype != torch.float32:
        tol += 2.0 ** (-8 if kind == "bf16" else -11) * 1.01                # the output's own rounding
    assert rel_err(c.double().cpu().numpy(), want.cpu().numpy()) <= tol


PACKED_CASES = _cases("bf16", 10, 404) + _cases("i8", 8, 505) + _cases("f16", 4, 606)


@pytest.mark.parametrize("case", PACKED_CASES, ids=lambda c: "{kind}-{batch}x{m}x{n}x{k}-pad{pad_a}{cin}{out}".format(
    cin="-cin" if c["c_in"] else "", out="-narrow" if c["narrow_out"] else "", **c))
def test_random_product_with_prepacked_b(device, case):
    """The same sweep with B packed by vecops_hip_pack_b (one packed operand for every batch): whatever the table plans
    for the pack, against float64 sums (int8 exactly)."""
    import torch
    from vecops_amd import capi
    kind, m, n, k, batch = case["kind"], case["m"], case["n"], case["k"], case["batch"]
    gen = torch.Generator(device="cpu").manual_seed(m * 7 + n * 13 + k)
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "i8": torch.int8}[kind]
    exact = kind == "i8"
    if exact:
        a = torch.randint(-128, 128, (batch, m, k + case["pad_a"]), generator=gen, dtype=torch.int8).to(device)[:, :, :k]
        b = torch.randint(-128, 128, (n, k), generator=gen, dtype=torch.int8).to(device)
    else:
        a = (torch.rand((batch, m, k + case["pad_a"]), generator=gen) * 2 - 1).to(dtype).to(device)[:, :, :k]
        b = (torch.rand((n, k), generator=gen) * 2 - 1).to(dtype).to(device)
    out_dtype = torch.int32 if exact else (dtype if case["narrow_out"] else torch.float32)
    c_in = None
    if case["c_in"]:
        c_in = (torch.randint(-1000, 1000, (batch, m, n), generator=gen, dtype=torch.int32) if exact
                else (torch.rand((batch, m, n), generator=gen) * 2 - 1).to(out_dtype)).to(device)
    c = torch.full((batch, m, n), -7 if exact else float("nan"), dtype=out_dtype, device=device)
    if batch == 1:
        a, c = a[0], c[0]
        c_in = None if c_in is None else c_in[0]
    packed = capi.pack_b(b)
    capi.matmul_packed_b(a, packed, c, c_in=c_in)
    torch.cuda.synchronize()
    want = torch.matmul(a.double(), b.double().t())
    if c_in is not None:
        want = want + c_in.double()
    if exact:
        assert torch.equal(c.to(torch.int64), want.to(torch.int64))
        return
    tol = fp32_tol(k)
    if out_dtype != torch.float32:
        tol += 2.0 ** (-8 if kind == "bf16" else -11) * 1.01
    assert rel_err(c.double().cpu().numpy(), want.cpu().numpy()) <= tol


F32_CASES = _cases("f32", 12, 707)


@pytest.mark.parametrize("case", F32_CASES, ids=lambda c: "f32-{batch}x{m}x{n}x{k}-{lay}{cin}-pad{pad_a}.{pad_b}".format(
    lay="kn" if c["b_as_kn"] else "nk", cin="-cin" if c["c_in"] else "", **c))
def test_random_fp32_compute_product(device, case):
    """fp32 operands multiplied in fp32 (the ring-of-stages kernel among the plans): against float64 sums."""
    import torch
    from vecops_amd import capi
    from test_matmul_gpu import fp32_compute_tol
    m, n, k, batch = case["m"], case["n"], case["k"], case["batch"]
    gen = torch.Generator(device="cpu").manual_seed(m * 3 + n * 5 + k)

    def operand(rows, cols, pad):
        return (torch.rand((batch, rows, cols + pad), generator=gen) * 2 - 1).to(device)[:, :, :cols]
    a = operand(m, k, case["pad_a"])
    b = operand(k, n, case["pad_b"]).transpose(1, 2) if case["b_as_kn"] else operand(n, k, case["pad_b"])
    c_in = (torch.rand((batch, m, n), generator=gen) * 2 - 1).to(device) if case["c_in"] else None
    c = torch.full((batch, m, n), float("nan"), dtype=torch.float32, device=device)
    if batch == 1:
        a, b, c = a[0], b[0], c[0]
        c_in = None if c_in is None else c_in[0]
    capi.matmul(a, b, c, c_in=c_in, compute=capi.COMPUTE_F32)
    torch.cuda.synchronize()
    want = torch.matmul(a.double(), b.double().transpose(-1, -2))
    if c_in is not None:
        want = want + c_in.double()
    assert rel_err(c.double().cpu().numpy(), want.cpu().numpy()) <= fp32_compute_tol(k)
