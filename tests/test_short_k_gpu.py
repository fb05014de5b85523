"""Products one matrix instruction deep (8 <= K <= 32, 16-bit compute, both operands K-contiguous) on the kernel that loads
its fragments straight from memory (tile_gemm_short_k.hip): what the library runs for a 128 x 128 plan of such a product
whose results leave as they are - fp32, bf16 or f16 into a C with contiguous, aligned rows and N a multiple of four / eight,
no C input, no fused transform; everything else about such shapes stays with the two-stage tile kernel, and is tested here
beside it.  A partial last chunk of K is the row's last eight elements with the overlap zeroed, so K = 8 .. 32 one by one;
rows padded to odd strides (no alignment of the operands is assumed); ragged M and N; batches; narrow outputs.  bf16 against
the oracle, everything against float64 sums of the same operands, and against the 256 x 256 tile's kernel."""
import numpy as np
import pytest

from conftest import rel_err
from vecops_amd import synth
from test_matmul_gpu import dev_bf16, fp32_tol

pytestmark = pytest.mark.gpu


def _request(capi, family="tile_128", split_k=1):
    return capi.family_request(family, capi.SELECT_REQUIRE, split_k=split_k)


@pytest.mark.parametrize("k", list(range(8, 33)))
def test_every_k_against_the_oracle(device, oracle, k):
    """3000 x 3000 x 17 is the benchmark's shape; here every K the kernel takes, on extents that leave part tiles."""
    import torch
    from vecops_amd import capi
    m, n = 200 + k, 264
    a_bits, b_bits = synth.bf16_round(synth.uniform_pm1(k, (m, k))), synth.bf16_round(synth.uniform_pm1(100 + k, (n, k)))
    a, b = dev_bf16(a_bits, device), dev_bf16(b_bits, device)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    other = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul_family(a, b, c, _request(capi))
    capi.matmul_family(a, b, other, _request(capi, "tile_256"))
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a_bits, b_bits, want, acc_f64=True, c_bf16=False)
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)
    assert rel_err(c.cpu().numpy(), other.cpu().numpy()) <= fp32_tol(k)


@pytest.mark.parametrize("kind", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("batch,m,n,k,pad", [(8, 3000, 3000, 17, 0), (1, 129, 257, 31, 3), (3, 65, 130, 9, 1), (1, 1000, 1001, 24, 0),
                                             (1, 64, 128, 32, 0), (2, 300, 520, 8, 5), (1, 1, 4100, 17, 0), (1, 2050, 3, 20, 2),
                                             (1, 4096, 4096, 32, 0)])
@pytest.mark.parametrize("narrow_out", [False, True])
def test_shapes_kinds_and_outputs(device, kind, batch, m, n, k, pad, narrow_out):
    """Operand rows padded by `pad` elements (rows start at any element); fp32 operands are multiplied as bf16."""
    import torch
    from vecops_amd import capi
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[kind]
    gen = torch.Generator(device="cpu").manual_seed(batch * 1000003 + m * 131 + n * 17 + k)
    a = (torch.rand((batch, m, k + pad), generator=gen) * 2 - 1).to(dtype).to(device)[:, :, :k]
    b = (torch.rand((batch, n, k + pad), generator=gen) * 2 - 1).to(dtype).to(device)[:, :, :k]
    out_dtype = torch.float32 if not narrow_out else (torch.bfloat16 if kind == "f32" else dtype)
    c = torch.full((batch, m, n), float("nan"), dtype=out_dtype, device=device)
    if batch == 1:
        a, b, c = a[0], b[0], c[0]
    capi.matmul_family(a, b, c, _request(capi))
    torch.cuda.synchronize()
    ar, br = (a.bfloat16(), b.bfloat16()) if kind == "f32" else (a, b)      # (torch rounds to nearest even, as the kernel does)
    want = torch.matmul(ar.double(), br.double().transpose(-1, -2))
    tol = fp32_tol(k)
    if narrow_out:
        tol += 2.0 ** (-11 if out_dtype == torch.float16 else -8) * 1.01
    assert rel_err(c.double().cpu().numpy(), want.cpu().numpy()) <= tol


@pytest.mark.parametrize("n", [520, 522])
def test_c_input_fused_transform_and_strided_c(device, n):
    """What the short-K kernel leaves to the two-stage kernel, on the same shapes."""
    import torch
    from vecops_amd import capi
    m, k = 333, 17
    gen = torch.Generator(device="cpu").manual_seed(n)
    a = (torch.rand((m, k), generator=gen) * 2 - 1).bfloat16().to(device)
    b = (torch.rand((n, k), generator=gen) * 2 - 1).bfloat16().to(device)
    cin = (torch.rand((m, n), generator=gen) * 2 - 1).to(device)
    want = torch.matmul(a.double(), b.double().t())
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul_family(a, b, c, _request(capi), c_in=cin)
    torch.cuda.synchronize()
    assert rel_err(c.double().cpu().numpy(), (want + cin.double()).cpu().numpy()) <= fp32_tol(k)
    # C as the transposed view of an [N,M] matrix: element by element through the general store
    ct = torch.full((n, m), float("nan"), dtype=torch.float32, device=device)
    capi.matmul_family(a, b, ct.t(), _request(capi))
    torch.cuda.synchronize()
    assert rel_err(ct.t().double().cpu().numpy(), want.cpu().numpy()) <= fp32_tol(k)
    # a fused transform - scale, shift and relu, to bf16 - on a shape the table plans as tile_128
    m2, n2 = 2000, n + 1536
    a2 = (torch.rand((m2, k), generator=gen) * 2 - 1).bfloat16().to(device)
    b2 = (torch.rand((n2, k), generator=gen) * 2 - 1).bfloat16().to(device)
    c16 = torch.full((m2, n2), float("nan"), dtype=torch.bfloat16, device=device)
    ep = capi.epilogue(activation="relu", scale=0.5, shift=0.25)
    plan = capi.plan_matmul_fused(a2, b2, c16, ep)
    assert capi.FAMILY_NAMES[plan.family] == "tile_128" and plan.split_k == 1
    capi.matmul_fused(a2, b2, c16, ep)
    torch.cuda.synchronize()
    fused = torch.clamp(torch.matmul(a2.double(), b2.double().t()) * 0.5 + 0.25, min=0.0)
    assert rel_err(c16.double().cpu().numpy(), fused.cpu().numpy()) <= fp32_tol(k) + 2.0 ** -8 * 1.01


@pytest.mark.parametrize("kind", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("narrow_out", [False, True])
@pytest.mark.parametrize("bias", [False, True])
def test_c_input_of_cs_type(device, kind, narrow_out, bias):
    """A C input of C's own element type with rows like C's - or one row for all (a bias: row stride 0) - is added by the
    short-K kernel itself: batches, ragged M, K = 17."""
    import torch
    from vecops_amd import capi
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[kind]
    batch, m, n, k = 2, 1000, 1032, 17
    gen = torch.Generator(device="cpu").manual_seed(17 + narrow_out + 2 * bias)
    a = (torch.rand((batch, m, k), generator=gen) * 2 - 1).to(dtype).to(device)
    b = (torch.rand((batch, n, k), generator=gen) * 2 - 1).to(dtype).to(device)
    out_dtype = torch.float32 if not narrow_out else (torch.bfloat16 if kind == "f32" else dtype)
    if bias:
        c_in = (torch.rand((batch, 1, n), generator=gen) * 2 - 1).to(out_dtype).to(device).expand(batch, m, n)
    else:
        c_in = (torch.rand((batch, m, n), generator=gen) * 2 - 1).to(out_dtype).to(device)
    c = torch.full((batch, m, n), float("nan"), dtype=out_dtype, device=device)
    capi.matmul_family(a, b, c, _request(capi), c_in=c_in)
    torch.cuda.synchronize()
    ar, br = (a.bfloat16(), b.bfloat16()) if kind == "f32" else (a, b)
    want = torch.matmul(ar.double(), br.double().transpose(-1, -2)) + c_in.double()
    tol = fp32_tol(k) + (2.0 ** (-11 if out_dtype == torch.float16 else -8) * 1.01 if narrow_out else 0.0)
    assert rel_err(c.double().cpu().numpy(), want.cpu().numpy()) <= tol


def _random_cases(count, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        out.append(dict(kind=str(rng.choice(["bf16", "f16", "f32"])), batch=int(rng.choice([1, 1, 2, 5])),
                        m=int(rng.integers(1, 1400)), n=int(rng.choice([4, 8, 12, 100, 128, 132, 1000, 1016, 1028, 2052, 3000, 777])),
                        k=int(rng.integers(8, 33)), pad_a=int(rng.choice([0, 1, 8])), pad_b=int(rng.choice([0, 3, 8])),
                        c_pad=int(rng.choice([0, 0, 8, 5])), narrow=bool(rng.random() < 0.5), c_in=str(rng.choice(["none", "same", "bias", "f32"]))))
    return out


@pytest.mark.parametrize("case", _random_cases(40, 2024), ids=lambda c: "{kind}-{batch}x{m}x{n}x{k}-{c_in}-{out}-pad{pad_a}.{pad_b}.{c_pad}".format(
    out="narrow" if c["narrow"] else "f32", **c))
def test_random_short_products(device, case):
    """Seeded random shapes through the table's own plan (whichever kernel that is): ragged extents, padded operand rows, a
    C whose rows are padded (aligned or not), C inputs of C's type, as a bias row, or of another type."""
    import torch
    from vecops_amd import capi
    kind, batch, m, n, k = case["kind"], case["batch"], case["m"], case["n"], case["k"]
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[kind]
    gen = torch.Generator(device="cpu").manual_seed(m * 7919 + n * 31 + k)
    a = (torch.rand((batch, m, k + case["pad_a"]), generator=gen) * 2 - 1).to(dtype).to(device)[:, :, :k]
    b = (torch.rand((batch, n, k + case["pad_b"]), generator=gen) * 2 - 1).to(dtype).to(device)[:, :, :k]
    out_dtype = torch.float32 if not case["narrow"] else (torch.bfloat16 if kind == "f32" else dtype)
    c = torch.full((batch, m, n + case["c_pad"]), float("nan"), dtype=out_dtype, device=device)[:, :, :n]
    c_in = None
    if case["c_in"] == "same":
        c_in = (torch.rand((batch, m, n), generator=gen) * 2 - 1).to(out_dtype).to(device)
    elif case["c_in"] == "bias":
        c_in = (torch.rand((batch, 1, n), generator=gen) * 2 - 1).to(out_dtype).to(device).expand(batch, m, n)
    elif case["c_in"] == "f32":
        c_in = (torch.rand((batch, m, n), generator=gen) * 2 - 1).to(device)
    if batch == 1:
        a, b, c = a[0], b[0], c[0]
        c_in = None if c_in is None else c_in[0]
    capi.matmul(a, b, c, c_in=c_in)
    torch.cuda.synchronize()
    ar, br = (a.bfloat16(), b.bfloat16()) if kind == "f32" else (a, b)
    want = torch.matmul(ar.double(), br.double().transpose(-1, -2))
    if c_in is not None:
        want = want + c_in.double()
    tol = fp32_tol(k) + (2.0 ** (-11 if out_dtype == torch.float16 else -8) * 1.01 if case["narrow"] else 0.0)
    assert rel_err(c.double().cpu().numpy(), want.cpu().numpy()) <= tol


def test_the_table_plans_the_benchmark_shape_on_it(device):
    """Batch 8 of 3000 x 3000 x 17 plans as tile_128 unsplit - the plan this kernel serves - and K = 33 or a B handed
    over as [K,N] still give right results on the two-stage kernel."""
    import torch
    from vecops_amd import capi
    a = torch.zeros((8, 3000, 17), dtype=torch.bfloat16, device=device)
    c = torch.empty((8, 3000, 3000), dtype=torch.float32, device=device)
    plan = capi.plan_matmul(a, a, c)
    assert capi.FAMILY_NAMES[plan.family] == "tile_128" and plan.split_k == 1
    gen = torch.Generator(device="cpu").manual_seed(7)
    for k, b_as_kn in ((33, False), (17, True)):
        x = (torch.rand((500, k), generator=gen) * 2 - 1).bfloat16().to(device)
        y = (torch.rand((k, 520) if b_as_kn else (520, k), generator=gen) * 2 - 1).bfloat16().to(device)
        yv = y.t() if b_as_kn else y
        out = torch.full((500, 520), float("nan"), dtype=torch.float32, device=device)
        capi.matmul_family(x, yv, out, _request(capi))
        torch.cuda.synchronize()
        want = torch.matmul(x.double(), yv.double().t())
        assert rel_err(out.double().cpu().numpy(), want.cpu().numpy()) <= fp32_tol(k)
