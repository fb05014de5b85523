"""The 192 x 192 workgroup tile (family tile_192), through the C ABI: 96 x 96 a wavefront on the 16x16 matrix instructions,
for bf16, f16 and signed 8-bit operands whose loads write LDS themselves (16-byte aligned bases and rows; both K-contiguous,
or 16-bit ones with B handed over as [K,N]).
The rule table plans it where its count fits one round that the other tiles' counts do not (3000^3: 256 tiles; 768 x 11008:
232).  bf16 against the oracle, f16 against float64 sums, int8 bit-exact (int32 sums, dequantised fp32); ragged extents, a K
that is no whole number of K tiles, K splits, batches, C inputs, narrow outputs; refusals where it cannot serve."""
import numpy as np
import pytest

from conftest import rel_err
from vecops_amd import synth
from test_matmul_gpu import dev_bf16, fp32_tol

pytestmark = pytest.mark.gpu


def _require(capi, split_k=0):
    return capi.family_request("tile_192", capi.SELECT_REQUIRE, split_k=split_k)


@pytest.mark.parametrize("m,n,k,split", [(192, 192, 512, 1), (3000, 3000, 264, 1), (500, 391, 1024, 1), (97, 1000, 520, 1),
                                         (770, 580, 2048, 3), (1, 200, 512, 1), (400, 100, 8, 1), (1000, 1000, 4096, 2)])
def test_bf16_against_the_oracle(device, oracle, m, n, k, split):
    import torch
    from vecops_amd import capi
    a_bits, b_bits = synth.bf16_round(synth.uniform_pm1(1, (m, k))), synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    a, b = dev_bf16(a_bits, device), dev_bf16(b_bits, device)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    request = _require(capi, split)
    plan = capi.plan_matmul_family(a, b, c, request)
    assert capi.FAMILY_NAMES[plan.family] == "tile_192" and plan.split_k == split
    capi.matmul_family(a, b, c, request)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a_bits, b_bits, want, acc_f64=True, c_bf16=False)
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("m,n,k,split", [(192, 192, 512, 1), (3000, 3000, 264, 1), (500, 392, 1024, 1), (97, 1000, 520, 1),
                                         (770, 584, 2048, 3), (1, 200, 512, 1), (400, 104, 8, 1), (1000, 1000, 4096, 2),
                                         (300, 8, 640, 1)])
def test_b_as_k_by_n(device, oracle, kind, m, n, k, split):
    """B stored [K,N] and handed over as the strided [N,K] view (N a multiple of eight): the tile lies [k][n] in LDS, 24
    chunk slots a row, and the fragment reads transpose.  bf16 against the oracle, f16 against float64 sums."""
    import torch
    from vecops_amd import capi
    request = _require(capi, split)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    if kind == "bf16":
        a_bits, b_bits = synth.bf16_round(synth.uniform_pm1(1, (m, k))), synth.bf16_round(synth.uniform_pm1(2, (k, n)))
        a, b = dev_bf16(a_bits, device), dev_bf16(b_bits, device)
        assert capi.FAMILY_NAMES[capi.plan_matmul_family(a, b.t(), c, request).family] == "tile_192"
        capi.matmul_family(a, b.t(), c, request)
        torch.cuda.synchronize()
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a_bits, np.ascontiguousarray(b_bits.T), want, acc_f64=True, c_bf16=False)
    else:
        ha, hb = synth.uniform_pm1(1, (m, k)).astype(np.float16), synth.uniform_pm1(2, (k, n)).astype(np.float16)
        a, b = torch.from_numpy(ha).to(device), torch.from_numpy(hb).to(device)
        capi.matmul_family(a, b.t(), c, request)
        torch.cuda.synchronize()
        want = (ha.astype(np.float64) @ hb.astype(np.float64)).astype(np.float32)
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)


@pytest.mark.parametrize("kind", ["bf16", "f16"])
def test_batches_c_input_and_narrow_output(device, kind):
    import torch
    from vecops_amd import capi
    dtype = torch.bfloat16 if kind == "bf16" else torch.float16
    batch, m, n, k = 3, 385, 577, 776
    gen = torch.Generator(device="cpu").manual_seed(11)
    a = (torch.rand((batch, m, k + 8), generator=gen) * 2 - 1).to(dtype).to(device)[:, :, :k]     # rows padded by 16 bytes
    b = (torch.rand((batch, n, k), generator=gen) * 2 - 1).to(dtype).to(device)
    c_in = (torch.rand((batch, m, n), generator=gen) * 2 - 1).to(dtype).to(device)
    c = torch.full((batch, m, n), float("nan"), dtype=dtype, device=device)
    capi.matmul_family(a, b, c, _require(capi), c_in=c_in)
    torch.cuda.synchronize()
    want = torch.matmul(a.double(), b.double().transpose(1, 2)) + c_in.double()
    assert rel_err(c.double().cpu().numpy(), want.cpu().numpy()) <= fp32_tol(k) + 2.0 ** (-8 if kind == "bf16" else -11) * 1.01


@pytest.mark.parametrize("m,n,k,split", [(192, 192, 256, 1), (1000, 777, 1040, 1), (2500, 2900, 512, 1), (300, 5000, 4096, 2)])
def test_int8_sums_bit_exact(device, m, n, k, split):
    import torch
    from vecops_amd import capi
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    c = torch.full((m, n), -7, dtype=torch.int32, device=device)
    capi.matmul_family(ta, tb, c, _require(capi, split))
    torch.cuda.synchronize()
    want = a.astype(np.int64) @ b.astype(np.int64).T
    assert np.array_equal(c.cpu().numpy().astype(np.int64), want)


def test_int8_dequantisation_on_the_tables_plan(device, oracle):
    """768 x 11008 x 2048 in int8: 232 tiles of 192 x 192, one round (129 big tiles would leave half the units idle); the
    dequantised output bit-exact against the oracle."""
    import torch
    from vecops_amd import capi
    m, n, k = 768, 11008, 2048
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    correction = ((synth.draws(5, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32)
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    plan = capi.plan_matmul(ta, tb, torch.empty((m, n), dtype=torch.int32, device=device))
    assert capi.FAMILY_NAMES[plan.family] == "tile_192" and plan.split_k == 1
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul_i8_dequant(ta, tb, torch.from_numpy(rs).to(device), torch.from_numpy(cs).to(device), c,
                           correction=torch.from_numpy(correction).to(device))
    torch.cuda.synchronize()
    want = oracle.matmul_i8_dequant(a, b, rs, cs, correction)
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_the_table_plans_one_round_of_them(device):
    """3000^3 in bf16, B as [N,K] or as [K,N]: 256 tiles of 192 x 192."""
    import torch
    from vecops_amd import capi
    gen = torch.Generator(device="cpu").manual_seed(3)
    a = (torch.randn((3000, 3000), generator=gen) * 0.05).bfloat16().to(device)
    b = (torch.randn((3000, 3000), generator=gen) * 0.05).bfloat16().to(device)
    c = torch.full((3000, 3000), float("nan"), dtype=torch.bfloat16, device=device)
    plan = capi.plan_matmul(a, b, c)
    assert capi.FAMILY_NAMES[plan.family] == "tile_192" and plan.split_k == 1 and plan.workspace_bytes == 0
    b_kn = b.t().contiguous()                    # the same matrix stored [K,N]
    assert capi.FAMILY_NAMES[capi.plan_matmul(a, b_kn.t(), c).family] == "tile_192"
    from_kn = torch.full((3000, 3000), float("nan"), dtype=torch.bfloat16, device=device)
    capi.matmul(a, b_kn.t(), from_kn)
    capi.matmul(a, b, c)
    other = torch.full((3000, 3000), float("nan"), dtype=torch.bfloat16, device=device)
    capi.matmul_family(a, b, other, capi.family_request("tile_256", capi.SELECT_REQUIRE, split_k=1))
    torch.cuda.synchronize()
    rows = torch.arange(0, 3000, 59, device=device)
    want = torch.matmul(a[rows].double(), b.double().t())
    assert rel_err(c[rows].double().cpu().numpy(), want.cpu().numpy()) <= fp32_tol(3000) + 2.0 ** -8 * 1.01
    assert torch.equal(c, other)      # the same matrix instruction over the same k in the same order
    assert torch.equal(c, from_kn)


@pytest.mark.parametrize("m,n,k,b_as_kn,family,split", [(2304, 2304, 8192, False, "tile_256", 3), (768, 3072, 12288, False, "tile_192", 4),
                                                         (768, 3072, 12288, True, "tile_192", 4), (1500, 3000, 8192, False, "tile_192", 2)])
def test_one_round_of_bigger_tiles_by_a_k_split(device, m, n, k, b_as_kn, family, split):
    """Where 128 x 128 pairs fill their round badly and K is long, the table plans one round of 256 x 256 or 192 x 192 tiles
    in two to four K parts (partial sums in the workspace, summed by the reduce kernel): sampled rows against float64."""
    import torch
    from vecops_amd import capi
    gen = torch.Generator(device="cpu").manual_seed(m + n + k)
    a = (torch.rand((m, k), generator=gen) * 2 - 1).bfloat16().to(device)
    b = (torch.rand((k, n) if b_as_kn else (n, k), generator=gen) * 2 - 1).bfloat16().to(device)
    bv = b.t() if b_as_kn else b
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    plan = capi.plan_matmul(a, bv, c)
    assert capi.FAMILY_NAMES[plan.family] == family and plan.split_k == split and plan.workspace_bytes == split * m * n * 4
    capi.matmul(a, bv, c)
    torch.cuda.synchronize()
    assert not torch.isnan(c).any()
    rows = torch.arange(0, m, 41, device=device)
    want = torch.matmul(a[rows].double(), bv.double().t())
    assert rel_err(c[rows].double().cpu().numpy(), want.cpu().numpy()) <= fp32_tol(k)


@pytest.mark.parametrize("b_as_kn", [False, True])
def test_fused_transform_on_the_tables_plan(device, b_as_kn):
    """3000 x 3000 x 520 with row and column scales, a shift, silu and a bias row, to bf16: the table plans 192 x 192 tiles;
    against the same operations in float64 (the bound: bf16's half unit in the last place on top of the sums')."""
    import torch
    from vecops_amd import capi
    m, n, k = 3000, 3000, 520
    gen = torch.Generator(device="cpu").manual_seed(9)
    a = (torch.rand((m, k), generator=gen) * 2 - 1).bfloat16().to(device)
    b = (torch.rand((k, n) if b_as_kn else (n, k), generator=gen) * 2 - 1).bfloat16().to(device)
    bv = b.t() if b_as_kn else b
    rs = (torch.rand(m, generator=gen) + 0.5).to(device)
    cs = (torch.rand(n, generator=gen) + 0.5).to(device)
    bias = (torch.rand((1, n), generator=gen) * 2 - 1).to(device).expand(m, n)
    c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
    ep = capi.epilogue(activation="silu", scale=0.125, shift=0.5, row_scales=rs, column_scales=cs)
    plan = capi.plan_matmul_fused(a, bv, c, ep, c_in=bias)
    assert capi.FAMILY_NAMES[plan.family] == "tile_192" and plan.split_k == 1
    capi.matmul_fused(a, bv, c, ep, c_in=bias)
    torch.cuda.synchronize()
    x = (torch.matmul(a.double(), bv.double().t()) + bias.double()) * rs.double()[:, None] * cs.double()[None, :] * 0.125 + 0.5
    want = x * torch.sigmoid(x)
    assert rel_err(c.double().cpu().numpy(), want.cpu().numpy()) <= 2.0 ** -8 * 1.01 + 1e-3    # (the fast exp and reciprocal)


def test_required_where_it_cannot_serve(device):
    import torch
    from vecops_amd import capi
    request, prefer = _require(capi), capi.family_request("tile_192", capi.SELECT_PREFER)

    def z(shape, dtype):
        return torch.zeros(shape, dtype=dtype, device=device)
    cases = {
        "fp32 operands": (z((400, 512), torch.float32), z((400, 512), torch.float32), torch.float32),
        "int8 with B as [K,N]": (z((400, 512), torch.int8), z((512, 400), torch.int8).t(), torch.int32),
        "B as [K,N] with N no multiple of eight": (z((400, 512), torch.bfloat16), z((512, 404), torch.bfloat16).t(), torch.float32),
        "rows not 16-byte aligned": (z((400, 516), torch.bfloat16)[:, :515], z((400, 516), torch.bfloat16)[:, :515], torch.float32),
        "unsigned a": (z((400, 512), torch.uint8), z((400, 512), torch.int8), torch.int32),
    }
    for name, (a, b, out) in cases.items():
        c = torch.zeros((a.shape[0], b.shape[0]), dtype=out, device=device)
        with pytest.raises(capi.VecopsHipError) as err:
            capi.matmul_family(a, b, c, request)
        assert err.value.code == 2, name                       # NotApplicable
        capi.matmul_family(a, b, c, prefer)                    # a preference falls back to the rule table's choice
        assert capi.FAMILY_NAMES[capi.plan_matmul_family(a, b, c, prefer).family] != "tile_192", name
    # a plan that names the family for such a call is refused by the planned entry point
    a, b = cases["fp32 operands"][:2]
    c = torch.zeros((400, 400), dtype=torch.float32, device=device)
    plan = capi.plan_matmul(a, b, c)
    plan.family = capi.FAMILY_CODES["tile_192"]
    with pytest.raises(capi.VecopsHipError):
        capi.matmul_planned(a, b, c, plan)
    torch.cuda.synchronize()
