"""The 256 x 352 workgroup tile (family tile_256x352), through the C ABI.  Signed 8-bit operands: int32 sums bit-exact
against exact integer arithmetic on shapes with one, two, three and more K tiles, ragged N (clamped rows, guarded
stores), several tile rows and columns; the dequantising epilogue bit-exact against the oracle (the same two
separately rounded multiplies, vecops matmul/Quantization.h:195-250) on a shape the rule table itself gives to this
tile; and the family request's error behaviour (a required family that cannot serve the operands is NotApplicable,
tests/ops/MatmulTest.cpp:514-536).  bf16 and f16 operands on the same tile: against float64 sums of the same
operands and against the 256 x 256 tile, to fp32 and to the operands' own type."""
import numpy as np
import pytest

from vecops_amd import synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("m,n,k", [(256, 352, 256), (256, 352, 384), (256, 352, 640), (256, 704, 512), (512, 1000, 512),
                                   (256, 180, 256), (768, 3000, 1024), (256, 356, 2048), (300, 352, 512), (1, 704, 256),
                                   (257, 1000, 384), (1500, 3000, 1024), (129, 356, 256)])
def test_wide_tile_int32_sums_are_exact(device, m, n, k):
    import torch
    from vecops_amd import capi
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    request = capi.family_request("tile_256x352", capi.SELECT_REQUIRE)
    c_store = torch.full((m, n + 12), -7, dtype=torch.int32, device=device)   # rows of C with a pad that must stay
    c = c_store[:, :n]
    assert capi.FAMILY_NAMES[capi.plan_matmul_family(ta, tb, c, request).family] == "tile_256x352"
    capi.matmul_family(ta, tb, c, request)
    torch.cuda.synchronize()
    want = (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32)
    assert np.array_equal(c.cpu().numpy(), want)
    assert bool((c_store[:, n:] == -7).all())


def test_wide_tile_extreme_operands_wrap_like_int32(device):
    """All operands -128: every product 16384, K = 32768 of them = 2^29 per sum... and K = 131072 wraps mod 2^32."""
    import torch
    from vecops_amd import capi
    m, n, k = 256, 352, 131072
    ta = torch.full((m, k), -128, dtype=torch.int8, device=device)
    tb = torch.full((n, k), -128, dtype=torch.int8, device=device)
    c = torch.zeros((m, n), dtype=torch.int32, device=device)
    capi.matmul_family(ta, tb, c, capi.family_request("tile_256x352", capi.SELECT_REQUIRE))
    torch.cuda.synchronize()
    want = np.int64(16384) * k % (1 << 32)
    assert bool((c.view(torch.int32).cpu().numpy().astype(np.int64) % (1 << 32) == want).all())


def test_wide_tile_is_the_tables_choice_and_dequantises_bit_exactly(device, oracle):
    """2048 x 11008 (the benchmark's extents) with a shorter K: 256 tiles of 256 x 352 = one round, which the rule table
    takes; per-token x per-channel dequantisation with a correction row, every output against the oracle."""
    import torch
    from vecops_amd import capi
    m, n, k = 2048, 11008, 1152
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    correction = ((synth.draws(5, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32)
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    plan = capi.plan_matmul(ta, tb, torch.empty((m, n), dtype=torch.int32, device=device))
    assert capi.FAMILY_NAMES[plan.family] == "tile_256x352" and plan.split_k == 1 and plan.workspace_bytes == 0
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul_i8_dequant(ta, tb, torch.from_numpy(rs).to(device), torch.from_numpy(cs).to(device), c,
                           correction=torch.from_numpy(correction).to(device))
    torch.cuda.synchronize()
    want = oracle.matmul_i8_dequant(a, b, rs, cs, correction)
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))
    # scales and correction at addresses that are not 16-byte aligned: the element-wise loads of the epilogue
    rs1, cs1, corr1 = (torch.zeros(x.size + 1, dtype=torch.from_numpy(x).dtype, device=device) for x in (rs, cs, correction))
    rs1[1:], cs1[1:], corr1[1:] = torch.from_numpy(rs).to(device), torch.from_numpy(cs).to(device), torch.from_numpy(correction).to(device)
    c.fill_(float("nan"))
    capi.matmul_i8_dequant(ta, tb, rs1[1:], cs1[1:], c, correction=corr1[1:])
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_wide_tile_with_prepacked_weights(device, oracle):
    """The same tile fed from vecops_hip_pack_b's layout (vecops' ops::matmul_pack, ops/MatmulPack.h:9-117), N ragged
    against the 32-row panels of the pack: dequantised output bit-exact against the oracle and bit-equal to the product
    with the plain operand."""
    import torch
    from vecops_amd import capi
    m, n, k = 2048, 11004, 1152
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    packed = capi.pack_b(tb)
    plan = capi.plan_matmul_packed_b(ta, packed, torch.empty((m, n), dtype=torch.int32, device=device))
    assert capi.FAMILY_NAMES[plan.family] == "tile_256x352"
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul_i8_dequant_packed_b(ta, packed, torch.from_numpy(rs).to(device), torch.from_numpy(cs).to(device), c)
    plain = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul_i8_dequant(ta, tb, torch.from_numpy(rs).to(device), torch.from_numpy(cs).to(device), plain)
    torch.cuda.synchronize()
    want = oracle.matmul_i8_dequant(a, b, rs, cs, None)
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert torch.equal(c.view(torch.int32), plain.view(torch.int32))
    # int32 sums through vecops_hip_matmul_packed_b
    ci = torch.full((m, n), -1, dtype=torch.int32, device=device)
    capi.matmul_packed_b(ta, packed, ci)
    torch.cuda.synchronize()
    rows = np.arange(0, m, 37)
    assert np.array_equal(ci.cpu().numpy()[rows], (a[rows].astype(np.int64) @ b.astype(np.int64).T).astype(np.int32))


def test_wide_tile_required_where_it_cannot_serve(device):
    import torch
    from vecops_amd import capi
    request = capi.family_request("tile_256x352", capi.SELECT_REQUIRE)
    prefer = capi.family_request("tile_256x352", capi.SELECT_PREFER)

    def i8(shape):
        return torch.zeros(shape, dtype=torch.int8, device=device)
    cases = {
        "K not a multiple of 128": (i8((256, 520)), i8((352, 520)), torch.int32),
        "a single K tile": (i8((256, 128)), i8((352, 128)), torch.int32),
        "fp32 operands": (torch.zeros((256, 512), dtype=torch.float32, device=device),
                          torch.zeros((352, 512), dtype=torch.float32, device=device), torch.float32),
        "bf16 operands, B as [K,N]": (torch.zeros((256, 512), dtype=torch.bfloat16, device=device),
                                      torch.zeros((512, 352), dtype=torch.bfloat16, device=device).t(), torch.float32),
        "unsigned a": (torch.zeros((256, 512), dtype=torch.uint8, device=device), i8((352, 512)), torch.int32),
    }
    for name, (a, b, out) in cases.items():
        c = torch.zeros((a.shape[0], b.shape[0]), dtype=out, device=device)
        with pytest.raises(capi.VecopsHipError) as err:
            capi.matmul_family(a, b, c, request)
        assert err.value.code == 2, name                       # NotApplicable
        capi.matmul_family(a, b, c, prefer)                    # a preference falls back to the rule table's choice
        assert capi.FAMILY_NAMES[capi.plan_matmul_family(a, b, c, prefer).family] != "tile_256x352", name
    # a fixed K split is not this family's either
    a, b = i8((256, 512)), i8((352, 512))
    c = torch.zeros((256, 352), dtype=torch.int32, device=device)
    with pytest.raises(capi.VecopsHipError):
        capi.matmul_family(a, b, c, capi.family_request("tile_256x352", capi.SELECT_REQUIRE, split_k=2))
    torch.cuda.synchronize()


@pytest.mark.parametrize("kind,out", [("bf16", "f32"), ("bf16", "own"), ("f16", "f32"), ("f16", "own")])
@pytest.mark.parametrize("m,n,k", [(256, 352, 128), (256, 352, 192), (512, 1000, 512), (256, 4, 256), (768, 3000, 1024),
                                   (256, 356, 2048), (300, 352, 256), (1, 704, 128), (1500, 3000, 512)])
def test_wide_tile_16_bit_operands(device, kind, out, m, n, k):
    import torch
    from vecops_amd import capi
    from conftest import rel_err
    from test_matmul_gpu import fp32_tol
    dtype = torch.bfloat16 if kind == "bf16" else torch.float16
    gen = torch.Generator().manual_seed(m + 3 * n + 7 * k)
    a = (torch.rand((m, k), generator=gen) * 2 - 1).to(dtype).to(device)
    b = (torch.rand((n, k), generator=gen) * 2 - 1).to(dtype).to(device)
    out_dtype = torch.float32 if out == "f32" else dtype
    c_store = torch.full((m, n + 12), -7.0, dtype=out_dtype, device=device)   # rows of C with a pad that must stay
    c = c_store[:, :n]
    request = capi.family_request("tile_256x352", capi.SELECT_REQUIRE)
    assert capi.FAMILY_NAMES[capi.plan_matmul_family(a, b, c, request).family] == "tile_256x352"
    capi.matmul_family(a, b, c, request)
    square = torch.empty((m, n), dtype=out_dtype, device=device)
    capi.matmul_family(a, b, square, capi.family_request("tile_256", capi.SELECT_REQUIRE, split_k=1))
    torch.cuda.synchronize()
    want = (a.double() @ b.double().t()).cpu().numpy()
    tol = fp32_tol(k) + (0.0 if out == "f32" else 2.0 ** (-8 if kind == "bf16" else -11) * 1.01)
    assert rel_err(c.double().cpu().numpy(), want) <= tol
    assert rel_err(c.double().cpu().numpy(), square.double().cpu().numpy()) <= tol   # the order of the fp32 sums may differ
    assert bool((c_store[:, n:] == -7.0).all())


def test_wide_tile_bf16_is_the_tables_choice_where_its_count_fits(device):
    """2048 x 11008 x 4096 in bf16 (B [N,K]): 256 tiles of 256 x 352 are one round; with prepacked weights too.  Every
    output enters a checksum (C v against A (B^T v) in float64)."""
    import torch
    from vecops_amd import capi
    m, n, k = 2048, 11008, 4096
    a = torch.from_numpy(synth.bf16_round(synth.normal(1, (m, k), 0.02)).view(np.int16)).to(device).view(torch.bfloat16)
    b = torch.from_numpy(synth.bf16_round(synth.normal(2, (n, k), 0.02)).view(np.int16)).to(device).view(torch.bfloat16)
    c = torch.empty((m, n), dtype=torch.float32, device=device)
    assert capi.FAMILY_NAMES[capi.plan_matmul(a, b, c).family] == "tile_256x352"
    capi.matmul(a, b, c)
    packed = capi.pack_b(b)
    assert capi.FAMILY_NAMES[capi.plan_matmul_packed_b(a, packed, c).family] == "tile_256x352"
    cp = torch.empty_like(c)
    capi.matmul_packed_b(a, packed, cp)
    torch.cuda.synchronize()
    assert torch.equal(c, cp)                                # the same loop on the same K order
    v = torch.from_numpy(np.random.default_rng(3).standard_normal(n)).to(device)
    got = c.double() @ v
    want = a.double() @ (b.double().t() @ v)
    scale = (a.double().abs() @ (b.double().abs().t() @ v.abs())).clamp(min=1e-30)
    assert float(((got - want).abs() / scale).max()) <= 2e-6 * k / 32


@pytest.mark.parametrize("kind,out", [("bf16", "bf16"), ("bf16", "f32"), ("i8", "i32"), ("i8", "u8"), ("i8", "f32")])
def test_wide_tile_c_input_and_fused_transform(device, kind, out):
    """A bias row (a C input of row stride 0), per-row and per-column scales, scale, shift and an activation on the
    256 x 352 tile: the finishing step is tile_gemm_kernel's own, so the result equals the same call with B handed
    over as [K,N] (which that tile does not serve) - bit for bit on the integer classes, up to the order of the fp32
    sums otherwise - and the formula of the header on float64 sums."""
    import torch
    from vecops_amd import capi
    from conftest import rel_err
    m, n = 1500, 11000                            # 6 x 32 = 192 tiles: the table's own choice ...
    k = 2048 if kind == "i8" else 512             # ... from nine K tiles of bytes on, five of 16-bit elements
    gen = torch.Generator().manual_seed(11)
    if kind == "i8":
        a = torch.randint(-128, 128, (m, k), generator=gen, dtype=torch.int8).to(device)
        b_kn = torch.randint(-128, 128, (k, n), generator=gen, dtype=torch.int8).to(device)
        bias = torch.randint(-5000, 5000, (1, n), generator=gen, dtype=torch.int32).to(device)
    else:
        a = (torch.rand((m, k), generator=gen) * 2 - 1).to(torch.bfloat16).to(device)
        b_kn = (torch.rand((k, n), generator=gen) * 2 - 1).to(torch.bfloat16).to(device)
        bias = (torch.rand((1, n), generator=gen) * 2 - 1).to(torch.bfloat16).to(device)
    b = b_kn.t().contiguous()                      # [N,K]: the 256 x 352 tile's layout
    out_dtype = {"bf16": torch.bfloat16, "f32": torch.float32, "i32": torch.int32, "u8": torch.uint8}[out]
    if out != "i32":
        rs = (torch.rand(m, generator=gen) * 0.5 + 0.75).to(device)
        cs = (torch.rand(n, generator=gen) * 0.5 + 0.75).to(device)
        mag = 2.5e-4 if kind == "i8" else 1.0
        ep = capi.epilogue(activation="relu" if out == "u8" else "silu", scale=0.5 * mag, shift=0.25, row_scales=rs, column_scales=cs)
    # (a C input under both scale vectors on int32 sums - the kernels' dequantisation stage - is not this tile's)
    with_bias = not (kind == "i8" and out != "i32")
    c_in = bias.expand(m, n) if with_bias else None
    c = torch.zeros((m, n), dtype=out_dtype, device=device)
    other = torch.zeros((m, n), dtype=out_dtype, device=device)
    if out == "i32":                                 # (no transform: the plain entry point with its C input)
        assert capi.FAMILY_NAMES[capi.plan_matmul(a, b, c, c_in=c_in).family] == "tile_256x352"
        capi.matmul(a, b, c, c_in=c_in)
        assert capi.FAMILY_NAMES[capi.plan_matmul(a, b_kn.t(), other, c_in=c_in).family] != "tile_256x352"
        capi.matmul(a, b_kn.t(), other, c_in=c_in)
    else:
        plan = capi.plan_matmul_fused(a, b, c, ep, c_in=c_in)
        assert capi.FAMILY_NAMES[plan.family] == "tile_256x352"
        capi.matmul_fused(a, b, c, ep, c_in=c_in)
        assert capi.FAMILY_NAMES[capi.plan_matmul_fused(a, b_kn.t(), other, ep, c_in=c_in).family] != "tile_256x352"
        capi.matmul_fused(a, b_kn.t(), other, ep, c_in=c_in)
    torch.cuda.synchronize()
    if kind == "i8":
        assert torch.equal(c, other)
    else:
        assert rel_err(c.double().cpu().numpy(), other.double().cpu().numpy()) <= 2e-6 * k / 32 + (2.0 ** -8 if out == "bf16" else 0.0)
    v = a.double() @ b.double().t() + (bias.double() if with_bias else 0.0)
    if out == "i32":
        assert torch.equal(c.to(torch.int64), v.to(torch.int64))
        return
    t = ((v * rs.double()[:, None]) * cs.double()[None, :]) * (0.5 * mag) + 0.25
    want = torch.relu(t) if out == "u8" else t * torch.sigmoid(t)
    if out == "u8":
        want = want.clamp(0, 255).floor()
        assert float((c.double() - want).abs().max()) <= 1.0      # truncation next to an integer boundary
    else:
        assert rel_err(c.double().cpu().numpy(), want.cpu().numpy()) <= 1e-4 + (2.0 ** -8 if out == "bf16" else 0.0)
