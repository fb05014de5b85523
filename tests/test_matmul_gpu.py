"""Parity of the gfx950 kernels, called through the C ABI (include/vecops_hip.h),
with the CPU oracle on the same seeded inputs, plus size-independent properties
at the full BASELINE sizes.

Tolerances: integer paths and the dequantisation epilogue are bit-exact.  fp32
outputs may differ from the oracle (fp64 accumulation) only through fp32
summation order: |got - want| <= 2e-6 * max(1, K/32) * max(1, |want|, |got|),
well inside the reference's own 8e-4 for fp32 outputs
(tests/ops/MatmulConversionTestCommon.h:79-83).  bf16 outputs: one bf16 ulp
(2^-7 relative; the reference allows 2e-2).
"""
import numpy as np
import pytest

from conftest import rel_err
from oracle import oracle as O
from vecops_amd import synth

pytestmark = pytest.mark.gpu


def fp32_tol(k):
    return 2e-6 * max(1.0, k / 32)


def dev_bf16(x_bits, device):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x_bits).view(np.int16)).to(device).view(torch.bfloat16)


def host_bits(t):
    import torch
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


REF_SHAPES = [(16, 16, 35), (16, 32, 67), (16, 48, 79), (1, 48, 79), (32, 16, 33), (48, 16, 65), (32, 32, 97),
              (16, 64, 67), (16, 80, 67), (16, 96, 67), (64, 16, 67), (80, 16, 67), (96, 16, 67), (37, 51, 79),
              (1, 128, 65), (512, 1, 256)]  # tests/ops/MatmulTest.cpp:434-452
TILE_SHAPES = [(256, 256, 64), (257, 255, 65), (512, 768, 1024), (300, 520, 1000), (1000, 130, 2048),
               (129, 129, 129), (64, 64, 8), (1024, 1024, 1024), (2048, 2048, 512)]


@pytest.mark.parametrize("m,n,k", REF_SHAPES + TILE_SHAPES)
def test_bf16_gemm_fp32_out(device, oracle, m, n, k):
    import torch
    from vecops_amd import capi
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul(dev_bf16(a, device), dev_bf16(b, device), c)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, acc_f64=True)
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)


@pytest.mark.parametrize("m,n,k", [(37, 51, 79), (256, 256, 256), (300, 520, 1000), (1024, 512, 2048)])
def test_bf16_out_is_rne_of_fp32_out(device, oracle, m, n, k):
    """Same kernel, same summation order: the bf16 output must be exactly the
    round-to-nearest-even of the fp32 output (docs/Tensor.md:253-299)."""
    import torch
    from vecops_amd import capi
    a = dev_bf16(synth.bf16_round(synth.uniform_pm1(1, (m, k))), device)
    b = dev_bf16(synth.bf16_round(synth.uniform_pm1(2, (n, k))), device)
    c32 = torch.empty((m, n), dtype=torch.float32, device=device)
    c16 = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    capi.matmul(a, b, c32)
    capi.matmul(a, b, c16)
    torch.cuda.synchronize()
    assert np.array_equal(host_bits(c16), oracle.bf16_from_f32(c32.cpu().numpy()))


def test_fp32_memory_bf16_compute(device, oracle):
    import torch
    from vecops_amd import capi
    for (m, n, k) in [(33, 65, 257), (256, 384, 512), (1024, 1024, 1024)]:
        a, b = synth.uniform_pm1(1, (m, k)), synth.uniform_pm1(2, (n, k))
        c = torch.empty((m, n), dtype=torch.float32, device=device)
        capi.matmul(torch.from_numpy(a).to(device), torch.from_numpy(b).to(device), c, compute=capi.COMPUTE_BF16)
        torch.cuda.synchronize()
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a, b, want, atom=O.ATOM_BF16F32, acc_f64=True)
        assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)
        # B as [K,N] row-major (BASELINE config 1 layout)
        b_kn = torch.from_numpy(np.ascontiguousarray(b.T)).to(device)
        c2 = torch.empty((m, n), dtype=torch.float32, device=device)
        capi.matmul(torch.from_numpy(a).to(device), b_kn.t(), c2)
        torch.cuda.synchronize()
        assert rel_err(c2.cpu().numpy(), want) <= fp32_tol(k)


def fp32_compute_tol(k):
    """fp32 products summed in fp32 in an unspecified order: a random walk of K roundings of
    half an ulp at the size of the partial sums (~sqrt(K)/3 for U[-1,1) operands), scaled like
    rel_err by max(1, |c|); a few sigma over a million outputs.  Operands rounded to bf16 would
    be off by 2^-9 * sqrt(K) - a hundred times more."""
    return max(2e-6, 1.2e-7 * k)


@pytest.mark.parametrize("m,n,k,layout", [(1024, 1024, 1024, "nn"), (1024, 1024, 1024, "nt"), (37, 51, 79, "nt"),
                                          (300, 520, 1001, "nn"), (257, 255, 65, "tn"), (64, 48, 4099, "nt"),
                                          (512, 768, 96, "nn")])
def test_fp32_compute(device, oracle, m, n, k, layout):
    """fp32 operands multiplied in fp32 (the SME_F32F32 atom, matmul/details/kernel/sme/Atoms.h:65-76;
    1024^3 with B as [K,N] is BASELINE configs[0]): operands must NOT be rounded to bf16."""
    import torch
    from vecops_amd import capi
    a, b = synth.uniform_pm1(1, (m, k)), synth.uniform_pm1(2, (n, k))
    ta = torch.from_numpy(a).to(device)
    if layout[0] == "t":
        ta = torch.from_numpy(np.ascontiguousarray(a.T)).to(device).t()
    tb = torch.from_numpy(b).to(device)
    if layout[1] == "n":
        tb = torch.from_numpy(np.ascontiguousarray(b.T)).to(device).t()       # B stored [K, N]
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul(ta, tb, c, compute=capi.COMPUTE_F32)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, atom=1, acc_f64=True)
    assert rel_err(c.cpu().numpy(), want) <= fp32_compute_tol(k)
    assert rel_err(want, (a.astype(np.float64) @ b.astype(np.float64).T)) <= 1e-6   # the oracle itself: plain fp64 product
    # accumulate into an fp32 C input, bf16 output
    cin = synth.uniform_pm1(3, (m, n))
    c16 = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    capi.matmul(ta, tb, c16, c_in=torch.from_numpy(cin).to(device), compute=capi.COMPUTE_F32)
    torch.cuda.synchronize()
    got16 = synth.bf16_to_f32(host_bits(c16))
    assert rel_err(got16, want + cin) <= 2.0 ** -8


@pytest.mark.parametrize("layout", ["nn", "tn", "tt", "inner2", "padded", "c_transposed", "offset2"])
def test_layouts(device, oracle, layout):
    """Strided views give the values of dense copies (tests/ops/MatmulOrientationTest.cpp:139,249;
    tests/ops/MatmulTest.cpp:220-279)."""
    import torch
    from vecops_amd import capi
    m, n, k = 70, 90, 130
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, acc_f64=True)
    ta, tb = dev_bf16(a, device), dev_bf16(b, device)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    if layout in ("nn", "tt"):
        tb = tb.t().contiguous().t()
    if layout in ("tn", "tt"):
        ta = ta.t().contiguous().t()
    if layout == "inner2":
        big_a = torch.zeros((m, 2 * k + 3), dtype=torch.bfloat16, device=device)
        big_b = torch.zeros((n, 2 * k + 5), dtype=torch.bfloat16, device=device)
        big_a[:, 0:2 * k:2] = ta
        big_b[:, 0:2 * k:2] = tb
        ta, tb = big_a[:, 0:2 * k:2], big_b[:, 0:2 * k:2]
    if layout == "padded":
        big_a = torch.zeros((m, k + 8), dtype=torch.bfloat16, device=device)
        big_a[:, :k] = ta
        ta = big_a[:, :k]
    if layout == "offset2":  # rows start 2 bytes off a 16-byte boundary
        flat = torch.zeros(m * k + 1, dtype=torch.bfloat16, device=device)
        flat[1:] = ta.reshape(-1)
        ta = flat[1:].view(m, k)
    if layout == "c_transposed":
        c = torch.full((n, m), float("nan"), dtype=torch.float32, device=device).t()
    capi.matmul(ta, tb, c)
    torch.cuda.synchronize()
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)


@pytest.mark.parametrize("a_t", [False, True])
@pytest.mark.parametrize("b_t", [False, True])
@pytest.mark.parametrize("c_t", [False, True])
@pytest.mark.parametrize("dtype", ["bf16", "i8"])
def test_eight_orientations(device, oracle, a_t, b_t, c_t, dtype):
    """Every combination of A, B and C held transposed in memory - the eight orientations of
    tests/ops/MatmulOrientationTest.cpp:139,249 - gives the values of the dense product, for a floating and an
    integer atom, on a shape with ragged tiles in every direction."""
    import torch
    from vecops_amd import capi
    m, n, k = 150, 203, 333
    if dtype == "bf16":
        a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
        b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
        ta, tb = dev_bf16(a, device), dev_bf16(b, device)
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a, b, want, acc_f64=True)
        out_dtype = torch.float32
    else:
        a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
        ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
        want = (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32)
        out_dtype = torch.int32
    if a_t:
        ta = ta.t().contiguous().t()      # [M,K] view of a [K,M] array
    if b_t:
        tb = tb.t().contiguous().t()      # [N,K] view of a [K,N] array: the conventional B
    if c_t:
        c = torch.zeros((n, m), dtype=out_dtype, device=device).t()
    else:
        c = torch.zeros((m, n), dtype=out_dtype, device=device)
    capi.matmul(ta, tb, c)
    torch.cuda.synchronize()
    if dtype == "bf16":
        assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)
    else:
        assert np.array_equal(c.cpu().numpy(), want)


TILE_FAMILIES = ["tile_256", "tile_128", "tile_64", "tile_256x128", "tile_128x256"]


@pytest.mark.parametrize("family", TILE_FAMILIES)
@pytest.mark.parametrize("dtype,layout", [("bf16", "nt"), ("bf16", "nn"), ("i8", "nt"), ("f32", "nn")])
def test_required_family_equals_the_oracle(device, oracle, family, dtype, layout):
    """The first tier of the owner selection: every tile family, required by the caller on one ragged shape (where the
    rule table itself would take 64x64 tiles and split K), gives the oracle's product - and the plan says so."""
    import torch
    from vecops_amd import capi
    m, n, k = 300, 520, 1000
    request = capi.family_request(family, capi.SELECT_REQUIRE)
    if dtype == "i8":
        a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
        ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
        c = torch.zeros((m, n), dtype=torch.int32, device=device)
        want = (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32)
    elif dtype == "f32":
        a, b = synth.uniform_pm1(1, (m, k)), synth.uniform_pm1(2, (n, k))
        ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
        c = torch.zeros((m, n), dtype=torch.float32, device=device)
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a, b, want, acc_f64=True)     # fp32 memory, bf16 compute
    else:
        a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
        b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
        ta, tb = dev_bf16(a, device), dev_bf16(b, device)
        c = torch.zeros((m, n), dtype=torch.float32, device=device)
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a, b, want, acc_f64=True)
    if layout == "nn":
        tb = tb.t().contiguous().t()
    plan = capi.plan_matmul_family(ta, tb, c, request)
    assert capi.FAMILY_NAMES[plan.family] == family
    capi.matmul_family(ta, tb, c, request)
    torch.cuda.synchronize()
    if dtype == "i8":
        assert np.array_equal(c.cpu().numpy(), want)
    else:
        assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)
    # and with the K split fixed by the caller (partial sums through the workspace)
    split = capi.family_request(family, capi.SELECT_REQUIRE, split_k=3)
    plan = capi.plan_matmul_family(ta, tb, c, split)
    assert plan.split_k == 3 and plan.workspace_bytes >= 3 * m * n * 4
    c.zero_()
    capi.matmul_family(ta, tb, c, split)
    torch.cuda.synchronize()
    if dtype == "i8":
        assert np.array_equal(c.cpu().numpy(), want)
    else:
        assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)


def test_required_family_that_cannot_serve_is_rejected(device, oracle):
    """family_selection::Require on a family that cannot serve the call is an error, not a fallback
    (tests/ops/MatmulTest.cpp:514-536: RequiredFamilyRuntimeRejectionPropagatesAsException, 128^3 bf16 there too);
    Prefer falls back to the rule table's choice."""
    import torch
    from vecops_amd import capi
    m = n = k = 128
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    ta, tb = dev_bf16(a, device), dev_bf16(b, device)
    c = torch.full((m, n), 7.0, dtype=torch.float32, device=device)
    with pytest.raises(capi.VecopsHipError) as info:
        capi.matmul_family(ta, tb, c, capi.family_request("skinny", capi.SELECT_REQUIRE))
    assert info.value.code == 2 and "skinny" in str(info.value)
    torch.cuda.synchronize()
    assert bool((c == 7.0).all())                                   # nothing was launched
    automatic = capi.plan_matmul(ta, tb, c)
    preferred = capi.plan_matmul_family(ta, tb, c, capi.family_request("skinny", capi.SELECT_PREFER))
    assert preferred.family == automatic.family and preferred.split_k == automatic.split_k
    capi.matmul_family(ta, tb, c, capi.family_request("skinny", capi.SELECT_PREFER))
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, acc_f64=True)
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)
    # the skinny family on one of its own shapes, required; and a tile family required on that shape
    m2, n2, k2 = 4, 1024, 512
    a2 = synth.bf16_round(synth.uniform_pm1(3, (m2, k2)))
    b2 = synth.bf16_round(synth.uniform_pm1(4, (n2, k2)))
    want2 = np.zeros((m2, n2), np.float32)
    oracle.matmul(a2, b2, want2, acc_f64=True)
    for family in ("skinny", "tile_64", "tile_128"):
        c2 = torch.zeros((m2, n2), dtype=torch.float32, device=device)
        request = capi.family_request(family, capi.SELECT_REQUIRE)
        assert capi.FAMILY_NAMES[capi.plan_matmul_family(dev_bf16(a2, device), dev_bf16(b2, device), c2, request).family] == family
        capi.matmul_family(dev_bf16(a2, device), dev_bf16(b2, device), c2, request)
        torch.cuda.synchronize()
        assert rel_err(c2.cpu().numpy(), want2) <= fp32_tol(k2), family
    # nothing to multiply: a tile family cannot be required of an empty product or of K = 0
    empty = torch.zeros((0, n), dtype=torch.float32, device=device)
    with pytest.raises(capi.VecopsHipError) as info:
        capi.matmul_family(ta[:0], tb, empty, capi.family_request("tile_128", capi.SELECT_REQUIRE))
    assert info.value.code == 2
    capi.matmul_family(ta[:0], tb, empty, capi.family_request("none", capi.SELECT_REQUIRE))


def test_batched_and_broadcast(device, oracle):
    """Rank 3: independent products over the batch; stride 0 broadcasts an operand
    (tests/ops/MatmulBatchTest.cpp:176-335)."""
    import torch
    from vecops_amd import capi
    batch, m, n, k = 5, 45, 67, 200
    a = synth.bf16_round(synth.uniform_pm1(1, (batch, m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (batch, n, k)))
    for share in (None, "a", "b"):
        ha = np.broadcast_to(a[0], a.shape) if share == "a" else a
        hb = np.broadcast_to(b[0], b.shape) if share == "b" else b
        ta = dev_bf16(a[0], device).expand(batch, m, k) if share == "a" else dev_bf16(a, device)
        tb = dev_bf16(b[0], device).expand(batch, n, k) if share == "b" else dev_bf16(b, device)
        c = torch.full((batch, m, n), float("nan"), dtype=torch.float32, device=device)
        capi.matmul(ta, tb, c)
        torch.cuda.synchronize()
        want = np.zeros((batch, m, n), np.float32)
        oracle.matmul(ha, hb, want, acc_f64=True)
        assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)
    # batch == 0: nothing to do, no error (ArchitectureFamily.h:1935-1938)
    capi.matmul(torch.empty((0, m, k), dtype=torch.bfloat16, device=device),
                torch.empty((0, n, k), dtype=torch.bfloat16, device=device),
                torch.empty((0, m, n), dtype=torch.float32, device=device))


@pytest.mark.parametrize("m,n,k,family", [(4187, 1100, 328, "tile_256x128"), (2111, 3643, 328, "tile_128x256"),
                                          (1938, 900, 72, "tile_128"), (2457, 3221, 328, "tile_256"), (2457, 3221, 72, "tile_128"),
                                          (900, 900, 72, "tile_64")])
def test_every_tile_family_ragged(device, oracle, m, n, k, family):
    """Each workgroup tile shape (required of the library, so that the case does not move with the rule table) on
    extents that leave partial tiles in M, N and K, with a bf16 C input and a bf16 output (RNE of the fp32 result of
    the same launch sequence)."""
    import torch
    from vecops_amd import capi
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    cin = synth.bf16_round(synth.uniform_pm1(3, (m, n)))
    ta, tb, tci = dev_bf16(a, device), dev_bf16(b, device), dev_bf16(cin, device)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    request = capi.family_request(family)
    assert capi.FAMILY_NAMES[capi.plan_matmul_family(ta, tb, c, request, c_in=tci).family] == family
    capi.matmul_family(ta, tb, c, request, c_in=tci)
    c16 = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    capi.matmul_family(ta, tb, c16, request, c_in=tci)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, cin=cin, acc_f64=True)
    got = c.cpu().numpy()
    assert rel_err(got, want) <= fp32_tol(k)
    assert np.array_equal(host_bits(c16), oracle.bf16_from_f32(got))


def test_shared_b_batch_is_folded(device, oracle):
    """One B for every batch and A / C rows running on from batch to batch: planned and run as a single
    [batch * M, K] x B product (tests/ops/MatmulBatchTest.cpp:301-335), with a per-batch C input, a bias
    row, and - rows not running on - the unfolded path giving the same values."""
    import torch
    from vecops_amd import capi
    batch, m, n, k = 64, 32, 2048, 264
    a = synth.bf16_round(synth.uniform_pm1(1, (batch, m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    cin = synth.uniform_pm1(3, (batch, m, n))
    ta, tb = dev_bf16(a, device), dev_bf16(b, device)[None].expand(batch, n, k)
    c = torch.full((batch, m, n), float("nan"), dtype=torch.float32, device=device)
    folded = capi.plan_matmul(ta, tb, c)
    apart = capi.plan_matmul(ta, dev_bf16(np.broadcast_to(b, (batch, n, k)).copy(), device), c)
    assert capi.FAMILY_NAMES[folded.family] in ("tile_128", "tile_256x128", "tile_128x256")
    assert capi.FAMILY_NAMES[apart.family] == "tile_64"
    hb = np.broadcast_to(b, (batch, n, k))
    for c_in, h_in in ((None, None), (torch.from_numpy(cin).to(device), cin),
                       (torch.from_numpy(cin[0, 0].copy()).to(device).expand(batch, m, n),
                        np.broadcast_to(cin[0, 0], (batch, m, n)))):
        c.fill_(float("nan"))
        capi.matmul(ta, tb, c, c_in=c_in)
        torch.cuda.synchronize()
        want = np.zeros((batch, m, n), np.float32)
        oracle.matmul(a, hb, want, cin=h_in, acc_f64=True)
        assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)
    # C with padded rows between batches: not foldable, same values
    c_store = torch.full((batch, m + 3, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul(ta, tb, c_store[:, :m])
    torch.cuda.synchronize()
    want = np.zeros((batch, m, n), np.float32)
    oracle.matmul(a, hb, want, acc_f64=True)
    assert rel_err(c_store[:, :m].cpu().numpy(), want) <= fp32_tol(k)
    assert torch.isnan(c_store[:, m:]).all()


@pytest.mark.parametrize("m,n,k", [(777, 1000, 3001), (1, 4097, 129), (255, 63, 8191), (3000, 3000, 17)])
def test_config3_irregular_batch8(device, oracle, m, n, k):
    """BASELINE config 3 at full size: batch 8, bf16 in, fp32 out.  All eight products run on the GPU; the oracle
    checks batches 0 and 7 in full and 302 sampled sums of every batch."""
    import torch
    from vecops_amd import capi
    batch = 8
    a = synth.bf16_round(synth.uniform_pm1(1, (batch, m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (batch, n, k)))
    c = torch.full((batch, m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul(dev_bf16(a, device), dev_bf16(b, device), c)
    torch.cuda.synchronize()
    got = c.cpu().numpy()
    assert np.isfinite(got).all()
    for bi in (0, 7):
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a[bi], b[bi], want, acc_f64=True)
        assert rel_err(got[bi], want) <= fp32_tol(k)
    # every batch against the oracle's sampled sums (a batch offset by one, a wrong batch stride or a skipped
    # batch would leave batches 0 and 7 right)
    rng = np.random.default_rng(m + n + k)
    for bi in range(batch):
        rows = np.concatenate([rng.integers(0, m, 300), [0, m - 1]])
        cols = np.concatenate([rng.integers(0, n, 300), [n - 1, 0]])
        want = oracle.matmul_sampled(a[bi], b[bi], rows, cols)
        assert rel_err(got[bi][rows, cols], want) <= fp32_tol(k), f"batch {bi}"


def test_explicit_c_input_and_aliasing(device, oracle):
    import torch
    from vecops_amd import capi
    for (m, n, k) in [(37, 51, 79), (300, 260, 512)]:
        a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
        b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
        cin = synth.uniform_pm1(3, (m, n))
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a, b, want, cin=cin, acc_f64=True)
        c = torch.from_numpy(cin.copy()).to(device)
        capi.matmul(dev_bf16(a, device), dev_bf16(b, device), c, c_in=c)   # Cin aliases Cout
        torch.cuda.synchronize()
        assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)
        # a broadcast row as C input (bias): stride 0 over rows
        bias = torch.from_numpy(cin[0].copy()).to(device)
        c2 = torch.empty((m, n), dtype=torch.float32, device=device)
        capi.matmul(dev_bf16(a, device), dev_bf16(b, device), c2, c_in=bias.expand(m, n))
        torch.cuda.synchronize()
        want2 = np.zeros((m, n), np.float32)
        oracle.matmul(a, b, want2, cin=np.broadcast_to(cin[0], (m, n)), acc_f64=True)
        assert rel_err(c2.cpu().numpy(), want2) <= fp32_tol(k)


def test_zero_extents(device):
    """K == 0 writes zeros (single C) or C_in (explicit C); zero M or N writes nothing
    (ops/Matmul.h:41-43; tests/ops/MatmulTest.cpp:456-457)."""
    import torch
    from vecops_amd import capi
    bf = torch.bfloat16
    c = torch.full((4, 5), 3.0, dtype=torch.float32, device=device)
    capi.matmul(torch.empty((4, 0), dtype=bf, device=device), torch.empty((5, 0), dtype=bf, device=device), c)
    torch.cuda.synchronize()
    assert torch.equal(c, torch.zeros_like(c))
    cin = torch.full((4, 5), 2.5, dtype=torch.float32, device=device)
    capi.matmul(torch.empty((4, 0), dtype=bf, device=device), torch.empty((5, 0), dtype=bf, device=device), c,
                c_in=cin)
    torch.cuda.synchronize()
    assert torch.equal(c, cin)
    capi.matmul(torch.empty((0, 16), dtype=bf, device=device), torch.empty((5, 16), dtype=bf, device=device),
                torch.empty((0, 5), dtype=torch.float32, device=device))
    capi.matmul(torch.empty((4, 16), dtype=bf, device=device), torch.empty((0, 16), dtype=bf, device=device),
                torch.empty((4, 0), dtype=torch.float32, device=device))
    torch.cuda.synchronize()


def test_invalid_arguments_are_rejected(device):
    import torch
    from vecops_amd import capi
    bf = torch.bfloat16
    a = torch.zeros((4, 8), dtype=bf, device=device)
    with pytest.raises(capi.VecopsHipError) as e:
        capi.matmul(a, torch.zeros((5, 9), dtype=bf, device=device), torch.zeros((4, 5), device=device))
    assert e.value.code == 1
    with pytest.raises(capi.VecopsHipError) as e:
        capi.matmul(a, torch.zeros((5, 8), dtype=bf, device=device), torch.zeros((4, 6), device=device))
    assert e.value.code == 1
    with pytest.raises(capi.VecopsHipError) as e:  # dtype combination outside the path
        capi.matmul(a, torch.zeros((5, 8), dtype=torch.int8, device=device), torch.zeros((4, 5), device=device))
    assert e.value.code == 2


@pytest.mark.parametrize("m,n,k", [(1, 14336, 4096), (16, 14336, 4096), (4, 4096, 11008), (3, 1000, 520),
                                   (2048, 7, 264), (5, 513, 64), (16, 600, 8200)])
def test_skinny_bf16_family(device, oracle, m, n, k):
    """One side at most 16 rows, the other long (the small-vector shapes of
    matmul/details/kernel/RuntimeDispatch.h:24-83): the skinny kernel, fp32 and bf16 outputs."""
    import torch
    from vecops_amd import capi
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    ta, tb = dev_bf16(a, device), dev_bf16(b, device)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    assert capi.FAMILY_NAMES[capi.plan_matmul(ta, tb, c).family] == "skinny"
    capi.matmul(ta, tb, c)
    c16 = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    capi.matmul(ta, tb, c16)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, acc_f64=True)
    got = c.cpu().numpy()
    assert rel_err(got, want) <= fp32_tol(k)
    assert np.array_equal(host_bits(c16), oracle.bf16_from_f32(got))


@pytest.mark.parametrize("compute", ["bf16", "f32"])
@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (4, 14336, 1024), (16, 1000, 520), (3000, 7, 264), (1, 513, 64)])
def test_skinny_f32_operand_family(device, oracle, compute, m, n, k):
    """fp32 memory on the skinny kernel, rounded to bf16 on the way in (AMX_BF16F32 with fp32 memory) or multiplied in
    fp32 (SME_F32F32): vecops' small-vector leaves serve every atom (matmul/details/kernel/amx/Backend.h:767-992).
    Either side narrow, fp32 and bf16 outputs; a K that is not a multiple of the lane's chunk keeps the tile path."""
    import torch
    from vecops_amd import capi
    a, b = synth.uniform_pm1(1, (m, k)).astype(np.float32), synth.uniform_pm1(2, (n, k)).astype(np.float32)
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    code = capi.COMPUTE_F32 if compute == "f32" else capi.COMPUTE_BF16
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    assert capi.FAMILY_NAMES[capi.plan_matmul(ta, tb, c, compute=code).family] == "skinny"
    capi.matmul(ta, tb, c, compute=code)
    c16 = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    capi.matmul(ta, tb, c16, compute=code)
    torch.cuda.synchronize()
    if compute == "f32":
        want = (a.astype(np.float64) @ b.astype(np.float64).T).astype(np.float32)
    else:
        want = np.zeros((m, n), np.float32)
        oracle.matmul(synth.bf16_round(a), synth.bf16_round(b), want, acc_f64=True)
    got = c.cpu().numpy()
    assert rel_err(got, want) <= fp32_tol(k)
    assert np.array_equal(host_bits(c16), oracle.bf16_from_f32(got))
    # K + 2: no longer whole chunks per lane - the tile kernels, same values on the common columns
    a2, b2 = np.pad(a, ((0, 0), (0, 2))), np.pad(b, ((0, 0), (0, 2)))
    ta2, tb2 = torch.from_numpy(a2).to(device), torch.from_numpy(b2).to(device)
    assert capi.FAMILY_NAMES[capi.plan_matmul(ta2, tb2, c, compute=code).family] != "skinny"
    c2 = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul(ta2, tb2, c2, compute=code)
    torch.cuda.synchronize()
    assert rel_err(c2.cpu().numpy(), want) <= fp32_tol(k)


def test_skinny_bf16_batched_strided(device, oracle):
    """Rank-3 batch with a broadcast narrow operand, padded rows of the wide operand and a
    transposed (column-major) output."""
    import torch
    from vecops_amd import capi
    batch, m, n, k = 3, 6, 1100, 776
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b_pad = synth.bf16_round(synth.uniform_pm1(2, (batch, n, k + 24)))
    tb = dev_bf16(b_pad, device)[:, :, :k]                              # row stride k + 24
    ta = dev_bf16(a, device)[None].expand(batch, m, k)                  # stride-0 batch
    c_t = torch.full((batch, n, m), float("nan"), dtype=torch.float32, device=device)
    c = c_t.transpose(1, 2)                                             # [batch, m, n] view, n stride m
    assert capi.FAMILY_NAMES[capi.plan_matmul(ta, tb, c).family] == "skinny"
    capi.matmul(ta, tb, c)
    torch.cuda.synchronize()
    want = np.zeros((batch, m, n), np.float32)
    oracle.matmul(np.broadcast_to(a, (batch, m, k)), b_pad[:, :, :k], want, acc_f64=True)
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)


# --- int8 -------------------------------------------------------------------------------

@pytest.mark.parametrize("m,n,k", [(19, 21, 69), (1, 128, 65), (128, 1, 65), (1, 16, 129), (35, 53, 257),
                                   (256, 256, 128), (300, 520, 1000), (1024, 768, 4096), (130, 140, 515)])
def test_int8_gemm_bit_exact(device, oracle, m, n, k):
    import torch
    from vecops_amd import capi
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    c = torch.full((m, n), -1, dtype=torch.int32, device=device)
    capi.matmul(torch.from_numpy(a).to(device), torch.from_numpy(b).to(device), c)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy(), oracle.matmul_i8_dense(a, b))


@pytest.mark.parametrize("signs", ["us", "su", "uu"])
@pytest.mark.parametrize("m,n,k", [(19, 21, 69), (1, 128, 65), (300, 520, 1000), (256, 256, 128), (64, 48, 8191)])
def test_unsigned_byte_operands_bit_exact(device, oracle, signs, m, n, k):
    """AMX_I8I32<A, B> with uint8 on either side (matmul/details/kernel/amx/Atoms.h:73-86): the
    unsigned side is staged as u - 128 and restored with row / column sums in the epilogue;
    every int32 must equal the oracle's plain integer sum (tile, split-K and ragged shapes)."""
    import torch
    from vecops_amd import capi
    def gen(seed, shape, unsigned):
        if unsigned:
            return (synth.draws(seed, shape[0] * shape[1]) % np.uint64(256)).astype(np.uint8).reshape(shape)
        return synth.int8_sym(seed, shape)
    a, b = gen(1, (m, k), signs[0] == "u"), gen(2, (n, k), signs[1] == "u")
    c = torch.full((m, n), -1, dtype=torch.int32, device=device)
    capi.matmul(torch.from_numpy(a).to(device), torch.from_numpy(b).to(device), c)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.int32)
    oracle.matmul(a, b, want, atom=2)
    assert np.array_equal(c.cpu().numpy(), want)
    assert np.array_equal(want, (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32))


def test_unsigned_bytes_batched_cin_and_wrap(device, oracle):
    """uint8 x uint8 with a rank-3 batch, a broadcast B, an int32 C input and accumulators that
    wrap (255 * 255 * K > 2^31)."""
    import torch
    from vecops_amd import capi
    batch, m, n, k = 3, 70, 33, 40000
    a = np.full((batch, m, k), 255, np.uint8)
    a[1] = (synth.draws(1, m * k) % np.uint64(256)).astype(np.uint8).reshape(m, k)
    b = np.full((n, k), 255, np.uint8)
    b[::2] = (synth.draws(2, ((n + 1) // 2) * k) % np.uint64(256)).astype(np.uint8).reshape(-1, k)
    cin = ((synth.draws(3, batch * m * n) % np.uint64(200001)).astype(np.int64) - 100000).astype(np.int32)
    cin = cin.reshape(batch, m, n)
    tb = torch.from_numpy(b).to(device)[None].expand(batch, n, k)          # stride-0 batch
    c = torch.zeros((batch, m, n), dtype=torch.int32, device=device)
    capi.matmul(torch.from_numpy(a).to(device), tb, c, c_in=torch.from_numpy(cin).to(device))
    torch.cuda.synchronize()
    want = (np.einsum("bmk,nk->bmn", a.astype(np.int64), b.astype(np.int64)) + cin).astype(np.uint64)
    want = (want & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.int32)
    assert np.array_equal(c.cpu().numpy(), want)


def test_int32_accumulator_wraps(device):
    """tests/ops/MatmulTest.cpp:1025-1055: 262145 products of 127*127 wrap mod 2^32."""
    import torch
    from vecops_amd import capi
    K = 262145
    a = torch.full((1, K), 127, dtype=torch.int8, device=device)
    c = torch.zeros((1, 1), dtype=torch.int32, device=device)
    capi.matmul(a, a.clone(), c)
    torch.cuda.synchronize()
    assert int(c.item()) == int(np.uint32((127 * 127 * K) % 2 ** 32).astype(np.int32))
    # a full tile of wrapping accumulators
    m = n = 64
    am = torch.full((m, K), 127, dtype=torch.int8, device=device)
    cm = torch.zeros((m, n), dtype=torch.int32, device=device)
    capi.matmul(am, am.clone(), cm)
    torch.cuda.synchronize()
    assert (cm.cpu().numpy() == np.uint32((127 * 127 * K) % 2 ** 32).astype(np.int32)).all()


def test_int8_c_input(device, oracle):
    import torch
    from vecops_amd import capi
    m, n, k = 35, 53, 257
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    cin = ((synth.draws(3, m * n) % np.uint64(200001)).astype(np.int64) - 100000).astype(np.int32).reshape(m, n)
    c = torch.zeros((m, n), dtype=torch.int32, device=device)
    capi.matmul(torch.from_numpy(a).to(device), torch.from_numpy(b).to(device), c,
                c_in=torch.from_numpy(cin).to(device))
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy(), oracle.matmul_i8_dense(a, b) + cin)


@pytest.mark.parametrize("m,n,k,corr", [(67, 129, 515, False), (67, 129, 515, True), (256, 384, 1024, False),
                                        (300, 1000, 2048, True), (1, 300, 4096, False), (16, 64, 100, True)])
def test_int8_dequant_bit_exact(device, oracle, m, n, k, corr):
    import torch
    from vecops_amd import capi
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    correction = ((synth.draws(5, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32) if corr else None
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul_i8_dequant(torch.from_numpy(a).to(device), torch.from_numpy(b).to(device),
                           torch.from_numpy(rs).to(device), torch.from_numpy(cs).to(device), c,
                           correction=torch.from_numpy(correction).to(device) if corr else None)
    torch.cuda.synchronize()
    want = oracle.matmul_i8_dequant(a, b, rs, cs, correction)
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("m,n,k", [(1, 11008, 4096), (16, 14336, 4096), (4, 4096, 11008), (3, 1000, 528),
                                   (2048, 7, 272), (5, 513, 128), (16, 600, 8208)])
def test_skinny_int8_family(device, oracle, m, n, k):
    """int8 decode shapes on the skinny kernel: int32 accumulators bit-exact, either side narrow."""
    import torch
    from vecops_amd import capi
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    c = torch.full((m, n), -1, dtype=torch.int32, device=device)
    assert capi.FAMILY_NAMES[capi.plan_matmul(ta, tb, c).family] == "skinny"
    capi.matmul(ta, tb, c)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy(), oracle.matmul_i8_dense(a, b))


@pytest.mark.parametrize("m,n,k,corr", [(1, 11008, 4096, False), (16, 11008, 4096, True), (7, 700, 1040, True),
                                        (2048, 7, 272, True)])
def test_skinny_int8_dequant_bit_exact(device, oracle, m, n, k, corr):
    """Decode-shaped quantised matmul (few tokens against the whole weight matrix): the skinny kernel with
    the dequantising epilogue when A is the narrow side, the tile kernel otherwise - same bits either way."""
    import torch
    from vecops_amd import capi
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    correction = ((synth.draws(5, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32) if corr else None
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul_i8_dequant(torch.from_numpy(a).to(device), torch.from_numpy(b).to(device),
                           torch.from_numpy(rs).to(device), torch.from_numpy(cs).to(device), c,
                           correction=torch.from_numpy(correction).to(device) if corr else None)
    torch.cuda.synchronize()
    want = oracle.matmul_i8_dequant(a, b, rs, cs, correction)
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_skinny_int8_wraps_and_batches(device):
    """Accumulators wrap mod 2^32 across the K slices of the eight wavefronts; rank-3 with a broadcast A."""
    import torch
    from vecops_amd import capi
    batch, m, n, k = 2, 3, 640, 140000 // 16 * 16
    a = torch.full((m, k), -128, dtype=torch.int8, device=device)
    b = torch.full((batch, n, k), -128, dtype=torch.int8, device=device)
    b[1, :, ::2] = 127
    c = torch.empty((batch, m, n), dtype=torch.int32, device=device)
    capi.matmul(a[None].expand(batch, m, k), b, c)
    torch.cuda.synchronize()
    want0 = np.int64(16384) * k
    want1 = np.int64(16384) * (k // 2) + np.int64(-128 * 127) * (k // 2)
    wrap = lambda v: int(((int(v) + 2 ** 31) % 2 ** 32) - 2 ** 31)
    assert (c[0] == wrap(want0)).all() and (c[1] == wrap(want1)).all()
    assert want0 > 2 ** 31  # the case does wrap


# --- full BASELINE sizes: size-independent properties -------------------------------------

def test_config2_bf16_4096_sampled_and_linear(device, oracle):
    """bf16 4096^3, B given as [K,N] row-major, bf16 out: 4096 sampled outputs
    against the oracle, and the whole output against fp32-out of the same kernel."""
    import torch
    from vecops_amd import capi
    n = 4096
    a = synth.bf16_round(synth.normal(1, (n, n), 0.02))
    b_kn = synth.bf16_round(synth.normal(2, (n, n), 0.02))      # [K, N]
    ta, tb = dev_bf16(a, device), dev_bf16(b_kn, device).t()    # strided [N, K] view
    c16 = torch.empty((n, n), dtype=torch.bfloat16, device=device)
    c32 = torch.empty((n, n), dtype=torch.float32, device=device)
    capi.matmul(ta, tb, c16)
    capi.matmul(ta, tb, c32)
    torch.cuda.synchronize()
    rng = np.random.default_rng(7)
    rows, cols = rng.integers(0, n, 4096), rng.integers(0, n, 4096)
    rows[:8] = [0, 0, n - 1, n - 1, 255, 256, 2047, 2048]
    cols[:8] = [0, n - 1, 0, n - 1, 256, 255, 2048, 2047]
    want = oracle.matmul_sampled(a, b_kn.T, rows, cols)
    got32 = c32.cpu().numpy()
    assert rel_err(got32[rows, cols], want) <= fp32_tol(n)
    assert np.array_equal(host_bits(c16), oracle.bf16_from_f32(got32))
    # linearity: (2A) B == 2 (A B) exactly in binary floating point
    c32b = torch.empty_like(c32)
    capi.matmul(ta * 2, tb, c32b)
    torch.cuda.synchronize()
    assert torch.equal(c32b, c32 * 2)


@pytest.mark.parametrize("layout", ["nt", "nn"])
def test_wide_ragged_bf16_sampled(device, oracle, layout):
    """Many 256-wide tiles with ragged N and a K tail: sampled outputs against the
    oracle, bf16 output against RNE of the fp32 output."""
    import torch
    from vecops_amd import capi
    m, n, k = 2048, 11000, 264
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    ta = dev_bf16(a, device)
    tb = dev_bf16(b, device) if layout == "nt" else dev_bf16(np.ascontiguousarray(b.T), device).t()
    c32 = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    c16 = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    capi.matmul(ta, tb, c32)
    capi.matmul(ta, tb, c16)
    torch.cuda.synchronize()
    rng = np.random.default_rng(11)
    rows, cols = rng.integers(0, m, 8192), rng.integers(0, n, 8192)
    rows[:6] = [0, 0, m - 1, m - 1, 255, 256]
    cols[:6] = [0, n - 1, 0, n - 1, 255, 256]
    got32 = c32.cpu().numpy()
    assert not np.isnan(got32).any()
    assert rel_err(got32[rows, cols], oracle.matmul_sampled(a, b, rows, cols)) <= fp32_tol(k)
    assert np.array_equal(host_bits(c16), oracle.bf16_from_f32(got32))


def test_config4_int8_full_size_checksum(device, oracle):
    """int8 2048x4096x11008: every int32 accumulator is checked by a checksum of
    checksums that is exact mod 2^32 (C v == A (B^T v) for a random integer v), the
    dequantised output is checked bit-for-bit against the epilogue applied to those
    accumulators, and 64 whole rows are compared with the oracle."""
    import torch
    from vecops_amd import capi
    m, k, n = 2048, 4096, 11008
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    acc = torch.empty((m, n), dtype=torch.int32, device=device)
    capi.matmul(ta, tb, acc)
    out = torch.empty((m, n), dtype=torch.float32, device=device)
    trs, tcs = torch.from_numpy(rs).to(device), torch.from_numpy(cs).to(device)
    capi.matmul_i8_dequant(ta, tb, trs, tcs, out)
    torch.cuda.synchronize()
    # checksum of checksums in int64 (no overflow: |v| < 2^15, |sum| < 2^63), reduced mod 2^32
    v = torch.from_numpy((synth.draws(9, n) % np.uint64(32768)).astype(np.int64)).to(device)
    lhs = (acc.to(torch.int64) * v[None, :]).sum(dim=1)
    btv = (tb.to(torch.int64) * v[:, None]).sum(dim=0)          # [K]
    rhs = (ta.to(torch.int64) * btv[None, :]).sum(dim=1)
    assert torch.equal(lhs & 0xFFFFFFFF, rhs & 0xFFFFFFFF)
    w = torch.from_numpy((synth.draws(10, m) % np.uint64(32768)).astype(np.int64)).to(device)
    lhs2 = (acc.to(torch.int64) * w[:, None]).sum(dim=0)
    atw = (ta.to(torch.int64) * w[:, None]).sum(dim=0)
    rhs2 = (tb.to(torch.int64) * atw[None, :]).sum(dim=1)
    assert torch.equal(lhs2 & 0xFFFFFFFF, rhs2 & 0xFFFFFFFF)
    # epilogue: two IEEE fp32 multiplies, row scale first
    expect = (acc.to(torch.float32) * trs[:, None]) * tcs[None, :]
    assert torch.equal(out.view(torch.int32), expect.view(torch.int32))
    rows = np.r_[0:32, m - 32:m]
    want = oracle.matmul_i8_dequant(a[rows], b, rs[rows], cs)
    assert np.array_equal(out[torch.from_numpy(rows).to(device)].cpu().numpy().view(np.uint32), want.view(np.uint32))


# --- weight-only int8, per-group scales (no reference counterpart: parity unpinned) ------------

@pytest.mark.parametrize("m", [1, 2, 3, 4, 7, 8, 16])
@pytest.mark.parametrize("n,k,group", [(14336, 4096, 128), (300, 512, 64), (17, 1024, 128), (4096, 11008, 128),
                                       (2064, 4096, 256), (2100, 4096, 128), (4100, 4096, 128), (4100, 4096, 256),
                                       (4100, 4096, 64), (4099, 4096, 32)])
def test_w8a16_group(device, oracle, m, n, k, group):
    """Checked against the fp64 brute force of the stated contract: fp32 accumulation
    over K=4096 plus the final bf16 rounding stay within one bf16 ulp (2^-7) of it."""
    import torch
    from vecops_amd import capi
    if n * k > 20e6 and m not in (1, 4, 16):
        pytest.skip("large case only at the BASELINE M values")
    x = synth.bf16_round(synth.normal(1, (m, k)))
    w = synth.int8_sym(2, (n, k))
    s = synth.scales(3, (n, k // group))
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
    capi.matmul_w8a16_group(dev_bf16(x, device), torch.from_numpy(w).to(device), torch.from_numpy(s).to(device), y,
                            group)
    torch.cuda.synchronize()
    _, want = oracle.matmul_w8a16_group(x, w, s, group)
    assert rel_err(synth.bf16_to_f32(host_bits(y)), want) <= 2 ** -7


@pytest.mark.parametrize("m", [1, 2, 4, 16])
@pytest.mark.parametrize("group", [128, 256])
def test_w8a16_group_strided_operands(device, oracle, m, group):
    """Rows of x, w and y that are longer than the operand (ldx, ldw, ldy beyond K, K and N) on the decode shape's
    kernels (K = 4096, N >= 4096, ragged N): the padding must neither be read into the sums nor written."""
    import torch
    from vecops_amd import capi
    n, k = 4100, 4096
    x = synth.bf16_round(synth.normal(5, (m, k)))
    w = synth.int8_sym(6, (n, k))
    s = synth.scales(7, (n, k // group))
    xp = torch.full((m, k + 64), float("nan"), dtype=torch.bfloat16, device=device)
    xp[:, :k] = dev_bf16(x, device)
    wp = torch.full((n, k + 256), 77, dtype=torch.int8, device=device)
    wp[:, :k] = torch.from_numpy(w).to(device)
    yp = torch.full((m, n + 24), 3.0, dtype=torch.bfloat16, device=device)
    capi.matmul_w8a16_group(xp[:, :k], wp[:, :k], torch.from_numpy(s).to(device), yp[:, :n], group)
    torch.cuda.synchronize()
    _, want = oracle.matmul_w8a16_group(x, w, s, group)
    assert rel_err(synth.bf16_to_f32(host_bits(yp[:, :n].contiguous())), want) <= 2 ** -7
    assert bool((yp[:, n:] == 3.0).all())


def test_w8a16_rejects_bad_arguments(device):
    import torch
    from vecops_amd import capi
    x = torch.zeros((17, 256), dtype=torch.bfloat16, device=device)
    w = torch.zeros((8, 256), dtype=torch.int8, device=device)
    s = torch.zeros((8, 2), device=device)
    y = torch.zeros((17, 8), dtype=torch.bfloat16, device=device)
    with pytest.raises(capi.VecopsHipError) as e:
        capi.matmul_w8a16_group(x, w, s, y, 128)
    assert e.value.code == 2                                   # m > 16 is another kernel family
    with pytest.raises(capi.VecopsHipError) as e:
        capi.matmul_w8a16_group(x[:4], w, s, y[:4], 100)
    assert e.value.code == 1


@pytest.mark.parametrize("kind,m,n,k,split", [("bf16", 640, 4096, 4096, 1), ("bf16", 896, 2560, 12288, 3), ("bf16", 1000, 2000, 8200, 4),
                                              ("i8", 768, 3072, 12288, 1), ("i8", 700, 4000, 8192, 1), ("i8", 700, 4000, 8208, 2)])
def test_mid_band_k_split(device, oracle, kind, m, n, k, split):
    """128 to 200 tiles of 128 x 128 with a long K: 128 x 128 tiles, whole on the four-stage kernel where it serves
    (one workgroup per compute unit) and with K split two to four ways otherwise - a K that is no whole number of K
    tiles, or many idle units and a very long K (partial sums in the workspace, summed in the order of the parts).
    Against the oracle (int8: exact), with a C input; the entry point that allocates nothing agrees within the bound."""
    import torch
    from vecops_amd import capi
    if kind == "bf16":
        a, b = synth.bf16_round(synth.uniform_pm1(1, (m, k))), synth.bf16_round(synth.uniform_pm1(2, (n, k)))
        ta, tb = dev_bf16(a, device), dev_bf16(b, device)
        cin = synth.uniform_pm1(3, (m, n)).astype(np.float32)
        c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    else:
        a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
        ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
        cin = (synth.draws(3, m * n) % np.uint64(1 << 20)).astype(np.int32).reshape(m, n)
        c = torch.full((m, n), -1, dtype=torch.int32, device=device)
    tci = torch.from_numpy(cin).to(device)
    plan = capi.plan_matmul(ta, tb, c, c_in=tci)
    assert capi.FAMILY_NAMES[plan.family] == "tile_128" and plan.split_k == split
    capi.matmul(ta, tb, c, c_in=tci)
    alone = torch.empty_like(c)
    capi.matmul_static_workspace(ta, tb, alone, c_in=tci)
    torch.cuda.synchronize()
    if kind == "bf16":
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a, b, want, cin=cin, acc_f64=True)
        assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)
        assert rel_err(alone.cpu().numpy(), want) <= fp32_tol(k)
    else:
        want = (a.astype(np.float64) @ b.astype(np.float64).T).astype(np.int64) + cin   # exact: sums stay below 2^53
        want = (want & 0xffffffff).astype(np.uint32).view(np.int32)
        assert np.array_equal(c.cpu().numpy(), want)
        assert np.array_equal(alone.cpu().numpy(), want)


@pytest.mark.parametrize("m,n,k,family,split", [(1024, 2048, 4096, "tile_128", 2), (1536, 1536, 1536, "tile_128", 1), (1408, 1408, 1408, "tile_64", 1)])
def test_fp32_operands_as_bf16_plans(device, m, n, k, family, split):
    """fp32 operands multiplied as bf16 (register-staged loads) around half the units' worth of 128 x 128 tiles: the table's
    plan - two K parts from 96 tiles and a long K - against float64 sums of the operands rounded to bf16."""
    import torch
    from vecops_amd import capi
    gen = torch.Generator(device="cpu").manual_seed(m + k)
    a = (torch.rand((m, k), generator=gen) * 2 - 1).to(device)
    b = (torch.rand((k, n), generator=gen) * 2 - 1).to(device)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    plan = capi.plan_matmul(a, b.t(), c)
    assert capi.FAMILY_NAMES[plan.family] == family and plan.split_k == split
    capi.matmul(a, b.t(), c)
    torch.cuda.synchronize()
    rows = torch.arange(0, m, 37, device=device)
    want = torch.matmul(a[rows].bfloat16().double(), b.bfloat16().double())
    assert rel_err(c[rows].double().cpu().numpy(), want.cpu().numpy()) <= fp32_tol(k)


@pytest.mark.parametrize("m,n,k,pad", [(768, 3072, 12288, 0), (768, 3072, 12289, 15)])
def test_mid_band_k_split_with_dequantisation(device, m, n, k, pad):
    """The mid band under the dequantising epilogue - unsplit on the four-stage kernel, and split (the epilogue applied
    by the kernel that sums the parts) for rows padded to 16 bytes around an odd K: bit for bit
    (float(acc + corr) * rs) * cs.  The workspace query, which is told extents only, must have answered for the split."""
    import torch
    from vecops_amd import capi
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    corr = ((synth.draws(5, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32)
    ta = torch.zeros(m, k + pad, dtype=torch.int8, device=device)
    tb = torch.zeros(n, k + pad, dtype=torch.int8, device=device)
    ta[:, :k], tb[:, :k] = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    # (whole K tiles and aligned rows run unsplit on the four-stage kernel; the odd K keeps the split)
    assert capi.lib().vecops_hip_matmul_i8_dequant_workspace(m, n, k) >= (2 * m * n * 4 if pad else 0)
    c = torch.full((m, n), float("nan"), device=device)
    capi.matmul_i8_dequant(ta[:, :k], tb[:, :k], torch.from_numpy(rs).to(device), torch.from_numpy(cs).to(device), c,
                           correction=torch.from_numpy(corr).to(device))
    torch.cuda.synchronize()
    acc = ((a.astype(np.float64) @ b.astype(np.float64).T).astype(np.int64) + corr[None, :]).astype(np.int32)   # exact in float64
    want = (acc.astype(np.float32) * rs[:, None].astype(np.float32)) * cs[None, :].astype(np.float32)
    assert np.array_equal(c.cpu().numpy(), want)


@pytest.mark.parametrize("kind,m,n,k", [("bf16", 1536, 11008, 2048), ("bf16", 1500, 11000, 2056), ("i8", 1536, 11008, 4096)])
def test_peeled_columns(device, oracle, kind, m, n, k):
    """Two rounds of 128 x 128 tiles and a few more: the rule table cuts the last columns of tiles off and runs them
    as a product of their own (few tiles, K split), so that the rest fills whole rounds.  Both parts against the
    oracle (int8: exact), with a C input; a required family runs the product whole."""
    import torch
    from vecops_amd import capi
    if kind == "bf16":
        a, b = synth.bf16_round(synth.uniform_pm1(1, (m, k))), synth.bf16_round(synth.uniform_pm1(2, (n, k)))
        ta, tb = dev_bf16(a, device), dev_bf16(b, device)
        if k % 64 == 0:
            tb = tb.t().contiguous().t()      # B stored [K,N]: with B [N,K] these extents take the 256 x 352 tile, which peels nothing
        cin = synth.uniform_pm1(3, (m, n)).astype(np.float32)
        c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    else:
        a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
        ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
        cin = (synth.draws(3, m * n) % np.uint64(1 << 20)).astype(np.int32).reshape(m, n)
        c = torch.full((m, n), -1, dtype=torch.int32, device=device)
    tci = torch.from_numpy(cin).to(device)
    if kind == "i8":
        tci = tci.t().contiguous().t()        # (a C input whose rows are not contiguous: not the 256 x 352 tile's)
    plan = capi.plan_matmul(ta, tb, c, c_in=tci)
    assert capi.FAMILY_NAMES[plan.family] == "tile_128" and plan.split_k == 1 and 0 < plan.peeled_columns <= 256
    whole_plan = capi.plan_matmul_family(ta, tb, c, capi.family_request("tile_128"), c_in=tci)
    assert whole_plan.peeled_columns == 0
    capi.matmul(ta, tb, c, c_in=tci)
    whole = torch.empty_like(c)
    capi.matmul_family(ta, tb, whole, capi.family_request("tile_128", split_k=1), c_in=tci)
    torch.cuda.synchronize()
    cut = n - plan.peeled_columns
    if kind == "bf16":
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a, b, want, cin=cin, acc_f64=True)
        got = c.cpu().numpy()
        assert rel_err(got[:, :cut], want[:, :cut]) <= fp32_tol(k) and rel_err(got[:, cut:], want[:, cut:]) <= fp32_tol(k)
        assert np.array_equal(got[:, :cut], whole.cpu().numpy()[:, :cut])   # the same kernel on the same tiles
    else:
        want = (a.astype(np.float64) @ b.astype(np.float64).T).astype(np.int64) + cin   # exact: sums stay below 2^53
        want = (want & 0xffffffff).astype(np.uint32).view(np.int32)
        assert np.array_equal(c.cpu().numpy(), want)
