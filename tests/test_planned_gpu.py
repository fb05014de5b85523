"""vecops_hip_matmul_planned: the prepared invocation (vecops ops/Matmul.h:183-500, docs/Runtime.md:196-206) - a plan
made once by the planning entries and handed to every later call.  The planned call must give the bits of the unplanned
one (same kernels), accept the plans of the family entry, and refuse plans that do not fit the operands."""
import numpy as np
import pytest

from conftest import rel_err
from vecops_amd import synth

pytestmark = pytest.mark.gpu


def _bf16(torch, device, seed, shape):
    bits = synth.bf16_round(synth.uniform_pm1(seed, shape))
    return bits, torch.from_numpy(bits.view(np.int16)).to(device).view(torch.bfloat16)


@pytest.mark.parametrize("m,n,k", [(300, 520, 1000), (255, 63, 8191), (1, 4097, 129), (1536, 11008, 2048), (768, 4096, 4096),
                                   (0, 5, 7), (5, 7, 0)])
def test_planned_call_equals_the_unplanned_one(device, oracle, m, n, k):
    import torch
    from vecops_amd import capi
    a_bits, a = _bf16(torch, device, 1, (m, k))
    b_bits, b = _bf16(torch, device, 2, (n, k))
    want = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    got = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    plan = capi.plan_matmul(a, b, got)
    capi.matmul(a, b, want)
    capi.matmul_planned(a, b, got, plan)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    if m and n:
        ref = np.zeros((m, n), np.float32)
        oracle.matmul(a_bits, b_bits, ref, acc_f64=True)
        assert rel_err(got.cpu().numpy(), ref) <= 2e-6 * max(1, k // 32)
    # the prepared form of the binding goes through the same entry
    run = capi.PreparedMatmul(a, b, got)
    got.fill_(float("nan"))
    run()
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))


def test_planned_call_takes_the_family_entrys_plans(device):
    import torch
    from vecops_amd import capi
    m, n, k = 300, 520, 1000
    _, a = _bf16(torch, device, 1, (m, k))
    _, b = _bf16(torch, device, 2, (n, k))
    for family, split in (("tile_256", 1), ("tile_128", 3), ("tile_64", 2), ("tile_128x256", 1)):
        request = capi.family_request(family, capi.SELECT_REQUIRE, split_k=split)
        want = torch.empty((m, n), dtype=torch.float32, device=device)
        capi.matmul_family(a, b, want, request)
        plan = capi.plan_matmul_family(a, b, want, request)
        got = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
        capi.matmul_planned(a, b, got, plan)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (family, split)


def test_planned_call_refuses_plans_that_do_not_fit(device):
    import torch
    from vecops_amd import capi
    m, n, k = 300, 520, 1000
    _, a = _bf16(torch, device, 1, (m, k))
    _, b = _bf16(torch, device, 2, (n, k))
    c = torch.full((m, n), 7.0, dtype=torch.float32, device=device)
    good = capi.plan_matmul(a, b, c)

    def broken(**fields):
        p = capi.Plan()
        for name, _ in capi.Plan._fields_:
            setattr(p, name, getattr(good, name))
        for name, value in fields.items():
            setattr(p, name, value)
        return p
    cases = {"the skinny family on a square product": broken(family=capi.FAMILY_CODES["skinny"], split_k=1),
             "the int8 tile on bf16 operands": broken(family=capi.FAMILY_CODES["tile_256x352"], split_k=1),
             "more parts than K tiles": broken(family=capi.FAMILY_CODES["tile_64"], split_k=1000),
             "no parts": broken(split_k=0),
             "the empty family on a product": broken(family=capi.FAMILY_CODES["none"], split_k=1),
             "peeled columns the table does not peel": broken(peeled_columns=128),
             "an unknown family": broken(family=99)}
    for name, plan in cases.items():
        with pytest.raises(capi.VecopsHipError) as err:
            capi.matmul_planned(a, b, c, plan)
        assert err.value.code == 1, name
    # a workspace that is too small for the plan's (recomputed) need
    split = capi.plan_matmul_family(a, b, c, capi.family_request("tile_64", capi.SELECT_REQUIRE, split_k=4))
    split.workspace_bytes = 0          # a lie: the need is recomputed, not trusted
    with pytest.raises(capi.VecopsHipError):
        lib = capi.lib()
        import ctypes as C
        oa, ob, oc = capi.operand(a), capi.operand(b), capi.operand(c)
        capi._check(lib.vecops_hip_matmul_planned(C.byref(oa), C.byref(ob), None, C.byref(oc), 0, C.byref(split), None, 0, None))
    torch.cuda.synchronize()
    assert float(c.min()) == 7.0 and float(c.max()) == 7.0     # nothing was launched


def test_config2_full_coverage_checksum(device):
    """bf16 4096^3 with B as [K,N] (the headline workload): every output enters a checksum - C v against A (B^T v) in
    float64 for two random vectors v and u^T C against (u^T A) B^T - so a tile written to the wrong place, or not at
    all, shows.  Tolerance: the fp32 output's rounding and summation order, 2e-6 * K / 32 relative to the sum of
    magnitudes that enter each checksum."""
    import torch
    from vecops_amd import capi
    n = 4096
    a = synth.bf16_round(synth.normal(1, (n, n), 0.02))
    b_kn = synth.bf16_round(synth.normal(2, (n, n), 0.02))
    ta = torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
    tb = torch.from_numpy(b_kn.view(np.int16)).to(device).view(torch.bfloat16).t()
    c = torch.full((n, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul(ta, tb, c)
    torch.cuda.synchronize()
    got = c.double()
    ad, bd = ta.double(), tb.double()                      # bd: [N, K]
    rng = np.random.default_rng(5)
    for _ in range(2):
        v = torch.from_numpy(rng.standard_normal(n)).to(device)
        u = torch.from_numpy(rng.standard_normal(n)).to(device)
        tol = 2e-6 * n / 32
        right, want_right = got @ v, ad @ (bd.t() @ v)
        scale_right = (ad.abs() @ (bd.abs().t() @ v.abs()))
        assert bool(((right - want_right).abs() <= tol * scale_right).all())
        left, want_left = u @ got, (u @ ad) @ bd.t()
        scale_left = (u.abs() @ ad.abs()) @ bd.abs().t()
        assert bool(((left - want_left).abs() <= tol * scale_left).all())
    # and the bf16 output of the same call sequence is the rounded fp32 output, element for element
    c16 = torch.empty((n, n), dtype=torch.bfloat16, device=device)
    capi.matmul(ta, tb, c16)
    torch.cuda.synchronize()
    assert torch.equal(c16, c.to(torch.bfloat16))


@pytest.mark.parametrize("out", ["bf16", "transposed"])
def test_peeled_columns_other_outputs(device, oracle, out):
    """The peeled-columns plan with a bf16 output and with a C whose columns are the contiguous direction
    (the transposed view of an [N, M] tensor): both parts against the oracle."""
    import torch
    from vecops_amd import capi
    m, n, k = 1536, 11008, 2048
    a_bits, a = _bf16(torch, device, 1, (m, k))
    b_bits, b = _bf16(torch, device, 2, (n, k))
    if out == "bf16":
        # (B stored [K,N]: with B [N,K] and a row-major bf16 C these extents take the 256 x 352 tile, which peels nothing)
        b = b.t().contiguous().t()
    if out == "bf16":
        c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
    else:
        c = torch.full((n, m), float("nan"), dtype=torch.float32, device=device).t()
    plan = capi.plan_matmul(a, b, c)
    assert plan.peeled_columns > 0
    capi.matmul(a, b, c)
    torch.cuda.synchronize()
    rows = np.arange(0, m, 29)
    want = np.zeros((len(rows), n), np.float32)
    oracle.matmul(np.ascontiguousarray(a_bits[rows]), b_bits, want, acc_f64=True)
    got = c.float().cpu().numpy()[rows]
    tol = 2e-6 * k / 32 + (2.0 ** -8 if out == "bf16" else 0.0)
    cut = n - plan.peeled_columns
    assert rel_err(got[:, :cut], want[:, :cut]) <= tol and rel_err(got[:, cut:], want[:, cut:]) <= tol
