"""Several independent products in one call (vecops_hip_matmul_grouped: irregular batches) and the mirror image of
the shared-B batch folding (one row of A for every batch, vecops' batch-columns flattening,
planning/families/ArchitectureBatchPlanner.h:82-160), through the C ABI against the oracle."""
import numpy as np
import pytest

from vecops_amd import synth

pytestmark = pytest.mark.gpu


def rel_err(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)) / np.maximum(1.0, np.abs(want))))


def fp32_tol(k):
    return 2e-6 * max(1.0, k / 32)


def dev_bf16(x_bits, device):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x_bits).view(np.int16)).to(device).view(torch.bfloat16)


def host_bits(t):
    import torch
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


BF16_GROUPS = {
    # every group in whole tiles of every candidate size
    "regular": [(256, 512, 128), (512, 256, 192), (256, 256, 64)],
    # ragged M, N and K; a single row; a group smaller than any tile
    "ragged": [(300, 200, 520), (64, 1000, 136), (1, 77, 64), (513, 257, 1000), (5, 3, 8)],
    # enough work for 128 x 128 tiles, and for 256 x 256 ones
    "medium": [(1000, 1300, 264), (700, 900, 264), (1500, 400, 520), (130, 2000, 72)],
    "large": [(2048, 2048, 520), (3000, 1000, 264), (1024, 4096, 136), (4000, 2000, 72), (2500, 2500, 200)],
    # more groups than one table chunk carries
    "many": [(40 + 7 * i, 300 - 5 * i, 64 + 8 * (i % 5)) for i in range(31)],
    # groups whose K the rule table splits (launches of their own, partial sums behind the table) among others
    "long_k": [(255, 63, 8191), (300, 200, 520), (100, 40, 4099), (700, 900, 264), (500, 300, 4100)],
}


@pytest.mark.parametrize("name", list(BF16_GROUPS))
def test_grouped_bf16_equals_the_oracle_and_the_single_calls(device, oracle, name):
    """bf16 groups of unlike shapes in one launch: fp32 and bf16 outputs, every other group with a C input; each
    group against the oracle, and bit-equal to vecops_hip_matmul on that group alone on the tile shape the grouped
    launch took (one of the three square ones), K unsplit: the same kernel body, the same order of sums.  (One
    exception: with K of 256 or less the single call's 128 x 128 tile multiplies on the 32x32 MFMA shape, the
    grouped launch's on the 16x16 one - another order of sums inside a K tile.)"""
    import torch
    from vecops_amd import capi
    shapes = BF16_GROUPS[name]
    ha, hb, hci, ta, tb, tc, tci = [], [], [], [], [], [], []
    for i, (m, n, k) in enumerate(shapes):
        ha.append(synth.bf16_round(synth.uniform_pm1(10 + i, (m, k))))
        hb.append(synth.bf16_round(synth.uniform_pm1(50 + i, (n, k))))
        hci.append(synth.uniform_pm1(90 + i, (m, n)).astype(np.float32) if i % 2 else None)
        ta.append(dev_bf16(ha[-1], device))
        tb.append(dev_bf16(hb[-1], device))
        tci.append(torch.from_numpy(hci[-1]).to(device) if hci[-1] is not None else None)
        tc.append(torch.full((m, n), float("nan"), dtype=torch.float32 if i % 3 else torch.bfloat16, device=device))
    capi.matmul_grouped(ta, tb, tc, c_in_list=tci)
    torch.cuda.synchronize()
    for i, (m, n, k) in enumerate(shapes):
        want = np.zeros((m, n), np.float32)
        oracle.matmul(ha[i], hb[i], want, cin=hci[i], acc_f64=True)
        if tc[i].dtype == torch.float32:
            assert rel_err(tc[i].cpu().numpy(), want) <= fp32_tol(k), (name, i)
        else:
            got = synth.bf16_to_f32(host_bits(tc[i]))
            assert rel_err(got, want) <= 2.0 ** -8 + fp32_tol(k), (name, i)
        same_bits = []
        for family in ("tile_256", "tile_128", "tile_64"):
            alone = torch.empty_like(tc[i])
            capi.matmul_family(ta[i], tb[i], alone, capi.family_request(family, split_k=1), c_in=tci[i])
            torch.cuda.synchronize()
            same_bits.append(np.array_equal(host_bits(tc[i]), host_bits(alone)))
        plan = capi.plan_matmul(ta[i], tb[i], tc[i], c_in=tci[i])
        if plan.split_k > 1:       # a group that splits K runs vecops_hip_matmul's own plan
            alone = torch.empty_like(tc[i])
            capi.matmul(ta[i], tb[i], alone, c_in=tci[i])
            torch.cuda.synchronize()
            assert np.array_equal(host_bits(tc[i]), host_bits(alone)), (name, i)
        else:
            assert any(same_bits) or k <= 256, (name, i)
    if name == "long_k":
        assert sum(capi.plan_matmul(ta[i], tb[i], tc[i], c_in=tci[i]).split_k > 1 for i in range(len(shapes))) >= 2


def test_grouped_int8_bit_exact_with_degenerate_groups(device, oracle):
    """int8 groups (int32 sums, exact), among them a group with K = 0 (c = c_in), one with no rows, and rank-3 groups
    (a batch inside a group)."""
    import torch
    from oracle import oracle as O
    from vecops_amd import capi
    shapes = [(300, 200, 520), (0, 64, 32), (64, 500, 0), (129, 131, 1000), (17, 900, 144), (700, 700, 256)]
    ha, hb, hci, ta, tb, tc, tci = [], [], [], [], [], [], []
    for i, (m, n, k) in enumerate(shapes):
        ha.append(synth.int8_sym(10 + i, (m, k)))
        hb.append(synth.int8_sym(50 + i, (n, k)))
        hci.append((synth.int8_sym(90 + i, (m, n)).astype(np.int32) * 1000) if i in (2, 3) else None)
        ta.append(torch.from_numpy(ha[-1]).to(device))
        tb.append(torch.from_numpy(hb[-1]).to(device))
        tci.append(torch.from_numpy(hci[-1]).to(device) if hci[-1] is not None else None)
        tc.append(torch.full((m, n), -7, dtype=torch.int32, device=device))
    # a rank-3 group: two batches of its own
    a3, b3 = synth.int8_sym(7, (2, 70, 200)), synth.int8_sym(8, (2, 90, 200))
    ta.append(torch.from_numpy(a3).to(device)); tb.append(torch.from_numpy(b3).to(device)); tci.append(None)
    tc.append(torch.full((2, 70, 90), -7, dtype=torch.int32, device=device))
    capi.matmul_grouped(ta, tb, tc, c_in_list=tci)
    torch.cuda.synchronize()
    for i, (m, n, k) in enumerate(shapes):
        want = np.zeros((m, n), np.int32)
        if m and n:
            oracle.matmul(ha[i], hb[i], want, cin=hci[i], atom=O.ATOM_I8I32, acc_f64=True, c_bf16=False)
        assert np.array_equal(tc[i].cpu().numpy(), want), i
    want3 = np.einsum("bmk,bnk->bmn", a3.astype(np.int64), b3.astype(np.int64)).astype(np.int32)
    assert np.array_equal(tc[-1].cpu().numpy(), want3)


def test_grouped_mixed_layouts_and_unaligned_operands(device, oracle):
    """Groups whose B is stored [K,N], groups with unaligned rows and views with gaps: the weakest loader any group
    needs serves them all; nothing outside a group's C is written."""
    import torch
    from vecops_amd import capi
    for layouts in (("kn", "kn", "kn"), ("kn", "nk", "kn"), ("nk", "odd", "nk"), ("gap", "gap", "nk")):
        shapes = [(200, 264, 136), (130, 520, 264), (384, 136, 72)]
        ha, hb, ta, tb, tc, stores = [], [], [], [], [], []
        for i, ((m, n, k), layout) in enumerate(zip(shapes, layouts)):
            if layout == "odd":
                k += 3                                                # rows no longer 16-byte aligned
            ha.append(synth.bf16_round(synth.uniform_pm1(20 + i, (m, k))))
            hb.append(synth.bf16_round(synth.uniform_pm1(60 + i, (n, k))))
            a, b = dev_bf16(ha[-1], device), dev_bf16(hb[-1], device)
            if layout == "kn":
                b = b.t().contiguous().t()                            # [N,K] view of a [K,N] row-major store
            store = torch.full((m + 2, n + 8), float("nan"), dtype=torch.float32, device=device)
            if layout == "gap":
                wide = torch.zeros((m, k + 8), dtype=torch.bfloat16, device=device)
                wide[:, :k] = a
                a = wide[:, :k]
            ta.append(a); tb.append(b); stores.append(store); tc.append(store[:m, :n])
        capi.matmul_grouped(ta, tb, tc)
        torch.cuda.synchronize()
        for i, (m, n, _) in enumerate(shapes):
            k = ha[i].shape[1]
            want = np.zeros((m, n), np.float32)
            oracle.matmul(ha[i], hb[i], want, acc_f64=True)
            assert rel_err(tc[i].cpu().numpy(), want) <= fp32_tol(k), (layouts, i)
            assert torch.isnan(stores[i][m:]).all() and torch.isnan(stores[i][:, n:]).all()


@pytest.mark.parametrize("kind", ["f32_as_bf16", "f32", "f16"])
def test_grouped_floating_classes_in_one_launch(device, oracle, kind):
    """fp32 operands in both compute types and f16 operands: groups of unlike shapes (ragged, a C input on every
    other one, enough tiles for the 128 x 128 shape) through the grouped launch, each against the oracle and
    bit-equal to the single call on one of the three square tile shapes, K unsplit (in fp32 compute; with bf16 or
    f16 compute the single call's 128 x 128 tile takes the other MFMA shape where K is 256 or less)."""
    import torch
    from vecops_amd import capi
    shapes = [(70, 90, 200), (300, 20, 64), (1000, 1300, 136), (700, 900, 264), (1, 33, 40), (513, 257, 96)]
    compute = capi.COMPUTE_F32 if kind == "f32" else capi.COMPUTE_BF16
    ha, hb, hci, ta, tb, tc, tci = [], [], [], [], [], [], []
    for i, (m, n, k) in enumerate(shapes):
        a, b = synth.uniform_pm1(10 + i, (m, k)), synth.uniform_pm1(50 + i, (n, k))
        if kind == "f16":
            a, b = a.astype(np.float16), b.astype(np.float16)
        ha.append(a)
        hb.append(b)
        hci.append(synth.uniform_pm1(90 + i, (m, n)).astype(np.float32) if i % 2 else None)
        ta.append(torch.from_numpy(a).to(device))
        tb.append(torch.from_numpy(b).to(device))
        tci.append(torch.from_numpy(hci[-1]).to(device) if hci[-1] is not None else None)
        tc.append(torch.full((m, n), float("nan"), dtype=torch.float32, device=device))
    capi.matmul_grouped(ta, tb, tc, c_in_list=tci, compute=compute)
    torch.cuda.synchronize()
    for i, (m, n, k) in enumerate(shapes):
        if kind == "f32_as_bf16":   # operands rounded to bf16 on the way in, products and sums in fp32
            a64, b64 = (synth.bf16_to_f32(synth.bf16_round(x)).astype(np.float64) for x in (ha[i], hb[i]))
        else:
            a64, b64 = ha[i].astype(np.float64), hb[i].astype(np.float64)
        want = a64 @ b64.T + (hci[i] if hci[i] is not None else 0.0)
        assert rel_err(tc[i].cpu().numpy(), want) <= fp32_tol(k), (kind, i)
        same_bits = []
        for family in ("tile_256", "tile_128", "tile_64"):
            alone = torch.empty_like(tc[i])
            capi.matmul_family(ta[i], tb[i], alone, capi.family_request(family, split_k=1), c_in=tci[i], compute=compute)
            torch.cuda.synchronize()
            same_bits.append(np.array_equal(tc[i].cpu().numpy(), alone.cpu().numpy()))
        assert any(same_bits) or (kind != "f32" and k <= 256), (kind, i)


def test_grouped_unsigned_sides_in_one_launch(device):
    """Groups with an unsigned 8-bit side (AMX_I8I32<uint8_t, int8_t>, <int8_t, uint8_t>, <uint8_t, uint8_t>; the
    reference's batch planner serves every atom alike, planning/families/ArchitectureFamily.h:430-463): one table,
    every group with its own sign flips and row-sum terms in the workspace.  Exact sums mod 2^32, ragged shapes, a
    C input on every other group, bytes of the full range; and the result of each group equals its single call's."""
    import torch
    from vecops_amd import capi

    def raw(seed, shape, unsigned):
        x = (synth.draws(seed, int(np.prod(shape))) % np.uint64(256)).astype(np.uint8).reshape(shape)
        return x if unsigned else x.view(np.int8)
    cases = [((70, 90, 200), True, False), ((300, 20, 64), True, True), ((1000, 1300, 136), False, True),
             ((513, 257, 96), True, True), ((1, 33, 40), True, False), ((700, 900, 1100), False, True)]
    ha, hb, hci, ta, tb, tc, tci = [], [], [], [], [], [], []
    for i, ((m, n, k), au, bu) in enumerate(cases):
        ha.append(raw(10 + i, (m, k), au))
        hb.append(raw(50 + i, (n, k), bu))
        hci.append(synth.int8_sym(90 + i, (m, n)).astype(np.int32) * 1000 if i % 2 else None)
        ta.append(torch.from_numpy(ha[-1]).to(device))
        tb.append(torch.from_numpy(hb[-1]).to(device))
        tci.append(torch.from_numpy(hci[-1]).to(device) if hci[-1] is not None else None)
        tc.append(torch.full((m, n), -1, dtype=torch.int32, device=device))
    capi.matmul_grouped(ta, tb, tc, c_in_list=tci)
    torch.cuda.synchronize()
    for i in range(len(cases)):
        want = ha[i].astype(np.int64) @ hb[i].astype(np.int64).T + (hci[i] if hci[i] is not None else 0)
        assert np.array_equal(tc[i].cpu().numpy(), (want & 0xffffffff).astype(np.uint32).view(np.int32)), cases[i]
        alone = torch.full_like(tc[i], -1)
        capi.matmul(ta[i], tb[i], alone, c_in=tci[i])
        torch.cuda.synchronize()
        assert torch.equal(alone, tc[i])
    # too small a workspace is refused before anything runs
    Operands = capi.Operand * len(cases)
    oa, ob, oc = (Operands(*map(capi.operand, xs)) for xs in (ta, tb, tc))
    need = capi.lib().vecops_hip_matmul_grouped_workspace(len(cases), oa, ob, None, oc, 0)
    assert need >= sum(4 * (m + n) for (m, n, _), _, _ in cases)
    ws = torch.empty(need, dtype=torch.uint8, device=device)
    assert capi.lib().vecops_hip_matmul_grouped(len(cases), oa, ob, None, oc, 0, ws.data_ptr(), need - 256, None) == 1


def test_grouped_other_classes_run_group_by_group(device, oracle):
    """Two unsigned-side groups, then a mix of classes (launches of their own): the same entry point."""
    import torch
    from vecops_amd import capi
    def u8(seed, shape):
        return (synth.int8_sym(seed, shape).astype(np.int16) + 128).astype(np.uint8)
    ua, ub = u8(1, (70, 200)), synth.int8_sym(2, (90, 200))
    va, vb = u8(3, (300, 64)), u8(4, (20, 64))
    c0 = torch.zeros((70, 90), dtype=torch.int32, device=device)
    c1 = torch.zeros((300, 20), dtype=torch.int32, device=device)
    capi.matmul_grouped([torch.from_numpy(ua).to(device), torch.from_numpy(va).to(device)],
                        [torch.from_numpy(ub).to(device), torch.from_numpy(vb).to(device)], [c0, c1])
    torch.cuda.synchronize()
    for a, b, c in ((ua, ub, c0), (va, vb, c1)):
        assert np.array_equal(c.cpu().numpy(), (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32))
    # a bf16 group beside an int8 group
    ha, hb = synth.bf16_round(synth.uniform_pm1(5, (100, 72))), synth.bf16_round(synth.uniform_pm1(6, (50, 72)))
    ia, ib = synth.int8_sym(7, (60, 144)), synth.int8_sym(8, (40, 144))
    cf = torch.full((100, 50), float("nan"), device=device)
    ci = torch.zeros((60, 40), dtype=torch.int32, device=device)
    capi.matmul_grouped([dev_bf16(ha, device), torch.from_numpy(ia).to(device)],
                        [dev_bf16(hb, device), torch.from_numpy(ib).to(device)], [cf, ci])
    torch.cuda.synchronize()
    want = np.zeros((100, 50), np.float32)
    oracle.matmul(ha, hb, want, acc_f64=True)
    assert rel_err(cf.cpu().numpy(), want) <= fp32_tol(72)
    assert np.array_equal(ci.cpu().numpy(), (ia.astype(np.int64) @ ib.astype(np.int64).T).astype(np.int32))
    # validation: a group whose operands disagree names the problem
    with pytest.raises(capi.VecopsHipError) as e:
        capi.matmul_grouped([dev_bf16(ha, device)], [dev_bf16(hb[:, :64], device)], [cf])
    assert e.value.code == 1
    capi.matmul_grouped([], [], [])                                   # no groups: nothing to do


@pytest.mark.parametrize("batch,n,k,dtype", [(8, 512, 264, "bf16"), (5, 1000, 1024, "bf16"), (16, 300, 520, "i8"), (3, 64, 72, "bf16")])
def test_shared_a_row_batch_is_folded(device, oracle, batch, n, k, dtype):
    """One row of A for every batch (M = 1, batch stride 0) against per-batch weights whose rows run on, the outputs
    laid end to end: planned and run as the [1, batch * N] product (vecops' batch-columns flattening); with gaps
    between the outputs of the batches the batched form gives the same values."""
    import torch
    from oracle import oracle as O
    from vecops_amd import capi
    if dtype == "bf16":
        a = synth.bf16_round(synth.uniform_pm1(1, (1, k)))
        b = synth.bf16_round(synth.uniform_pm1(2, (batch, n, k)))
        ta, tb = dev_bf16(a, device).expand(batch, 1, k), dev_bf16(b, device)
        want = np.zeros((batch, 1, n), np.float32)
        oracle.matmul(np.broadcast_to(a, (batch, 1, k)), b, want, acc_f64=True)
        c = torch.full((batch, 1, n), float("nan"), device=device)
    else:
        a, b = synth.int8_sym(1, (1, k)), synth.int8_sym(2, (batch, n, k))
        ta, tb = torch.from_numpy(a).to(device).expand(batch, 1, k), torch.from_numpy(b).to(device)
        want = np.einsum("k,bnk->bn", a[0].astype(np.int64), b.astype(np.int64)).astype(np.int32).reshape(batch, 1, n)
        c = torch.full((batch, 1, n), -7, dtype=torch.int32, device=device)
    folded = capi.plan_matmul(ta, tb, c)
    gapped_store = torch.zeros((batch, 1, n + 8), dtype=c.dtype, device=device)
    unfolded = capi.plan_matmul(ta, tb, gapped_store[:, :, :n])
    capi.matmul(ta, tb, c)
    capi.matmul(ta, tb, gapped_store[:, :, :n])
    torch.cuda.synchronize()
    for got in (c, gapped_store[:, :, :n]):
        if dtype == "bf16":
            assert rel_err(got.cpu().numpy(), want) <= fp32_tol(k)
        else:
            assert np.array_equal(got.cpu().numpy(), want)
    assert (gapped_store[:, :, n:] == 0).all()
    if batch * n >= 512 and k % 16 == 0:
        assert capi.FAMILY_NAMES[folded.family] == "skinny"          # one long GEMV instead of `batch` short ones
    else:
        assert folded.family == unfolded.family or unfolded.split_k >= 1


def test_prepared_grouped_call_repeats_the_plain_one(device):
    """capi.PreparedGrouped: descriptors and workspace built once, every call one foreign call; same bits as
    matmul_grouped, call after call."""
    import torch
    from vecops_amd import capi
    shapes = [(300, 200, 520), (64, 1000, 136), (1, 77, 64), (1000, 1300, 264)]
    a_list = [dev_bf16(synth.bf16_round(synth.uniform_pm1(10 + i, (m, k))), device) for i, (m, n, k) in enumerate(shapes)]
    b_list = [dev_bf16(synth.bf16_round(synth.uniform_pm1(40 + i, (n, k))), device) for i, (m, n, k) in enumerate(shapes)]
    want = [torch.empty((m, n), dtype=torch.float32, device=device) for m, n, k in shapes]
    capi.matmul_grouped(a_list, b_list, want)
    got = [torch.full((m, n), float("nan"), dtype=torch.float32, device=device) for m, n, k in shapes]
    run = capi.PreparedGrouped(a_list, b_list, got)
    for _ in range(3):
        for t in got:
            t.fill_(float("nan"))
        run()
        torch.cuda.synchronize()
        assert all(torch.equal(g, w) for g, w in zip(got, want))
