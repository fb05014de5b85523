"""fp64 operands (vecops' SME_F64F64 atom, matmul/details/kernel/sme/Atoms.h:108-112) through the C ABI against the
oracle.  The reference's own build of this atom needs an SME machine, so the oracle's fp64 path is pinned by the
mathematics in tests/test_oracle.py; here the GPU kernel meets it: bit for bit where every product and sum is exact
(small integers), within the reordering bound of an fp64 sum otherwise."""
import numpy as np
import pytest

from oracle import oracle as O
from vecops_amd import synth

pytestmark = pytest.mark.gpu


def f64(seed, shape):
    return (synth.uniform_pm1(seed, shape).astype(np.float64) + synth.uniform_pm1(seed + 100, shape).astype(np.float64) * 2.0 ** -25)


def bound(a, b, k):
    """|fl(sum) - sum| <= k * eps * sum |x||y| for any order of an fp64 sum of k products."""
    return k * 2.0 ** -52 * (np.abs(a) @ np.abs(b).T)


@pytest.mark.parametrize("m,n,k", [(16, 16, 4), (19, 21, 65), (1, 128, 65), (128, 1, 33), (37, 51, 79), (256, 256, 64),
                                   (300, 520, 1000), (1024, 768, 2048), (130, 140, 515), (5, 3, 1)])
def test_f64_gemm_against_the_oracle(device, oracle, m, n, k):
    import torch
    from vecops_amd import capi
    a, b, cin = f64(1, (m, k)), f64(2, (n, k)), f64(3, (m, n))
    ta, tb, tci = (torch.from_numpy(x).to(device) for x in (a, b, cin))
    c = torch.full((m, n), float("nan"), dtype=torch.float64, device=device)
    plan = capi.plan_matmul(ta, tb, c)
    assert capi.FAMILY_NAMES[plan.family] == "tile_128" and plan.split_k == 1 and plan.workspace_bytes == 0
    capi.matmul(ta, tb, c)
    c2 = torch.full((m, n), float("nan"), dtype=torch.float64, device=device)
    capi.matmul(ta, tb, c2, c_in=tci)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float64)
    oracle.matmul(a, b, want, atom=O.ATOM_F64F64)
    assert (np.abs(c.cpu().numpy() - want) <= 2 * bound(a, b, k) + 1e-300).all()
    want2 = np.zeros((m, n), np.float64)
    oracle.matmul(a, b, want2, cin=cin, atom=O.ATOM_F64F64)
    assert (np.abs(c2.cpu().numpy() - want2) <= 2 * bound(a, b, k) + 2.0 ** -52 * np.abs(want2)).all()


def test_f64_exact_on_small_integers_and_beyond_fp32(device, oracle):
    """Integer-valued operands: every product and partial sum is exact in fp64, so any order gives the same bits -
    and the values (up to 2^40) are out of reach of an fp32 or bf16 path."""
    import torch
    from vecops_amd import capi
    m, n, k = 200, 136, 520
    a = (synth.draws(1, m * k) % np.uint64(2 ** 20)).astype(np.float64).reshape(m, k) - 2.0 ** 19
    b = (synth.draws(2, n * k) % np.uint64(2 ** 20)).astype(np.float64).reshape(n, k) - 2.0 ** 19
    c = torch.empty((m, n), dtype=torch.float64, device=device)
    capi.matmul(torch.from_numpy(a).to(device), torch.from_numpy(b).to(device), c)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float64)
    oracle.matmul(a, b, want, atom=O.ATOM_F64F64)
    exact = (a.astype(object) @ b.astype(object).T).astype(np.float64) if m * n * k < 2e6 else want
    assert np.array_equal(c.cpu().numpy(), want) and np.array_equal(want, exact)
    assert np.abs(want).max() > 2.0 ** 40


def test_f64_layouts_batches_and_degenerate_extents(device, oracle):
    """B stored [K,N], a transposed A, a column-major C, padded rows, a rank-3 batch with a broadcast B (folded into rows)
    and one with per-batch operands, C_in aliasing C, K = 0, empty M / N / batch."""
    import torch
    from vecops_amd import capi
    m, n, k = 150, 90, 133
    a, b = f64(1, (m, k)), f64(2, (n, k))
    want = np.zeros((m, n), np.float64)
    oracle.matmul(a, b, want, atom=O.ATOM_F64F64)
    tol = 2 * bound(a, b, k)
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    views = {
        "b_kn": (ta, tb.t().contiguous().t(), torch.empty((m, n), dtype=torch.float64, device=device)),
        "a_t": (ta.t().contiguous().t(), tb, torch.empty((m, n), dtype=torch.float64, device=device)),
        "c_t": (ta, tb, torch.empty((n, m), dtype=torch.float64, device=device).t()),
        "padded": (torch.zeros((m, k + 3), dtype=torch.float64, device=device)[:, :k].copy_(ta), tb,
                   torch.full((m + 2, n + 5), float("nan"), dtype=torch.float64, device=device)[:m, :n]),
    }
    for name, (va, vb, vc) in views.items():
        capi.matmul(va, vb, vc)
        torch.cuda.synchronize()
        assert (np.abs(vc.cpu().numpy() - want) <= tol).all(), name
    # batches: shared B (rows of a and c run on: one [batch * M, K] product) and per-batch B
    batch = 3
    a3, b3 = f64(5, (batch, m, k)), f64(6, (batch, n, k))
    c3 = torch.empty((batch, m, n), dtype=torch.float64, device=device)
    capi.matmul(torch.from_numpy(a3).to(device), tb.unsqueeze(0).expand(batch, n, k), c3)
    c4 = torch.empty((batch, m, n), dtype=torch.float64, device=device)
    capi.matmul(torch.from_numpy(a3).to(device), torch.from_numpy(b3).to(device), c4)
    torch.cuda.synchronize()
    for i in range(batch):
        w = np.zeros((m, n), np.float64)
        oracle.matmul(a3[i], b, w, atom=O.ATOM_F64F64)
        assert (np.abs(c3[i].cpu().numpy() - w) <= 2 * bound(a3[i], b, k)).all()
        oracle.matmul(a3[i], b3[i], w, atom=O.ATOM_F64F64)
        assert (np.abs(c4[i].cpu().numpy() - w) <= 2 * bound(a3[i], b3[i], k)).all()
    # C_in aliasing C, K = 0, empty extents
    acc = torch.ones((m, n), dtype=torch.float64, device=device)
    capi.matmul(ta, tb, acc, c_in=acc)
    torch.cuda.synchronize()
    assert (np.abs(acc.cpu().numpy() - (want + 1.0)) <= tol + 2.0 ** -52 * np.abs(want + 1.0)).all()
    z = torch.full((4, 5), float("nan"), dtype=torch.float64, device=device)
    capi.matmul(torch.empty((4, 0), dtype=torch.float64, device=device), torch.empty((5, 0), dtype=torch.float64, device=device), z)
    torch.cuda.synchronize()
    assert (z == 0).all()
    capi.matmul(torch.empty((0, 8), dtype=torch.float64, device=device), torch.zeros((5, 8), dtype=torch.float64, device=device),
                torch.empty((0, 5), dtype=torch.float64, device=device))
    with pytest.raises(capi.VecopsHipError) as e:                     # fp64 operands write fp64
        capi.matmul(ta, tb, torch.empty((m, n), dtype=torch.float32, device=device))
    assert e.value.code == 2
    with pytest.raises(capi.VecopsHipError) as e:                     # only the fp64 kernel's own tile can be required
        capi.matmul_family(ta, tb, torch.empty((m, n), dtype=torch.float64, device=device),
                           capi.family_request("tile_256", capi.SELECT_REQUIRE))
    assert e.value.code == 2
