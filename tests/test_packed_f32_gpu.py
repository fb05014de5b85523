"""Packing for the fp32-compute atom (ops::MatmulPack is generic over atoms, ops/MatmulPack.h:9-117; SME_F32F32,
matmul/details/kernel/sme/Atoms.h:96): an fp32 operand packed with its elements kept fp32 (vecops_hip_pack_as with packed
dtype f32) and the products against it, either side and both.  The pack is a permutation plus zero padding, checked
byte for byte against the numpy restatement of the layout; the products are checked against fp64 within the fp32
summation-order bound and, where the plain fp32-compute kernel runs the same tile, bit for bit against it."""
import numpy as np
import pytest

from conftest import rel_err
from vecops_amd import synth
from test_matmul_gpu import fp32_tol
from test_packed_gpu import packed_layout_numpy

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,k", [(1, 1), (19, 35), (32, 32), (33, 129), (300, 1000)])
def test_pack_f32_layout(device, n, k):
    import torch
    from vecops_amd import capi
    b = synth.uniform_pm1(7, (n, k))
    want = packed_layout_numpy(b, 4)
    assert capi.lib().vecops_hip_packed_b_bytes(capi.F32, n, k) == want.size
    padded = torch.full((n, k + 3), -99.0, dtype=torch.float32, device=device)
    padded[:, :k] = torch.from_numpy(b).to(device)
    for source in (torch.from_numpy(b).to(device), padded[:, :k], torch.from_numpy(np.ascontiguousarray(b.T)).to(device).t()):
        packed = capi.pack_b(source, compute=capi.COMPUTE_F32)
        torch.cuda.synchronize()
        assert packed.dtype == capi.F32
        assert np.array_equal(packed.storage.cpu().numpy()[:want.size], want)
    # without the compute type an fp32 source still packs as bf16
    assert capi.pack_b(torch.from_numpy(b).to(device)).dtype == capi.BF16


@pytest.mark.parametrize("m,n,k", [(35, 53, 257), (64, 64, 32), (300, 520, 1000), (1024, 1024, 1024), (2, 700, 144),
                                   (513, 257, 96), (1536, 2048, 520)])
def test_packed_f32_products(device, m, n, k):
    """B packed, A packed and both, against fp64; operands that bf16 rounding would visibly change."""
    import torch
    from vecops_amd import capi
    a, b = synth.uniform_pm1(1, (m, k)), synth.uniform_pm1(2, (n, k))
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    want = a.astype(np.float64) @ b.astype(np.float64).T
    pa, pb = capi.pack_a(ta, compute=capi.COMPUTE_F32), capi.pack_b(tb, compute=capi.COMPUTE_F32)
    plain = torch.full((m, n), float("nan"), device=device)
    capi.matmul(ta, tb, plain, compute=capi.COMPUTE_F32)
    for run in (lambda c: capi.matmul_packed_b(ta, pb, c), lambda c: capi.matmul_packed_a(pa, tb, c),
                lambda c: capi.matmul_packed_ab(pa, pb, c)):
        c = torch.full((m, n), float("nan"), device=device)
        run(c)
        torch.cuda.synchronize()
        got = c.cpu().numpy()
        assert rel_err(got, want) <= fp32_tol(k)
        # fp32 products: far inside what rounding the operands to bf16 leaves (about 1e-3 of the largest element here)
        assert rel_err(got, want) <= 1e-4
    assert rel_err(plain.cpu().numpy(), want) <= fp32_tol(k)


def test_packed_f32_batched_cin_strides_and_rejections(device):
    """One packed B for every batch of a rank-3 A, a C input, a strided A and a transposed C; operand classes that do not
    go with an f32 pack are refused."""
    import torch
    from vecops_amd import capi
    batch, m, n, k = 3, 70, 130, 264
    a, b = synth.uniform_pm1(1, (batch, m, k + 5)), synth.uniform_pm1(2, (n, k))
    cin = synth.uniform_pm1(3, (batch, m, n))
    ta = torch.from_numpy(a).to(device)[:, :, :k]
    pb = capi.pack_b(torch.from_numpy(b).to(device), compute=capi.COMPUTE_F32)
    store = torch.full((batch, n, m), float("nan"), device=device)
    c = store.transpose(1, 2)
    capi.matmul_packed_b(ta, pb, c, c_in=torch.from_numpy(cin).to(device))
    torch.cuda.synchronize()
    want = cin.astype(np.float64) + np.einsum("bmk,nk->bmn", a[:, :, :k].astype(np.float64), b.astype(np.float64))
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)
    with pytest.raises(capi.VecopsHipError) as err:        # a bf16 a does not multiply an f32 pack
        capi.matmul_packed_b(torch.zeros((4, k), dtype=torch.bfloat16, device=device), pb,
                             torch.empty((4, n), dtype=torch.float32, device=device))
    assert err.value.code == 2
    import ctypes as C
    ob = capi.operand(torch.zeros((8, 64), dtype=torch.bfloat16, device=device))
    buf = torch.empty(1 << 16, dtype=torch.uint8, device=device)
    assert capi.lib().vecops_hip_pack_as(C.byref(ob), capi.F32, buf.data_ptr(), 1 << 16, None) == 2   # bf16 does not widen
    of = capi.operand(torch.zeros((8, 64), device=device))
    assert capi.lib().vecops_hip_pack_as(C.byref(of), capi.F32, buf.data_ptr(), 16, None) == 1        # too small
    assert capi.lib().vecops_hip_pack_as(C.byref(of), capi.F16, buf.data_ptr(), 1 << 16, None) == 2   # f32 does not pack as half
