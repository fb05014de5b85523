"""Prepacked B operand (vecops_hip_pack_b / vecops_hip_matmul_packed_b) through the C ABI.

Packing is a permutation plus zero padding (ops/MatmulPack.h:16-21), so every
check is exact: the packed bytes against a numpy restatement of the documented
layout, and the packed matmul against the plain matmul of the same library bit
for bit as well as against the CPU oracle (integer: bit-exact; fp32 outputs:
the summation-order tolerance of test_matmul_gpu).  Shapes follow
tests/ops/MatmulPackTest.cpp:299-336 (full blocks and ragged tails) and
:354-433 (compensated pack, zero extents).
"""
import numpy as np
import pytest

from conftest import rel_err
from oracle import oracle as O
from vecops_amd import synth
from test_matmul_gpu import dev_bf16, fp32_tol, host_bits

pytestmark = pytest.mark.gpu


def packed_layout_numpy(b: np.ndarray, elem_bytes: int) -> np.ndarray:
    """[panel][k-step][k-half][row 32][k EPC] with zero padding, as bytes."""
    n, k = b.shape
    epc = 16 // elem_bytes
    ktile = 8 * epc
    kp = (k + ktile - 1) // ktile * ktile
    npad = (n + 31) // 32 * 32
    full = np.zeros((npad, kp), dtype=b.dtype)
    full[:n, :k] = b
    blocks = full.reshape(npad // 32, 32, kp // (2 * epc), 2, epc)  # [panel][row][k-step][half][k]
    return np.ascontiguousarray(blocks.transpose(0, 2, 3, 1, 4)).view(np.uint8).reshape(-1)


@pytest.mark.parametrize("n,k", [(16, 32), (19, 35), (1, 1), (32, 64), (33, 129), (300, 1000), (256, 4096)])
def test_pack_b_bf16_layout(device, n, k):
    import torch
    from vecops_amd import capi
    bits = synth.bf16_round(synth.uniform_pm1(7, (n, k)))
    packed = capi.pack_b(dev_bf16(bits, device))
    torch.cuda.synchronize()
    want = packed_layout_numpy(bits, 2)
    assert capi.lib().vecops_hip_packed_b_bytes(capi.BF16, n, k) == want.size
    assert np.array_equal(packed.storage.cpu().numpy()[:want.size], want)


@pytest.mark.parametrize("n,k", [(16, 64), (19, 67), (23, 71), (31, 79), (300, 1000)])
def test_pack_b_i8_layout_strided_source(device, n, k):
    import torch
    from vecops_amd import capi
    b = synth.int8_sym(8, (n, k))
    # K-contiguous with a padded row stride, and the transposed ([K,N] row-major) source
    padded = torch.full((n, k + 3), -99, dtype=torch.int8, device=device)
    padded[:, :k] = torch.from_numpy(b).to(device)
    want = packed_layout_numpy(b, 1)
    for source in (padded[:, :k], torch.from_numpy(np.ascontiguousarray(b.T)).to(device).t()):
        packed = capi.pack_b(source)
        torch.cuda.synchronize()
        assert np.array_equal(packed.storage.cpu().numpy()[:want.size], want)


def test_pack_b_f32_source_rounds_to_bf16(device, oracle):
    import torch
    from vecops_amd import capi
    n, k = 37, 131
    b = synth.uniform_pm1(9, (n, k))
    packed = capi.pack_b(torch.from_numpy(b).to(device))
    torch.cuda.synchronize()
    want = packed_layout_numpy(oracle.bf16_from_f32(b), 2)
    assert packed.dtype == capi.BF16
    assert np.array_equal(packed.storage.cpu().numpy()[:want.size], want)


PACKED_SHAPES = [(16, 16, 35), (37, 51, 79), (1, 128, 65), (512, 1, 256), (257, 255, 65), (300, 520, 1000),
                 (129, 129, 129), (64, 64, 8), (1024, 1024, 1024), (2048, 2048, 512), (16, 4096, 4096),
                 (1000, 130, 2048), (512, 768, 4096 + 64)]


@pytest.mark.parametrize("m,n,k", PACKED_SHAPES)
def test_packed_bf16_matmul(device, oracle, m, n, k):
    import torch
    from vecops_amd import capi
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    da, db = dev_bf16(a, device), dev_bf16(b, device)
    packed = capi.pack_b(db)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul_packed_b(da, packed, c)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, acc_f64=True)
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)
    # bf16 output = RNE of the fp32 output of the same kernel
    c16 = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    capi.matmul_packed_b(da, packed, c16)
    torch.cuda.synchronize()
    assert np.array_equal(host_bits(c16), oracle.bf16_from_f32(c.cpu().numpy()))


@pytest.mark.parametrize("m,n,k", [(19, 21, 69), (1, 128, 65), (128, 1, 65), (35, 53, 257), (256, 256, 128),
                                   (300, 520, 1000), (1024, 768, 4096), (130, 140, 515), (16, 64, 8191)])
def test_packed_int8_matmul_bit_exact(device, oracle, m, n, k):
    import torch
    from vecops_amd import capi
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    packed = capi.pack_b(torch.from_numpy(b).to(device))
    c = torch.full((m, n), -1, dtype=torch.int32, device=device)
    capi.matmul_packed_b(torch.from_numpy(a).to(device), packed, c)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy(), oracle.matmul_i8_dense(a, b))


@pytest.mark.parametrize("m,n,k", [(19, 21, 69), (1, 128, 65), (35, 53, 257), (256, 256, 128), (300, 520, 1000),
                                   (1024, 768, 4096), (64, 48, 8191), (2, 33, 262145)])
def test_packed_int8_b_with_unsigned_a_bit_exact(device, oracle, m, n, k):
    """uint8 activations against int8-packed weights (the atom AMX_I8I32<uint8_t, int8_t> that
    ops::matmul_pack_b_compensated exists for): a is staged as a - 128 and 128 * sum_k b[n,k], summed from the
    packed rows, is added back; every int32 equals the exact integer sum mod 2^32 (tile, split-K, ragged shapes,
    and a K long enough for the sums of 255 * 127 to wrap)."""
    import torch
    from vecops_amd import capi
    a = (synth.draws(1, m * k) % np.uint64(256)).astype(np.uint8).reshape(m, k)
    b = synth.int8_sym(2, (n, k))
    if k > 100000:
        a[0], b[0] = 255, 127                                   # 262145 * 255 * 127 > 2^31
    packed = capi.pack_b(torch.from_numpy(b).to(device))
    c = torch.full((m, n), -1, dtype=torch.int32, device=device)
    capi.matmul_packed_b(torch.from_numpy(a).to(device), packed, c)
    torch.cuda.synchronize()
    exact = a.astype(np.int64) @ b.astype(np.int64).T
    assert np.array_equal(c.cpu().numpy(), (exact & 0xffffffff).astype(np.uint32).view(np.int32))
    if k < 100000:
        want = np.zeros((m, n), np.int32)
        oracle.matmul(a, b, want, atom=2)
        assert np.array_equal(c.cpu().numpy(), want)


def test_packed_int8_b_with_unsigned_a_batched(device):
    """One packed operand for every batch of a rank-3 uint8 a, with an int32 C input."""
    import torch
    from vecops_amd import capi
    batch, m, n, k = 3, 70, 200, 300
    a = (synth.draws(1, batch * m * k) % np.uint64(256)).astype(np.uint8).reshape(batch, m, k)
    b = synth.int8_sym(2, (n, k))
    cin = ((synth.draws(3, batch * m * n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32).reshape(batch, m, n)
    packed = capi.pack_b(torch.from_numpy(b).to(device))
    c = torch.full((batch, m, n), -1, dtype=torch.int32, device=device)
    capi.matmul_packed_b(torch.from_numpy(a).to(device), packed, c, c_in=torch.from_numpy(cin).to(device))
    torch.cuda.synchronize()
    want = np.einsum("bmk,nk->bmn", a.astype(np.int64), b.astype(np.int64)) + cin
    assert np.array_equal(c.cpu().numpy(), want.astype(np.int32))


@pytest.mark.parametrize("m,n,k,corr", [(67, 129, 515, True), (256, 384, 1024, False), (300, 1000, 2048, True),
                                        (1, 300, 4096, False)])
def test_packed_int8_dequant_bit_exact(device, oracle, m, n, k, corr):
    import torch
    from vecops_amd import capi
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    correction = ((synth.draws(5, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32) if corr else None
    packed = capi.pack_b(torch.from_numpy(b).to(device))
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    capi.matmul_i8_dequant_packed_b(torch.from_numpy(a).to(device), packed, torch.from_numpy(rs).to(device),
                                    torch.from_numpy(cs).to(device), c,
                                    correction=torch.from_numpy(correction).to(device) if corr else None)
    torch.cuda.synchronize()
    want = oracle.matmul_i8_dequant(a, b, rs, cs, correction)
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_packed_fp32_a_batched_cin_and_strides(device, oracle):
    """fp32 A (rounded to bf16 like the plain path) of rank 3 with padded rows, one packed B for
    every batch, an explicit bf16 C input and a C with padded rows."""
    import torch
    from vecops_amd import capi
    batch, m, n, k = 3, 70, 200, 333
    a = synth.uniform_pm1(1, (batch, m, k))
    b = synth.uniform_pm1(2, (n, k))
    cin = synth.bf16_round(synth.uniform_pm1(3, (batch, m, n)))
    a_dev = torch.zeros((batch, m, k + 5), dtype=torch.float32, device=device)
    a_dev[:, :, :k] = torch.from_numpy(a).to(device)
    c_store = torch.full((batch, m, n + 8), float("nan"), dtype=torch.float32, device=device)
    c = c_store[:, :, :n]
    packed = capi.pack_b(torch.from_numpy(b).to(device))
    capi.matmul_packed_b(a_dev[:, :, :k], packed, c, c_in=dev_bf16(cin, device))
    torch.cuda.synchronize()
    got = c.cpu().numpy()
    b3 = np.broadcast_to(b, (batch, n, k))
    want = np.zeros((batch, m, n), np.float32)
    oracle.matmul(a, np.ascontiguousarray(b3), want, cin=cin, atom=O.ATOM_BF16F32, acc_f64=True)
    assert rel_err(got, want) <= fp32_tol(k)
    assert torch.isnan(c_store[:, :, n:]).all()
    # identical, bit for bit, to the plain path on the unpacked operand on the 256 x 256 tiles (the packed kernel's
    # MFMA shape and order of sums)
    c_plain = torch.empty((batch, m, n), dtype=torch.float32, device=device)
    capi.matmul_family(a_dev[:, :, :k], torch.from_numpy(np.ascontiguousarray(b3)).to(device), c_plain,
                       capi.family_request("tile_256", split_k=capi.plan_matmul_packed_b(a_dev[:, :, :k], packed, c).split_k),
                       c_in=dev_bf16(cin, device))
    torch.cuda.synchronize()
    assert np.array_equal(got, c_plain.cpu().numpy())


def test_packed_full_size_bf16_sampled(device, oracle):
    """4096^3 (the headline shape): sampled rows and columns against the oracle, and the whole
    result against the plain tile kernel on the unpacked operand."""
    import torch
    from vecops_amd import capi
    m = n = k = 4096
    a = synth.bf16_round(synth.normal(11, (m, k)))
    b = synth.bf16_round(synth.normal(12, (n, k)))
    da, db = dev_bf16(a, device), dev_bf16(b, device)
    packed = capi.pack_b(db)
    c = torch.empty((m, n), dtype=torch.float32, device=device)
    capi.matmul_packed_b(da, packed, c)
    c_plain = torch.empty((m, n), dtype=torch.float32, device=device)
    capi.matmul(da, db, c_plain)
    torch.cuda.synchronize()
    rows = np.array([0, 1, 31, 32, 255, 256, 1000, 2047, 2048, 4095])
    cols = np.array([0, 7, 31, 32, 33, 255, 256, 3000, 4064, 4095])
    rr, cc = (x.reshape(-1) for x in np.meshgrid(rows, cols, indexing="ij"))
    want = oracle.matmul_sampled(a, b, rr, cc)
    got = c.cpu().numpy()
    assert rel_err(got[rr, cc], want) <= fp32_tol(k)
    # (the plain kernel's 256 x 256 tile of aligned bf16 operands sums 32 k per matrix instruction, the packed kernel
    # 16: the two agree up to the order of the fp32 sums)
    assert rel_err(got, c_plain.cpu().numpy()) <= fp32_tol(k)


def test_pack_b_compensated_reference_case(device):
    """tests/ops/MatmulPackTest.cpp:354-377: N=33, K=129, row stride K+3, zero point 3."""
    import torch
    from vecops_amd import capi
    n, k, zp = 33, 129, 3
    nn, kk = np.meshgrid(np.arange(n), np.arange(k), indexing="ij")
    logical = ((nn * 17 + kk * 3) % 61 - 30).astype(np.int8)
    store = torch.full((n, k + 3), -99, dtype=torch.int8, device=device)
    store[:, :k] = torch.from_numpy(logical).to(device)
    packed, comp = capi.pack_b(store[:, :k], a_zero_point=zp)
    torch.cuda.synchronize()
    want = packed_layout_numpy(logical, 1)
    assert np.array_equal(packed.storage.cpu().numpy()[:want.size], want)
    assert np.array_equal(comp.cpu().numpy(), (-zp * logical.astype(np.int64).sum(axis=1)).astype(np.int32))
    # used as the stride-0 C input of a u8 x s8 product it removes A's zero point:
    # sum_k (ua - zp) * b = sum_k ua * b + comp
    m = 21
    ua = (synth.draws(4, m * k) % np.uint64(256)).astype(np.uint8).reshape(m, k)
    c = torch.empty((m, n), dtype=torch.int32, device=device)
    cin = comp.view(1, n).expand(m, n)
    capi.matmul(torch.from_numpy(ua).to(device), store[:, :k], c, c_in=cin)
    torch.cuda.synchronize()
    want_c = (ua.astype(np.int64) - zp) @ logical.astype(np.int64).T
    assert np.array_equal(c.cpu().numpy(), want_c.astype(np.int32))
    # and the same against the packed operand itself: AMX_I8I32<uint8_t, int8_t> with a packed B and its
    # sidecar (ops/MatmulPack.h:52-58)
    c2 = torch.full((m, n), -1, dtype=torch.int32, device=device)
    capi.matmul_packed_b(torch.from_numpy(ua).to(device), packed, c2, c_in=cin)
    torch.cuda.synchronize()
    assert np.array_equal(c2.cpu().numpy(), want_c.astype(np.int32))


def test_packed_zero_extents_and_rejections(device):
    """tests/ops/MatmulPackTest.cpp:401-459: zero K writes a zero compensation, zero N writes nothing."""
    import torch
    from vecops_amd import capi
    b = torch.empty((17, 0), dtype=torch.int8, device=device)
    packed, comp = capi.pack_b(b, a_zero_point=3)
    torch.cuda.synchronize()
    assert capi.lib().vecops_hip_packed_b_bytes(capi.I8, 17, 0) == 0
    assert (comp == 0).all()
    # K == 0: C = C_in (or zeros)
    a = torch.empty((5, 0), dtype=torch.int8, device=device)
    c = torch.full((5, 17), -1, dtype=torch.int32, device=device)
    capi.matmul_packed_b(a, packed, c)
    torch.cuda.synchronize()
    assert (c == 0).all()
    # N == 0: nothing to do
    empty = capi.pack_b(torch.empty((0, 67), dtype=torch.int8, device=device))
    capi.matmul_packed_b(torch.zeros((5, 67), dtype=torch.int8, device=device), empty,
                         torch.empty((5, 0), dtype=torch.int32, device=device))
    # mismatched operand classes and a short buffer are refused
    pb = capi.pack_b(torch.zeros((8, 64), dtype=torch.bfloat16, device=device))
    with pytest.raises(capi.VecopsHipError) as err:
        capi.matmul_packed_b(torch.zeros((4, 64), dtype=torch.int8, device=device), pb,
                             torch.empty((4, 8), dtype=torch.int32, device=device))
    assert err.value.code == 2
    ob = capi.operand(torch.zeros((40, 64), dtype=torch.int8, device=device))
    import ctypes as C
    rc = capi.lib().vecops_hip_pack_b(C.byref(ob), packed.storage.data_ptr(), 16, None)
    assert rc == 1
    with pytest.raises(capi.VecopsHipError) as err:        # 32-bit integers have no packed form
        capi.pack_b(torch.zeros((4, 8), dtype=torch.int32, device=device))
    assert err.value.code == 2
