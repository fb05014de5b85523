"""Packing of either operand and of both (vecops' ops::matmul_pack with Operand::A / Operand::B,
tests/ops/MatmulMixedPackingTest.cpp: every atom supports either packed operand and both), and packed operands of
every signedness (AMX_I8I32<A, B> with A, B in {int8, uint8}, :131-153), through the C ABI.  Packing is a permutation,
so integer results are exact and floating ones equal the plain product of the same library bit for bit."""
import numpy as np
import pytest

from conftest import rel_err
from vecops_amd import synth
from test_matmul_gpu import dev_bf16, fp32_tol, host_bits
from test_packed_gpu import packed_layout_numpy

pytestmark = pytest.mark.gpu


def conversion_value(count, seed, unsigned):
    """tests/ops/MatmulConversionTestCommon.h:62-70 for the integral types: the operands of the reference's tests."""
    low = 0 if unsigned else -3
    return (low + (np.arange(count, dtype=np.int64) * 5 + seed) % 7).astype(np.uint8 if unsigned else np.int8)


def bytes_operand(seed, shape, unsigned):
    raw = (synth.draws(seed, int(np.prod(shape))) % np.uint64(256)).astype(np.uint8).reshape(shape)
    return raw if unsigned else raw.view(np.int8)


def exact_i32(a, b):
    return ((a.astype(np.int64) @ b.astype(np.int64).T) & 0xffffffff).astype(np.uint32).view(np.int32)


SIGNS = [(False, False), (False, True), (True, False), (True, True)]


@pytest.mark.parametrize("a_unsigned,b_unsigned", SIGNS)
def test_reference_mixed_packing_case(device, a_unsigned, b_unsigned):
    """The reference's own case (19 x 21 x 65, conversion_value operands) for each signedness: A packed, B packed, both."""
    import torch
    from vecops_amd import capi
    m, n, k = 19, 21, 65
    a = conversion_value(m * k, 3, a_unsigned).reshape(m, k)
    b = conversion_value(n * k, 11, b_unsigned).reshape(n, k)
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    want = exact_i32(a, b)
    pa, pb = capi.pack_a(ta), capi.pack_b(tb)
    for run in (lambda c: capi.matmul_packed_a(pa, tb, c), lambda c: capi.matmul_packed_b(ta, pb, c),
                lambda c: capi.matmul_packed_ab(pa, pb, c)):
        c = torch.full((m, n), -1, dtype=torch.int32, device=device)
        run(c)
        torch.cuda.synchronize()
        assert np.array_equal(c.cpu().numpy(), want)


def test_unsigned_operand_packs_as_its_signed_image(device):
    """A uint8 operand is stored as b - 128 (bytes xor 0x80) in the documented layout, padding zero."""
    import torch
    from vecops_amd import capi
    b = bytes_operand(5, (45, 133), True)
    packed = capi.pack_b(torch.from_numpy(b).to(device))
    assert packed.dtype == capi.U8
    want = packed_layout_numpy((b ^ 0x80).view(np.int8), 1)
    got = packed.storage.cpu().numpy()[:want.size]
    # padding (rows past N, k past K) stays zero, it is not the image of zero
    mask = packed_layout_numpy(np.ones(b.shape, np.int8), 1).astype(bool)
    assert np.array_equal(got[mask], want[mask]) and not got[~mask].any()


@pytest.mark.parametrize("m,n,k", [(35, 53, 257), (256, 256, 128), (300, 520, 1000), (1024, 768, 4096), (2, 33, 262145),
                                   (1, 700, 144)])
@pytest.mark.parametrize("a_unsigned,b_unsigned", [(False, True), (True, True)])
def test_packed_unsigned_b_bit_exact(device, oracle, m, n, k, a_unsigned, b_unsigned):
    """AMX_I8I32<int8_t, uint8_t> and <uint8_t, uint8_t> against a packed B: exact sums mod 2^32 over tile shapes,
    split-K, ragged extents and a K long enough to wrap."""
    import torch
    from vecops_amd import capi
    a, b = bytes_operand(1, (m, k), a_unsigned), bytes_operand(2, (n, k), b_unsigned)
    if k > 100000:
        a[0], b[0] = (255 if a_unsigned else 127), 255
    packed = capi.pack_b(torch.from_numpy(b).to(device))
    c = torch.full((m, n), -1, dtype=torch.int32, device=device)
    capi.matmul_packed_b(torch.from_numpy(a).to(device), packed, c)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy(), exact_i32(a, b))
    if k < 5000:
        want = np.zeros((m, n), np.int32)
        oracle.matmul(a, b, want, atom=2)
        assert np.array_equal(c.cpu().numpy(), want)


@pytest.mark.parametrize("m,n,k", [(19, 21, 69), (128, 1, 65), (300, 520, 1000), (768, 1024, 520), (1000, 16, 4096)])
def test_packed_a_int8_with_c_input_and_batches(device, m, n, k):
    """A packed, int8 / uint8 b of rank 2 and 3 (the one packed a serves every batch), int32 C input."""
    import torch
    from vecops_amd import capi
    for a_unsigned, b_unsigned in SIGNS:
        a, b = bytes_operand(1, (m, k), a_unsigned), bytes_operand(2, (3, n, k), b_unsigned)
        cin = ((synth.draws(3, 3 * m * n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32).reshape(3, m, n)
        pa = capi.pack_a(torch.from_numpy(a).to(device))
        c = torch.full((3, m, n), -1, dtype=torch.int32, device=device)
        capi.matmul_packed_a(pa, torch.from_numpy(b).to(device), c, c_in=torch.from_numpy(cin).to(device))
        c2 = torch.full((m, n), -1, dtype=torch.int32, device=device)
        capi.matmul_packed_a(pa, torch.from_numpy(b[1]).to(device), c2)
        torch.cuda.synchronize()
        want = np.einsum("mk,bnk->bmn", a.astype(np.int64), b.astype(np.int64))
        assert np.array_equal(c.cpu().numpy(), ((want + cin) & 0xffffffff).astype(np.uint32).view(np.int32))
        assert np.array_equal(c2.cpu().numpy(), (want[1] & 0xffffffff).astype(np.uint32).view(np.int32))


@pytest.mark.parametrize("m,n,k", [(19, 21, 65), (300, 520, 1000), (1024, 768, 264), (257, 255, 4096)])
@pytest.mark.parametrize("out", ["f32", "bf16"])
def test_packed_a_and_both_bf16_equal_the_plain_product(device, oracle, m, n, k, out):
    """bf16 (AMX_BF16F32): A packed, and both packed, against the oracle and against the plain product of this
    library - bit for bit where the plain call runs its tile kernels without a K split."""
    import torch
    from vecops_amd import capi
    a, b = synth.bf16_round(synth.uniform_pm1(1, (m, k))), synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    cin = synth.uniform_pm1(3, (m, n)).astype(np.float32)
    ta, tb, tci = dev_bf16(a, device), dev_bf16(b, device), torch.from_numpy(cin).to(device)
    dtype = torch.float32 if out == "f32" else torch.bfloat16
    pa, pb = capi.pack_a(ta), capi.pack_b(tb)
    plain = torch.empty((m, n), dtype=dtype, device=device)
    plan = capi.plan_matmul(ta, tb, plain, c_in=tci)
    capi.matmul(ta, tb, plain, c_in=tci)
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, cin=cin, acc_f64=True)
    for run in (lambda c: capi.matmul_packed_a(pa, tb, c, c_in=tci), lambda c: capi.matmul_packed_ab(pa, pb, c, c_in=tci)):
        c = torch.full((m, n), float("nan"), dtype=dtype, device=device)
        run(c)
        torch.cuda.synchronize()
        got = c.cpu().numpy() if out == "f32" else synth.bf16_to_f32(host_bits(c))
        assert rel_err(got, want) <= fp32_tol(k) + (2.0 ** -8 if out == "bf16" else 0.0)
        if plan.split_k == 1 and capi.FAMILY_NAMES[plan.family] != "skinny" and out == "f32":
            # the same K order per accumulator whichever operand takes which path
            assert rel_err(got, plain.cpu().numpy()) <= fp32_tol(k)


def test_packed_a_f16_and_f32_sources(device, oracle):
    """Half operands (AMX_F16F32) and an fp32 b against a bf16-packed a."""
    import torch
    from vecops_amd import capi
    m, n, k = 130, 200, 264
    a, b = synth.uniform_pm1(1, (m, k)).astype(np.float16), synth.uniform_pm1(2, (n, k)).astype(np.float16)
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    c = torch.full((m, n), float("nan"), device=device)
    capi.matmul_packed_a(capi.pack_a(ta), tb, c)
    cb = torch.full((m, n), float("nan"), device=device)
    capi.matmul_packed_ab(capi.pack_a(ta), capi.pack_b(tb), cb)
    torch.cuda.synchronize()
    want = a.astype(np.float64) @ b.astype(np.float64).T
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k) and rel_err(cb.cpu().numpy(), want) <= fp32_tol(k)
    a16 = synth.bf16_round(synth.uniform_pm1(3, (m, k)))
    b32 = synth.uniform_pm1(4, (n, k)).astype(np.float32)
    c.fill_(float("nan"))
    capi.matmul_packed_a(capi.pack_a(dev_bf16(a16, device)), torch.from_numpy(b32).to(device), c)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a16, synth.bf16_round(b32), want, acc_f64=True)
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)


def test_packed_sides_zero_extents_and_rejections(device):
    import torch
    from vecops_amd import capi
    b = torch.zeros((8, 64), dtype=torch.int8, device=device)
    pa = capi.pack_a(torch.zeros((0, 64), dtype=torch.int8, device=device))
    capi.matmul_packed_a(pa, b, torch.empty((0, 8), dtype=torch.int32, device=device))
    pa0 = capi.pack_a(torch.zeros((4, 0), dtype=torch.int8, device=device))
    c = torch.full((4, 8), 7, dtype=torch.int32, device=device)
    capi.matmul_packed_a(pa0, torch.zeros((8, 0), dtype=torch.int8, device=device), c)
    capi.matmul_packed_ab(pa0, capi.pack_b(torch.zeros((8, 0), dtype=torch.int8, device=device)), c)
    torch.cuda.synchronize()
    assert (c == 0).all()                                            # K == 0: the empty sum
    pa = capi.pack_a(torch.zeros((4, 64), dtype=torch.int8, device=device))
    with pytest.raises(capi.VecopsHipError) as e:                    # an 8-bit packed a needs an 8-bit b
        capi.matmul_packed_a(pa, torch.zeros((8, 64), dtype=torch.bfloat16, device=device),
                             torch.empty((4, 8), dtype=torch.float32, device=device))
    assert e.value.code == 2
    with pytest.raises(capi.VecopsHipError) as e:                    # c must be [M, N]
        capi.matmul_packed_a(pa, b, torch.empty((8, 4), dtype=torch.int32, device=device))
    assert e.value.code == 1
