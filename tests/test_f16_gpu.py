"""IEEE half operands (vecops' AMX_F16F32 / SME_F16F32 atoms, matmul/details/kernel/amx/Atoms.h:62-71) on
the GPU against the oracle's F16 atom.  The reference's own build of this atom needs AMX-FP16, which the
build host lacks, so the oracle side is pinned by closed forms only (tests/test_oracle.py): half products
are exact in fp32, the sums are compared with the bound used for bf16 (summation order), a half output
within one half ulp."""
import numpy as np
import pytest

from conftest import rel_err
from oracle import oracle as O
from vecops_amd import synth

pytestmark = pytest.mark.gpu


def _half(seed, shape):
    return synth.uniform_pm1(seed, shape).astype(np.float16)


def _dev(x, device):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).to(device)


SHAPES = [(256, 512, 256), (300, 260, 1000), (37, 51, 79), (2457, 1221, 72), (255, 63, 8191), (1, 4097, 129)]


@pytest.mark.parametrize("m,n,k", SHAPES, ids=["x".join(map(str, s)) for s in SHAPES])
@pytest.mark.parametrize("out", ["f32", "f16"])
def test_f16_matmul_against_oracle(device, oracle, m, n, k, out):
    import torch
    from vecops_amd import capi
    a, b = _half(1, (m, k)), _half(2, (n, k))
    want = np.zeros((m, n), np.float32 if out == "f32" else np.float16)
    oracle.matmul(a, b, want, atom=O.ATOM_F16F32, acc_f64=True)
    c = torch.full((m, n), float("nan"), dtype=torch.float32 if out == "f32" else torch.float16, device=device)
    capi.matmul(_dev(a, device), _dev(b, device), c)
    torch.cuda.synchronize()
    got = c.cpu().numpy()
    if out == "f32":
        assert rel_err(got, want) <= 2e-6 * max(1.0, k / 32)
    else:
        assert rel_err(got.astype(np.float32), want.astype(np.float32)) <= 2.0 ** -10
        assert (got.view(np.uint16) != want.view(np.uint16)).mean() < 0.02


def test_f16_layouts_c_input_and_batches(device, oracle):
    import torch
    from vecops_amd import capi
    m, n, k, batch = 130, 264, 200, 3
    a, b = _half(1, (batch, m, k)), _half(2, (batch, n, k))
    cin = _half(3, (batch, m, n))
    want = np.zeros((batch, m, n), np.float16)
    oracle.matmul(a, b, want, cin=cin, atom=O.ATOM_F16F32, acc_f64=True)
    ta, tb, tcin = _dev(a, device), _dev(b, device), _dev(cin, device)
    c = torch.zeros((batch, m, n), dtype=torch.float16, device=device)
    capi.matmul(ta, tb, c, c_in=tcin)
    assert rel_err(c.cpu().numpy().astype(np.float32), want.astype(np.float32)) <= 2.0 ** -10
    # B handed over as [K,N] row-major (strides (1, N)); the C-input aliases the output
    b_kn = tb.transpose(1, 2).contiguous().transpose(1, 2)
    assert b_kn.stride() == (k * n, 1, n)
    acc = tcin.clone()
    capi.matmul(ta, b_kn, acc, c_in=acc)
    assert rel_err(acc.cpu().numpy().astype(np.float32), want.astype(np.float32)) <= 2.0 ** -10
    # fp32 C-input and output, shared B (the batch is folded into one product)
    want32 = np.zeros((batch, m, n), np.float32)
    cin32 = synth.uniform_pm1(4, (batch, m, n))
    oracle.matmul(a, np.broadcast_to(b[0], (batch, n, k)), want32, cin=cin32, atom=O.ATOM_F16F32, acc_f64=True)
    c32 = torch.zeros((batch, m, n), device=device)
    capi.matmul(ta, tb[0].unsqueeze(0).expand(batch, n, k), c32, c_in=_dev(cin32, device))
    assert rel_err(c32.cpu().numpy(), want32) <= 2e-6 * max(1.0, k / 32)


def test_f16_fused_and_dtype_rules(device, oracle):
    import torch
    from vecops_amd import capi
    m, n, k = 67, 136, 96
    a, b = _half(1, (m, k)), _half(2, (n, k))
    bias = synth.uniform_pm1(3, (n,))
    acc = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, acc, cin=np.broadcast_to(bias, (m, n)), atom=O.ATOM_F16F32, acc_f64=True)
    want = oracle.fused_outputs(acc, np.float32, activation=1, scale=0.5)
    c = torch.zeros((m, n), device=device)
    capi.matmul_fused(_dev(a, device), _dev(b, device), c, capi.epilogue(activation="relu", scale=0.5),
                      c_in=_dev(bias, device).reshape(1, n).expand(m, n))
    assert rel_err(c.cpu().numpy(), want) <= 2e-6 * max(1.0, k / 32)
    with pytest.raises(capi.VecopsHipError) as info:          # half operands do not write bf16
        capi.matmul(_dev(a, device), _dev(b, device), torch.zeros((m, n), dtype=torch.bfloat16, device=device))
    assert info.value.code == 2
    with pytest.raises(capi.VecopsHipError) as info:          # nor mix with bf16 operands
        capi.matmul(_dev(a, device), torch.zeros((n, k), dtype=torch.bfloat16, device=device), c)
    assert info.value.code == 2


@pytest.mark.parametrize("narrow,wide,k", [(1, 14336, 4096), (4, 4096, 1024), (16, 2048, 4096), (3, 600, 136)])
@pytest.mark.parametrize("out", ["f32", "f16"])
def test_f16_skinny_family(device, oracle, narrow, wide, k, out):
    """Half operands on the skinny kernels (v_mfma_f32_16x16x32_f16), either operand the narrow one."""
    import torch
    from vecops_amd import capi
    for m, n in ((narrow, wide), (wide, narrow)):
        a, b = _half(1, (m, k)), _half(2, (n, k))
        ta, tb = _dev(a, device), _dev(b, device)
        c = torch.full((m, n), float("nan"), dtype=torch.float32 if out == "f32" else torch.float16, device=device)
        assert capi.FAMILY_NAMES[capi.plan_matmul(ta, tb, c).family] == "skinny"
        capi.matmul(ta, tb, c)
        torch.cuda.synchronize()
        want = np.zeros((m, n), np.float32 if out == "f32" else np.float16)
        oracle.matmul(a, b, want, atom=O.ATOM_F16F32, acc_f64=True)
        got = c.cpu().numpy()
        if out == "f32":
            assert rel_err(got, want) <= 2e-6 * max(1.0, k / 32)
        else:
            assert rel_err(got.astype(np.float32), want.astype(np.float32)) <= 2.0 ** -10


@pytest.mark.parametrize("m,n,k", [(300, 260, 1000), (37, 51, 79), (512, 768, 512), (2, 3, 64, 40, 200)][:3] + [(2457, 1221, 72)])
def test_f16_prepacked_b(device, oracle, m, n, k):
    """Half weights packed once (the 16-bit permutation of the bf16 pack): equal to the plain product on the 256 x 256
    tiles up to the order of the fp32 sums (the packed kernel multiplies on v_mfma_f32_32x32x16_f16, the plain tile of
    aligned operands on v_mfma_f32_16x16x32_f16: 16 against 32 k per instruction)."""
    import torch
    from vecops_amd import capi
    a, b = _half(1, (m, k)), _half(2, (n, k))
    ta, tb = _dev(a, device), _dev(b, device)
    packed = capi.pack_b(tb)
    assert packed.dtype == capi.F16
    for dt in (torch.float32, torch.float16):
        c, ref = (torch.full((m, n), float("nan"), dtype=dt, device=device) for _ in range(2))
        capi.matmul_packed_b(ta, packed, c)
        split_k = capi.plan_matmul_packed_b(ta, packed, c).split_k          # the same partition of K
        capi.matmul_family(ta, tb, ref, capi.family_request("tile_256", split_k=split_k))
        torch.cuda.synchronize()
        tol = 2e-6 * max(1.0, k / 32) if dt == torch.float32 else 2.0 ** -10
        assert rel_err(c.float().cpu().numpy(), ref.float().cpu().numpy()) <= tol
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, atom=O.ATOM_F16F32, acc_f64=True)
    c = torch.empty((m, n), device=device)
    capi.matmul_packed_b(ta, packed, c)
    assert rel_err(c.cpu().numpy(), want) <= 2e-6 * max(1.0, k / 32)
    with pytest.raises(capi.VecopsHipError):                 # a bf16 a against f16-packed weights
        capi.matmul_packed_b(ta.to(torch.bfloat16), packed, c)
