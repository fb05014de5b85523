"""The four-stage 128 x 128 kernel (tile_gemm_deep128.hip): what the library runs when a product gives a compute unit at
most one 128 x 128 workgroup (256 workgroups or fewer, operands aligned and K-contiguous - or, 16-bit ones, B handed
over as [K,N] -, K in whole K tiles).
Checked against the oracle, against exact integer sums, and against the two-stage kernel of the same tile - which a
K that is no whole number of K tiles, or more than 256 workgroups, still selects - on ragged extents, batches, K
splits, C inputs, bf16 outputs and a transposed C."""
import numpy as np
import pytest

from conftest import rel_err
from oracle import oracle as O
from vecops_amd import synth
from test_matmul_gpu import dev_bf16, fp32_tol

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("m,n,k,split", [(1024, 1024, 512, 1), (300, 520, 1024, 1), (513, 257, 576, 3), (128, 128, 512, 1),
                                         (1000, 2000, 640, 1), (700, 900, 2048, 2), (1, 129, 512, 1), (2000, 2048, 512, 1)])
def test_deep_kernel_bf16_against_the_oracle(device, oracle, m, n, k, split):
    import torch
    from vecops_amd import capi
    a_bits, b_bits = synth.bf16_round(synth.uniform_pm1(1, (m, k))), synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    a, b = dev_bf16(a_bits, device), dev_bf16(b_bits, device)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    request = capi.family_request("tile_128", capi.SELECT_REQUIRE, split_k=split)
    capi.matmul_family(a, b, c, request)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a_bits, b_bits, want, acc_f64=True, c_bf16=False)
    assert rel_err(c.cpu().numpy(), want) <= fp32_tol(k)


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("m,n,k,split", [(1024, 1024, 512, 1), (300, 520, 1024, 1), (513, 264, 576, 3), (128, 128, 512, 1),
                                         (1000, 2000, 640, 1), (700, 904, 2048, 2), (1, 136, 512, 1), (100, 8, 512, 1),
                                         (2000, 2048, 512, 1)])
def test_deep_kernel_b_as_k_by_n(device, oracle, kind, m, n, k, split):
    """B stored [K,N] and handed over as the strided [N,K] view (N a multiple of eight: the rows are 16-byte aligned):
    the tile lies [k][n] in LDS and the fragment reads transpose.  bf16 against the oracle, f16 against float64 sums of
    the same operands."""
    import torch
    from vecops_amd import capi
    request = capi.family_request("tile_128", capi.SELECT_REQUIRE, split_k=split)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    if kind == "bf16":
        a_bits, b_bits = synth.bf16_round(synth.uniform_pm1(1, (m, k))), synth.bf16_round(synth.uniform_pm1(2, (k, n)))
        a, b = dev_bf16(a_bits, device), dev_bf16(b_bits, device)
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


@pytest.mark.parametrize("m,n,k,split", [(1024, 4096, 4096, 1), (300, 520, 1024, 1), (513, 257, 1152, 3), (768, 4096, 4096, 1),
                                         (96, 100, 262144, 1)])
def test_deep_kernel_int8_exact(device, m, n, k, split):
    """Exact int32 sums (a K long enough to wrap among them), equal bit for bit to every other family's."""
    import torch
    from vecops_amd import capi
    raw = lambda seed, shape: (synth.draws(seed, int(np.prod(shape))) % np.uint64(256)).astype(np.uint8).reshape(shape).view(np.int8)  # noqa: E731
    a, b = raw(1, (m, k)), raw(2, (n, k))
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    c = torch.full((m, n), -1, dtype=torch.int32, device=device)
    capi.matmul_family(ta, tb, c, capi.family_request("tile_128", capi.SELECT_REQUIRE, split_k=split))
    other = torch.full((m, n), -1, dtype=torch.int32, device=device)
    capi.matmul_family(ta, tb, other, capi.family_request("tile_64", capi.SELECT_REQUIRE, split_k=1))
    torch.cuda.synchronize()
    assert torch.equal(c, other)
    rows = np.arange(0, m, max(1, m // 16))
    want = (a[rows].astype(np.int64) @ b.astype(np.int64).T & 0xffffffff).astype(np.uint32).view(np.int32)
    assert np.array_equal(c.cpu().numpy()[rows], want)


@pytest.mark.parametrize("kind", ["bf16", "f16", "i8"])
@pytest.mark.parametrize("m,n,k", [(1024, 4096, 1024), (300, 520, 1024), (513, 257, 1152), (128, 100, 512), (256, 4096, 4096),
                                   (2, 640, 2048)])
def test_deep_kernel_prepacked_b(device, kind, m, n, k):
    """B packed by vecops_hip_pack_b: the pack keeps its order in LDS; the product equals the plain operand's bit for
    bit (the same kernel's loop on the same K order; integer sums in any case), K splits of the plan included."""
    import torch
    from vecops_amd import capi
    gen = torch.Generator().manual_seed(m + n + k)
    if kind == "i8":
        a = torch.randint(-128, 128, (m, k), generator=gen, dtype=torch.int8).to(device)
        b = torch.randint(-128, 128, (n, k), generator=gen, dtype=torch.int8).to(device)
        c = torch.full((m, n), -1, dtype=torch.int32, device=device)
    else:
        dtype = torch.bfloat16 if kind == "bf16" else torch.float16
        a = (torch.rand((m, k), generator=gen) * 2 - 1).to(dtype).to(device)
        b = (torch.rand((n, k), generator=gen) * 2 - 1).to(dtype).to(device)
        c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    packed = capi.pack_b(b)
    plan = capi.plan_matmul_packed_b(a, packed, c)
    if m * n >= 128 * 128 * 96:
        assert capi.FAMILY_NAMES[plan.family] == "tile_128"          # 96 to 256 tiles: whole, on the four-stage kernel
    capi.matmul_packed_b(a, packed, c)
    plain = torch.empty_like(c)
    capi.matmul_family(a, b, plain, capi.family_request("tile_128", capi.SELECT_REQUIRE, split_k=max(int(plan.split_k), 1)))
    torch.cuda.synchronize()
    if kind == "i8" or capi.FAMILY_NAMES[plan.family] == "tile_128":
        assert torch.equal(c, plain)
    want = a.double() @ b.double().t()
    if kind == "i8":
        assert torch.equal(c.to(torch.int64), want.to(torch.int64))
    else:
        assert rel_err(c.double().cpu().numpy(), want.cpu().numpy()) <= fp32_tol(k)


def test_deep_kernel_batches_cin_bf16_out_transposed_c(device, oracle):
    import torch
    from vecops_amd import capi
    batch, m, n, k = 3, 200, 330, 768
    a_bits = synth.bf16_round(synth.uniform_pm1(1, (batch, m, k)))
    b_bits = synth.bf16_round(synth.uniform_pm1(2, (batch, n, k)))
    cin_bits = synth.bf16_round(synth.uniform_pm1(3, (batch, m, n)))
    a, b, cin = dev_bf16(a_bits, device), dev_bf16(b_bits, device), dev_bf16(cin_bits, device)
    store = torch.full((batch, n, m), float("nan"), dtype=torch.bfloat16, device=device)
    c = store.transpose(1, 2)
    plan = capi.plan_matmul(a, b, c, c_in=cin)
    assert capi.FAMILY_NAMES[plan.family] in ("tile_128", "tile_64")
    capi.matmul_family(a, b, c, capi.family_request("tile_128", capi.SELECT_REQUIRE, split_k=1), c_in=cin)
    torch.cuda.synchronize()
    want = np.zeros((batch, m, n), np.uint16)
    for i in range(batch):
        oracle.matmul(a_bits[i], b_bits[i], want[i], cin=cin_bits[i], acc_f64=True)
    got = c.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    f = lambda bits: (bits.astype(np.uint32) << 16).view(np.float32)  # noqa: E731
    assert rel_err(f(got), f(want)) <= 2.0 ** -7


def test_the_table_plans_one_workgroup_per_unit(device):
    """1024 x 4096 x 4096 and its neighbours: the plan is the unsplit 128 x 128 tile, and it equals the two-stage kernel's
    result (which a K of one element more, padded operands apart, selects) up to the order of the fp32 sums."""
    import torch
    from vecops_amd import capi
    for (m, n, k), b_as_kn in (((1024, 4096, 4096), False), ((768, 4096, 4096), False), ((512, 4096, 4096), False),
                               ((2048, 2048, 2048), False), ((1024, 4096, 4096), True), ((512, 4096, 4096), True)):
        a_bits = synth.bf16_round(synth.normal(1, (m, k), 0.02))
        b_bits = synth.bf16_round(synth.normal(2, (k, n) if b_as_kn else (n, k), 0.02))
        a, b = dev_bf16(a_bits, device), dev_bf16(b_bits, device)
        b = b.t() if b_as_kn else b
        c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
        plan = capi.plan_matmul(a, b, c)
        assert capi.FAMILY_NAMES[plan.family] == "tile_128" and plan.split_k == 1 and plan.workspace_bytes == 0
        capi.matmul(a, b, c)
        big = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
        capi.matmul_family(a, b, big, capi.family_request("tile_256", capi.SELECT_REQUIRE, split_k=1))
        torch.cuda.synchronize()
        scale = float(big.abs().max())
        assert float((c - big).abs().max()) <= scale * fp32_tol(k)
