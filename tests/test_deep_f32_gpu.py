"""fp32 compute on the ring-of-stages kernel (tile_gemm_deep_f32.hip): what the library runs for fp32 products of at
most one 64 x 64 or 128 x 128 workgroup per compute unit (256 workgroups or fewer, aligned operands, B K-contiguous or
[K,N] with N a multiple of four, K in whole K tiles of 32).  Against the oracle's fp32 atom, and against the two-stage
kernel of another tile family, whose sums it repeats bit for bit (the same matrix instructions in the same order)."""
import numpy as np
import pytest

from conftest import rel_err
from oracle import oracle as O  # noqa: F401
from vecops_amd import synth
from test_matmul_gpu import fp32_compute_tol, host_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("b_as_kn", [True, False])
@pytest.mark.parametrize("m,n,k,family,split,batch", [(1024, 1024, 1024, "tile_64", 1, 1), (300, 520, 512, "tile_64", 1, 1),
                                                      (513, 260, 576, "tile_128", 3, 1), (1000, 2000, 512, "tile_128", 1, 1),
                                                      (64, 64, 256, "tile_64", 1, 1), (1, 132, 512, "tile_64", 1, 1),
                                                      (100, 4, 256, "tile_64", 1, 1), (200, 300, 768, "tile_64", 1, 3),
                                                      (700, 900, 2048, "tile_128", 2, 1)])
def test_ring_kernel_against_the_oracle(device, oracle, m, n, k, family, split, batch, b_as_kn):
    import torch
    from vecops_amd import capi
    a = synth.uniform_pm1(1, (batch, m, k))
    b = synth.uniform_pm1(2, (batch, n, k))
    ta = torch.from_numpy(a).to(device)
    tb = (torch.from_numpy(np.ascontiguousarray(b.transpose(0, 2, 1))).to(device).transpose(1, 2) if b_as_kn
          else torch.from_numpy(b).to(device))
    c = torch.full((batch, m, n), float("nan"), dtype=torch.float32, device=device)
    other = torch.full((batch, m, n), float("nan"), dtype=torch.float32, device=device)
    if batch == 1:
        ta, tb, c, other = ta[0], tb[0], c[0], other[0]
    capi.matmul_family(ta, tb, c, capi.family_request(family, capi.SELECT_REQUIRE, split_k=split), compute=capi.COMPUTE_F32)
    capi.matmul_family(ta, tb, other, capi.family_request("tile_256", capi.SELECT_REQUIRE, split_k=1), compute=capi.COMPUTE_F32)
    torch.cuda.synchronize()
    got = c.cpu().numpy().reshape(batch, m, n)
    for i in range(batch):
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a[i], b[i], want, atom=1, acc_f64=True)
        assert rel_err(got[i], want) <= fp32_compute_tol(k)
    if split == 1:
        assert torch.equal(c, other)        # k summed in the same order by the same instructions


def test_ring_kernel_c_input_and_bf16_output(device, oracle):
    import torch
    from vecops_amd import capi
    m, n, k = 520, 1024, 1024
    a, b, cin = synth.uniform_pm1(1, (m, k)), synth.uniform_pm1(2, (k, n)), synth.uniform_pm1(3, (m, n))
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device).t()
    plan = capi.plan_matmul(ta, tb, torch.empty((m, n), dtype=torch.float32, device=device), compute=capi.COMPUTE_F32)
    assert capi.FAMILY_NAMES[plan.family] == "tile_64" and plan.split_k == 1     # 9 x 16 tiles: one workgroup per unit at most
    c16 = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    capi.matmul(ta, tb, c16, c_in=torch.from_numpy(cin).to(device), compute=capi.COMPUTE_F32)
    torch.cuda.synchronize()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, np.ascontiguousarray(b.T), want, atom=1, acc_f64=True)
    assert rel_err(synth.bf16_to_f32(host_bits(c16)), want + cin) <= 2.0 ** -8


def test_fp32_compute_prefers_small_tiles_on_a_part_filled_round(device):
    """1536^3 in fp32: 144 tiles of 128 x 128 leave 112 compute units idle; 576 of 64 x 64 give every unit two or three."""
    import torch
    from vecops_amd import capi
    a = torch.zeros((1536, 1536), dtype=torch.float32, device=device)
    c = torch.empty((1536, 1536), dtype=torch.float32, device=device)
    assert capi.FAMILY_NAMES[capi.plan_matmul(a, a, c, compute=capi.COMPUTE_F32).family] == "tile_64"
    big = torch.zeros((2048, 2048), dtype=torch.float32, device=device)
    assert capi.FAMILY_NAMES[capi.plan_matmul(big, big, torch.empty_like(big), compute=capi.COMPUTE_F32).family] == "tile_128"
    assert capi.FAMILY_NAMES[capi.plan_matmul(a.bfloat16(), a.bfloat16(), c).family] != "tile_64"   # the 16-bit classes keep their rules
