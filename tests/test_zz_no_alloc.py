"""The entry point that takes no workspace (vecops_hip_matmul_static_workspace): its split-K partial sums and
unsigned-operand terms live in a buffer the library's code object owns on each GPU.  Same kernels as
vecops_hip_matmul, so the results must agree bit for bit - on two calls in a row, the second smaller than the
first (the buffer keeps the first call's contents), and against the oracle."""
import numpy as np
import pytest

from vecops_amd import capi, synth
from conftest import rel_err

pytestmark = pytest.mark.gpu


def _bf16(torch, device, seed, shape):
    bits = synth.bf16_round(synth.uniform_pm1(seed, shape))
    return bits, torch.from_numpy(bits.view(np.int16)).to(device).view(torch.bfloat16)


def test_static_workspace_split_k_twice_in_a_row(device, oracle):
    import torch
    # both shapes are split along K (few output tiles, long K): the partial sums go through the scratch
    for call, (m, n, k) in enumerate([(255, 63, 8191), (100, 40, 4099)]):
        a_bits, a = _bf16(torch, device, 31 + call, (m, k))
        b_bits, b = _bf16(torch, device, 41 + call, (n, k))
        plan = capi.plan_matmul(a, b, torch.empty((m, n), dtype=torch.float32, device=device))
        assert plan.split_k > 1 and 0 < plan.workspace_bytes <= capi.lib().vecops_hip_static_workspace_bytes()
        want = capi.matmul(a, b, torch.empty((m, n), dtype=torch.float32, device=device))
        got = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
        capi.matmul_static_workspace(a, b, got)      # warm-up: the kernels' code and the scratch address are set up once
        torch.cuda.synchronize()
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        # free device memory as the driver sees it (an allocation inside the library would not show in torch's own
        # counter, which is kept as a second check)
        import gc
        gc.collect()     # (tensors of earlier tests must not be freed between the two readings)
        before_driver, before_torch = torch.cuda.mem_get_info(device)[0], torch.cuda.memory_allocated(device)
        capi.matmul_static_workspace(a, b, got)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(device)[0] >= before_driver      # nothing was taken from the device
        assert torch.cuda.memory_allocated(device) <= before_torch
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), f"call {call}: differs from vecops_hip_matmul"
        ref = np.zeros((m, n), np.float32)
        oracle.matmul(a_bits, b_bits, ref, acc_f64=True)
        assert rel_err(got.cpu().numpy(), ref) <= 2e-6 * max(1, k // 32)


def test_static_workspace_unsigned_operands_and_c_input(device, oracle):
    import torch
    from oracle import oracle as O
    # u8 x u8 with split-K: partial sums and both operands' row sums share the scratch; int32, bit-exact
    for call, (m, n, k) in enumerate([(70, 130, 2100), (33, 65, 1029)]):
        a = (synth.draws(51 + call, m * k) % np.uint64(256)).astype(np.uint8).reshape(m, k)
        b = (synth.draws(61 + call, n * k) % np.uint64(256)).astype(np.uint8).reshape(n, k)
        cin = synth.int8_sym(71 + call, (m, n)).astype(np.int32) * 1000
        ta, tb, tc = (torch.from_numpy(x).to(device) for x in (a, b, cin))
        plan = capi.plan_matmul(ta, tb, torch.empty((m, n), dtype=torch.int32, device=device), c_in=tc)
        assert plan.workspace_bytes > 0
        want = capi.matmul(ta, tb, torch.empty((m, n), dtype=torch.int32, device=device), c_in=tc)
        got = torch.zeros((m, n), dtype=torch.int32, device=device)
        capi.matmul_static_workspace(ta, tb, got, c_in=tc)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        ref = np.zeros((m, n), np.int32)
        oracle.matmul(a, b, ref, cin=cin, atom=O.ATOM_I8I32)
        assert np.array_equal(got.cpu().numpy(), ref)


def test_static_workspace_shrinks_a_split_that_does_not_fit(device, oracle):
    """bf16, 64 tiles of 128 x 128 and a long K: vecops_hip_matmul splits K in four (16 MiB of partial sums); this
    entry point runs the product with a split that fits instead of refusing it."""
    import torch
    m, n, k = 512, 2048, 16384
    a, b = synth.bf16_round(synth.uniform_pm1(81, (m, k))), synth.bf16_round(synth.uniform_pm1(82, (n, k)))
    ta = torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
    tb = torch.from_numpy(b.view(np.int16)).to(device).view(torch.bfloat16)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    plan = capi.plan_matmul(ta, tb, c)
    assert plan.workspace_bytes > capi.lib().vecops_hip_static_workspace_bytes()
    capi.matmul_static_workspace(ta, tb, c)
    torch.cuda.synchronize()
    rows = np.arange(0, m, 61)
    want = synth.bf16_to_f32(a[rows]).astype(np.float64) @ synth.bf16_to_f32(b).astype(np.float64).T
    assert rel_err(c.cpu().numpy()[rows], want) <= 2e-6 * max(1, k // 32)


def test_static_workspace_rejects_what_does_not_fit(device):
    import torch
    # the row sums of an unsigned operand take 4 bytes per row: 2.2 M rows do not fit the 8 MiB buffer, and
    # the call is refused before anything is launched
    limit = capi.lib().vecops_hip_static_workspace_bytes()
    assert limit == 8 << 20
    m, n, k = 2_200_000, 8, 16
    a = torch.zeros((m, k), dtype=torch.uint8, device=device)
    b = torch.zeros((n, k), dtype=torch.uint8, device=device)
    c = torch.full((m, n), 7, dtype=torch.int32, device=device)
    assert capi.plan_matmul(a, b, c).workspace_bytes > limit
    with pytest.raises(capi.VecopsHipError) as info:
        capi.matmul_static_workspace(a, b, c)
    assert info.value.code == 2 and "scratch" in str(info.value)
    torch.cuda.synchronize()
    assert int(c.min()) == 7 and int(c.max()) == 7
