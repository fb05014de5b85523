"""fp32 activations quantised on the way in (vecops' RuntimePerRowAsymmetricQuantizeTransform,
matmul/Quantization.h:91-146) through the C ABI: vecops_hip_quantize_rows and the one-call pipeline
vecops_hip_matmul_runtime_quant (tests/ops/MatmulConversionTestCommon.h:1437-1540), bit for bit against the
golden vectors of the real vecops build and against the oracle."""
import os

import numpy as np
import pytest

from golden_cases import (QUANT_BATCHED_CASES, QUANT_CASES, QUANT_EDGE_ZERO_POINTS, make_quant_batched_inputs,
                          make_quant_inputs, quant_batched_by_oracle, quant_edge_inputs)
from oracle import oracle as O
from vecops_amd import synth

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vecops_quant_golden.npz"))


def dev(x, device):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).to(device)


def test_quantize_rows_edge_values_and_double_rounding(device):
    import torch
    from vecops_amd import capi
    a, _, mult = quant_edge_inputs()
    for zp in QUANT_EDGE_ZERO_POINTS:
        q = torch.full(a.shape, 99, dtype=torch.uint8, device=device)
        capi.quantize_rows(dev(a, device), dev(mult, device), zp, q)
        assert np.array_equal(q.cpu().numpy().astype(np.int32), GOLD[f"edge_zp{zp}"]), zp
    fa, fm = GOLD["fma_a"], GOLD["fma_multipliers"]
    q = torch.zeros(fa.shape, dtype=torch.uint8, device=device)
    capi.quantize_rows(dev(fa, device), dev(fm, device), -15, q)
    assert np.array_equal(q.cpu().numpy().astype(np.int32), GOLD["fma_bytes"])       # 1 everywhere; a fused rounding gives 0


@pytest.mark.parametrize("batch,m,k", [(1, 19, 69), (1, 1, 1), (3, 37, 130), (1, 300, 4096), (2, 5, 3)])
def test_quantize_rows_strided_and_batched(device, oracle, batch, m, k):
    """Rank 2 and 3, row strides wider than K on both sides, K not a multiple of four, a transposed source."""
    import torch
    from vecops_amd import capi
    mult = (np.float32(3.0) + synth.uniform_pm1(1, (batch * m,))).astype(np.float32)
    x = (synth.uniform_pm1(2, (batch * m, k)) * np.float32(60.0)).astype(np.float32)
    want = oracle.quantize_rows(x, mult, 100).reshape(batch, m, k)
    store = torch.full((batch, m, k + 5), float("nan"), device=device)
    store[:, :, :k] = dev(x.reshape(batch, m, k), device)
    qstore = torch.full((batch, m, k + 3), 77, dtype=torch.uint8, device=device)
    xv, qv = store[:, :, :k], qstore[:, :, :k]
    if batch == 1:
        xv, qv = xv[0], qv[0]
    capi.quantize_rows(xv, dev(mult, device), 100, qv)
    assert np.array_equal(qstore[:, :, :k].cpu().numpy(), want)
    assert (qstore[:, :, k:] == 77).all()
    if batch == 1:                                                   # source stored [K,M]
        xt = dev(np.ascontiguousarray(x.T), device).t()
        q2 = torch.zeros((m, k), dtype=torch.uint8, device=device)
        capi.quantize_rows(xt, dev(mult, device), 100, q2)
        assert np.array_equal(q2.cpu().numpy(), want[0])


@pytest.mark.parametrize("case", QUANT_CASES, ids=lambda c: c["name"])
def test_runtime_quant_pipeline_golden(device, case):
    import torch
    from vecops_amd import capi
    inp = make_quant_inputs(case)
    c = torch.full((case["m"], case["n"]), float("nan"), device=device)
    capi.matmul_runtime_quant(dev(inp["a"], device), dev(inp["multipliers"], device), case["zp"], dev(inp["b"], device),
                              dev(inp["row_scales"], device), dev(inp["column_scales"], device), c,
                              correction=dev(inp["correction"], device))
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint32), GOLD[case["name"] + "_f32"].view(np.uint32))


@pytest.mark.parametrize("m,n,k", [(2048, 1100, 4096), (1, 300, 512), (16, 4096, 4096), (255, 63, 8191)])
def test_runtime_quant_pipeline_against_the_oracle(device, oracle, m, n, k):
    """Tile, split-K and narrow shapes; B given [K,N]; no correction row."""
    import torch
    from vecops_amd import capi
    mult = (np.float32(2.0) + synth.uniform_pm1(1, (m,))).astype(np.float32)
    a = ((synth.uniform_pm1(2, (m, k)) * np.float32(140.0) + np.float32(120.0)) / mult[:, None]).astype(np.float32)
    b = synth.int8_sym(3, (n, k))
    rs, cs = (np.float32(1.0) / mult).astype(np.float32), synth.scales(4, n)
    q = oracle.quantize_rows(a, mult, 8)
    acc = np.zeros((m, n), np.int32)
    oracle.matmul(q, b, acc, atom=O.ATOM_I8I32, acc_f64=True, c_bf16=False)
    want = oracle.fused_outputs(acc, np.float32, row_scales=rs, column_scales=cs)
    bt = dev(np.ascontiguousarray(b.T), device).t()                  # [N,K] view of a [K,N] array
    c = torch.full((m, n), float("nan"), device=device)
    capi.matmul_runtime_quant(dev(a, device), dev(mult, device), 8, bt, dev(rs, device), dev(cs, device), c)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("case", QUANT_CASES, ids=lambda c: c["name"])
def test_runtime_quant_pipeline_packed_weights_golden(device, case):
    """The reference test's own operands: B packed first, the compensated pack's sidecar as the correction row
    (tests/ops/MatmulConversionTestCommon.h:1484-1510, ops/MatmulPack.h:52-58)."""
    import torch
    from vecops_amd import capi
    inp = make_quant_inputs(case)
    packed, comp = capi.pack_b(dev(inp["b"], device), a_zero_point=case["zp"])
    assert np.array_equal(comp.cpu().numpy(), inp["correction"])
    c = torch.full((case["m"], case["n"]), float("nan"), device=device)
    capi.matmul_runtime_quant_packed_b(dev(inp["a"], device), dev(inp["multipliers"], device), case["zp"], packed,
                                       dev(inp["row_scales"], device), dev(inp["column_scales"], device), c, correction=comp)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint32), GOLD[case["name"] + "_f32"].view(np.uint32))


def test_runtime_quant_batched_activations_shared_weights(device, oracle):
    """Rank-3 a and c against one b (vecops' BroadcastB case, row scales indexed batch * M + row,
    tests/ops/MatmulConversionTestCommon.h:1277-1434): the batches fold into rows."""
    import torch
    from vecops_amd import capi
    batch, m, n, k = 3, 37, 150, 300
    mult = (np.float32(2.0) + synth.uniform_pm1(1, (batch * m,))).astype(np.float32)
    a = ((synth.uniform_pm1(2, (batch * m, k)) * np.float32(140.0) + np.float32(120.0)) / mult[:, None]).astype(np.float32)
    b = synth.int8_sym(3, (n, k))
    rs, cs = (np.float32(1.0) / mult).astype(np.float32), synth.scales(4, n)
    corr = (-8 * b.astype(np.int64).sum(axis=1)).astype(np.int32)
    acc = (oracle.quantize_rows(a, mult, 8).astype(np.int64) @ b.astype(np.int64).T + corr).astype(np.int32)
    want = oracle.fused_outputs(acc, np.float32, row_scales=rs, column_scales=cs).reshape(batch, m, n)
    c = torch.full((batch, m, n), float("nan"), device=device)
    capi.matmul_runtime_quant(dev(a.reshape(batch, m, k), device), dev(mult, device), 8, dev(b, device), dev(rs, device),
                              dev(cs, device), c, correction=dev(corr, device))
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))
    # rows that do not run on from batch to batch in a: quantised from where they are, the product still folds
    gapped = torch.zeros((batch, m + 1, k), device=device)
    gapped[:, :m] = dev(a.reshape(batch, m, k), device)
    c.fill_(float("nan"))
    capi.matmul_runtime_quant(gapped[:, :m], dev(mult, device), 8, dev(b, device), dev(rs, device), dev(cs, device), c,
                              correction=dev(corr, device))
    # ... and in c: batch by batch
    cg = torch.full((batch, m + 2, n), float("nan"), device=device)
    capi.matmul_runtime_quant(gapped[:, :m], dev(mult, device), 8, dev(b, device), dev(rs, device), dev(cs, device), cg[:, :m],
                              correction=dev(corr, device))
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert np.array_equal(cg[:, :m].cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert torch.isnan(cg[:, m:]).all()


@pytest.mark.parametrize("case", QUANT_BATCHED_CASES, ids=[c["name"] for c in QUANT_BATCHED_CASES])
def test_runtime_quant_batched_golden(device, case):
    """Shared or per-batch activations and weights (tests/ops/MatmulConversionTestCommon.h:1277-1434; a batch stride of
    0 shares an operand): bit for bit against the outputs of the real vecops build."""
    import torch
    from vecops_amd import capi
    inp = make_quant_batched_inputs(case)
    batch, m, n, k = case["batch"], case["m"], case["n"], case["k"]
    a = dev(inp["a"], device).expand(batch, m, k)                   # a leading extent of 1 becomes batch stride 0
    b = dev(inp["b"], device).expand(batch, n, k)
    c = torch.full((batch, m, n), float("nan"), device=device)
    capi.matmul_runtime_quant(a, dev(inp["multipliers"], device), inp["zero_point"], b, dev(inp["row_scales"], device),
                              dev(inp["column_scales"], device), c, correction=dev(inp["correction"], device))
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint32), GOLD[case["name"] + "_f32"].view(np.uint32))


@pytest.mark.parametrize("batch,m,n,k,shared_a,shared_b", [(4, 300, 520, 1030, False, False), (5, 64, 1000, 4096, True, False),
                                                           (3, 7, 2048, 512, False, False), (6, 130, 130, 129, False, True)])
def test_runtime_quant_batched_against_the_oracle(device, oracle, batch, m, n, k, shared_a, shared_b):
    """Bigger batched shapes (several tiles per batch, a skinny M, K with a tail), operands with gaps between rows and
    batches, and the explicit batch strides of vecops_hip_matmul_runtime_quant_batched - among them one set of scales
    for per-batch activations (stride 0), which the conventional entry cannot say."""
    import torch
    from vecops_amd import capi
    case = {"kind": "seeded", "batch": batch, "m": m, "n": n, "k": k, "shared_a": shared_a, "shared_b": shared_b}
    inp = make_quant_batched_inputs(case)
    want = quant_batched_by_oracle(oracle, inp, batch)
    ab, bb = inp["a"].shape[0], inp["b"].shape[0]
    a_store = torch.full((ab, m + 1, k + 4), float("nan"), device=device)
    a_store[:, :m, :k] = dev(inp["a"], device)
    b_store = torch.full((bb, n + 2, k + 16), 99, dtype=torch.int8, device=device)
    b_store[:, :n, :k] = dev(inp["b"], device)
    a, b = a_store[:, :m, :k].expand(batch, m, k), b_store[:, :n, :k].expand(batch, n, k)
    c_store = torch.full((batch, m + 3, n + 4), float("nan"), device=device)
    c = c_store[:, :m, :n]
    mult, rs, cs = dev(inp["multipliers"], device), dev(inp["row_scales"], device), dev(inp["column_scales"], device)
    corr = dev(inp["correction"], device)
    capi.matmul_runtime_quant(a, mult, inp["zero_point"], b, rs, cs, c, correction=corr)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert torch.isnan(c_store[:, m:]).all() and torch.isnan(c_store[:, :, n:]).all()
    # the same through the explicit strides
    c_store.fill_(float("nan"))
    capi.matmul_runtime_quant_batched(a, mult, inp["zero_point"], 0 if shared_a else m, b, rs, cs, c, correction=corr,
                                      correction_batch_stride=0 if shared_b else n)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))
    if not shared_a:
        # per-batch activations under ONE set of multipliers / scales (those of batch 0) and one correction row
        inp0 = dict(inp, multipliers=np.tile(inp["multipliers"][:m], batch), row_scales=np.tile(inp["row_scales"][:m], batch),
                    correction=np.tile(inp["correction"][:n], bb))
        want0 = quant_batched_by_oracle(oracle, inp0, batch)
        c_store.fill_(float("nan"))
        capi.matmul_runtime_quant_batched(a, mult, inp["zero_point"], 0, b, rs, cs, c, correction=corr, correction_batch_stride=0)
        torch.cuda.synchronize()
        assert np.array_equal(c.cpu().numpy().view(np.uint32), want0.view(np.uint32))


def test_runtime_quant_zero_extents_and_rejections(device):
    import torch
    from vecops_amd import capi
    one = torch.ones(4, device=device)
    c = torch.full((4, 6), float("nan"), device=device)
    corr = torch.arange(6, dtype=torch.int32, device=device)
    capi.matmul_runtime_quant(torch.empty((4, 0), device=device), one, 3, torch.empty((6, 0), dtype=torch.int8, device=device),
                              one, torch.ones(6, device=device), c, correction=corr)
    torch.cuda.synchronize()
    assert torch.equal(c, corr.float().expand(4, 6))                  # K == 0: the correction row, dequantised
    capi.matmul_runtime_quant(torch.empty((0, 8), device=device), one, 3, torch.zeros((6, 8), dtype=torch.int8, device=device),
                              one, torch.ones(6, device=device), torch.empty((0, 6), device=device))
    with pytest.raises(capi.VecopsHipError) as e:                     # bf16 activations are not this entry's business
        capi.matmul_runtime_quant(torch.zeros((4, 8), dtype=torch.bfloat16, device=device), one, 3,
                                  torch.zeros((6, 8), dtype=torch.int8, device=device), one, torch.ones(6, device=device), c)
    assert e.value.code == 2
    with pytest.raises(capi.VecopsHipError) as e:
        capi.quantize_rows(torch.zeros((4, 8), device=device), one, 3, torch.zeros((4, 9), dtype=torch.uint8, device=device))
    assert e.value.code == 1
