"""The whole drop-in path on the GPU: vecops Operator -> dispatch policy -> recipe
-> HipExecutableProvider -> Executable -> artifact DSO -> C ABI -> gfx950 kernel,
with host tensors (staged inside the artifact) and with device tensors (used in
place), checked against the oracle.  Runs against the restated runtime and against
the plug-in compiled into the vecops tree's own runtime where oracle/_ref holds it."""
import os

import numpy as np
import pytest

from conftest import rel_err
from oracle import oracle as O
from vecops_amd import host_api as H
from vecops_amd import synth

pytestmark = pytest.mark.gpu
# the same plug-in compiled against the reference's own runtime sources (a checker build: oracle/Makefile, target ref)
UPSTREAM_LIB = os.path.join(H.ROOT, "oracle", "_ref", "libvecops_hip_host_upstream.so")
FLAVORS = [H.HOST_LIB] + ([UPSTREAM_LIB] if os.path.exists(UPSTREAM_LIB) else [])


@pytest.fixture(scope="module", params=FLAVORS, ids=lambda p: "upstream" if "upstream" in p else "restated")
def host(request, device):
    return H.HostLibrary(request.param)


def fp32_tol(k):
    return 2e-6 * max(1.0, k / 32)


@pytest.mark.parametrize("m,n,k", [(37, 51, 79), (300, 260, 1000), (255, 63, 8191)])
def test_matmul_bf16_host_tensors(host, oracle, m, n, k):
    op = host.operator("vecops::matmul")
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    c = np.full((m, n), np.nan, np.float32)
    frame = H.Frame([a, b, None, c], outputs=(3,))
    assert op.workspace(frame) == 0          # host callers cannot supply device scratch
    op.invoke(frame)
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, acc_f64=True)
    assert rel_err(c, want) <= fp32_tol(k)


def test_matmul_host_strided_views_and_aliased_c_input(host, oracle):
    op = host.operator("vecops::matmul")
    m, n, k = 33, 47, 130
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b_kn = np.ascontiguousarray(synth.bf16_round(synth.uniform_pm1(2, (n, k))).T)   # [K,N] row-major
    b = b_kn.T
    store = np.full((m, 2 * n), -5.0, np.float32)
    store[:, 0:2 * n:2] = synth.uniform_pm1(3, (m, n))
    c = store[:, 0:2 * n:2]                                                        # every other column
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, cin=c.copy(), acc_f64=True)
    op.invoke(H.Frame([a, b, c, c], outputs=(3,)))                                   # C input aliases the output
    assert rel_err(c, want) <= fp32_tol(k)
    assert (store[:, 1:2 * n:2] == -5.0).all()                                       # gaps untouched


def test_matmul_device_tensors_and_workspace(host, oracle, device):
    import torch
    op = host.operator("vecops::matmul")
    m, n, k = 255, 63, 8191                   # tiny output, long K: split-K needs caller workspace
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    ta = torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
    tb = torch.from_numpy(b.view(np.int16)).to(device).view(torch.bfloat16)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    frame = H.Frame([ta, tb, None, c], outputs=(3,))
    assert op.resolve(frame).endswith("memory=device;backend=hip-gfx950")
    need = op.workspace(frame)
    assert need > 0
    with pytest.raises(H.HostError) as e:     # Executable::invoke rejects too little workspace (Executable.cpp:291-295)
        op.invoke(frame)
    assert e.value.code == 1 and "workspace bytes" in e.value.message
    ws = torch.empty(need, dtype=torch.uint8, device=device)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        op.invoke(frame, workspace=ws.data_ptr(), workspace_size=need, stream=stream.cuda_stream)
    # the ABI is synchronous: the result is visible as soon as invoke returns
    got = c.cpu().numpy()
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, acc_f64=True)
    assert rel_err(got, want) <= fp32_tol(k)


def test_matmul_required_family(host, oracle, device):
    """The `Family` specialization through Operator::invoke: the required family computes the product (host and device
    tensors); a family that cannot serve the call is "not applicable" from the artifact, nothing is written."""
    import torch
    op = host.operator("vecops::matmul")
    m, n, k = 300, 260, 1000
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, acc_f64=True)
    for family in (1, 2, 3, 6, 7, 9):
        c = np.full((m, n), np.nan, np.float32)
        op.invoke(H.Frame([a, b, None, c], outputs=(3,)), {"Family": family})
        assert rel_err(c, want) <= fp32_tol(k), family
    ta = torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
    tb = torch.from_numpy(b.view(np.int16)).to(device).view(torch.bfloat16)
    tc = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    frame = H.Frame([ta, tb, None, tc], outputs=(3,))
    assert "family=tile_128;memory=device" in op.resolve(frame, {"Family": 2})
    need = op.workspace(frame, {"Family": 2})
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=device)
    op.invoke(frame, {"Family": 2}, workspace=ws.data_ptr(), workspace_size=need)
    assert rel_err(tc.cpu().numpy(), want) <= fp32_tol(k)
    c = np.full((m, n), 7.0, np.float32)
    with pytest.raises(H.HostError) as e:        # the skinny family cannot serve 300 x 260 x 1000
        op.invoke(H.Frame([a, b, None, c], outputs=(3,)), {"Family": 4})
    assert e.value.code == 2 and "skinny" in e.value.message
    assert (c == 7.0).all()
    with pytest.raises(H.HostError) as e:        # nor the 256 x 352 tile a K of 1000 (no whole number of K tiles)
        op.invoke(H.Frame([a, b, None, c], outputs=(3,)), {"Family": 8})
    assert e.value.code == 2 and (c == 7.0).all()
    # ... and serves its own shapes
    m2, n2, k2 = 4, 1024, 512
    a2 = synth.bf16_round(synth.uniform_pm1(3, (m2, k2)))
    b2 = synth.bf16_round(synth.uniform_pm1(4, (n2, k2)))
    c2 = np.full((m2, n2), np.nan, np.float32)
    op.invoke(H.Frame([a2, b2, None, c2], outputs=(3,)), {"Family": 4})
    want2 = np.zeros((m2, n2), np.float32)
    oracle.matmul(a2, b2, want2, acc_f64=True)
    assert rel_err(c2, want2) <= fp32_tol(k2)
    # 8-bit integers, bit-exact
    ai, bi = synth.int8_sym(5, (m, k)), synth.int8_sym(6, (n, k))
    ci = np.zeros((m, n), np.int32)
    op.invoke(H.Frame([ai, bi, None, ci], outputs=(3,)), {"Family": 6})
    assert np.array_equal(ci, (ai.astype(np.int64) @ bi.astype(np.int64).T).astype(np.int32))


def test_matmul_rank3_fp32_and_int8(host, oracle, device):
    import torch
    op = host.operator("vecops::matmul")
    batch, m, n, k = 3, 40, 56, 96
    a, b = synth.uniform_pm1(1, (batch, m, k)), synth.uniform_pm1(2, (n, k))
    c = np.zeros((batch, m, n), np.float32)
    bb = np.broadcast_to(b, (batch, n, k))    # stride-0 batch
    op.invoke(H.Frame([a, bb, None, c], outputs=(3,)))
    want = np.zeros((batch, m, n), np.float32)
    oracle.matmul(a, bb, want, atom=O.ATOM_BF16F32, acc_f64=True)
    assert rel_err(c, want) <= fp32_tol(k)
    ai, bi = synth.int8_sym(3, (130, 515)), synth.int8_sym(4, (140, 515))
    ci = torch.zeros((130, 140), dtype=torch.int32, device=device)
    op.invoke(H.Frame([torch.from_numpy(ai).to(device), torch.from_numpy(bi).to(device), None, ci], outputs=(3,)))
    assert np.array_equal(ci.cpu().numpy(), oracle.matmul_i8_dense(ai, bi))
    # unsigned activations against signed weights, host tensors: the same recipe and artifact
    au = (synth.draws(5, 130 * 515) % np.uint64(256)).astype(np.uint8).reshape(130, 515)
    cu = np.zeros((130, 140), np.int32)
    op.invoke(H.Frame([au, bi, None, cu], outputs=(3,)))
    assert np.array_equal(cu, (au.astype(np.int64) @ bi.astype(np.int64).T).astype(np.int32))


def test_matmul_fp32_compute_operator(host, oracle):
    """ComputeType=Float32 selects the fp32-compute artifact: operands are not rounded to bf16."""
    op = host.operator("vecops::matmul")
    m, n, k = 96, 80, 300
    a, b = synth.uniform_pm1(1, (m, k)), synth.uniform_pm1(2, (n, k))
    c = np.zeros((m, n), np.float32)
    op.invoke(H.Frame([a, b, None, c], outputs=(3,)), {"ComputeType": ("dtype", H.F32)})
    exact = a.astype(np.float64) @ b.astype(np.float64).T
    assert rel_err(c, exact) <= 1.2e-7 * k
    c_bf16_compute = np.zeros((m, n), np.float32)
    op.invoke(H.Frame([a, b, None, c_bf16_compute], outputs=(3,)))
    assert rel_err(c_bf16_compute, exact) > 1e-3        # the default rounds the operands to bf16


def test_matmul_i8_dequant_operator(host, oracle, device):
    import torch
    op = host.operator("vecops::matmul_i8_dequant")
    m, n, k = 67, 129, 515
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    corr = ((synth.draws(5, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32)
    want = oracle.matmul_i8_dequant(a, b, rs, cs, corr)
    c = np.zeros((m, n), np.float32)
    op.invoke(H.Frame([a, b, rs, cs, corr, c], outputs=(5,)))
    assert np.array_equal(c.view(np.uint32), want.view(np.uint32))
    tc = torch.zeros((m, n), dtype=torch.float32, device=device)
    to = lambda x: torch.from_numpy(x).to(device)  # noqa: E731
    op.invoke(H.Frame([to(a), to(b), to(rs), to(cs), None, tc], outputs=(5,)))
    assert np.array_equal(tc.cpu().numpy().view(np.uint32), oracle.matmul_i8_dequant(a, b, rs, cs).view(np.uint32))


def test_matmul_f16_operator(host, oracle, device):
    import torch
    op = host.operator("vecops::matmul")
    m, n, k = 130, 264, 200
    a = synth.uniform_pm1(1, (m, k)).astype(np.float16)
    b = synth.uniform_pm1(2, (n, k)).astype(np.float16)
    want = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, want, atom=O.ATOM_F16F32, acc_f64=True)
    c = np.full((m, n), np.nan, np.float32)
    op.invoke(H.Frame([a, b, None, c], outputs=(3,)))                       # host tensors, staged
    assert rel_err(c, want) <= fp32_tol(k)
    th = torch.zeros((m, n), dtype=torch.float16, device=device)
    frame = H.Frame([torch.from_numpy(a).to(device), torch.from_numpy(b).to(device), None, th], outputs=(3,))
    assert op.resolve(frame) == "vecops::matmul;operands=f16;compute=f16;memory=device;backend=hip-gfx950"
    op.invoke(frame)
    assert rel_err(th.cpu().numpy().astype(np.float32), want) <= 2.0 ** -10


def test_matmul_fused_operator(host, oracle, device):
    """vecops::matmul_fused through the Operator: int8 with an int32 bias row, both scale vectors, a shift and
    requantisation to uint8 (host tensors, staged); bf16 with a bias row and silu to bf16 (device tensors)."""
    import torch
    op = host.operator("vecops::matmul_fused")
    m, n, k = 67, 129, 515
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m) * np.float32(64), synth.scales(4, n)
    bias = ((synth.draws(5, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32)
    acc = np.zeros((m, n), np.int32)
    oracle.matmul(a, b, acc, cin=np.broadcast_to(bias, (m, n)), atom=O.ATOM_I8I32, acc_f64=True, c_bf16=False)
    want = oracle.fused_outputs(acc, np.uint8, row_scales=rs, column_scales=cs, shift=128.0)
    assert (want == 0).any() and (want == 255).any()
    c = np.full((m, n), 9, np.uint8)
    bias_rows = np.broadcast_to(bias, (m, n))                                  # row stride 0
    frame = H.Frame([a, b, bias_rows, rs, cs, 0, 1.0, 128.0, 0.0, 0.0, c], outputs=(10,))
    assert op.resolve(frame) == "vecops::matmul_fused;operands=i8;memory=host;backend=hip-gfx950"
    op.invoke(frame)
    assert np.array_equal(c, want)
    # relu on the same sums, fp32 out, device tensors
    to = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(device)  # noqa: E731
    want_relu = oracle.fused_outputs(acc, np.float32, column_scales=cs, scale=-0.5, activation=1)
    tc = torch.full((m, n), float("nan"), device=device)
    tbias = to(bias).reshape(1, n).expand(m, n)
    frame = H.Frame([to(a), to(b), tbias, None, to(cs), 1, -0.5, 0.0, 0.0, 0.0, tc], outputs=(10,))
    assert op.resolve(frame).endswith("operands=i8;memory=device;backend=hip-gfx950")
    op.invoke(frame)
    assert np.array_equal(tc.cpu().numpy().view(np.uint32), want_relu.view(np.uint32))
    # bf16 operands, fp32 bias row, silu, bf16 out
    m, n, k = 130, 270, 200
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    fbias = synth.uniform_pm1(3, (n,))
    facc = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, facc, cin=np.broadcast_to(fbias, (m, n)), acc_f64=True, c_bf16=False)
    want16 = oracle.fused_outputs(facc, np.uint16, activation=4)
    ta = torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
    tb = torch.from_numpy(b.view(np.int16)).to(device).view(torch.bfloat16)
    tc16 = torch.zeros((m, n), dtype=torch.bfloat16, device=device)
    frame = H.Frame([ta, tb, to(fbias).reshape(1, n).expand(m, n), None, None, 4, 1.0, 0.0, 0.0, 0.0, tc16], outputs=(10,))
    assert op.resolve(frame) == "vecops::matmul_fused;operands=bf16;memory=device;backend=hip-gfx950"
    op.invoke(frame)
    got16 = tc16.view(torch.int16).cpu().numpy().view(np.uint16)
    assert rel_err(synth.bf16_to_f32(got16), synth.bf16_to_f32(want16)) <= 2 ** -7


def test_packed_b_operators(host, oracle, device):
    """vecops::matmul_pack_b then vecops::matmul_packed_b through the Operator: results equal vecops::matmul's on
    the unpacked operand bit for bit (host tensors staged, device tensors in place), the compensation row equals
    -zp * sum_k b[n,k], and one packed operand serves every batch of a rank-3 a."""
    import torch
    from vecops_amd import capi
    pack, mul, plain = (host.operator("vecops::matmul_pack_b"), host.operator("vecops::matmul_packed_b"),
                        host.operator("vecops::matmul"))
    # int8, host tensors, compensated pack
    m, n, k = 67, 129, 515
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    size = capi.lib().vecops_hip_packed_b_bytes(capi.I8, n, k)
    packed, comp = np.zeros(size, np.uint8), np.zeros(n, np.int32)
    frame = H.Frame([b, 7, packed, comp], outputs=(2, 3))
    assert pack.resolve(frame) == "vecops::matmul_pack_b;operands=i8;memory=host;backend=hip-gfx950"
    pack.invoke(frame)
    assert np.array_equal(comp, (-7 * b.astype(np.int64).sum(axis=1)).astype(np.int32))
    want = np.zeros((m, n), np.int32)
    oracle.matmul(a, b, want, atom=O.ATOM_I8I32, acc_f64=True, c_bf16=False)
    c = np.full((m, n), -1, np.int32)
    mul.invoke(H.Frame([a, packed, None, c], outputs=(3,)))
    assert np.array_equal(c, want)
    corr = np.broadcast_to(comp, (m, n))                                      # the sidecar as a stride-0 C-input row
    mul.invoke(H.Frame([a, packed, corr, c], outputs=(3,)))
    assert np.array_equal(c, want + comp[None, :])
    ua = (a.astype(np.int16) + 7).clip(0, 255).astype(np.uint8)                # asymmetric activations, zero point 7
    mul.invoke(H.Frame([ua, packed, corr, c], outputs=(3,)))                   # = sum_k (ua - 7) * b
    assert np.array_equal(c, ((ua.astype(np.int64) - 7) @ b.astype(np.int64).T).astype(np.int32))
    # bf16 from an fp32 source, device tensors, rank-3 a with a workspace when the plan asks for one
    batch, m, n, k = 3, 50, 200, 1000
    a = synth.bf16_round(synth.uniform_pm1(1, (batch, m, k)))
    bf = synth.uniform_pm1(2, (n, k))
    ta = torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
    tbf = torch.from_numpy(bf).to(device)
    tb = torch.from_numpy(synth.bf16_round(bf).view(np.int16)).to(device).view(torch.bfloat16)
    tp = torch.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.BF16, n, k), dtype=torch.uint8, device=device)
    frame = H.Frame([tbf, 0, tp, None], outputs=(2,))
    assert pack.resolve(frame) == "vecops::matmul_pack_b;operands=bf16;memory=device;backend=hip-gfx950"
    pack.invoke(frame)
    tc = torch.full((batch, m, n), float("nan"), device=device)
    frame = H.Frame([ta, tp, None, tc], outputs=(3,))
    need = mul.workspace(frame)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
    mul.invoke(frame, workspace=ws.data_ptr(), workspace_size=need)
    tref = torch.full((batch, m, n), float("nan"), device=device)
    frame = H.Frame([ta, tb.unsqueeze(0).expand(batch, n, k), None, tref], outputs=(3,))
    need = plain.workspace(frame)
    ws2 = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
    plain.invoke(frame, workspace=ws2.data_ptr(), workspace_size=need)
    torch.cuda.synchronize()
    got = tc.cpu().numpy()
    wantf = np.zeros((batch, m, n), np.float32)
    for i in range(batch):
        oracle.matmul(a[i], synth.bf16_round(bf), wantf[i], acc_f64=True, c_bf16=False)
    assert rel_err(got, wantf) <= fp32_tol(k)
    assert rel_err(got, tref.cpu().numpy()) <= fp32_tol(k)
    # a packed tensor of the wrong size is an invalid argument, not a fault
    with pytest.raises(H.HostError) as e:
        mul.invoke(H.Frame([ta, tp[:64], None, tc], outputs=(3,)))
    assert e.value.code == 1
    # half operands (AMX_F16F32): their own recipes and artifacts, f32 and f16 outputs, host and device tensors
    m, n, k = 70, 130, 264
    ah, bh = synth.uniform_pm1(5, (m, k)).astype(np.float16), synth.uniform_pm1(6, (n, k)).astype(np.float16)
    wanth = ah.astype(np.float64) @ bh.astype(np.float64).T
    packed = np.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.F16, n, k), np.uint8)
    frame = H.Frame([bh, 0, packed, None], outputs=(2,))
    assert pack.resolve(frame) == "vecops::matmul_pack_b;operands=f16;memory=host;backend=hip-gfx950"
    pack.invoke(frame)
    ch = np.full((m, n), np.nan, np.float32)
    frame = H.Frame([ah, packed, None, ch], outputs=(3,))
    assert mul.resolve(frame) == "vecops::matmul_packed_b;operands=f16;memory=host;backend=hip-gfx950"
    mul.invoke(frame)
    assert rel_err(ch, wanth) <= fp32_tol(k)
    th, tph = torch.from_numpy(ah).to(device), torch.from_numpy(packed).to(device)
    tch = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    frame = H.Frame([th, tph, None, tch], outputs=(3,))
    assert mul.resolve(frame) == "vecops::matmul_packed_b;operands=f16;memory=device;backend=hip-gfx950"
    need = mul.workspace(frame)
    wsh = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
    mul.invoke(frame, workspace=wsh.data_ptr(), workspace_size=need)
    torch.cuda.synchronize()
    assert np.array_equal(tch.cpu().numpy().view(np.uint16), ch.astype(np.float16).view(np.uint16))   # RNE of the fp32 result
    with pytest.raises(H.HostError):                                         # a bf16 output does not go with half operands
        mul.invoke(H.Frame([th, tph, None, torch.empty((m, n), dtype=torch.bfloat16, device=device)], outputs=(3,)))


def test_matmul_runtime_quant_operator(host, device):
    """vecops::matmul_runtime_quant through the Operator, host tensors (staged) and device tensors (in place, with
    the workspace the artifact asks for): the golden case of the real vecops build, bit for bit."""
    import torch
    from golden_cases import QUANT_CASES, make_quant_inputs
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vecops_quant_golden.npz"))
    op = host.operator("vecops::matmul_runtime_quant")
    case = QUANT_CASES[1]
    inp = make_quant_inputs(case)
    want = gold[case["name"] + "_f32"]
    c = np.full((case["m"], case["n"]), np.nan, np.float32)
    frame = H.Frame([inp["a"], inp["b"], inp["multipliers"], case["zp"], inp["row_scales"], inp["column_scales"],
                     inp["correction"], c], outputs=(7,))
    assert "memory=host" in op.resolve(frame)
    op.invoke(frame)
    assert np.array_equal(c.view(np.uint32), want.view(np.uint32))
    to = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(device)  # noqa: E731
    tc = torch.full((case["m"], case["n"]), float("nan"), device=device)
    frame = H.Frame([to(inp["a"]), to(inp["b"]), to(inp["multipliers"]), case["zp"], to(inp["row_scales"]),
                     to(inp["column_scales"]), to(inp["correction"]), tc], outputs=(7,))
    assert "memory=device" in op.resolve(frame)
    need = op.workspace(frame)
    assert need >= case["m"] * case["k"]                                      # the quantised activations live there
    ws = torch.empty(need, dtype=torch.uint8, device=device)
    op.invoke(frame, workspace=ws.data_ptr(), workspace_size=need)
    torch.cuda.synchronize()
    assert np.array_equal(tc.cpu().numpy().view(np.uint32), want.view(np.uint32))
    with pytest.raises(H.HostError) as e:                                      # too little workspace is an error, not a fault
        op.invoke(frame, workspace=ws.data_ptr(), workspace_size=16)
    assert e.value.code == 1


def test_matmul_w8a16_group_operator(host, oracle, device):
    import torch
    op = host.operator("vecops::matmul_w8a16_group")
    for m, n, k, g in [(1, 512, 1024, 128), (4, 300, 512, 64)]:
        x = synth.bf16_round(synth.normal(1, (m, k)))
        w = synth.int8_sym(2, (n, k))
        s = synth.scales(3, (n, k // g))
        _, want = oracle.matmul_w8a16_group(x, w, s, g)
        y = np.zeros((m, n), np.uint16)
        op.invoke(H.Frame([x, w, s, y], outputs=(3,)), {"G": g})
        assert rel_err(synth.bf16_to_f32(y), want) <= 2 ** -7
        ty = torch.zeros((m, n), dtype=torch.bfloat16, device=device)
        tx = torch.from_numpy(x.view(np.int16)).to(device).view(torch.bfloat16)
        op.invoke(H.Frame([tx, torch.from_numpy(w).to(device), torch.from_numpy(s).to(device), ty], outputs=(3,)),
                  {"G": g})
        got = ty.view(torch.int16).cpu().numpy().view(np.uint16)
        assert np.array_equal(got, y)         # host-staged and in-place runs agree bit for bit
    with pytest.raises(H.HostError) as e:     # M > 16 is not the skinny family
        op.invoke(H.Frame([np.zeros((17, 256), np.uint16), np.zeros((8, 256), np.int8), np.zeros((8, 2), np.float32),
                           np.zeros((17, 8), np.uint16)], outputs=(3,)))
    assert e.value.code in (2, 3)


def test_mixed_placement_is_refused(host, device):
    import torch
    op = host.operator("vecops::matmul")
    a = np.zeros((4, 8), np.uint16)
    tb = torch.zeros((5, 8), dtype=torch.bfloat16, device=device)
    with pytest.raises(H.HostError) as e:
        op.invoke(H.Frame([a, tb, None, np.zeros((4, 5), np.float32)], outputs=(3,)))
    assert e.value.code in (2, 3)


def _conversion_value(count, seed, unsigned):
    """tests/ops/MatmulConversionTestCommon.h:62-70 for the integral types: the operands of the reference's tests."""
    low = 0 if unsigned else -3
    return (low + (np.arange(count, dtype=np.int64) * 5 + seed) % 7).astype(np.uint8 if unsigned else np.int8)


@pytest.mark.parametrize("a_unsigned,b_unsigned", [(False, False), (False, True), (True, False), (True, True)])
def test_mixed_packing_case_through_the_operators(host, a_unsigned, b_unsigned):
    """tests/ops/MatmulMixedPackingTest.cpp:24-28 through the Operator surface: the reference's own 19 x 21 x 65 case with
    its conversion_value operands, for each signedness, with A packed (vecops::matmul_pack_a / matmul_packed_a) and
    with B packed (vecops::matmul_pack_b / matmul_packed_b); a packed operand of unsigned bytes is announced by the
    PackedType specialization value.  Exact int32 sums."""
    from vecops_amd import capi
    m, n, k = 19, 21, 65
    a = _conversion_value(m * k, 3, a_unsigned).reshape(m, k)
    b = _conversion_value(n * k, 11, b_unsigned).reshape(n, k)
    want = (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32)
    u8 = {"PackedType": ("dtype", H.U8)}
    # B packed
    packed_b = np.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.U8 if b_unsigned else capi.I8, n, k), np.uint8)
    frame = H.Frame([b, 0, packed_b, None], outputs=(2,))
    pack_b = host.operator("vecops::matmul_pack_b")
    assert f"operands={'u8' if b_unsigned else 'i8'};" in pack_b.resolve(frame)
    pack_b.invoke(frame)
    c = np.full((m, n), -1, np.int32)
    mul_b = host.operator("vecops::matmul_packed_b")
    frame = H.Frame([a, packed_b, None, c], outputs=(3,))
    assert ("packed=u8" in mul_b.resolve(frame, u8 if b_unsigned else None)) == b_unsigned
    mul_b.invoke(frame, u8 if b_unsigned else None)
    assert np.array_equal(c, want)
    # A packed
    packed_a = np.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.U8 if a_unsigned else capi.I8, m, k), np.uint8)
    frame = H.Frame([a, packed_a], outputs=(1,))
    pack_a = host.operator("vecops::matmul_pack_a")
    assert pack_a.resolve(frame) == f"vecops::matmul_pack_a;operands={'u8' if a_unsigned else 'i8'};memory=host;backend=hip-gfx950"
    pack_a.invoke(frame)
    c = np.full((m, n), -1, np.int32)
    mul_a = host.operator("vecops::matmul_packed_a")
    frame = H.Frame([packed_a, b, None, c], outputs=(3,))
    assert ("packed=u8" in mul_a.resolve(frame, u8 if a_unsigned else None)) == a_unsigned
    mul_a.invoke(frame, u8 if a_unsigned else None)
    assert np.array_equal(c, want)
    # with the wrong announcement the bytes are read as the other signedness: the sums differ by 128 * the row sums
    if a_unsigned:
        mul_a.invoke(frame)
        assert np.array_equal(c, want - 128 * b.astype(np.int64).sum(axis=1)[None, :].astype(np.int32))


def test_packed_a_operators(host, oracle, device):
    """vecops::matmul_pack_a then vecops::matmul_packed_a on larger shapes: int8 bit for bit against vecops::matmul
    (host tensors), bf16 from an fp32 source on device tensors with one packed a serving every batch of a rank-3 b and
    a C-input, half operands to a half output; too small a packed buffer is an invalid argument."""
    import torch
    from vecops_amd import capi
    pack, mul, plain = (host.operator("vecops::matmul_pack_a"), host.operator("vecops::matmul_packed_a"),
                        host.operator("vecops::matmul"))
    m, n, k = 129, 67, 515
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    packed = np.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.I8, m, k), np.uint8)
    pack.invoke(H.Frame([a, packed], outputs=(1,)))
    want = np.zeros((m, n), np.int32)
    plain.invoke(H.Frame([a, b, None, want], outputs=(3,)))
    assert np.array_equal(want, (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32))
    c = np.full((m, n), -1, np.int32)
    mul.invoke(H.Frame([packed, b, None, c], outputs=(3,)))
    assert np.array_equal(c, want)
    cin = synth.int8_sym(3, (m, n)).astype(np.int32)
    mul.invoke(H.Frame([packed, b, cin, c], outputs=(3,)))
    assert np.array_equal(c, want + cin)
    with pytest.raises(H.HostError) as e:
        pack.invoke(H.Frame([a, np.zeros(16, np.uint8)], outputs=(1,)))
    assert e.value.code == 1 and "bytes" in e.value.message
    with pytest.raises(H.HostError) as e:
        mul.invoke(H.Frame([packed[:64], b, None, c], outputs=(3,)))
    assert e.value.code == 1
    # bf16 packed from fp32, device tensors, rank-3 b
    batch, m, n, k = 3, 200, 50, 1000
    af = synth.uniform_pm1(1, (m, k))
    b = synth.bf16_round(synth.uniform_pm1(2, (batch, n, k)))
    taf = torch.from_numpy(af).to(device)
    tb = torch.from_numpy(b.view(np.int16)).to(device).view(torch.bfloat16)
    tp = torch.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.BF16, m, k), dtype=torch.uint8, device=device)
    frame = H.Frame([taf, tp], outputs=(1,))
    assert pack.resolve(frame) == "vecops::matmul_pack_a;operands=bf16;memory=device;backend=hip-gfx950"
    pack.invoke(frame)
    cin = synth.uniform_pm1(4, (batch, m, n))
    tcin = torch.from_numpy(cin).to(device)
    tc = torch.full((batch, m, n), float("nan"), device=device)
    frame = H.Frame([tp, tb, tcin, tc], outputs=(3,))
    assert mul.resolve(frame) == "vecops::matmul_packed_a;operands=bf16;memory=device;backend=hip-gfx950"
    need = mul.workspace(frame)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
    mul.invoke(frame, workspace=ws.data_ptr(), workspace_size=need)
    torch.cuda.synchronize()
    wantf = np.zeros((batch, m, n), np.float32)
    for i in range(batch):
        oracle.matmul(synth.bf16_round(af), b[i], wantf[i], cin=cin[i], acc_f64=True, c_bf16=False)
    assert rel_err(tc.cpu().numpy(), wantf) <= fp32_tol(k)
    # half operands, host tensors, half output
    m, n, k = 130, 70, 264
    ah, bh = synth.uniform_pm1(5, (m, k)).astype(np.float16), synth.uniform_pm1(6, (n, k)).astype(np.float16)
    packed = np.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.F16, m, k), np.uint8)
    pack.invoke(H.Frame([ah, packed], outputs=(1,)))
    ch = np.full((m, n), np.nan, np.float16)
    frame = H.Frame([packed, bh, None, ch], outputs=(3,))
    assert mul.resolve(frame) == "vecops::matmul_packed_a;operands=f16;memory=host;backend=hip-gfx950"
    mul.invoke(frame)
    wanth = ah.astype(np.float64) @ bh.astype(np.float64).T
    assert rel_err(ch.astype(np.float64), wanth) <= 2e-3


def test_fp32_compute_pack_through_the_operators(host, device):
    """ComputeType = Float32 on the pack and on the product: fp32 operands packed as fp32 and multiplied in fp32, B
    side on host tensors and A side on device tensors, against fp64 far inside what bf16 rounding would leave."""
    import torch
    from vecops_amd import capi
    f32 = {"ComputeType": ("dtype", H.F32)}
    m, n, k = 70, 130, 520
    a, b = synth.uniform_pm1(1, (m, k)), synth.uniform_pm1(2, (n, k))
    want = a.astype(np.float64) @ b.astype(np.float64).T
    packed = np.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.F32, n, k), np.uint8)
    host.operator("vecops::matmul_pack_b").invoke(H.Frame([b, 0, packed, None], outputs=(2,)), f32)
    c = np.full((m, n), np.nan, np.float32)
    host.operator("vecops::matmul_packed_b").invoke(H.Frame([a, packed, None, c], outputs=(3,)), f32)
    assert rel_err(c, want) <= 1e-5
    ta, tb = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    tp = torch.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.F32, m, k), dtype=torch.uint8, device=device)
    host.operator("vecops::matmul_pack_a").invoke(H.Frame([ta, tp], outputs=(1,)), f32)
    tc = torch.full((m, n), float("nan"), device=device)
    mul_a = host.operator("vecops::matmul_packed_a")
    frame = H.Frame([tp, tb, None, tc], outputs=(3,))
    need = mul_a.workspace(frame, f32)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
    mul_a.invoke(frame, f32, workspace=ws.data_ptr(), workspace_size=need)
    torch.cuda.synchronize()
    assert rel_err(tc.cpu().numpy(), want) <= 1e-5
    # the bf16 pack of the same source, for contrast: the rounding of the weights is visible
    host.operator("vecops::matmul_pack_b").invoke(H.Frame([b, 0, packed, None], outputs=(2,)))
    host.operator("vecops::matmul_packed_b").invoke(H.Frame([a, packed, None, c], outputs=(3,)))
    assert rel_err(c, want) > 1e-4
