"""The Torch registration facade (vecops_amd/torch_bridge.py), counterpart of vecops.ops.torch.register
(python/vecops/ops/torch.py:35-86): name validation, idempotent registration, schemas with mutable outputs,
Meta dispatch, error mapping without a GPU; on the GPU, results through torch.ops equal the C ABI's."""
import numpy as np
import pytest
import torch

from vecops_amd import capi
from vecops_amd import host_api as H
from vecops_amd import synth
from vecops_amd import torch_bridge as tb


def test_name_validation():
    for bad in ("matmul", "a::b::c"):
        with pytest.raises(ValueError, match="library::name"):
            tb.register(bad)
    for bad in ("::matmul", "lib::"):
        with pytest.raises(ValueError, match="must not be empty"):
            tb.register(bad)
    with pytest.raises(ValueError, match="no HIP operator"):
        tb.register("vecops_hip_t::transpose")
    with pytest.raises(TypeError):
        tb.register("vecops_hip_t::matmul", dispatch=object())


def test_registration_is_idempotent_and_schemas_mark_outputs():
    first = tb.register("vecops_hip_t::matmul")
    assert tb.register("vecops_hip_t::matmul") is first
    assert tb.vecops_hip_t.matmul is first
    with pytest.raises(AttributeError):
        tb.no_such_library
    ns = tb.register_all("vecops_hip_t")
    assert sorted(vars(ns)) == ["matmul", "matmul_fused", "matmul_i8_dequant", "matmul_pack_a", "matmul_pack_b",
                                "matmul_packed_a", "matmul_packed_b", "matmul_runtime_quant", "matmul_w8a16_group"]
    pack = str(torch.ops.vecops_hip_t.matmul_pack_b.default._schema)
    assert "int a_zero_point" in pack and "Tensor(a!) packed" in pack and "Tensor(b!)? compensation" in pack
    schema = str(torch.ops.vecops_hip_t.matmul.default._schema)
    assert "Tensor? c_in" in schema and "Tensor(a!) c" in schema and "int ComputeType=-1" in schema
    assert "-> ()" in schema
    fused = str(torch.ops.vecops_hip_t.matmul_fused.default._schema)
    assert "int activation" in fused and "float scale" in fused and "Tensor(a!) c" in fused
    assert "int G=-1" in str(torch.ops.vecops_hip_t.matmul_w8a16_group.default._schema)


def test_meta_tensors_and_argument_checks():
    mm = tb.register("vecops_hip_t::matmul")
    a = torch.empty(4, 8, dtype=torch.bfloat16, device="meta")
    b = torch.empty(5, 8, dtype=torch.bfloat16, device="meta")
    c = torch.empty(4, 5, device="meta")
    assert mm(a, b, None, c) is c                        # the caller's own output object comes back
    with pytest.raises(TypeError, match="positional"):
        mm(a, b, c)
    with pytest.raises(TypeError, match="unknown specialization"):
        mm(a, b, None, c, Group=3)


@pytest.mark.skipif(torch.cuda.is_available(), reason="this case is the no-GPU error path")
def test_host_tensors_without_a_gpu_report_an_execution_error():
    mm = tb.register("vecops_hip_t::matmul")
    a, b, c = torch.zeros(4, 8, dtype=torch.bfloat16), torch.zeros(5, 8, dtype=torch.bfloat16), torch.zeros(4, 5)
    with pytest.raises(H.HostError) as e:                # resolved, loaded, run() stops at "no HIP device"
        mm(a, b, None, c)
    assert e.value.code == 6
    with pytest.raises(H.HostError) as e:                # schema violations surface as InvalidArgument
        mm(a, torch.zeros(5, 9, dtype=torch.bfloat16), None, c)
    assert e.value.code == 1 and "K" in e.value.message


# ---- GPU ------------------------------------------------------------------------------------------

def _bf16(x, device):
    return torch.from_numpy(synth.bf16_round(x).view(np.int16)).to(device).view(torch.bfloat16)


@pytest.mark.gpu
def test_torch_ops_matmul_equals_the_c_abi(device):
    from vecops_amd import capi
    ns = tb.register_all("vecops_hip_t")
    m, n, k = 300, 260, 1000
    a, b = _bf16(synth.uniform_pm1(1, (m, k)), device), _bf16(synth.uniform_pm1(2, (n, k)), device)
    want = torch.empty(m, n, device=device)
    capi.matmul(a, b, want)
    c = torch.full((m, n), float("nan"), device=device)
    assert ns.matmul(a, b, None, c) is c
    assert torch.equal(c, want)
    # and against an independent product of the same bf16 values in float64 (not only against the C ABI)
    exact_bf16 = a.double() @ b.double().T
    assert float(((c.double() - exact_bf16).abs() / exact_bf16.abs().clamp(min=1.0)).max()) <= 2e-6 * k / 32
    # the raw torch.ops symbol, on a stream of its own, with a C-input that aliases the output
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        acc = torch.ones(m, n, device=device)
        torch.ops.vecops_hip_t.matmul(a, b, acc, acc)
    side.synchronize()
    want2 = torch.empty(m, n, device=device)
    capi.matmul(a, b, want2, c_in=torch.ones(m, n, device=device))
    assert torch.equal(acc, want2)
    # fp32 operands: the ComputeType specialization picks the artifact (torch dtype or VecopsDType number)
    a32, b32 = torch.randn(64, 96, device=device), torch.randn(80, 96, device=device)
    c_bf, c_f32 = torch.empty(64, 80, device=device), torch.empty(64, 80, device=device)
    ns.matmul(a32, b32, None, c_bf)
    ns.matmul(a32, b32, None, c_f32, ComputeType=torch.float32)
    exact = a32.double() @ b32.double().T
    assert (c_f32.double() - exact).abs().max() < 1e-4 < (c_bf.double() - exact).abs().max()
    # split-K shape: the workspace comes from torch's allocator, its size is cached per signature
    a, b = _bf16(synth.uniform_pm1(3, (255, 8191)), device), _bf16(synth.uniform_pm1(4, (63, 8191)), device)
    c1, c2, want = (torch.empty(255, 63, device=device) for _ in range(3))
    ns.matmul(a, b, None, c1)
    ns.matmul(a, b, None, c2)
    capi.matmul(a, b, want)
    assert torch.equal(c1, want) and torch.equal(c2, want)


@pytest.mark.gpu
def test_torch_ops_quantised_operators(device, oracle):
    ns = tb.register_all("vecops_hip_t")
    m, n, k = 67, 129, 515
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    to = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(device)  # noqa: E731
    c = torch.zeros(m, n, device=device)
    ns.matmul_i8_dequant(to(a), to(b), to(rs), to(cs), None, c)
    want = oracle.matmul_i8_dequant(a, b, rs, cs)
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))
    # fused: dequantisation, silu, fp32 out; and requantisation to uint8
    acc = oracle.matmul_i8_dense(a, b)
    y = torch.zeros(m, n, device=device)
    ns.matmul_fused(to(a), to(b), None, to(rs), to(cs), 1, 1.0, 0.0, 0.0, 0.0, y)
    want_relu = oracle.fused_outputs(acc, np.float32, row_scales=rs, column_scales=cs, activation=1)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), want_relu.view(np.uint32))
    q = torch.zeros(m, n, dtype=torch.uint8, device=device)
    ns.matmul_fused(to(a), to(b), None, None, to(cs), 0, 0.5, 128, 0.0, 0.0, q)      # an int where a float goes
    assert np.array_equal(q.cpu().numpy(), oracle.fused_outputs(acc, np.uint8, column_scales=cs, scale=0.5, shift=128.0))
    # weight-only GEMV with the group size as a specialization value
    k, n = 512, 256
    x = synth.bf16_round(synth.normal(5, (2, k)))
    w = synth.int8_sym(6, (n, k))
    s = synth.scales(7, (n, k // 64))
    yb = torch.zeros(2, n, dtype=torch.bfloat16, device=device)
    ns.matmul_w8a16_group(torch.from_numpy(x.view(np.int16)).to(device).view(torch.bfloat16), to(w), to(s), yb, G=64)
    bits, exact = oracle.matmul_w8a16_group(x, w, s, 64)
    got = synth.bf16_to_f32(yb.view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)
    assert np.abs(got - exact).max() <= 2 ** -7 * np.abs(exact).max()


@pytest.mark.gpu
def test_torch_ops_runtime_quant(device, oracle):
    ns = tb.register_all("vecops_hip_t")
    to = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(device)  # noqa: E731
    m, n, k = 70, 130, 260
    mult = (np.float32(2.0) + synth.uniform_pm1(1, (m,))).astype(np.float32)
    a = ((synth.uniform_pm1(2, (m, k)) * np.float32(140.0) + np.float32(120.0)) / mult[:, None]).astype(np.float32)
    b = synth.int8_sym(3, (n, k))
    rs, cs = (np.float32(1.0) / mult).astype(np.float32), synth.scales(4, n)
    corr = (-9 * b.astype(np.int64).sum(axis=1)).astype(np.int32)
    acc = oracle.quantize_rows(a, mult, 9).astype(np.int64) @ b.astype(np.int64).T + corr
    want = oracle.fused_outputs(acc.astype(np.int32), np.float32, row_scales=rs, column_scales=cs)
    c = torch.zeros(m, n, device=device)
    assert ns.matmul_runtime_quant(to(a), to(b), to(mult), 9, to(rs), to(cs), to(corr), c) is c
    assert np.array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.gpu
def test_torch_ops_packed_b(device):
    """Pack once through torch.ops, multiply twice: int8 bit-equal to vecops::matmul on the unpacked operand, bf16
    equal up to the order of the fp32 sums (the packed kernel multiplies on another MFMA shape than the small tiles
    of the plain one) and bit-equal to the C ABI's packed product."""
    ns = tb.register_all("vecops_hip_t")
    to = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(device)  # noqa: E731
    m, n, k = 70, 300, 520
    a, b = to(synth.int8_sym(1, (m, k))), to(synth.int8_sym(2, (n, k)))
    packed = torch.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.I8, n, k), dtype=torch.uint8, device=device)
    comp = torch.zeros(n, dtype=torch.int32, device=device)
    outs = ns.matmul_pack_b(b, -3, packed, comp)
    assert outs[0] is packed and outs[1] is comp
    assert torch.equal(comp, (3 * b.to(torch.int64).sum(dim=1)).to(torch.int32))
    assert ns.matmul_pack_b(b, 0, packed, None) is packed                       # without the sidecar
    c, want = (torch.zeros(m, n, dtype=torch.int32, device=device) for _ in range(2))
    ns.matmul_packed_b(a, packed, None, c)
    ns.matmul(a, b, None, want)
    assert torch.equal(c, want)
    af, bf = _bf16(synth.uniform_pm1(3, (m, k)), device), _bf16(synth.uniform_pm1(4, (n, k)), device)
    pf = torch.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.BF16, n, k), dtype=torch.uint8, device=device)
    ns.matmul_pack_b(bf, 0, pf, None)
    cin = torch.from_numpy(synth.uniform_pm1(5, (m, n))).to(device)
    c1, c2 = torch.zeros(m, n, device=device), torch.zeros(m, n, device=device)
    ns.matmul_packed_b(af, pf, cin, c1)
    ns.matmul(af, bf, cin, c2)
    assert torch.allclose(c1, c2, rtol=0.0, atol=float(np.abs(c2.cpu().numpy()).max()) * 2e-6 * (k / 32))
    c3 = torch.zeros(m, n, device=device)
    capi.matmul_packed_b(af, capi.pack_b(bf), c3, c_in=cin)
    assert torch.equal(c1, c3)


@pytest.mark.gpu
def test_torch_ops_packed_a_and_unsigned_weights(device):
    """Side A and unsigned weights through torch.ops: pack A once, multiply by dense B; pack uint8 weights and announce
    them with PackedType - int32 sums exact against the plain operator."""
    ns = tb.register_all("vecops_hip_t")
    to = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(device)  # noqa: E731
    m, n, k = 300, 70, 520
    a, b = to(synth.int8_sym(1, (m, k))), to(synth.int8_sym(2, (n, k)))
    packed = torch.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.I8, m, k), dtype=torch.uint8, device=device)
    assert ns.matmul_pack_a(a, packed) is packed
    c, want = (torch.zeros(m, n, dtype=torch.int32, device=device) for _ in range(2))
    ns.matmul_packed_a(packed, b, None, c)
    ns.matmul(a, b, None, want)
    assert torch.equal(c, want)
    ub = to((synth.int8_sym(3, (n, k)).astype(np.int16) + 128).astype(np.uint8))
    pu = torch.zeros(capi.lib().vecops_hip_packed_b_bytes(capi.U8, n, k), dtype=torch.uint8, device=device)
    ns.matmul_pack_b(ub, 0, pu, None)
    ns.matmul_packed_b(a, pu, None, c, PackedType=torch.uint8)
    ns.matmul(a, ub, None, want)
    assert torch.equal(c, want)


@pytest.mark.gpu
def test_torch_ops_host_tensors_are_staged(device):
    ns = tb.register_all("vecops_hip_t")
    a = torch.from_numpy(synth.uniform_pm1(1, (33, 70)))
    b = torch.from_numpy(synth.uniform_pm1(2, (47, 70)))
    c = torch.zeros(33, 47)
    ns.matmul(a, b, None, c, ComputeType=torch.float32)
    assert (c.double() - a.double() @ b.double().T).abs().max() < 1e-4


@pytest.mark.gpu
def test_bridge_entry_on_device_tensors_with_its_own_scratch(device, oracle):
    """vecops_operator_bridge_invoke_v1 called directly (what a generated extension does): device tensors, no workspace
    in the call record - the bridge supplies the split-K scratch from its per-thread buffer - against the oracle; a
    caller-supplied workspace and the stream-ordered flag give the same bits."""
    host = H.HostLibrary()
    op = host.operator("vecops::matmul")
    for m, n, k in ((300, 260, 1000), (64, 48, 4099), (255, 63, 8191)):  # the last one splits K: it needs a workspace
        a, b = synth.bf16_round(synth.uniform_pm1(1, (m, k))), synth.bf16_round(synth.uniform_pm1(2, (n, k)))
        ta = torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
        tb_ = torch.from_numpy(b.view(np.int16)).to(device).view(torch.bfloat16)
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a, b, want, acc_f64=True)
        c = torch.full((m, n), float("nan"), device=device)
        frame = H.Frame([ta, tb_, None, c], outputs=(3,))
        torch.cuda.synchronize()
        op.bridge_invoke(frame)                                       # synchronous: the result is there on return
        got = c.cpu().numpy()
        assert np.max(np.abs(got - want) / np.maximum(1.0, np.abs(want))) <= 2e-6 * max(1.0, k / 32)
        need = op.workspace(frame)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
        c2 = torch.full((m, n), float("nan"), device=device)
        stream = torch.cuda.current_stream().cuda_stream
        op.bridge_invoke(H.Frame([ta, tb_, None, c2], outputs=(3,)), workspace=ws.data_ptr(), workspace_size=need,
                         stream=stream, stream_ordered=True)
        c3 = torch.full((m, n), float("nan"), device=device)
        op.bridge_invoke(H.Frame([ta, tb_, None, c3], outputs=(3,)), stream=stream, stream_ordered=True)   # bridge scratch: waits
        assert np.array_equal(c3.cpu().numpy(), got)
        torch.cuda.synchronize()
        assert np.array_equal(c2.cpu().numpy(), got)
    assert need > 0
    with pytest.raises(H.HostError) as e:                             # a workspace that is too small is refused, not used
        op.bridge_invoke(H.Frame([ta, tb_, None, c], outputs=(3,)), workspace=ws.data_ptr(), workspace_size=0)
    assert e.value.code != 0


@pytest.mark.gpu
def test_torch_ops_concurrent_callers_compile_and_the_oracle(device, oracle):
    """Callers on several host threads (python/tests/test_torch.py:125-134 of vecops), the operator inside a
    torch.compile'd function (:146-152), and - unlike the comparison with this library's own C ABI - every result
    against the CPU oracle."""
    from concurrent.futures import ThreadPoolExecutor
    ns = tb.register_all("vecops_hip_t")
    m, n, k = 200, 136, 520
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    tb_ = torch.from_numpy(b.view(np.int16)).to(device).view(torch.bfloat16)

    def expected(a):
        want = np.zeros((m, n), np.float32)
        oracle.matmul(a, b, want, acc_f64=True)
        return want

    inputs = [synth.bf16_round(synth.uniform_pm1(10 + i, (m, k))) for i in range(4)]

    def threaded_call(i):
        ta = torch.from_numpy(inputs[i].view(np.int16)).to(device).view(torch.bfloat16)
        out = torch.full((m, n), float("nan"), device=device)
        for _ in range(5):
            ns.matmul(ta, tb_, None, out)
        torch.cuda.synchronize()
        return out.cpu().numpy()

    with ThreadPoolExecutor(max_workers=4) as executor:
        results = list(executor.map(threaded_call, range(4)))
    for i, got in enumerate(results):
        want = expected(inputs[i])
        assert np.max(np.abs(got - want) / np.maximum(1.0, np.abs(want))) <= 2e-6 * max(1.0, k / 32), i

    ta = torch.from_numpy(inputs[0].view(np.int16)).to(device).view(torch.bfloat16)

    def compiled_call(x, w, destination):
        torch.ops.vecops_hip_t.matmul(x, w, None, destination)
        return destination

    compiled = torch.compile(compiled_call, backend="eager", fullgraph=True)
    out = torch.full((m, n), float("nan"), device=device)
    assert compiled(ta, tb_, out) is out
    torch.cuda.synchronize()
    want = expected(inputs[0])
    assert np.max(np.abs(out.cpu().numpy() - want) / np.maximum(1.0, np.abs(want))) <= 2e-6 * max(1.0, k / 32)
    # fake-tensor propagation of the registered operator (schema, Meta kernel, aliasing of the output)
    torch.library.opcheck(torch.ops.vecops_hip_t.matmul.default, (ta, tb_, None, torch.empty(m, n, device=device)),
                          test_utils=("test_schema", "test_faketensor"))
