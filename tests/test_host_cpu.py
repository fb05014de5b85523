"""The C++ host layer without a GPU: ABI layout, artifact loading, schema
validation, dispatch, provider behaviour and error mapping - the checks vecops
runs against its fake backend in tests/runtime/RuntimeTest.cpp:302-347,468,
502-506,557-562, here against the real HIP artifacts (whose run() stops at
"no HIP device" on a host without one).  Every test runs against the restated
runtime and, where oracle/_ref holds it, against the plug-in compiled into the
vecops tree's own runtime."""
import ctypes as C
import os
import shutil
import subprocess
import threading

import numpy as np
import pytest

from vecops_amd import host_api as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# the same plug-in compiled against the reference's own runtime sources (a checker build: oracle/Makefile, target ref)
UPSTREAM_LIB = os.path.join(H.ROOT, "oracle", "_ref", "libvecops_hip_host_upstream.so")
FLAVORS = [H.HOST_LIB] + ([UPSTREAM_LIB] if os.path.exists(UPSTREAM_LIB) else [])


@pytest.fixture(scope="module", params=FLAVORS, ids=lambda p: "upstream" if "upstream" in p else "restated")
def host(request):
    return H.HostLibrary(request.param)


def bf16(shape):
    return np.zeros(shape, np.uint16)


ABI_PROBE = r"""
#include <stdio.h>
#include <stddef.h>
#include HEADER_CALL
#include HEADER_KERNEL
#define S(T) printf(#T " %zu\n", sizeof(T))
#define O(T, F) printf(#T "." #F " %zu\n", offsetof(T, F))
int main(void) {
  S(VecopsError); O(VecopsError, code); O(VecopsError, message); O(VecopsError, message_capacity); O(VecopsError, message_required);
  S(VecopsTensorView); O(VecopsTensorView, data); O(VecopsTensorView, byte_offset); O(VecopsTensorView, device_type);
  O(VecopsTensorView, device_index); O(VecopsTensorView, dtype); O(VecopsTensorView, rank); O(VecopsTensorView, sizes);
  O(VecopsTensorView, strides); O(VecopsTensorView, flags);
  S(VecopsScalar); O(VecopsScalar, dtype); O(VecopsScalar, value);
  S(VecopsValue); O(VecopsValue, kind); O(VecopsValue, value);
  S(VecopsExecutionContext); O(VecopsExecutionContext, requested_threads); O(VecopsExecutionContext, stream);
  O(VecopsExecutionContext, user_data); O(VecopsExecutionContext, flags); O(VecopsExecutionContext, workspace_provider);
  O(VecopsExecutionContext, thread_pool); O(VecopsExecutionContext, allocation_observer);
  S(VecopsCall); O(VecopsCall, num_values); O(VecopsCall, values); O(VecopsCall, workspace); O(VecopsCall, workspace_size);
  O(VecopsCall, context);
  S(VecopsDimensionConstraint); O(VecopsDimensionConstraint, kind); O(VecopsDimensionConstraint, value);
  O(VecopsDimensionConstraint, lower_bound); O(VecopsDimensionConstraint, upper_bound); O(VecopsDimensionConstraint, alignment);
  S(VecopsTensorParameter); O(VecopsTensorParameter, dtype_mask); O(VecopsTensorParameter, device_type);
  O(VecopsTensorParameter, device_index); O(VecopsTensorParameter, rank); O(VecopsTensorParameter, optional);
  O(VecopsTensorParameter, dimension_constraint_stride); O(VecopsTensorParameter, sizes); O(VecopsTensorParameter, strides);
  O(VecopsTensorParameter, required_flags);
  S(VecopsScalarParameter); S(VecopsParameterDescriptor); O(VecopsParameterDescriptor, kind); O(VecopsParameterDescriptor, name);
  O(VecopsParameterDescriptor, constraint);
  S(VecopsKernelDescriptorV1); O(VecopsKernelDescriptorV1, abi_version_major); O(VecopsKernelDescriptorV1, abi_version_minor);
  O(VecopsKernelDescriptorV1, operator_name); O(VecopsKernelDescriptorV1, specialization_key);
  O(VecopsKernelDescriptorV1, num_parameters); O(VecopsKernelDescriptorV1, parameter_stride); O(VecopsKernelDescriptorV1, parameters);
  O(VecopsKernelDescriptorV1, workspace); O(VecopsKernelDescriptorV1, run); O(VecopsKernelDescriptorV1, flags);
  printf("enum %d %d %d %d %d %d %d %d\n", VECOPS_STATUS_EXECUTION_ERROR, VECOPS_DEVICE_PRIVATE, VECOPS_DTYPE_BF16,
         VECOPS_DTYPE_F32, VECOPS_DTYPE_I8, VECOPS_VALUE_TENSOR, (int)VECOPS_TENSOR_WRITE, VECOPS_DIM_DYNAMIC);
  printf("symbol %s %u %u\n", VECOPS_KERNEL_QUERY_SYMBOL_V1, VECOPS_KERNEL_ABI_VERSION_MAJOR, VECOPS_KERNEL_ABI_VERSION_MINOR);
  return 0;
}
"""


def _probe(tmp_path, tag, include_dir, call_header, kernel_header):
    src = tmp_path / f"probe_{tag}.c"
    src.write_text(ABI_PROBE)
    exe = tmp_path / f"probe_{tag}"
    subprocess.run(["gcc", "-I", include_dir, f'-DHEADER_CALL="{call_header}"', f'-DHEADER_KERNEL="{kernel_header}"',
                    str(src), "-o", str(exe)], check=True)
    return subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout


def test_abi_layout(tmp_path):
    ours = _probe(tmp_path, "ours", os.path.join(ROOT, "vecops_amd", "host", "include"), "vecops_rt/abi.h",
                  "vecops_rt/abi.h")
    facts = dict(line.rsplit(" ", 1) for line in ours.splitlines() if not line.startswith(("enum", "symbol")))
    for name, size in H.ABI_SIZES.items():
        assert int(facts[name]) == size == C.sizeof({"VecopsTensorView": H.TensorView, "VecopsScalar": H.Scalar,
                                                     "VecopsValue": H.Value,
                                                     "VecopsExecutionContext": H.ExecutionContext}[name])
    assert "symbol vecops_kernel_query_v1 1 1" in ours
    assert "enum 6 255 11 12 2 1 2 2" in ours
    if os.path.isdir("/root/reference/include/vecops/runtime"):
        # byte-for-byte the same layout as vecops' own runtime/CallAbi.h and runtime/KernelAbi.h
        theirs = _probe(tmp_path, "ref", "/root/reference/include", "vecops/runtime/CallAbi.h",
                        "vecops/runtime/KernelAbi.h")
        assert ours == theirs


def test_host_library_exports_every_declared_symbol(host):
    import ctypes
    import re
    text = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include",
                             "vecops_hip_host.h")).read()
    names = sorted(set(re.findall(r"VECOPS_HIP_HOST_EXPORT[^;(]*?\b(vecops_(?:hip_host|operator_bridge)_\w+)\s*\(", text)))
    assert len(names) == 10 and "vecops_operator_bridge_invoke_v1" in names
    lib = ctypes.CDLL(H.HOST_LIB)
    for name in names:
        assert getattr(lib, name) is not None
    for name in ("vecops::matmul", "vecops::matmul_fused", "vecops::matmul_i8_dequant", "vecops::matmul_runtime_quant",
                 "vecops::matmul_pack_b", "vecops::matmul_packed_b", "vecops::matmul_w8a16_group"):
        assert host.operator(name) is not None
    with pytest.raises(Exception):
        host.operator("vecops::no_such_operator")


def test_every_artifact_loads_with_its_key(host):
    files = sorted(os.listdir(H.ARTIFACT_DIR))
    assert len(files) == 102  # 40 + (8 required families x {bf16, i8} + 15 unsigned-weight, side-A and fp32-pack kinds) x {host, device}
    for f in files:
        name, key = host.load_artifact(os.path.join(H.ARTIFACT_DIR, f))
        assert key.startswith(name + ";") and key.endswith(";backend=hip-gfx950")
        assert f == "".join(ch if (ch.isalnum() or ch in "_.=-") else "_" for ch in key) + ".so"
    # exactly one exported symbol of ours per artifact
    out = subprocess.run(["nm", "-D", "--defined-only", os.path.join(H.ARTIFACT_DIR, files[0])], capture_output=True,
                         text=True).stdout
    assert [l.split()[-1] for l in out.splitlines() if " T " in l] == ["vecops_kernel_query_v1"]


def test_loader_error_mapping(host, tmp_path):
    with pytest.raises(H.HostError) as e:       # unloadable -> LoadError (Executable.cpp:208-218)
        host.load_artifact(str(tmp_path / "missing.so"))
    assert e.value.code == 5
    with pytest.raises(H.HostError) as e:       # a DSO without the query symbol -> AbiMismatch (:219-229)
        host.load_artifact(os.path.join(ROOT, "oracle", "libvecops_oracle.so"))
    assert e.value.code == 4 and "vecops_kernel_query_v1" in e.value.message


def test_resolve_picks_recipe_by_dtype_and_placement(host):
    op = host.operator("vecops::matmul")
    a32, b32, c32 = np.zeros((4, 8), np.float32), np.zeros((5, 8), np.float32), np.zeros((4, 5), np.float32)
    assert op.resolve(H.Frame([a32, b32, None, c32], outputs=(3,))) == \
        "vecops::matmul;operands=f32;compute=bf16;memory=host;backend=hip-gfx950"
    assert op.resolve(H.Frame([bf16((4, 8)), bf16((5, 8)), None, c32], outputs=(3,))) == \
        "vecops::matmul;operands=bf16;compute=bf16;memory=host;backend=hip-gfx950"
    ah, bh = np.zeros((4, 8), np.float16), np.zeros((5, 8), np.float16)
    for ch in (c32, np.zeros((4, 5), np.float16)):          # half operands write fp32 or half
        assert op.resolve(H.Frame([ah, bh, None, ch], outputs=(3,))) == \
            "vecops::matmul;operands=f16;compute=f16;memory=host;backend=hip-gfx950"
    with pytest.raises(H.HostError) as e:                   # ... not bf16
        op.resolve(H.Frame([ah, bh, None, bf16((4, 5))], outputs=(3,)))
    assert e.value.code in (2, 3)
    ai, bi, ci = np.zeros((4, 8), np.int8), np.zeros((5, 8), np.int8), np.zeros((4, 5), np.int32)
    assert op.resolve(H.Frame([ai, bi, None, ci], outputs=(3,))) == \
        "vecops::matmul;operands=i8;compute=i32;memory=host;backend=hip-gfx950"
    dev = lambda dtype, shape: {"data": 0x10000, "dtype": dtype, "shape": shape,  # noqa: E731
                                "strides": (shape[-1], 1) if len(shape) == 2 else (shape[1] * shape[2], shape[2], 1),
                                "device_type": H.DEVICE_PRIVATE}
    f = H.Frame([dev(H.BF16, (2, 4, 8)), dev(H.BF16, (2, 5, 8)), None, dev(H.BF16, (2, 4, 5))], outputs=(3,))
    assert op.resolve(f) == "vecops::matmul;operands=bf16;compute=bf16;memory=device;backend=hip-gfx950"
    # explicit ComputeType specialization (bf16 is what the x86 reference path computes in)
    assert "compute=bf16" in op.resolve(H.Frame([a32, b32, None, c32], outputs=(3,)), {"ComputeType": ("dtype", H.BF16)})
    # true fp32 compute (the SME_F32F32 atom) is a specialization of its own
    assert op.resolve(H.Frame([a32, b32, None, c32], outputs=(3,)), {"ComputeType": ("dtype", H.F32)}) == \
        "vecops::matmul;operands=f32;compute=f32;memory=host;backend=hip-gfx950"
    with pytest.raises(H.HostError) as e:       # bf16 operands cannot ask for fp32 compute
        op.resolve(H.Frame([bf16((8, 16)), bf16((8, 16)), None, np.zeros((8, 8), np.float32)], outputs=(3,)),
                   {"ComputeType": ("dtype", H.F32)})
    assert e.value.code in (2, 3)
    w = host.operator("vecops::matmul_w8a16_group")
    x, wq, s, y = bf16((4, 256)), np.zeros((8, 256), np.int8), np.zeros((8, 2), np.float32), bf16((4, 8))
    assert w.resolve(H.Frame([x, wq, s, y], outputs=(3,))) == \
        "vecops::matmul_w8a16_group;G=128;memory=host;backend=hip-gfx950"
    s4 = np.zeros((8, 4), np.float32)
    assert "G=64" in w.resolve(H.Frame([x, wq, s4, y], outputs=(3,)), {"G": 64})
    with pytest.raises(H.HostError) as e:       # valid call, no artifact for G=32 -> NotFound from the provider
        w.resolve(H.Frame([x, wq, np.zeros((8, 8), np.float32), y], outputs=(3,)), {"G": 32})
    assert e.value.code == 3


def test_family_specialization_is_part_of_the_key(host):
    """`Family` on vecops::matmul: the kernel family the call requires (vecops' family_selection::Require<F> is part
    of MatmulConfig, i.e. of the specialization); each family has artifacts of its own for bf16 and 8-bit operands."""
    op = host.operator("vecops::matmul")
    a, b, c = bf16((4, 8)), bf16((5, 8)), np.zeros((4, 5), np.float32)
    names = {1: "tile_256", 2: "tile_128", 3: "tile_64", 4: "skinny", 6: "tile_256x128", 7: "tile_128x256", 8: "tile_256x352",
             9: "tile_192"}
    for code, name in names.items():
        assert op.resolve(H.Frame([a, b, None, c], outputs=(3,)), {"Family": code}) == \
            f"vecops::matmul;operands=bf16;compute=bf16;family={name};memory=host;backend=hip-gfx950"
    ai, bi, ci = np.zeros((4, 8), np.int8), np.zeros((5, 8), np.uint8), np.zeros((4, 5), np.int32)
    assert op.resolve(H.Frame([ai, bi, None, ci], outputs=(3,)), {"Family": 2}) == \
        "vecops::matmul;operands=i8;compute=i32;family=tile_128;memory=host;backend=hip-gfx950"
    # 0 = automatic: the plain artifact
    assert "family" not in op.resolve(H.Frame([a, b, None, c], outputs=(3,)), {"Family": 0})
    for bad in (5, 10, -1):                      # zero_k, unknown numbers: nothing a caller can require
        with pytest.raises(H.HostError) as e:
            op.resolve(H.Frame([a, b, None, c], outputs=(3,)), {"Family": bad})
        assert e.value.code in (1, 2, 3)
    a32, b32, c32 = np.zeros((4, 8), np.float32), np.zeros((5, 8), np.float32), np.zeros((4, 5), np.float32)
    with pytest.raises(H.HostError) as e:        # fp32 operands: no such artifacts
        op.resolve(H.Frame([a32, b32, None, c32], outputs=(3,)), {"Family": 2})
    assert e.value.code in (2, 3)


def test_schema_validation(host):
    op = host.operator("vecops::matmul")
    c = np.zeros((4, 5), np.float32)
    ok = [bf16((4, 8)), bf16((5, 8)), None, c]
    op.resolve(H.Frame(ok, outputs=(3,)))
    cases = [
        ([bf16((4, 8)), bf16((5, 9)), None, c], "K"),                            # K mismatch
        ([bf16((4, 8)), bf16((5, 8)), None, np.zeros((4, 6), np.float32)], "c must be"),
        ([bf16((4, 8)), bf16((5, 8)), np.zeros((4, 6), np.float32), c], "c_in"),
        ([bf16((2, 4, 8)), bf16((3, 5, 8)), None, np.zeros((2, 4, 5), np.float32)], "batch"),
        ([bf16((4, 8)), bf16((2, 5, 8)), None, c], "rank"),
        ([bf16((4, 8)), bf16((5, 8)), None, None], "not optional"),
        ([bf16((4, 8)), bf16((5, 8)), c], "expects 4 arguments"),
        ([np.zeros((4, 8), np.int32), bf16((5, 8)), None, c], "dtype"),
    ]
    for args, needle in cases:
        with pytest.raises(H.HostError) as e:
            op.resolve(H.Frame(args, outputs=(len(args) - 1,)))
        assert e.value.code == 1 and needle in e.value.message, (needle, e.value.message)
    with pytest.raises(H.HostError) as e:       # output without write access
        op.resolve(H.Frame(ok, outputs=()))
    assert e.value.code == 1 and "access" in e.value.message
    with pytest.raises(H.HostError) as e:       # operand dtypes no recipe takes
        op.resolve(H.Frame([bf16((4, 8)), np.zeros((5, 8), np.int8), None, c], outputs=(3,)))
    assert e.value.code in (2, 3)
    deq = host.operator("vecops::matmul_i8_dequant")
    a, b = np.zeros((4, 8), np.int8), np.zeros((5, 8), np.int8)
    with pytest.raises(H.HostError) as e:
        deq.resolve(H.Frame([a, b, np.zeros(3, np.float32), np.zeros(5, np.float32), None, c], outputs=(5,)))
    assert e.value.code == 1 and "row_scales" in e.value.message


def test_fused_operator_resolution_and_validation(host):
    """vecops::matmul_fused: eleven positional values (five of them scalars), one artifact per operand class."""
    op = host.operator("vecops::matmul_fused")
    c = np.zeros((4, 5), np.float32)
    scalars = [1, 1.0, 0.0, 0.0, 0.0]                      # activation relu, no scale, no shift, clamp bounds unused
    frame = lambda a, b, cin, rs, cs, out, sc=scalars: H.Frame([a, b, cin, rs, cs] + sc + [out], outputs=(10,))  # noqa: E731
    assert op.resolve(frame(bf16((4, 8)), bf16((5, 8)), None, None, None, c)) == \
        "vecops::matmul_fused;operands=bf16;memory=host;backend=hip-gfx950"
    f32 = np.zeros((4, 8), np.float32)
    assert "operands=f32" in op.resolve(frame(f32, np.zeros((5, 8), np.float32), None, None, None, c))
    assert "operands=f16" in op.resolve(frame(np.zeros((4, 8), np.float16), np.zeros((5, 8), np.float16), None, None,
                                              None, np.zeros((4, 5), np.float16)))
    a8, b8 = np.zeros((4, 8), np.int8), np.zeros((5, 8), np.int8)
    bias = np.zeros((4, 5), np.int32)
    for out in (c, np.zeros((4, 5), np.uint8), np.zeros((4, 5), np.int8)):
        assert op.resolve(frame(a8, b8, bias, np.zeros(4, np.float32), np.zeros(5, np.float32), out)) == \
            "vecops::matmul_fused;operands=i8;memory=host;backend=hip-gfx950"
    bad = [
        (frame(a8, b8, None, np.zeros(3, np.float32), None, c), 1, "row_scales"),
        (frame(a8, b8, None, None, np.zeros(6, np.float32), c), 1, "column_scales"),
        (frame(a8, b8, None, None, None, c, [7, 1.0, 0.0, 0.0, 0.0]), 1, "activation"),
        (frame(a8, b8, None, None, None, c, [1.5, 1.0, 0.0, 0.0, 0.0]), 1, "activation"),      # a float where an int goes
        (frame(bf16((4, 8)), bf16((5, 9)), None, None, None, c), 1, "K"),
    ]
    for fr, code, needle in bad:
        with pytest.raises(H.HostError) as e:
            op.resolve(fr)
        assert e.value.code == code and needle in e.value.message, (needle, e.value.message)
    with pytest.raises(H.HostError) as e:                  # int32 sums cannot leave as bf16: no recipe takes it
        op.resolve(frame(a8, b8, None, None, None, bf16((4, 5))))
    assert e.value.code in (2, 3)
    with pytest.raises(H.HostError) as e:                  # bf16 sums cannot leave as bytes
        op.resolve(frame(bf16((4, 8)), bf16((5, 8)), None, None, None, np.zeros((4, 5), np.uint8)))
    assert e.value.code in (2, 3)


def test_packed_b_operators_resolution_and_validation(host):
    """vecops::matmul_pack_b / vecops::matmul_packed_b: the packed operand is an opaque byte tensor; the pack's
    class follows the source dtype, the multiply's class follows a."""
    pack = host.operator("vecops::matmul_pack_b")
    packed = np.zeros(4096, np.uint8)
    comp = np.zeros(5, np.int32)
    pf = lambda b, zp, p, c: H.Frame([b, zp, p, c], outputs=(2, 3))  # noqa: E731
    assert pack.resolve(pf(bf16((5, 8)), 0, packed, None)) == \
        "vecops::matmul_pack_b;operands=bf16;memory=host;backend=hip-gfx950"
    assert "operands=bf16" in pack.resolve(pf(np.zeros((5, 8), np.float32), 0, packed, None))   # rounded while packing
    assert pack.resolve(pf(np.zeros((5, 8), np.int8), 3, packed, comp)) == \
        "vecops::matmul_pack_b;operands=i8;memory=host;backend=hip-gfx950"
    for fr, needle in [(pf(bf16((5, 8)), 0, packed, comp), "int8"),
                       (pf(np.zeros((5, 8), np.int8), 3, packed, np.zeros(4, np.int32)), "N entries"),
                       (pf(np.zeros((5, 8), np.int8), 1.5, packed, None), "a_zero_point")]:
        with pytest.raises(H.HostError) as e:
            pack.resolve(fr)
        assert e.value.code == 1 and needle in e.value.message, (needle, e.value.message)
    assert pack.resolve(pf(np.zeros((5, 8), np.float16), 0, packed, None)) == \
        "vecops::matmul_pack_b;operands=f16;memory=host;backend=hip-gfx950"        # half operands: a recipe of their own
    assert pack.resolve(pf(np.zeros((5, 8), np.uint8), 0, packed, None)) == \
        "vecops::matmul_pack_b;operands=u8;memory=host;backend=hip-gfx950"         # unsigned weights (AMX_I8I32<.., uint8_t>)
    with pytest.raises(H.HostError) as e:                  # the compensated pack is the signed-weights atom's
        pack.resolve(pf(np.zeros((5, 8), np.uint8), 3, packed, comp))
    assert e.value.code == 1 and "int8" in e.value.message

    mul = host.operator("vecops::matmul_packed_b")
    mf = lambda a, cin, c: H.Frame([a, packed, cin, c], outputs=(3,))  # noqa: E731
    c = np.zeros((4, 5), np.float32)
    assert mul.resolve(mf(bf16((4, 8)), None, c)) == "vecops::matmul_packed_b;operands=bf16;memory=host;backend=hip-gfx950"
    assert "operands=bf16" in mul.resolve(mf(bf16((2, 4, 8)), None, bf16((2, 4, 5))))
    assert "operands=f32" in mul.resolve(mf(np.zeros((4, 8), np.float32), c, c))
    assert "operands=i8" in mul.resolve(mf(np.zeros((4, 8), np.int8), None, np.zeros((4, 5), np.int32)))
    assert "operands=i8" in mul.resolve(mf(np.zeros((4, 8), np.uint8), None, np.zeros((4, 5), np.int32)))   # u8 x packed s8
    assert "operands=f16" in mul.resolve(mf(np.zeros((4, 8), np.float16), None, np.zeros((4, 5), np.float16)))
    with pytest.raises(H.HostError) as e:                  # half operands write fp32 or half, not bf16
        mul.resolve(mf(np.zeros((4, 8), np.float16), None, bf16((4, 5))))
    assert e.value.code in (2, 3)
    for fr, needle in [(mf(bf16((4, 8)), None, np.zeros((3, 5), np.float32)), "[.., M, N]"),
                       (mf(bf16((2, 4, 8)), None, np.zeros((3, 4, 5), np.float32)), "batch"),
                       (mf(bf16((4, 8)), np.zeros((4, 6), np.float32), c), "c_in")]:
        with pytest.raises(H.HostError) as e:
            mul.resolve(fr)
        assert e.value.code == 1 and needle in e.value.message, (needle, e.value.message)
    with pytest.raises(H.HostError) as e:                  # int32 sums do not leave as fp32 here
        mul.resolve(mf(np.zeros((4, 8), np.int8), None, c))
    assert e.value.code in (2, 3)
    # a packed tensor that is too small for N x K is refused by the artifact's workspace query
    with pytest.raises(H.HostError) as e:
        mul.workspace(H.Frame([bf16((4, 8)), np.zeros(16, np.uint8), None, c], outputs=(3,)))
    assert e.value.code == 1 and "bytes" in e.value.message
    # unsigned packed weights: the PackedType specialization value names what the opaque bytes hold
    i32 = np.zeros((4, 5), np.int32)
    u8 = {"PackedType": ("dtype", H.U8)}
    assert mul.resolve(mf(np.zeros((4, 8), np.int8), None, i32), u8) == \
        "vecops::matmul_packed_b;operands=i8;packed=u8;memory=host;backend=hip-gfx950"
    assert "packed=u8" in mul.resolve(mf(np.zeros((4, 8), np.uint8), None, i32), u8)
    assert "packed=" not in mul.resolve(mf(np.zeros((4, 8), np.int8), None, i32), {"PackedType": ("dtype", H.I8)})
    for fr, spec, needle in [(mf(bf16((4, 8)), None, c), u8, "8-bit"),
                             (mf(np.zeros((4, 8), np.int8), None, i32), {"PackedType": 3}, "DType")]:
        with pytest.raises(H.HostError) as e:
            mul.resolve(fr, spec)
        assert e.value.code == 1 and needle in e.value.message, (needle, e.value.message)


def test_fp32_compute_pack_resolution(host):
    """The pack of the fp32-compute atom (ops::MatmulPack over SME_F32F32): ComputeType = Float32 on the pack keeps an
    fp32 source's elements fp32, and on the product selects the recipe that multiplies in fp32; either side."""
    f32 = {"ComputeType": ("dtype", H.F32)}
    packed = np.zeros(4096, np.uint8)
    src = np.zeros((5, 8), np.float32)
    pack_b, pack_a = host.operator("vecops::matmul_pack_b"), host.operator("vecops::matmul_pack_a")
    assert pack_b.resolve(H.Frame([src, 0, packed, None], outputs=(2,)), f32) == \
        "vecops::matmul_pack_b;operands=f32;memory=host;backend=hip-gfx950"
    assert "operands=bf16" in pack_b.resolve(H.Frame([src, 0, packed, None], outputs=(2,)))
    assert "operands=bf16" in pack_b.resolve(H.Frame([src, 0, packed, None], outputs=(2,)), {"ComputeType": ("dtype", H.BF16)})
    assert pack_a.resolve(H.Frame([src, packed], outputs=(1,)), f32) == \
        "vecops::matmul_pack_a;operands=f32;memory=host;backend=hip-gfx950"
    assert "operands=bf16" in pack_b.resolve(H.Frame([bf16((5, 8)), 0, packed, None], outputs=(2,)), f32)   # bf16 stays bf16
    c = np.zeros((4, 5), np.float32)
    mul_b, mul_a = host.operator("vecops::matmul_packed_b"), host.operator("vecops::matmul_packed_a")
    assert mul_b.resolve(H.Frame([np.zeros((4, 8), np.float32), packed, None, c], outputs=(3,)), f32) == \
        "vecops::matmul_packed_b;operands=f32;compute=f32;memory=host;backend=hip-gfx950"
    assert mul_b.resolve(H.Frame([np.zeros((4, 8), np.float32), packed, None, c], outputs=(3,))) == \
        "vecops::matmul_packed_b;operands=f32;memory=host;backend=hip-gfx950"              # fp32 rows against a bf16 pack
    assert mul_a.resolve(H.Frame([packed, np.zeros((5, 8), np.float32), c, c], outputs=(3,)), f32) == \
        "vecops::matmul_packed_a;operands=f32;compute=f32;memory=host;backend=hip-gfx950"
    with pytest.raises(H.HostError) as e:                  # fp32 products leave as fp32
        mul_b.resolve(H.Frame([np.zeros((4, 8), np.float32), packed, None, bf16((4, 5))], outputs=(3,)), f32)
    assert e.value.code in (2, 3)


def test_packed_a_operators_resolution_and_validation(host):
    """vecops::matmul_pack_a / vecops::matmul_packed_a (ops::matmul_pack with Operand::A, ops/MatmulPack.h:81-96):
    the packed operand comes first, M is taken from c and K from b; every class of the B side has its mirror."""
    pack = host.operator("vecops::matmul_pack_a")
    packed = np.zeros(4096, np.uint8)
    pf = lambda a: H.Frame([a, packed], outputs=(1,))  # noqa: E731
    for src, name in [(bf16((5, 8)), "bf16"), (np.zeros((5, 8), np.float32), "bf16"), (np.zeros((5, 8), np.float16), "f16"),
                      (np.zeros((5, 8), np.int8), "i8"), (np.zeros((5, 8), np.uint8), "u8")]:
        assert pack.resolve(pf(src)) == f"vecops::matmul_pack_a;operands={name};memory=host;backend=hip-gfx950"
    with pytest.raises(H.HostError) as e:
        pack.resolve(pf(np.zeros((5, 8), np.int32)))
    assert e.value.code in (1, 2, 3)

    mul = host.operator("vecops::matmul_packed_a")
    mf = lambda b, cin, c: H.Frame([packed, b, cin, c], outputs=(3,))  # noqa: E731
    c = np.zeros((4, 5), np.float32)
    key = "vecops::matmul_packed_a;operands={};memory=host;backend=hip-gfx950"
    assert mul.resolve(mf(bf16((5, 8)), None, c)) == key.format("bf16")
    assert mul.resolve(mf(bf16((2, 5, 8)), None, bf16((2, 4, 5)))) == key.format("bf16")   # one packed a, every batch of b
    assert mul.resolve(mf(np.zeros((5, 8), np.float32), c, c)) == key.format("f32")
    assert mul.resolve(mf(np.zeros((5, 8), np.float16), None, np.zeros((4, 5), np.float16))) == key.format("f16")
    i32 = np.zeros((4, 5), np.int32)
    assert mul.resolve(mf(np.zeros((5, 8), np.int8), None, i32)) == key.format("i8")
    assert mul.resolve(mf(np.zeros((5, 8), np.uint8), None, i32)) == key.format("i8")       # s8-packed a x u8 b
    assert mul.resolve(mf(np.zeros((5, 8), np.int8), None, i32), {"PackedType": ("dtype", H.U8)}) == key.format("i8;packed=u8")
    for fr, needle in [(mf(bf16((5, 8)), None, np.zeros((4, 6), np.float32)), "[.., M, N]"),
                       (mf(bf16((2, 5, 8)), None, np.zeros((3, 4, 5), np.float32)), "batch"),
                       (mf(bf16((5, 8)), np.zeros((3, 5), np.float32), c), "c_in")]:
        with pytest.raises(H.HostError) as e:
            mul.resolve(fr)
        assert e.value.code == 1 and needle in e.value.message, (needle, e.value.message)
    with pytest.raises(H.HostError) as e:                  # int32 sums do not leave as fp32 here
        mul.resolve(mf(np.zeros((5, 8), np.int8), None, c))
    assert e.value.code in (2, 3)
    with pytest.raises(H.HostError) as e:                  # too small for M x K
        mul.workspace(H.Frame([np.zeros(16, np.uint8), bf16((5, 8)), None, c], outputs=(3,)))
    assert e.value.code == 1 and "bytes" in e.value.message


def test_runtime_quant_operator_resolution_and_validation(host):
    """vecops::matmul_runtime_quant: eight positional values, the zero point a scalar in the middle."""
    op = host.operator("vecops::matmul_runtime_quant")
    a, b, c = np.zeros((4, 8), np.float32), np.zeros((5, 8), np.int8), np.zeros((4, 5), np.float32)
    m4, n5 = np.ones(4, np.float32), np.ones(5, np.float32)
    fr = lambda *v: H.Frame(list(v), outputs=(7,))  # noqa: E731
    assert op.resolve(fr(a, b, m4, 7, m4, n5, None, c)) == \
        "vecops::matmul_runtime_quant;operands=f32_i8;epilogue=row_col_dequant;memory=host;backend=hip-gfx950"
    assert op.resolve(fr(a, b, m4, 7, m4, n5, np.zeros(5, np.int32), c)).startswith("vecops::matmul_runtime_quant;")
    for frame, needle in [(fr(a, b, np.ones(3, np.float32), 7, m4, n5, None, c), "multipliers"),
                          (fr(a, b, m4, 7, m4, np.ones(6, np.float32), None, c), "column_scales"),
                          (fr(a, b, m4, 7, m4, n5, np.zeros(4, np.int32), c), "correction"),
                          (fr(a, b, m4, 7.5, m4, n5, None, c), "zero_point"),
                          (fr(a, np.zeros((5, 9), np.int8), m4, 7, m4, n5, None, c), "K")]:
        with pytest.raises(H.HostError) as e:
            op.resolve(frame)
        assert e.value.code == 1 and needle in e.value.message, (needle, e.value.message)
    with pytest.raises(H.HostError) as e:                  # activations that are already bytes go to vecops::matmul_fused
        op.resolve(fr(np.zeros((4, 8), np.uint8), b, m4, 7, m4, n5, None, c))
    assert e.value.code in (1, 2, 3)


def test_provider_without_artifacts_reports_not_found(host, tmp_path):
    op = host.operator("vecops::matmul", str(tmp_path))
    with pytest.raises(H.HostError) as e:
        op.resolve(H.Frame([bf16((4, 8)), bf16((5, 8)), None, np.zeros((4, 5), np.float32)], outputs=(3,)))
    assert e.value.code == 3 and "no HIP artifact" in e.value.message


def test_artifact_with_the_wrong_key_is_rejected(host, tmp_path):
    """A file in the bf16 slot that is really the int8 artifact: the provider (and
    Operator.cpp:250-253 behind it) must refuse it with AbiMismatch (RuntimeTest.cpp:502-506)."""
    bf = "vecops__matmul_operands=bf16_compute=bf16_memory=host_backend=hip-gfx950.so"
    i8 = "vecops__matmul_operands=i8_compute=i32_memory=host_backend=hip-gfx950.so"
    shutil.copy(os.path.join(H.ARTIFACT_DIR, i8), tmp_path / bf)
    op = host.operator("vecops::matmul", str(tmp_path))
    with pytest.raises(H.HostError) as e:
        op.resolve(H.Frame([bf16((4, 8)), bf16((5, 8)), None, np.zeros((4, 5), np.float32)], outputs=(3,)))
    assert e.value.code == 4


def test_concurrent_resolution(host):
    """Provider thread-safety (RuntimeTest.cpp:512-547): many threads resolving the same and different keys."""
    op = host.operator("vecops::matmul")
    frames = [H.Frame([bf16((4, 8)), bf16((5, 8)), None, np.zeros((4, 5), np.float32)], outputs=(3,)),
              H.Frame([np.zeros((4, 8), np.int8), np.zeros((5, 8), np.int8), None, np.zeros((4, 5), np.int32)],
                      outputs=(3,))]
    keys, errors = [], []

    def work(i):
        try:
            for _ in range(20):
                keys.append(op.resolve(frames[i % 2]))
        except Exception as exc:  # pragma: no cover
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(8)]
    [t.start() for t in threads]
    [t.join() for t in threads]
    assert not errors and len(keys) == 160 and len(set(keys)) == 2


def test_invoke_without_a_gpu_is_an_execution_error(host):
    """On a host with no HIP device the artifact's run() reports
    VECOPS_STATUS_EXECUTION_ERROR through VecopsError; nothing falls back to the CPU."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    op = host.operator("vecops::matmul")
    c = np.full((4, 5), 7.0, np.float32)
    with pytest.raises(H.HostError) as e:
        op.invoke(H.Frame([bf16((4, 8)), bf16((5, 8)), None, c], outputs=(3,)))
    assert e.value.code == 6 and "no HIP device" in e.value.message
    assert (c == 7.0).all()


def test_bridge_records_have_the_reference_layout(tmp_path):
    """VecopsSpecializationArgument and the bridge entry's prototype (runtime/OperatorBridgeAbi.h) as restated in
    vecops_rt/abi.h: same sizes and offsets as vecops' own header, and the ctypes mirror agrees."""
    probe = r"""
#include <stddef.h>
#include <stdio.h>
#include HEADER
int main(void) {
  printf("%zu %zu %zu %zu %zu %u %u\n", sizeof(VecopsSpecializationArgument), offsetof(VecopsSpecializationArgument, kind),
         offsetof(VecopsSpecializationArgument, name), offsetof(VecopsSpecializationArgument, value), sizeof(VecopsCall),
         (unsigned)VECOPS_SPECIALIZATION_CONST_INT, (unsigned)VECOPS_SPECIALIZATION_DTYPE);
  int32_t (*entry)(uint64_t, const VecopsCall*, uint32_t, const VecopsSpecializationArgument*, VecopsError*) =
      vecops_operator_bridge_invoke_v1;
  return entry == 0;
}
"""
    def run(tag, include_dir, header):
        src = tmp_path / f"bridge_{tag}.c"
        src.write_text(probe)
        obj = tmp_path / f"bridge_{tag}.o"
        # compile only: the prototype must accept the assignment; the numbers come from a second, linkable program
        subprocess.run(["gcc", "-c", "-I", include_dir, f'-DHEADER="{header}"', str(src), "-o", str(obj)], check=True)
        src2 = tmp_path / f"bridge_{tag}_sizes.c"
        src2.write_text(probe.replace("vecops_operator_bridge_invoke_v1;", "0;").replace("return entry == 0;", "return entry != 0;"))
        exe = tmp_path / f"bridge_{tag}_sizes"
        subprocess.run(["gcc", "-I", include_dir, f'-DHEADER="{header}"', str(src2), "-o", str(exe)], check=True)
        return subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    ours = run("ours", os.path.join(ROOT, "vecops_amd", "host", "include"), "vecops_rt/abi.h")
    sizes = [int(v) for v in ours.split()]
    assert sizes[0] == C.sizeof(H.SpecializationArgument) and sizes[3] == H.SpecializationArgument.value.offset
    assert sizes[4] == C.sizeof(H.Call) and sizes[5:] == [1, 2]
    if os.path.isdir("/root/reference/include/vecops/runtime"):
        assert ours == run("ref", "/root/reference/include", "vecops/runtime/OperatorBridgeAbi.h")


def test_bridge_entry_validates_handles_and_records(host):
    """vecops_operator_bridge_invoke_v1 without a GPU: unknown and stale handles, malformed records and schema errors
    come back as status codes with the message in the caller's VecopsError (python/bindings/module.cpp:1223-1239)."""
    op = host.operator("vecops::matmul")
    a, b, c = bf16((4, 8)), bf16((5, 8)), np.zeros((4, 5), np.float32)
    frame = H.Frame([a, b, None, c], outputs=(3,))
    with pytest.raises(H.HostError) as e:
        op.bridge_invoke(frame, handle=987654321)
    assert e.value.code == 1 and "handle" in e.value.message
    handle = op.bridge_handle()
    assert handle != 0 and op.bridge_handle() == handle
    with pytest.raises(H.HostError) as e:                      # K differs: the schema's relation validator, through the bridge
        op.bridge_invoke(H.Frame([a, bf16((5, 9)), None, c], outputs=(3,)))
    assert e.value.code == 1 and "K" in e.value.message
    with pytest.raises(H.HostError) as e:                      # an unknown specialization kind
        sp = (H.SpecializationArgument * 1)()
        sp[0].struct_size, sp[0].kind, sp[0].name = C.sizeof(H.SpecializationArgument), 7, b"ComputeType"
        call = H.Call(C.sizeof(H.Call), len(frame.values), C.cast(frame.values, C.c_void_p), None, 0, None)
        msg = C.create_string_buffer(256)
        err = H.Error(C.sizeof(H.Error), 0, C.cast(msg, C.c_void_p), 256, 0)
        rc = host.lib.vecops_operator_bridge_invoke_v1(handle, C.byref(call), 1, sp, C.byref(err))
        assert rc == 1 and err.code == 1 and err.message_required == len(msg.value) + 1
        raise H.HostError(rc, msg.value.decode())
    assert "specialization" in e.value.message
    short = H.Call(8, 0, None, None, 0, None)                   # a call record shorter than the ABI's
    assert host.lib.vecops_operator_bridge_invoke_v1(handle, C.byref(short), 0, None, None) == 1
    # a handle dies with its registration and is never handed out again
    host.lib.vecops_hip_host_bridge_unregister(handle)
    with pytest.raises(H.HostError) as e:
        op.bridge_invoke(frame, handle=handle)
    assert e.value.code == 1
    op._bridge = 0
    assert op.bridge_handle() > handle
