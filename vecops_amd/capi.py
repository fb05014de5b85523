"""ctypes binding of ``libvecops_hip.so`` (``include/vecops_hip.h``).

There is no CPU fallback: loading fails loudly when the HIP library has not been
built, and every call goes to the GPU kernels.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libvecops_hip.so")

# VecopsDType numbers
I8, U8, I32, F16, BF16, F32, F64 = 2, 3, 6, 10, 11, 12, 13
COMPUTE_BF16, COMPUTE_F32 = 0, 1
FAMILY_NAMES = {0: "none", 1: "tile_256", 2: "tile_128", 3: "tile_64", 4: "skinny", 5: "zero_k", 6: "tile_256x128",
                7: "tile_128x256", 8: "tile_256x352", 9: "tile_192"}
STATUS_NAMES = {0: "Ok", 1: "InvalidArgument", 2: "NotApplicable", 3: "NotFound", 4: "AbiMismatch", 5: "LoadError",
                6: "ExecutionError", 7: "InternalError"}

EXPORTS = [
    "vecops_hip_abi_version", "vecops_hip_last_error", "vecops_hip_device_count", "vecops_hip_plan_matmul",
    "vecops_hip_matmul", "vecops_hip_matmul_planned", "vecops_hip_matmul_i8_dequant", "vecops_hip_matmul_i8_dequant_workspace",
    "vecops_hip_matmul_w8a16_group", "vecops_hip_packed_b_bytes", "vecops_hip_pack_b", "vecops_hip_pack_b_compensated",
    "vecops_hip_pack_as", "vecops_hip_plan_matmul_packed_b", "vecops_hip_matmul_packed_b", "vecops_hip_matmul_i8_dequant_packed_b",
    "vecops_hip_plan_matmul_fused", "vecops_hip_matmul_fused", "vecops_hip_quantize_rows",
    "vecops_hip_matmul_runtime_quant_workspace", "vecops_hip_matmul_runtime_quant",
    "vecops_hip_matmul_runtime_quant_packed_b_workspace", "vecops_hip_matmul_runtime_quant_packed_b",
    "vecops_hip_static_workspace_bytes", "vecops_hip_matmul_static_workspace",
    "vecops_hip_mfma_stream_ops", "vecops_hip_mfma_stream",
    "vecops_hip_mfma_stream_shape_ops", "vecops_hip_mfma_stream_shape", "vecops_hip_read_stream",
    "vecops_hip_plan_matmul_family", "vecops_hip_matmul_family",
    "vecops_hip_matmul_runtime_quant_batched_workspace", "vecops_hip_matmul_runtime_quant_batched",
    "vecops_hip_matmul_grouped_workspace", "vecops_hip_matmul_grouped",
    "vecops_hip_pack_a", "vecops_hip_plan_matmul_packed_a", "vecops_hip_matmul_packed_a",
    "vecops_hip_matmul_packed_ab_workspace", "vecops_hip_matmul_packed_ab",
]

ACT_NONE, ACT_RELU, ACT_CLAMP, ACT_SIGMOID, ACT_SILU = 0, 1, 2, 3, 4
ACTIVATIONS = {None: ACT_NONE, "none": ACT_NONE, "relu": ACT_RELU, "clamp": ACT_CLAMP, "sigmoid": ACT_SIGMOID,
               "silu": ACT_SILU}
EPILOGUE_SCALE, EPILOGUE_SHIFT = 1, 2


class Operand(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_uint32), ("rank", C.c_uint32), ("sizes", C.c_int64 * 3),
                ("strides", C.c_int64 * 3)]


class Plan(C.Structure):
    _fields_ = [("family", C.c_uint32), ("split_k", C.c_uint32), ("vector_a", C.c_uint32), ("vector_b", C.c_uint32),
                ("b_layout", C.c_uint32), ("peeled_columns", C.c_uint32), ("workspace_bytes", C.c_uint64)]


class Epilogue(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("activation", C.c_uint32), ("flags", C.c_uint32), ("scale", C.c_float),
                ("shift", C.c_float), ("clamp_lo", C.c_float), ("clamp_hi", C.c_float), ("row_scales", C.c_void_p),
                ("column_scales", C.c_void_p)]


class FamilyRequest(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("selection", C.c_uint32), ("family", C.c_uint32), ("split_k", C.c_uint32)]


SELECT_AUTOMATIC, SELECT_PREFER, SELECT_REQUIRE = 0, 1, 2
FAMILY_CODES = {name: code for code, name in FAMILY_NAMES.items()}


def family_request(family, selection=SELECT_REQUIRE, split_k: int = 0) -> FamilyRequest:
    """`family`: a name of FAMILY_NAMES or its number; the counterpart of family_selection::Require<F> / Prefer<F>."""
    r = FamilyRequest()
    r.struct_size = C.sizeof(FamilyRequest)
    r.selection = selection
    r.family = FAMILY_CODES[family] if isinstance(family, str) else int(family)
    r.split_k = split_k
    return r


class VecopsHipError(RuntimeError):
    def __init__(self, code: int, message: str) -> None:
        super().__init__(f"{STATUS_NAMES.get(code, code)}: {message}")
        self.code = code


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with vecops_amd.build.build_all() "
                               "(there is no CPU fallback for the HIP path)")
        L = C.CDLL(LIB_PATH)
        L.vecops_hip_abi_version.restype = C.c_uint32
        L.vecops_hip_last_error.restype = C.c_char_p
        L.vecops_hip_device_count.restype = C.c_int32
        P = C.POINTER(Operand)
        L.vecops_hip_plan_matmul.argtypes = [P, P, P, P, C.c_uint32, C.POINTER(Plan)]
        L.vecops_hip_matmul.argtypes = [P, P, P, P, C.c_uint32, C.c_void_p, C.c_uint64, C.c_void_p]
        L.vecops_hip_static_workspace_bytes.restype = C.c_uint64
        R = C.POINTER(FamilyRequest)
        L.vecops_hip_plan_matmul_family.argtypes = [P, P, P, P, C.c_uint32, R, C.POINTER(Plan)]
        L.vecops_hip_matmul_family.argtypes = [P, P, P, P, C.c_uint32, R, C.c_void_p, C.c_uint64, C.c_void_p]
        L.vecops_hip_matmul_planned.argtypes = [P, P, P, P, C.c_uint32, C.POINTER(Plan), C.c_void_p, C.c_uint64, C.c_void_p]
        L.vecops_hip_mfma_stream_ops.restype = C.c_uint64
        L.vecops_hip_mfma_stream_ops.argtypes = [C.c_uint32, C.c_int32, C.c_int32]
        L.vecops_hip_mfma_stream.argtypes = [C.c_uint32, C.c_void_p, C.c_uint64, C.c_int32, C.c_int32, C.c_void_p,
                                             C.c_void_p]
        L.vecops_hip_mfma_stream_shape_ops.restype = C.c_uint64
        L.vecops_hip_mfma_stream_shape_ops.argtypes = [C.c_uint32, C.c_uint32, C.c_int32, C.c_int32]
        L.vecops_hip_mfma_stream_shape.argtypes = [C.c_uint32, C.c_uint32, C.c_void_p, C.c_uint64, C.c_int32, C.c_int32,
                                                   C.c_void_p, C.c_void_p]
        L.vecops_hip_read_stream.argtypes = [C.c_void_p, C.c_uint64, C.c_int32, C.c_void_p, C.c_void_p]
        L.vecops_hip_matmul_static_workspace.argtypes = [P, P, P, P, C.c_uint32, C.c_void_p]
        L.vecops_hip_matmul_i8_dequant.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p,
                                                   C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64,
                                                   C.c_int64, C.c_int64, C.c_void_p, C.c_uint64, C.c_void_p]
        L.vecops_hip_matmul_i8_dequant_workspace.restype = C.c_uint64
        L.vecops_hip_matmul_i8_dequant_workspace.argtypes = [C.c_int64] * 3
        L.vecops_hip_matmul_w8a16_group.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p,
                                                    C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                                                    C.c_int64, C.c_void_p]
        L.vecops_hip_packed_b_bytes.restype = C.c_uint64
        L.vecops_hip_packed_b_bytes.argtypes = [C.c_uint32, C.c_int64, C.c_int64]
        L.vecops_hip_pack_b.argtypes = [P, C.c_void_p, C.c_uint64, C.c_void_p]
        L.vecops_hip_pack_b_compensated.argtypes = [P, C.c_int32, C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]
        L.vecops_hip_pack_as.argtypes = [P, C.c_uint32, C.c_void_p, C.c_uint64, C.c_void_p]
        L.vecops_hip_plan_matmul_packed_b.argtypes = [P, C.c_uint32, C.c_int64, P, P, C.POINTER(Plan)]
        L.vecops_hip_matmul_packed_b.argtypes = [P, C.c_void_p, C.c_uint32, C.c_int64, P, P, C.c_void_p, C.c_uint64,
                                                 C.c_void_p]
        L.vecops_hip_matmul_i8_dequant_packed_b.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p,
                                                            C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64,
                                                            C.c_int64, C.c_void_p, C.c_uint64, C.c_void_p]
        E = C.POINTER(Epilogue)
        L.vecops_hip_quantize_rows.argtypes = [P, C.c_void_p, C.c_int32, P, C.c_void_p]
        L.vecops_hip_matmul_runtime_quant_workspace.restype = C.c_uint64
        L.vecops_hip_matmul_runtime_quant_workspace.argtypes = [P, P, P]
        L.vecops_hip_matmul_runtime_quant.argtypes = [P, C.c_void_p, C.c_int32, P, C.c_void_p, C.c_void_p, C.c_void_p, P,
                                                      C.c_void_p, C.c_uint64, C.c_void_p]
        L.vecops_hip_matmul_runtime_quant_packed_b_workspace.restype = C.c_uint64
        L.vecops_hip_matmul_runtime_quant_packed_b_workspace.argtypes = [P, C.c_int64, P]
        L.vecops_hip_matmul_runtime_quant_packed_b.argtypes = [P, C.c_void_p, C.c_int32, C.c_void_p, C.c_int64, C.c_void_p,
                                                               C.c_void_p, C.c_void_p, P, C.c_void_p, C.c_uint64,
                                                               C.c_void_p]
        L.vecops_hip_matmul_runtime_quant_batched_workspace.restype = C.c_uint64
        L.vecops_hip_matmul_runtime_quant_batched_workspace.argtypes = [P, C.c_int64, P, C.c_int64, P]
        L.vecops_hip_matmul_runtime_quant_batched.argtypes = [P, C.c_void_p, C.c_int32, C.c_int64, P, C.c_void_p, C.c_int64,
                                                              C.c_void_p, C.c_void_p, P, C.c_void_p, C.c_uint64, C.c_void_p]
        L.vecops_hip_pack_a.argtypes = [P, C.c_void_p, C.c_uint64, C.c_void_p]
        L.vecops_hip_plan_matmul_packed_a.argtypes = [C.c_uint32, C.c_int64, P, P, P, C.POINTER(Plan)]
        L.vecops_hip_matmul_packed_a.argtypes = [C.c_void_p, C.c_uint32, C.c_int64, P, P, P, C.c_void_p, C.c_uint64,
                                                 C.c_void_p]
        L.vecops_hip_matmul_packed_ab_workspace.restype = C.c_uint64
        L.vecops_hip_matmul_packed_ab_workspace.argtypes = [C.c_uint32, C.c_int64, C.c_uint32, C.c_int64, C.c_int64, P, P]
        L.vecops_hip_matmul_packed_ab.argtypes = [C.c_void_p, C.c_uint32, C.c_int64, C.c_void_p, C.c_uint32, C.c_int64,
                                                  C.c_int64, P, P, C.c_void_p, C.c_uint64, C.c_void_p]
        L.vecops_hip_matmul_grouped_workspace.restype = C.c_uint64
        L.vecops_hip_matmul_grouped_workspace.argtypes = [C.c_uint32, P, P, P, P, C.c_uint32]
        L.vecops_hip_matmul_grouped.argtypes = [C.c_uint32, P, P, P, P, C.c_uint32, C.c_void_p, C.c_uint64, C.c_void_p]
        L.vecops_hip_plan_matmul_fused.argtypes = [P, P, P, P, C.c_uint32, E, C.POINTER(Plan)]
        L.vecops_hip_matmul_fused.argtypes = [P, P, P, P, C.c_uint32, E, C.c_void_p, C.c_uint64, C.c_void_p]
        _lib = L
    return _lib


def _check(rc: int) -> None:
    if rc != 0:
        raise VecopsHipError(rc, lib().vecops_hip_last_error().decode())


def _torch_dtype_code(t) -> int:
    import torch
    return {torch.int8: I8, torch.uint8: U8, torch.int32: I32, torch.float16: F16, torch.bfloat16: BF16,
            torch.float32: F32, torch.float64: F64}[t.dtype]


def operand(t) -> Operand:
    """Describe a torch tensor (rank 2 or 3, any strides) living in device memory."""
    o = Operand()
    o.data = t.data_ptr()
    o.dtype = _torch_dtype_code(t)
    o.rank = t.dim()
    for i in range(t.dim()):
        o.sizes[i] = t.shape[i]
        o.strides[i] = t.stride(i)
    return o


def _stream_handle(stream) -> int:
    import torch
    s = stream if stream is not None else torch.cuda.current_stream()
    return s.cuda_stream


def plan_matmul(a, b, c, c_in=None, compute=COMPUTE_BF16) -> Plan:
    plan = Plan()
    oa, ob, oc = operand(a), operand(b), operand(c)
    oi = operand(c_in) if c_in is not None else None
    _check(lib().vecops_hip_plan_matmul(C.byref(oa), C.byref(ob), C.byref(oi) if oi is not None else None,
                                        C.byref(oc), compute, C.byref(plan)))
    return plan


def matmul(a, b, c, c_in=None, compute=COMPUTE_BF16, workspace=None, stream=None):
    """c[..,M,N] = c_in + a[..,M,K] . b[..,N,K]^T on the GPU; returns c.

    Mirrors ``ops::matmul(config)(workspace, m, n, k, A, B[, Cin], C)``: the caller
    allocates the output; a workspace tensor is allocated here when the plan needs
    one and none is passed.  Such a workspace comes from torch's allocator, which orders its reuse on torch's CURRENT
    stream: pass ``stream`` only when it is that stream (the default), or pass a workspace of your own that outlives
    the work on the stream you name.
    """
    import torch
    plan = plan_matmul(a, b, c, c_in, compute)
    if plan.workspace_bytes and (workspace is None or workspace.numel() * workspace.element_size()
                                 < plan.workspace_bytes):
        workspace = torch.empty(plan.workspace_bytes, dtype=torch.uint8, device=c.device)
    oa, ob, oc = operand(a), operand(b), operand(c)
    oi = operand(c_in) if c_in is not None else None
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul(C.byref(oa), C.byref(ob), C.byref(oi) if oi is not None else None, C.byref(oc),
                                   compute, ws_ptr, ws_size, _stream_handle(stream)))
    return c


def matmul_planned(a, b, c, plan: Plan, c_in=None, compute=COMPUTE_BF16, workspace=None, stream=None):
    """``matmul`` with a plan made beforehand (``plan_matmul`` / ``plan_matmul_family`` on operands of the same
    metadata): ``vecops_hip_matmul_planned``."""
    import torch
    if plan.workspace_bytes and (workspace is None or workspace.numel() * workspace.element_size() < plan.workspace_bytes):
        workspace = torch.empty(plan.workspace_bytes, dtype=torch.uint8, device=c.device)
    oa, ob, oc = operand(a), operand(b), operand(c)
    oi = operand(c_in) if c_in is not None else None
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_planned(C.byref(oa), C.byref(ob), C.byref(oi) if oi is not None else None, C.byref(oc),
                                           compute, C.byref(plan), ws_ptr, ws_size, _stream_handle(stream)))
    return c


class PreparedMatmul:
    """``matmul`` on fixed operands with everything but the launch done once: the descriptors, the plan and the
    workspace are built here, a call is one foreign call (the counterpart of vecops' prepared invocation,
    ``ops::matmul(config).prepare(...)`` / docs/Runtime.md:196-206).  The tensors must stay alive and in place; the
    stream is the one that was current at preparation unless ``stream`` is given."""

    def __init__(self, a, b, c, c_in=None, compute=COMPUTE_BF16, workspace=None, stream=None):
        import torch
        self.plan = plan_matmul(a, b, c, c_in, compute)
        need = int(self.plan.workspace_bytes)
        if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
            workspace = torch.empty(need, dtype=torch.uint8, device=c.device)
        self._keep = (a, b, c, c_in, workspace)
        self._oa, self._ob, self._oc = operand(a), operand(b), operand(c)
        self._oi = operand(c_in) if c_in is not None else None
        ws_ptr = workspace.data_ptr() if workspace is not None else None
        ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
        self._args = (C.byref(self._oa), C.byref(self._ob), C.byref(self._oi) if self._oi is not None else None,
                      C.byref(self._oc), compute, C.byref(self.plan), ws_ptr, ws_size, _stream_handle(stream))
        self._fn = lib().vecops_hip_matmul_planned

    def __call__(self):
        rc = self._fn(*self._args)
        if rc != 0:
            _check(rc)
        return self._keep[2]


def plan_matmul_family(a, b, c, request: FamilyRequest, c_in=None, compute=COMPUTE_BF16) -> Plan:
    plan = Plan()
    oa, ob, oc = operand(a), operand(b), operand(c)
    oi = operand(c_in) if c_in is not None else None
    _check(lib().vecops_hip_plan_matmul_family(C.byref(oa), C.byref(ob), C.byref(oi) if oi is not None else None,
                                               C.byref(oc), compute, C.byref(request), C.byref(plan)))
    return plan


def matmul_family(a, b, c, request: FamilyRequest, c_in=None, compute=COMPUTE_BF16, workspace=None, stream=None):
    """``matmul`` on the kernel family the caller prefers or requires (``family_request``)."""
    import torch
    plan = plan_matmul_family(a, b, c, request, c_in, compute)
    if plan.workspace_bytes and (workspace is None or workspace.numel() * workspace.element_size()
                                 < plan.workspace_bytes):
        workspace = torch.empty(plan.workspace_bytes, dtype=torch.uint8, device=c.device)
    oa, ob, oc = operand(a), operand(b), operand(c)
    oi = operand(c_in) if c_in is not None else None
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_family(C.byref(oa), C.byref(ob), C.byref(oi) if oi is not None else None,
                                          C.byref(oc), compute, C.byref(request), ws_ptr, ws_size, _stream_handle(stream)))
    return c


def matmul_static_workspace(a, b, c, c_in=None, compute=COMPUTE_BF16, stream=None):
    """``matmul`` for callers that cannot allocate: split-K partials go to the library's own per-GPU buffer
    (``vecops_hip_matmul_static_workspace``); nothing is allocated here either."""
    oa, ob, oc = operand(a), operand(b), operand(c)
    oi = operand(c_in) if c_in is not None else None
    _check(lib().vecops_hip_matmul_static_workspace(C.byref(oa), C.byref(ob), C.byref(oi) if oi is not None else None,
                                                    C.byref(oc), compute, _stream_handle(stream)))
    return c


def mfma_stream(operands, workgroups: int, iters: int, out, stream=None, shape: int = 0) -> int:
    """Launches the matrix-core yardstick on the values of `operands` (bf16 or int8 tensor) with the 32x32 (shape 0) or
    the 16x16 (shape 1) matrix instructions; returns the operations (2 per multiply-add) the launch performs."""
    code = _torch_dtype_code(operands)
    _check(lib().vecops_hip_mfma_stream_shape(code, shape, operands.data_ptr(), operands.numel() * operands.element_size(),
                                              workgroups, iters, out.data_ptr(), _stream_handle(stream)))
    return lib().vecops_hip_mfma_stream_shape_ops(code, shape, workgroups, iters)


def read_stream(src, workgroups: int, out, stream=None) -> int:
    """Launches the read-only yardstick over the bytes of `src`; returns the bytes one launch reads."""
    nbytes = src.numel() * src.element_size() // 16 * 16
    _check(lib().vecops_hip_read_stream(src.data_ptr(), nbytes, workgroups, out.data_ptr(), _stream_handle(stream)))
    return nbytes


def epilogue(activation=None, scale=None, shift=None, row_scales=None, column_scales=None, clamp=(0.0, 0.0)) -> Epilogue:
    """The fused output transform of ``matmul_fused``: ``act(((v * row_scales[row]) * column_scales[col]) * scale
    + shift)`` on ``v = float(c_in + a . b^T)``; scale tensors are fp32 and live on the device."""
    e = Epilogue()
    e.struct_size = C.sizeof(Epilogue)
    e.activation = ACTIVATIONS[activation] if not isinstance(activation, int) else activation
    e.flags = (EPILOGUE_SCALE if scale is not None else 0) | (EPILOGUE_SHIFT if shift is not None else 0)
    e.scale = 0.0 if scale is None else scale
    e.shift = 0.0 if shift is None else shift
    e.clamp_lo, e.clamp_hi = clamp
    e.row_scales = row_scales.data_ptr() if row_scales is not None else None
    e.column_scales = column_scales.data_ptr() if column_scales is not None else None
    return e


def plan_matmul_fused(a, b, c, ep: Epilogue, c_in=None, compute=COMPUTE_BF16) -> Plan:
    plan = Plan()
    oa, ob, oc = operand(a), operand(b), operand(c)
    oi = operand(c_in) if c_in is not None else None
    _check(lib().vecops_hip_plan_matmul_fused(C.byref(oa), C.byref(ob), C.byref(oi) if oi is not None else None,
                                              C.byref(oc), compute, C.byref(ep), C.byref(plan)))
    return plan


def matmul_fused(a, b, c, ep: Epilogue, c_in=None, compute=COMPUTE_BF16, workspace=None, stream=None):
    """c = convert(transform(c_in + a . b^T)) with the output transform ``ep`` (see ``epilogue``) fused into the
    kernel's store; a bias is a ``c_in`` whose row stride is 0.  Mirrors ``tensor::output<Acc>(c, transform)``."""
    import torch
    plan = plan_matmul_fused(a, b, c, ep, c_in, compute)
    if plan.workspace_bytes and (workspace is None or workspace.numel() * workspace.element_size()
                                 < plan.workspace_bytes):
        workspace = torch.empty(plan.workspace_bytes, dtype=torch.uint8, device=c.device)
    oa, ob, oc = operand(a), operand(b), operand(c)
    oi = operand(c_in) if c_in is not None else None
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_fused(C.byref(oa), C.byref(ob), C.byref(oi) if oi is not None else None,
                                         C.byref(oc), compute, C.byref(ep), ws_ptr, ws_size, _stream_handle(stream)))
    return c


def matmul_i8_dequant(a, b, row_scales, column_scales, c, correction=None, workspace=None, stream=None):
    import torch
    m, k = a.shape
    n = b.shape[0]
    assert a.stride(1) == 1 and b.stride(1) == 1 and c.stride(1) == 1
    need = lib().vecops_hip_matmul_i8_dequant_workspace(m, n, k)
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=c.device)
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_i8_dequant(
        a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), row_scales.data_ptr(), column_scales.data_ptr(),
        correction.data_ptr() if correction is not None else None, c.data_ptr(), c.stride(0), m, n, k, ws_ptr,
        ws_size, _stream_handle(stream)))
    return c


def quantize_rows(x, multipliers, zero_point: int, q, stream=None):
    """q = u8(x * multipliers[row] + zero_point): vecops' per-row asymmetric quantisation of fp32 activations."""
    ox, oq = operand(x), operand(q)
    _check(lib().vecops_hip_quantize_rows(C.byref(ox), multipliers.data_ptr(), int(zero_point), C.byref(oq),
                                          _stream_handle(stream)))
    return q


def matmul_runtime_quant(a, multipliers, zero_point: int, b, row_scales, column_scales, c, correction=None,
                         workspace=None, stream=None):
    """c = dequantise(quantise(a) . b^T + correction): fp32 a quantised on the way in, int8 b, fp32 c."""
    import torch
    oa, ob, oc = operand(a), operand(b), operand(c)
    need = lib().vecops_hip_matmul_runtime_quant_workspace(C.byref(oa), C.byref(ob), C.byref(oc))
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=c.device)
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_runtime_quant(
        C.byref(oa), multipliers.data_ptr(), int(zero_point), C.byref(ob),
        correction.data_ptr() if correction is not None else None, row_scales.data_ptr(), column_scales.data_ptr(),
        C.byref(oc), ws_ptr, ws_size, _stream_handle(stream)))
    return c


def matmul_runtime_quant_batched(a, multipliers, zero_point: int, scale_batch_stride: int, b, row_scales, column_scales, c,
                                 correction=None, correction_batch_stride: int = 0, workspace=None, stream=None):
    """``matmul_runtime_quant`` on rank-3 operands with the batch strides of the scale vectors and of the correction
    rows given (vecops' ``batch_stride`` of the runtime quantise / dequantise transforms)."""
    import torch
    oa, ob, oc = operand(a), operand(b), operand(c)
    need = lib().vecops_hip_matmul_runtime_quant_batched_workspace(C.byref(oa), int(scale_batch_stride), C.byref(ob),
                                                                   int(correction_batch_stride), C.byref(oc))
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=c.device)
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_runtime_quant_batched(
        C.byref(oa), multipliers.data_ptr(), int(zero_point), int(scale_batch_stride), C.byref(ob),
        correction.data_ptr() if correction is not None else None, int(correction_batch_stride), row_scales.data_ptr(),
        column_scales.data_ptr(), C.byref(oc), ws_ptr, ws_size, _stream_handle(stream)))
    return c


def matmul_grouped(a_list, b_list, c_list, c_in_list=None, compute: int = 0, workspace=None, stream=None):
    """Several independent products ``c[i] = c_in[i] + a[i] . b[i]^T`` in one call (irregular batches): groups of
    one operand class (bf16, f16, int8, fp32) run as one launch.  ``c_in_list`` entries may be None."""
    import torch
    count = len(a_list)
    if not (len(b_list) == count and len(c_list) == count and (c_in_list is None or len(c_in_list) == count)):
        raise ValueError("matmul_grouped: lists differ in length")
    Operands = Operand * max(count, 1)
    oa, ob, oc = Operands(*map(operand, a_list)), Operands(*map(operand, b_list)), Operands(*map(operand, c_list))
    oi = None
    if c_in_list is not None:
        oi = Operands(*[operand(t) if t is not None else Operand() for t in c_in_list])
    need = lib().vecops_hip_matmul_grouped_workspace(count, oa, ob, oi, oc, compute)
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=c_list[0].device)
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_grouped(count, oa, ob, oi, oc, compute, ws_ptr, ws_size, _stream_handle(stream)))
    return c_list


class PreparedGrouped:
    """``matmul_grouped`` on fixed operands with the descriptors and the workspace built once: a call is one foreign
    call (the library plans the groups anew each time - they are a handful of integer comparisons a group).  The
    tensors must stay alive and in place."""

    def __init__(self, a_list, b_list, c_list, c_in_list=None, compute: int = 0, workspace=None, stream=None):
        import torch
        count = len(a_list)
        if not (len(b_list) == count and len(c_list) == count and (c_in_list is None or len(c_in_list) == count)):
            raise ValueError("matmul_grouped: lists differ in length")
        Operands = Operand * max(count, 1)
        self._oa, self._ob, self._oc = Operands(*map(operand, a_list)), Operands(*map(operand, b_list)), Operands(*map(operand, c_list))
        self._oi = None
        if c_in_list is not None:
            self._oi = Operands(*[operand(t) if t is not None else Operand() for t in c_in_list])
        need = lib().vecops_hip_matmul_grouped_workspace(count, self._oa, self._ob, self._oi, self._oc, compute)
        if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
            workspace = torch.empty(need, dtype=torch.uint8, device=c_list[0].device)
        self._keep = (a_list, b_list, c_list, c_in_list, workspace)
        ws_ptr = workspace.data_ptr() if workspace is not None else None
        ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
        self._args = (count, self._oa, self._ob, self._oi, self._oc, compute, ws_ptr, ws_size, _stream_handle(stream))
        self._fn = lib().vecops_hip_matmul_grouped

    def __call__(self):
        rc = self._fn(*self._args)
        if rc != 0:
            _check(rc)
        return self._keep[2]


def matmul_runtime_quant_packed_b(a, multipliers, zero_point: int, packed, row_scales, column_scales, c, correction=None,
                                  workspace=None, stream=None):
    """``matmul_runtime_quant`` against weights packed once by ``pack_b`` (int8)."""
    import torch
    oa, oc = operand(a), operand(c)
    need = lib().vecops_hip_matmul_runtime_quant_packed_b_workspace(C.byref(oa), packed.n, C.byref(oc))
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=c.device)
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_runtime_quant_packed_b(
        C.byref(oa), multipliers.data_ptr(), int(zero_point), packed.storage.data_ptr(), packed.n,
        correction.data_ptr() if correction is not None else None, row_scales.data_ptr(), column_scales.data_ptr(),
        C.byref(oc), ws_ptr, ws_size, _stream_handle(stream)))
    return c


def matmul_w8a16_group(x, w, scales, y, group: int, stream=None):
    m, k = x.shape
    n = w.shape[0]
    assert x.stride(1) == 1 and w.stride(1) == 1 and y.stride(1) == 1 and scales.is_contiguous()
    _check(lib().vecops_hip_matmul_w8a16_group(x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0),
                                               scales.data_ptr(), y.data_ptr(), y.stride(0), m, n, k, group,
                                               _stream_handle(stream)))
    return y


class PackedB:
    """A [N,K] operand (or, from ``pack_a``, an [M,K] one: ``n`` then counts its rows) in the packed layout of
    ``vecops_hip_pack_b``: ``storage`` (uint8 tensor), ``dtype`` (BF16, F16, I8 or U8), ``n`` and ``k`` - the counterpart
    of a tensor over ``matmul::packed_layout<Atom, Operand::B>``."""

    def __init__(self, storage, dtype: int, n: int, k: int) -> None:
        self.storage, self.dtype, self.n, self.k = storage, dtype, n, k


def pack_b(b, a_zero_point=None, stream=None, compute: int = 0):
    """Pack b ([N,K]; bf16, f16, f32, int8 or uint8) once for any number of ``matmul_packed_b`` calls.  An fp32 source
    is rounded to bf16 unless ``compute`` is ``COMPUTE_F32``, which keeps fp32 elements (the fp32-compute atom).

    With ``a_zero_point`` (int8 b only) also returns the int32[N] compensation row
    ``-a_zero_point * sum_k b[n,k]`` (``ops::matmul_pack_b_compensated``).
    """
    import torch
    n, k = b.shape
    dtype = (I8 if b.dtype == torch.int8 else U8 if b.dtype == torch.uint8 else F16 if b.dtype == torch.float16
             else F32 if b.dtype == torch.float32 and compute == COMPUTE_F32 else BF16)
    size = lib().vecops_hip_packed_b_bytes(dtype, n, k)
    storage = torch.empty(max(size, 16), dtype=torch.uint8, device=b.device)
    ob = operand(b)
    if a_zero_point is None:
        _check(lib().vecops_hip_pack_as(C.byref(ob), dtype, storage.data_ptr(), size, _stream_handle(stream)))
        return PackedB(storage, dtype, n, k)
    comp = torch.empty(n, dtype=torch.int32, device=b.device)
    _check(lib().vecops_hip_pack_b_compensated(C.byref(ob), a_zero_point, storage.data_ptr(), size, comp.data_ptr(),
                                               _stream_handle(stream)))
    return PackedB(storage, dtype, n, k), comp


def pack_a(a, stream=None, compute: int = 0) -> PackedB:
    """Pack a ([M,K]) for ``matmul_packed_a`` / ``matmul_packed_ab`` (``ops::matmul_pack`` with ``Operand::A``)."""
    return pack_b(a, stream=stream, compute=compute)


def matmul_packed_a(packed: PackedB, b, c, c_in=None, workspace=None, stream=None):
    """c[..,M,N] = c_in + A . b[..,N,K]^T with A packed by ``pack_a``; returns c."""
    import torch
    plan = Plan()
    ob, oc = operand(b), operand(c)
    oi = operand(c_in) if c_in is not None else None
    oi_ref = C.byref(oi) if oi is not None else None
    _check(lib().vecops_hip_plan_matmul_packed_a(packed.dtype, packed.n, C.byref(ob), oi_ref, C.byref(oc), C.byref(plan)))
    if plan.workspace_bytes and (workspace is None or workspace.numel() * workspace.element_size() < plan.workspace_bytes):
        workspace = torch.empty(plan.workspace_bytes, dtype=torch.uint8, device=c.device)
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_packed_a(packed.storage.data_ptr(), packed.dtype, packed.n, C.byref(ob), oi_ref,
                                            C.byref(oc), ws_ptr, ws_size, _stream_handle(stream)))
    return c


def matmul_packed_ab(packed_a: PackedB, packed_b: PackedB, c, c_in=None, workspace=None, stream=None):
    """c[M,N] = c_in + A . B^T with both operands packed (``pack_a``, ``pack_b``); returns c."""
    import torch
    if packed_a.k != packed_b.k:
        raise ValueError("matmul_packed_ab: the packed operands differ in K")
    oc = operand(c)
    oi = operand(c_in) if c_in is not None else None
    oi_ref = C.byref(oi) if oi is not None else None
    need = lib().vecops_hip_matmul_packed_ab_workspace(packed_a.dtype, packed_a.n, packed_b.dtype, packed_b.n, packed_a.k,
                                                       oi_ref, C.byref(oc))
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=c.device)
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_packed_ab(packed_a.storage.data_ptr(), packed_a.dtype, packed_a.n,
                                             packed_b.storage.data_ptr(), packed_b.dtype, packed_b.n, packed_a.k, oi_ref,
                                             C.byref(oc), ws_ptr, ws_size, _stream_handle(stream)))
    return c


def plan_matmul_packed_b(a, packed: PackedB, c, c_in=None) -> Plan:
    plan = Plan()
    oa, oc = operand(a), operand(c)
    oi = operand(c_in) if c_in is not None else None
    _check(lib().vecops_hip_plan_matmul_packed_b(C.byref(oa), packed.dtype, packed.n,
                                                 C.byref(oi) if oi is not None else None, C.byref(oc), C.byref(plan)))
    return plan


def matmul_packed_b(a, packed: PackedB, c, c_in=None, workspace=None, stream=None):
    """c[..,M,N] = c_in + a[..,M,K] . B^T with B packed by ``pack_b``; returns c."""
    import torch
    plan = plan_matmul_packed_b(a, packed, c, c_in)
    if plan.workspace_bytes and (workspace is None or workspace.numel() * workspace.element_size()
                                 < plan.workspace_bytes):
        workspace = torch.empty(plan.workspace_bytes, dtype=torch.uint8, device=c.device)
    oa, oc = operand(a), operand(c)
    oi = operand(c_in) if c_in is not None else None
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_packed_b(C.byref(oa), packed.storage.data_ptr(), packed.dtype, packed.n,
                                            C.byref(oi) if oi is not None else None, C.byref(oc), ws_ptr, ws_size,
                                            _stream_handle(stream)))
    return c


def matmul_i8_dequant_packed_b(a, packed: PackedB, row_scales, column_scales, c, correction=None, workspace=None,
                               stream=None):
    import torch
    m, k = a.shape
    n = packed.n
    assert a.stride(1) == 1 and c.stride(1) == 1 and packed.dtype == I8 and packed.k == k
    need = lib().vecops_hip_matmul_i8_dequant_workspace(m, n, k)
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=c.device)
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_size = workspace.numel() * workspace.element_size() if workspace is not None else 0
    _check(lib().vecops_hip_matmul_i8_dequant_packed_b(
        a.data_ptr(), a.stride(0), packed.storage.data_ptr(), row_scales.data_ptr(), column_scales.data_ptr(),
        correction.data_ptr() if correction is not None else None, c.data_ptr(), c.stride(0), m, n, k, ws_ptr,
        ws_size, _stream_handle(stream)))
    return c
