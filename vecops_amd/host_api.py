"""ctypes binding of the C++ host layer (``include/vecops_hip_host.h``): vecops
``Operator`` objects built from this repository's schema, recipes, dispatch policy
and HIP executable provider.  Used by the tests to drive the whole
Operator -> recipe -> provider -> Executable -> artifact DSO -> kernel path."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
HOST_LIB = os.path.join(HERE, "lib", "libvecops_hip_host.so")
ARTIFACT_DIR = os.path.join(HERE, "lib", "artifacts")

DEVICE_CPU, DEVICE_PRIVATE = 1, 255
READ, WRITE = 1, 2
I8, U8, I32, F16, BF16, F32 = 2, 3, 6, 10, 11, 12
I64, F64 = 8, 13


class TensorView(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("data", C.c_void_p), ("byte_offset", C.c_uint64),
                ("device_type", C.c_uint32), ("device_index", C.c_int32), ("dtype", C.c_uint32), ("rank", C.c_uint32),
                ("sizes", C.POINTER(C.c_int64)), ("strides", C.POINTER(C.c_int64)), ("flags", C.c_uint64)]


class ScalarStorage(C.Union):
    _fields_ = [("i64", C.c_int64), ("u64", C.c_uint64), ("f64", C.c_double)]


class Scalar(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("dtype", C.c_uint32), ("value", ScalarStorage)]


class _ValueUnion(C.Union):
    _fields_ = [("tensor", TensorView), ("scalar", Scalar)]


class Value(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("kind", C.c_uint32), ("value", _ValueUnion)]


class ExecutionContext(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("requested_threads", C.c_uint32), ("stream", C.c_void_p),
                ("user_data", C.c_void_p), ("flags", C.c_uint64), ("workspace_provider", C.c_void_p),
                ("thread_pool", C.c_void_p), ("allocation_observer", C.c_void_p)]


class Specialization(C.Structure):
    _fields_ = [("name", C.c_char_p), ("kind", C.c_int32), ("value", C.c_int64)]


# layout facts of vecops' runtime/CallAbi.h on LP64, checked by tests/test_host_cpu.py
ABI_SIZES = {"VecopsTensorView": 64, "VecopsScalar": 16, "VecopsValue": 72, "VecopsExecutionContext": 56}

_NP_CODES = {np.dtype(np.int8): I8, np.dtype(np.uint8): U8, np.dtype(np.int32): I32, np.dtype(np.float32): F32,
             np.dtype(np.float16): F16}


class SpecializationValue(C.Union):
    _fields_ = [("integer", C.c_int64), ("dtype", C.c_uint32)]


class SpecializationArgument(C.Structure):
    """VecopsSpecializationArgument of the process-local bridge (vecops runtime/OperatorBridgeAbi.h:44-57)."""
    _fields_ = [("struct_size", C.c_uint32), ("kind", C.c_uint32), ("name", C.c_char_p), ("value", SpecializationValue)]


class Call(C.Structure):
    """VecopsCall (vecops runtime/CallAbi.h): the positional values, the caller's workspace, the context."""
    _fields_ = [("struct_size", C.c_uint32), ("num_values", C.c_uint32), ("values", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_size", C.c_uint64), ("context", C.c_void_p)]


class Error(C.Structure):
    """VecopsError: code and a caller-owned message buffer."""
    _fields_ = [("struct_size", C.c_uint32), ("code", C.c_int32), ("message", C.c_void_p),
                ("message_capacity", C.c_size_t), ("message_required", C.c_size_t)]


class Frame:
    """Positional VecopsValue records for one call; keeps the size/stride arrays alive."""

    def __init__(self, args, outputs=()):
        self.values = (Value * len(args))()
        self._keep = []
        for i, arg in enumerate(args):
            v = self.values[i]
            v.struct_size = C.sizeof(Value)
            if arg is None:
                v.kind = 0
                continue
            if isinstance(arg, (int, float)) and not isinstance(arg, bool):   # scalar argument
                v.kind = 2
                v.value.scalar.struct_size = C.sizeof(Scalar)
                if isinstance(arg, int):
                    v.value.scalar.dtype, v.value.scalar.value.i64 = I64, arg
                else:
                    v.value.scalar.dtype, v.value.scalar.value.f64 = F64, arg
                continue
            v.kind = 1
            t = v.value.tensor
            t.struct_size = C.sizeof(TensorView)
            t.flags = READ | (WRITE if i in outputs else 0)
            if isinstance(arg, dict):          # explicit description
                t.data, t.dtype, t.device_type = arg["data"], arg["dtype"], arg.get("device_type", DEVICE_CPU)
                shape, strides = arg["shape"], arg["strides"]
                t.flags = arg.get("flags", t.flags)
            elif isinstance(arg, np.ndarray):
                t.data, t.device_type = arg.ctypes.data, DEVICE_CPU
                t.dtype = arg.view_dtype if hasattr(arg, "view_dtype") else _NP_CODES.get(arg.dtype, BF16)
                shape, strides = arg.shape, [s // arg.itemsize for s in arg.strides]
                self._keep.append(arg)
            else:                               # torch tensor, on the GPU or in host memory
                import torch
                on_host = arg.device.type == "cpu"
                t.data, t.device_type = arg.data_ptr(), (DEVICE_CPU if on_host else DEVICE_PRIVATE)
                t.device_index = 0 if on_host else (arg.device.index or 0)
                t.dtype = {torch.int8: I8, torch.uint8: U8, torch.int32: I32, torch.bfloat16: BF16,
                           torch.float32: F32, torch.float16: F16}[arg.dtype]
                shape, strides = tuple(arg.shape), tuple(arg.stride())
                self._keep.append(arg)
            t.rank = len(shape)
            sizes = (C.c_int64 * max(1, len(shape)))(*shape)
            strd = (C.c_int64 * max(1, len(shape)))(*strides)
            self._keep += [sizes, strd]
            t.sizes, t.strides = sizes, strd


# VECOPS_HIP_CONTEXT_STREAM_ORDERED: device-memory artifacts return once their kernels are enqueued on the stream
CONTEXT_STREAM_ORDERED = 1


class HostError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"status {code}: {message}")
        self.code, self.message = code, message


class HostLibrary:
    def __init__(self, path=HOST_LIB):
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with vecops_amd.build.build_all()")
        L = self.lib = C.CDLL(path)
        L.vecops_hip_host_operator_create.restype = C.c_void_p
        L.vecops_hip_host_operator_create.argtypes = [C.c_char_p, C.c_char_p]
        L.vecops_hip_host_operator_destroy.argtypes = [C.c_void_p]
        L.vecops_hip_host_runtime_flavor.restype = C.c_char_p
        common = [C.c_void_p, C.POINTER(Value), C.c_uint32, C.POINTER(Specialization), C.c_uint32]
        L.vecops_hip_host_operator_resolve.argtypes = common + [C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t]
        L.vecops_hip_host_operator_workspace.argtypes = common + [C.POINTER(C.c_uint64), C.c_char_p, C.c_size_t]
        L.vecops_hip_host_operator_invoke.argtypes = common + [C.c_void_p, C.c_uint64, C.POINTER(ExecutionContext),
                                                              C.c_char_p, C.c_size_t]
        L.vecops_hip_host_load_artifact.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t,
                                                    C.c_char_p, C.c_size_t]
        L.vecops_hip_host_bridge_register.restype = C.c_uint64
        L.vecops_hip_host_bridge_register.argtypes = [C.c_void_p]
        L.vecops_hip_host_bridge_unregister.argtypes = [C.c_uint64]
        L.vecops_operator_bridge_invoke_v1.argtypes = [C.c_uint64, C.POINTER(Call), C.c_uint32,
                                                       C.POINTER(SpecializationArgument), C.POINTER(Error)]

    def flavor(self) -> str:
        return self.lib.vecops_hip_host_runtime_flavor().decode()

    def operator(self, name: str, artifact_dir: str = ARTIFACT_DIR) -> "HostOperator":
        handle = self.lib.vecops_hip_host_operator_create(name.encode(), artifact_dir.encode())
        if not handle:
            raise ValueError(f"unknown operator {name}")
        return HostOperator(self, handle)

    def load_artifact(self, path: str):
        name, key, msg = C.create_string_buffer(256), C.create_string_buffer(512), C.create_string_buffer(1024)
        rc = self.lib.vecops_hip_host_load_artifact(path.encode(), name, 256, key, 512, msg, 1024)
        if rc != 0:
            raise HostError(rc, msg.value.decode())
        return name.value.decode(), key.value.decode()


def _bridge_specs(specializations):
    items = list((specializations or {}).items())
    arr = (SpecializationArgument * max(1, len(items)))()
    for i, (k, v) in enumerate(items):
        arr[i].struct_size = C.sizeof(SpecializationArgument)
        arr[i].name = k.encode()
        if isinstance(v, tuple):        # ("dtype", code)
            arr[i].kind, arr[i].value.dtype = 2, v[1]
        else:
            arr[i].kind, arr[i].value.integer = 1, int(v)
    return arr, len(items)


def _specs(specializations):
    items = list((specializations or {}).items())
    arr = (Specialization * max(1, len(items)))()
    for i, (k, v) in enumerate(items):
        arr[i].name = k.encode()
        if isinstance(v, tuple):        # ("dtype", code)
            arr[i].kind, arr[i].value = 1, v[1]
        else:
            arr[i].kind, arr[i].value = 0, int(v)
    return arr, len(items)


class HostOperator:
    def __init__(self, lib: HostLibrary, handle):
        self._lib, self._h = lib, handle

    def __del__(self):
        try:
            if getattr(self, "_bridge", 0):
                self._lib.lib.vecops_hip_host_bridge_unregister(self._bridge)
            self._lib.lib.vecops_hip_host_operator_destroy(self._h)
        except Exception:
            pass

    def bridge_handle(self) -> int:
        """Registers the operator with the process-local bridge (once) and returns its handle."""
        if not getattr(self, "_bridge", 0):
            self._bridge = self._lib.lib.vecops_hip_host_bridge_register(self._h)
            if not self._bridge:
                raise RuntimeError("bridge registration failed")
        return self._bridge

    def bridge_invoke(self, frame: Frame, specializations=None, workspace=None, workspace_size=0, stream=None,
                      handle=None, stream_ordered=False):
        """One foreign call through vecops_operator_bridge_invoke_v1: validation, dispatch, resolution, workspace
        (the bridge's own scratch when none is given) and the artifact's run callback, synchronous."""
        ctx = ExecutionContext()
        ctx.struct_size = C.sizeof(ExecutionContext)
        ctx.stream = stream
        ctx.flags = CONTEXT_STREAM_ORDERED if stream_ordered else 0
        call = Call(C.sizeof(Call), len(frame.values), C.cast(frame.values, C.c_void_p), workspace, workspace_size,
                    C.cast(C.pointer(ctx), C.c_void_p))
        msg = C.create_string_buffer(1024)
        err = Error(C.sizeof(Error), 0, C.cast(msg, C.c_void_p), 1024, 0)
        sp, n = _bridge_specs(specializations)
        rc = self._lib.lib.vecops_operator_bridge_invoke_v1(self.bridge_handle() if handle is None else handle,
                                                            C.byref(call), n, sp, C.byref(err))
        if rc != 0:
            raise HostError(rc, msg.value.decode())

    def resolve(self, frame: Frame, specializations=None) -> str:
        key, msg = C.create_string_buffer(512), C.create_string_buffer(1024)
        sp, n = _specs(specializations)
        rc = self._lib.lib.vecops_hip_host_operator_resolve(self._h, frame.values, len(frame.values), sp, n, key, 512,
                                                            msg, 1024)
        if rc != 0:
            raise HostError(rc, msg.value.decode())
        return key.value.decode()

    def workspace(self, frame: Frame, specializations=None) -> int:
        size, msg = C.c_uint64(0), C.create_string_buffer(1024)
        sp, n = _specs(specializations)
        rc = self._lib.lib.vecops_hip_host_operator_workspace(self._h, frame.values, len(frame.values), sp, n,
                                                              C.byref(size), msg, 1024)
        if rc != 0:
            raise HostError(rc, msg.value.decode())
        return size.value

    def invoke(self, frame: Frame, specializations=None, workspace=None, workspace_size=0, stream=None,
               stream_ordered=False):
        msg = C.create_string_buffer(1024)
        sp, n = _specs(specializations)
        ctx = ExecutionContext()
        ctx.struct_size = C.sizeof(ExecutionContext)
        ctx.stream = stream
        ctx.flags = CONTEXT_STREAM_ORDERED if stream_ordered else 0
        rc = self._lib.lib.vecops_hip_host_operator_invoke(self._h, frame.values, len(frame.values), sp, n, workspace,
                                                           workspace_size, C.byref(ctx), msg, 1024)
        if rc != 0:
            raise HostError(rc, msg.value.decode())
