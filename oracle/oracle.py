"""TEST INFRASTRUCTURE ONLY: ctypes access to the CPU checkers.

``Oracle``    - oracle/libvecops_oracle.so, the C restatement of the vecops matmul
                semantics (oracle/vecops_oracle.c).
``Reference`` - oracle/_ref/libvecops_ref.so, the real vecops CPU matmul compiled
                from its own sources (oracle/ref_harness.cpp); present only where
                it was built, usable only on an x86 host with AMX.

Only tests, the smoke check and the benchmark's CPU-baseline leg import this
module.  The product path never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

# VecopsDType numeric values (runtime/CallAbi.h:62-91)
I8, U8, I32, F16, BF16, F32, F64 = 2, 3, 6, 10, 11, 12, 13
ATOM_BF16F32, ATOM_F32F32, ATOM_I8I32, ATOM_F16F32, ATOM_F64F64 = 0, 1, 2, 3, 4
SHAPE_AMX_BF16, SHAPE_AMX_I8_SAME, SHAPE_AMX_I8_MIXED, SHAPE_SME_F16, SHAPE_SME_OTHER = range(5)


class _Tensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int32), ("rank", C.c_int32),
                ("sizes", C.c_int64 * 3), ("strides", C.c_int64 * 3)]


def _np_dtype_code(arr: np.ndarray, bf16: bool) -> int:
    if arr.dtype == np.float32:
        return F32
    if arr.dtype == np.float64:
        return F64
    if arr.dtype == np.float16:
        return F16
    if arr.dtype == np.uint16:
        return BF16 if bf16 else F16
    if arr.dtype == np.int8:
        return I8
    if arr.dtype == np.uint8:
        return U8
    if arr.dtype == np.int32:
        return I32
    raise TypeError(f"unsupported dtype {arr.dtype}")


def _tensor(arr: np.ndarray, bf16: bool = True) -> _Tensor:
    """Describe a numpy array (any strides, rank 2 or 3); uint16 arrays hold bf16 bits."""
    t = _Tensor()
    t.data = arr.ctypes.data
    t.dtype = _np_dtype_code(arr, bf16)
    t.rank = arr.ndim
    for i in range(arr.ndim):
        t.sizes[i] = arr.shape[i]
        assert arr.strides[i] % arr.itemsize == 0
        t.strides[i] = arr.strides[i] // arr.itemsize
    return t


def build_oracle() -> str:
    path = os.path.join(HERE, "libvecops_oracle.so")
    subprocess.run(["make", "-C", HERE, "-B", "all"], check=True, capture_output=True)
    return path


def build_reference() -> str | None:
    """Compile the real reference when its tree is present (build container only)."""
    if not os.path.isdir("/root/reference/include/vecops"):
        return None
    subprocess.run(["make", "-C", HERE, "ref"], check=True, capture_output=True)
    return os.path.join(HERE, "_ref", "libvecops_ref.so")


class Oracle:
    def __init__(self) -> None:
        path = os.path.join(HERE, "libvecops_oracle.so")
        if not os.path.exists(path):
            build_oracle()
        self.lib = C.CDLL(path)
        L = self.lib
        L.vo_bf16_from_f32.restype = C.c_uint16
        L.vo_bf16_from_f32.argtypes = [C.c_float]
        L.vo_f32_from_bf16.restype = C.c_float
        L.vo_f32_from_bf16.argtypes = [C.c_uint16]
        L.vo_f32_to_i32_sat.restype = C.c_int32
        L.vo_f32_to_i32_sat.argtypes = [C.c_float]
        L.vo_bf16_from_f32_array.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        L.vo_f16_from_f32_array.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        L.vo_f32_from_f16.restype = C.c_float
        L.vo_f32_from_f16.argtypes = [C.c_uint16]
        L.vo_matmul.argtypes = [C.POINTER(_Tensor)] * 4 + [C.c_int, C.c_int]
        L.vo_matmul_sampled.argtypes = [C.POINTER(_Tensor)] * 2 + [C.c_int, C.c_void_p, C.c_void_p, C.c_int64,
                                                                   C.c_void_p]
        L.vo_matmul_i8_dense.argtypes = [C.c_void_p] * 3 + [C.c_int64] * 3
        L.vo_matmul_i8_dequant.argtypes = [C.c_void_p] * 6 + [C.c_int64] * 3
        L.vo_matmul_w8a16_group.argtypes = [C.c_void_p] * 5 + [C.c_int64] * 4
        L.vo_fused_outputs.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_uint32,
                                       C.c_float, C.c_float, C.c_int, C.c_float, C.c_float, C.c_int, C.c_void_p]
        for name in ("vo_amx_small_vector_profitable", "vo_sme_small_vector_profitable"):
            getattr(L, name).argtypes = [C.c_int, C.c_int64, C.c_int64, C.c_int64]
        L.vo_quantize_rows_u8.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_int32, C.c_void_p,
                                          C.c_int64]
        L.vo_quantize_rows_u8.restype = None
        L.vo_small_area_profitable.argtypes = [C.c_int64] * 4
        L.vo_threads.restype = C.c_int
        L.vo_matmul_bf16_dense.argtypes = [C.c_void_p] * 4 + [C.c_int64] * 3
        L.vo_amx_residual_split_profitable.argtypes = [C.c_int64] * 3

    # -- conversions ---------------------------------------------------------
    def bf16_from_f32(self, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.shape, dtype=np.uint16)
        self.lib.vo_bf16_from_f32_array(x.ctypes.data, out.ctypes.data, x.size)
        return out

    def f16_from_f32(self, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.shape, dtype=np.uint16)
        self.lib.vo_f16_from_f32_array(x.ctypes.data, out.ctypes.data, x.size)
        return out

    @staticmethod
    def f32_from_bf16(bits: np.ndarray) -> np.ndarray:
        return (bits.astype(np.uint32) << 16).view(np.float32)

    # -- matmul --------------------------------------------------------------
    def matmul(self, a, b, c, cin=None, atom=ATOM_BF16F32, acc_f64=False, c_bf16=True):
        """c[...] = cin + a . b^T in place; arrays may be arbitrarily strided views."""
        ta, tb, tc = _tensor(a), _tensor(b), _tensor(c, c_bf16)
        tci = _tensor(cin, c_bf16) if cin is not None else None
        rc = self.lib.vo_matmul(C.byref(ta), C.byref(tb), C.byref(tci) if tci is not None else None, C.byref(tc),
                                atom, 1 if acc_f64 else 0)
        if rc != 0:
            raise ValueError("vo_matmul rejected the operand shapes")
        return c

    def matmul_sampled(self, a, b, rows, cols, atom=ATOM_BF16F32) -> np.ndarray:
        rows = np.ascontiguousarray(rows, dtype=np.int64)
        cols = np.ascontiguousarray(cols, dtype=np.int64)
        out = np.empty(rows.size, dtype=np.float64)
        ta, tb = _tensor(a), _tensor(b)
        rc = self.lib.vo_matmul_sampled(C.byref(ta), C.byref(tb), atom, rows.ctypes.data, cols.ctypes.data,
                                        rows.size, out.ctypes.data)
        if rc != 0:
            raise ValueError("vo_matmul_sampled rejected the operand shapes")
        return out

    def threads(self) -> int:
        return int(self.lib.vo_threads())

    def matmul_bf16_dense(self, a_bits: np.ndarray, b_bits: np.ndarray, out_bf16: bool = False) -> np.ndarray:
        """Vectorised all-core bf16 product on dense operands (CPU-baseline kernel)."""
        a_bits = np.ascontiguousarray(a_bits, dtype=np.uint16)
        b_bits = np.ascontiguousarray(b_bits, dtype=np.uint16)
        m, k = a_bits.shape
        n = b_bits.shape[0]
        c = np.empty((m, n), dtype=np.uint16 if out_bf16 else np.float32)
        self.lib.vo_matmul_bf16_dense(a_bits.ctypes.data, b_bits.ctypes.data, None if out_bf16 else c.ctypes.data,
                                      c.ctypes.data if out_bf16 else None, m, n, k)
        return c

    def matmul_i8_dense(self, a: np.ndarray, b: np.ndarray) -> np.ndarray:
        a = np.ascontiguousarray(a, dtype=np.int8)
        b = np.ascontiguousarray(b, dtype=np.int8)
        c = np.empty((a.shape[0], b.shape[0]), dtype=np.int32)
        self.lib.vo_matmul_i8_dense(a.ctypes.data, b.ctypes.data, c.ctypes.data, a.shape[0], b.shape[0], a.shape[1])
        return c

    def matmul_i8_dequant(self, a, b, row_scales, column_scales, correction=None) -> np.ndarray:
        a = np.ascontiguousarray(a, dtype=np.int8)
        b = np.ascontiguousarray(b, dtype=np.int8)
        rs = np.ascontiguousarray(row_scales, dtype=np.float32)
        cs = np.ascontiguousarray(column_scales, dtype=np.float32)
        corr = np.ascontiguousarray(correction, dtype=np.int32) if correction is not None else None
        c = np.empty((a.shape[0], b.shape[0]), dtype=np.float32)
        self.lib.vo_matmul_i8_dequant(a.ctypes.data, b.ctypes.data, rs.ctypes.data, cs.ctypes.data,
                                      corr.ctypes.data if corr is not None else None, c.ctypes.data, a.shape[0],
                                      b.shape[0], a.shape[1])
        return c

    def quantize_rows(self, a, multipliers, zero_point: int) -> np.ndarray:
        """uint8 [M,K]: the per-row asymmetric quantisation of fp32 activations (vo_quantize_rows_u8)."""
        a = np.ascontiguousarray(a, dtype=np.float32)
        mult = np.ascontiguousarray(multipliers, dtype=np.float32)
        assert a.ndim == 2 and mult.shape == (a.shape[0],)
        q = np.empty(a.shape, dtype=np.uint8)
        self.lib.vo_quantize_rows_u8(a.ctypes.data, a.shape[0], a.shape[1], a.shape[1], mult.ctypes.data,
                                     int(zero_point), q.ctypes.data, a.shape[1])
        return q

    def fused_outputs(self, acc, out_dtype, *, activation=0, scale=None, shift=None, row_scales=None,
                      column_scales=None, lo=0.0, hi=0.0) -> np.ndarray:
        """The fused output transform on an [M,N] accumulator matrix (int32 or float32, C-input already
        added); out_dtype float32, uint16 (bf16 bits), uint8 or int8."""
        acc = np.ascontiguousarray(acc)
        assert acc.ndim == 2 and acc.dtype in (np.int32, np.float32)
        out_dtype = np.dtype(out_dtype)
        code = {np.dtype(np.float32): 12, np.dtype(np.uint16): 11, np.dtype(np.uint8): 3, np.dtype(np.int8): 2}[out_dtype]
        rs = np.ascontiguousarray(row_scales, dtype=np.float32) if row_scales is not None else None
        cs = np.ascontiguousarray(column_scales, dtype=np.float32) if column_scales is not None else None
        out = np.empty(acc.shape, dtype=out_dtype)
        rc = self.lib.vo_fused_outputs(acc.ctypes.data, 1 if acc.dtype == np.int32 else 0, acc.shape[0], acc.shape[1],
                                       rs.ctypes.data if rs is not None else None,
                                       cs.ctypes.data if cs is not None else None,
                                       (1 if scale is not None else 0) | (2 if shift is not None else 0),
                                       0.0 if scale is None else scale, 0.0 if shift is None else shift, activation,
                                       lo, hi, code, out.ctypes.data)
        if rc != 0:
            raise ValueError("vo_fused_outputs rejected its arguments")
        return out

    def matmul_w8a16_group(self, x_bits, w, scales, group: int):
        """Returns (y bf16 bits [M,N], y as float64 [M,N])."""
        x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
        w = np.ascontiguousarray(w, dtype=np.int8)
        scales = np.ascontiguousarray(scales, dtype=np.float32)
        M, K = x_bits.shape
        N = w.shape[0]
        y = np.empty((M, N), dtype=np.uint16)
        y64 = np.empty((M, N), dtype=np.float64)
        rc = self.lib.vo_matmul_w8a16_group(x_bits.ctypes.data, w.ctypes.data, scales.ctypes.data, y.ctypes.data,
                                            y64.ctypes.data, M, N, K, group)
        if rc != 0:
            raise ValueError("K must be a multiple of the group size")
        return y, y64

    # -- dispatch predicates -----------------------------------------------------
    def amx_small_vector_profitable(self, shape, m, n, k) -> bool:
        return bool(self.lib.vo_amx_small_vector_profitable(shape, m, n, k))

    def sme_small_vector_profitable(self, shape, m, n, k) -> bool:
        return bool(self.lib.vo_sme_small_vector_profitable(shape, m, n, k))

    def small_area_profitable(self, m, n, k, limit) -> bool:
        return bool(self.lib.vo_small_area_profitable(m, n, k, limit))

    def amx_residual_split_profitable(self, m, n, k) -> bool:
        return bool(self.lib.vo_amx_residual_split_profitable(m, n, k))


def _strides3(arr: np.ndarray):
    s = (C.c_int64 * 3)()
    for i in range(arr.ndim):
        s[i] = arr.strides[i] // arr.itemsize
    return s


class FusedSpec(C.Structure):
    """Mirror of FusedSpec in oracle/ref_harness.cpp."""
    _fields_ = [("activation", C.c_int32), ("flags", C.c_uint32), ("scale", C.c_float), ("shift", C.c_float),
                ("lo", C.c_float), ("hi", C.c_float), ("column_scales", C.c_void_p)]


class Reference:
    """The real vecops CPU matmul (AMX).  ``Reference.load()`` returns None when the
    library was not built or the host cannot run it."""

    def __init__(self, lib) -> None:
        self.lib = lib

    @staticmethod
    def load() -> "Reference | None":
        path = os.path.join(HERE, "_ref", "libvecops_ref.so")
        if not os.path.exists(path):
            return None
        try:
            with open("/proc/cpuinfo") as f:
                flags = f.read()
            if "amx_tile" not in flags or "avx512f" not in flags:
                return None
            lib = C.CDLL(path)
        except OSError:
            return None
        lib.vref_available.restype = C.c_int
        if lib.vref_available() != 1:
            return None
        return Reference(lib)

    def _call2(self, fn, a, b, c, cin=None):
        m, k = a.shape
        n = b.shape[0]
        args = [C.c_void_p(a.ctypes.data), C.c_void_p(b.ctypes.data), C.c_void_p(c.ctypes.data)]
        if cin is not False:
            args.append(C.c_void_p(cin.ctypes.data) if cin is not None else C.c_void_p(None))
        args += [C.c_int64(m), C.c_int64(n), C.c_int64(k), _strides3(a), _strides3(b), _strides3(c)]
        rc = fn(*args)
        if rc != 0:
            raise RuntimeError("reference matmul unavailable")
        return c

    def matmul_bf16_f32(self, a, b, c, cin=None):
        return self._call2(self.lib.vref_matmul_bf16_f32, a, b, c, cin)

    def matmul_bf16_bf16(self, a, b, c):
        return self._call2(self.lib.vref_matmul_bf16_bf16, a, b, c, False)

    def matmul_f32_f32(self, a, b, c, cin=None):
        return self._call2(self.lib.vref_matmul_f32_f32, a, b, c, cin)

    def matmul_f32_bf16(self, a, b, c):
        return self._call2(self.lib.vref_matmul_f32_bf16, a, b, c, False)

    def matmul_i8_i32(self, a, b, c, cin=None):
        return self._call2(self.lib.vref_matmul_i8_i32, a, b, c, cin)

    def matmul_u8i8_i32(self, a, b, c):
        return self._call2(self.lib.vref_matmul_u8i8_i32, a, b, c, False)

    def matmul_bf16_f32_batched(self, a, b, c):
        batch, m, k = a.shape
        n = b.shape[1]
        rc = self.lib.vref_matmul_bf16_f32_batched(
            C.c_void_p(a.ctypes.data), C.c_void_p(b.ctypes.data), C.c_void_p(c.ctypes.data), C.c_int64(batch),
            C.c_int64(m), C.c_int64(n), C.c_int64(k), _strides3(a), _strides3(b), _strides3(c))
        if rc != 0:
            raise RuntimeError("reference matmul unavailable")
        return c

    def dense_bf16_bf16(self, a, b, c, b_is_kn: bool = False):
        """c = a . b^T on dense row-major tensors (the reference's fastest form): a [M,K], b [N,K] - or [K,N] seen
        through the transposed view when b_is_kn -, c [M,N], all bf16 bits."""
        m, k = a.shape
        n = c.shape[1]
        assert a.flags["C_CONTIGUOUS"] and b.flags["C_CONTIGUOUS"] and c.flags["C_CONTIGUOUS"]
        rc = self.lib.vref_dense_bf16_bf16(C.c_void_p(a.ctypes.data), C.c_void_p(b.ctypes.data), C.c_void_p(c.ctypes.data),
                                           C.c_int64(m), C.c_int64(n), C.c_int64(k), 1 if b_is_kn else 0)
        if rc != 0:
            raise RuntimeError("reference matmul unavailable")
        return c

    def matmul_runtime_quant(self, a, b, multipliers, zero_point, correction, row_scales=None, column_scales=None):
        """fp32 a quantised on the way in (per-row multiplier, zero point) x int8 b + correction row;
        int32 sums, or the dequantised fp32 when both scale vectors are given."""
        a = np.ascontiguousarray(a, dtype=np.float32)
        b = np.ascontiguousarray(b, dtype=np.int8)
        m, k = a.shape
        n = b.shape[0]
        mult = np.ascontiguousarray(multipliers, dtype=np.float32)
        corr = np.ascontiguousarray(correction, dtype=np.int32)
        if row_scales is not None:
            rs = np.ascontiguousarray(row_scales, dtype=np.float32)
            cs = np.zeros(n + 64, dtype=np.float32)  # unmasked vector load past n (Quantization.h:229-231)
            cs[:n] = column_scales
            c = np.empty((m, n), dtype=np.float32)
            rs_ptr, cs_ptr = C.c_void_p(rs.ctypes.data), C.c_void_p(cs.ctypes.data)
        else:
            c = np.empty((m, n), dtype=np.int32)
            rs_ptr, cs_ptr = None, None
        rc = self.lib.vref_matmul_runtime_quant(
            C.c_void_p(a.ctypes.data), C.c_void_p(b.ctypes.data), C.c_void_p(mult.ctypes.data), C.c_int32(zero_point),
            rs_ptr, cs_ptr, C.c_void_p(corr.ctypes.data), C.c_void_p(c.ctypes.data), C.c_int64(m), C.c_int64(n),
            C.c_int64(k))
        if rc != 0:
            raise RuntimeError("reference matmul unavailable")
        return c

    def matmul_runtime_quant_batched(self, a, b, multipliers, zero_point, row_scales, column_scales, correction,
                                     batch=None):
        """The batched runtime-quantised product of tests/ops/MatmulConversionTestCommon.h:1277-1434 on the real
        vecops build.  a [batch or 1, M, K] f32 and b [batch or 1, N, K] i8 (a leading extent of 1 = shared by every
        batch, batch stride 0); multipliers / row_scales [a's batches * M]; correction [b's batches * N]."""
        a = np.ascontiguousarray(a, dtype=np.float32)
        b = np.ascontiguousarray(b, dtype=np.int8)
        batch = max(a.shape[0], b.shape[0]) if batch is None else batch
        m, k = a.shape[1:]
        n = b.shape[1]
        mult = np.ascontiguousarray(multipliers, dtype=np.float32)
        rs = np.ascontiguousarray(row_scales, dtype=np.float32)
        corr = np.ascontiguousarray(correction, dtype=np.int32)
        assert mult.size == a.shape[0] * m and rs.size == mult.size and corr.size == b.shape[0] * n
        cs = np.zeros(n + 64, dtype=np.float32)  # unmasked vector load past n (Quantization.h:229-231)
        cs[:n] = column_scales
        c = np.empty((batch, m, n), dtype=np.float32)
        rc = self.lib.vref_matmul_runtime_quant_batched(
            C.c_void_p(a.ctypes.data), C.c_void_p(b.ctypes.data), C.c_void_p(mult.ctypes.data), C.c_int32(zero_point),
            C.c_void_p(rs.ctypes.data), C.c_void_p(cs.ctypes.data), C.c_void_p(corr.ctypes.data),
            C.c_void_p(c.ctypes.data), C.c_int64(batch), C.c_int64(m), C.c_int64(n), C.c_int64(k),
            C.c_int(1 if a.shape[0] == 1 and batch > 1 else 0), C.c_int(1 if b.shape[0] == 1 and batch > 1 else 0))
        if rc != 0:
            raise RuntimeError("reference matmul unavailable")
        return c

    def matmul_i8_dequant(self, a, b, row_scales, column_scales, correction=None):
        a = np.ascontiguousarray(a, dtype=np.int8)
        b = np.ascontiguousarray(b, dtype=np.int8)
        m, k = a.shape
        n = b.shape[0]
        rs = np.ascontiguousarray(row_scales, dtype=np.float32)
        cs = np.zeros(n + 64, dtype=np.float32)  # unmasked vector load past n (Quantization.h:229-231)
        cs[:n] = column_scales
        corr = np.ascontiguousarray(correction, dtype=np.int32) if correction is not None else None
        c = np.empty((m, n), dtype=np.float32)
        rc = self.lib.vref_matmul_i8_dequant(
            C.c_void_p(a.ctypes.data), C.c_void_p(b.ctypes.data), C.c_void_p(rs.ctypes.data),
            C.c_void_p(cs.ctypes.data), C.c_void_p(corr.ctypes.data if corr is not None else None),
            C.c_void_p(c.ctypes.data), C.c_int64(m), C.c_int64(n), C.c_int64(k))
        if rc != 0:
            raise RuntimeError("reference matmul unavailable")
        return c

    def matmul_fused(self, a, b, bias, out_dtype, *, activation=0, scale=None, column_scales=None, shift=None,
                     lo=0.0, hi=0.0):
        """bf16 (uint16 bits) or int8 operands through the reference with a fused output transform:
        convert(act(((A.B^T + bias) * scale) * column_scales[col] + shift)); out_dtype is a numpy dtype
        (float32, uint16 = bf16 bits, uint8, int8)."""
        m, k = a.shape
        n = b.shape[0]
        a = np.ascontiguousarray(a)
        b = np.ascontiguousarray(b)
        cs = None
        if column_scales is not None:
            cs = np.zeros(n + 64, dtype=np.float32)  # unmasked vector load past n
            cs[:n] = column_scales
        spec = FusedSpec(activation, (1 if scale is not None else 0) | (2 if shift is not None else 0),
                         0.0 if scale is None else scale, 0.0 if shift is None else shift, lo, hi,
                         cs.ctypes.data if cs is not None else None)
        integer = a.dtype == np.int8
        if bias is not None:
            bias = np.ascontiguousarray(bias, dtype=np.int32 if integer else np.float32)
        out_dtype = np.dtype(out_dtype)
        kind = {np.dtype(np.float32): 0, np.dtype(np.uint16): 1, np.dtype(np.uint8): 3, np.dtype(np.int8): 4}[out_dtype]
        c = np.zeros((m, n), dtype=out_dtype)
        fn = self.lib.vref_matmul_i8_fused if integer else self.lib.vref_matmul_bf16_fused
        rc = fn(C.c_void_p(a.ctypes.data), C.c_void_p(b.ctypes.data),
                C.c_void_p(bias.ctypes.data if bias is not None else None), C.c_void_p(c.ctypes.data), C.c_int(kind),
                C.c_int64(m), C.c_int64(n), C.c_int64(k), C.byref(spec))
        if rc != 0:
            raise RuntimeError("reference fused matmul unavailable (rc=%d)" % rc)
        return c

    def predicate(self, name: str, *args) -> bool:
        fn = getattr(self.lib, "vref_" + name)
        fn.argtypes = [C.c_int] + [C.c_int64] * (len(args) - 1) if "small_vector" in name else [C.c_int64] * len(args)
        return bool(fn(*args))
