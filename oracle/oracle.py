"""ctypes binding of the CPU oracle (oracle/bitnet_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of the benchmark.  The shipped package never imports it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libbitnet_oracle.so")

_f32p = C.POINTER(C.c_float)
_u8p = C.POINTER(C.c_uint8)
_i8p = C.POINTER(C.c_int8)
_i32p = C.POINTER(C.c_int32)


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds).  Returns the path of the library."""
    src = os.path.join(_HERE, "bitnet_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_SO)
        L.orc_pack_ternary_bits.argtypes = [_f32p, C.c_size_t, C.c_float, C.c_float, _u8p]
        L.orc_pack_ternary_bits.restype = None
        L.orc_quantize_ternary.argtypes = [_f32p, C.c_size_t, _u8p, _f32p, _f32p]
        L.orc_quantize_ternary.restype = C.c_uint64
        L.orc_get_value.argtypes = [_u8p, C.c_size_t, C.c_size_t]
        L.orc_get_value.restype = C.c_int8
        L.orc_dequantize_ternary.argtypes = [_u8p, C.c_size_t, C.c_float, _f32p]
        L.orc_dequantize_ternary.restype = None
        L.orc_ternary_matmul.argtypes = [_u8p, C.c_float, _u8p, C.c_float, C.c_size_t,
                                         C.c_size_t, C.c_size_t, _f32p, _i32p]
        L.orc_ternary_matmul.restype = None
        L.orc_execute_ternary.argtypes = [_f32p, _f32p, C.c_size_t, C.c_size_t, C.c_size_t,
                                          _f32p, _i32p]
        L.orc_execute_ternary.restype = C.c_int
        L.orc_packed_size.argtypes = [C.POINTER(C.c_size_t), C.c_size_t, C.c_int]
        L.orc_packed_size.restype = C.c_int64
        L.orc_alignment.argtypes = [C.c_int]
        L.orc_alignment.restype = C.c_size_t
        L.orc_act_quant_i8.argtypes = [_f32p, C.c_size_t, C.c_size_t, _i8p, _f32p, _i32p]
        L.orc_act_quant_i8.restype = None
        L.orc_matmul_i8_ternary.argtypes = [_i8p, _f32p, _u8p, C.c_float, C.c_size_t,
                                            C.c_size_t, C.c_size_t, _f32p, _i32p]
        L.orc_matmul_i8_ternary.restype = None
        L.orc_unpack_values.argtypes = [_u8p, C.c_size_t, _i8p]
        L.orc_unpack_values.restype = None
        _lib = L
    return _lib


def _p(a, t):
    return a.ctypes.data_as(t)


def _f32(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.float32))


class TernaryTensor:
    """Fields of the reference's TernaryTensor (quantization.rs:249-260)."""

    def __init__(self, packed_data, shape, scale, threshold, element_count, survivors=0):
        self.packed_data = packed_data      # np.uint8 [ceil(n/4)]
        self.shape = list(shape)
        self.scale = np.float32(scale)
        self.threshold = np.float32(threshold)
        self.element_count = int(element_count)
        self.survivors = int(survivors)

    def memory_size(self):
        return int(self.packed_data.size)

    def compression_ratio(self):
        return np.float32(np.float32(self.element_count * 4) / np.float32(self.memory_size()))

    def get_value(self, index):
        return int(lib().orc_get_value(_p(self.packed_data, _u8p), self.element_count, index))

    def values(self):
        out = np.empty(self.element_count, dtype=np.int8)
        lib().orc_unpack_values(_p(self.packed_data, _u8p), self.element_count, _p(out, _i8p))
        return out


def quantize_ternary(x) -> TernaryTensor:
    x = _f32(x)
    n = x.size
    packed = np.zeros((n + 3) // 4, dtype=np.uint8)
    if packed.size == 0:
        packed = np.zeros(1, dtype=np.uint8)[:0]
    scale = C.c_float()
    thr = C.c_float()
    # a zero-length numpy array still has a valid (dummy) data pointer
    cnt = lib().orc_quantize_ternary(_p(x, _f32p), n, _p(packed, _u8p), C.byref(scale),
                                     C.byref(thr))
    return TernaryTensor(packed, x.shape, scale.value, thr.value, n, cnt)


def pack_ternary_bits(x, threshold) -> np.ndarray:
    x = _f32(x)
    packed = np.zeros((x.size + 3) // 4, dtype=np.uint8)
    lib().orc_pack_ternary_bits(_p(x, _f32p), x.size, np.float32(threshold), 1.0,
                                _p(packed, _u8p))
    return packed


def dequantize_ternary(t: TernaryTensor) -> np.ndarray:
    out = np.empty(t.element_count, dtype=np.float32)
    lib().orc_dequantize_ternary(_p(t.packed_data, _u8p), t.element_count, t.scale,
                                 _p(out, _f32p))
    return out.reshape(t.shape)


def ternary_matmul(a: TernaryTensor, b: TernaryTensor, m, n, k):
    """execute_ternary_matmul (kernels.rs:134-178): returns (f32 [m,n], int32 [m,n])."""
    if a.shape != [m, k] or b.shape != [k, n]:
        raise ValueError(
            "Matrix dimension mismatch: A=%s, B=%s, expected A=[%d,%d], B=[%d,%d]"
            % (a.shape, b.shape, m, k, k, n))
    out = np.empty((m, n), dtype=np.float32)
    acc = np.empty((m, n), dtype=np.int32)
    lib().orc_ternary_matmul(_p(a.packed_data, _u8p), a.scale, _p(b.packed_data, _u8p), b.scale,
                             m, n, k, _p(out, _f32p), _p(acc, _i32p))
    return out, acc


def execute_ternary(a, b):
    """CompiledKernel::execute, TernaryMatMul arm (kernels.rs:271-283) with m,n,k
    taken from the inputs.  Returns (f32 [m,n], int32 [m,n])."""
    a = _f32(a)
    b = _f32(b)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    out = np.empty((m, n), dtype=np.float32)
    acc = np.empty((m, n), dtype=np.int32)
    rc = lib().orc_execute_ternary(_p(a, _f32p), _p(b, _f32p), m, n, k, _p(out, _f32p),
                                   _p(acc, _i32p))
    if rc != 0:
        raise MemoryError("oracle allocation failed")
    return out, acc


def act_quant_i8(x):
    """Build-defined per-token absmax int8 quantiser: (q int8 [m,k], scale f32 [m], rowsum i32 [m])."""
    x = _f32(x)
    m, k = x.shape
    q = np.empty((m, k), dtype=np.int8)
    scale = np.empty(m, dtype=np.float32)
    rowsum = np.empty(m, dtype=np.int32)
    lib().orc_act_quant_i8(_p(x, _f32p), m, k, _p(q, _i8p), _p(scale, _f32p), _p(rowsum, _i32p))
    return q, scale, rowsum


def matmul_i8_ternary(q, act_scale, b: TernaryTensor):
    q = np.ascontiguousarray(q, dtype=np.int8)
    act_scale = _f32(act_scale)
    m, k = q.shape
    k2, n = b.shape
    assert k == k2 and act_scale.size == m
    out = np.empty((m, n), dtype=np.float32)
    acc = np.empty((m, n), dtype=np.int32)
    lib().orc_matmul_i8_ternary(_p(q, _i8p), _p(act_scale, _f32p), _p(b.packed_data, _u8p),
                                b.scale, m, n, k, _p(out, _f32p), _p(acc, _i32p))
    return out, acc


def packed_size(shape, dtype_code):
    arr = (C.c_size_t * len(shape))(*shape)
    return int(lib().orc_packed_size(arr, len(shape), dtype_code))


def alignment(dtype_code):
    return int(lib().orc_alignment(dtype_code))
