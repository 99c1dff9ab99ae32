"""ctypes binding of libronn_bitnet_hip.so (the C ABI in include/ronn_bitnet_hip.h).

The library carries the hand-written gfx950 kernels.  There is no CPU fallback: if
the library is missing, or no MI355X is visible when a context is created, the
call raises.
"""
from __future__ import annotations

import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libronn_bitnet_hip.so")

RBN_OK = 0
RBN_ERR_INVALID = -1
RBN_ERR_HIP = -2
RBN_ERR_OOM = -3
RBN_ERR_UNSUPPORTED = -4
RBN_ERR_NO_DEVICE = -5

SUM_STRICT_SEQ = 0
SUM_TREE = 1
GEMV_MAX_M = 16
GEMV_GROUP_MAX = 32
FLAG_HISTORY_OVERFLOW = 1

# dtype codes of rbn_tensor_bytes (declaration order of the reference's DataType)
DT_F32, DT_F16, DT_BF16, DT_I8, DT_I32, DT_I64, DT_U8, DT_U32, DT_BOOL, DT_F64 = range(10)


class DeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128),
        ("arch", C.c_char * 64),
        ("compute_units", C.c_int),
        ("clock_khz", C.c_int),
        ("mem_clock_khz", C.c_int),
        ("mem_bus_bits", C.c_int),
        ("hbm_bytes", C.c_uint64),
        ("l2_bytes", C.c_uint64),
    ]


class GemvProblem(C.Structure):
    """rbn_gemv_problem: one GEMV of a grouped launch (device pointers)."""
    _fields_ = [
        ("d_q", C.c_void_p),
        ("d_act_scale", C.c_void_p),
        ("d_rowsum", C.c_void_p),
        ("d_tiled", C.c_void_p),
        ("d_out", C.c_void_p),
        ("d_acc", C.c_void_p),
        ("w_scale", C.c_float),
        ("reserved", C.c_uint32),
    ]


class RbnError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("%s (rbn status %d)" % (message, code))
        self.code = code
        self.message = message


_vp = C.c_void_p
_u64 = C.c_uint64
_f32p = C.POINTER(C.c_float)
_u64p = C.POINTER(C.c_uint64)

# name -> (restype, argtypes).  Every symbol include/ronn_bitnet_hip.h declares.
SIGNATURES = {
    "rbn_version": (C.c_char_p, []),
    "rbn_last_error": (C.c_char_p, []),
    "rbn_device_count": (C.c_int, []),
    "rbn_ctx_create": (C.c_int, [C.c_int, C.POINTER(_vp)]),
    "rbn_ctx_destroy": (C.c_int, [_vp]),
    "rbn_get_device_info": (C.c_int, [_vp, C.POINTER(DeviceInfo)]),
    "rbn_malloc": (C.c_int, [_vp, C.c_size_t, C.POINTER(_vp)]),
    "rbn_free": (C.c_int, [_vp, _vp]),
    "rbn_h2d": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "rbn_d2h": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "rbn_d2d": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "rbn_fill_u8": (C.c_int, [_vp, _vp, C.c_int, C.c_size_t]),
    "rbn_sync": (C.c_int, [_vp]),
    "rbn_memory_info": (C.c_int, [_vp, _u64p, _u64p]),
    "rbn_tensor_bytes": (C.c_int64, [_u64, C.c_int]),
    "rbn_tensor_alignment": (C.c_size_t, [C.c_int]),
    "rbn_packed_capacity": (C.c_size_t, [_u64]),
    "rbn_tiled_bytes": (C.c_size_t, [_u64, _u64]),
    "rbn_act_pitch": (C.c_size_t, [_u64]),
    "rbn_timer_start": (C.c_int, [_vp]),
    "rbn_timer_stop": (C.c_int, [_vp, _f32p]),
    "rbn_graph_begin_capture": (C.c_int, [_vp]),
    "rbn_graph_end_capture": (C.c_int, [_vp, C.POINTER(_vp)]),
    "rbn_graph_launch": (C.c_int, [_vp, _vp]),
    "rbn_graph_destroy": (C.c_int, [_vp, _vp]),
    "rbn_abs_sum_f32": (C.c_int, [_vp, _vp, _u64, C.c_int, C.c_int, C.c_float, _f32p, _u64p]),
    "rbn_pack_ternary": (C.c_int, [_vp, _vp, _u64, C.c_float, _vp]),
    "rbn_quantize_ternary": (C.c_int, [_vp, _vp, _u64, C.c_int, _vp, _f32p, _f32p, _u64p]),
    "rbn_dequantize_ternary": (C.c_int, [_vp, _vp, _u64, C.c_float, _vp]),
    "rbn_unpack_ternary_i8": (C.c_int, [_vp, _vp, _u64, _u64, _u64, _vp, _vp]),
    "rbn_tile_weights": (C.c_int, [_vp, _vp, _u64, _u64, _vp]),
    "rbn_act_quant_i8": (C.c_int, [_vp, _vp, _u64, _u64, _vp, _vp, _vp]),
    "rbn_act_quant_ternary": (C.c_int, [_vp, _vp, _u64, _u64, C.c_int, _vp, _vp, _vp, _f32p, _f32p]),
    "rbn_gemv_t2_i8": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_float, _u64, _u64, _u64, _vp, _vp]),
    "rbn_gemv_t2_i8_kernel_time": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_float, _u64, _u64, _u64, _vp, _vp,
                                             C.POINTER(C.c_float)]),
    "rbn_gemv_t2_i8_grouped": (C.c_int, [_vp, C.POINTER(GemvProblem), _u64, _u64, _u64, _u64]),
    "rbn_gemm_t2_i8_skinny": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_float, _u64, _u64, _u64, _vp, _vp]),
    "rbn_skinny_launch_shape": (C.c_int, [_u64, _u64, _u64, C.POINTER(C.c_int32)]),
    "rbn_gemm_t2_i8_skinny_static": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_float, _u64, _u64, _u64, _vp, _vp]),
    "rbn_gemm_t2_i8_mfma": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_float, _u64, _u64, _u64, _vp, _vp]),
    "rbn_bitlinear_gemv_f32": (C.c_int, [_vp, _vp, _vp, _vp, C.c_float, _vp, C.c_float, _u64, _u64, _vp, _vp]),
    "rbn_embed_f32": (C.c_int, [_vp, _vp, _vp, _u64, _u64, _u64, _vp]),
    "rbn_rmsnorm_quant_i8": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_float, _u64, _u64, _vp, _vp, _vp]),
    "rbn_rope_kv_store_f16": (C.c_int, [_vp, _vp, _vp, _u64, _u64, _u64, C.c_float, _vp, _vp, _u64]),
    "rbn_attention_f16kv": (C.c_int, [_vp, _vp, _vp, _u64, _u64, _u64, _vp, _vp, _u64, _vp]),
    "rbn_attention_decode_f16kv": (C.c_int, [_vp, _vp, _vp, _u64, _u64, C.c_float, _vp, _vp, _u64, _vp]),
    "rbn_swiglu_f32": (C.c_int, [_vp, _vp, _u64, _u64, _vp]),
    "rbn_argmax_f32": (C.c_int, [_vp, _vp, _u64, _vp, _vp, _vp, _u64]),
    "rbn_greedy_next_f32": (C.c_int, [_vp, _vp, _u64, _vp, _vp, _vp, _u64, _vp, _u64, _vp]),
    "rbn_device_flags": (C.c_int, [_vp, C.POINTER(C.c_uint32)]),
    "rbn_add_i32": (C.c_int, [_vp, _vp, C.c_int32]),
    "rbn_synth_normal_device_f32": (C.c_int, [_vp, _u64, C.c_float, _vp, _u64]),
    "rbn_probe_mfma_i8": (C.c_int, [_vp, C.c_int, C.POINTER(C.c_double)]),
    "rbn_probe_empty_launch": (C.c_int, [_vp]),
    "rbn_probe_stream_read": (C.c_int, [_vp, _vp, _u64, C.c_int]),
    "rbn_matmul_kernel_choice": (C.c_int, [_u64, _u64, _u64]),
    "rbn_matmul_t2_i8": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_float, _u64, _u64, _u64, _vp, _vp]),
    "rbn_execute_ternary_matmul": (C.c_int, [_vp, _vp, _vp, _u64, _u64, _u64, C.c_int, _vp, _vp]),
    "rbn_synth_normal_f32": (None, [_u64, C.c_double, _u64, _u64, _vp]),
}

_lib = None


def load():
    """Loads the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C ronn_amd/csrc`.  There is no CPU fallback." % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError names a missing export
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc):
    if rc != RBN_OK:
        raise RbnError(rc, load().rbn_last_error().decode("utf-8", "replace"))
