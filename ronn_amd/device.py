"""Device context and buffers over the C ABI (numpy on the host side).

Everything here forwards to libronn_bitnet_hip.so; nothing computes on the CPU.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import check


class DeviceBuffer:
    """A device allocation owned by a Context (rbn_malloc / rbn_free)."""

    def __init__(self, ctx: "Context", nbytes: int):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(ctx.lib.rbn_malloc(ctx.handle, self.nbytes, C.byref(p)))
        self.ptr = p.value

    def free(self):
        if self.ptr is not None and self.ctx.handle is not None:
            check(self.ctx.lib.rbn_free(self.ctx.handle, self.ptr))
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def upload(self, array: np.ndarray):
        a = np.ascontiguousarray(array)
        if a.nbytes > self.nbytes:
            raise ValueError("upload of %d bytes into a %d-byte buffer" % (a.nbytes, self.nbytes))
        check(self.ctx.lib.rbn_h2d(self.ctx.handle, self.ptr, a.ctypes.data, a.nbytes))
        return self

    def download(self, dtype, count: int, offset_bytes: int = 0) -> np.ndarray:
        out = np.empty(int(count), dtype=dtype)
        if out.nbytes + offset_bytes > self.nbytes:
            raise ValueError("download beyond the end of the buffer")
        check(self.ctx.lib.rbn_d2h(self.ctx.handle, out.ctypes.data, self.ptr + offset_bytes,
                                   out.nbytes))
        return out


class Context:
    """One GPU, one stream (rbn_ctx)."""

    def __init__(self, device: int = 0):
        self.lib = _lib.load()
        h = C.c_void_p()
        check(self.lib.rbn_ctx_create(int(device), C.byref(h)))
        self.handle = h.value
        self.device = int(device)

    def close(self):
        if self.handle is not None:
            self.lib.rbn_ctx_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- buffers ---------------------------------------------------------------
    def alloc(self, nbytes: int) -> DeviceBuffer:
        return DeviceBuffer(self, nbytes)

    def to_device(self, array: np.ndarray) -> DeviceBuffer:
        a = np.ascontiguousarray(array)
        return self.alloc(max(a.nbytes, 1)).upload(a)

    def sync(self):
        check(self.lib.rbn_sync(self.handle))

    def device_info(self) -> dict:
        info = _lib.DeviceInfo()
        check(self.lib.rbn_get_device_info(self.handle, C.byref(info)))
        return {
            "name": info.name.decode(), "arch": info.arch.decode(),
            "compute_units": info.compute_units, "clock_khz": info.clock_khz,
            "mem_clock_khz": info.mem_clock_khz, "mem_bus_bits": info.mem_bus_bits,
            "hbm_bytes": info.hbm_bytes, "l2_bytes": info.l2_bytes,
        }

    def memory_info(self):
        a, p = C.c_uint64(), C.c_uint64()
        check(self.lib.rbn_memory_info(self.handle, C.byref(a), C.byref(p)))
        return a.value, p.value

    # -- timing ------------------------------------------------------------------
    def timer_start(self):
        check(self.lib.rbn_timer_start(self.handle))

    def timer_stop(self) -> float:
        ms = C.c_float()
        check(self.lib.rbn_timer_stop(self.handle, C.byref(ms)))
        return ms.value

    # -- HIP graphs ------------------------------------------------------------------
    def graph_begin(self):
        check(self.lib.rbn_graph_begin_capture(self.handle))

    def graph_end(self):
        g = C.c_void_p()
        check(self.lib.rbn_graph_end_capture(self.handle, C.byref(g)))
        return g.value

    def graph_launch(self, graph):
        check(self.lib.rbn_graph_launch(self.handle, graph))

    def graph_destroy(self, graph):
        check(self.lib.rbn_graph_destroy(self.handle, graph))

    # -- (1) ternarize + pack ------------------------------------------------------
    def abs_sum(self, d_x: DeviceBuffer, n: int, mode=_lib.SUM_STRICT_SEQ, mask_threshold=None):
        s, cnt = C.c_float(), C.c_uint64()
        use_mask = 0 if mask_threshold is None else 1
        thr = 0.0 if mask_threshold is None else float(mask_threshold)
        check(self.lib.rbn_abs_sum_f32(self.handle, d_x.ptr, n, mode, use_mask, thr, C.byref(s),
                                       C.byref(cnt)))
        return np.float32(s.value), cnt.value

    def pack_ternary(self, d_x: DeviceBuffer, n: int, threshold, d_packed: DeviceBuffer = None):
        if d_packed is None:
            d_packed = self.alloc(self.lib.rbn_packed_capacity(n))
        check(self.lib.rbn_pack_ternary(self.handle, d_x.ptr, n, float(threshold), d_packed.ptr))
        return d_packed

    def quantize_ternary(self, d_x: DeviceBuffer, n: int, mode=_lib.SUM_STRICT_SEQ,
                         d_packed: DeviceBuffer = None):
        """Returns (d_packed, scale, threshold, survivors)."""
        if d_packed is None:
            d_packed = self.alloc(self.lib.rbn_packed_capacity(n))
        scale, thr, cnt = C.c_float(), C.c_float(), C.c_uint64()
        check(self.lib.rbn_quantize_ternary(self.handle, d_x.ptr, n, mode, d_packed.ptr,
                                            C.byref(scale), C.byref(thr), C.byref(cnt)))
        return d_packed, np.float32(scale.value), np.float32(thr.value), cnt.value

    def dequantize_ternary(self, d_packed: DeviceBuffer, n: int, scale) -> DeviceBuffer:
        d_out = self.alloc(max(4 * n, 4))
        check(self.lib.rbn_dequantize_ternary(self.handle, d_packed.ptr, n, float(scale),
                                              d_out.ptr))
        return d_out

    def tile_weights(self, d_packed: DeviceBuffer, K: int, N: int) -> DeviceBuffer:
        d_tiled = self.alloc(self.lib.rbn_tiled_bytes(K, N))
        check(self.lib.rbn_tile_weights(self.handle, d_packed.ptr, K, N, d_tiled.ptr))
        return d_tiled

    # -- (2) activations -------------------------------------------------------------
    def act_pitch(self, K: int) -> int:
        return int(self.lib.rbn_act_pitch(K))

    def alloc_acts(self, M: int, K: int):
        return (self.alloc(M * self.act_pitch(K)), self.alloc(4 * M), self.alloc(4 * M))

    def act_quant_i8(self, d_x: DeviceBuffer, M: int, K: int, bufs=None):
        """Returns (d_q [M,pitch] int8, d_act_scale [M] f32, d_rowsum [M] i32)."""
        d_q, d_s, d_r = bufs if bufs is not None else self.alloc_acts(M, K)
        check(self.lib.rbn_act_quant_i8(self.handle, d_x.ptr, M, K, d_q.ptr, d_s.ptr, d_r.ptr))
        return d_q, d_s, d_r

    def act_quant_ternary(self, d_x: DeviceBuffer, M: int, K: int, mode=_lib.SUM_STRICT_SEQ,
                          bufs=None):
        """Returns (d_q, d_act_scale, d_rowsum, scale, threshold)."""
        d_q, d_s, d_r = bufs if bufs is not None else self.alloc_acts(M, K)
        scale, thr = C.c_float(), C.c_float()
        check(self.lib.rbn_act_quant_ternary(self.handle, d_x.ptr, M, K, mode, d_q.ptr, d_s.ptr,
                                             d_r.ptr, C.byref(scale), C.byref(thr)))
        return d_q, d_s, d_r, np.float32(scale.value), np.float32(thr.value)

    def unpack_ternary_i8(self, d_packed: DeviceBuffer, rows: int, cols: int, pitch: int = None):
        pitch = cols if pitch is None else pitch
        d_q = self.alloc(max(rows * pitch, 1))
        d_r = self.alloc(max(4 * rows, 4))
        check(self.lib.rbn_unpack_ternary_i8(self.handle, d_packed.ptr, rows, cols, pitch, d_q.ptr,
                                             d_r.ptr))
        return d_q, d_r

    # -- (3)(4)(5) matmul ----------------------------------------------------------------
    def _mm(self, fn, acts, d_tiled, w_scale, M, K, N, want_acc, d_out=None, d_acc=None):
        d_q, d_s, d_r = acts
        if d_out is None:
            d_out = self.alloc(4 * M * N)
        if want_acc and d_acc is None:
            d_acc = self.alloc(4 * M * N)
        check(fn(self.handle, d_q.ptr, d_s.ptr, d_r.ptr, d_tiled.ptr, float(w_scale), M, K, N,
                 d_acc.ptr if d_acc is not None else None, d_out.ptr))
        return d_out, d_acc

    def gemv(self, acts, d_tiled, w_scale, M, K, N, want_acc=False, d_out=None, d_acc=None):
        return self._mm(self.lib.rbn_gemv_t2_i8, acts, d_tiled, w_scale, M, K, N, want_acc, d_out,
                        d_acc)

    def gemv_kernel_time_us(self, acts, d_tiled, w_scale, M, K, N, d_out) -> float:
        """One GEMV launch; returns the duration of the dispatch from its own timestamps."""
        d_q, d_s, d_r = acts
        us = C.c_float()
        check(self.lib.rbn_gemv_t2_i8_kernel_time(self.handle, d_q.ptr, d_s.ptr, d_r.ptr, d_tiled.ptr,
                                                  float(w_scale), M, K, N, None, d_out.ptr, C.byref(us)))
        return us.value

    def gemv_problems(self, problems):
        """Host array of rbn_gemv_problem from (acts, d_tiled, w_scale, d_out, d_acc or None) tuples."""
        arr = (_lib.GemvProblem * len(problems))()
        for p, (acts, d_tiled, w_scale, d_out, d_acc) in zip(arr, problems):
            p.d_q, p.d_act_scale, p.d_rowsum = acts[0].ptr, acts[1].ptr, acts[2].ptr
            p.d_tiled, p.d_out = d_tiled.ptr, d_out.ptr
            p.d_acc = d_acc.ptr if d_acc is not None else None
            p.w_scale, p.reserved = float(w_scale), 0
        return arr

    def gemv_grouped(self, problems, M, K, N, first=0, count=None):
        """One launch of problems[first:first+count] (an array from gemv_problems), all of shape (M, K, N)."""
        count = len(problems) - first if count is None else count
        check(self.lib.rbn_gemv_t2_i8_grouped(
            self.handle, C.cast(C.byref(problems, first * C.sizeof(_lib.GemvProblem)), C.POINTER(_lib.GemvProblem)),
            count, M, K, N))

    def skinny(self, acts, d_tiled, w_scale, M, K, N, want_acc=False, d_out=None, d_acc=None):
        return self._mm(self.lib.rbn_gemm_t2_i8_skinny, acts, d_tiled, w_scale, M, K, N, want_acc,
                        d_out, d_acc)

    def skinny_static(self, acts, d_tiled, w_scale, M, K, N, want_acc=False, d_out=None, d_acc=None):
        """rbn_gemm_t2_i8_skinny with the split-k exchange in the library's static device array."""
        return self._mm(self.lib.rbn_gemm_t2_i8_skinny_static, acts, d_tiled, w_scale, M, K, N, want_acc,
                        d_out, d_acc)

    def gemm(self, acts, d_tiled, w_scale, M, K, N, want_acc=False, d_out=None, d_acc=None):
        return self._mm(self.lib.rbn_gemm_t2_i8_mfma, acts, d_tiled, w_scale, M, K, N, want_acc,
                        d_out, d_acc)

    def matmul(self, acts, d_tiled, w_scale, M, K, N, want_acc=False, d_out=None, d_acc=None):
        return self._mm(self.lib.rbn_matmul_t2_i8, acts, d_tiled, w_scale, M, K, N, want_acc,
                        d_out, d_acc)

    def probe_mfma_i8(self, operand_kind: int) -> float:
        """Dense int8 MFMA rate of this machine in TOP/s (0 constant, 1 int8 x ternary, 2 int8 x int8)."""
        tops = C.c_double()
        check(self.lib.rbn_probe_mfma_i8(self.handle, operand_kind, C.byref(tops)))
        return tops.value

    # -- whole execute() -------------------------------------------------------------------
    def execute_ternary_matmul(self, a: np.ndarray, b: np.ndarray, mode=_lib.SUM_STRICT_SEQ,
                               want_acc=True):
        a = np.ascontiguousarray(a, dtype=np.float32)
        b = np.ascontiguousarray(b, dtype=np.float32)
        M, K = a.shape
        K2, N = b.shape
        if K != K2:
            raise ValueError("inner dimensions differ")
        out = np.empty((M, N), dtype=np.float32)
        acc = np.empty((M, N), dtype=np.int32) if want_acc else None
        check(self.lib.rbn_execute_ternary_matmul(
            self.handle, a.ctypes.data, b.ctypes.data, M, N, K, mode, out.ctypes.data,
            acc.ctypes.data if want_acc else None))
        return out, acc


def synth_normal(seed: int, sigma: float, shape, first: int = 0) -> np.ndarray:
    """Deterministic N(0, sigma^2) f32 tensor from the library's counter-based generator."""
    count = int(np.prod(shape))
    out = np.empty(count, dtype=np.float32)
    _lib.load().rbn_synth_normal_f32(int(seed), float(sigma), int(first), count, out.ctypes.data)
    return out.reshape(shape)
