"""Python face of the BitNet execution provider (include/ronn_bitnet_provider.h).

A thin ctypes layer over the C++ provider mirror that lives in the shared library
(ronn_amd/csrc/host/).  Names follow the reference's
crates/ronn-providers/src/bitnet/{provider,kernels,quantization,allocator}.rs and
crates/ronn-core/src/types.rs, so tests written against the reference read the same.
Nothing here computes: every call lands in the HIP library.
"""
from __future__ import annotations

import ctypes as C
import enum
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np

from . import _lib


class Error(RuntimeError):
    """The reference's anyhow::Error: carries the same message text."""


class DataType(enum.IntEnum):          # types.rs:39-60
    F32 = 0
    F16 = 1
    BF16 = 2
    I8 = 3
    I32 = 4
    I64 = 5
    U8 = 6
    U32 = 7
    Bool = 8
    F64 = 9


class ProviderId(enum.IntEnum):        # types.rs:24-35
    CPU = 0
    GPU = 1
    WebAssembly = 2
    BitNet = 3
    Custom = 4


ProviderType = ProviderId              # types.rs:20


class QuantizationMethod(enum.IntEnum):  # quantization.rs:13-20
    Binary = 0
    Ternary = 1
    AsymmetricBinary = 2


class OptimizationLevel(enum.IntEnum):  # types.rs:281-291
    NONE = 0
    Basic = 1
    Aggressive = 2
    Custom = 3


class PerformanceProfile(enum.IntEnum):  # types.rs:244-254
    CPU = 0
    GPU = 1
    MemoryOptimized = 2
    PowerEfficient = 3


class TensorLayout(enum.IntEnum):
    RowMajor = 0
    ColumnMajor = 1


class Tensor:
    """Host tensor with the four operations the provider uses (tensor.rs:40, :165, :170, :217)."""

    def __init__(self, array: np.ndarray, dtype: DataType, layout: TensorLayout):
        self._a = array
        self._dtype = dtype
        self._layout = layout

    @staticmethod
    def from_data(data, shape: Sequence[int], dtype: DataType = DataType.F32,
                  layout: TensorLayout = TensorLayout.RowMajor) -> "Tensor":
        a = np.ascontiguousarray(np.asarray(data, dtype=np.float32)).reshape(-1)
        if a.size != int(np.prod(shape, dtype=np.int64)):
            raise Error("shape mismatch: %d values for shape %s" % (a.size, list(shape)))
        return Tensor(a.reshape(tuple(shape)), dtype, layout)

    def shape(self) -> List[int]:
        return list(self._a.shape)

    def dtype(self) -> DataType:
        return self._dtype

    def to_vec(self) -> np.ndarray:
        return self._a.reshape(-1)

    def numpy(self) -> np.ndarray:
        return self._a


@dataclass
class GraphNode:                       # types.rs:121-135
    id: int
    op_type: str
    attributes: Dict[str, object] = field(default_factory=dict)
    inputs: List[str] = field(default_factory=list)
    outputs: List[str] = field(default_factory=list)
    name: Optional[str] = None


@dataclass
class SubGraph:                        # types.rs:348-358
    nodes: List[GraphNode]
    edges: list = field(default_factory=list)
    inputs: List[str] = field(default_factory=list)
    outputs: List[str] = field(default_factory=list)


@dataclass
class OperatorSpec:                    # types.rs:335-345
    op_type: str
    input_types: List[DataType] = field(default_factory=list)
    output_types: List[DataType] = field(default_factory=list)
    attributes: Dict[str, object] = field(default_factory=dict)


@dataclass
class ProviderConfig:                  # types.rs:268-278
    thread_count: Optional[int] = None
    memory_limit: Optional[int] = None
    optimization_level: OptimizationLevel = OptimizationLevel.Basic
    custom_options: Dict[str, str] = field(default_factory=dict)


@dataclass
class KernelStats:                     # types.rs:179-189
    execution_count: int = 0
    average_time_us: float = 0.0
    min_time_us: float = 0.0
    max_time_us: float = 0.0


@dataclass
class MemoryUsage:                     # types.rs:168-176
    peak_bytes: int = 0
    current_bytes: int = 0
    allocation_count: int = 0


@dataclass
class MemoryInfo:                      # types.rs:324-332
    total_bytes: int = 0
    allocated_bytes: int = 0
    peak_bytes: int = 0


@dataclass
class TensorBuffer:                    # types.rs:306-316 (ptr is a device address here)
    ptr: int
    size: int
    alignment: int
    memory_type: str = "DeviceMemory"


class _Config(C.Structure):
    _fields_ = [("quantization_method", C.c_int), ("enable_kernel_caching", C.c_int),
                ("max_cache_size", C.c_uint64), ("enable_mixed_precision", C.c_int),
                ("memory_optimization_level", C.c_int), ("enable_simd", C.c_int),
                ("activation", C.c_int), ("strict_reference_sum", C.c_int), ("device", C.c_int)]


@dataclass
class BitNetProviderConfig:            # provider.rs:41-68 (+ activation, strict_reference_sum, device)
    quantization_method: QuantizationMethod = QuantizationMethod.Ternary
    enable_kernel_caching: bool = True
    max_cache_size: int = 64 * 1024 * 1024
    enable_mixed_precision: bool = True
    memory_optimization_level: int = 2
    enable_simd: bool = True
    activation: str = "ternary"        # "ternary" (as the reference) or "int8"
    strict_reference_sum: bool = True
    device: int = 0

    def _to_c(self) -> _Config:
        return _Config(int(self.quantization_method), int(self.enable_kernel_caching),
                       int(self.max_cache_size), int(self.enable_mixed_precision),
                       int(self.memory_optimization_level), int(self.enable_simd),
                       1 if self.activation == "int8" else 0, int(self.strict_reference_sum),
                       int(self.device))

    @staticmethod
    def _from_c(c: _Config) -> "BitNetProviderConfig":
        return BitNetProviderConfig(QuantizationMethod(c.quantization_method),
                                    bool(c.enable_kernel_caching), int(c.max_cache_size),
                                    bool(c.enable_mixed_precision), int(c.memory_optimization_level),
                                    bool(c.enable_simd), "int8" if c.activation == 1 else "ternary",
                                    bool(c.strict_reference_sum), int(c.device))


_vp = C.c_void_p
_u64 = C.c_uint64
_u64p = C.POINTER(C.c_uint64)
_f32p = C.POINTER(C.c_float)
_strs = C.POINTER(C.c_char_p)

PROVIDER_SIGNATURES = {
    "rbp_last_error": (C.c_char_p, []),
    "rbp_default_config": (None, [C.POINTER(_Config)]),
    "rbp_provider_create": (C.c_int, [C.POINTER(_Config), C.POINTER(_vp)]),
    "rbp_provider_destroy": (C.c_int, [_vp]),
    "rbp_provider_id": (C.c_int, [_vp]),
    "rbp_provider_get_config": (C.c_int, [_vp, C.POINTER(_Config)]),
    "rbp_provider_supports": (C.c_int, [_vp, C.c_char_p]),
    "rbp_provider_estimate_speedup": (C.c_float, [_vp, C.c_char_p]),
    "rbp_provider_capability": (C.c_int, [_vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "rbp_provider_has_data_type": (C.c_int, [_vp, C.c_int]),
    "rbp_provider_configure": (C.c_int, [_vp, _u64, C.c_int, _strs, _strs, C.c_int]),
    "rbp_provider_shutdown": (C.c_int, [_vp]),
    "rbp_provider_compile_subgraph": (C.c_int, [_vp, _strs, C.c_int, C.POINTER(_vp)]),
    "rbp_allocate": (C.c_int, [_vp, _u64p, C.c_int, C.c_int, C.POINTER(_vp), _u64p, _u64p]),
    "rbp_deallocate": (C.c_int, [_vp, _vp, _u64, _u64]),
    "rbp_memory_info": (C.c_int, [_vp, _u64p, _u64p, _u64p]),
    "rbp_provider_memory_stats": (C.c_int, [_vp, _u64p, _u64p, _u64p, _f32p]),
    "rbp_create_ternary_matmul_kernel": (C.c_int, [_vp, _u64, _u64, _u64, C.POINTER(_vp)]),
    "rbp_kernel_destroy": (C.c_int, [_vp]),
    "rbp_kernel_execute": (C.c_int, [_vp, C.c_int, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(C.c_int),
                                     C.POINTER(C.c_int), _vp, _u64, _u64p]),
    "rbp_kernel_stats": (C.c_int, [_vp, _u64p, C.POINTER(C.c_double), C.POINTER(C.c_double),
                                   C.POINTER(C.c_double)]),
    "rbp_kernel_memory_usage": (C.c_int, [_vp, _u64p, _u64p, _u64p]),
    "rbp_quantize_ternary": (C.c_int, [_vp, _vp, _u64p, C.c_int, C.c_int, C.POINTER(_vp)]),
    "rbp_ternary_destroy": (C.c_int, [_vp]),
    "rbp_ternary_info": (C.c_int, [_vp, _f32p, _f32p, _u64p, _u64p, _f32p]),
    "rbp_ternary_packed": (C.c_int, [_vp, _vp, _u64]),
    "rbp_ternary_get_value": (C.c_int, [_vp, _u64]),
    "rbp_dequantize_ternary": (C.c_int, [_vp, _vp, _vp, _u64]),
    "rbp_ternary_from_parts": (C.c_int, [_vp, _u64, _u64p, C.c_int, C.c_float, C.c_float, C.POINTER(_vp)]),
    "rbp_ternary_shape": (C.c_int, [_vp, _u64p, C.POINTER(C.c_int)]),
    "rbp_ternary_save": (C.c_int, [_vp, C.c_char_p]),
    "rbp_ternary_load": (C.c_int, [C.c_char_p, C.POINTER(_vp)]),
    "rbp_kernel_execute_prepacked": (C.c_int, [_vp, _vp, _u64p, C.c_int, _vp, _vp, _u64, _u64p]),
    "rbp_kernel_execute_group": (C.c_int, [_vp, C.c_int, _vp, _vp, _u64p, _u64p, _vp, _u64, C.POINTER(C.c_int)]),
}

_bound = None


def _api():
    global _bound
    if _bound is None:
        lib = _lib.load()
        for name, (res, args) in PROVIDER_SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _bound = lib
    return _bound


def _check(rc):
    if rc != 0:
        raise Error(_api().rbp_last_error().decode("utf-8", "replace"))


def _shape_arg(shape):
    return (C.c_uint64 * max(len(shape), 1))(*[int(d) for d in shape])


class TernaryTensor:
    """quantization.rs:249-292."""

    def __init__(self, handle, shape):
        self._h = handle
        self.shape = list(shape)
        s, t, r = C.c_float(), C.c_float(), C.c_float()
        n, m = C.c_uint64(), C.c_uint64()
        _check(_api().rbp_ternary_info(handle, C.byref(s), C.byref(t), C.byref(n), C.byref(m),
                                       C.byref(r)))
        self.scale = np.float32(s.value)
        self.threshold = np.float32(t.value)
        self.element_count = n.value
        self._memory_size = m.value
        self._ratio = np.float32(r.value)
        self.packed_data = np.zeros(m.value, dtype=np.uint8)
        if m.value:
            _check(_api().rbp_ternary_packed(handle, self.packed_data.ctypes.data, m.value))

    @classmethod
    def from_parts(cls, packed_data, shape, scale, threshold) -> "TernaryTensor":
        """A tensor from fields produced elsewhere (e.g. an offline quantiser); checked
        against the invariants of quantize_ternary.  Needs no GPU."""
        packed = np.ascontiguousarray(packed_data, dtype=np.uint8)
        h = _vp()
        _check(_api().rbp_ternary_from_parts(packed.ctypes.data, packed.size, _shape_arg(shape), len(shape),
                                             float(scale), float(threshold), C.byref(h)))
        return cls(h.value, shape)

    def save(self, path: str):
        """Writes the packed-weight file (format: csrc/host/bitnet_provider.hpp)."""
        _check(_api().rbp_ternary_save(self._h, str(path).encode()))

    @classmethod
    def load(cls, path: str) -> "TernaryTensor":
        h = _vp()
        _check(_api().rbp_ternary_load(str(path).encode(), C.byref(h)))
        shape, ndim = (C.c_uint64 * 8)(), C.c_int()
        _check(_api().rbp_ternary_shape(h.value, shape, C.byref(ndim)))
        return cls(h.value, [int(shape[i]) for i in range(ndim.value)])

    def memory_size(self) -> int:
        return self._memory_size

    def compression_ratio(self) -> float:
        return self._ratio

    def get_value(self, index: int) -> int:
        return int(_api().rbp_ternary_get_value(self._h, int(index)))

    def __del__(self):
        try:
            _api().rbp_ternary_destroy(self._h)
        except Exception:
            pass


class BitNetQuantizer:
    """quantization.rs:24-208, ternary half; bound to a provider's device."""

    def __init__(self, method: QuantizationMethod, provider: "BitNetExecutionProvider"):
        self.method = method
        self._provider = provider

    def quantize_ternary(self, tensor: Tensor) -> TernaryTensor:
        data = np.ascontiguousarray(tensor.to_vec(), dtype=np.float32)
        shape = tensor.shape()
        h = _vp()
        _check(_api().rbp_quantize_ternary(self._provider._h, data.ctypes.data, _shape_arg(shape),
                                           len(shape), int(tensor.dtype()), C.byref(h)))
        return TernaryTensor(h.value, shape)

    def dequantize_ternary(self, t: TernaryTensor) -> Tensor:
        out = np.empty(t.element_count, dtype=np.float32)
        _check(_api().rbp_dequantize_ternary(self._provider._h, t._h, out.ctypes.data, out.size))
        return Tensor(out.reshape(tuple(t.shape)), DataType.F32, TensorLayout.RowMajor)

    def quantize_binary(self, tensor: Tensor):
        raise Error("Binary quantization is outside this build: it implements the ternary path")


class BitNetKernel:
    """CompiledKernel (types.rs:153-165) as BitNetKernel implements it (kernels.rs:254-328)."""

    def __init__(self, handle):
        self._h = handle

    def execute(self, inputs: Sequence[Tensor]) -> List[Tensor]:
        n = len(inputs)
        arrays = [np.ascontiguousarray(t.to_vec(), dtype=np.float32) for t in inputs]
        shapes = [_shape_arg(t.shape()) for t in inputs]
        data_p = (_vp * max(n, 1))(*[a.ctypes.data for a in arrays])
        shape_p = (_vp * max(n, 1))(*[C.cast(s, _vp).value for s in shapes])
        ndims = (C.c_int * max(n, 1))(*[len(t.shape()) for t in inputs])
        dtypes = (C.c_int * max(n, 1))(*[int(t.dtype()) for t in inputs])
        cap = 1
        if n >= 2 and len(inputs[0].shape()) == 2 and len(inputs[1].shape()) == 2:
            cap = max(1, inputs[0].shape()[0] * inputs[1].shape()[1])
        out = np.empty(cap, dtype=np.float32)
        out_shape = (C.c_uint64 * 2)()
        _check(_api().rbp_kernel_execute(self._h, n, data_p, shape_p, ndims, dtypes, out.ctypes.data,
                                         cap, out_shape))
        m, nn = out_shape[0], out_shape[1]
        return [Tensor(out[:m * nn].reshape(m, nn), DataType.F32, TensorLayout.RowMajor)]

    def execute_group(self, inputs: Sequence[Tensor]) -> List[Tensor]:
        """Several independent TernaryMatMul nodes of one shape, passed as the pairs
        (A_0, B_0, A_1, B_1, ...): result i is what execute([A_i, B_i]) returns.  In the decode
        regime the nodes share one GPU launch; `last_group_launches` holds the number of
        matmul launches the call issued."""
        if len(inputs) == 0 or len(inputs) % 2:
            raise Error("Ternary MatMul group requires pairs of inputs (A_i, B_i)")
        for t in inputs:
            if t.dtype() != DataType.F32:
                raise Error("BitNet quantization requires FP32 input tensors")
        n = len(inputs) // 2
        a0, b0 = inputs[0], inputs[1]
        if len(a0.shape()) != 2 or len(b0.shape()) != 2:
            raise Error("Matrix dimension mismatch: A=%s, B=%s, expected A=[m,k], B=[k,n]"
                        % (a0.shape(), b0.shape()))
        for i in range(1, n):
            # the C entry point takes one shape for the whole group, so this is checked here
            if inputs[2 * i].shape() != a0.shape() or inputs[2 * i + 1].shape() != b0.shape():
                raise Error("Ternary MatMul group: node %d has A=%s, B=%s, the group's shape is A=%s, B=%s"
                            % (i, inputs[2 * i].shape(), inputs[2 * i + 1].shape(), a0.shape(), b0.shape()))
        a_arr = [np.ascontiguousarray(inputs[2 * i].to_vec(), dtype=np.float32) for i in range(n)]
        b_arr = [np.ascontiguousarray(inputs[2 * i + 1].to_vec(), dtype=np.float32) for i in range(n)]
        m, nn = a0.shape()[0], b0.shape()[1]
        cap = max(1, m * nn)
        outs = [np.empty(cap, dtype=np.float32) for _ in range(n)]
        pa = (_vp * n)(*[x.ctypes.data for x in a_arr])
        pb = (_vp * n)(*[x.ctypes.data for x in b_arr])
        po = (_vp * n)(*[x.ctypes.data for x in outs])
        launches = C.c_int(0)
        _check(_api().rbp_kernel_execute_group(self._h, n, pa, pb, _shape_arg(a0.shape()), _shape_arg(b0.shape()),
                                               po, cap, C.byref(launches)))
        self.last_group_launches = launches.value
        return [Tensor(o[:m * nn].reshape(m, nn), DataType.F32, TensorLayout.RowMajor) for o in outs]

    def execute_prepacked(self, a: Tensor, weights: "TernaryTensor") -> Tensor:
        """TernaryMatMul with weights that are already ternarised (a loaded weight file)."""
        arr = np.ascontiguousarray(a.to_vec(), dtype=np.float32)
        cap = max(1, a.shape()[0] * (weights.shape[1] if len(weights.shape) == 2 else 1))
        out = np.empty(cap, dtype=np.float32)
        out_shape = (C.c_uint64 * 2)()
        _check(_api().rbp_kernel_execute_prepacked(self._h, arr.ctypes.data, _shape_arg(a.shape()),
                                                   len(a.shape()), weights._h, out.ctypes.data, cap,
                                                   out_shape))
        m, nn = out_shape[0], out_shape[1]
        return Tensor(out[:m * nn].reshape(m, nn), DataType.F32, TensorLayout.RowMajor)

    def get_performance_stats(self) -> KernelStats:
        c, a, lo, hi = C.c_uint64(), C.c_double(), C.c_double(), C.c_double()
        _check(_api().rbp_kernel_stats(self._h, C.byref(c), C.byref(a), C.byref(lo), C.byref(hi)))
        return KernelStats(c.value, a.value, lo.value, hi.value)

    def get_memory_usage(self) -> MemoryUsage:
        p, c, n = C.c_uint64(), C.c_uint64(), C.c_uint64()
        _check(_api().rbp_kernel_memory_usage(self._h, C.byref(p), C.byref(c), C.byref(n)))
        return MemoryUsage(p.value, c.value, n.value)

    def __del__(self):
        try:
            _api().rbp_kernel_destroy(self._h)
        except Exception:
            pass


class BitNetMemoryAllocator:
    """TensorAllocator (types.rs:294-303) with the reference's size rules (allocator.rs:39-75)."""

    def __init__(self, provider: "BitNetExecutionProvider"):
        self._provider = provider

    def allocate(self, shape: Sequence[int], dtype: DataType) -> TensorBuffer:
        p, size, align = _vp(), C.c_uint64(), C.c_uint64()
        _check(_api().rbp_allocate(self._provider._h, _shape_arg(shape), len(shape), int(dtype),
                                   C.byref(p), C.byref(size), C.byref(align)))
        return TensorBuffer(p.value, size.value, align.value)

    def deallocate(self, buffer: TensorBuffer) -> None:
        _check(_api().rbp_deallocate(self._provider._h, buffer.ptr, buffer.size, buffer.alignment))

    def get_memory_info(self) -> MemoryInfo:
        t, a, p = C.c_uint64(), C.c_uint64(), C.c_uint64()
        _check(_api().rbp_memory_info(self._provider._h, C.byref(t), C.byref(a), C.byref(p)))
        return MemoryInfo(t.value, a.value, p.value)


class BitNetExecutionProvider:
    """ExecutionProvider (types.rs:192-213) as provider.rs:245-386 implements it."""

    def __init__(self, config: Optional[BitNetProviderConfig] = None):
        cfg = (config or BitNetProviderConfig())._to_c()
        h = _vp()
        _check(_api().rbp_provider_create(C.byref(cfg), C.byref(h)))
        self._h = h.value

    @staticmethod
    def with_config(config: BitNetProviderConfig) -> "BitNetExecutionProvider":
        return BitNetExecutionProvider(config)

    def provider_id(self) -> ProviderId:
        return ProviderId(_api().rbp_provider_id(self._h))

    def get_config(self) -> BitNetProviderConfig:
        c = _Config()
        _check(_api().rbp_provider_get_config(self._h, C.byref(c)))
        return BitNetProviderConfig._from_c(c)

    @property
    def config(self) -> BitNetProviderConfig:
        return self.get_config()

    def get_memory_stats(self) -> dict:                              # provider.rs:121-123
        b, t, saved, ratio = C.c_uint64(), C.c_uint64(), C.c_uint64(), C.c_float()
        _check(_api().rbp_provider_memory_stats(self._h, C.byref(b), C.byref(t), C.byref(saved), C.byref(ratio)))
        return {"binary_tensor_count": b.value, "ternary_tensor_count": t.value,
                "memory_saved_bytes": saved.value, "average_compression_ratio": ratio.value}

    def supports_operation(self, op_type: str) -> bool:
        return bool(_api().rbp_provider_supports(self._h, op_type.encode()))

    def can_handle(self, operators: Sequence[OperatorSpec]) -> List[bool]:
        return [self.supports_operation(op.op_type) for op in operators]

    def estimate_speedup(self, op_spec: OperatorSpec) -> float:
        return float(_api().rbp_provider_estimate_speedup(self._h, op_spec.op_type.encode()))

    def get_capability(self) -> dict:
        n, prof = C.c_int(), C.c_int()
        _check(_api().rbp_provider_capability(self._h, C.byref(n), C.byref(prof)))
        ops = {op for op in ("MatMul", "Gemm", "Conv", "Add", "Sub", "Mul", "And", "Or", "Xor",
                             "BatchNormalization", "ReLU", "Sigmoid", "LSTM", "Softmax")
               if self.supports_operation(op)}
        assert len(ops) == n.value
        return {"supported_ops": ops,
                "data_types": [d for d in DataType
                               if _api().rbp_provider_has_data_type(self._h, int(d))],
                "performance_profile": PerformanceProfile(prof.value)}

    def compile_subgraph(self, subgraph: SubGraph) -> BitNetKernel:
        ops = [n.op_type.encode() for n in subgraph.nodes]
        arr = (C.c_char_p * max(len(ops), 1))(*ops)
        h = _vp()
        _check(_api().rbp_provider_compile_subgraph(self._h, arr, len(ops), C.byref(h)))
        return BitNetKernel(h.value)

    def get_allocator(self) -> BitNetMemoryAllocator:
        return BitNetMemoryAllocator(self)

    def configure(self, config: ProviderConfig) -> None:
        keys = [k.encode() for k in config.custom_options]
        vals = [str(v).encode() for v in config.custom_options.values()]
        ka = (C.c_char_p * max(len(keys), 1))(*keys)
        va = (C.c_char_p * max(len(vals), 1))(*vals)
        _check(_api().rbp_provider_configure(self._h, int(config.memory_limit or 0),
                                             int(config.optimization_level), ka, va, len(keys)))

    def shutdown(self) -> None:
        _check(_api().rbp_provider_shutdown(self._h))

    def quantizer(self) -> BitNetQuantizer:
        return BitNetQuantizer(self.get_config().quantization_method, self)

    def create_ternary_matmul_kernel(self, m: int, n: int, k: int) -> BitNetKernel:
        h = _vp()
        _check(_api().rbp_create_ternary_matmul_kernel(self._h, m, n, k, C.byref(h)))
        return BitNetKernel(h.value)

    def __del__(self):
        try:
            _api().rbp_provider_destroy(self._h)
        except Exception:
            pass


def create_bitnet_provider() -> BitNetExecutionProvider:              # provider.rs:389-391
    return BitNetExecutionProvider()


def create_bitnet_provider_with_config(config: BitNetProviderConfig) -> BitNetExecutionProvider:
    return BitNetExecutionProvider(config)                            # provider.rs:394-398
