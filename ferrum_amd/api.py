"""Host-side mirror of Ferrum's quantized-matmul operator interface over the C ABI.

Names, argument meaning and error behaviour follow the reference so that
tests read like its own:

* ``QuantizationFormat``, ``QuantizedMatrix.from_reader``,
  ``QuantizedExpertMatrix.new``          src/quantization.rs:6-194
* ``DType``, ``Tensor.from_f32`` / ``to_f32`` / ``view``   src/tensor/mod.rs
* ``Device.project_quantized``           src/ops/transformer.rs:96-297
* ``Device.embedding_gather_quantized``  src/ops/transformer.rs:299-360
* ``Device.moe_route`` / ``expert_assign`` / ``expert_project_quantized`` /
  ``expert_silu_mul`` / ``expert_combine``   src/ops/mod.rs:23-551
* ``MoeRoutingPolicy``                   src/model/architecture.rs

Everything computes on the GPU through ``libferrum_hip.so``.  There is no CPU
path: importing this module raises if the library has not been built
(``python -m ferrum_amd.build``).
"""
from __future__ import annotations

import ctypes
import enum
import math
import os
import sys
import time
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("FERRUM_HIP_LIB") or os.path.join(_HERE, "lib", "libferrum_hip.so")


class Error(Exception):
    """ferrum::Error (src/error.rs:3-51); ``kind`` is the variant name."""
    kind = "Error"

    def __init__(self, message: str = ""):
        super().__init__(f"{self.kind}: {message}")
        self.message = message


def _variant(name):
    return type(name, (Error,), {"kind": name})


ShapeError = _variant("Shape")
DTypeError = _variant("DType")
DeviceMismatch = _variant("DeviceMismatch")
RangeError = _variant("Range")
DispatchError = _variant("Dispatch")
SynchronizationError = _variant("Synchronization")
AllocationError = _variant("Allocation")
GgufError = _variant("Gguf")
WeightError = _variant("Weight")
ParameterError = _variant("Parameter")
TokenError = _variant("Token")
ValidationError = _variant("Validation")
ConfigError = _variant("Config")   # host-side only (src/error.rs: Error::Config)

_ERRORS = {1: ShapeError, 2: DTypeError, 3: DeviceMismatch, 4: RangeError, 5: DispatchError,
           6: SynchronizationError, 7: AllocationError, 8: GgufError, 9: WeightError,
           10: ParameterError, 11: TokenError, 12: ValidationError}


class _View(ctypes.Structure):
    _fields_ = [("buffer", ctypes.c_void_p), ("offset", ctypes.c_size_t), ("dtype", ctypes.c_uint32)]


class _Props(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 128), ("arch", ctypes.c_char * 64),
                ("compute_units", ctypes.c_int32), ("wavefront", ctypes.c_int32),
                ("clock_khz", ctypes.c_int32), ("memory_clock_khz", ctypes.c_int32),
                ("memory_bus_bits", ctypes.c_int32), ("lds_bytes_per_block", ctypes.c_int32),
                ("global_bytes", ctypes.c_uint64), ("l2_bytes", ctypes.c_uint64)]


class _Policy(ctypes.Structure):
    _fields_ = [("experts", ctypes.c_uint32), ("top_k", ctypes.c_uint32),
                ("sigmoid", ctypes.c_uint32), ("normalize_top_k_prob", ctypes.c_uint32),
                ("normalization_epsilon", ctypes.c_float), ("routed_scaling_factor", ctypes.c_float)]


# every symbol include/ferrum_hip.h declares: (restype, argtypes)
_P, _SZ, _U32, _U64, _I32, _I64 = (ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32,
                                   ctypes.c_uint64, ctypes.c_int32, ctypes.c_int64)
_VP = ctypes.POINTER(_View)
SYMBOLS = {
    "fh_device_create": (_I32, [_I32, ctypes.POINTER(_P)]),
    "fh_device_destroy": (None, [_P]),
    "fh_device_properties": (_I32, [_P, ctypes.POINTER(_Props)]),
    "fh_synchronize": (_I32, [_P]),
    "fh_last_error": (ctypes.c_char_p, []),
    "fh_last_operation": (ctypes.c_char_p, [_P]),
    "fh_device_stream": (_P, [_P]),
    "fh_set_tuning": (_I32, [_P, ctypes.c_char_p, _I64]),
    "fh_get_tuning": (_I32, [_P, ctypes.c_char_p, ctypes.POINTER(_I64)]),
    "fh_buffer_alloc": (_I32, [_P, _SZ, ctypes.POINTER(_P)]),
    "fh_buffer_free": (None, [_P]),
    "fh_buffer_size": (_SZ, [_P]),
    "fh_buffer_device_ptr": (_P, [_P]),
    "fh_buffer_upload": (_I32, [_P, _SZ, _P, _SZ]),
    "fh_buffer_download": (_I32, [_P, _SZ, _P, _SZ]),
    "fh_buffer_fill_zero": (_I32, [_P, _SZ, _SZ]),
    "fh_qmatrix_create": (_I32, [_P, _U32, _U64, _U64, _U64, _P, _SZ, ctypes.POINTER(_P)]),
    "fh_qmatrix_destroy": (None, [_P]),
    "fh_qmatrix_rows": (_U64, [_P]),
    "fh_qmatrix_columns": (_U64, [_P]),
    "fh_qmatrix_experts": (_U64, [_P]),
    "fh_qmatrix_ggml_type": (_U32, [_P]),
    "fh_qmatrix_byte_size": (_SZ, [_P]),
    "fh_qmatrix_device_ptr": (_P, [_P]),
    "fh_dequantize": (_I32, [_P, _P, _VP]),
    "fh_embedding_gather_quantized": (_I32, [_P, _P, ctypes.POINTER(_U32), _SZ, _VP]),
    "fh_project_quantized": (_I32, [_P, _P, _VP, _U32, _VP]),
    "fh_project_quantized_no_alloc": (_I32, [_P, _P, _VP, _U32, _VP]),
    "fh_probe_read": (_I32, [_P, _P]),
    "fh_probe_mfma": (_I32, [_P, _U32, _U32, _U32, ctypes.POINTER(ctypes.c_double)]),
    "fh_probe_coissue": (_I32, [_P, _U32, _U32, _U32, _U32]),
    "fh_argmax_rows": (_I32, [_P, _VP, _U32, _U32, _VP]),
    "fh_add_rmsnorm": (_I32, [_P, _VP, _VP, _VP, _U32, _U32, ctypes.c_float, _VP, _VP]),
    "fh_moe_route": (_I32, [_P, _VP, _U32, _VP, ctypes.POINTER(_Policy), _VP]),
    "fh_moe_route_ranked": (_I32, [_P, _VP, _U32, ctypes.POINTER(_Policy), _VP, _VP, _U32, _VP, _VP]),
    "fh_moe_ffn": (_I32, [_P, _VP, _VP, _U32, _VP, ctypes.POINTER(_Policy), _P, _P, _P, _P, _VP, _VP]),
    "fh_expert_combine_shared": (_I32, [_P, _VP, _VP, _U32, _U32, _U32, _VP, _VP, _VP]),
    "fh_hybrid_moe_route": (_I32, [_P, _VP, _U32, ctypes.POINTER(_Policy), _VP, _VP, _U32, _VP, _VP, _VP]),
    "fh_hybrid_project": (_I32, [_P, _P, _VP, _U32, _VP, _U32]),
    "fh_hybrid_project_id": (_I32, [_P, _P, _VP, _VP, _U32, _U32, _VP]),
    "fh_hybrid_project_id_with_shared": (_I32, [_P, _P, _P, _VP, _VP, _U32, _U32, _U32, _VP, _VP, _VP]),
    "fh_hybrid_moe_map": (_I32, [_P, _VP, _U32, _U32, _VP, _VP, _VP]),
    "fh_hybrid_moe_gather": (_I32, [_P, _VP, _VP, _U32, _U32, _U32, _VP]),
    "fh_hybrid_project_mm_id": (_I32, [_P, _P, _VP, _VP, _U32, _VP]),
    "fh_hybrid_project_mm_id_with_shared": (_I32, [_P, _P, _P, _VP, _VP, _U32, _U32, _VP, _VP, _VP]),
    "fh_hybrid_moe_combine": (_I32, [_P, _VP, _VP, _VP, _VP, _VP, _U32, _U32, _U32, _VP]),
    "fh_expert_assign": (_I32, [_P, _VP, _U32, _U32, _VP, _U32, _VP]),
    "fh_expert_project_quantized": (_I32, [_P, _P, _VP, _U32, _VP, _VP]),
    "fh_expert_project_fused": (_I32, [_P, _P, _VP, _U32, _U32, _U32, _VP, _VP]),
    "fh_project_silu_mul_quantized": (_I32, [_P, _P, _VP, _U32, _VP]),
    "fh_expert_project_with_shared": (_I32, [_P, _P, _P, _VP, _U32, _U32, _U32, _VP, _VP, _VP, _VP]),
    "fh_expert_silu_mul": (_I32, [_P, _VP, _U32, _U32, _VP]),
    "fh_expert_combine": (_I32, [_P, _VP, _VP, _U32, _U32, _U32, _VP]),
    "fh_execution_begin": (_I32, [_P]),
    "fh_execution_end": (_I32, [_P, ctypes.POINTER(_P)]),
    "fh_graph_launch": (_I32, [_P]),
    "fh_graph_destroy": (None, [_P]),
    "fh_event_create": (_I32, [_P, ctypes.POINTER(_P)]),
    "fh_event_destroy": (None, [_P]),
    "fh_event_record": (_I32, [_P]),
    "fh_event_elapsed_ms": (_I32, [_P, _P, ctypes.POINTER(ctypes.c_float)]),
}


def load_library(path: str = LIB_PATH) -> ctypes.CDLL:
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it with `python -m ferrum_amd.build` "
                          "(there is no CPU fallback)")
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


_lib = load_library()


def _check(status: int):
    if status != 0:
        message = _lib.fh_last_error().decode("utf-8", "replace")
        raise _ERRORS.get(status, Error)(message)


class DType(enum.IntEnum):
    F32 = 0
    F16 = 1
    BF16 = 2

    def size_bytes(self) -> int:
        return 4 if self == DType.F32 else 2


class QuantizationFormat(enum.Enum):
    Q8_0 = 8       # the hybrid engine's Format::Q8_0: 34-byte blocks of 32 weights (src/loader/gguf.rs:99)
    Q4_K = 12
    Q5_K = 13
    Q6_K = 14
    IQ4_XS = 23    # the hybrid engine's Format::Iq4Xs (src/hybrid/weights.rs:38-60)

    @staticmethod
    def from_ggml_type(type_id: int) -> "QuantizationFormat":
        try:
            return QuantizationFormat(type_id)
        except ValueError:
            raise GgufError(f"unsupported quantized weight type {type_id}") from None

    def ggml_type(self) -> int:
        return self.value

    def block_elements(self) -> int:
        """Weights per block: a row is a whole number of them (256, or 32 for Q8_0)."""
        return 32 if self.value == 8 else 256

    def block_bytes(self) -> int:
        return {8: 34, 12: 144, 13: 176, 14: 210, 23: 136}[self.value]


def _f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(a)
    if nan.any():
        rounded[nan] = ((bits[nan] >> 16) | 0x40).astype(np.uint16)
    return rounded


def encode(values: np.ndarray, dtype: DType) -> np.ndarray:
    """f32 -> storage bytes (round to nearest even), as Tensor::from_f32 does."""
    a = np.ascontiguousarray(values, dtype=np.float32)
    if dtype == DType.F32:
        return a
    if dtype == DType.F16:
        with np.errstate(over="ignore"):
            return a.astype(np.float16)
    return _f32_to_bf16_bits(a)


def decode(raw: np.ndarray, dtype: DType) -> np.ndarray:
    if dtype == DType.F32:
        return raw.view(np.float32).copy()
    if dtype == DType.F16:
        return raw.view(np.float16).astype(np.float32)
    return (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32)


class Buffer:
    def __init__(self, device: "Device", nbytes: int):
        self.device = device
        handle = ctypes.c_void_p()
        _check(_lib.fh_buffer_alloc(device._handle, nbytes, ctypes.byref(handle)))
        self._handle = handle
        self.nbytes = nbytes

    def upload(self, offset: int, data: np.ndarray):
        data = np.ascontiguousarray(data)
        _check(_lib.fh_buffer_upload(self._handle, offset, data.ctypes.data, data.nbytes))

    def download(self, offset: int, nbytes: int) -> np.ndarray:
        out = np.empty(nbytes, dtype=np.uint8)
        _check(_lib.fh_buffer_download(self._handle, offset, out.ctypes.data, nbytes))
        return out

    def device_ptr(self) -> int:
        return _lib.fh_buffer_device_ptr(self._handle) or 0

    def __del__(self):
        if sys.is_finalizing():   # the HIP runtime may already be gone at interpreter exit
            return
        h, self._handle = getattr(self, "_handle", None), None
        if h:
            _lib.fh_buffer_free(h)


class Tensor:
    """Dense row-major tensor: a typed window on a Buffer."""

    def __init__(self, buffer: Buffer, offset: int, shape, dtype: DType):
        self.buffer, self.offset, self.dtype = buffer, offset, DType(dtype)
        self._shape = tuple(int(d) for d in shape)

    @staticmethod
    def zeros(device: "Device", shape, dtype: DType) -> "Tensor":
        shape = tuple(int(d) for d in shape)
        n = int(np.prod(shape, dtype=np.int64)) if shape else 1
        return Tensor(Buffer(device, max(n, 1) * DType(dtype).size_bytes()), 0, shape, dtype)

    @staticmethod
    def from_f32(device: "Device", shape, dtype: DType, values) -> "Tensor":
        shape = tuple(int(d) for d in shape)
        a = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)
        if a.size != int(np.prod(shape, dtype=np.int64)):
            raise ShapeError("value count does not match shape")
        t = Tensor.zeros(device, shape, dtype)
        if a.size:
            t.buffer.upload(0, encode(a, DType(dtype)))
        return t

    @staticmethod
    def from_bits(device: "Device", shape, values_u32) -> "Tensor":
        """F32-typed carrier of raw 32-bit words (the reference stores ids so)."""
        a = np.ascontiguousarray(values_u32, dtype=np.uint32).reshape(-1)
        t = Tensor.zeros(device, shape, DType.F32)
        t.buffer.upload(0, a)
        return t

    def shape(self):
        return self._shape

    def numel(self) -> int:
        return int(np.prod(self._shape, dtype=np.int64)) if self._shape else 1

    def byte_size(self) -> int:
        return self.numel() * self.dtype.size_bytes()

    def view(self, element_offset: int, shape) -> "Tensor":
        shape = tuple(int(d) for d in shape)
        n = int(np.prod(shape, dtype=np.int64))
        if element_offset < 0 or element_offset + n > self.numel():
            raise RangeError("view exceeds tensor")
        return Tensor(self.buffer, self.offset + element_offset * self.dtype.size_bytes(), shape,
                      self.dtype)

    def to_f32(self) -> np.ndarray:
        raw = self.buffer.download(self.offset, self.byte_size())
        return decode(raw, self.dtype).reshape(self._shape)

    def raw(self) -> np.ndarray:
        return self.buffer.download(self.offset, self.byte_size())

    def _view(self) -> _View:
        return _View(self.buffer._handle, self.offset, int(self.dtype))


@dataclass
class Output:
    """src/ops/mod.rs:8-21: the result tensor plus Metrics.operation / bytes."""
    tensor: Tensor
    operation: str
    bytes_read: int = 0
    bytes_written: int = 0


class QuantizedMatrix:
    """Row-major [rows, columns] matrix of verbatim GGUF super-blocks."""

    def __init__(self, device, handle, rows, columns, fmt):
        self.device, self._handle = device, handle
        self._rows, self._columns, self._format = rows, columns, fmt

    @staticmethod
    def from_reader(device: "Device", rows: int, columns: int, fmt: QuantizationFormat, fill,
                    experts: int = 1) -> "QuantizedMatrix":
        """``fill(destination)`` writes the packed payload into a uint8 array,
        like the reference's FnOnce(&mut [u8]) reader."""
        total_rows = rows * experts
        if total_rows == 0 or columns == 0 or columns % fmt.block_elements() != 0:
            raise ShapeError(f"{fmt.name} matrix requires nonempty rows and columns divisible by "
                             f"block size {fmt.block_elements()}")
        byte_len = total_rows * (columns // fmt.block_elements()) * fmt.block_bytes()
        destination = np.zeros(byte_len, dtype=np.uint8)
        fill(destination)
        return QuantizedMatrix.from_bytes(device, rows, columns, fmt, destination, experts)

    @staticmethod
    def from_bytes(device, rows, columns, fmt, payload, experts: int = 1) -> "QuantizedMatrix":
        ggml = fmt.value if isinstance(fmt, QuantizationFormat) else int(fmt)
        payload = np.ascontiguousarray(payload, dtype=np.uint8)
        handle = ctypes.c_void_p()
        _check(_lib.fh_qmatrix_create(device._handle, ggml, rows, columns, experts,
                                      payload.ctypes.data, payload.nbytes, ctypes.byref(handle)))
        return QuantizedMatrix(device, handle, rows * experts, columns, QuantizationFormat(ggml))

    def rows(self) -> int:
        return self._rows

    def columns(self) -> int:
        return self._columns

    def format(self) -> QuantizationFormat:
        return self._format

    def byte_size(self) -> int:
        return int(_lib.fh_qmatrix_byte_size(self._handle))

    def device_ptr(self) -> int:
        return _lib.fh_qmatrix_device_ptr(self._handle) or 0

    def __del__(self):
        if sys.is_finalizing():   # the HIP runtime may already be gone at interpreter exit
            return
        h, self._handle = getattr(self, "_handle", None), None
        if h:
            _lib.fh_qmatrix_destroy(h)


class QuantizedExpertMatrix:
    """[experts, rows_per_expert, columns] stored as one packed matrix with the
    expert axis flattened into rows."""

    def __init__(self, device, handle, experts, rows_per_expert, columns, fmt):
        self.device, self._handle = device, handle
        self._experts, self._rows, self._columns, self._format = experts, rows_per_expert, columns, fmt

    @staticmethod
    def new(device, payload, fmt: QuantizationFormat, experts: int, rows_per_expert: int,
            columns: int) -> "QuantizedExpertMatrix":
        if experts == 0 or rows_per_expert == 0:
            raise ShapeError("quantized expert matrix row geometry mismatch")
        payload = np.ascontiguousarray(payload, dtype=np.uint8)
        handle = ctypes.c_void_p()
        _check(_lib.fh_qmatrix_create(device._handle, fmt.value, rows_per_expert, columns, experts,
                                      payload.ctypes.data, payload.nbytes, ctypes.byref(handle)))
        return QuantizedExpertMatrix(device, handle, experts, rows_per_expert, columns, fmt)

    def experts(self) -> int:
        return self._experts

    def rows_per_expert(self) -> int:
        return self._rows

    def columns(self) -> int:
        return self._columns

    def format(self) -> QuantizationFormat:
        return self._format

    def byte_size(self) -> int:
        return int(_lib.fh_qmatrix_byte_size(self._handle))

    def matrix_view(self) -> QuantizedMatrix:
        """The flattened [experts*rows, columns] matrix (shares storage; the
        returned object does not own the handle)."""
        m = QuantizedMatrix(self.device, None, self._experts * self._rows, self._columns, self._format)
        m._borrowed = self._handle
        return m

    def __del__(self):
        if sys.is_finalizing():   # the HIP runtime may already be gone at interpreter exit
            return
        h, self._handle = getattr(self, "_handle", None), None
        if h:
            _lib.fh_qmatrix_destroy(h)


class MoeScoringFunction(enum.Enum):
    Softmax = 0
    Sigmoid = 1


@dataclass
class MoeRoutingPolicy:
    experts: int
    top_k: int
    scoring_function: MoeScoringFunction = MoeScoringFunction.Softmax
    normalize_top_k_prob: bool = True
    normalization_epsilon: float = 0.0
    routed_scaling_factor: float = 1.0
    use_expert_bias: bool = False

    @staticmethod
    def softmax(experts: int, top_k: int) -> "MoeRoutingPolicy":
        return MoeRoutingPolicy(experts, top_k)

    def _c(self) -> _Policy:
        return _Policy(self.experts, self.top_k,
                       int(self.scoring_function == MoeScoringFunction.Sigmoid),
                       int(self.normalize_top_k_prob), self.normalization_epsilon,
                       self.routed_scaling_factor)


@dataclass
class MoeStats:
    """What SparseMoe.forward did since the last take_stats (MoeStats, src/nn/moe.rs:75-116).
    Durations are host seconds spent enqueueing; routing runs on the device, so the set of
    active experts is never read back and `active_experts_known` turns false with the first
    forward pass."""
    router_projection_enqueue: float = 0.0
    routing: float = 0.0
    routing_boundary_wait: float = 0.0
    expert_dispatch: float = 0.0
    combine_dispatch: float = 0.0
    active_experts: int = 0
    active_experts_known: bool = True
    assignments: int = 0
    peak_temporary_bytes: int = 0

    def merge(self, other: "MoeStats") -> None:
        self.router_projection_enqueue += other.router_projection_enqueue
        self.routing += other.routing
        self.routing_boundary_wait += other.routing_boundary_wait
        self.expert_dispatch += other.expert_dispatch
        self.combine_dispatch += other.combine_dispatch
        self.active_experts += other.active_experts
        self.active_experts_known = self.active_experts_known and other.active_experts_known
        self.assignments += other.assignments
        self.peak_temporary_bytes = max(self.peak_temporary_bytes, other.peak_temporary_bytes)


class Event:
    def __init__(self, device: "Device"):
        handle = ctypes.c_void_p()
        _check(_lib.fh_event_create(device._handle, ctypes.byref(handle)))
        self._handle = handle

    def record(self):
        _check(_lib.fh_event_record(self._handle))

    def elapsed_ms(self, stop: "Event") -> float:
        ms = ctypes.c_float()
        _check(_lib.fh_event_elapsed_ms(self._handle, stop._handle, ctypes.byref(ms)))
        return float(ms.value)

    def __del__(self):
        if sys.is_finalizing():   # the HIP runtime may already be gone at interpreter exit
            return
        h, self._handle = getattr(self, "_handle", None), None
        if h:
            _lib.fh_event_destroy(h)


class Graph:
    """A recorded batch of operator calls (the reference's Execution scope),
    replayable with launch()."""

    def __init__(self, device: "Device", handle):
        self.device, self._handle = device, handle

    def launch(self):
        _check(_lib.fh_graph_launch(self._handle))

    def __del__(self):
        if sys.is_finalizing():   # the HIP runtime may already be gone at interpreter exit
            return
        h, self._handle = getattr(self, "_handle", None), None
        if h:
            _lib.fh_graph_destroy(h)


class Execution:
    """with device.execution() as e: ...ops with preallocated outputs...; e.graph.launch()"""

    def __init__(self, device: "Device"):
        self.device, self.graph = device, None

    def __enter__(self):
        _check(_lib.fh_execution_begin(self.device._handle))
        return self

    def __exit__(self, exc_type, exc, tb):
        handle = ctypes.c_void_p()
        status = _lib.fh_execution_end(self.device._handle, ctypes.byref(handle))
        if exc_type is None:
            _check(status)
            self.graph = Graph(self.device, handle)
        elif handle:
            _lib.fh_graph_destroy(handle)
        return False


class Device:
    """One gfx950 GPU and its stream (the reference's MetalDevice)."""

    def __init__(self, ordinal: int = 0):
        handle = ctypes.c_void_p()
        _check(_lib.fh_device_create(ordinal, ctypes.byref(handle)))
        self._handle = handle

    @staticmethod
    def new(ordinal: int = 0) -> "Device":
        return Device(ordinal)

    def properties(self) -> dict:
        p = _Props()
        _check(_lib.fh_device_properties(self._handle, ctypes.byref(p)))
        return {f: (getattr(p, f).decode() if isinstance(getattr(p, f), bytes) else getattr(p, f))
                for f, _ in _Props._fields_}

    def synchronize(self):
        _check(_lib.fh_synchronize(self._handle))

    def last_operation(self) -> str:
        return _lib.fh_last_operation(self._handle).decode()

    def set_tuning(self, key: str, value: int):
        _check(_lib.fh_set_tuning(self._handle, key.encode(), value))

    def get_tuning(self, key: str) -> int:
        v = ctypes.c_int64()
        _check(_lib.fh_get_tuning(self._handle, key.encode(), ctypes.byref(v)))
        return int(v.value)

    def set_k_quant_gemv_ksplit(self, simds: int):
        self.set_tuning("k_quant_gemv_ksplit", simds)

    def set_moe_routing_temporary_limit(self, nbytes: int):
        """Bound on the routing temporaries of one SparseMoe chunk
        (set_moe_routing_temporary_limit, src/metal/legacy.rs:520-534; 128 MiB at first)."""
        self.set_tuning("moe_routing_temporary_limit", nbytes)

    def moe_routing_temporary_limit(self) -> int:
        return self.get_tuning("moe_routing_temporary_limit")

    def event(self) -> Event:
        return Event(self)

    def execution(self) -> Execution:
        return Execution(self)

    # ---- operators ---------------------------------------------------------

    def dequantize(self, weight, dtype: DType = DType.F32) -> Tensor:
        rows = weight.rows() if isinstance(weight, QuantizedMatrix) else weight.experts() * weight.rows_per_expert()
        out = Tensor.zeros(self, (rows, weight.columns()), dtype)
        v = out._view()
        _check(_lib.fh_dequantize(self._handle, _handle_of(weight), ctypes.byref(v)))
        return out

    def embedding_gather_quantized(self, weight: QuantizedMatrix, tokens, output_dtype: DType) -> Output:
        ids = np.ascontiguousarray(tokens, dtype=np.uint32)
        out = Tensor.zeros(self, (ids.size, weight.columns()), output_dtype)
        v = out._view()
        _check(_lib.fh_embedding_gather_quantized(
            self._handle, _handle_of(weight), ids.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)),
            ids.size, ctypes.byref(v)))
        return Output(out, self.last_operation())

    def project_quantized(self, a: Tensor, weight: QuantizedMatrix, out_dtype: DType | None = None,
                          out: Tensor | None = None, silu_mul: bool = False) -> Output:
        """``silu_mul=True`` takes ``a`` as [M, 2K] (gate first) and projects
        round(round(silu(gate)) * up), as expert_silu_mul followed by this call would."""
        dims = a.shape()
        if (len(dims) != 2 or dims[1] != weight.columns() * (2 if silu_mul else 1)
                or dims[1] > 0xFFFFFFFF - 32):
            raise ShapeError("quantized projection requires [M,K] matching [N,K]")
        if a.buffer.device is not self or weight.device is not self:
            raise DeviceMismatch("tensor or weight belongs to another device")
        m, n = dims[0], weight.rows()
        dtype = a.dtype if out_dtype is None else DType(out_dtype)
        if out is None:
            out = Tensor.zeros(self, (m, n), dtype)
        if m == 0:
            return Output(out, "")
        xv, yv = a._view(), out._view()
        call = _lib.fh_project_silu_mul_quantized if silu_mul else _lib.fh_project_quantized
        _check(call(self._handle, _handle_of(weight), ctypes.byref(xv), m, ctypes.byref(yv)))
        return Output(out, self.last_operation(), a.byte_size() + weight.byte_size(), out.byte_size())

    def project_quantized_no_alloc(self, a: Tensor, weight, out: Tensor) -> Output:
        """fh_project_quantized_no_alloc: the per-row GEMV kernels with the library's fixed
        scratch; the caller brings the output, nothing is allocated on the device."""
        dims = a.shape()
        if len(dims) != 2 or dims[1] != weight.columns() or out.shape() != (dims[0], weight.rows()):
            raise ShapeError("quantized projection requires [M,K] matching [N,K]")
        xv, yv = a._view(), out._view()
        _check(_lib.fh_project_quantized_no_alloc(self._handle, _handle_of(weight), ctypes.byref(xv), dims[0],
                                                  ctypes.byref(yv)))
        return Output(out, self.last_operation(), a.byte_size() + weight.byte_size(), out.byte_size())

    def probe_read(self, weight) -> None:
        """fh_probe_read: reads every byte of a resident matrix with 128-bit loads and
        writes nothing (a measurement kernel; the reference has none)."""
        _check(_lib.fh_probe_read(self._handle, _handle_of(weight)))

    def probe_mfma(self, shape: int, groups: int, iterations: int) -> float:
        """fh_probe_mfma: an MFMA issue loop from registers (shape 0 = 16x16x32 f16,
        1 = 32x32x16 f16, 2 = 32x32x16 f16 on pseudo-random operands); returns the
        floating-point operations of the launch."""
        flops = ctypes.c_double()
        _check(_lib.fh_probe_mfma(self._handle, shape, groups, iterations, ctypes.byref(flops)))
        return float(flops.value)

    def probe_coissue(self, groups: int, iterations: int, mfma: bool, valu_rounds: int) -> None:
        """fh_probe_coissue: an MFMA wave and a VALU wave on every SIMD, either or both."""
        _check(_lib.fh_probe_coissue(self._handle, groups, iterations, int(mfma), valu_rounds))

    def argmax_rows(self, logits: Tensor) -> Tensor:
        """[rows, 2] F32 carrier of u32 bits: first maximal index and a non-finite flag
        (MetalDevice::argmax_rows, src/ops/transformer.rs:768-792)."""
        dims = logits.shape()
        if len(dims) != 2 or 0 in dims or dims[1] > 0xFFFFFFFF:
            raise ShapeError("argmax requires nonempty [rows,width]")
        if logits.buffer.device is not self:
            raise DeviceMismatch("tensor belongs to another device")
        out = Tensor.zeros(self, (dims[0], 2), DType.F32)
        lv, ov = logits._view(), out._view()
        _check(_lib.fh_argmax_rows(self._handle, ctypes.byref(lv), dims[0], dims[1], ctypes.byref(ov)))
        return out

    def add_rmsnorm(self, a: Tensor, b: Tensor, weight: Tensor, epsilon: float,
                    residual: Tensor | None = None, normed: Tensor | None = None) -> tuple[Tensor, Tensor]:
        """(residual, normed): residual = a + b in the operands' dtype, normed =
        rmsnorm(residual) * weight (MetalDevice::add_rmsnorm, src/ops/mod.rs:762-820).
        `residual` / `normed` may be passed in to reuse buffers."""
        dims = a.shape()
        if len(dims) == 0 or dims[-1] == 0 or a.numel() == 0:
            raise ShapeError("last dimension must be nonzero")
        width = dims[-1]
        if a.shape() != b.shape() or a.dtype != b.dtype or weight.dtype != a.dtype:
            raise ShapeError("fused add+RMSNorm operands must match")
        if weight.shape() != (width,) or width > 0xFFFFFFFF - 256:
            raise ShapeError("RMSNorm weight must match the last dimension")
        if not math.isfinite(epsilon) or epsilon <= 0:
            raise ParameterError("epsilon must be finite and positive")
        if any(t.buffer.device is not self for t in (a, b, weight)):
            raise DeviceMismatch("tensor belongs to another device")
        residual = residual if residual is not None else Tensor.zeros(self, dims, a.dtype)
        normed = normed if normed is not None else Tensor.zeros(self, dims, a.dtype)
        views = [t._view() for t in (a, b, weight, residual, normed)]
        _check(_lib.fh_add_rmsnorm(self._handle, ctypes.byref(views[0]), ctypes.byref(views[1]),
                                   ctypes.byref(views[2]), a.numel() // width, width, epsilon,
                                   ctypes.byref(views[3]), ctypes.byref(views[4])))
        return residual, normed

    def moe_route(self, logits: Tensor, selection_bias: Tensor | None, policy: MoeRoutingPolicy,
                  out: Tensor | None = None) -> Tensor:
        dims = logits.shape()
        if len(dims) != 2 or dims[0] == 0 or dims[1] == 0 or dims[1] != policy.experts:
            raise ShapeError("invalid sparse routing geometry")
        if selection_bias is not None and (selection_bias.shape() != (policy.experts,)
                                           or selection_bias.dtype != DType.F32):
            raise ShapeError("invalid sparse routing geometry")
        if out is None:
            out = Tensor.zeros(self, (dims[0] * max(policy.top_k, 1), 3), DType.F32)
        lv, ov, pc = logits._view(), out._view(), policy._c()
        bv = selection_bias._view() if selection_bias is not None else None
        _check(_lib.fh_moe_route(self._handle, ctypes.byref(lv), dims[0],
                                 ctypes.byref(bv) if bv is not None else None, ctypes.byref(pc),
                                 ctypes.byref(ov)))
        return out

    def moe_route_ranked(self, logits: Tensor, policy: MoeRoutingPolicy, x: Tensor | None = None,
                         gate_vector: Tensor | None = None, want_gate: bool = False):
        """The hybrid engine's router (h_moe_route, src/metal/shaders/hybrid.metal:2259-2319):
        metadata rows in selection order, and the shared-expert gate
        sigmoid(dot(x[t], gate_vector)) per token (ones without a vector).
        Returns (metadata, shared_gate or None)."""
        dims = logits.shape()
        if len(dims) != 2 or dims[0] == 0 or dims[1] != policy.experts:
            raise ShapeError("invalid sparse routing geometry")
        if gate_vector is not None and (x is None or x.shape() != (dims[0], gate_vector.shape()[0])
                                        or gate_vector.dtype != DType.F32):
            raise ShapeError("the shared-expert gate needs x [tokens, hidden] and an f32 vector [hidden]")
        meta = Tensor.zeros(self, (dims[0] * policy.top_k, 3), DType.F32)
        gate = Tensor.zeros(self, (dims[0],), DType.F32) if (want_gate or gate_vector is not None) else None
        lv, mv, pc = logits._view(), meta._view(), policy._c()
        xv = x._view() if gate_vector is not None else None
        wv = gate_vector._view() if gate_vector is not None else None
        gv = gate._view() if gate is not None else None
        ref = lambda v: ctypes.byref(v) if v is not None else None
        _check(_lib.fh_moe_route_ranked(self._handle, ctypes.byref(lv), dims[0], ctypes.byref(pc), ref(xv), ref(wv),
                                        gate_vector.shape()[0] if gate_vector is not None else 0,
                                        ctypes.byref(mv), ref(gv)))
        return meta, gate

    # ---- the hybrid engine's routed FFN in its own layout (ids / weights as plain arrays) ----

    def hybrid_moe_route(self, logits: Tensor, policy: MoeRoutingPolicy, x: Tensor | None = None,
                         gate_vector: Tensor | None = None):
        """h_moe_route (src/metal/shaders/hybrid.metal:2259-2319): (ids, weights, shared_gate),
        ids and weights [tokens * top_k] in selection order, ids as u32 bits in an F32 carrier."""
        dims = logits.shape()
        if len(dims) != 2 or dims[0] == 0 or dims[1] != policy.experts:
            raise ShapeError("invalid sparse routing geometry")
        if gate_vector is not None and (x is None or x.shape() != (dims[0], gate_vector.shape()[0])
                                        or gate_vector.dtype != DType.F32):
            raise ShapeError("the shared-expert gate needs x [tokens, hidden] and an f32 vector [hidden]")
        ids = Tensor.zeros(self, (dims[0] * policy.top_k,), DType.F32)
        weights = Tensor.zeros(self, (dims[0] * policy.top_k,), DType.F32)
        gate = Tensor.zeros(self, (dims[0],), DType.F32)
        lv, iv, wtv, gv, pc = logits._view(), ids._view(), weights._view(), gate._view(), policy._c()
        xv = x._view() if gate_vector is not None else None
        wv = gate_vector._view() if gate_vector is not None else None
        ref = lambda v: ctypes.byref(v) if v is not None else None
        _check(_lib.fh_hybrid_moe_route(self._handle, ctypes.byref(lv), dims[0], ctypes.byref(pc), ref(xv), ref(wv),
                                        gate_vector.shape()[0] if gate_vector is not None else 0,
                                        ctypes.byref(iv), ctypes.byref(wtv), ctypes.byref(gv)))
        return ids, weights, gate

    def hybrid_project(self, weight: QuantizedMatrix, x: Tensor, exact: bool = False,
                       out_dtype: DType | None = None) -> Output:
        """HybridModel::project (src/hybrid/engine.rs:3407-3500): exact f32 weights for 1..4 rows
        (or always with `exact`), f16 tiles from 5 rows on."""
        dims = x.shape()
        if len(dims) != 2 or dims[0] == 0 or dims[1] != weight.columns():
            raise ShapeError("quantized projection requires [M,K] matching [N,K]")
        y = Tensor.zeros(self, (dims[0], weight.rows()), out_dtype or x.dtype)
        xv, yv = x._view(), y._view()
        _check(_lib.fh_hybrid_project(self._handle, _handle_of(weight), ctypes.byref(xv), dims[0], ctypes.byref(yv),
                                      1 if exact else 0))
        return Output(y, self.last_operation(), x.byte_size() + weight.byte_size(), y.byte_size())

    def hybrid_project_id(self, weight: "QuantizedExpertMatrix", x: Tensor, ids: Tensor, routes: int, x_div: int,
                          out_dtype: DType | None = None) -> Tensor:
        """HybridModel::project_id (src/hybrid/engine.rs:3113-3148): route r multiplies activation
        row r / x_div by expert ids[r]."""
        if (routes == 0 or x_div == 0 or routes % x_div or ids.shape() != (routes,) or ids.dtype != DType.F32
                or x.shape() != (routes // x_div, weight.columns())):
            raise ShapeError("expert projection geometry")
        y = Tensor.zeros(self, (routes, weight.rows_per_expert()), out_dtype or x.dtype)
        xv, iv, yv = x._view(), ids._view(), y._view()
        _check(_lib.fh_hybrid_project_id(self._handle, _handle_of(weight), ctypes.byref(xv), ctypes.byref(iv), routes,
                                         x_div, ctypes.byref(yv)))
        return y

    def hybrid_project_id_with_shared(self, weight: "QuantizedExpertMatrix", shared_weight: "QuantizedMatrix",
                                      x: Tensor, ids: Tensor, routes: int, x_div: int, tokens: int,
                                      shared_x: Tensor | None = None):
        """``hybrid_project_id`` and, in the same launch, the shared expert's projection of every
        token with the dense ``shared_weight``: from ``shared_x`` [tokens, K] when given (the down
        projection), else from the token rows ``x`` (gate, up).  Returns (y [routes, N],
        shared_y [tokens, N])."""
        if (routes == 0 or x_div == 0 or routes % x_div or ids.shape() != (routes,) or ids.dtype != DType.F32
                or x.shape() != (routes // x_div, weight.columns()) or tokens == 0
                or (shared_x is None and tokens != routes // x_div)
                or (shared_x is not None and (shared_x.shape() != (tokens, weight.columns())
                                              or shared_x.dtype != x.dtype))
                or shared_weight.rows() != weight.rows_per_expert() or shared_weight.columns() != weight.columns()
                or shared_weight.format().ggml_type() != weight.format().ggml_type()):
            raise ShapeError("expert projection geometry")
        y = Tensor.zeros(self, (routes, weight.rows_per_expert()), x.dtype)
        ys = Tensor.zeros(self, (tokens, weight.rows_per_expert()), x.dtype)
        xv, iv, yv, ysv = x._view(), ids._view(), y._view(), ys._view()
        sxv = shared_x._view() if shared_x is not None else None
        _check(_lib.fh_hybrid_project_id_with_shared(
            self._handle, _handle_of(weight), _handle_of(shared_weight), ctypes.byref(xv), ctypes.byref(iv), routes,
            x_div, tokens, ctypes.byref(sxv) if sxv is not None else None, ctypes.byref(yv), ctypes.byref(ysv)))
        return y, ys

    def hybrid_moe_map(self, ids: Tensor, experts: int):
        """h_moe_map (hybrid.metal:2321-2358): (offsets [experts + 1], sorted [routes], position
        [routes]) as u32 bits in F32 carriers."""
        routes = ids.numel()
        if routes == 0 or ids.dtype != DType.F32:
            raise ShapeError("route map needs routes")
        offsets = Tensor.zeros(self, (experts + 1,), DType.F32)
        order = Tensor.zeros(self, (routes,), DType.F32)
        position = Tensor.zeros(self, (routes,), DType.F32)
        iv, ov, sv, pv = ids._view(), offsets._view(), order._view(), position._view()
        _check(_lib.fh_hybrid_moe_map(self._handle, ctypes.byref(iv), experts, routes, ctypes.byref(ov),
                                      ctypes.byref(sv), ctypes.byref(pv)))
        return offsets, order, position

    def hybrid_moe_gather(self, x: Tensor, order: Tensor, used: int) -> Tensor:
        """h_moe_gather (hybrid.metal:2360-2370): out[p] = x[sorted[p] / used]."""
        dims, routes = x.shape(), order.numel()
        if len(dims) != 2 or used == 0 or routes != dims[0] * used:
            raise ShapeError("route gather needs [tokens, hidden] and tokens * used routes")
        out = Tensor.zeros(self, (routes, dims[1]), x.dtype)
        xv, sv, ov = x._view(), order._view(), out._view()
        _check(_lib.fh_hybrid_moe_gather(self._handle, ctypes.byref(xv), ctypes.byref(sv), dims[1], used, routes,
                                         ctypes.byref(ov)))
        return out

    def hybrid_project_mm_id(self, weight: "QuantizedExpertMatrix", x: Tensor, offsets: Tensor,
                             out_dtype: DType | None = None) -> Tensor:
        """HybridModel::project_mm_id (src/hybrid/engine.rs:3150-3220): rows offsets[e] ..
        offsets[e + 1] of the expert-sorted x are multiplied by expert e."""
        dims = x.shape()
        if len(dims) != 2 or dims[0] == 0 or dims[1] != weight.columns() or offsets.shape() != (weight.experts() + 1,):
            raise ShapeError("expert projection geometry")
        y = Tensor.zeros(self, (dims[0], weight.rows_per_expert()), out_dtype or x.dtype)
        xv, fv, yv = x._view(), offsets._view(), y._view()
        _check(_lib.fh_hybrid_project_mm_id(self._handle, _handle_of(weight), ctypes.byref(xv), ctypes.byref(fv),
                                            dims[0], ctypes.byref(yv)))
        return y

    def hybrid_project_mm_id_with_shared(self, weight: "QuantizedExpertMatrix", shared_weight: "QuantizedMatrix",
                                         x: Tensor, offsets: Tensor, shared_x: Tensor):
        """``hybrid_project_mm_id`` and, in the same launch, the shared expert's dense projection of
        ``shared_x`` [tokens, K].  Returns (y [routes, N], shared_y [tokens, N])."""
        dims, sd = x.shape(), shared_x.shape()
        if (len(dims) != 2 or dims[0] == 0 or dims[1] != weight.columns() or offsets.shape() != (weight.experts() + 1,)
                or len(sd) != 2 or sd[0] == 0 or sd[1] != dims[1] or shared_x.dtype != x.dtype
                or shared_weight.rows() != weight.rows_per_expert() or shared_weight.columns() != weight.columns()
                or shared_weight.format().ggml_type() != weight.format().ggml_type()):
            raise ShapeError("expert projection geometry")
        y = Tensor.zeros(self, (dims[0], weight.rows_per_expert()), x.dtype)
        ys = Tensor.zeros(self, (sd[0], weight.rows_per_expert()), x.dtype)
        xv, fv, sxv, yv, ysv = x._view(), offsets._view(), shared_x._view(), y._view(), ys._view()
        _check(_lib.fh_hybrid_project_mm_id_with_shared(
            self._handle, _handle_of(weight), _handle_of(shared_weight), ctypes.byref(xv), ctypes.byref(fv), dims[0],
            sd[0], ctypes.byref(sxv), ctypes.byref(yv), ctypes.byref(ysv)))
        return y, ys

    def hybrid_moe_combine(self, down: Tensor, weights: Tensor, position: Tensor | None, shared: Tensor,
                           shared_gate: Tensor, used: int) -> Tensor:
        """h_moe_combine (hybrid.metal:2372-2388), f32: the weighted sum of each token's routed rows
        (row = position[route], or the route itself when position is None) plus gate * shared."""
        tokens, hidden = shared.shape()
        if (down.shape() != (tokens * used, hidden) or weights.numel() != tokens * used
                or shared_gate.shape() != (tokens,) or (position is not None and position.numel() != tokens * used)):
            raise ShapeError("expert combine geometry mismatch")
        out = Tensor.zeros(self, (tokens, hidden), DType.F32)
        views = [t._view() if t is not None else None for t in (down, weights, position, shared, shared_gate, out)]
        ref = lambda v: ctypes.byref(v) if v is not None else None
        _check(_lib.fh_hybrid_moe_combine(self._handle, ref(views[0]), ref(views[1]), ref(views[2]), ref(views[3]),
                                          ref(views[4]), hidden, used, tokens, ref(views[5])))
        return out

    def expert_combine_shared(self, input: Tensor, metadata: Tensor, tokens: int, hidden: int, top_k: int,
                              shared: Tensor, shared_gate: Tensor | None = None,
                              out: Tensor | None = None) -> Tensor:
        """h_moe_combine (hybrid.metal:2374-2388): the weighted sum of the routed rows plus
        shared_gate[t] * shared[t] (gate 1 when absent)."""
        if (input.shape() != (tokens * top_k, hidden) or metadata.shape() != (tokens * top_k, 3)
                or shared.shape() != (tokens, hidden) or shared.dtype != input.dtype
                or (shared_gate is not None and shared_gate.shape() != (tokens,))):
            raise ShapeError("expert combine geometry mismatch")
        if out is None:
            out = Tensor.zeros(self, (tokens, hidden), input.dtype)
        iv, mv, sv, ov = input._view(), metadata._view(), shared._view(), out._view()
        gv = shared_gate._view() if shared_gate is not None else None
        _check(_lib.fh_expert_combine_shared(self._handle, ctypes.byref(iv), ctypes.byref(mv), tokens, hidden,
                                             top_k, ctypes.byref(sv),
                                             ctypes.byref(gv) if gv is not None else None, ctypes.byref(ov)))
        return out

    def expert_assign(self, hidden: Tensor, metadata: Tensor, top_k: int,
                      out: Tensor | None = None) -> Tensor:
        x, meta = hidden.shape(), metadata.shape()
        if (len(x) != 2 or x[0] == 0 or x[1] == 0 or len(meta) != 2 or meta[1] != 3 or top_k == 0
                or x[0] * top_k != meta[0] or metadata.dtype != DType.F32):
            raise ShapeError("expert assignments require [S,H] and [S*top_k,3]")
        if out is None:
            out = Tensor.zeros(self, (meta[0], x[1]), hidden.dtype)
        hv, mv, ov = hidden._view(), metadata._view(), out._view()
        _check(_lib.fh_expert_assign(self._handle, ctypes.byref(hv), x[0], x[1], ctypes.byref(mv),
                                     top_k, ctypes.byref(ov)))
        return out

    def expert_project_quantized(self, input: Tensor, metadata: Tensor,
                                 weight: QuantizedExpertMatrix, features: int, experts: int,
                                 out_dtype: DType | None = None, out: Tensor | None = None,
                                 form: str = "rows") -> Tensor:
        """``form``: "rows" reads input [A, K]; "gather" reads input as hidden
        [tokens, K] and uses row token(a) (expert_assign folded in); "silu_mul"
        reads input [A, 2K] and applies expert_silu_mul on the way in."""
        x, meta = input.shape(), metadata.shape()
        code = {"rows": 0, "gather": 1, "silu_mul": 2}[form]
        width = features * (2 if code == 2 else 1)
        if (len(x) != 2 or x[0] == 0 or x[1] != width or len(meta) != 2 or meta[1] != 3 or meta[0] == 0
                or (code != 1 and meta[0] != x[0])
                or metadata.dtype != DType.F32 or experts == 0 or weight.experts() != experts
                or weight.columns() != features or weight.rows_per_expert() == 0
                or input.buffer.device is not self or metadata.buffer.device is not self
                or weight.device is not self):
            raise ShapeError("quantized expert projection geometry mismatch")
        dtype = input.dtype if out_dtype is None else DType(out_dtype)
        if out is None:
            out = Tensor.zeros(self, (meta[0], weight.rows_per_expert()), dtype)
        xv, mv, ov = input._view(), metadata._view(), out._view()
        if code == 0:
            _check(_lib.fh_expert_project_quantized(self._handle, weight._handle, ctypes.byref(xv), x[0],
                                                    ctypes.byref(mv), ctypes.byref(ov)))
        else:
            _check(_lib.fh_expert_project_fused(self._handle, weight._handle, ctypes.byref(xv), x[0], code,
                                                meta[0], ctypes.byref(mv), ctypes.byref(ov)))
        return out

    def expert_project_with_shared(self, input: Tensor, metadata: Tensor, weight: QuantizedExpertMatrix,
                                   shared_weight: QuantizedMatrix, tokens: int, form: str,
                                   shared_input: Tensor | None = None, out: Tensor | None = None,
                                   shared_out: Tensor | None = None):
        """The routed projection of ``expert_project_quantized(form=...)`` and, in the same
        launch, the shared expert's dense projection of every token: ``form="gather"`` reads
        both from ``input`` [tokens, K]; ``form="silu_mul"`` reads the routed rows from
        ``input`` [A, 2K] and the shared ones from ``shared_input`` [tokens, 2K].  Returns
        (routed [A, N], shared [tokens, N])."""
        code = {"gather": 1, "silu_mul": 2}[form]
        x, meta, k = input.shape(), metadata.shape(), weight.columns()
        if (len(x) != 2 or len(meta) != 2 or meta[1] != 3 or meta[0] == 0 or tokens == 0
                or metadata.dtype != DType.F32
                or x != ((tokens, k) if code == 1 else (meta[0], 2 * k))
                or (code == 2) != (shared_input is not None)
                or (shared_input is not None and (shared_input.shape() != (tokens, 2 * k)
                                                  or shared_input.dtype != input.dtype))
                or shared_weight.rows() != weight.rows_per_expert() or shared_weight.columns() != k
                or shared_weight.format().ggml_type() != weight.format().ggml_type()
                or input.buffer.device is not self or metadata.buffer.device is not self
                or weight.device is not self or shared_weight.device is not self):
            raise ShapeError("quantized expert projection geometry mismatch")
        n = weight.rows_per_expert()
        if out is None:
            out = Tensor.zeros(self, (meta[0], n), input.dtype)
        if shared_out is None:
            shared_out = Tensor.zeros(self, (tokens, n), input.dtype)
        xv, mv, ov, sov = input._view(), metadata._view(), out._view(), shared_out._view()
        sxv = shared_input._view() if shared_input is not None else None
        _check(_lib.fh_expert_project_with_shared(
            self._handle, weight._handle, _handle_of(shared_weight), ctypes.byref(xv), tokens, code, meta[0],
            ctypes.byref(mv), ctypes.byref(sxv) if sxv is not None else None, ctypes.byref(ov),
            ctypes.byref(sov)))
        return out, shared_out

    def expert_silu_mul(self, input: Tensor, intermediate: int, out: Tensor | None = None) -> Tensor:
        x = input.shape()
        if len(x) != 2 or intermediate == 0 or intermediate * 2 != x[1]:
            raise ShapeError("packed expert activation geometry mismatch")
        if out is None:
            out = Tensor.zeros(self, (x[0], intermediate), input.dtype)
        iv, ov = input._view(), out._view()
        _check(_lib.fh_expert_silu_mul(self._handle, ctypes.byref(iv), x[0], intermediate,
                                       ctypes.byref(ov)))
        return out

    def expert_combine(self, input: Tensor, metadata: Tensor, tokens: int, hidden: int,
                       top_k: int, out: Tensor | None = None) -> Tensor:
        x = input.shape()
        if (top_k == 0 or hidden == 0 or x != (tokens * top_k, hidden)
                or metadata.shape() != (x[0], 3) or metadata.dtype != DType.F32):
            raise ShapeError("expert combine geometry mismatch")
        if out is None:
            out = Tensor.zeros(self, (tokens, hidden), input.dtype)
        iv, mv, ov = input._view(), metadata._view(), out._view()
        _check(_lib.fh_expert_combine(self._handle, ctypes.byref(iv), ctypes.byref(mv), tokens,
                                      hidden, top_k, ctypes.byref(ov)))
        return out

    def __del__(self):
        if sys.is_finalizing():   # the HIP runtime may already be gone at interpreter exit
            return
        h, self._handle = getattr(self, "_handle", None), None
        if h:
            _lib.fh_device_destroy(h)


class SparseMoe:
    """Routed expert FFN, the orchestration of SparseMoe::forward
    (src/nn/moe.rs:222-390): route -> assign -> gate|up projection -> SiLU*up ->
    down projection -> weighted combine.  The reference computes the router
    logits with a dense linear layer of its own; that layer is not part of the
    quantized path, so `forward` takes the logits.  With `workspace(tokens)`
    every intermediate is allocated ahead, which lets a forward pass be
    recorded into an execution."""

    def __init__(self, device: "Device", input_experts: QuantizedExpertMatrix,
                 output_experts: QuantizedExpertMatrix, routing: MoeRoutingPolicy,
                 selection_bias: Tensor | None = None, shared_input: QuantizedMatrix | None = None,
                 shared_output: QuantizedMatrix | None = None):
        """``shared_input`` [2*I_s, H] (gate rows first) and ``shared_output`` [H, I_s]: a
        shared expert that every token runs next to its routed ones, as the hybrid engine's
        moe_ffn does (src/hybrid/engine.rs:2925); its output is added in the combine,
        scaled by ``forward``'s ``shared_gate`` when given."""
        e, two_i, h = input_experts.experts(), input_experts.rows_per_expert(), input_experts.columns()
        if (two_i == 0 or two_i % 2 or output_experts.experts() != e
                or output_experts.rows_per_expert() != h or output_experts.columns() * 2 != two_i
                or routing.experts != e or routing.top_k == 0 or routing.top_k > e
                or routing.use_expert_bias != (selection_bias is not None)
                or input_experts.device is not device or output_experts.device is not device):
            raise ConfigError("invalid sparse expert weight geometry")
        if (shared_input is None) != (shared_output is None) or (shared_input is not None and (
                shared_input.columns() != h or shared_output.rows() != h or shared_input.rows() == 0
                or shared_input.rows() != 2 * shared_output.columns()
                or shared_input.device is not device or shared_output.device is not device)):
            raise ConfigError("invalid shared expert weight geometry")
        self.device, self.routing, self.selection_bias = device, routing, selection_bias
        self.input_experts, self.output_experts = input_experts, output_experts
        self.shared_input, self.shared_output = shared_input, shared_output
        self.expert_count, self.hidden_size, self.intermediate_size = e, h, two_i // 2
        # the shared expert can ride in the routed launches when it has an expert's shape and format
        self._shared_rides = (shared_input is not None and shared_input.rows() == two_i
                              and shared_input.format().ggml_type() == input_experts.format().ggml_type()
                              and shared_output.format().ggml_type() == output_experts.format().ggml_type())
        self._ws = None
        self._stats = MoeStats()
        # most f32 assignments that take the fused per-assignment kernels (f32 rows have no
        # grouped form by default, and the per-assignment SiLU is recomputed by every workgroup);
        # also the most assignments whose shared expert rides in the routed launches
        self.fused_max_assignments = 31
        # False: expert_assign and expert_silu_mul always run as launches of their own
        self.fuse_inputs = True

    def workspace(self, tokens: int, dtype: DType):
        a, h, i = tokens * self.routing.top_k, self.hidden_size, self.intermediate_size
        d = self.device
        self._ws = {"tokens": tokens, "dtype": dtype,
                    "metadata": Tensor.zeros(d, (a, 3), DType.F32),
                    "assigned": Tensor.zeros(d, (a, h), dtype),
                    "projected": Tensor.zeros(d, (a, 2 * i), dtype),
                    "activated": Tensor.zeros(d, (a, i), dtype),
                    "expert_output": Tensor.zeros(d, (a, h), dtype),
                    "combined": Tensor.zeros(d, (tokens, h), dtype)}
        if self.shared_input is not None:
            si = self.shared_output.columns()
            self._ws.update({"shared_projected": Tensor.zeros(d, (tokens, 2 * si), dtype),
                             "shared_activated": Tensor.zeros(d, (tokens, si), dtype),
                             "shared_output": Tensor.zeros(d, (tokens, h), dtype)})
        return self._ws

    def forward_in_one_call(self, hidden: Tensor, router_logits: Tensor, shared_gate: Tensor | None = None,
                            out: Tensor | None = None) -> Tensor:
        """fh_moe_ffn: the steps of ``forward`` (inputs folded into the projections) enqueued by
        one library call, temporaries in the library's workspace; the same bits."""
        dims = hidden.shape()
        if len(dims) != 2 or dims[1] != self.hidden_size or dims[0] == 0:
            raise ShapeError("sparse expert input requires [tokens,hidden]")
        if router_logits.shape() != (dims[0], self.expert_count):
            raise ShapeError("router logits require [tokens,experts]")
        if shared_gate is not None and shared_gate.numel() != dims[0]:
            raise ShapeError("shared gate requires one value per token")
        if out is None:
            out = Tensor.zeros(self.device, dims, hidden.dtype)
        hv, lv, ov, pc = hidden._view(), router_logits._view(), out._view(), self.routing._c()
        bv = self.selection_bias._view() if self.selection_bias is not None else None
        gv = shared_gate._view() if shared_gate is not None else None
        ref = lambda v: ctypes.byref(v) if v is not None else None
        _check(_lib.fh_moe_ffn(self.device._handle, ctypes.byref(hv), ctypes.byref(lv), dims[0], ref(bv), ctypes.byref(pc),
                               self.input_experts._handle, self.output_experts._handle,
                               _handle_of(self.shared_input) if self.shared_input is not None else None,
                               _handle_of(self.shared_output) if self.shared_output is not None else None,
                               ref(gv), ctypes.byref(ov)))
        return out

    def take_stats(self) -> MoeStats:
        """The statistics gathered since the last call, which start afresh (take_stats,
        src/nn/moe.rs:218-220)."""
        taken, self._stats = self._stats, MoeStats()
        return taken

    def temporary_bytes(self, tokens: int, dtype: DType) -> int:
        """Routing temporaries of `tokens` tokens as the reference counts them
        (src/nn/moe.rs:232-249, :306-316): per assignment the assigned row, the gate|up
        row, the activated row and the projected output row plus one routing record; per
        token its logits and its combined row."""
        per_assignment = (2 * self.hidden_size + 3 * self.intermediate_size) * dtype.size_bytes() + 12
        per_token = per_assignment * self.routing.top_k + (self.expert_count + self.hidden_size) * dtype.size_bytes()
        return tokens * per_token

    def forward(self, hidden: Tensor, router_logits: Tensor, shared_gate: Tensor | None = None) -> Tensor:
        """Tokens are taken in chunks whose routing temporaries stay under the device's
        moe_routing_temporary_limit (src/nn/moe.rs:250-256); every chunk's combine writes its
        rows of one output tensor, so nothing is read back between chunks."""
        dims = hidden.shape()
        if len(dims) != 2 or dims[1] != self.hidden_size or dims[0] == 0:
            raise ShapeError("sparse expert input requires [tokens,hidden]")
        if hidden.buffer.device is not self.device:
            raise DeviceMismatch("tensor belongs to another device")
        if router_logits.shape() != (dims[0], self.expert_count):
            raise ShapeError("router logits require [tokens,experts]")
        if shared_gate is not None and shared_gate.numel() != dims[0]:
            raise ShapeError("shared gate requires one value per token")
        tokens = dims[0]
        per_token = self.temporary_bytes(1, hidden.dtype)
        chunk_tokens = min(tokens, max(1, self.device.moe_routing_temporary_limit() // per_token))
        stats = MoeStats(active_experts_known=False)
        if chunk_tokens == tokens:
            ws = self._ws if self._ws and self._ws["tokens"] == tokens and self._ws["dtype"] == hidden.dtype else {}
            out = self._forward_chunk(hidden, router_logits, shared_gate, ws, None, stats)
        else:
            out = Tensor.zeros(self.device, (tokens, self.hidden_size), hidden.dtype)
            for start in range(0, tokens, chunk_tokens):
                count = min(chunk_tokens, tokens - start)
                gate = None if shared_gate is None else shared_gate.view(start, (count,))
                self._forward_chunk(hidden.view(start * self.hidden_size, (count, self.hidden_size)),
                                    router_logits.view(start * self.expert_count, (count, self.expert_count)),
                                    gate, {}, out.view(start * self.hidden_size, (count, self.hidden_size)), stats)
        self._stats.merge(stats)
        return out

    def _forward_chunk(self, hidden, router_logits, shared_gate, ws, out, stats):
        dims = hidden.shape()
        d, k = self.device, self.routing.top_k
        stats.assignments += dims[0] * k
        stats.peak_temporary_bytes = max(stats.peak_temporary_bytes, self.temporary_bytes(dims[0], hidden.dtype))
        combined = out if out is not None else ws.get("combined")
        t0 = time.perf_counter()
        metadata = d.moe_route(router_logits, self.selection_bias, self.routing, out=ws.get("metadata"))
        t1 = time.perf_counter()
        stats.routing += t1 - t0
        if self.shared_input is not None:
            return self._forward_with_shared(hidden, metadata, shared_gate, ws, combined, stats, t1)
        if self.fuse_inputs and (dims[0] * k <= self.fused_max_assignments or hidden.dtype != DType.F32):
            # the copy and the activation ride inside the projections: per assignment in
            # decode, and in the grouped kernel's gather of an expert's rows beyond it
            projected = d.expert_project_quantized(hidden, metadata, self.input_experts, self.hidden_size,
                                                   self.expert_count, out=ws.get("projected"), form="gather")
            expert_output = d.expert_project_quantized(projected, metadata, self.output_experts,
                                                       self.intermediate_size, self.expert_count,
                                                       out=ws.get("expert_output"), form="silu_mul")
        else:
            assigned = d.expert_assign(hidden, metadata, k, out=ws.get("assigned"))
            projected = d.expert_project_quantized(assigned, metadata, self.input_experts, self.hidden_size,
                                                   self.expert_count, out=ws.get("projected"))
            activated = d.expert_silu_mul(projected, self.intermediate_size, out=ws.get("activated"))
            expert_output = d.expert_project_quantized(activated, metadata, self.output_experts,
                                                       self.intermediate_size, self.expert_count,
                                                       out=ws.get("expert_output"))
        t2 = time.perf_counter()
        stats.expert_dispatch += t2 - t1
        result = d.expert_combine(expert_output, metadata, dims[0], self.hidden_size, k, out=combined)
        stats.combine_dispatch += time.perf_counter() - t2
        return result

    def _forward_with_shared(self, hidden, metadata, shared_gate, ws, combined, stats, t1):
        d, k, tokens = self.device, self.routing.top_k, hidden.shape()[0]
        a = tokens * k
        if self.fuse_inputs and self._shared_rides and (a <= self.fused_max_assignments or hidden.dtype != DType.F32):
            # four launches: the shared expert's rows are batch entries of the routed ones in
            # decode and further token groups of the grouped kernel beyond it
            projected, shared_projected = d.expert_project_with_shared(
                hidden, metadata, self.input_experts, self.shared_input, tokens, "gather",
                out=ws.get("projected"), shared_out=ws.get("shared_projected"))
            expert_output, shared_output = d.expert_project_with_shared(
                projected, metadata, self.output_experts, self.shared_output, tokens, "silu_mul",
                shared_input=shared_projected, out=ws.get("expert_output"), shared_out=ws.get("shared_output"))
        else:
            fused = self.fuse_inputs and (a <= self.fused_max_assignments or hidden.dtype != DType.F32)
            if fused:
                projected = d.expert_project_quantized(hidden, metadata, self.input_experts, self.hidden_size,
                                                       self.expert_count, out=ws.get("projected"), form="gather")
                expert_output = d.expert_project_quantized(projected, metadata, self.output_experts,
                                                           self.intermediate_size, self.expert_count,
                                                           out=ws.get("expert_output"), form="silu_mul")
            else:
                assigned = d.expert_assign(hidden, metadata, k, out=ws.get("assigned"))
                projected = d.expert_project_quantized(assigned, metadata, self.input_experts, self.hidden_size,
                                                       self.expert_count, out=ws.get("projected"))
                activated = d.expert_silu_mul(projected, self.intermediate_size, out=ws.get("activated"))
                expert_output = d.expert_project_quantized(activated, metadata, self.output_experts,
                                                           self.intermediate_size, self.expert_count,
                                                           out=ws.get("expert_output"))
            shared_projected = d.project_quantized(hidden, self.shared_input, out=ws.get("shared_projected")).tensor
            if self.fuse_inputs and tokens <= self.fused_max_assignments:
                shared_output = d.project_quantized(shared_projected, self.shared_output, out=ws.get("shared_output"),
                                                    silu_mul=True).tensor
            else:
                shared_activated = d.expert_silu_mul(shared_projected, self.shared_output.columns(),
                                                     out=ws.get("shared_activated"))
                shared_output = d.project_quantized(shared_activated, self.shared_output,
                                                    out=ws.get("shared_output")).tensor
        t2 = time.perf_counter()
        stats.expert_dispatch += t2 - t1
        result = d.expert_combine_shared(expert_output, metadata, tokens, self.hidden_size, k, shared_output,
                                         shared_gate, out=combined)
        stats.combine_dispatch += time.perf_counter() - t2
        return result


def _handle_of(weight):
    h = getattr(weight, "_handle", None)
    return h if h else getattr(weight, "_borrowed", None)
