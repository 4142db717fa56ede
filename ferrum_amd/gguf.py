"""Bounds-checked GGUF v2/v3 index and tensor reads: the host-side reader that
feeds packed K-quant tensors to the device verbatim.

It mirrors ``GgufReader`` of the reference (src/loader/gguf.rs:162-530): the
same block-size table (``block_layout``, :91-121), limits, alignment rule
(``general.alignment``, default 32), descriptor validation, overlap check and
error texts' meaning; ``TensorInfo.logical_matrix_shape`` /
``logical_expert_shape`` (:133-157) turn GGUF's fastest-first dimensions into
``[rows, columns]`` / ``[experts, rows, columns]``.  Tensor payloads are read
on demand.  Every failure is ``api.GgufError``.
"""
from __future__ import annotations

import io
import os
import struct
from dataclasses import dataclass

MAGIC = b"GGUF"
MAX_TENSORS = 1_000_000
MAX_METADATA = 1_000_000
MAX_ARRAY_ITEMS = 4_000_000
MAX_STRING_BYTES = 16 * 1024 * 1024
MAX_TENSOR_NAME_BYTES = 64
MAX_UNTAGGED_TENSOR_NAME_BYTES = 256

# type id -> (elements per block, bytes per block)
_BLOCKS = {
    0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 36),
    10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292),
    18: (256, 98), 20: (32, 18), 21: (256, 110), 22: (256, 82), 23: (256, 136), 30: (1, 2), 42: (64, 18),
}

_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<B", 10: "<Q", 11: "<q", 12: "<d"}
STRING, ARRAY, BOOL = 8, 9, 7


def _error(message: str):
    from . import api
    return api.GgufError(message)


def block_layout(type_id: int) -> tuple[int, int]:
    """(elements, bytes) of one block of a GGML tensor type."""
    try:
        return _BLOCKS[type_id]
    except KeyError:
        raise _error(f"unsupported GGML tensor type {type_id}") from None


@dataclass
class MetadataValue:
    type_id: int          # MetadataType
    value: object         # python scalar, str, or list for arrays
    element_type: int | None = None


@dataclass
class TensorInfo:
    name: str
    dimensions: list      # GGUF order: dimension zero is the contiguous one
    type_id: int
    offset: int           # relative to the aligned start of the tensor-data section
    byte_len: int

    def logical_matrix_shape(self):
        if len(self.dimensions) != 2:
            raise _error(f"tensor {self.name} is rank {len(self.dimensions)}, expected a matrix")
        return [self.dimensions[1], self.dimensions[0]]

    def logical_expert_shape(self):
        if len(self.dimensions) != 3:
            raise _error(f"tensor {self.name} is rank {len(self.dimensions)}, expected an expert matrix")
        return [self.dimensions[2], self.dimensions[1], self.dimensions[0]]


class GgufReader:
    def __init__(self, stream, max_array_items: int | None = None, require_architecture: bool = True):
        self._f = stream
        self._f.seek(0, os.SEEK_END)
        self.file_len = self._f.tell()
        self._f.seek(0)
        self._parse(MAX_ARRAY_ITEMS if max_array_items is None else max_array_items, require_architecture,
                    skipping=max_array_items is not None)

    @staticmethod
    def open(path: str) -> "GgufReader":
        try:
            return GgufReader(builtins_open(path))
        except OSError as e:
            raise _error(f"{path}: {e}") from None

    @staticmethod
    def open_untagged(path: str) -> "GgufReader":
        try:
            return GgufReader(builtins_open(path), require_architecture=False)
        except OSError as e:
            raise _error(f"{path}: {e}") from None

    @staticmethod
    def from_bytes(data: bytes, **kw) -> "GgufReader":
        return GgufReader(io.BytesIO(data), **kw)

    # ---- primitives -------------------------------------------------------
    def _take(self, n: int, what: str) -> bytes:
        data = self._f.read(n)
        if len(data) != n:
            raise _error(f"unexpected end of file while reading {what}")
        return data

    def _scalar(self, fmt: str, what: str):
        return struct.unpack(fmt, self._take(struct.calcsize(fmt), what))[0]

    def _string(self, what: str) -> str:
        n = self._scalar("<Q", what)
        if n > MAX_STRING_BYTES or n > self.file_len:
            raise _error(f"{what} length {n} is unreasonable")
        try:
            return self._take(n, what).decode("utf-8")
        except UnicodeDecodeError:
            raise _error(f"{what} is not valid UTF-8") from None

    def _value(self, type_id: int, max_items: int, skipping: bool) -> MetadataValue:
        if type_id in _SCALARS:
            v = self._scalar(_SCALARS[type_id], "metadata value")
            if type_id == BOOL:
                if v > 1:
                    raise _error(f"invalid bool value {v}")
                v = bool(v)
            return MetadataValue(type_id, v)
        if type_id == STRING:
            return MetadataValue(type_id, self._string("metadata string"))
        if type_id == ARRAY:
            element = self._scalar("<I", "array element type")
            if element == ARRAY or (element not in _SCALARS and element != STRING):
                raise _error(f"unsupported metadata type {element}")
            count = self._scalar("<Q", "array length")
            if count > MAX_ARRAY_ITEMS or count > self.file_len:
                raise _error(f"unreasonable metadata array length {count}")
            keep = not (skipping and count > max_items)
            values = []
            for _ in range(count):
                v = self._value(element, max_items, skipping).value
                if keep:
                    values.append(v)
            return MetadataValue(type_id, values, element)
        raise _error(f"unsupported metadata type {type_id}")

    # ---- header -----------------------------------------------------------
    def _parse(self, max_items: int, require_architecture: bool, skipping: bool):
        if self._take(4, "magic") != MAGIC:
            raise _error("invalid magic; expected GGUF")
        self.version = self._scalar("<I", "version")
        if self.version not in (2, 3):
            raise _error(f"unsupported version {self.version}")
        tensor_count = self._scalar("<Q", "tensor count")
        metadata_count = self._scalar("<Q", "metadata count")
        if tensor_count > MAX_TENSORS or metadata_count > MAX_METADATA:
            raise _error(f"unreasonable descriptor counts: {tensor_count} tensors, {metadata_count} metadata entries")

        self.metadata = {}
        for _ in range(metadata_count):
            key = self._string("metadata key")
            value = self._value(self._scalar("<I", "metadata value type"), max_items, skipping)
            if key in self.metadata:
                raise _error(f"duplicate metadata key {key}")
            self.metadata[key] = value

        alignment = self.metadata.get("general.alignment")
        if alignment is None:
            self.alignment = 32
        elif alignment.type_id != 4:
            raise _error("general.alignment must have uint32 type")
        else:
            self.alignment = alignment.value
        if self.alignment < 8 or self.alignment % 8:
            raise _error(f"general.alignment must be a positive multiple of 8, got {self.alignment}")
        architecture = self.metadata.get("general.architecture")
        if require_architecture and (architecture is None or architecture.type_id != STRING):
            raise _error("missing or invalid general.architecture metadata")

        self.tensors = {}
        quantized = False
        max_name = MAX_TENSOR_NAME_BYTES if require_architecture else MAX_UNTAGGED_TENSOR_NAME_BYTES
        for _ in range(tensor_count):
            name = self._string("tensor name")
            if len(name.encode("utf-8")) > max_name:
                raise _error(f"tensor name exceeds {max_name} bytes")
            rank = self._scalar("<I", "tensor rank")
            if not 1 <= rank <= 4:
                raise _error(f"tensor {name} has unsupported rank {rank}")
            dims = [self._scalar("<Q", "tensor dimension") for _ in range(rank)]
            if any(d == 0 for d in dims):
                raise _error(f"tensor {name} has an empty dimension")
            type_id = self._scalar("<I", "tensor type")
            offset = self._scalar("<Q", "tensor data offset")
            try:
                elements_per, bytes_per = block_layout(type_id)
            except Exception as e:
                raise _error(f"tensor {name}: {e.message}") from None
            elements = 1
            for d in dims:
                elements *= d
            if elements >= 1 << 63:
                raise _error(f"tensor {name} element count overflow")
            if dims[0] % elements_per:
                raise _error(f"tensor {name} fastest dimension {dims[0]} is not divisible by block size "
                             f"{elements_per} for type {type_id}")
            byte_len = elements // elements_per * bytes_per
            if offset % self.alignment:
                raise _error(f"tensor {name} offset {offset} is not aligned to {self.alignment}")
            quantized |= type_id not in (0, 1, 30)
            if name in self.tensors:
                raise _error(f"duplicate tensor name {name}")
            self.tensors[name] = TensorInfo(name, dims, type_id, offset, byte_len)

        end = self._f.tell()
        self.tensor_data_offset = -(-end // self.alignment) * self.alignment
        ranges = []
        for t in self.tensors.values():
            start = self.tensor_data_offset + t.offset
            stop = start + t.byte_len
            if stop > self.file_len:
                raise _error(f"tensor {t.name} range {start}..{stop} exceeds file length {self.file_len}")
            ranges.append((start, stop, t.name))
        ranges.sort()
        for left, right in zip(ranges, ranges[1:]):
            if left[1] > right[0]:
                raise _error(f"tensor ranges overlap: {left[2]} and {right[2]}")
        version = self.metadata.get("general.quantization_version")
        if require_architecture and quantized and (version is None or version.type_id != 4):
            raise _error("quantized tensor file is missing uint32 general.quantization_version")

    # ---- tensors ----------------------------------------------------------
    def metadata_value(self, key: str):
        return self.metadata.get(key)

    def tensor(self, name: str) -> TensorInfo:
        try:
            return self.tensors[name]
        except KeyError:
            raise _error(f"missing tensor {name}") from None

    def read_tensor_into(self, name: str, out) -> None:
        """Fills the writable buffer `out` (exactly byte_len bytes) with the tensor's payload."""
        info = self.tensor(name)
        view = memoryview(out).cast("B")
        if len(view) != info.byte_len:
            raise _error(f"tensor {name} needs {info.byte_len} bytes, the buffer holds {len(view)}")
        self._f.seek(self.tensor_data_offset + info.offset)
        if self._f.readinto(view) != info.byte_len:
            raise _error(f"short read of tensor {name}")

    def stream_tensor(self, name: str, chunk_bytes: int, consume) -> None:
        """Calls consume(offset, bytes) for successive chunks of the payload."""
        info = self.tensor(name)
        if chunk_bytes <= 0:
            raise _error("stream chunk size must be positive")
        self._f.seek(self.tensor_data_offset + info.offset)
        done = 0
        while done < info.byte_len:
            data = self._take(min(chunk_bytes, info.byte_len - done), f"tensor {name}")
            consume(done, data)
            done += len(data)

    def tensors_equal_payload(self, left: str, right: str) -> bool:
        """True when two tensors have the same dimensions, type and bytes (tied
        embeddings stored twice); compared through bounded reads."""
        a, b = self.tensor(left), self.tensor(right)
        if (a.dimensions, a.type_id, a.byte_len) != (b.dimensions, b.type_id, b.byte_len):
            return False
        step = 256 * 1024
        for offset in range(0, a.byte_len, step):
            n = min(step, a.byte_len - offset)
            self._f.seek(self.tensor_data_offset + a.offset + offset)
            x = self._take(n, f"tensor {left}")
            self._f.seek(self.tensor_data_offset + b.offset + offset)
            if x != self._take(n, f"tensor {right}"):
                return False
        return True

    def read_stacked_experts(self, gate_name: str, up_name: str):
        return _read_stacked_experts(self, gate_name, up_name)

    def quantized_input_experts(self, device, gate_name: str, up_name: str):
        """gate|up expert tensors as one api.QuantizedExpertMatrix of [experts, 2I, H]
        (load_quantized_input_experts, src/model/lfm2_moe/gguf.rs:466-534)."""
        from . import api
        payload, fmt, experts, rows_per_expert, columns = self.read_stacked_experts(gate_name, up_name)
        return api.QuantizedExpertMatrix.new(device, payload, fmt, experts, rows_per_expert, columns)

    # ---- device upload ----------------------------------------------------
    def quantized_matrix(self, device, name: str):
        """A rank-2 Q4_K / Q6_K tensor as api.QuantizedMatrix, blocks uploaded verbatim."""
        from . import api
        info = self.tensor(name)
        rows, columns = info.logical_matrix_shape()
        fmt = api.QuantizationFormat.from_ggml_type(info.type_id)
        return api.QuantizedMatrix.from_reader(device, rows, columns, fmt,
                                               lambda buffer: self.read_tensor_into(name, buffer))

    def quantized_expert_matrix(self, device, name: str):
        """A rank-3 tensor as api.QuantizedExpertMatrix ([experts, rows, columns])."""
        import numpy as np
        from . import api
        info = self.tensor(name)
        experts, rows, columns = info.logical_expert_shape()
        fmt = api.QuantizationFormat.from_ggml_type(info.type_id)
        payload = np.empty(info.byte_len, dtype=np.uint8)
        self.read_tensor_into(name, payload)
        return api.QuantizedExpertMatrix.new(device, payload, fmt, experts, rows, columns)


def _read_stacked_experts(reader: "GgufReader", gate_name: str, up_name: str):
    """Host side of load_quantized_input_experts (src/model/lfm2_moe/gguf.rs:466-534): the
    gate and up expert tensors ([experts, I, H] each) interleaved per expert into
    [experts, 2I, H] rows, gate first, streamed 64 rows at a time.  Returns
    (payload uint8 array, format, experts, rows_per_expert, columns)."""
    import numpy as np
    from . import api
    gate, up = reader.tensor(gate_name), reader.tensor(up_name)
    experts, intermediate, hidden = gate.logical_expert_shape()
    if up.logical_expert_shape() != [experts, intermediate, hidden] or up.type_id != gate.type_id:
        raise api.WeightError(f"{up_name}: gate and up expert tensors differ in shape or type")
    fmt = api.QuantizationFormat.from_ggml_type(gate.type_id)
    row_bytes = hidden // fmt.block_elements() * fmt.block_bytes()
    component_bytes = experts * intermediate * row_bytes
    rows_per_expert = 2 * intermediate
    payload = np.empty(experts * rows_per_expert * row_bytes, dtype=np.uint8)
    view = payload.reshape(experts, 2, intermediate, row_bytes)
    for component, name in enumerate((gate_name, up_name)):
        info = reader.tensor(name)
        if info.byte_len != component_bytes:
            raise api.WeightError(f"{name}: expected {component_bytes} packed expert bytes")
        written = 0

        def place(offset, chunk, component=component, name=name):
            nonlocal written
            if len(chunk) % row_bytes:
                raise _error(f"tensor {name} stream ended inside an expert row")
            rows = np.frombuffer(chunk, dtype=np.uint8).reshape(-1, row_bytes)
            first = offset // row_bytes
            for i, row in enumerate(rows):
                expert, within = divmod(first + i, intermediate)
                if expert >= experts:
                    raise _error(f"tensor {name} contains too many expert rows")
                view[expert, component, within] = row
            written += len(chunk)

        reader.stream_tensor(name, row_bytes * 64, place)
        if written != component_bytes:
            raise _error(f"tensor {name} streamed {written} bytes, expected {component_bytes}")
    return payload, fmt, experts, rows_per_expert, hidden


def builtins_open(path: str):
    return open(path, "rb")
