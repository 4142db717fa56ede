"""ctypes front end of the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this package.  The product (``ferrum_amd``) never does: it fails loudly when
its HIP library is missing instead of falling back to anything here.

Arrays are numpy; shapes follow Ferrum's conventions (packed weights are
row-major ``[rows=N, columns=K]`` super-blocks, activations ``[M, K]``).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libferrum_oracle.so")

Q4_K = 12
Q6_K = 14
F32, F16, BF16 = 0, 1, 2


def build() -> str:
    """Compile the C restatement (always recompiles)."""
    subprocess.run(["make", "-C", _HERE, "-B", "libferrum_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load() -> ctypes.CDLL:
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    c = ctypes
    u8p, f32p = c.POINTER(c.c_uint8), c.POINTER(c.c_float)
    sz, u32, i32 = c.c_size_t, c.c_uint32, c.c_int
    lib.fo_f16_to_f32.restype = c.c_float
    lib.fo_f16_to_f32.argtypes = [c.c_uint16]
    lib.fo_f32_to_f16.restype = c.c_uint16
    lib.fo_f32_to_f16.argtypes = [c.c_float]
    lib.fo_f32_to_bf16.restype = c.c_uint16
    lib.fo_f32_to_bf16.argtypes = [c.c_float]
    lib.fo_round_storage_array.restype = None
    lib.fo_round_storage_array.argtypes = [f32p, sz, u32, f32p]
    lib.fo_block_bytes.restype = sz
    lib.fo_block_bytes.argtypes = [u32]
    lib.fo_row_bytes.restype = sz
    lib.fo_row_bytes.argtypes = [u32, sz]
    lib.fo_columns_ok.restype = ctypes.c_int
    lib.fo_columns_ok.argtypes = [u32, sz]
    lib.fo_q4_k_scale_min.restype = None
    lib.fo_q4_k_scale_min.argtypes = [u8p, u32, c.POINTER(u32), c.POINTER(u32)]
    lib.fo_dequantize.restype = i32
    lib.fo_dequantize.argtypes = [u32, u8p, sz, sz, f32p]
    lib.fo_weight.restype = c.c_float
    lib.fo_weight.argtypes = [u32, u8p, sz, sz, sz]
    lib.fo_validate_payload.restype = i32
    lib.fo_validate_payload.argtypes = [u32, u8p, sz]
    lib.fo_project_f32seq.restype = i32
    lib.fo_project_f32seq.argtypes = [u32, u8p, sz, sz, f32p, sz, f32p, i32, i32, i32]
    lib.fo_project_f64.restype = i32
    lib.fo_project_f64.argtypes = [u32, u8p, sz, sz, f32p, sz, f32p, i32, i32]
    lib.fo_select_routes.restype = i32
    lib.fo_select_routes.argtypes = [f32p, sz, sz, sz, i32, i32, c.c_float, c.c_float, f32p, f32p]
    lib.fo_expert_assign.restype = None
    lib.fo_expert_assign.argtypes = [f32p, f32p, sz, sz, f32p]
    lib.fo_expert_project.restype = i32
    lib.fo_expert_project.argtypes = [u32, u8p, sz, sz, sz, f32p, f32p, sz, f32p, i32, i32, i32]
    lib.fo_expert_silu_mul.restype = None
    lib.fo_expert_silu_mul.argtypes = [f32p, sz, sz, u32, f32p]
    lib.fo_select_routes_ranked.restype = i32
    lib.fo_select_routes_ranked.argtypes = [f32p, sz, sz, sz, i32, i32, f32p]
    lib.fo_shared_gate.restype = None
    lib.fo_shared_gate.argtypes = [f32p, f32p, sz, sz, f32p]
    lib.fo_expert_combine_shared.restype = None
    lib.fo_expert_combine_shared.argtypes = [f32p, f32p, sz, sz, sz, u32, f32p, f32p, f32p]
    u32p = c.POINTER(c.c_uint32)
    lib.fo_moe_map.restype = None
    lib.fo_moe_map.argtypes = [u32p, sz, sz, u32p, u32p, u32p]
    lib.fo_hybrid_combine.restype = None
    lib.fo_hybrid_combine.argtypes = [f32p, f32p, u32p, f32p, f32p, sz, sz, sz, f32p]
    lib.fo_add_rmsnorm.restype = None
    lib.fo_add_rmsnorm.argtypes = [f32p, f32p, f32p, sz, sz, ctypes.c_float, ctypes.c_uint32, f32p, f32p]
    lib.fo_argmax_rows.restype = None
    lib.fo_argmax_rows.argtypes = [f32p, sz, sz, ctypes.POINTER(ctypes.c_uint32)]
    lib.fo_expert_combine.restype = None
    lib.fo_expert_combine.argtypes = [f32p, f32p, sz, sz, sz, u32, f32p]
    return lib


_lib = _load()


def _u8(a: np.ndarray):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8))


def _f32(a: np.ndarray):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _packed(packed) -> np.ndarray:
    return np.ascontiguousarray(np.frombuffer(packed, dtype=np.uint8)
                                if not isinstance(packed, np.ndarray) else packed, dtype=np.uint8)


def block_bytes(ggml_type: int) -> int:
    return int(_lib.fo_block_bytes(ggml_type))


def row_bytes(ggml_type: int, cols: int) -> int:
    """Bytes of one packed row: whole super-blocks, or for Q8_0 whole 34-byte blocks of 32 weights."""
    if not _lib.fo_columns_ok(ggml_type, cols):
        raise ValueError("unsupported format or a row that is not whole blocks")
    return int(_lib.fo_row_bytes(ggml_type, cols))


def f16_to_f32(bits: int) -> float:
    return float(_lib.fo_f16_to_f32(bits))


def f32_to_f16(value) -> int:
    return int(_lib.fo_f32_to_f16(ctypes.c_float(value)))


def f32_to_bf16(value) -> int:
    return int(_lib.fo_f32_to_bf16(ctypes.c_float(value)))


def round_storage(values, dtype: int) -> np.ndarray:
    a = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty_like(a)
    _lib.fo_round_storage_array(_f32(a), a.size, dtype, _f32(out))
    return out


def q4_k_scale_min(scales12, group: int):
    s = np.ascontiguousarray(scales12, dtype=np.uint8)
    assert s.size == 12
    sc, mn = ctypes.c_uint32(), ctypes.c_uint32()
    _lib.fo_q4_k_scale_min(_u8(s), group, ctypes.byref(sc), ctypes.byref(mn))
    return sc.value, mn.value


def dequantize(ggml_type: int, packed, rows: int, cols: int) -> np.ndarray:
    p = _packed(packed)
    assert p.size == rows * row_bytes(ggml_type, cols), "packed length"
    out = np.empty((rows, cols), dtype=np.float32)
    rc = _lib.fo_dequantize(ggml_type, _u8(p), rows, cols, _f32(out))
    if rc:
        raise ValueError("unsupported format or a row that is not whole blocks")
    return out


def weight(ggml_type: int, packed, row: int, column: int, cols: int) -> float:
    p = _packed(packed)
    return float(_lib.fo_weight(ggml_type, _u8(p), row, column, cols))


def validate_payload(ggml_type: int, payload) -> int:
    p = _packed(payload)
    return int(_lib.fo_validate_payload(ggml_type, _u8(p), p.size))


def project(ggml_type: int, packed, n: int, k: int, x, *, accumulate: str = "f32",
            weight_round: int = 0, out_round: int = 0, threads: int = 1) -> np.ndarray:
    """Y[M,N] = X[M,K] . W[N,K]^T.  accumulate 'f32' (sequential, K ascending)
    or 'f64'."""
    p = _packed(packed)
    xa = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    m = xa.shape[0]
    assert p.size == n * row_bytes(ggml_type, k), "packed length"
    y = np.empty((m, n), dtype=np.float32)
    if accumulate == "f32":
        rc = _lib.fo_project_f32seq(ggml_type, _u8(p), n, k, _f32(xa), m, _f32(y), weight_round,
                                    out_round, threads)
    elif accumulate == "f64":
        rc = _lib.fo_project_f64(ggml_type, _u8(p), n, k, _f32(xa), m, _f32(y), weight_round,
                                 threads)
        if out_round:
            y = round_storage(y, out_round)
    else:
        raise ValueError(accumulate)
    if rc:
        raise ValueError("unsupported format or geometry")
    return y


def select_routes(logits, experts: int, top_k: int, *, sigmoid: bool = False,
                  normalize: bool = True, eps: float = 0.0, scaling: float = 1.0,
                  bias=None) -> np.ndarray:
    lg = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1, experts)
    tokens = lg.shape[0]
    meta = np.empty((tokens * top_k, 3), dtype=np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    rc = _lib.fo_select_routes(_f32(lg), tokens, experts, top_k, int(sigmoid), int(normalize),
                               eps, scaling, None if b is None else _f32(b), _f32(meta))
    if rc:
        raise ValueError(f"select_routes failed ({rc})")
    return meta


def expert_assign(hidden, metadata) -> np.ndarray:
    h = np.ascontiguousarray(hidden, dtype=np.float32)
    meta = np.ascontiguousarray(metadata, dtype=np.float32)
    out = np.empty((meta.shape[0], h.shape[1]), dtype=np.float32)
    _lib.fo_expert_assign(_f32(h), _f32(meta), meta.shape[0], h.shape[1], _f32(out))
    return out


def expert_project(ggml_type: int, packed, experts: int, rows: int, k: int, x, metadata, *,
                   weight_round: int = 0, out_round: int = 0, accumulate: str = "f32") -> np.ndarray:
    p = _packed(packed)
    xa = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    meta = np.ascontiguousarray(metadata, dtype=np.float32)
    assert meta.shape == (xa.shape[0], 3)
    assert p.size == experts * rows * row_bytes(ggml_type, k), "packed length"
    y = np.empty((xa.shape[0], rows), dtype=np.float32)
    rc = _lib.fo_expert_project(ggml_type, _u8(p), experts, rows, k, _f32(xa), _f32(meta),
                                xa.shape[0], _f32(y), weight_round, out_round,
                                int(accumulate == "f64"))
    if rc:
        raise ValueError("unsupported format or geometry")
    return y


def expert_silu_mul(packed_rows, intermediate: int, dtype: int = F32) -> np.ndarray:
    a = np.ascontiguousarray(packed_rows, dtype=np.float32).reshape(-1, 2 * intermediate)
    out = np.empty((a.shape[0], intermediate), dtype=np.float32)
    _lib.fo_expert_silu_mul(_f32(a), a.shape[0], intermediate, dtype, _f32(out))
    return out


def select_routes_ranked(logits, experts: int, top_k: int, sigmoid: bool = False,
                         normalize: bool = True) -> np.ndarray:
    """h_moe_route (hybrid.metal:2259-2319): metadata rows in selection order."""
    a = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1, experts)
    out = np.empty((a.shape[0] * top_k, 3), dtype=np.float32)
    status = _lib.fo_select_routes_ranked(_f32(a), a.shape[0], experts, top_k, int(sigmoid), int(normalize), _f32(out))
    if status:
        raise ValueError(f"ranked routing failed with status {status}")
    return out


def shared_gate(x, w) -> np.ndarray:
    a = np.ascontiguousarray(x, dtype=np.float32)
    v = np.ascontiguousarray(w, dtype=np.float32)
    out = np.empty(a.shape[0], dtype=np.float32)
    _lib.fo_shared_gate(_f32(a), _f32(v), a.shape[0], a.shape[1], _f32(out))
    return out


def expert_combine_shared(values, metadata, tokens: int, hidden: int, top_k: int, shared, gate=None,
                          dtype: int = F32) -> np.ndarray:
    v = np.ascontiguousarray(values, dtype=np.float32).reshape(tokens * top_k, hidden)
    meta = np.ascontiguousarray(metadata, dtype=np.float32)
    sh = np.ascontiguousarray(shared, dtype=np.float32).reshape(tokens, hidden)
    g = None if gate is None else np.ascontiguousarray(gate, dtype=np.float32)
    out = np.empty((tokens, hidden), dtype=np.float32)
    _lib.fo_expert_combine_shared(_f32(v), _f32(meta), tokens, hidden, top_k, dtype, _f32(sh),
                                  _f32(g) if g is not None else None, _f32(out))
    return out


def _u32(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))


def moe_map(ids, experts: int):
    """(offsets, sorted, position) of h_moe_map (src/metal/shaders/hybrid.metal:2321-2358);
    entries of routes whose id is not an expert are 0xffffffff."""
    i = np.ascontiguousarray(ids, dtype=np.uint32).reshape(-1)
    offsets = np.zeros(experts + 1, dtype=np.uint32)
    order = np.full(i.size, 0xFFFFFFFF, dtype=np.uint32)
    position = np.full(i.size, 0xFFFFFFFF, dtype=np.uint32)
    _lib.fo_moe_map(_u32(i), experts, i.size, _u32(offsets), _u32(order), _u32(position))
    return offsets, order, position


def hybrid_combine(down, weights, position, shared, shared_gate, used: int) -> np.ndarray:
    """h_moe_combine (src/metal/shaders/hybrid.metal:2372-2388) in f32, rank order."""
    sh = np.ascontiguousarray(shared, dtype=np.float32)
    tokens, hidden = sh.shape
    d = np.ascontiguousarray(down, dtype=np.float32).reshape(tokens * used, hidden)
    w = np.ascontiguousarray(weights, dtype=np.float32).reshape(-1)
    g = np.ascontiguousarray(shared_gate, dtype=np.float32).reshape(-1)
    p = None if position is None else np.ascontiguousarray(position, dtype=np.uint32).reshape(-1)
    out = np.empty((tokens, hidden), dtype=np.float32)
    _lib.fo_hybrid_combine(_f32(d), _f32(w), _u32(p) if p is not None else None, _f32(sh), _f32(g), hidden, used,
                           tokens, _f32(out))
    return out


def add_rmsnorm(a, b, weight, eps: float, dtype: int = F32):
    """(residual, normed) of [rows, width] operands: the storage-rounded sum and the
    reference's float64 CPU rmsnorm of it (add_rmsnorm, src/metal/shaders/ops.metal:99-124;
    src/reference.rs:23-35)."""
    x = np.ascontiguousarray(a, dtype=np.float32)
    y = np.ascontiguousarray(b, dtype=np.float32)
    w = np.ascontiguousarray(weight, dtype=np.float32)
    assert x.ndim == 2 and x.shape == y.shape and w.shape == (x.shape[1],)
    residual, normed = np.empty_like(x), np.empty_like(x)
    _lib.fo_add_rmsnorm(_f32(x), _f32(y), _f32(w), x.shape[0], x.shape[1], eps, dtype, _f32(residual),
                        _f32(normed))
    return residual, normed


def argmax_rows(logits) -> np.ndarray:
    """[rows, 2] uint32: first maximal index and a non-finite flag (argmax_rows,
    src/metal/shaders/ops.metal:2438-2464)."""
    a = np.ascontiguousarray(logits, dtype=np.float32)
    out = np.empty((a.shape[0], 2), dtype=np.uint32)
    _lib.fo_argmax_rows(_f32(a), a.shape[0], a.shape[1], out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)))
    return out


def expert_combine(values, metadata, tokens: int, hidden: int, top_k: int,
                   dtype: int = F32) -> np.ndarray:
    v = np.ascontiguousarray(values, dtype=np.float32).reshape(tokens * top_k, hidden)
    meta = np.ascontiguousarray(metadata, dtype=np.float32)
    out = np.empty((tokens, hidden), dtype=np.float32)
    _lib.fo_expert_combine(_f32(v), _f32(meta), tokens, hidden, top_k, dtype, _f32(out))
    return out
