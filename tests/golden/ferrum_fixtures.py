"""Closed-form test data of Ferrum's own quantized-matmul tests, rebuilt in numpy.

The reference stores no binary vectors for this path: every Q4_K / Q6_K test
builds its packed bytes, activations and expected values from integer
formulas.  Those formulas are restated here so the same bytes and the same
per-element expectations exist without running the reference:

* ``q4k_packed`` / ``q4k_value``   src/ops/transformer.rs:2833-2956 (qk_tests)
* ``q5k_packed`` / ``q5k_value``   the Q5_K branch of the same tests (:2843-2847, 2887-2892, 2946-2952)
* ``q6k_packed`` / ``q6k_value``   src/ops/transformer.rs:4102-4169 (q6_k_tests)
* ``qk_q6_packed`` / ``qk_q6_value``  the Q6_K branch inside qk_tests
                                   (src/ops/transformer.rs:2863-2878, 2924-2936)
* ``q4k_input`` / ``q6k_input``    :2958-2962 and :4171-4175
* ``xorshift_blocks`` / ``xorshift_uniform``  src/diffusion/tests.rs:9-19, 769-795
* ``iq_random_blocks`` / ``iq_random``        src/hybrid/iq_tests.rs:1233-1262

The per-element ``*_value`` functions are evaluated in float32 numpy with one
rounding per operation, in the reference's order, and are independent of the
C oracle: tests compare the two bitwise.
"""
from __future__ import annotations

import numpy as np

Q4_K, Q5_K, Q6_K = 12, 13, 14
F = np.float32


def _f16_bytes(value: float) -> bytes:
    return np.array([value], dtype=np.float32).astype(np.float16).tobytes()


# --------------------------------------------------------------- qk_tests

def _qk_scales(row: int, block: int) -> np.ndarray:
    i = np.arange(12)
    return ((row * 47 + block * 31 + i * 53 + 0x9D) & 255).astype(np.uint8)


def _qk_qbyte(row, block, index):
    return (row * 17 + block * 43 + index * 29 + 0x6B) & 255


def _qk_q4_parameters(row: int):
    return F(0.00390625) + F(row) * F(0.00048828125), F(0.015625)


def q4k_packed(rows: int, columns: int) -> np.ndarray:
    out = bytearray()
    idx = np.arange(128)
    for row in range(rows):
        for block in range(columns // 256):
            d, dmin = _qk_q4_parameters(row)
            out += _f16_bytes(d) + _f16_bytes(dmin)
            out += _qk_scales(row, block).tobytes()
            out += _qk_qbyte(row, block, idx).astype(np.uint8).tobytes()
    return np.frombuffer(bytes(out), dtype=np.uint8).copy()


def _unpack_scale_min(scales: np.ndarray, group: int):
    if group < 4:
        return int(scales[group] & 63), int(scales[group + 4] & 63)
    return (int(scales[group + 4] & 15) | (int(scales[group - 4] >> 6) << 4),
            int(scales[group + 4] >> 4) | (int(scales[group] >> 6) << 4))


def q4k_value(row: int, column: int) -> np.float32:
    block, within = divmod(column, 256)
    group, lane, chunk = within // 32, within % 32, within // 64
    byte = _qk_qbyte(row, block, chunk * 32 + lane)
    nibble = byte & 15 if group % 2 == 0 else byte >> 4
    d, dmin = _qk_q4_parameters(row)
    scale, minimum = _unpack_scale_min(_qk_scales(row, block), group)
    return F(F(F(d * F(scale)) * F(nibble)) - F(dmin * F(minimum)))


def _qk_q5_parameters(block: int):
    return F(0.001953125) + F(block) / F(4096.0), F(0.0078125)


def q5k_packed(rows: int, columns: int) -> np.ndarray:
    out = bytearray()
    for row in range(rows):
        for block in range(columns // 256):
            d, dmin = _qk_q5_parameters(block)
            out += _f16_bytes(d) + _f16_bytes(dmin)
            out += _qk_scales(row, block).tobytes()
            out += _qk_qbyte(row + 7, block, np.arange(32)).astype(np.uint8).tobytes()
            out += _qk_qbyte(row, block, np.arange(128)).astype(np.uint8).tobytes()
    return np.frombuffer(bytes(out), dtype=np.uint8).copy()


def q5k_value(row: int, column: int) -> np.float32:
    block, within = divmod(column, 256)
    group, lane, chunk = within // 32, within % 32, within // 64
    byte = _qk_qbyte(row, block, chunk * 32 + lane)
    nibble = byte & 15 if group % 2 == 0 else byte >> 4
    high = (_qk_qbyte(row + 7, block, lane) >> group) & 1
    d, dmin = _qk_q5_parameters(block)
    scale, minimum = _unpack_scale_min(_qk_scales(row, block), group)
    return F(F(F(d * F(scale)) * F(nibble | (high << 4))) - F(dmin * F(minimum)))


def q5k_dense(rows: int, columns: int) -> np.ndarray:
    return np.array([[q5k_value(r, c) for c in range(columns)] for r in range(rows)], dtype=F)


def q4k_dense(rows: int, columns: int) -> np.ndarray:
    return np.array([[q4k_value(r, c) for c in range(columns)] for r in range(rows)], dtype=F)


def q4k_input(rows: int, columns: int) -> np.ndarray:
    i = np.arange(rows * columns, dtype=np.int64)
    return (((i * 41 + 11) % 127).astype(F) / F(113.0) - F(0.55)).astype(F).reshape(rows, columns)


def qk_q6_packed(rows: int, columns: int) -> np.ndarray:
    out = bytearray()
    for row in range(rows):
        for block in range(columns // 256):
            out += _qk_qbyte(row, block, np.arange(128)).astype(np.uint8).tobytes()
            out += _qk_qbyte(row + 5, block, np.arange(64)).astype(np.uint8).tobytes()
            s = ((row * 7 + block * 3 + np.arange(16) * 5) % 15 - 7).astype(np.int8)
            out += s.tobytes()
            out += _f16_bytes(F(0.015625) + F(row) / F(4096.0))
    return np.frombuffer(bytes(out), dtype=np.uint8).copy()


def qk_q6_value(row: int, column: int) -> np.float32:
    block, within = divmod(column, 256)
    group, lane = within // 32, within % 32
    half_block, slice_ = group // 4, group % 4
    byte = _qk_qbyte(row, block, half_block * 64 + (slice_ & 1) * 32 + lane)
    low = byte & 15 if slice_ < 2 else byte >> 4
    high = (_qk_qbyte(row + 5, block, half_block * 32 + lane) >> (slice_ * 2)) & 3
    q = (low | (high << 4)) - 32
    scale_index = half_block * 8 + slice_ * 2 + lane // 16
    scale = (row * 7 + block * 3 + scale_index * 5) % 15 - 7
    d = F(0.015625) + F(row) / F(4096.0)
    return F(F(d * F(scale)) * F(q))


# -------------------------------------------------------------- q6_k_tests

def _q6_byte(row, block, index):
    return (row * 13 + block * 7 + index * 17 + 3) & 255


def _q6_scale(row, block, index):
    return (row * 3 + block * 5 + index * 7) % 9 - 4


def _q6_block_scale(row: int, block: int) -> np.float32:
    return F(0.125) if (row + block) % 2 == 0 else F(-0.0625)


def q6k_packed(rows: int, columns: int) -> np.ndarray:
    out = bytearray()
    for row in range(rows):
        for block in range(columns // 256):
            out += _q6_byte(row, block, np.arange(128)).astype(np.uint8).tobytes()
            out += _q6_byte(row + 11, block, np.arange(64)).astype(np.uint8).tobytes()
            out += _q6_scale(row, block, np.arange(16)).astype(np.int8).tobytes()
            out += _f16_bytes(_q6_block_scale(row, block))
    return np.frombuffer(bytes(out), dtype=np.uint8).copy()


def q6k_value(row: int, column: int) -> np.float32:
    block, within = divmod(column, 256)
    group, lane = within // 32, within % 32
    half_block, slice_ = group // 4, group % 4
    ql = _q6_byte(row, block, half_block * 64 + (slice_ % 2) * 32 + lane)
    ql_bits = ql & 15 if slice_ < 2 else ql >> 4
    qh = _q6_byte(row + 11, block, half_block * 32 + lane)
    high = (qh >> (slice_ * 2)) & 3
    quant = (ql_bits | (high << 4)) - 32
    scale = _q6_scale(row, block, half_block * 8 + slice_ * 2 + lane // 16)
    return F(F(_q6_block_scale(row, block) * F(scale)) * F(quant))


def q6k_dense(rows: int, columns: int) -> np.ndarray:
    return np.array([[q6k_value(r, c) for c in range(columns)] for r in range(rows)], dtype=F)


def q6k_input(rows: int, columns: int) -> np.ndarray:
    i = np.arange(rows * columns, dtype=np.int64)
    return (((i * 19 + 7) % 127).astype(F) / F(113.0) - F(0.56)).astype(F).reshape(rows, columns)


def expected_f32seq(x: np.ndarray, dense: np.ndarray) -> np.ndarray:
    """`.sum::<f32>()` of x*w over K ascending, per (m, n)."""
    m, k = x.shape
    n = dense.shape[0]
    out = np.zeros((m, n), dtype=F)
    for c in range(k):
        out = (out + (x[:, c:c + 1] * dense[:, c][None, :]).astype(F)).astype(F)
    return out


# ------------------------------------------------- xorshift block generators

_M64 = (1 << 64) - 1


def _xorshift_bytes(state: int, count: int) -> np.ndarray:
    out = np.empty(count, dtype=np.uint8)
    x = state
    for i in range(count):
        x ^= (x << 13) & _M64
        x ^= x >> 7
        x ^= (x << 17) & _M64
        out[i] = (x >> 32) & 255
    return out


def xorshift_blocks(ggml_type: int, count: int) -> np.ndarray:
    """kquant::blocks (src/diffusion/tests.rs:769-795): random bytes whose f16
    scales are overwritten with small finite values."""
    block = 144 if ggml_type == Q4_K else 210
    data = _xorshift_bytes(((block * 0x9E3779B97F4A7C15) & _M64) | 1, count * block)
    data = data.reshape(count, block)
    for b in data:
        s0 = np.frombuffer(_f16_bytes(F(0.002) + F(0.002) * F(b[4]) / F(255.0)), dtype=np.uint8)
        s1 = np.frombuffer(_f16_bytes(F(0.002) + F(0.002) * F(b[5]) / F(255.0)), dtype=np.uint8)
        if ggml_type == Q6_K:
            b[208:210] = s0
        else:
            b[0:2] = s0
            b[2:4] = s1
    return data.reshape(-1).copy()


def hybrid_random_blocks(blocks: int, block: int, seed: int) -> np.ndarray:
    """`random_blocks(blocks, block, seed)` of the hybrid engine's format tests
    (src/hybrid/iq_tests.rs:1231-1249): xorshift bytes, with the f16 at the start of
    every block forced to 0.02 + 0.01 * byte0 / 255."""
    data = _xorshift_bytes(((seed * 0x9E3779B97F4A7C15) & _M64) | 1, blocks * block).reshape(blocks, block)
    for b in data:
        scale = F(0.02) + F(0.01) * F(b[0]) / F(255.0)
        b[0:2] = np.frombuffer(_f16_bytes(scale), dtype=np.uint8)
    return data.reshape(-1).copy()


IQ4_VALUES = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=F)


def iq4_nl_dense(blocks: np.ndarray) -> np.ndarray:
    """`dequant_iq4_nl` (src/hybrid/iq_tests.rs:1606-1620; the same walk at
    src/hybrid/ple.rs:150-158): 18-byte blocks of 32 values, byte j holds values j (low
    nibble) and j + 16 (high), each d * VALUES[nibble]."""
    b = np.asarray(blocks, dtype=np.uint8).reshape(-1, 18)
    d = b[:, 0:2].copy().view(np.float16).astype(F)            # [blocks, 1]
    out = np.empty((b.shape[0], 32), dtype=F)
    out[:, :16] = d * IQ4_VALUES[b[:, 2:] & 15]
    out[:, 16:] = d * IQ4_VALUES[b[:, 2:] >> 4]
    return out


def iq4_xs_pack(d, ls, index) -> np.ndarray:
    """IQ4_XS blocks (block_iq4_xs, src/metal/shaders/hybrid.metal:27) from their fields:
    `d` [blocks] f16-representable, `ls` [blocks, 8] in 0..63, `index` [blocks, 256] in 0..15."""
    d = np.asarray(d, dtype=np.float16).reshape(-1)
    ls = np.asarray(ls, dtype=np.uint32).reshape(d.size, 8)
    index = np.asarray(index, dtype=np.uint8).reshape(d.size, 8, 32)
    out = np.zeros((d.size, 136), dtype=np.uint8)
    out[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    high = sum(((ls[:, i] >> 4) & 3) << (2 * i) for i in range(8)).astype(np.uint16)
    out[:, 2:4] = high.view(np.uint8).reshape(-1, 2)
    for pair in range(4):
        out[:, 4 + pair] = (ls[:, 2 * pair] & 15) | ((ls[:, 2 * pair + 1] & 15) << 4)
    out[:, 8:] = (index[:, :, :16] | (index[:, :, 16:] << 4)).reshape(d.size, 128)
    return out


def deterministic(n: int) -> np.ndarray:
    """`reference::deterministic(n)`: ((73 i + 19) mod 257 - 128) / 73 in f32
    (src/reference.rs:67-71), the input of the reference's elementwise and norm tests."""
    i = np.arange(n, dtype=np.int64)
    return ((i * 73 + 19) % 257 - 128).astype(F) / F(73.0)


def xorshift_uniform(n: int, seed: int, multiplier: int = 0x9E3779B97F4A7C15) -> np.ndarray:
    """`random(n, seed)`: uniform in [-1, 1) (src/diffusion/tests.rs:9-19; the
    hybrid twin at src/hybrid/iq_tests.rs:1251-1262 uses 0x2545F4914F6CDD1D)."""
    x = ((seed * multiplier) & _M64) | 1
    out = np.empty(n, dtype=F)
    for i in range(n):
        x ^= (x << 13) & _M64
        x ^= x >> 7
        x ^= (x << 17) & _M64
        out[i] = F(F(x >> 40) / F(1 << 24)) * F(2.0) - F(1.0)
    return out


def iq_random_blocks(blocks: int, block: int, seed: int) -> np.ndarray:
    """random_blocks (src/hybrid/iq_tests.rs:1233-1249): bytes 0..2 hold an f16
    scale in 0.02..0.03."""
    data = _xorshift_bytes(((seed * 0x9E3779B97F4A7C15) & _M64) | 1, blocks * block)
    data = data.reshape(blocks, block)
    for b in data:
        b[0:2] = np.frombuffer(_f16_bytes(F(0.02) + F(0.01) * F(b[0]) / F(255.0)), dtype=np.uint8)
    return data.reshape(-1).copy()
