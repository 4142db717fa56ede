"""Seeded synthetic GGUF super-blocks and activations.

The distributions are the ones the benchmark configurations state:

* Q4_K block (144 B): f16 ``d = |N(0,1)|*0.01``, f16 ``dmin = |N(0,1)|*0.005``,
  eight 6-bit scales and eight 6-bit minimums uniform in 0..63 packed into 12
  bytes, 256 nibbles uniform in 0..15.
* Q6_K block (210 B): 256 six-bit values uniform in 0..63 split into the
  ``ql`` / ``qh`` planes, 16 int8 scales uniform in -64..63, f16
  ``d = |N(0,1)|*0.002``.
* activations: N(0,1), f32, optionally rounded to f16.

Everything derives from one integer seed through numpy's PCG64 stream, so
the CPU oracle and the GPU consume identical bytes.
"""
from __future__ import annotations

import numpy as np

Q8_0, Q4_K, Q5_K, Q6_K, IQ4_XS = 8, 12, 13, 14, 23
BLOCK_BYTES = {Q8_0: 272, Q4_K: 144, Q5_K: 176, Q6_K: 210, IQ4_XS: 136}    # per 256 weights


def rng(seed: int, stream: int = 0) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(np.random.SeedSequence([seed, stream])))


def pack_q4_k_scales(sc: np.ndarray, mn: np.ndarray) -> np.ndarray:
    """Inverse of the 6-bit unpack: ``sc``/``mn`` are ``[blocks, 8]`` in 0..63,
    the result ``[blocks, 12]`` bytes.  Groups 0..3 sit in the low six bits of
    bytes 0..3 (scales) and 4..7 (minimums); groups 4..7 put their low nibbles
    in bytes 8..11 and their top two bits in bits 6..7 of bytes 0..7."""
    sc = np.asarray(sc, dtype=np.uint8)
    mn = np.asarray(mn, dtype=np.uint8)
    out = np.zeros(sc.shape[:-1] + (12,), dtype=np.uint8)
    out[..., 0:4] = sc[..., 0:4] | ((sc[..., 4:8] >> 4) << 6)
    out[..., 4:8] = mn[..., 0:4] | ((mn[..., 4:8] >> 4) << 6)
    out[..., 8:12] = (sc[..., 4:8] & 15) | ((mn[..., 4:8] & 15) << 4)
    return out


def q4_k_blocks(count: int, g: np.random.Generator) -> np.ndarray:
    blocks = np.empty((count, 144), dtype=np.uint8)
    d = (np.abs(g.standard_normal(count)) * 0.01).astype(np.float32).astype(np.float16)
    dmin = (np.abs(g.standard_normal(count)) * 0.005).astype(np.float32).astype(np.float16)
    blocks[:, 0:2] = d.view(np.uint8).reshape(count, 2)
    blocks[:, 2:4] = dmin.view(np.uint8).reshape(count, 2)
    sc = g.integers(0, 64, (count, 8), dtype=np.uint8)
    mn = g.integers(0, 64, (count, 8), dtype=np.uint8)
    blocks[:, 4:16] = pack_q4_k_scales(sc, mn)
    nib = g.integers(0, 16, (count, 4, 2, 32), dtype=np.uint8)      # [chunk][low/high][lane]
    blocks[:, 16:] = (nib[:, :, 0, :] | (nib[:, :, 1, :] << 4)).reshape(count, 128)
    return blocks


def q5_k_blocks(count: int, g: np.random.Generator) -> np.ndarray:
    """Q4_K's header and scales, then qh[32] (bit 2*chunk + half of byte l is the fifth bit
    of that group's weight l) and qs[128]."""
    blocks = np.empty((count, 176), dtype=np.uint8)
    d = (np.abs(g.standard_normal(count)) * 0.005).astype(np.float32).astype(np.float16)
    dmin = (np.abs(g.standard_normal(count)) * 0.005).astype(np.float32).astype(np.float16)
    blocks[:, 0:2] = d.view(np.uint8).reshape(count, 2)
    blocks[:, 2:4] = dmin.view(np.uint8).reshape(count, 2)
    sc = g.integers(0, 64, (count, 8), dtype=np.uint8)
    mn = g.integers(0, 64, (count, 8), dtype=np.uint8)
    blocks[:, 4:16] = pack_q4_k_scales(sc, mn)
    q = g.integers(0, 32, (count, 4, 2, 32), dtype=np.uint8)        # [chunk][low/high][lane]
    low, top = q & 15, q >> 4
    blocks[:, 48:] = (low[:, :, 0, :] | (low[:, :, 1, :] << 4)).reshape(count, 128)
    qh = np.zeros((count, 32), dtype=np.uint8)
    for chunk in range(4):
        for half in range(2):
            qh |= top[:, chunk, half, :] << (2 * chunk + half)
    blocks[:, 16:48] = qh
    return blocks


def pack_q6_k_quants(q: np.ndarray):
    """``q`` is ``[blocks, 256]`` in 0..63 (the stored value, i.e. weight+32).
    Returns (ql ``[blocks,128]``, qh ``[blocks,64]``)."""
    q = np.asarray(q, dtype=np.uint8).reshape(-1, 2, 4, 32)           # [half][slice][lane]
    low, high = q & 15, q >> 4
    ql = np.empty((q.shape[0], 2, 2, 32), dtype=np.uint8)             # [half][slice&1][lane]
    ql[:, :, 0, :] = low[:, :, 0, :] | (low[:, :, 2, :] << 4)
    ql[:, :, 1, :] = low[:, :, 1, :] | (low[:, :, 3, :] << 4)
    qh = (high[:, :, 0, :] | (high[:, :, 1, :] << 2) | (high[:, :, 2, :] << 4)
          | (high[:, :, 3, :] << 6))
    return ql.reshape(-1, 128), qh.reshape(-1, 64)


def q6_k_blocks(count: int, g: np.random.Generator) -> np.ndarray:
    blocks = np.empty((count, 210), dtype=np.uint8)
    q = g.integers(0, 64, (count, 256), dtype=np.uint8)
    ql, qh = pack_q6_k_quants(q)
    blocks[:, 0:128] = ql
    blocks[:, 128:192] = qh
    blocks[:, 192:208] = g.integers(-64, 64, (count, 16), dtype=np.int8).view(np.uint8)
    d = (np.abs(g.standard_normal(count)) * 0.002).astype(np.float32).astype(np.float16)
    blocks[:, 208:210] = d.view(np.uint8).reshape(count, 2)
    return blocks


def iq4_xs_blocks(count: int, g: np.random.Generator) -> np.ndarray:
    """f16 d, u16 scales_h, scales_l[4], qs[128]: every 6-bit sub-block scale and every
    codebook index is drawn uniformly."""
    blocks = np.empty((count, 136), dtype=np.uint8)
    d = (np.abs(g.standard_normal(count)) * 0.0005).astype(np.float32).astype(np.float16)
    blocks[:, 0:2] = d.view(np.uint8).reshape(count, 2)
    ls = g.integers(0, 64, (count, 8), dtype=np.uint16)
    high = np.zeros(count, dtype=np.uint16)
    for i in range(8):
        high |= (ls[:, i] >> 4) << (2 * i)
    blocks[:, 2:4] = high.view(np.uint8).reshape(count, 2)
    low = (ls & 15).astype(np.uint8)
    blocks[:, 4:8] = low[:, 0::2] | (low[:, 1::2] << 4)
    blocks[:, 8:] = g.integers(0, 256, (count, 128), dtype=np.uint8)
    return blocks


def q8_0_blocks(count: int, g: np.random.Generator) -> np.ndarray:
    """`count` runs of 256 weights: eight 34-byte blocks (f16 d, int8 qs[32]) each."""
    blocks = np.empty((count * 8, 34), dtype=np.uint8)
    d = (np.abs(g.standard_normal(count * 8)) * 0.0005).astype(np.float32).astype(np.float16)
    blocks[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    blocks[:, 2:] = g.integers(-128, 128, (count * 8, 32), dtype=np.int8).view(np.uint8)
    return blocks.reshape(count, 272)


def matrix(ggml_type: int, rows: int, cols: int, seed: int, stream: int = 0) -> np.ndarray:
    """Packed row-major ``[rows, cols]`` matrix as a flat uint8 array."""
    g = rng(seed, stream)
    if ggml_type == Q8_0 and cols % 32 == 0 and cols % 256:
        # rows of 32 n weights that do not end on a run of eight blocks: whole runs, cut to length
        blocks = rows * (cols // 32)
        return q8_0_blocks((blocks + 7) // 8, g).reshape(-1)[:blocks * 34].copy()
    if cols % 256:
        raise ValueError("columns must be a multiple of 256 (of 32 for Q8_0)")
    count = rows * (cols // 256)
    if ggml_type == Q4_K:
        return q4_k_blocks(count, g).reshape(-1)
    if ggml_type == Q5_K:
        return q5_k_blocks(count, g).reshape(-1)
    if ggml_type == Q6_K:
        return q6_k_blocks(count, g).reshape(-1)
    if ggml_type == IQ4_XS:
        return iq4_xs_blocks(count, g).reshape(-1)
    if ggml_type == Q8_0:
        return q8_0_blocks(count, g).reshape(-1)
    raise ValueError(f"unsupported ggml type {ggml_type}")


def activations(m: int, k: int, seed: int, stream: int = 1000, f16: bool = False) -> np.ndarray:
    x = rng(seed, stream).standard_normal((m, k)).astype(np.float32)
    if f16:
        x = x.astype(np.float16).astype(np.float32)
    return x
