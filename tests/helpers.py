"""Shared helpers for the parity tests."""
import contextlib

import numpy as np

import oracle


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def rel_l2(got, want):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float(np.linalg.norm(got - want) / np.linalg.norm(want))


def max_rel(got, want):
    """Largest |got-want| / max(|want|, floor): the reference's own tolerance
    form abs <= tol*max(|ref|, floor) (src/ops/transformer.rs:3023), with the
    floor set to the RMS of the reference so near-zero outputs of a
    zero-mean product do not dominate."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    floor = float(np.sqrt(np.mean(want * want)))
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), floor)))


def assert_matmul_parity(got, want, what, max_rel_tol=1e-3, l2_tol=1e-5):
    assert np.abs(want).max() > 1e-3, f"{what}: reference is vacuous"
    l2, mr = rel_l2(got, want), max_rel(got, want)
    assert l2 <= l2_tol, f"{what}: relative L2 {l2:.3e} > {l2_tol:.0e}"
    assert mr <= max_rel_tol, f"{what}: max relative error {mr:.3e} > {max_rel_tol:.0e}"
    return l2, mr


def oracle_columns(ggml_type, packed, n, k, rows, x, **kw):
    """Oracle projection restricted to the weight rows in `rows` (a sample of
    output columns), for shapes whose full product is too slow on the CPU."""
    row_bytes = oracle.row_bytes(ggml_type, k)
    sub = np.ascontiguousarray(packed.reshape(n, row_bytes)[rows]).reshape(-1)
    return oracle.project(ggml_type, sub, len(rows), k, x, **kw)


@contextlib.contextmanager
def fma_gemv(d):
    """Dense Q4_K and Q6_K GEMVs inside the block take the FMA kernel, the one the fused and
    per-assignment launches run on, so results can be compared with them bit for bit (the
    streamed matrix-core GEMV sums in another order and agrees to the matmul tolerance)."""
    before = d.get_tuning("gemv_stream")
    d.set_tuning("gemv_stream", 0)
    try:
        yield
    finally:
        d.set_tuning("gemv_stream", before)
