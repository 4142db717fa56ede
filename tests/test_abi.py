"""CPU-only checks of the drop-in boundary: the shared library loads and exports
every symbol include/ferrum_hip.h declares, and the host mirror's own
validation (no GPU work) behaves like the reference's."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ferrum_hip.h")
# measurement kernels, declared apart from the operator surface
PROBE_HEADER = os.path.join(ROOT, "include", "ferrum_hip_probe.h")


def declared_symbols(path=None):
    texts = [open(p).read() for p in ([path] if path else [HEADER, PROBE_HEADER])]
    text = re.sub(r"/\*.*?\*/", "", "\n".join(texts), flags=re.S)
    return sorted(set(re.findall(r"\b(fh_[a-z0-9_]+)\s*\(", text)))


def test_measurement_kernels_stay_out_of_the_operator_header():
    assert not [n for n in declared_symbols(HEADER) if n.startswith("fh_probe_")]
    assert declared_symbols(PROBE_HEADER) == ["fh_probe_coissue", "fh_probe_mfma", "fh_probe_read"]


def test_library_exports_every_declared_symbol():
    from ferrum_amd import api
    lib = ctypes.CDLL(api.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 30
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    # the python binding table covers the header exactly
    assert sorted(api.SYMBOLS) == names


def test_header_cites_a_reference_interface_for_each_operator():
    text = open(HEADER).read()
    for op in ("fh_project_quantized", "fh_moe_route", "fh_expert_assign",
               "fh_expert_project_quantized", "fh_expert_silu_mul", "fh_expert_combine",
               "fh_qmatrix_create", "fh_embedding_gather_quantized"):
        before = text[:text.index(op + "(")]
        comment = before[before.rindex("/*"):]
        assert re.search(r"src/[a-z_/]+\.(rs|metal):\d+", comment), op


def test_error_codes_mirror_the_reference_variants():
    from ferrum_amd import api
    text = open(HEADER).read()
    codes = dict(re.findall(r"FH_ERR_([A-Z_]+) = (\d+)", text))
    assert {int(v) for v in codes.values()} == set(api._ERRORS)
    assert api._ERRORS[int(codes["SHAPE"])].kind == "Shape"
    assert api._ERRORS[int(codes["DEVICE_MISMATCH"])].kind == "DeviceMismatch"
    assert api._ERRORS[int(codes["WEIGHT"])].kind == "Weight"


def test_format_geometry_matches_ggml():
    # src/quantization.rs:302-313, src/loader/gguf.rs:933-963
    from ferrum_amd import api
    q4 = api.QuantizationFormat.from_ggml_type(12)
    q6 = api.QuantizationFormat.from_ggml_type(14)
    assert (q4.ggml_type(), q4.block_elements(), q4.block_bytes()) == (12, 256, 144)
    assert (q6.ggml_type(), q6.block_elements(), q6.block_bytes()) == (14, 256, 210)
    with pytest.raises(api.GgufError):
        api.QuantizationFormat.from_ggml_type(5)


def test_storage_encoding_rounds_like_the_oracle():
    import oracle
    from ferrum_amd import api
    rng = np.random.default_rng(2)
    v = np.concatenate([rng.standard_normal(2000).astype(np.float32),
                        np.array([1.00390625, 1.01171875, np.inf, -0.0], dtype=np.float32)])
    for dtype, code in ((api.DType.F16, oracle.F16), (api.DType.BF16, oracle.BF16)):
        back = api.decode(api.encode(v, dtype).view(np.uint8), dtype)
        assert np.array_equal(back.view(np.uint32), oracle.round_storage(v, code).view(np.uint32))


def test_synthetic_blocks_have_the_stated_distributions():
    import oracle
    from ferrum_amd import synth
    rows, cols = 64, 1024
    p4 = synth.matrix(12, rows, cols, seed=5).reshape(-1, 144)
    d = p4[:, 0:2].copy().view(np.float16).astype(np.float64).reshape(-1)
    dmin = p4[:, 2:4].copy().view(np.float16).astype(np.float64).reshape(-1)
    assert 0.006 < d.mean() < 0.010 and 0.003 < dmin.mean() < 0.005     # E|N(0,1)| = 0.798
    nib = np.concatenate([p4[:, 16:] & 15, p4[:, 16:] >> 4])
    assert abs(nib.mean() - 7.5) < 0.1
    assert oracle.validate_payload(12, p4.reshape(-1)) == 0
    p6 = synth.matrix(14, rows, cols, seed=5)
    dense = oracle.dequantize(14, p6, rows, cols)
    b6 = p6.reshape(-1, 210)
    d6 = b6[:, 208:210].copy().view(np.float16).astype(np.float32).reshape(-1)
    sc = b6[:, 192:208].view(np.int8).astype(np.float32)
    # stored quant = dense / (d*scale) + 32 must be uniform in 0..63
    blk = dense.reshape(-1, 16, 16)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = blk / (d6[:, None, None] * sc[:, :, None]) + 32
    q = q[np.isfinite(q)]
    assert np.all(np.abs(q - np.round(q)) < 1e-3) and q.min() >= -0.01 and q.max() <= 63.01
    assert abs(q.mean() - 31.5) < 0.3
    assert sc.min() == -64 and sc.max() == 63
    # same seed, same bytes
    assert np.array_equal(p6, synth.matrix(14, rows, cols, seed=5))
