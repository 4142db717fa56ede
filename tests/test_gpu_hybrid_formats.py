"""GPU parity of the hybrid engine's IQ4_XS and Q8_0 (GGML types 23 and 8, Format::Iq4Xs /
Format::Q8_0, src/hybrid/weights.rs:29-60) through every kernel family, against the CPU
oracle and through the C ABI.

The reference tests its IQ formats with random blocks, shapes (rows, cols) = (13, 1024),
M in {1, 3, 16, 64}, f32 activations and |err| <= 5e-3 * max|ref| against the float64
product of the CPU dequant (src/hybrid/iq_tests.rs:1300-1337); those cases are replayed
here with its block generator, then held to this build's bars (dequant bit-exact, matmul
max-rel 1e-3 and rel-L2 1e-5) at larger shapes on seeded blocks.
"""
import numpy as np
import pytest

import ferrum_fixtures as fx
import oracle
from helpers import assert_matmul_parity, bits, oracle_columns
from ferrum_amd import synth

pytestmark = pytest.mark.gpu

IQ4_XS, Q8_0 = 23, 8
NAME = {IQ4_XS: "iq4_xs", Q8_0: "q8_0"}
UNIT = {IQ4_XS: 136, Q8_0: 272}            # bytes per 256 weights
FORMATS = pytest.mark.parametrize("ggml", [IQ4_XS, Q8_0], ids=["iq4_xs", "q8_0"])


def reference_blocks(ggml, rows, cols, seed_offset=0):
    """random_blocks(.., block, block as u64) as the reference's format tests call it for
    their own kinds: the GGML block size is both the stride and the seed
    (src/hybrid/iq_tests.rs:1308)."""
    block = 136 if ggml == IQ4_XS else 34
    return fx.hybrid_random_blocks(rows * cols * UNIT[ggml] // 256 // block, block, seed_offset + block)


@pytest.fixture(scope="module")
def api():
    from ferrum_amd import api as module
    return module


@pytest.fixture(scope="module")
def d(api):
    return api.Device.new()


def qm(api, d, rows, cols, packed, ggml=IQ4_XS):
    return api.QuantizedMatrix.from_bytes(d, rows, cols, api.QuantizationFormat(ggml), packed)


@FORMATS
def test_dequantize_and_gather_are_bit_exact(api, d, ggml):
    for rows, cols, packed in ((13, 1024, reference_blocks(ggml, 13, 1024)),
                               (257, 2560, synth.matrix(ggml, 257, 2560, seed=301))):
        w = qm(api, d, rows, cols, packed, ggml)
        assert w.byte_size() == rows * (cols // 256) * UNIT[ggml]
        want = oracle.dequantize(ggml, packed, rows, cols)
        out = d.dequantize(w)
        assert d.last_operation() == f"dequantize_{NAME[ggml]}"
        assert np.array_equal(bits(out.to_f32()), bits(want))
        for dtype, code in ((api.DType.F16, oracle.F16), (api.DType.BF16, oracle.BF16)):
            assert np.array_equal(bits(d.dequantize(w, dtype).to_f32()),
                                  bits(oracle.round_storage(want, code).reshape(rows, cols)))
        ids = [rows - 1, 0, 3, 3]
        got = d.embedding_gather_quantized(w, ids, api.DType.F32)
        assert got.operation == f"embedding_gather_{NAME[ggml]}"
        assert np.array_equal(bits(got.tensor.to_f32()), bits(want[ids]))


@FORMATS
def test_projections_replay_the_reference_iq_cases(api, d, ggml):
    # iq_projections_match_the_cpu_dequant (src/hybrid/iq_tests.rs:1300-1337)
    rows, cols = 13, 1024
    packed = reference_blocks(ggml, rows, cols)
    w = qm(api, d, rows, cols, packed, ggml)
    dense = oracle.dequantize(ggml, packed, rows, cols).astype(np.float64)
    for m in (1, 3, 16, 64):
        x = fx.xorshift_uniform(m * cols, m, multiplier=0x2545F4914F6CDD1D).reshape(m, cols)
        out = d.project_quantized(api.Tensor.from_f32(d, x.shape, api.DType.F32, x), w)
        assert out.operation == (f"{NAME[ggml]}_gemv_factored" if m == 1 else f"{NAME[ggml]}_gemm")
        want = x.astype(np.float64) @ dense.T
        scale = np.abs(want).max()
        assert scale > 1e-2
        assert np.abs(out.tensor.to_f32() - want).max() <= 5e-3 * scale       # the reference's bound
        assert_matmul_parity(out.tensor.to_f32(), want, f"{NAME[ggml]} m={m}")     # this build's


@pytest.mark.parametrize("n,k,m,dtype_name", [(4099, 5120, 1, "F32"), (1003, 4864, 1, "F32"), (5120, 17408, 1, "F32"),
                                              (17408, 5120, 1, "F32"), (515, 1280, 3, "F32"), (515, 1280, 1, "F16"),
                                              (515, 1280, 1, "BF16")])
@FORMATS
def test_gemv_matches_the_f64_oracle(api, d, ggml, n, k, m, dtype_name):
    dtype = api.DType[dtype_name]
    code = {"F32": oracle.F32, "F16": oracle.F16, "BF16": oracle.BF16}[dtype_name]
    packed = synth.matrix(ggml, n, k, seed=n + k)
    w = qm(api, d, n, k, packed, ggml)
    x = oracle.round_storage(synth.activations(m, k, seed=11), code).reshape(m, k)
    out = d.project_quantized(api.Tensor.from_f32(d, x.shape, dtype, x), w, out_dtype=api.DType.F32)
    rows = np.unique(np.concatenate([np.arange(0, 40), np.arange(n - 40, n), synth.rng(12).integers(0, n, 64)]))
    want = oracle_columns(ggml, packed, n, k, rows, x, accumulate="f64")
    assert_matmul_parity(out.tensor.to_f32()[:, rows], want, f"{NAME[ggml]} {n}x{k} m={m} {dtype_name}")
    if k == 17408:
        assert out.operation == f"{NAME[ggml]}_gemv_ksplit"


@pytest.mark.parametrize("m,n,dtype_name", [(8, 1100, "F16"), (20, 1100, "BF16"), (50, 1100, "F16"), (130, 1000, "F16"),
                                            (130, 16000, "BF16"), (300, 33000, "F16"), (300, 33000, "BF16")])
@FORMATS
def test_tile_kernels_match_the_rounded_weight_oracle(api, d, ggml, m, n, dtype_name):
    # register-dequant kernel (M <= 64), 64- and 128-wide tiles, and the 256-row tile
    k = 768
    dtype = api.DType[dtype_name]
    code = oracle.F16 if dtype_name == "F16" else oracle.BF16
    packed = synth.matrix(ggml, n, k, seed=311 + n)
    w = qm(api, d, n, k, packed, ggml)
    x = oracle.round_storage(synth.activations(m, k, seed=312), code).reshape(m, k)
    d.set_tuning("gemm_resident", 0)   # the square tiles: rows this short would otherwise stay in LDS,
    d.set_tuning("gemm_wide_shape", 0) # and 130 x 16000 would fill the chip with 128-row tiles of the 32x32x16 form
    try:
        out = d.project_quantized(api.Tensor.from_f32(d, x.shape, dtype, x), w, out_dtype=api.DType.F32)
    finally:
        d.set_tuning("gemm_resident", 1)
        d.set_tuning("gemm_wide_shape", 1)
    suffix = {8: "_skinny", 20: "_skinny", 50: "_skinny", 130: "", 300: "_m256"}[m]
    assert out.operation == f"{NAME[ggml]}_gemm_mfma{suffix}"
    rows = np.unique(np.concatenate([np.arange(0, 150), np.arange(n - 150, n), synth.rng(313).integers(0, n, 64)]))
    want = oracle_columns(ggml, packed, n, k, rows, x, weight_round=code, accumulate="f64")
    assert_matmul_parity(out.tensor.to_f32()[:, rows], want, f"{NAME[ggml]} tile m={m} n={n}")


@FORMATS
def test_tile_values_are_the_dequantised_weights_rounded_once(api, d, ggml):
    # X = identity rows: the product reads the tile values themselves
    n, k = 200, 256
    packed = synth.matrix(ggml, n, k, seed=321)
    w = qm(api, d, n, k, packed, ggml)
    dense = oracle.dequantize(ggml, packed, n, k)
    eye = np.eye(k, dtype=np.float32)
    for dtype, code in ((api.DType.F16, oracle.F16), (api.DType.BF16, oracle.BF16)):
        for m0, m1 in ((0, 40), (40, 256)):              # register-dequant kernel, then the tiles
            x = eye[m0:m1]
            out = d.project_quantized(api.Tensor.from_f32(d, x.shape, dtype, x), w, out_dtype=api.DType.F32)
            want = oracle.round_storage(dense[:, m0:m1].T.copy(), code).reshape(m1 - m0, n)
            # equal as numbers: a zero scale or quant gives -0 in the decoder and +0 from a sum
            got = out.tensor.to_f32()
            assert np.array_equal(got, want), (dtype, out.operation, np.argwhere(got != want)[:4])
            nonzero = want != 0
            assert np.array_equal(bits(got[nonzero]), bits(want[nonzero]))


@FORMATS
def test_expert_projection_per_assignment_and_grouped(api, d, ggml):
    # iq_expert_projections_match_the_cpu_dequant (src/hybrid/iq_tests.rs:1398-1437) in shape:
    # each route multiplies its own expert's slice
    experts, rows, cols = 3, 13, 1024
    packed = reference_blocks(ggml, experts * rows, cols, seed_offset=7)
    w = api.QuantizedExpertMatrix.new(d, packed, api.QuantizationFormat(ggml), experts, rows, cols)
    ids = [2, 0, 1, 1, 2]
    a = len(ids)
    meta = np.zeros((a, 3), dtype=np.uint32)
    meta[:, 0] = ids
    meta[:, 1] = np.arange(a)
    meta[:, 2] = np.float32(1.0).view(np.uint32)
    x = fx.xorshift_uniform(a * cols, 11, multiplier=0x2545F4914F6CDD1D).reshape(a, cols)
    got = d.expert_project_quantized(api.Tensor.from_f32(d, x.shape, api.DType.F32, x),
                                     api.Tensor.from_bits(d, meta.shape, meta), w, cols, experts).to_f32()
    assert d.last_operation() == f"expert_project_{NAME[ggml]}_factored"
    want = oracle.expert_project(ggml, packed, experts, rows, cols, x, meta.view(np.float32), accumulate="f64")
    assert np.abs(got - want).max() <= 5e-3 * np.abs(want).max()
    assert_matmul_parity(got, want, f"{NAME[ggml]} routes")

    # the grouped MFMA form: many assignments, f16 rows, ragged expert sizes (one empty)
    experts, rows, cols, a = 6, 200, 768, 150
    packed = synth.matrix(ggml, experts * rows, cols, seed=331)
    w = api.QuantizedExpertMatrix.new(d, packed, api.QuantizationFormat(ggml), experts, rows, cols)
    rng = synth.rng(332)
    ids = rng.choice([0, 1, 2, 4, 5], size=a, p=[0.4, 0.05, 0.25, 0.2, 0.1])   # expert 3 gets nothing
    meta = np.zeros((a, 3), dtype=np.uint32)
    meta[:, 0] = np.sort(ids)
    meta[:, 1] = rng.integers(0, 64, a)
    meta[:, 2] = np.float32(1.0).view(np.uint32)
    x = oracle.round_storage(synth.activations(a, cols, seed=333) * 0.25, oracle.F16).reshape(a, cols)
    got = d.expert_project_quantized(api.Tensor.from_f32(d, x.shape, api.DType.F16, x),
                                     api.Tensor.from_bits(d, meta.shape, meta), w, cols, experts,
                                     out_dtype=api.DType.F32).to_f32()
    assert d.last_operation() == f"expert_project_{NAME[ggml]}_grouped_mfma"
    want = oracle.expert_project(ggml, packed, experts, rows, cols, x, meta.view(np.float32), accumulate="f64",
                                 weight_round=oracle.F16)
    assert_matmul_parity(got, want, f"{NAME[ggml]} grouped routes")


@FORMATS
def test_validation(api, d, ggml):
    rows, cols = 4, 512
    packed = synth.matrix(ggml, rows, cols, seed=341)
    bad = packed.copy()
    bad[1] = 0x7c                                       # d = +inf in the first block
    with pytest.raises(api.WeightError):
        qm(api, d, rows, cols, bad, ggml)
    if ggml == IQ4_XS:
        ok = packed.copy()
        ok[2:4] = 0xff                                  # scales_h is not a float: any bits are fine
        qm(api, d, rows, cols, ok, ggml)
    else:
        bad = packed.copy()
        bad[34 * 11 + 1] = 0x7e                         # NaN scale in the twelfth 34-byte block
        with pytest.raises(api.WeightError):
            qm(api, d, rows, cols, bad, ggml)
        with pytest.raises(api.ShapeError):             # a row is whole 32-weight blocks
            qm(api, d, rows, 304, packed[: rows * 9 * 34], ggml)
    with pytest.raises(api.Error):
        qm(api, d, rows, cols, packed[:-1], ggml)
