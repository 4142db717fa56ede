"""GPU parity of the dense path (dequantize, GEMV, small-M, tile GEMM) against
the CPU oracle, through the C ABI.

The first half replays the reference's own test cases for this path
(src/ops/transformer.rs qk_tests / q6_k_tests, src/diffusion/tests.rs:716-761)
with its closed-form inputs and its tolerances; the second half applies the
benchmark's bars (dequant bit-exact; max relative error 1e-3 and relative L2
1e-5 with f32 accumulation) at the benchmark shapes on seeded synthetic blocks.
"""
import numpy as np
import pytest

import ferrum_fixtures as fx
import oracle
from helpers import assert_matmul_parity, bits, fma_gemv, oracle_columns, rel_l2
from ferrum_amd import synth

pytestmark = pytest.mark.gpu

Q4_K, Q6_K = 12, 14


@pytest.fixture(scope="module")
def api():
    from ferrum_amd import api as module
    return module


@pytest.fixture(scope="module")
def d(api):
    return api.Device.new()


def qm(api, d, ggml, rows, cols, packed):
    fmt = api.QuantizationFormat(ggml)
    return api.QuantizedMatrix.from_reader(d, rows, cols, fmt, lambda dst: np.copyto(dst, packed))


# ------------------------------------------------------------- dequantize

@pytest.mark.parametrize("ggml,rows,cols", [(Q4_K, 5, 512), (Q6_K, 5, 512), (Q4_K, 133, 2560),
                                            (Q6_K, 133, 2560)])
def test_dequantize_is_bit_exact_on_reference_fixtures(api, d, ggml, rows, cols):
    packed = fx.q4k_packed(rows, cols) if ggml == Q4_K else fx.q6k_packed(rows, cols)
    w = qm(api, d, ggml, rows, cols, packed)
    assert w.byte_size() == rows * (cols // 256) * (144 if ggml == Q4_K else 210)
    got = d.dequantize(w).to_f32()
    assert np.array_equal(bits(got), bits(oracle.dequantize(ggml, packed, rows, cols)))


@pytest.mark.parametrize("ggml", [Q4_K, Q6_K])
def test_dequantize_is_bit_exact_on_synthetic_blocks_in_every_dtype(api, d, ggml):
    rows, cols = 257, 5120
    packed = synth.matrix(ggml, rows, cols, seed=1234)
    w = qm(api, d, ggml, rows, cols, packed)
    want = oracle.dequantize(ggml, packed, rows, cols)
    assert np.array_equal(bits(d.dequantize(w).to_f32()), bits(want))
    for dtype, code in ((api.DType.F16, oracle.F16), (api.DType.BF16, oracle.BF16)):
        got = d.dequantize(w, dtype).to_f32()
        assert np.array_equal(bits(got), bits(oracle.round_storage(want, code).reshape(rows, cols)))


def test_embedding_gather_decodes_selected_rows(api, d):
    # src/ops/transformer.rs:3307-3329 and :4351-4369: bitwise after BF16 rounding
    for ggml, packed in ((Q4_K, fx.q4k_packed(5, 512)), (Q6_K, fx.q6k_packed(5, 512))):
        w = qm(api, d, ggml, 5, 512, packed)
        ids = [4, 0, 3]
        out = d.embedding_gather_quantized(w, ids, api.DType.BF16)
        assert out.operation == ("embedding_gather_q4_k" if ggml == Q4_K else "embedding_gather_q6_k")
        dense = oracle.dequantize(ggml, packed, 5, 512)
        want = oracle.round_storage(dense[ids], oracle.BF16).reshape(3, 512)
        assert np.array_equal(bits(out.tensor.to_f32()), bits(want))
        with pytest.raises(api.TokenError):
            d.embedding_gather_quantized(w, [5], api.DType.BF16)


# ---------------------------------------------- the reference's GEMV / GEMM cases

def test_q4_k_gemv_gemm_cover_blocks_and_batch_tails(api, d):
    # src/ops/transformer.rs:2982-3002
    n, k = 5, 512
    packed = fx.q4k_packed(n, k)
    w = qm(api, d, Q4_K, n, k, packed)
    for m in (1, 2, 3, 4, 5, 7):
        values = fx.q4k_input(m, k)
        x = api.Tensor.from_f32(d, (m, k), api.DType.F32, values)
        actual = d.project_quantized(x, w).tensor.to_f32()
        reference = oracle.project(Q4_K, packed, n, k, values)
        assert np.abs(actual - reference).max() <= 2.0e-4, m


def test_q6_k_gemv_gemm_cover_superblock_and_batch_tails(api, d):
    # src/ops/transformer.rs:4251-4269
    n, k = 5, 512
    packed = fx.q6k_packed(n, k)
    w = qm(api, d, Q6_K, n, k, packed)
    for m in (1, 2, 3, 4, 5, 7):
        values = fx.q6k_input(m, k)
        x = api.Tensor.from_f32(d, (m, k), api.DType.F32, values)
        actual = d.project_quantized(x, w).tensor.to_f32()
        reference = oracle.project(Q6_K, packed, n, k, values)
        assert np.abs(actual - reference).max() <= 0.02, m
        # far tighter than the reference asks: f32 parity
        assert np.abs(actual - reference).max() <= 1e-4 * max(1.0, np.abs(reference).max())


@pytest.mark.parametrize("ggml", [Q4_K, Q6_K])
def test_gemv_ksplit_covers_row_and_block_tails(api, d, ggml):
    # src/ops/transformer.rs:3004-3029 and :4190-4214: 133 rows leave a partial
    # row tile; 10 and 19 super-blocks leave partial strides for every split.
    with pytest.raises(api.ParameterError):
        d.set_k_quant_gemv_ksplit(3)
    try:
        for n, k in ((133, 2560), (6, 4864)):
            packed = fx.q4k_packed(n, k) if ggml == Q4_K else fx.q6k_packed(n, k)
            values = fx.q4k_input(1, k) if ggml == Q4_K else fx.q6k_input(1, k)
            w = qm(api, d, ggml, n, k, packed)
            x = api.Tensor.from_f32(d, (1, k), api.DType.F32, values)
            reference = oracle.project(ggml, packed, n, k, values)
            outputs = []
            for simds in (1, 2, 4, 8):
                d.set_k_quant_gemv_ksplit(simds)
                out = d.project_quantized(x, w)
                name = "q4_k" if ggml == Q4_K else "q6_k"
                assert out.operation == (f"{name}_gemv_ksplit" if simds > 1 else f"{name}_gemv_factored")
                actual = out.tensor.to_f32()
                assert np.all(np.abs(actual - reference) <= 1.0e-3 * np.maximum(np.abs(reference), 1.0)), \
                    (n, k, simds)
                # segments meet in a fixed order: a second launch gives the same bits
                again = d.project_quantized(x, w).tensor.to_f32()
                assert np.array_equal(bits(actual), bits(again))
                outputs.append(actual)
    finally:
        d.set_k_quant_gemv_ksplit(0)


@pytest.mark.parametrize("dtype_name", ["F16", "BF16"])
def test_gemv_accepts_half_precision_activations(api, d, dtype_name):
    n, k = 133, 1024
    dtype = api.DType[dtype_name]
    code = oracle.F16 if dtype_name == "F16" else oracle.BF16
    for ggml in (Q4_K, Q6_K):
        packed = fx.q4k_packed(n, k) if ggml == Q4_K else fx.q6k_packed(n, k)
        w = qm(api, d, ggml, n, k, packed)
        values = fx.q4k_input(1, k)
        x = api.Tensor.from_f32(d, (1, k), dtype, values)
        rounded = x.to_f32()
        assert np.array_equal(rounded, oracle.round_storage(values, code).reshape(1, k))
        out = d.project_quantized(x, w)                      # output dtype = input dtype
        want = oracle.project(ggml, packed, n, k, rounded, accumulate="f64")
        assert np.array_equal(out.tensor.to_f32(), oracle.round_storage(out.tensor.to_f32(), code).reshape(1, n))
        assert rel_l2(out.tensor.to_f32(), want) <= (1e-3 if dtype_name == "F16" else 6e-3)
        out32 = d.project_quantized(x, w, out_dtype=api.DType.F32).tensor.to_f32()
        assert_matmul_parity(out32, want, f"{dtype_name} gemv")


def test_k_quant_gemms_match_the_cpu_dequant(api, d):
    # src/diffusion/tests.rs:716-761: F16 activations, M=200, K=512, N=100,
    # f64-accumulated CPU dequant, worst error <= 2e-3 * max|ref|.
    m, k, n = 200, 512, 100
    x = oracle.round_storage(fx.xorshift_uniform(m * k, 31), oracle.F16).reshape(m, k)
    for ggml in (Q4_K, Q6_K):
        packed = fx.xorshift_blocks(ggml, n * k // 256)
        w = qm(api, d, ggml, n, k, packed)
        xt = api.Tensor.from_f32(d, (m, k), api.DType.F16, x)
        out = d.project_quantized(xt, w, out_dtype=api.DType.F32)
        assert out.operation.startswith("q4_k_gemm_mfma" if ggml == Q4_K else "q6_k_gemm_mfma")
        got = out.tensor.to_f32()
        want = oracle.project(ggml, packed, n, k, x, accumulate="f64")
        scale = np.abs(want).max()
        assert scale > 0.1, "reference is vacuous"
        assert np.abs(got - want).max() <= 2e-3 * scale
        # against the tile-dtype oracle (weights rounded to f16 first) the
        # result is f32-accumulation accurate
        tile = oracle.project(ggml, packed, n, k, x, accumulate="f64", weight_round=oracle.F16)
        assert_matmul_parity(got, tile, "f16 tile gemm")


def test_bf16_tile_gemm_covers_row_output_and_group_tails(api, d):
    # src/ops/transformer.rs:3115-3175: (N, K) = (65, 512), M in {4, 8, 15, 35},
    # BF16 activations, weights rounded to BF16, result stored as BF16, abs <= 0.04.
    n, k = 65, 512
    for ggml, tol in ((Q4_K, 0.04), (Q6_K, 0.12)):
        packed = fx.q4k_packed(n, k) if ggml == Q4_K else fx.q6k_packed(n, k)
        w = qm(api, d, ggml, n, k, packed)
        for m in (4, 8, 15, 35):
            values = fx.q4k_input(m, k) if ggml == Q4_K else fx.q6k_input(m, k)
            x = api.Tensor.from_f32(d, (m, k), api.DType.BF16, values)
            rounded = x.to_f32()
            expected = oracle.project(ggml, packed, n, k, rounded, weight_round=oracle.BF16,
                                      out_round=oracle.BF16)
            out = d.project_quantized(x, w)
            assert "gemm_mfma" in out.operation
            assert np.abs(out.tensor.to_f32() - expected).max() <= tol, (ggml, m)


@pytest.mark.parametrize("ggml,dtype_name", [(Q4_K, "F16"), (Q6_K, "BF16")])
def test_tile_gemm_both_tile_sizes_match_the_f16_tile_oracle(api, d, ggml, dtype_name):
    # M = 130 rows: N = 16000 takes 128 x 128 tiles (250 workgroups), N = 1000 takes
    # 64 x 64 tiles; both have ragged last tiles in M and N.  Oracle on sampled columns.
    k, m = 512, 130
    dtype = api.DType[dtype_name]
    code = oracle.F16 if dtype_name == "F16" else oracle.BF16
    x = oracle.round_storage(synth.activations(m, k, seed=91), code).reshape(m, k)
    xt = api.Tensor.from_f32(d, x.shape, dtype, x)
    for n in (16000, 1000):
        packed = synth.matrix(ggml, n, k, seed=92 + n)
        w = qm(api, d, ggml, n, k, packed)
        d.set_tuning("gemm_resident", 0)   # rows this short would otherwise stay in LDS (tested below),
        d.set_tuning("gemm_wide_shape", 0) # and the 128-row tiles of the 32x32x16 form would take 16000 columns
        try:
            out = d.project_quantized(xt, w, out_dtype=api.DType.F32)
        finally:
            d.set_tuning("gemm_resident", 1)
            d.set_tuning("gemm_wide_shape", 1)
        assert out.operation == ("q4_k_gemm_mfma" if ggml == Q4_K else "q6_k_gemm_mfma")
        got = out.tensor.to_f32()
        rows = np.unique(np.concatenate([np.arange(0, 130), np.arange(n - 70, n),
                                         synth.rng(93).integers(0, n, 64)]))
        want = oracle_columns(ggml, packed, n, k, rows, x, weight_round=code, accumulate="f64")
        assert_matmul_parity(got[:, rows], want, f"tile gemm n={n}")


@pytest.mark.parametrize("ggml,dtype_name", [(Q4_K, "F16"), (Q4_K, "BF16"), (synth.Q5_K, "F16"),
                                             (synth.Q5_K, "BF16"), (Q6_K, "F16"), (Q6_K, "BF16")])
def test_register_dequant_gemm_up_to_64_rows(api, d, ggml, dtype_name):
    # 33..64 rows stay on the kernel that dequantises in registers (four 16-row MFMA
    # operands per wave); 65 is the first row count on the 256-row tile.  N = 1100 leaves
    # a ragged last row group.
    n, k = 1100, 1280
    dtype = api.DType[dtype_name]
    code = oracle.F16 if dtype_name == "F16" else oracle.BF16
    packed = synth.matrix(ggml, n, k, seed=131)
    w = qm(api, d, ggml, n, k, packed)
    for m in (32, 33, 49, 64, 65):
        x = oracle.round_storage(synth.activations(m, k, seed=132 + m), code).reshape(m, k)
        d.set_tuning("gemm_resident", 0)   # rows too long for LDS take these kernels; these would fit
        try:
            out = d.project_quantized(api.Tensor.from_f32(d, x.shape, dtype, x), w, out_dtype=api.DType.F32)
        finally:
            d.set_tuning("gemm_resident", 1)
        assert out.operation.endswith("_skinny") == (m <= 64), (m, out.operation)
        want = oracle.project(ggml, packed, n, k, x, weight_round=code, accumulate="f64")
        assert_matmul_parity(out.tensor.to_f32(), want, f"{dtype_name} m={m}")


@pytest.mark.parametrize("ggml", [Q4_K, Q6_K])
def test_f32_activations_take_the_tile_kernels_from_a_chosen_row_count(api, d, ggml):
    # HybridModel::project (src/hybrid/engine.rs:3407-3500) sends f32 activations to f16
    # tiles from 5 rows on; here that is opt-in, and below the threshold (or with the key at
    # 0) every row keeps exact f32 weights.
    n, k = 1100, 1024
    packed = synth.matrix(ggml, n, k, seed=121)
    w = qm(api, d, ggml, n, k, packed)
    d.set_tuning("gemm_f32_min_rows", 5)
    try:
        for m in (4, 5, 16, 40, 130):
            x = synth.activations(m, k, seed=122 + m)
            out = d.project_quantized(api.Tensor.from_f32(d, x.shape, api.DType.F32, x), w)
            assert out.tensor.dtype == api.DType.F32
            if m < 5:
                assert out.operation.endswith("_gemm") and "mfma" not in out.operation
                want = oracle.project(ggml, packed, n, k, x, accumulate="f64")
            else:
                assert "gemm_mfma" in out.operation
                want = oracle.project(ggml, packed, n, k, oracle.round_storage(x, oracle.F16).reshape(m, k),
                                      weight_round=oracle.F16, accumulate="f64")
            assert_matmul_parity(out.tensor.to_f32(), want, f"f32 activations m={m}")
    finally:
        d.set_tuning("gemm_f32_min_rows", 0)
    x = synth.activations(16, k, seed=123)
    exact = d.project_quantized(api.Tensor.from_f32(d, x.shape, api.DType.F32, x), w)
    assert "mfma" not in exact.operation
    assert_matmul_parity(exact.tensor.to_f32(), oracle.project(ggml, packed, n, k, x, accumulate="f64"), "exact f32")
    with pytest.raises(api.ParameterError):
        d.set_tuning("gemm_f32_min_rows", 1)


# ------------------------------------------------------- benchmark shapes

def check_gemv(api, d, ggml, n, k, seed, l2_tol=1e-5):
    packed = synth.matrix(ggml, n, k, seed)
    x = synth.activations(1, k, seed)
    w = qm(api, d, ggml, n, k, packed)
    xt = api.Tensor.from_f32(d, (1, k), api.DType.F32, x)
    got = d.project_quantized(xt, w).tensor.to_f32()
    want64 = oracle.project(ggml, packed, n, k, x, accumulate="f64", threads=8)
    want32 = oracle.project(ggml, packed, n, k, x, accumulate="f32", threads=8)
    l2, mr = assert_matmul_parity(got, want64, f"gemv {ggml} {n}x{k} vs f64", l2_tol=l2_tol)
    # the reference's sequential-f32 answer, whose own rounding error grows with K
    assert_matmul_parity(got, want32, f"gemv {ggml} {n}x{k} vs f32seq", l2_tol=l2_tol)
    assert l2 <= rel_l2(want32, want64) * 1.5 + 1e-7, "GPU is less accurate than the sequential CPU sum"


# The streamed matrix-core GEMV (dense Q4_K and Q6_K): row lengths on both sides of its per-wave
# block budgets, tile heights 1..16, every activation dtype, batched rows; rows too long for one
# tile (more than 48 super-blocks, or 16 rows of them past 64 KB) are cut into 2 to 6 K segments.
# Q6_K rows take it when they hold an even number of super-blocks (their 210-byte blocks then start
# on a dword).
STREAM_SHAPES = [(Q4_K, n, k) for n, k in [(37, 256), (133, 2560), (300, 4864), (1100, 5120), (4100, 2048), (70, 6144),
                                           (33, 8192), (20, 12288), (100, 12544), (777, 14336), (530, 17408),
                                           (64, 34816)]]
STREAM_SHAPES += [(Q6_K, n, k) for n, k in [(37, 512), (133, 2560), (300, 4608), (1100, 5120), (4100, 2048), (70, 6144),
                                            (33, 8192), (200, 9728), (20, 12288), (100, 12800), (777, 14336),
                                            (530, 17408), (64, 34816)]]


@pytest.mark.parametrize("ggml,n,k", STREAM_SHAPES)
@pytest.mark.parametrize("dtype", ["F32", "F16", "BF16"])
def test_streamed_gemv_matches_the_oracle(api, d, ggml, n, k, dtype):
    code = {"F32": oracle.F32, "F16": oracle.F16, "BF16": oracle.BF16}[dtype]
    name = "q4_k" if ggml == Q4_K else "q6_k"
    packed = synth.matrix(ggml, n, k, seed=n + k)
    w = qm(api, d, ggml, n, k, packed)
    d.set_tuning("gemv_stream", 2)   # also where the matrix is small enough for the FMA kernel to win
    for m in ((1, 3) if dtype == "F32" else (1,)):   # 16-bit rows beyond the first take the tile kernels
        x = oracle.round_storage(synth.activations(m, k, seed=7 * n + m), code).reshape(m, k)
        xt = api.Tensor.from_f32(d, (m, k), getattr(api.DType, dtype), x)
        out = d.project_quantized(xt, w, out_dtype=api.DType.F32)
        if m > 1:
            assert out.operation == name + "_gemm"
        elif ggml == Q4_K:
            assert out.operation == ("q4_k_gemv_ksplit" if k > 12288 else "q4_k_gemv_factored")
        else:
            assert out.operation in ("q6_k_gemv_ksplit", "q6_k_gemv_factored")
            assert k <= 12288 or out.operation == "q6_k_gemv_ksplit"
        segmented = out.operation.endswith("ksplit")
        want = oracle.project(ggml, packed, n, k, x, accumulate="f64")
        assert_matmul_parity(out.tensor.to_f32(), want, f"streamed gemv {name} {n}x{k} {dtype} m={m}")
        if segmented:   # the segments are added in a fixed order
            again = d.project_quantized(xt, w, out_dtype=api.DType.F32).tensor.to_f32()
            assert np.array_equal(bits(again), bits(out.tensor.to_f32()))
        with fma_gemv(d):
            other = d.project_quantized(xt, w, out_dtype=api.DType.F32).tensor.to_f32()
        assert rel_l2(out.tensor.to_f32(), other) <= 1e-5 and not np.array_equal(bits(out.tensor.to_f32()), bits(other))
        # tiles of up to 14 rows are loaded block by block by the waves that multiply them, taller
        # ones row by row by all waves: the same arithmetic either way
        d.set_tuning("gemv_stream_own_loads", 0)
        try:
            by_rows = d.project_quantized(xt, w, out_dtype=api.DType.F32).tensor.to_f32()
        finally:
            d.set_tuning("gemv_stream_own_loads", 1)
        assert np.array_equal(bits(by_rows), bits(out.tensor.to_f32()))
    d.set_tuning("gemv_stream", 1)


def test_large_q6_k_output_matrix_streams_in_uncut_sixteen_row_tiles(api, d):
    # a million super-blocks in rows the FMA kernel cannot cut evenly over its block slots (20 per row):
    # sixteen rows of 5120 Q6_K weights are a 67 KB tile
    n, k = 52000, 5120
    base = synth.matrix(Q6_K, 2000, k, seed=97).reshape(2000, -1)
    packed = np.tile(base, (n // 2000, 1)).reshape(-1)
    w = qm(api, d, Q6_K, n, k, packed)
    for dtype, code in (("F32", oracle.F32), ("F16", oracle.F16)):
        x = oracle.round_storage(synth.activations(1, k, seed=98), code).reshape(1, k)
        xt = api.Tensor.from_f32(d, (1, k), getattr(api.DType, dtype), x)
        out = d.project_quantized(xt, w, out_dtype=api.DType.F32)
        assert out.operation == "q6_k_gemv_factored"
        got = out.tensor.to_f32()
        rows = np.unique(np.concatenate([np.arange(0, 40), np.arange(n - 40, n), synth.rng(99).integers(0, n, 120)]))
        want = oracle_columns(Q6_K, packed, n, k, rows, x, accumulate="f64")
        assert_matmul_parity(got[:, rows], want, f"streamed q6_k {n}x{k} {dtype}")
        with fma_gemv(d):
            other = d.project_quantized(xt, w, out_dtype=api.DType.F32).tensor.to_f32()
        # another kernel, another order of summation: equal to the tolerance and not to the bit
        assert rel_l2(got, other) <= 1e-5 and not np.array_equal(bits(got), bits(other))
        assert np.array_equal(bits(got[0, :2000]), bits(got[0, 2000:4000]))   # the rows repeat


@pytest.mark.parametrize("ggml", [Q4_K, Q6_K])
def test_streamed_gemv_scales_every_chunk_by_itself(api, d, ggml):
    # activations whose 64-value chunks differ by dozens of orders of magnitude, zero chunks, one
    # value per chunk: the power-of-two scale of a chunk (Q6_K: of a 16-weight group) keeps 22 bits
    # of each
    n, k = 64, 2048
    packed = synth.matrix(ggml, n, k, seed=91)
    w = qm(api, d, ggml, n, k, packed)
    d.set_tuning("gemv_stream", 2)
    x = synth.activations(1, k, seed=92).reshape(k // 64, 64)
    x *= np.float32(10.0) ** np.linspace(-30, 30, k // 64, dtype=np.float32)[:, None]
    x[3] = 0
    x[5, 1:] = 0
    x = x.reshape(1, k)
    got = d.project_quantized(api.Tensor.from_f32(d, (1, k), api.DType.F32, x), w).tensor.to_f32()
    want = oracle.project(ggml, packed, n, k, x, accumulate="f64")
    assert rel_l2(got, want) <= 1e-5
    # each chunk alone: what the huge chunks would hide
    for chunk in (0, 5, 16, 31):
        part = np.zeros_like(x).reshape(k // 64, 64)
        part[chunk] = x.reshape(k // 64, 64)[chunk]
        part = part.reshape(1, k)
        got = d.project_quantized(api.Tensor.from_f32(d, (1, k), api.DType.F32, part), w).tensor.to_f32()
        want = oracle.project(ggml, packed, n, k, part, accumulate="f64")
        assert rel_l2(got, want) <= 1e-5, chunk
    if ggml == Q6_K:
        # sixteen-value groups of one chunk that differ as much: each has a scale of its own
        part = np.zeros((k // 16, 16), np.float32)
        part[8:12] = synth.activations(1, 64, seed=93).reshape(4, 16) * np.float32(10.0) ** np.array([-20, 0, 11, 25], np.float32)[:, None]
        part = part.reshape(1, k)
        got = d.project_quantized(api.Tensor.from_f32(d, (1, k), api.DType.F32, part), w).tensor.to_f32()
        for group in range(8, 12):
            alone = np.zeros((k // 16, 16), np.float32)
            alone[group] = part.reshape(k // 16, 16)[group]
            one = d.project_quantized(api.Tensor.from_f32(d, (1, k), api.DType.F32, alone.reshape(1, k)), w).tensor.to_f32()
            assert rel_l2(one, oracle.project(ggml, packed, n, k, alone.reshape(1, k), accumulate="f64")) <= 1e-5, group
        assert rel_l2(got, oracle.project(ggml, packed, n, k, part, accumulate="f64")) <= 1e-5
    # non-finite activations reach the rows they touch
    bad = x.copy()
    bad[0, 7] = np.inf
    got = d.project_quantized(api.Tensor.from_f32(d, (1, k), api.DType.F32, bad), w).tensor.to_f32()
    assert not np.isfinite(got).any()
    d.set_tuning("gemv_stream", 1)


def test_config0_q4_k_gemv_4096(api, d):
    check_gemv(api, d, Q4_K, 4096, 4096, seed=1)


@pytest.mark.parametrize("n,k", [(5120, 5120), (17408, 5120), (5120, 17408)])
def test_config1_q4_k_decode_shapes(api, d, n, k):
    check_gemv(api, d, Q4_K, n, k, seed=2)


@pytest.mark.parametrize("n,k", [(5120, 17408), (151936, 5120)])
def test_config2_q6_k_gemv(api, d, n, k):
    check_gemv(api, d, Q6_K, n, k, seed=3)


@pytest.mark.parametrize("m", [8, 16, 128, 512])
def test_config3_q4_k_gemm_5120_17408(api, d, m):
    n, k = 17408, 5120
    packed = synth.matrix(Q4_K, n, k, seed=4)
    x = synth.activations(m, k, seed=4, f16=True)
    w = qm(api, d, Q4_K, n, k, packed)
    xt = api.Tensor.from_f32(d, (m, k), api.DType.F16, x)
    full = d.project_quantized(xt, w, out_dtype=api.DType.F32)
    got = full.tensor.to_f32()
    rows = np.sort(synth.rng(4, 77).choice(n, size=192, replace=False))
    rows[:4] = [0, 1, 2, 3]
    rows[-2:] = [n - 2, n - 1]
    rows = np.unique(rows)
    tile = oracle_columns(Q4_K, packed, n, k, rows, x, accumulate="f64", weight_round=oracle.F16,
                          threads=8)
    assert_matmul_parity(got[:, rows], tile, f"gemm M={m} vs f16-tile oracle")
    plain = oracle_columns(Q4_K, packed, n, k, rows, x, accumulate="f64", threads=8)
    # distance to the unrounded CPU reference: only the f16 tile rounding
    assert rel_l2(got[:, rows], plain) <= 4e-4
    # linearity in M: row i of the product depends only on row i of X.  The 256-row tile has two
    # forms that sum in different orders and are chosen by shape, so each is held fixed in turn.
    if m >= 16:
        xt2 = api.Tensor.from_f32(d, (m // 2, k), api.DType.F16, x[: m // 2])
        before = d.get_tuning("gemm_wide_shape")
        try:
            for shape in (0, 2):
                d.set_tuning("gemm_wide_shape", shape)
                whole = d.project_quantized(xt, w, out_dtype=api.DType.F32)
                half = d.project_quantized(xt2, w, out_dtype=api.DType.F32)
                if half.operation == whole.operation:
                    assert np.array_equal(half.tensor.to_f32(), whole.tensor.to_f32()[: m // 2])
                else:  # another kernel, another summation order
                    assert_matmul_parity(half.tensor.to_f32(), got[: m // 2], f"gemm M={m // 2} vs M={m}")
                assert_matmul_parity(whole.tensor.to_f32()[:, rows], tile, f"gemm M={m}, tile form {shape}")
        finally:
            d.set_tuning("gemm_wide_shape", before)


@pytest.mark.parametrize("m", [8, 512])
def test_config3_every_column_against_a_closed_form(api, d, m):
    # All 17408 columns, which a sample of columns cannot vouch for: row n keeps one super-block,
    # number n % 20, and zero blocks (d = dmin = 0) elsewhere, so y[:, n] is a 256-term product the
    # host evaluates for every column.
    n, k = 17408, 5120
    nb = k // 256
    blocks = synth.matrix(Q4_K, n, 256, seed=401).reshape(n, 144)
    packed = np.zeros((n, nb, 144), np.uint8)
    keep = np.arange(n) % nb
    packed[np.arange(n), keep] = blocks
    x = synth.activations(m, k, seed=402, f16=True)
    w = qm(api, d, Q4_K, n, k, packed.reshape(-1))
    out = d.project_quantized(api.Tensor.from_f32(d, (m, k), api.DType.F16, x), w, out_dtype=api.DType.F32)
    got = out.tensor.to_f32()
    dense = oracle.round_storage(oracle.dequantize(Q4_K, blocks.reshape(-1), n, 256), oracle.F16).astype(np.float64)
    want = np.empty((m, n), np.float64)
    for b in range(nb):
        rows = np.nonzero(keep == b)[0]
        want[:, rows] = x[:, 256 * b:256 * (b + 1)].astype(np.float64) @ dense[rows].T
    assert_matmul_parity(got, want, f"every column at M={m} ({out.operation})")
    worst = np.abs(got - want).max(axis=0)
    assert worst.max() <= 1e-3 * np.abs(want).max(), int(worst.argmax())


# ------------------------------------------------------------ error behaviour

def test_project_rejects_bad_geometry_and_foreign_buffers(api, d):
    packed = fx.q4k_packed(5, 512)
    w = qm(api, d, Q4_K, 5, 512, packed)
    with pytest.raises(api.ShapeError):
        d.project_quantized(api.Tensor.zeros(d, (1, 256), api.DType.F32), w)
    with pytest.raises(api.ShapeError):
        d.project_quantized(api.Tensor.zeros(d, (512,), api.DType.F32), w)
    other = api.Device.new()
    foreign = api.Tensor.zeros(other, (1, 512), api.DType.F32)
    with pytest.raises(api.DeviceMismatch):
        d.project_quantized(foreign, w)
    x = api.Tensor.zeros(d, (2, 512), api.DType.F32)
    with pytest.raises(api.RangeError):
        d.project_quantized(x.view(0, (1, 512)), w, out=x.view(0, (1, 5)))     # aliasing
    with pytest.raises(api.RangeError):
        d.project_quantized(x.view(1, (1, 512)), w)                            # misaligned view


def test_quantized_matrix_validation(api, d):
    # src/quantization.rs:93-103, :212-261 and qk_tests "reject partial blocks"
    fmt = api.QuantizationFormat.Q4_K
    with pytest.raises(api.ShapeError):
        api.QuantizedMatrix.from_reader(d, 3, 255, fmt, lambda dst: None)
    with pytest.raises(api.ShapeError):
        api.QuantizedMatrix.from_reader(d, 0, 256, fmt, lambda dst: None)
    good = fx.q4k_packed(2, 256)
    with pytest.raises(api.GgufError):
        api.QuantizedMatrix.from_bytes(d, 2, 256, fmt, good[:-1])
    with pytest.raises(api.ShapeError):
        api.QuantizedMatrix.from_bytes(d, 3, 256, fmt, good)
    bad = good.copy()
    bad[146:148] = np.frombuffer(np.float16(np.nan).tobytes(), np.uint8)
    with pytest.raises(api.WeightError):
        api.QuantizedMatrix.from_bytes(d, 2, 256, fmt, bad)
    bad6 = fx.q6k_packed(2, 256)
    bad6[208:210] = np.frombuffer(np.float16(np.inf).tobytes(), np.uint8)
    with pytest.raises(api.WeightError):
        api.QuantizedMatrix.from_bytes(d, 2, 256, api.QuantizationFormat.Q6_K, bad6)
    with pytest.raises(api.GgufError):
        api.QuantizationFormat.from_ggml_type(5)
    assert api.QuantizationFormat.from_ggml_type(12).block_bytes() == 144
    assert api.QuantizationFormat.from_ggml_type(14).block_bytes() == 210


# ------------------------------------------------------------ executions

def test_recorded_execution_replays_bitwise_with_eager_work_in_between(api, d):
    # Execution (src/metal/mod.rs:263-278): calls recorded once, replayed many times
    n, k = 1024, 2048
    w = qm(api, d, Q4_K, n, k, synth.matrix(Q4_K, n, k, seed=101))
    x = api.Tensor.from_f32(d, (1, k), api.DType.F32, synth.activations(1, k, seed=102))
    x8 = api.Tensor.from_f32(d, (8, k), api.DType.F16, synth.activations(8, k, seed=103, f16=True))
    y, y8 = api.Tensor.zeros(d, (1, n), api.DType.F32), api.Tensor.zeros(d, (8, n), api.DType.F32)
    eager = d.project_quantized(x, w).tensor.raw()
    eager8 = d.project_quantized(x8, w, out_dtype=api.DType.F32).tensor.raw()
    with d.execution() as ex:
        d.project_quantized(x, w, out=y)
        d.project_quantized(x8, w, out=y8)
        with pytest.raises(api.Error):
            api.Tensor.zeros(d, (4,), api.DType.F32)          # allocation is refused while recording
        with pytest.raises(api.Error):
            y.to_f32()                                         # so is a download
    for _ in range(3):
        ex.graph.launch()
        assert np.array_equal(y.raw(), eager) and np.array_equal(y8.raw(), eager8)
        y.buffer.upload(0, np.zeros(n, np.float32))            # eager work between the replays
        d.project_quantized(x8, w)
        d.synchronize()


def test_a_recorded_execution_survives_the_growth_of_the_scratch(api, d):
    # a recorded long-K GEMV carries the address of the device scratch (partial sums, counters);
    # an eager call that outgrows the scratch afterwards must not take that memory away
    n, k = 2048, 17408
    w = qm(api, d, Q4_K, n, k, synth.matrix(Q4_K, n, k, seed=121))
    x = api.Tensor.from_f32(d, (1, k), api.DType.F32, synth.activations(1, k, seed=122))
    y = api.Tensor.zeros(d, (1, n), api.DType.F32)
    eager = d.project_quantized(x, w)
    assert eager.operation == "q4_k_gemv_ksplit"
    with d.execution() as ex:
        d.project_quantized(x, w, out=y)
    ex.graph.launch()
    assert np.array_equal(y.raw(), eager.tensor.raw())
    # 3000 x 5120 f32 rows rounded to f16 in the scratch: 30 MB, beyond the 16 MB it starts with
    kb, nbig, mb = 5120, 256, 3000
    wb = qm(api, d, Q4_K, nbig, kb, synth.matrix(Q4_K, nbig, kb, seed=123))
    xb = api.Tensor.from_f32(d, (mb, kb), api.DType.F32, synth.activations(mb, kb, seed=124))
    d.set_tuning("gemm_f32_min_rows", 2)
    try:
        big = d.project_quantized(xb, wb)
    finally:
        d.set_tuning("gemm_f32_min_rows", 0)
    assert "mfma" in big.operation
    for _ in range(2):
        y.buffer.upload(0, np.zeros(n, np.float32))
        ex.graph.launch()
        assert np.array_equal(y.raw(), eager.tensor.raw())
        d.project_quantized(x, w)          # eager work on the new scratch in between
        d.synchronize()


def test_f32_batches_of_any_size_run_through_the_long_k_gemv(api, d):
    # q4_k_gemm accepts any M (src/metal/shaders/ops.metal:1102-1121): a long-K projection of 110 f32
    # rows needs more row-tile counters than one launch has, so the batch is cut into runs
    n, k, m = 5120, 17408, 110
    packed = synth.matrix(Q4_K, n, k, seed=131)
    w = qm(api, d, Q4_K, n, k, packed)
    x = synth.activations(m, k, seed=132)
    out = d.project_quantized(api.Tensor.from_f32(d, (m, k), api.DType.F32, x), w)
    assert out.operation == "q4_k_gemm"
    got = out.tensor.to_f32()
    first = d.project_quantized(api.Tensor.from_f32(d, (60, k), api.DType.F32, x[:60]), w).tensor.to_f32()
    last = d.project_quantized(api.Tensor.from_f32(d, (50, k), api.DType.F32, x[60:]), w).tensor.to_f32()
    assert np.array_equal(bits(got[:60]), bits(first)) and np.array_equal(bits(got[60:]), bits(last))
    rows = np.unique(synth.rng(133).integers(0, n, 48))
    picked = [0, 59, 60, 101, 102, 103, 109]
    want = oracle_columns(Q4_K, packed, n, k, rows, x[picked], accumulate="f64")
    assert_matmul_parity(got[picked][:, rows], want, "f32 batch through the K-split GEMV")


def test_wide_gemm_covers_every_column_of_its_tiles(api, d):
    # 300 rows x 36864 columns: the 256-row tile kernel with 136 columns per workgroup; the last
    # columns of a workgroup's tile (the ninth MFMA column tile) are the ones checked
    n, k, m = 36864, 512, 300
    packed = synth.matrix(Q4_K, n, k, seed=141)
    w = qm(api, d, Q4_K, n, k, packed)
    x = synth.activations(m, k, seed=142, f16=True)
    d.set_tuning("gemm_wide_shape", 0)     # the 16x16x32 form, whose tiles have the ninth column tile
    try:
        out = d.project_quantized(api.Tensor.from_f32(d, (m, k), api.DType.F16, x), w, out_dtype=api.DType.F32)
    finally:
        d.set_tuning("gemm_wide_shape", 1)
    assert out.operation == "q4_k_gemm_mfma_m256"
    got = out.tensor.to_f32()
    for width in (128, 136, 144):      # whichever width the plan chose, its tiles' last 16 columns
        rows = np.concatenate([np.arange(t * width + width - 16, t * width + width) for t in (0, 1, 100, n // width - 1)])
        rows = rows[rows < n]
        want = oracle_columns(Q4_K, packed, n, k, rows, x, accumulate="f64", weight_round=oracle.F16)
        assert_matmul_parity(got[:, rows], want, f"columns at the end of {width}-wide tiles")
    rows = np.arange(n - 40, n)
    want = oracle_columns(Q4_K, packed, n, k, rows, x, accumulate="f64", weight_round=oracle.F16)
    assert_matmul_parity(got[:, rows], want, "last columns")


@pytest.mark.parametrize("ggml", [12, 13, 14, 23, 8], ids=["q4_k", "q5_k", "q6_k", "iq4_xs", "q8_0"])
@pytest.mark.parametrize("dtype", ["F16", "BF16"])
def test_wide_gemm_on_the_32x32x16_instruction(api, d, ggml, dtype):
    # the tiles built on v_mfma_f32_32x32x16, each forced in turn: 256 rows x 160 / 128 columns and
    # 128 rows x 160 / 128 / 64 columns.  300 rows leave the last row tile 44 rows, 8072 columns
    # leave the last workgroup 72, 8 or 8 of its columns.  Every output of the first is checked
    # against the oracle; the others add the same products in the same order, so they must give
    # its bits, and so must whichever tile the library picks by itself.
    n, k, m = 8072, 512, 300
    packed = synth.matrix(ggml, n, k, seed=171)
    w = qm(api, d, ggml, n, k, packed)
    code = oracle.F16 if dtype == "F16" else oracle.BF16
    x = oracle.round_storage(synth.activations(m, k, seed=172), code).reshape(m, k)
    xt = api.Tensor.from_f32(d, (m, k), getattr(api.DType, dtype), x)
    shape, tile = d.get_tuning("gemm_wide_shape"), d.get_tuning("gemm_wide32_tile")
    results = {}
    try:
        d.set_tuning("gemm_wide_shape", 2)
        for forced in (25, 24, 15, 14, 12, 0):
            d.set_tuning("gemm_wide32_tile", forced)
            out = d.project_quantized(xt, w, out_dtype=api.DType.F32)
            assert out.operation.endswith("_gemm_mfma_m256")
            results[forced] = out.tensor.to_f32()
        d.set_tuning("gemm_wide_shape", 0)
        other = d.project_quantized(xt, w, out_dtype=api.DType.F32)
        assert other.operation.endswith("_gemm_mfma_m256")
    finally:
        d.set_tuning("gemm_wide_shape", shape)
        d.set_tuning("gemm_wide32_tile", tile)
    want = oracle.project(ggml, packed, n, k, x, accumulate="f64", weight_round=code, threads=8)
    assert_matmul_parity(results[25], want, "every output of the 256 x 160 tiles")
    for forced, got in results.items():
        assert np.array_equal(bits(got), bits(results[25])), f"tile {forced} against 256 x 160"
    assert_matmul_parity(results[25], other.tensor.to_f32(), "against the 16x16x32 tiles", l2_tol=2e-6)


@pytest.mark.parametrize("m", [80, 128, 200, 330, 512])
def test_the_tile_picked_by_row_count_gives_the_bits_of_the_largest(api, d, m):
    # 17000 columns at every row count that changes the tile (128 x 68 of the 96-column tile up to
    # 128 rows, 128 x 160 up to 256, 128 x 128 up to 384, 256 x 160 beyond); the pick and the forced
    # 128 x 64 and 128 x 96 tiles against the forced 256 x 160 tile.
    n, k = 17000, 2816
    w = qm(api, d, Q4_K, n, k, synth.matrix(Q4_K, n, k, seed=173))
    x = synth.activations(m, k, seed=174, f16=True)
    xt = api.Tensor.from_f32(d, (m, k), api.DType.F16, x)
    tile, resident, shape = d.get_tuning("gemm_wide32_tile"), d.get_tuning("gemm_resident"), d.get_tuning("gemm_wide_shape")
    try:
        d.set_tuning("gemm_resident", 0)      # at 80 rows its estimate is close to the tile's,
        d.set_tuning("gemm_wide_shape", 2)    # at 512 the 16x16x32 form's, whose bits differ
        picked = d.project_quantized(xt, w, out_dtype=api.DType.F32)
        d.set_tuning("gemm_wide32_tile", 25)
        largest = d.project_quantized(xt, w, out_dtype=api.DType.F32)
        for forced in (12, 13):
            d.set_tuning("gemm_wide32_tile", forced)
            assert np.array_equal(d.project_quantized(xt, w, out_dtype=api.DType.F32).tensor.raw(), largest.tensor.raw())
    finally:
        d.set_tuning("gemm_wide32_tile", tile)
        d.set_tuning("gemm_resident", resident)
        d.set_tuning("gemm_wide_shape", shape)
    assert picked.operation == largest.operation == "q4_k_gemm_mfma_m256"
    assert np.array_equal(picked.tensor.raw(), largest.tensor.raw())


@pytest.mark.parametrize("ggml", [12, 13, 14, 23, 8], ids=["q4_k", "q5_k", "q6_k", "iq4_xs", "q8_0"])
@pytest.mark.parametrize("m,n,k,dtype", [(2, 17000, 5120, "F16"), (9, 4100, 5120, "BF16"), (16, 17000, 4096, "F16"),
                                         (8, 1000, 2048, "F16"), (16, 20000, 768, "BF16")])
def test_few_rows_deal_a_tiles_super_blocks_over_the_waves(api, d, ggml, m, n, k, dtype):
    # up to 16 rows and at most five 16-row weight tiles per compute unit: every wave of the
    # workgroup takes some super-blocks of every tile and the partial sums meet in LDS.  Rows of 1 -
    # 20 super-blocks (8 and 16 waves), one to five tiles per workgroup, a ragged last tile, every
    # format; against the tile-rounded oracle on sampled columns and against the kernel that
    # gives a wave whole tiles (the same products, added in another order).
    packed = synth.matrix(ggml, n, k, seed=181 + m)
    w = qm(api, d, ggml, n, k, packed)
    code = oracle.F16 if dtype == "F16" else oracle.BF16
    x = oracle.round_storage(synth.activations(m, k, seed=182), code).reshape(m, k)
    xt = api.Tensor.from_f32(d, (m, k), getattr(api.DType, dtype), x)
    out = d.project_quantized(xt, w, out_dtype=api.DType.F32)
    assert out.operation.endswith("_gemm_mfma_resident")
    d.set_tuning("gemm_few_tiles_split", 0)
    try:
        whole = d.project_quantized(xt, w, out_dtype=api.DType.F32)
    finally:
        d.set_tuning("gemm_few_tiles_split", 1)
    assert whole.operation == out.operation
    got = out.tensor.to_f32()
    rows = np.unique(np.concatenate([np.arange(0, 40), np.arange(n - 40, n), synth.rng(183).integers(0, n, 80)]))
    want = oracle_columns(ggml, packed, n, k, rows, x, weight_round=code, accumulate="f64")
    assert_matmul_parity(got[:, rows], want, "dealt super-blocks against the tile-rounded oracle")
    assert_matmul_parity(got, whole.tensor.to_f32(), "against whole tiles per wave", l2_tol=2e-6)
    assert not np.array_equal(got, np.zeros_like(got))
    half = d.project_quantized(xt, w, out_dtype=getattr(api.DType, dtype))      # 16-bit output: the scalar stores
    assert np.array_equal(half.tensor.to_f32(), oracle.round_storage(got, code).reshape(m, n))


@pytest.mark.parametrize("ggml,m,dtype", [(12, 130, "F16"), (12, 300, "BF16"), (14, 200, "F16"), (8, 130, "F16")],
                         ids=["q4_k-130", "q4_k-300-bf16", "q6_k-200", "q8_0-130"])
def test_rows_too_long_for_lds_take_the_128_row_tiles(api, d, ggml, m, dtype):
    # K = 17408 (the 27B model's down projection): no 16 rows of it fit LDS, so from 65 rows on the
    # choice is between the tiles only.  5120 columns are too few for 256-row tiles to fill the chip
    # and enough for 128 x 64 ones (160 or 240 workgroups), the default; the square tiles
    # (tuning gemm_wide_shape 0) give the reference bits of the same products in another order.
    n, k = 5120, 17408
    packed = synth.matrix(ggml, n, k, seed=191)
    w = qm(api, d, ggml, n, k, packed)
    code = oracle.F16 if dtype == "F16" else oracle.BF16
    x = oracle.round_storage(synth.activations(m, k, seed=192), code).reshape(m, k)
    xt = api.Tensor.from_f32(d, (m, k), getattr(api.DType, dtype), x)
    out = d.project_quantized(xt, w, out_dtype=api.DType.F32)
    d.set_tuning("gemm_wide_shape", 0)
    try:
        square = d.project_quantized(xt, w, out_dtype=api.DType.F32)
    finally:
        d.set_tuning("gemm_wide_shape", 1)
    assert out.operation.endswith("_gemm_mfma_m256") == (m > 128) and square.operation.endswith("_gemm_mfma")
    got = out.tensor.to_f32()
    rows = np.unique(np.concatenate([np.arange(0, 70), np.arange(n - 70, n), synth.rng(193).integers(0, n, 60)]))
    want = oracle_columns(ggml, packed, n, k, rows, x, weight_round=code, accumulate="f64")
    assert_matmul_parity(got[:, rows], want, "rows of 17408 on the tiles")
    assert_matmul_parity(got, square.tensor.to_f32(), "against the square tiles", l2_tol=2e-6)


def test_objects_may_outlive_their_device(api):
    # buffers, matrices and recorded executions hold the device object: releasing them after
    # fh_device_destroy (any order a garbage collector may pick) is safe
    import gc
    dev = api.Device.new()
    n, k = 64, 512
    w = qm(api, dev, Q4_K, n, k, synth.matrix(Q4_K, n, k, seed=151))
    x = api.Tensor.from_f32(dev, (1, k), api.DType.F32, synth.activations(1, k, seed=152))
    y = api.Tensor.zeros(dev, (1, n), api.DType.F32)
    with dev.execution() as ex:
        dev.project_quantized(x, w, out=y)
    ex.graph.launch()
    want = y.to_f32().copy()
    handle, dev._handle = dev._handle, None
    api._lib.fh_device_destroy(handle)
    with pytest.raises(api.Error):
        y.to_f32()                                  # the device is gone: a clear error, not a crash
    with pytest.raises(api.Error):
        ex.graph.launch()
    del ex, w, x, y
    gc.collect()
    assert np.abs(want).max() > 0


def test_releases_asked_for_while_recording_wait_for_its_end(api, d):
    import gc
    n, k = 512, 1024
    packed = synth.matrix(Q4_K, n, k, seed=111)
    w = qm(api, d, Q4_K, n, k, packed)
    x = api.Tensor.from_f32(d, (1, k), api.DType.F32, synth.activations(1, k, seed=112))
    y = api.Tensor.zeros(d, (1, n), api.DType.F32)
    want = d.project_quantized(x, w).tensor.raw()
    with d.execution() as old:
        d.project_quantized(x, w, out=y)
    old.graph.launch()
    spare_w = qm(api, d, Q4_K, n, k, packed)
    spare_t = api.Tensor.zeros(d, (64, 64), api.DType.F32)
    with d.execution() as ex:
        d.project_quantized(x, w, out=y)
        # dropping a graph, a matrix and a tensor here must not disturb the recording
        del old, spare_w, spare_t
        gc.collect()
        d.project_quantized(x, w, out=y)
    y.buffer.upload(0, np.zeros(n, np.float32))
    ex.graph.launch()
    assert np.array_equal(y.raw(), want)
    assert np.array_equal(d.project_quantized(x, w).tensor.raw(), want)


# ------------------------------------------------------------- greedy selection

@pytest.mark.parametrize("dtype_name", ["F32", "F16", "BF16"])
def test_argmax_rows_matches_the_oracle(api, d, dtype_name):
    dtype = api.DType[dtype_name]
    code = {"F32": oracle.F32, "F16": oracle.F16, "BF16": oracle.BF16}[dtype_name]
    rng = synth.rng(131)
    for rows, width in ((1, 1), (3, 33), (4, 1024), (5, 4099), (2, 151936)):
        x = oracle.round_storage(rng.standard_normal((rows, width)).astype(np.float32), code).reshape(rows, width)
        if width > 40:
            x[0, 5] = x[0, width - 3] = 9.0
            if rows > 2:
                x[1, 9] = np.inf
                x[2, 0] = np.nan
            if rows > 3:
                x[3, 2047 % width] = np.nan
        got = d.argmax_rows(api.Tensor.from_f32(d, x.shape, dtype, x))
        assert d.last_operation() == "argmax_rows"
        want = oracle.argmax_rows(x)
        assert np.array_equal(got.raw().view(np.uint32).reshape(rows, 2), want), (rows, width)
    with pytest.raises(api.ShapeError):
        d.argmax_rows(api.Tensor.zeros(d, (4,), dtype))


def test_lm_head_projection_then_argmax_picks_the_oracle_token(api, d):
    n, k = 4096, 1024
    packed = synth.matrix(Q6_K, n, k, seed=141)
    w = qm(api, d, Q6_K, n, k, packed)
    x = synth.activations(1, k, seed=142)
    logits = d.project_quantized(api.Tensor.from_f32(d, x.shape, api.DType.F32, x), w).tensor
    picked = d.argmax_rows(logits).raw().view(np.uint32)
    want = oracle.project(Q6_K, packed, n, k, x, accumulate="f64")
    assert picked[1] == 0 and picked[0] == int(np.argmax(logits.to_f32()))
    top2 = np.sort(want[0])[-2:]
    if top2[1] - top2[0] > 1e-3 * abs(top2[1]):      # unambiguous in the oracle too
        assert picked[0] == int(np.argmax(want))


# ----------------------------------------------------------------------- Q5_K

Q5_K = 13


def test_q5_k_dequantize_and_gather_are_bit_exact(api, d):
    for rows, cols, packed in ((5, 512, fx.q5k_packed(5, 512)), (133, 2560, fx.q5k_packed(133, 2560)),
                               (257, 1024, synth.matrix(Q5_K, 257, 1024, seed=181))):
        w = qm(api, d, Q5_K, rows, cols, packed)
        assert w.byte_size() == rows * (cols // 256) * 176
        want = oracle.dequantize(Q5_K, packed, rows, cols)
        assert np.array_equal(bits(d.dequantize(w).to_f32()), bits(want))
        assert np.array_equal(bits(d.dequantize(w, api.DType.BF16).to_f32()),
                              bits(oracle.round_storage(want, oracle.BF16).reshape(rows, cols)))
        ids = [rows - 1, 0, 3]
        got = d.embedding_gather_quantized(w, ids, api.DType.F32)
        assert got.operation == "embedding_gather_q5_k"
        assert np.array_equal(bits(got.tensor.to_f32()), bits(want[ids]))


def test_q5_k_gemv_and_small_batches_replay_the_reference_cases(api, d):
    # q4_k_and_q5_k_gemv_gemm_cover_blocks_and_batch_tails (src/ops/transformer.rs:2982-3002):
    # (N, K) = (5, 512), M in 1..7 except 6, f32, abs <= 2e-4 against the f32-sequential sum
    n, k = 5, 512
    packed = fx.q5k_packed(n, k)
    w = qm(api, d, Q5_K, n, k, packed)
    for m in (1, 2, 3, 4, 5, 7):
        x = fx.q4k_input(m, k)
        out = d.project_quantized(api.Tensor.from_f32(d, x.shape, api.DType.F32, x), w)
        assert out.operation == ("q5_k_gemv_factored" if m == 1 else "q5_k_gemm")
        want = oracle.project(Q5_K, packed, n, k, x, accumulate="f32")
        assert np.abs(out.tensor.to_f32() - want).max() <= 2e-4, m


@pytest.mark.parametrize("n,k,m,dtype_name", [(4099, 5120, 1, "F32"), (1003, 4864, 1, "F32"), (5120, 17408, 1, "F32"),
                                              (515, 1280, 3, "F32"), (515, 1280, 1, "F16"), (515, 1280, 4, "BF16")])
def test_q5_k_projection_matches_the_f64_oracle(api, d, n, k, m, dtype_name):
    dtype = api.DType[dtype_name]
    code = {"F32": oracle.F32, "F16": oracle.F16, "BF16": oracle.BF16}[dtype_name]
    packed = synth.matrix(Q5_K, n, k, seed=n + k)
    w = qm(api, d, Q5_K, n, k, packed)
    x = oracle.round_storage(synth.activations(m, k, seed=11), code).reshape(m, k)
    out = d.project_quantized(api.Tensor.from_f32(d, x.shape, dtype, x), w, out_dtype=api.DType.F32)
    rows = np.unique(np.concatenate([np.arange(0, 40), np.arange(n - 40, n), synth.rng(12).integers(0, n, 64)]))
    tiles = m > 1 and dtype_name != "F32"            # 16-bit batches take the tile kernels: weights rounded once
    want = oracle_columns(Q5_K, packed, n, k, rows, x, accumulate="f64", **({"weight_round": code} if tiles else {}))
    assert_matmul_parity(out.tensor.to_f32()[:, rows], want, f"q5_k {n}x{k} m={m} {dtype_name}")
    if k == 17408:
        assert out.operation == "q5_k_gemv_ksplit"


@pytest.mark.parametrize("m,n,dtype_name", [(8, 1100, "F16"), (20, 1100, "BF16"), (130, 1000, "F16"),
                                            (130, 16000, "BF16"), (300, 33000, "F16")])
def test_q5_k_tile_kernels_match_the_rounded_weight_oracle(api, d, m, n, dtype_name):
    # skinny (M <= 32), 64- and 128-wide tiles, and the 256-row tile (33000 columns x 2 row tiles)
    k = 512
    dtype = api.DType[dtype_name]
    code = oracle.F16 if dtype_name == "F16" else oracle.BF16
    packed = synth.matrix(Q5_K, n, k, seed=201 + n)
    w = qm(api, d, Q5_K, n, k, packed)
    x = oracle.round_storage(synth.activations(m, k, seed=202), code).reshape(m, k)
    d.set_tuning("gemm_resident", 0)       # the square tiles, which rows longer than LDS still take
    d.set_tuning("gemm_wide_shape", 0)     # where too few 256-row tiles would fill the chip (128-row ones do)
    try:
        out = d.project_quantized(api.Tensor.from_f32(d, x.shape, dtype, x), w, out_dtype=api.DType.F32)
    finally:
        d.set_tuning("gemm_resident", 1)
        d.set_tuning("gemm_wide_shape", 1)
    want_name = {8: "q5_k_gemm_mfma_skinny", 20: "q5_k_gemm_mfma_skinny", 130: "q5_k_gemm_mfma",
                 300: "q5_k_gemm_mfma_m256"}[m]
    assert out.operation == want_name
    rows = np.unique(np.concatenate([np.arange(0, 140), np.arange(n - 80, n), synth.rng(203).integers(0, n, 64)]))
    want = oracle_columns(Q5_K, packed, n, k, rows, x, weight_round=code, accumulate="f64")
    assert_matmul_parity(out.tensor.to_f32()[:, rows], want, f"q5_k tile m={m} n={n}")
    # the bf16 reference case: result stored in the activation dtype
    if m == 20:
        stored = d.project_quantized(api.Tensor.from_f32(d, x.shape, dtype, x), w).tensor.to_f32()
        assert np.array_equal(bits(stored), bits(oracle.round_storage(out.tensor.to_f32(), code).reshape(m, n)))


def test_q5_k_expert_projection_and_validation(api, d):
    experts, rows, cols, a = 4, 40, 768, 9
    packed = synth.matrix(Q5_K, experts * rows, cols, seed=191)
    w = api.QuantizedExpertMatrix.new(d, packed, api.QuantizationFormat(Q5_K), experts, rows, cols)
    meta = np.zeros((a, 3), dtype=np.uint32)
    meta[:, 0] = [0, 3, 1, 1, 2, 7, 0, 3, 2]          # 7 does not exist: a zero row
    meta[:, 1] = np.arange(a)
    meta[:, 2] = np.float32(1.0).view(np.uint32)
    x = synth.activations(a, cols, seed=192)
    got = d.expert_project_quantized(api.Tensor.from_f32(d, x.shape, api.DType.F32, x),
                                     api.Tensor.from_bits(d, meta.shape, meta), w, cols, experts)
    assert d.last_operation() == "expert_project_q5_k_factored"
    got = got.to_f32()
    safe = meta.copy(); safe[5, 0] = 0
    want = oracle.expert_project(Q5_K, packed, experts, rows, cols, x, safe.view(np.float32), accumulate="f64")
    valid = np.arange(a) != 5
    assert np.all(got[5] == 0)
    assert_matmul_parity(got[valid], want[valid], "q5_k expert projection")
    bad = packed.copy()
    bad[1] = 0x7c                                       # d = +inf in the first block
    with pytest.raises(api.WeightError):
        api.QuantizedMatrix.from_bytes(d, experts * rows, cols, api.QuantizationFormat(Q5_K), bad)
    with pytest.raises(api.Error):
        api.QuantizedMatrix.from_bytes(d, experts * rows, cols, api.QuantizationFormat(Q5_K), packed[:-1])


IQ4_XS, Q8_0 = 23, 8


# Rows that fit LDS for their whole length (K <= 2560 for groups of 32 rows, K <= 5120 for groups
# of 16), two rows or more: the kernel that keeps a group of rows resident and streams the
# weights past them.  Ragged row groups, ragged row tiles, more pieces than compute units, both
# group sizes, every format, both 16-bit dtypes.
@pytest.mark.parametrize("ggml,m,n,k,dtype_name", [
    (Q4_K, 70, 1000, 768, "F16"), (Q4_K, 200, 50, 4096, "BF16"), (Q4_K, 2000, 1000, 256, "F16"),
    (Q4_K, 40, 300, 5120, "F16"), (Q4_K, 2, 1000, 768, "F16"), (Q4_K, 16, 100, 4096, "BF16"), (Q6_K, 17, 530, 1024, "F16"), (Q5_K, 64, 1000, 512, "F16"),
    (Q5_K, 130, 1000, 512, "BF16"), (Q6_K, 97, 530, 1024, "F16"), (Q6_K, 65, 40, 2560, "F16"),
    (IQ4_XS, 300, 300, 512, "F16"), (Q8_0, 129, 260, 1280, "BF16")])
def test_rows_resident_gemm_matches_the_rounded_weight_oracle(api, d, ggml, m, n, k, dtype_name):
    dtype = api.DType[dtype_name]
    code = oracle.F16 if dtype_name == "F16" else oracle.BF16
    packed = synth.matrix(ggml, n, k, seed=301 + n + m)
    w = qm(api, d, ggml, n, k, packed)
    x = oracle.round_storage(synth.activations(m, k, seed=302 + m), code).reshape(m, k)
    xt = api.Tensor.from_f32(d, x.shape, dtype, x)
    out = d.project_quantized(xt, w, out_dtype=api.DType.F32)
    assert out.operation.endswith("_gemm_mfma_resident")
    rows = np.unique(np.concatenate([np.arange(0, min(n, 48)), np.arange(max(0, n - 40), n),
                                     synth.rng(303).integers(0, n, 32)]))
    want = oracle_columns(ggml, packed, n, k, rows, x, weight_round=code, accumulate="f64")
    got = out.tensor.to_f32()
    assert_matmul_parity(got[:, rows], want, f"rows-resident m={m} n={n} k={k}")
    # stored in the activation dtype (packed stores where rows allow, element stores on ragged ones)
    stored = d.project_quantized(xt, w)
    assert stored.operation == out.operation
    assert np.array_equal(bits(stored.tensor.to_f32()), bits(oracle.round_storage(got, code).reshape(m, n)))
    # every row group and tile was written: the square tiles give the same product
    d.set_tuning("gemm_resident", 0)
    try:
        tiles = d.project_quantized(xt, w, out_dtype=api.DType.F32)
    finally:
        d.set_tuning("gemm_resident", 1)
    assert not tiles.operation.endswith("_resident")
    assert rel_l2(got, tiles.tensor.to_f32()) <= 1e-5
