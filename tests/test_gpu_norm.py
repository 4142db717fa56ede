"""GPU parity of the residual add fused with RMSNorm, through the C ABI.

The cases are the reference's own (fused_add_rmsnorm_matches_separate_kernels_bitwise,
src/ops/transformer.rs:1345-1393: three dtypes, rows x width in {1x896, 37x2048, 5x64,
3x1000}, inputs from reference::deterministic) plus decode- and prefill-sized rows.  The
residual is bit-exact (a storage-rounded f32 sum); the normalised rows are held to the CPU
reference's float64 evaluation: 2e-6 relative for f32 (the reference's smoke test allows
2e-4, src/main.rs:62), one unit in the last place of the storage type for f16 / bf16.
"""
import numpy as np
import pytest

import ferrum_fixtures as fx
import oracle
from helpers import bits

pytestmark = pytest.mark.gpu

EPS = 1e-6


@pytest.fixture(scope="module")
def api():
    from ferrum_amd import api as module
    return module


@pytest.fixture(scope="module")
def d(api):
    return api.Device.new()


def operands(api, d, rows, width, dtype_name):
    dtype = api.DType[dtype_name]
    n = rows * width
    a = api.Tensor.from_f32(d, (rows, width), dtype, fx.deterministic(n))
    b = api.Tensor.from_f32(d, (rows, width), dtype, fx.deterministic(n + 11)[11:])
    w = api.Tensor.from_f32(d, (width,), dtype, 1.0 + fx.deterministic(width + 3)[3:])
    return a, b, w


def check(api, a, b, w, residual, normed, dtype_name):
    code = {"F32": oracle.F32, "F16": oracle.F16, "BF16": oracle.BF16}[dtype_name]
    want_residual, want_normed = oracle.add_rmsnorm(a.to_f32(), b.to_f32(), w.to_f32(), EPS, code)
    assert np.array_equal(bits(residual.to_f32()), bits(want_residual))
    got = normed.to_f32()
    if dtype_name == "F32":
        assert np.abs(got - want_normed).max() <= 2e-6 * np.abs(want_normed).max()
        assert np.allclose(got, want_normed, rtol=2e-6, atol=1e-7)
    else:
        # one rounding of a value that is itself a few f32 ulps from the float64 one:
        # equal to the rounded float64 value or its neighbour in the storage type
        rounded = oracle.round_storage(want_normed, code).reshape(got.shape)
        ulp = np.abs(rounded) * (2.0 ** -10 if dtype_name == "F16" else 2.0 ** -7)
        assert np.all(np.abs(got - rounded) <= ulp + 1e-7)
        assert (got != rounded).mean() < 0.01


@pytest.mark.parametrize("dtype_name", ["F32", "F16", "BF16"])
@pytest.mark.parametrize("rows,width", [(1, 896), (37, 2048), (5, 64), (3, 1000), (1, 5120), (512, 5120),
                                        (3, 8192), (2, 8196), (2, 16384), (2, 1001), (1, 17408)])
def test_add_rmsnorm_matches_the_cpu_reference(api, d, rows, width, dtype_name):
    a, b, w = operands(api, d, rows, width, dtype_name)
    residual, normed = d.add_rmsnorm(a, b, w, EPS)
    assert d.last_operation() == "add_rmsnorm"
    assert residual.shape() == (rows, width) and normed.dtype == a.dtype
    check(api, a, b, w, residual, normed, dtype_name)


def test_add_rmsnorm_reuses_output_buffers_and_rejects_bad_operands(api, d):
    a, b, w = operands(api, d, 4, 512, "F32")
    residual = api.Tensor.zeros(d, (4, 512), api.DType.F32)
    normed = api.Tensor.zeros(d, (4, 512), api.DType.F32)
    r2, n2 = d.add_rmsnorm(a, b, w, EPS, residual=residual, normed=normed)
    assert r2 is residual and n2 is normed
    check(api, a, b, w, residual, normed, "F32")
    with pytest.raises(api.RangeError):
        d.add_rmsnorm(a, b, w, EPS, residual=a, normed=normed)       # outputs may not alias operands
    with pytest.raises(api.RangeError):
        d.add_rmsnorm(a, b, w, EPS, residual=residual, normed=residual)
    with pytest.raises(api.ParameterError):
        d.add_rmsnorm(a, b, w, 0.0)
    with pytest.raises(api.ParameterError):
        d.add_rmsnorm(a, b, w, float("nan"))
    with pytest.raises(api.ShapeError):
        d.add_rmsnorm(a, b, api.Tensor.zeros(d, (511,), api.DType.F32), EPS)
    with pytest.raises(api.ShapeError):
        d.add_rmsnorm(a, api.Tensor.zeros(d, (4, 512), api.DType.F16), w, EPS)
    with pytest.raises(api.ShapeError):
        d.add_rmsnorm(a, api.Tensor.zeros(d, (2, 1024), api.DType.F32), w, EPS)
    other = api.Device.new()
    with pytest.raises(api.DeviceMismatch):
        d.add_rmsnorm(a, b, api.Tensor.zeros(other, (512,), api.DType.F32), EPS)


def test_norm_feeds_the_projection(api, d):
    # the decode chain of a layer: residual add + norm, then the quantised projection of the
    # normalised row; against the oracle's chain on the same inputs
    from ferrum_amd import synth
    n, k = 1100, 5120
    a, b, w = operands(api, d, 1, k, "F32")
    packed = synth.matrix(12, n, k, seed=141)
    weight = api.QuantizedMatrix.from_bytes(d, n, k, api.QuantizationFormat(12), packed)
    _, normed = d.add_rmsnorm(a, b, w, EPS)
    out = d.project_quantized(normed, weight).tensor.to_f32()
    _, want_normed = oracle.add_rmsnorm(a.to_f32(), b.to_f32(), w.to_f32(), EPS)
    want = oracle.project(12, packed, n, k, want_normed, accumulate="f64")
    assert np.linalg.norm(out - want) <= 1e-5 * np.linalg.norm(want)
