"""The entry point that allocates nothing, through the C ABI: fh_project_quantized_no_alloc
against fh_project_quantized on long rows (K segments: partial sums and counters in the
library's fixed scratch), two calls in a row, the second one smaller."""
import numpy as np
import pytest

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


def run_pair(api, d, ggml, n, k, m, dtype, seed):
    packed = synth.matrix(ggml, n, k, seed)
    w = api.QuantizedMatrix.from_bytes(d, n, k, api.QuantizationFormat(ggml), packed)
    x = api.Tensor.from_f32(d, (m, k), dtype, synth.activations(m, k, seed + 1))
    want = d.project_quantized(x, w, out_dtype=api.DType.F32)
    out = api.Tensor.from_f32(d, (m, n), api.DType.F32, np.full((m, n), np.nan, np.float32))
    got = d.project_quantized_no_alloc(x, w, out)
    return got, want


def test_no_alloc_projection_matches_the_allocating_one_on_two_calls_in_a_row(api, d):
    f32 = api.DType.F32
    # 68 super-blocks per row: three K segments, partial sums and counters in the fixed scratch
    got, want = run_pair(api, d, Q4_K, 5120, 17408, 1, f32, seed=501)
    assert got.operation == want.operation == "q4_k_gemv_ksplit"
    assert np.array_equal(got.tensor.raw(), want.tensor.raw())
    assert np.abs(want.tensor.to_f32()).max() > 1e-3
    # the second call is smaller and finds the scratch as the first left it
    got, want = run_pair(api, d, Q6_K, 700, 17408, 2, f32, seed=503)
    assert got.operation == "q6_k_gemv_ksplit"
    assert np.array_equal(got.tensor.raw(), want.tensor.raw())
    got, want = run_pair(api, d, Q4_K, 300, 1024, 1, api.DType.F16, seed=505)   # short rows: no scratch at all
    assert np.array_equal(got.tensor.raw(), want.tensor.raw())


def test_no_alloc_projection_rejects_what_the_fixed_scratch_cannot_hold(api, d):
    n, k, m = 5120, 17408, 20   # 3 segments x 20 rows x 5120 floats = 1.2 MB of partial sums
    w = api.QuantizedMatrix.from_bytes(d, n, k, api.QuantizationFormat(Q4_K), synth.matrix(Q4_K, n, k, seed=507))
    x = api.Tensor.from_f32(d, (m, k), api.DType.F32, synth.activations(m, k, seed=508))
    out = api.Tensor.zeros(d, (m, n), api.DType.F32)
    with pytest.raises(api.ShapeError, match="fixed scratch"):
        d.project_quantized_no_alloc(x, w, out)
    assert not out.to_f32().any()
    # and the next call still works
    got, want = run_pair(api, d, Q4_K, 1024, 17408, 1, api.DType.F32, seed=509)
    assert np.array_equal(got.tensor.raw(), want.tensor.raw())
