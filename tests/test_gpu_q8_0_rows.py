"""Q8_0 matrices whose rows are 32 n weights long with n not a multiple of 8 (the reference's
geometry is the 34-byte block of 32, src/loader/gguf.rs:99; a row is `cols / 32 * 34` bytes,
src/hybrid/weights.rs:1167), through every entry point that takes a matrix.

Two anchors per case: the CPU oracle at the matrix's own geometry, and the same entry point on
the matrix with every row completed to a run of eight blocks by empty ones and the activations
zero-filled to that width, whose result must be the same bits (the added terms are exact zeros).
"""
import numpy as np
import pytest

import oracle
from helpers import assert_matmul_parity, bits, oracle_columns, rel_l2
from ferrum_amd import synth

pytestmark = pytest.mark.gpu

Q8_0 = 8


@pytest.fixture(scope="module")
def api():
    from ferrum_amd import api as module
    return module


@pytest.fixture(scope="module")
def d(api):
    return api.Device.new()


def stored_width(cols):
    return (cols + 255) // 256 * 256


def completed(packed, rows, cols):
    """The payload with every row completed to a run of eight blocks by empty blocks."""
    width = stored_width(cols)
    out = np.zeros((rows, width // 32 * 34), dtype=np.uint8)
    out[:, : cols // 32 * 34] = packed.reshape(rows, cols // 32 * 34)
    return out.reshape(-1)


def widened(x, cols, parts=1):
    """[rows, parts * cols] -> [rows, parts * stored width], zeros in the added columns."""
    rows = x.shape[0]
    out = np.zeros((rows, parts, stored_width(cols)), dtype=np.float32)
    out[:, :, :cols] = x.reshape(rows, parts, cols)
    return out.reshape(rows, -1)


def both(api, d, rows, cols, seed, experts=1):
    packed = synth.matrix(Q8_0, experts * rows, cols, seed=seed)
    fmt = api.QuantizationFormat.Q8_0
    if experts == 1:
        own = api.QuantizedMatrix.from_bytes(d, rows, cols, fmt, packed)
        wide = api.QuantizedMatrix.from_bytes(d, rows, stored_width(cols), fmt, completed(packed, rows, cols))
    else:
        own = api.QuantizedExpertMatrix.new(d, packed, fmt, experts, rows, cols)
        wide = api.QuantizedExpertMatrix.new(d, completed(packed, experts * rows, cols), fmt, experts, rows,
                                             stored_width(cols))
    return packed, own, wide


def tensor(api, d, values, dtype):
    return api.Tensor.from_f32(d, values.shape, dtype, values)


CODE = {"F32": 0, "F16": 1, "BF16": 2}


@pytest.mark.parametrize("rows,cols", [(13, 32), (5, 288), (257, 2880), (3, 224)])
def test_dequantize_and_gather_are_bit_exact(api, d, rows, cols):
    packed = synth.matrix(Q8_0, rows, cols, seed=401 + cols)
    assert packed.size == rows * (cols // 32) * 34
    w = api.QuantizedMatrix.from_bytes(d, rows, cols, api.QuantizationFormat.Q8_0, packed)
    assert (w.rows(), w.columns(), w.byte_size()) == (rows, cols, packed.size)
    want = oracle.dequantize(Q8_0, packed, rows, cols)
    assert want.shape == (rows, cols)
    assert np.array_equal(bits(d.dequantize(w).to_f32()), bits(want))
    for dtype, code in ((api.DType.F16, oracle.F16), (api.DType.BF16, oracle.BF16)):
        assert np.array_equal(bits(d.dequantize(w, dtype).to_f32()),
                              bits(oracle.round_storage(want, code).reshape(rows, cols)))
    ids = [rows - 1, 0, 2, 2]
    got = d.embedding_gather_quantized(w, ids, api.DType.F32)
    assert got.operation == "embedding_gather_q8_0"
    assert np.array_equal(bits(got.tensor.to_f32()), bits(want[ids]))


@pytest.mark.parametrize("n,k,m,dtype_name", [(1003, 2880, 1, "F32"), (515, 288, 1, "F32"), (64, 32, 1, "F32"),
                                              (5120, 17440, 1, "F32"), (515, 2880, 3, "F32"), (515, 2880, 1, "F16"),
                                              (515, 2912, 1, "BF16")])
def test_few_rows_match_the_f64_oracle_and_the_completed_matrix(api, d, n, k, m, dtype_name):
    dtype = api.DType[dtype_name]
    packed, own, wide = both(api, d, n, k, seed=n + k)
    x = oracle.round_storage(synth.activations(m, k, seed=411), CODE[dtype_name]).reshape(m, k)
    out = d.project_quantized(tensor(api, d, x, dtype), own, out_dtype=api.DType.F32)
    assert out.operation.startswith("q8_0_gem")
    rows = np.unique(np.concatenate([np.arange(0, min(n, 40)), np.arange(max(n - 40, 0), n)]))
    want = oracle_columns(Q8_0, packed, n, k, rows, x, accumulate="f64")
    assert_matmul_parity(out.tensor.to_f32()[:, rows], want, f"q8_0 {n}x{k} m={m} {dtype_name}")
    same = d.project_quantized(tensor(api, d, widened(x, k), dtype), wide, out_dtype=api.DType.F32)
    assert same.operation == out.operation
    assert np.array_equal(bits(out.tensor.to_f32()), bits(same.tensor.to_f32()))


@pytest.mark.parametrize("m,n,dtype_name", [(8, 1100, "F16"), (50, 1100, "BF16"), (130, 1000, "F16"), (300, 3000, "F16")])
def test_tile_kernels_match_the_rounded_weight_oracle_and_the_completed_matrix(api, d, m, n, dtype_name):
    k = 800                                    # 25 blocks: three runs and one block
    dtype = api.DType[dtype_name]
    code = CODE[dtype_name]
    packed, own, wide = both(api, d, n, k, seed=421 + n)
    x = oracle.round_storage(synth.activations(m, k, seed=422), code).reshape(m, k)
    out = d.project_quantized(tensor(api, d, x, dtype), own, out_dtype=api.DType.F32)
    assert out.operation.startswith("q8_0_gemm_mfma")
    rows = np.unique(np.concatenate([np.arange(0, 150), np.arange(n - 150, n)]))
    want = oracle_columns(Q8_0, packed, n, k, rows, x, weight_round=code, accumulate="f64")
    assert_matmul_parity(out.tensor.to_f32()[:, rows], want, f"q8_0 tile m={m} n={n}")
    same = d.project_quantized(tensor(api, d, widened(x, k), dtype), wide, out_dtype=api.DType.F32)
    assert same.operation == out.operation
    assert np.array_equal(bits(out.tensor.to_f32()), bits(same.tensor.to_f32()))


def test_tile_values_are_the_dequantised_weights_rounded_once(api, d):
    n, k = 200, 288
    packed, own, _ = both(api, d, n, k, seed=431)
    dense = oracle.dequantize(Q8_0, packed, n, k)
    eye = np.eye(k, dtype=np.float32)
    for dtype, code in ((api.DType.F16, oracle.F16), (api.DType.BF16, oracle.BF16)):
        for m0, m1 in ((0, 40), (40, 288)):
            got = d.project_quantized(tensor(api, d, eye[m0:m1], dtype), own, out_dtype=api.DType.F32).tensor.to_f32()
            want = oracle.round_storage(dense[:, m0:m1].T.copy(), code).reshape(m1 - m0, n)
            assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype_name,m", [("F32", 1), ("F16", 3), ("F16", 40)])
def test_silu_mul_input(api, d, dtype_name, m):
    n, k = 515, 800
    dtype, code = api.DType[dtype_name], CODE[dtype_name]
    packed, own, wide = both(api, d, n, k, seed=441)
    packed_x = oracle.round_storage(synth.activations(m, 2 * k, seed=442), code).reshape(m, 2 * k)
    out = d.project_quantized(tensor(api, d, packed_x, dtype), own, out_dtype=api.DType.F32, silu_mul=True)
    act = oracle.expert_silu_mul(packed_x, k, code)
    want = oracle.project(Q8_0, packed, n, k, act, accumulate="f64")
    assert_matmul_parity(out.tensor.to_f32(), want, f"q8_0 silu m={m}")
    same = d.project_quantized(tensor(api, d, widened(packed_x, k, 2), dtype), wide, out_dtype=api.DType.F32,
                               silu_mul=True)
    assert np.array_equal(bits(out.tensor.to_f32()), bits(same.tensor.to_f32()))


@pytest.mark.parametrize("m", [1, 3, 16, 64])
def test_hybrid_projection_tiers(api, d, m):
    n, k = 300, 2880
    packed, own, wide = both(api, d, n, k, seed=451)
    x = synth.activations(m, k, seed=452)
    out = d.hybrid_project(own, tensor(api, d, x, api.DType.F32))
    assert out.operation == {1: "h_mv_q8_0", 3: "h_mvb_q8_0", 16: "h_mms_q8_0", 64: "h_mm_q8_0"}[m]
    if m < 5:
        want = oracle.project(Q8_0, packed, n, k, x, accumulate="f64")
    else:
        want = oracle.project(Q8_0, packed, n, k, oracle.round_storage(x, oracle.F16).reshape(m, k),
                              weight_round=oracle.F16, accumulate="f64")
    assert_matmul_parity(out.tensor.to_f32(), want, f"q8_0 hybrid m={m}")
    same = d.hybrid_project(wide, tensor(api, d, widened(x, k), api.DType.F32))
    assert np.array_equal(bits(out.tensor.to_f32()), bits(same.tensor.to_f32()))


def routes_of(ids, tokens=None):
    meta = np.zeros((len(ids), 3), dtype=np.uint32)
    meta[:, 0] = ids
    meta[:, 1] = np.arange(len(ids)) if tokens is None else tokens
    meta[:, 2] = np.float32(1.0).view(np.uint32)
    return meta


@pytest.mark.parametrize("form", ["rows", "gather", "silu_mul"])
@pytest.mark.parametrize("assignments,dtype_name", [(5, "F32"), (7, "F16"), (150, "F16"), (150, "BF16")])
def test_expert_projection_in_every_input_form(api, d, form, assignments, dtype_name):
    experts, rows, k, tokens = 6, 200, 800, 40
    dtype, code = api.DType[dtype_name], CODE[dtype_name]
    packed, own, wide = both(api, d, rows, k, seed=461, experts=experts)
    rng = synth.rng(462 + assignments)
    ids = np.sort(rng.choice([0, 1, 2, 4, 5], size=assignments))          # expert 3 gets nothing
    token_of = rng.integers(0, tokens, assignments)
    meta = routes_of(ids, token_of)
    mt = api.Tensor.from_bits(d, meta.shape, meta)
    if form == "rows":
        x = oracle.round_storage(synth.activations(assignments, k, seed=463) * 0.25, code).reshape(assignments, k)
        per_assignment, parts = x, 1
    elif form == "gather":
        x = oracle.round_storage(synth.activations(tokens, k, seed=464) * 0.25, code).reshape(tokens, k)
        per_assignment, parts = x[token_of], 1
    else:
        x = oracle.round_storage(synth.activations(assignments, 2 * k, seed=465), code).reshape(assignments, 2 * k)
        per_assignment, parts = oracle.expert_silu_mul(x, k, code), 2
    got = d.expert_project_quantized(tensor(api, d, x, dtype), mt, own, k, experts, out_dtype=api.DType.F32, form=form)
    operation = d.last_operation()
    grouped = assignments >= 32 and dtype_name != "F32"
    assert ("grouped" in operation) == grouped
    want = oracle.expert_project(Q8_0, packed, experts, rows, k, per_assignment, meta.view(np.float32), accumulate="f64",
                                 weight_round=code if grouped else 0)
    assert_matmul_parity(got.to_f32(), want, f"q8_0 routes {form} a={assignments}")
    same = d.expert_project_quantized(tensor(api, d, widened(x, k, parts), dtype), mt, wide, stored_width(k), experts,
                                      out_dtype=api.DType.F32, form=form)
    assert d.last_operation() == operation
    assert np.array_equal(bits(got.to_f32()), bits(same.to_f32()))


@pytest.mark.parametrize("tokens", [2, 60])
def test_shared_expert_rides_in_both_forms(api, d, tokens):
    experts, rows, k, top_k = 4, 192, 800, 2
    packed, own, wide = both(api, d, rows, k, seed=471, experts=experts)
    spacked, sown, swide = both(api, d, rows, k, seed=472)
    dtype, code = api.DType.F16, oracle.F16
    rng = synth.rng(473)
    a = tokens * top_k
    ids = rng.integers(0, experts, a)
    meta = routes_of(ids, np.repeat(np.arange(tokens), top_k))
    mt = api.Tensor.from_bits(d, meta.shape, meta)
    x = oracle.round_storage(synth.activations(tokens, k, seed=474) * 0.25, code).reshape(tokens, k)
    routed, shared = d.expert_project_with_shared(tensor(api, d, x, dtype), mt, own, sown, tokens, "gather")
    want = oracle.expert_project(Q8_0, packed, experts, rows, k, x[meta[:, 1]], meta.view(np.float32), accumulate="f64",
                                 weight_round=code if a >= 32 else 0)
    swant = oracle.project(Q8_0, spacked, rows, k, x, accumulate="f64", weight_round=code if a >= 32 else 0)
    assert rel_l2(routed.to_f32(), want) <= 1e-3 and rel_l2(shared.to_f32(), swant) <= 1e-3
    r2, s2 = d.expert_project_with_shared(tensor(api, d, widened(x, k), dtype), mt, wide, swide, tokens, "gather")
    assert np.array_equal(routed.raw(), r2.raw()) and np.array_equal(shared.raw(), s2.raw())
    packed_x = oracle.round_storage(synth.activations(a, 2 * k, seed=475), code).reshape(a, 2 * k)
    shared_x = oracle.round_storage(synth.activations(tokens, 2 * k, seed=476), code).reshape(tokens, 2 * k)
    routed, shared = d.expert_project_with_shared(tensor(api, d, packed_x, dtype), mt, own, sown, tokens, "silu_mul",
                                                  shared_input=tensor(api, d, shared_x, dtype))
    want = oracle.expert_project(Q8_0, packed, experts, rows, k, oracle.expert_silu_mul(packed_x, k, code),
                                 meta.view(np.float32), accumulate="f64", weight_round=code if a >= 32 else 0)
    swant = oracle.project(Q8_0, spacked, rows, k, oracle.expert_silu_mul(shared_x, k, code), accumulate="f64",
                           weight_round=code if a >= 32 else 0)
    assert rel_l2(routed.to_f32(), want) <= 1e-3 and rel_l2(shared.to_f32(), swant) <= 1e-3
    r2, s2 = d.expert_project_with_shared(tensor(api, d, widened(packed_x, k, 2), dtype), mt, wide, swide, tokens,
                                          "silu_mul", shared_input=tensor(api, d, widened(shared_x, k, 2), dtype))
    assert np.array_equal(routed.raw(), r2.raw()) and np.array_equal(shared.raw(), s2.raw())


def test_hybrid_routed_projections(api, d):
    experts, rows, k, tokens, used = 5, 160, 800, 12, 3
    packed, own, wide = both(api, d, rows, k, seed=481, experts=experts)
    spacked, sown, swide = both(api, d, rows, k, seed=482)
    rng = synth.rng(483)
    routes = tokens * used
    ids = rng.integers(0, experts, routes).astype(np.uint32)
    it = api.Tensor.from_bits(d, (routes,), ids)
    x = synth.activations(tokens, k, seed=484)
    xt, xw = tensor(api, d, x, api.DType.F32), tensor(api, d, widened(x, k), api.DType.F32)
    # project_id: route r multiplies row r / used by expert ids[r]; the shared expert reads the token rows
    y, ys = d.hybrid_project_id_with_shared(own, sown, xt, it, routes, used, tokens)
    meta = routes_of(ids)
    want = oracle.expert_project(Q8_0, packed, experts, rows, k, np.repeat(x, used, axis=0), meta.view(np.float32),
                                 accumulate="f64")
    assert_matmul_parity(y.to_f32(), want, "q8_0 project_id")
    assert_matmul_parity(ys.to_f32(), oracle.project(Q8_0, spacked, rows, k, x, accumulate="f64"), "q8_0 project_id shared")
    y2, ys2 = d.hybrid_project_id_with_shared(wide, swide, xw, it, routes, used, tokens)
    assert np.array_equal(y.raw(), y2.raw()) and np.array_equal(ys.raw(), ys2.raw())
    plain = d.hybrid_project_id(own, xt, it, routes, used)
    assert np.array_equal(plain.raw(), y.raw())
    # project_mm_id: expert-sorted rows and offsets, f32 rows rounded to f16 on the way in
    offsets, order, position = d.hybrid_moe_map(it, experts)
    sorted_x = d.hybrid_moe_gather(xt, order, used)
    host_order = order.raw().view(np.uint32)
    z, zs = d.hybrid_project_mm_id_with_shared(own, sown, sorted_x, offsets, xt)
    x16 = oracle.round_storage(x, oracle.F16).reshape(tokens, k)
    sorted_meta = routes_of(ids[host_order])
    want = oracle.expert_project(Q8_0, packed, experts, rows, k, x16[host_order // used], sorted_meta.view(np.float32),
                                 accumulate="f64", weight_round=oracle.F16)
    assert_matmul_parity(z.to_f32(), want, "q8_0 project_mm_id")
    assert_matmul_parity(zs.to_f32(), oracle.project(Q8_0, spacked, rows, k, x16, accumulate="f64", weight_round=oracle.F16),
                         "q8_0 project_mm_id shared")
    sorted_wide = d.hybrid_moe_gather(xw, order, used)
    z2, zs2 = d.hybrid_project_mm_id_with_shared(wide, swide, sorted_wide, offsets, xw)
    assert np.array_equal(z.raw(), z2.raw()) and np.array_equal(zs.raw(), zs2.raw())
    assert np.array_equal(d.hybrid_project_mm_id(own, sorted_x, offsets).raw(), z.raw())


@pytest.mark.parametrize("dtype_name,tokens,shared", [("F16", 1, True), ("F16", 3, False), ("F16", 70, True), ("F32", 5, True)])
def test_routed_ffn_in_one_call_and_as_separate_calls(api, d, dtype_name, tokens, shared):
    # hidden 800 and intermediate 288: both projections' rows end inside a run of eight blocks
    experts, hidden, inter, top_k = 8, 800, 288, 2
    dtype, code = api.DType[dtype_name], CODE[dtype_name]
    fmt = api.QuantizationFormat.Q8_0
    pin = synth.matrix(Q8_0, experts * 2 * inter, hidden, seed=491)
    pout = synth.matrix(Q8_0, experts * hidden, inter, seed=492)
    win = api.QuantizedExpertMatrix.new(d, pin, fmt, experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, pout, fmt, experts, hidden, inter)
    kw = {}
    if shared:
        psin, psout = synth.matrix(Q8_0, 2 * inter, hidden, seed=493), synth.matrix(Q8_0, hidden, inter, seed=494)
        kw = dict(shared_input=api.QuantizedMatrix.from_bytes(d, 2 * inter, hidden, fmt, psin),
                  shared_output=api.QuantizedMatrix.from_bytes(d, hidden, inter, fmt, psout))
    moe = api.SparseMoe(d, win, wout, api.MoeRoutingPolicy(experts, top_k), **kw)
    x = oracle.round_storage(synth.activations(tokens, hidden, seed=495) * 4, code).reshape(tokens, hidden)
    logits = synth.rng(496).standard_normal((tokens, experts)).astype(np.float32)
    xt, lt = tensor(api, d, x, dtype), tensor(api, d, logits, api.DType.F32)
    stepwise = moe.forward(xt, lt)
    one_call = moe.forward_in_one_call(xt, lt)
    assert np.array_equal(stepwise.raw(), one_call.raw())
    out = api.Tensor.zeros(d, (tokens, hidden), dtype)
    with d.execution() as ex:                 # the temporaries have their size: the call can be recorded
        moe.forward_in_one_call(xt, lt, out=out)
    ex.graph.launch()
    d.synchronize()
    assert np.array_equal(out.raw(), one_call.raw())
    meta = oracle.select_routes(logits, experts, top_k)
    up = oracle.round_storage(oracle.expert_project(Q8_0, pin, experts, 2 * inter, hidden,
                                                    oracle.expert_assign(x, meta), meta), code)
    down = oracle.round_storage(oracle.expert_project(Q8_0, pout, experts, hidden, inter,
                                                      oracle.expert_silu_mul(up, inter, code), meta), code)
    if shared:
        sup = oracle.round_storage(oracle.project(Q8_0, psin, 2 * inter, hidden, x), code)
        sdown = oracle.round_storage(oracle.project(Q8_0, psout, hidden, inter, oracle.expert_silu_mul(sup, inter, code)), code)
        want = oracle.expert_combine_shared(down, meta, tokens, hidden, top_k, sdown, None, dtype=code)
    else:
        want = oracle.expert_combine(down, meta, tokens, hidden, top_k, dtype=code)
    assert np.abs(want).max() > 1e-3
    assert rel_l2(one_call.to_f32(), want) <= (1e-5 if dtype_name == "F32" else 3e-3)


def test_recorded_projection_and_what_is_refused(api, d):
    n, k, m = 515, 2880, 2
    packed, own, _ = both(api, d, n, k, seed=501)
    x = synth.activations(m, k, seed=502)
    xt = tensor(api, d, x, api.DType.F32)
    want = d.project_quantized(xt, own).tensor
    out = api.Tensor.zeros(d, (m, n), api.DType.F32)
    with d.execution() as ex:
        d.project_quantized(xt, own, out=out)
    for _ in range(2):
        ex.graph.launch()
        d.synchronize()
        assert np.array_equal(out.raw(), want.raw())
        api._check(api._lib.fh_buffer_fill_zero(out.buffer._handle, 0, out.byte_size()))
        d.synchronize()
    # the entry point that allocates nothing has no room for the widened activations
    with pytest.raises(api.ShapeError, match="stored padded"):
        d.project_quantized_no_alloc(xt, own, out)
    # an output on top of the activations is refused as for any other matrix
    square = api.QuantizedMatrix.from_bytes(d, k, k, api.QuantizationFormat.Q8_0, synth.matrix(Q8_0, k, k, seed=503))
    xs = tensor(api, d, synth.activations(1, k, seed=504), api.DType.F32)
    with pytest.raises(api.RangeError):
        d.project_quantized(xs, square, out=xs)
    # a row is whole 32-weight blocks
    with pytest.raises(api.ShapeError, match="block size 32"):
        api.QuantizedMatrix.from_bytes(d, 4, 48, api.QuantizationFormat.Q8_0, packed[: 4 * 34])
    with pytest.raises(api.Error):
        api.QuantizedMatrix.from_bytes(d, 4, 288, api.QuantizationFormat.Q8_0, packed[: 4 * 9 * 34 - 1])
    bad = packed[: 4 * 9 * 34].copy()
    bad[34 * 20 + 1] = 0x7c                     # an infinite scale in a block past the first run
    with pytest.raises(api.WeightError):
        api.QuantizedMatrix.from_bytes(d, 4, 288, api.QuantizationFormat.Q8_0, bad)
