"""GPU parity of the mixture-of-experts stages against the CPU oracle, through
the C ABI.  Cases follow src/nn/moe.rs:666-819 (router), the expert
projection tests of src/ops/transformer.rs:3331-3388 / 4371-4424, and the
35B-A3B style configuration of the benchmark (hidden 2048, 256 experts,
intermediate 512, top-8)."""
import numpy as np
import pytest

import ferrum_fixtures as fx
import oracle
from helpers import assert_matmul_parity, bits, fma_gemv, rel_l2
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


def route_both(api, d, logits, policy, bias=None, dtype=None):
    dtype = api.DType.F32 if dtype is None else dtype
    lt = api.Tensor.from_f32(d, logits.shape, dtype, logits)
    bt = None if bias is None else api.Tensor.from_f32(d, (policy.experts,), api.DType.F32, bias)
    got = d.moe_route(lt, bt, policy).to_f32()
    want = oracle.select_routes(lt.to_f32(), policy.experts, policy.top_k,
                                sigmoid=policy.scoring_function == api.MoeScoringFunction.Sigmoid,
                                normalize=policy.normalize_top_k_prob,
                                eps=policy.normalization_epsilon,
                                scaling=policy.routed_scaling_factor, bias=bias)
    return got, want


def assert_routes(got, want):
    assert np.array_equal(bits(got[:, 0]), bits(want[:, 0])), "expert ids"
    assert np.array_equal(bits(got[:, 1]), bits(want[:, 1])), "token ids"
    assert np.abs(got[:, 2] - want[:, 2]).max() <= 2e-6, "route weights"


def test_router_preserves_cpu_top_k_order_and_weights(api, d):
    # src/nn/moe.rs:741-819
    logits = np.array([[0, 0, 0, 0, 0], [2, 0.5, -1, 1.5, 0]], dtype=np.float32)
    bias = np.array([0.1, 0.05, 0.1, -0.3, 0.1], dtype=np.float32)
    for scoring, use_bias in ((api.MoeScoringFunction.Sigmoid, True),
                              (api.MoeScoringFunction.Softmax, True),
                              (api.MoeScoringFunction.Softmax, False)):
        policy = api.MoeRoutingPolicy(5, 3, scoring, True, 1e-6, 1.25, use_bias)
        got, want = route_both(api, d, logits, policy, bias if use_bias else None, api.DType.BF16)
        assert_routes(got, want)
    # expert_assign gathers the token rows named by the metadata
    policy = api.MoeRoutingPolicy(5, 3, api.MoeScoringFunction.Softmax, True, 1e-6, 1.25)
    lt = api.Tensor.from_f32(d, (2, 5), api.DType.BF16, logits)
    meta = d.moe_route(lt, None, policy)
    hidden = api.Tensor.from_f32(d, (2, 1), api.DType.BF16, [1.0, 2.0])
    assigned = d.expert_assign(hidden, meta, 3).to_f32().reshape(-1)
    tokens = bits(meta.to_f32()[:, 1])
    assert np.array_equal(assigned, np.array([1.0, 2.0], dtype=np.float32)[tokens])


def test_router_literal_cases(api, d):
    # src/nn/moe.rs:666-739
    policy = api.MoeRoutingPolicy(3, 2, api.MoeScoringFunction.Sigmoid, True, 1e-6, 1.5)
    got, want = route_both(api, d, np.array([[0.0, 2.0, -2.0]], dtype=np.float32), policy)
    assert_routes(got, want)
    assert bits(got[:, 0]).tolist() == [0, 1] and abs(got[0, 2] + got[1, 2] - 1.5) < 2e-6
    policy = api.MoeRoutingPolicy(3, 2, api.MoeScoringFunction.Sigmoid, True, 1e-6, 1.0, True)
    got, want = route_both(api, d, np.array([[2.0, 1.0, 0.0]], dtype=np.float32), policy,
                           np.array([-10.0, 0.0, 2.0], dtype=np.float32))
    assert_routes(got, want)
    assert bits(got[:, 0]).tolist() == [1, 2]


@pytest.mark.parametrize("tokens", [1, 512])
def test_router_256_experts_top8(api, d, tokens):
    logits = synth.rng(9, tokens).standard_normal((tokens, 256)).astype(np.float32)
    policy = api.MoeRoutingPolicy(256, 8, api.MoeScoringFunction.Softmax, True, 0.0, 1.0)
    got, want = route_both(api, d, logits, policy)
    assert_routes(got, want)
    assert np.allclose(got[:, 2].reshape(tokens, 8).sum(1), 1.0, atol=1e-5)
    # ids ascend within a token
    ids = bits(got[:, 0]).reshape(tokens, 8).astype(np.int64)
    assert np.all(np.diff(ids, axis=1) > 0)


def test_router_rejects_invalid_geometry(api, d):
    lt = api.Tensor.zeros(d, (2, 5), api.DType.F32)
    with pytest.raises(api.ShapeError):
        d.moe_route(lt, None, api.MoeRoutingPolicy(5, 0))
    with pytest.raises(api.ShapeError):
        d.moe_route(lt, None, api.MoeRoutingPolicy(5, 6))
    with pytest.raises(api.ShapeError):
        d.moe_route(lt, None, api.MoeRoutingPolicy(4, 2))
    with pytest.raises(api.ShapeError):
        d.moe_route(lt, None, api.MoeRoutingPolicy(5, 17))
    with pytest.raises(api.ShapeError):
        d.moe_route(lt, None, api.MoeRoutingPolicy(5, 2, routed_scaling_factor=0.0))


@pytest.mark.parametrize("ggml", [Q4_K, Q6_K])
def test_expert_projection_uses_assignment_metadata(api, d, ggml):
    # src/ops/transformer.rs:3331-3388: 3 experts x 5 rows, ids [2, 1, 2, 0],
    # BF16 activations and outputs, abs <= 0.06 (Q4_K) / 0.12 (Q6_K)
    experts, rows, cols = 3, 5, 512
    expert_ids = [2, 1, 2, 0]
    packed = fx.q4k_packed(experts * rows, cols) if ggml == Q4_K else fx.q6k_packed(experts * rows, cols)
    fmt = api.QuantizationFormat(ggml)
    w = api.QuantizedExpertMatrix.new(d, packed, fmt, experts, rows, cols)
    values = fx.q4k_input(len(expert_ids), cols)
    x = api.Tensor.from_f32(d, (len(expert_ids), cols), api.DType.BF16, values)
    meta_bits = np.zeros((len(expert_ids), 3), dtype=np.uint32)
    meta_bits[:, 0] = expert_ids
    meta_bits[:, 1] = np.arange(len(expert_ids))
    meta_bits[:, 2] = np.float32(1.0).view(np.uint32)
    meta = api.Tensor.from_bits(d, (len(expert_ids), 3), meta_bits)
    actual = d.expert_project_quantized(x, meta, w, cols, experts).to_f32()
    expected = oracle.expert_project(ggml, packed, experts, rows, cols, x.to_f32(), meta.to_f32(),
                                     out_round=oracle.BF16)
    assert np.abs(actual - expected).max() <= (0.06 if ggml == Q4_K else 0.12)
    exact = d.expert_project_quantized(x, meta, w, cols, experts, out_dtype=api.DType.F32).to_f32()
    want64 = oracle.expert_project(ggml, packed, experts, rows, cols, x.to_f32(), meta.to_f32(),
                                   accumulate="f64")
    assert_matmul_parity(exact, want64, "expert projection")
    with pytest.raises(api.ShapeError):
        d.expert_project_quantized(x, meta, w, cols, experts + 1)


def test_silu_mul_and_combine_keep_the_storage_rounding_points(api, d):
    rng = synth.rng(21)
    # 96 / 64 columns take the eight-wide kernels, 10 / 6 the element-wise ones
    cases = [(24, 96, 6, 4, 64, dt) for dt in ((api.DType.F32, oracle.F32), (api.DType.F16, oracle.F16),
                                               (api.DType.BF16, oracle.BF16))]
    cases += [(12, 10, 4, 3, 6, dt) for dt in ((api.DType.F32, oracle.F32), (api.DType.BF16, oracle.BF16))]
    for a, inter, tokens, top_k, hidden, (dtype, code) in cases:
        packed_rows = (rng.standard_normal((a, 2 * inter)) * 2).astype(np.float32)
        t = api.Tensor.from_f32(d, packed_rows.shape, dtype, packed_rows)
        got = d.expert_silu_mul(t, inter).to_f32()
        want = oracle.expert_silu_mul(t.to_f32(), inter, code)
        if dtype == api.DType.F32:
            assert np.abs(got - want).max() <= 1e-6 * max(1.0, np.abs(want).max())
        else:
            # expf may differ in the last ulp between libm and the GPU; after
            # storage rounding at most a rare one-step difference remains
            step = 2.0 ** (-10 if dtype == api.DType.F16 else -7)
            assert np.all(np.abs(got - want) <= step * np.maximum(np.abs(want), 1e-3))
            assert np.mean(got != want) < 0.01

        values = rng.standard_normal((tokens * top_k, hidden)).astype(np.float32)
        logits = rng.standard_normal((tokens, 16)).astype(np.float32)
        meta_np = oracle.select_routes(logits, 16, top_k)
        vt = api.Tensor.from_f32(d, values.shape, dtype, values)
        mt = api.Tensor.from_bits(d, meta_np.shape, meta_np.view(np.uint32))
        got = d.expert_combine(vt, mt, tokens, hidden, top_k).to_f32()
        want = oracle.expert_combine(vt.to_f32(), meta_np, tokens, hidden, top_k, code)
        assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("tokens", [1, 48])
def test_routed_ffn_pipeline_matches_the_oracle(api, d, tokens):
    # hidden 2048, intermediate 512, top-8; 16 experts keep the CPU side quick
    hidden, inter, experts, top_k = 2048, 512, 16, 8
    w_in = synth.matrix(Q4_K, experts * 2 * inter, hidden, seed=31)
    w_out = synth.matrix(Q4_K, experts * hidden, inter, seed=32)
    x = synth.activations(tokens, hidden, seed=33, f16=True)
    logits = synth.rng(34).standard_normal((tokens, experts)).astype(np.float32)
    fmt = api.QuantizationFormat.Q4_K
    win = api.QuantizedExpertMatrix.new(d, w_in, fmt, experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, w_out, fmt, experts, hidden, inter)
    policy = api.MoeRoutingPolicy(experts, top_k)

    xt = api.Tensor.from_f32(d, x.shape, api.DType.F32, x)
    meta = d.moe_route(api.Tensor.from_f32(d, logits.shape, api.DType.F32, logits), None, policy)
    assigned = d.expert_assign(xt, meta, top_k)
    up = d.expert_project_quantized(assigned, meta, win, hidden, experts)
    act = d.expert_silu_mul(up, inter)
    down = d.expert_project_quantized(act, meta, wout, inter, experts)
    got = d.expert_combine(down, meta, tokens, hidden, top_k).to_f32()

    m = oracle.select_routes(logits, experts, top_k)
    assert np.array_equal(bits(meta.to_f32()[:, :2]), bits(m[:, :2]))
    o_assigned = oracle.expert_assign(x, m)
    o_up = oracle.expert_project(Q4_K, w_in, experts, 2 * inter, hidden, o_assigned, m, accumulate="f64")
    o_act = oracle.expert_silu_mul(o_up, inter)
    o_down = oracle.expert_project(Q4_K, w_out, experts, hidden, inter, o_act, m, accumulate="f64")
    want = oracle.expert_combine(o_down, m, tokens, hidden, top_k)
    assert np.abs(want).max() > 1e-2
    assert rel_l2(got, want) <= 2e-5
    assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max()) * 8


def _routing_rows(expert_ids):
    meta = np.zeros((len(expert_ids), 3), dtype=np.uint32)
    meta[:, 0] = expert_ids
    meta[:, 1] = np.arange(len(expert_ids))
    meta[:, 2] = np.float32(1.0).view(np.uint32)
    return meta


@pytest.mark.parametrize("ggml,dtype", [(Q4_K, "F16"), (Q4_K, "BF16"), (Q6_K, "F16"), (13, "F16")])
def test_grouped_expert_projection_matches_the_oracle_and_the_direct_form(api, d, ggml, dtype):
    # 6 experts x 72 rows (a ragged last row tile), K = 768.  Expert 3 gets no
    # assignment, expert 1 gets 37 (more than one pass of 32 tokens), expert 5
    # a single one, and two assignments carry an expert id that does not exist.
    experts, rows, cols = 6, 72, 768
    rng = synth.rng(51)
    ids = np.concatenate([np.full(37, 1), np.full(9, 0), np.full(17, 2), np.full(12, 4), [5], [9, 77]])
    rng.shuffle(ids)
    packed = synth.matrix(ggml, experts * rows, cols, seed=52)
    w = api.QuantizedExpertMatrix.new(d, packed, api.QuantizationFormat(ggml), experts, rows, cols)
    dt = getattr(api.DType, dtype)
    code = oracle.F16 if dtype == "F16" else oracle.BF16
    x = api.Tensor.from_f32(d, (len(ids), cols), dt, synth.activations(len(ids), cols, seed=53))
    meta = api.Tensor.from_bits(d, (len(ids), 3), _routing_rows(ids))
    valid = ids < experts

    got = d.expert_project_quantized(x, meta, w, cols, experts, out_dtype=api.DType.F32)
    assert d.last_operation() == {Q4_K: "expert_project_q4_k_grouped_mfma", 13: "expert_project_q5_k_grouped_mfma",
                                  Q6_K: "expert_project_q6_k_grouped_mfma"}[ggml]
    got = got.to_f32()
    safe = _routing_rows(np.where(valid, ids, 0)).view(np.float32)
    tile = oracle.expert_project(ggml, packed, experts, rows, cols, x.to_f32(), safe,
                                 weight_round=code, accumulate="f64")
    full = oracle.expert_project(ggml, packed, experts, rows, cols, x.to_f32(), safe, accumulate="f64")
    assert np.all(got[~valid] == 0), "rows of unknown experts are zero"
    assert_matmul_parity(got[valid], tile[valid], "grouped expert projection (tile-rounded weights)")
    assert rel_l2(got[valid], full[valid]) <= (6e-4 if dtype == "F16" else 5e-3)

    d.set_tuning("expert_grouped_min_assignments", 0)
    try:
        direct = d.expert_project_quantized(x, meta, w, cols, experts, out_dtype=api.DType.F32)
        assert d.last_operation().endswith("_factored")
        direct = direct.to_f32()
    finally:
        d.set_tuning("expert_grouped_min_assignments", 32)
    assert_matmul_parity(direct[valid], full[valid], "direct expert projection")
    assert np.all(direct[~valid] == 0)

    half = d.expert_project_quantized(x, meta, w, cols, experts).to_f32()   # output in the input dtype
    assert np.array_equal(bits(half), bits(oracle.round_storage(got, code)))


@pytest.mark.parametrize("dtype", ["F16", "BF16"])
@pytest.mark.parametrize("cols,crowd", [(256, 37), (512, 37), (512, 11), (768, 37), (1024, 11), (1024, 37)])
@pytest.mark.parametrize("ggml", [Q4_K, Q6_K])
def test_grouped_projection_with_short_rows_streams_weights_through_lds(api, d, ggml, cols, crowd, dtype):
    # Rows of one to four super-blocks and a whole number of 16-row tiles: every wave copies its
    # weight tiles into a ring in LDS.  The same call with the ring switched off loads them straight
    # into registers and multiplies in the same order, so the bits agree.  `crowd` assignments
    # for expert 1: 37 take two passes of 32 tokens, 11 fit one 16-token tile.
    experts, rows = 5, 80
    rng = synth.rng(61)
    ids = np.concatenate([np.full(crowd, 1), np.full(9, 0), np.full(13, 2), [4], [9, 77]])
    rng.shuffle(ids)
    packed = synth.matrix(ggml, experts * rows, cols, seed=62)
    w = api.QuantizedExpertMatrix.new(d, packed, api.QuantizationFormat(ggml), experts, rows, cols)
    dt = getattr(api.DType, dtype)
    code = oracle.F16 if dtype == "F16" else oracle.BF16
    x = api.Tensor.from_f32(d, (len(ids), cols), dt, synth.activations(len(ids), cols, seed=63))
    meta = api.Tensor.from_bits(d, (len(ids), 3), _routing_rows(ids))
    valid = ids < experts

    got = d.expert_project_quantized(x, meta, w, cols, experts, out_dtype=api.DType.F32)
    assert d.last_operation() == {Q4_K: "expert_project_q4_k_grouped_mfma", Q6_K: "expert_project_q6_k_grouped_mfma"}[ggml]
    got = got.to_f32()
    d.set_tuning("expert_weight_ring", 0)
    try:
        registers = d.expert_project_quantized(x, meta, w, cols, experts, out_dtype=api.DType.F32).to_f32()
    finally:
        d.set_tuning("expert_weight_ring", 1)
    assert np.array_equal(bits(got), bits(registers))
    safe = _routing_rows(np.where(valid, ids, 0)).view(np.float32)
    tile = oracle.expert_project(ggml, packed, experts, rows, cols, x.to_f32(), safe, weight_round=code, accumulate="f64")
    assert np.all(got[~valid] == 0), "rows of unknown experts are zero"
    assert_matmul_parity(got[valid], tile[valid], "grouped expert projection, weights through LDS")
    half = d.expert_project_quantized(x, meta, w, cols, experts).to_f32()   # output in the input dtype
    assert np.array_equal(bits(half), bits(oracle.round_storage(got, code)))


@pytest.mark.parametrize("tokens", [1, 512])
def test_a3b_style_ffn_with_shared_expert(api, d, tokens):
    # hidden 2048, 256 experts of intermediate 512, top-8 after softmax with
    # renormalised weights, plus one always-on shared expert; f16 activations.
    hidden, inter, experts, top_k = 2048, 512, 256, 8
    fmt = api.QuantizationFormat.Q4_K
    # 256 distinct experts would take the CPU side minutes: 8 distinct weight
    # sets are tiled 32 times, which leaves routing, grouping and addressing
    # at full size while the oracle evaluates 8 experts' worth of rows
    distinct = 8
    w_in8 = synth.matrix(Q4_K, distinct * 2 * inter, hidden, seed=61).reshape(distinct, -1)
    w_out8 = synth.matrix(Q4_K, distinct * hidden, inter, seed=62).reshape(distinct, -1)
    w_in = np.tile(w_in8, (experts // distinct, 1)).reshape(-1)
    w_out = np.tile(w_out8, (experts // distinct, 1)).reshape(-1)
    s_in = synth.matrix(Q4_K, 2 * inter, hidden, seed=63)
    s_out = synth.matrix(Q4_K, hidden, inter, seed=64)
    # the synthetic weights are O(1), so unit activations would overflow f16 after two
    # chained projections; 2^-6 keeps every stage inside the f16 range
    x = synth.activations(tokens, hidden, seed=65, f16=True) * np.float32(2.0 ** -6)
    logits = synth.rng(66).standard_normal((tokens, experts)).astype(np.float32)

    win = api.QuantizedExpertMatrix.new(d, w_in, fmt, experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, w_out, fmt, experts, hidden, inter)
    sin = api.QuantizedMatrix.from_bytes(d, 2 * inter, hidden, fmt, s_in)
    sout = api.QuantizedMatrix.from_bytes(d, hidden, inter, fmt, s_out)
    policy = api.MoeRoutingPolicy(experts, top_k)
    f16, f32 = api.DType.F16, api.DType.F32

    xt = api.Tensor.from_f32(d, x.shape, f16, x)
    meta = d.moe_route(api.Tensor.from_f32(d, logits.shape, f32, logits), None, policy)
    assigned = d.expert_assign(xt, meta, top_k)
    up = d.expert_project_quantized(assigned, meta, win, hidden, experts)
    assert d.last_operation() == ("expert_project_q4_k_grouped_mfma" if tokens > 1
                                  else "expert_project_q4_k_factored")
    act = d.expert_silu_mul(up, inter)
    down = d.expert_project_quantized(act, meta, wout, inter, experts)
    routed = d.expert_combine(down, meta, tokens, hidden, top_k).to_f32()
    s_up = d.project_quantized(xt, sin).tensor
    s_act = d.expert_silu_mul(s_up, inter)
    shared = d.project_quantized(s_act, sout).tensor.to_f32()
    got = routed + shared

    m = oracle.select_routes(logits, experts, top_k)
    assert np.array_equal(bits(meta.to_f32()[:, :2]), bits(m[:, :2]))
    # a token's output depends on its own eight routes only: the oracle follows
    # every token at T = 1 and a sample of 24 tokens at T = 512
    picked = np.arange(tokens) if tokens <= 24 else np.sort(synth.rng(67).choice(tokens, 24, replace=False))
    m = m.reshape(tokens, top_k, 3)[picked].reshape(-1, 3).copy()
    m[:, 1] = np.repeat(np.arange(len(picked), dtype=np.uint32), top_k).view(np.float32)
    x, got, tokens = x[picked], got[picked], len(picked)
    folded = m.copy()
    folded_ids = m[:, 0].view(np.uint32) % distinct
    folded[:, 0] = folded_ids.astype(np.uint32).view(np.float32)
    tile = oracle.F16 if tokens > 1 else 0     # one token runs the f32-weight GEMV form
    o_up = oracle.expert_project(Q4_K, w_in8.reshape(-1), distinct, 2 * inter, hidden,
                                 oracle.expert_assign(x, m), folded, weight_round=tile,
                                 out_round=oracle.F16, accumulate="f64")
    o_act = oracle.expert_silu_mul(o_up, inter, oracle.F16)
    o_down = oracle.expert_project(Q4_K, w_out8.reshape(-1), distinct, hidden, inter, o_act, folded,
                                   weight_round=tile, out_round=oracle.F16, accumulate="f64")
    o_routed = oracle.expert_combine(o_down, m, tokens, hidden, top_k, oracle.F16)
    stile = oracle.F16 if tokens > 1 else 0
    o_sup = oracle.round_storage(oracle.project(Q4_K, s_in, 2 * inter, hidden, x, accumulate="f64",
                                                weight_round=stile), oracle.F16)
    o_sact = oracle.expert_silu_mul(o_sup, inter, oracle.F16)
    o_shared = oracle.round_storage(oracle.project(Q4_K, s_out, hidden, inter, o_sact, accumulate="f64",
                                                   weight_round=stile), oracle.F16)
    want = o_routed + o_shared
    assert np.abs(want).max() > 1e-2
    # every stage stores f16, so a last-place difference in an intermediate moves
    # the result by about one f16 step of that stage
    assert rel_l2(got, want) <= 2e-3
    assert np.abs(got - want).max() <= 4e-3 * np.abs(want).max()


def _scaled_d(blocks, power):
    """Q4_K blocks [.., 144] with every block's f16 d multiplied by 2^power (exponent bits)."""
    out = blocks.copy()
    d = out[..., 0:2].copy().view(np.uint16)
    assert ((d >> 10) & 31).min() >= 1 and ((d >> 10) & 31).max() + power < 31
    out[..., 0:2] = (d + np.uint16(power << 10)).view(np.uint8)
    return out


@pytest.mark.parametrize("tokens", [1, 512])
def test_a3b_ffn_as_benchmarked_with_256_distinct_experts(api, d, tokens):
    # The path bench.py times: SparseMoe.forward with the shared expert riding in the routed launches,
    # hidden 2048, 256 experts of intermediate 512, top-8, f16.  Every expert is different, every
    # token is checked, and the host side still evaluates one expert per token: expert e is the base
    # expert with (a) its output rows rotated by 8e, (b) its up rows scaled by 2^((e / 2) % 4), an exact
    # scaling because the minimums are zero, and (c) for odd e the gate / up rows rotated by 256, with the
    # down projection's two column blocks swapped to match.  So routed_e(x) = 2^c roll(routed_base(x)).
    hidden, inter, experts, top_k = 2048, 512, 256, 8
    fmt = api.QuantizationFormat.Q4_K
    base_in = synth.matrix(Q4_K, 2 * inter, hidden, seed=201).reshape(2 * inter, hidden // 256, 144).copy()
    base_out = synth.matrix(Q4_K, hidden, inter, seed=202).reshape(hidden, inter // 256, 144).copy()
    for blocks in (base_in, base_out):
        blocks[..., 2:4] = 0                                     # dmin = 0
        small = blocks[..., 0:2].copy().view(np.uint16) < (1 << 10)
        blocks[..., 0:2] = np.where(small, np.uint16(0x2000), blocks[..., 0:2].copy().view(np.uint16)).view(np.uint8)
    w_in = np.empty((experts,) + base_in.shape, np.uint8)
    w_out = np.empty((experts,) + base_out.shape, np.uint8)
    power = lambda e: (e // 2) % 4
    for e in range(experts):
        s = 256 * (e % 2)
        w_in[e, :inter] = np.roll(base_in[:inter], -s, axis=0)
        w_in[e, inter:] = _scaled_d(np.roll(base_in[inter:], -s, axis=0), power(e))
        w_out[e] = np.roll(np.roll(base_out, -8 * e, axis=0), -(s // 256), axis=1)
    s_in = synth.matrix(Q4_K, 2 * inter, hidden, seed=203)
    s_out = synth.matrix(Q4_K, hidden, inter, seed=204)
    x = synth.activations(tokens, hidden, seed=205, f16=True) * np.float32(2.0 ** -9)
    logits = synth.rng(206).standard_normal((tokens, experts)).astype(np.float32)

    win = api.QuantizedExpertMatrix.new(d, w_in.reshape(-1), fmt, experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, w_out.reshape(-1), fmt, experts, hidden, inter)
    sin = api.QuantizedMatrix.from_bytes(d, 2 * inter, hidden, fmt, s_in)
    sout = api.QuantizedMatrix.from_bytes(d, hidden, inter, fmt, s_out)
    moe = api.SparseMoe(d, win, wout, api.MoeRoutingPolicy(experts, top_k), shared_input=sin, shared_output=sout)
    xt = api.Tensor.from_f32(d, x.shape, api.DType.F16, x)
    got = moe.forward(xt, api.Tensor.from_f32(d, logits.shape, api.DType.F32, logits)).to_f32()
    assert d.last_operation() in ("expert_combine", "h_moe_combine", "expert_combine_shared")

    code = oracle.F16
    tile = code if tokens > 1 else 0                # one token runs on exact f32 weights
    meta = oracle.select_routes(logits, experts, top_k)
    up = oracle.round_storage(oracle.project(Q4_K, base_in.reshape(-1), 2 * inter, hidden, x, accumulate="f64",
                                             weight_round=tile, threads=8), code)
    act = oracle.expert_silu_mul(up, inter, code)
    down = oracle.round_storage(oracle.project(Q4_K, base_out.reshape(-1), hidden, inter, act, accumulate="f64",
                                               weight_round=tile, threads=8), code)
    ids = meta[:, 0].copy().view(np.uint32)
    toks = meta[:, 1].copy().view(np.uint32)
    rows = np.stack([np.float32(2.0 ** power(int(e))) * np.roll(down[t], -8 * int(e)) for e, t in zip(ids, toks)])
    sup = oracle.round_storage(oracle.project(Q4_K, s_in, 2 * inter, hidden, x, accumulate="f64", weight_round=tile,
                                              threads=8), code)
    sdown = oracle.round_storage(oracle.project(Q4_K, s_out, hidden, inter, oracle.expert_silu_mul(sup, inter, code),
                                                accumulate="f64", weight_round=tile, threads=8), code)
    want = oracle.expert_combine_shared(rows, meta, tokens, hidden, top_k, sdown, None, dtype=code)
    assert np.isfinite(want).all() and np.abs(want).max() > 1e-3
    if tokens > 1:
        assert len(np.unique(ids)) == experts       # every expert is hit
    assert rel_l2(got, want) <= 3e-3
    per_token = np.linalg.norm(got - want, axis=1) / np.linalg.norm(want, axis=1)
    assert per_token.max() <= 1e-2, int(per_token.argmax())
    # The call bench.py times at both token counts is the single-call form (fh_moe_ffn): the same bits as
    # the separate calls, and so the same distance to the host statement.
    fused = moe.forward_in_one_call(xt, api.Tensor.from_f32(d, logits.shape, api.DType.F32, logits)).to_f32()
    assert np.array_equal(fused.view(np.uint32), got.view(np.uint32))
    assert rel_l2(fused, want) <= 3e-3


# ------------------------------------------------------- decode-sized fusions

@pytest.mark.parametrize("ggml,dtype", [(Q4_K, "F32"), (Q4_K, "F16"), (Q4_K, "BF16"), (Q6_K, "F16"), (Q6_K, "F32")])
def test_fused_expert_projections_give_the_bits_of_the_separate_calls(api, d, ggml, dtype):
    # 3 tokens x top-2 over 5 experts; hidden 768 -> 2 x 256 -> 768
    experts, hidden, inter, tokens, top_k = 5, 768, 256, 3, 2
    dt = getattr(api.DType, dtype)
    code = {"F32": oracle.F32, "F16": oracle.F16, "BF16": oracle.BF16}[dtype]
    w_in = synth.matrix(ggml, experts * 2 * inter, hidden, seed=61)
    w_out = synth.matrix(ggml, experts * hidden, inter, seed=62)
    fmt = api.QuantizationFormat(ggml)
    win = api.QuantizedExpertMatrix.new(d, w_in, fmt, experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, w_out, fmt, experts, hidden, inter)
    meta = np.zeros((tokens * top_k, 3), dtype=np.uint32)
    meta[:, 0] = [1, 4, 0, 1, 2, 3]
    meta[:, 1] = [0, 0, 1, 1, 2, 2]
    meta[:, 2] = np.float32(0.5).view(np.uint32)
    mt = api.Tensor.from_bits(d, meta.shape, meta)
    x = oracle.round_storage(synth.activations(tokens, hidden, seed=63) * np.float32(2.0 ** -10), code).reshape(tokens, hidden)
    xt = api.Tensor.from_f32(d, x.shape, dt, x)

    assigned = d.expert_assign(xt, mt, top_k)
    up = d.expert_project_quantized(assigned, mt, win, hidden, experts)
    fused_up = d.expert_project_quantized(xt, mt, win, hidden, experts, form="gather")
    assert d.last_operation().endswith("_factored")
    assert np.array_equal(up.raw(), fused_up.raw())

    act = d.expert_silu_mul(up, inter)
    down = d.expert_project_quantized(act, mt, wout, inter, experts)
    fused_down = d.expert_project_quantized(up, mt, wout, inter, experts, form="silu_mul")
    assert np.array_equal(down.raw(), fused_down.raw())

    # and against the oracle end to end (f64 accumulation, storage rounding at the same points)
    m = meta.view(np.float32)
    o_up = oracle.round_storage(oracle.expert_project(ggml, w_in, experts, 2 * inter, hidden,
                                                      oracle.expert_assign(x, m), m, accumulate="f64"), code)
    o_up = o_up.reshape(tokens * top_k, 2 * inter)
    assert rel_l2(fused_up.to_f32(), o_up) <= (1e-5 if dtype == "F32" else 2e-3)
    o_act = oracle.expert_silu_mul(fused_up.to_f32(), inter, code)
    o_down = oracle.expert_project(ggml, w_out, experts, hidden, inter, o_act, m, accumulate="f64")
    assert rel_l2(fused_down.to_f32(), o_down) <= (1e-5 if dtype == "F32" else 2e-3)

    with pytest.raises(api.ShapeError):
        d.expert_project_quantized(xt, mt, wout, inter, experts, form="gather")      # K mismatch
    with pytest.raises(api.ShapeError):
        d.expert_project_quantized(assigned, mt, wout, inter, experts, form="silu_mul")


@pytest.mark.parametrize("dtype,m", [("F32", 1), ("F32", 3), ("F16", 1), ("BF16", 1)])
def test_dense_projection_with_silu_mul_input_matches_the_two_calls(api, d, dtype, m):
    n, k = 520, 1024
    dt = getattr(api.DType, dtype)
    code = {"F32": oracle.F32, "F16": oracle.F16, "BF16": oracle.BF16}[dtype]
    packed = synth.matrix(Q4_K, n, k, seed=71)
    w = api.QuantizedMatrix.from_bytes(d, n, k, api.QuantizationFormat(Q4_K), packed)
    gate_up = oracle.round_storage(synth.activations(m, 2 * k, seed=72), code).reshape(m, 2 * k)
    t = api.Tensor.from_f32(d, gate_up.shape, dt, gate_up)
    with fma_gemv(d):   # the fused form runs on the FMA kernel
        two = d.project_quantized(d.expert_silu_mul(t, k), w).tensor
    one = d.project_quantized(t, w, silu_mul=True).tensor
    assert np.array_equal(one.raw(), two.raw())
    streamed = d.project_quantized(d.expert_silu_mul(t, k), w).tensor
    assert rel_l2(streamed.to_f32(), one.to_f32()) <= (1e-5 if dtype == "F32" else 2e-3)
    want = oracle.project(Q4_K, packed, n, k, oracle.expert_silu_mul(gate_up, k, code), accumulate="f64")
    assert rel_l2(one.to_f32(), want) <= (1e-5 if dtype == "F32" else 2e-3)
    with pytest.raises(api.ShapeError):
        d.project_quantized(api.Tensor.zeros(d, (m, k), dt), w, silu_mul=True)


# one and three tokens take the per-assignment kernels; 20 and 300 the grouped kernel, whose
# gather of an expert's rows reads the token rows itself (16 and then 32 tokens a pass) and
# whose SiLU * up rows the library writes into its scratch
@pytest.mark.parametrize("tokens", [1, 3, 20, 300])
def test_sparse_moe_fused_inputs_match_the_separate_steps(api, d, tokens):
    experts, hidden, inter, top_k = 16, 512, 256, 4
    fmt = api.QuantizationFormat(Q4_K)
    win = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * 2 * inter, hidden, seed=81), fmt,
                                        experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * hidden, inter, seed=82), fmt,
                                         experts, hidden, inter)
    moe = api.SparseMoe(d, win, wout, api.MoeRoutingPolicy(experts, top_k))
    x = synth.activations(tokens, hidden, seed=83, f16=True) * np.float32(2.0 ** -4)
    logits = synth.rng(84).standard_normal((tokens, experts)).astype(np.float32)
    xt = api.Tensor.from_f32(d, x.shape, api.DType.F16, x)
    lt = api.Tensor.from_f32(d, logits.shape, api.DType.F32, logits)
    fused = moe.forward(xt, lt)
    fused_op = d.last_operation()
    moe.fuse_inputs = False
    separate = moe.forward(xt, lt)
    assert np.array_equal(fused.raw(), separate.raw())
    assert np.abs(fused.to_f32()).max() > 1e-3
    meta = d.moe_route(lt, None, moe.routing)
    d.expert_project_quantized(xt, meta, win, hidden, experts, form="gather")
    assert d.last_operation() == ("expert_project_q4_k_grouped_mfma" if tokens * top_k >= 32 else "expert_project_q4_k_factored")


@pytest.mark.parametrize("dtype", ["F16", "BF16"])
def test_grouped_input_forms_when_an_experts_rows_do_not_fit_lds(api, d, dtype):
    # 32 rows of 2816 halves are more than the kernel's LDS: the library writes the gathered
    # and the activated rows out itself and the result is still that of the separate steps
    experts, hidden, inter, top_k, tokens = 4, 2816, 2816, 2, 40
    fmt = api.QuantizationFormat(Q4_K)
    win = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * 2 * inter, hidden, seed=85), fmt,
                                        experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * hidden, inter, seed=86), fmt,
                                         experts, hidden, inter)
    moe = api.SparseMoe(d, win, wout, api.MoeRoutingPolicy(experts, top_k))
    dt = getattr(api.DType, dtype)
    x = synth.activations(tokens, hidden, seed=87, f16=True) * np.float32(2.0 ** -5)
    logits = synth.rng(88).standard_normal((tokens, experts)).astype(np.float32)
    xt = api.Tensor.from_f32(d, x.shape, dt, x)
    lt = api.Tensor.from_f32(d, logits.shape, api.DType.F32, logits)
    fused = moe.forward(xt, lt)
    moe.fuse_inputs = False
    separate = moe.forward(xt, lt)
    assert np.array_equal(fused.raw(), separate.raw())
    assert np.abs(fused.to_f32()).max() > 1e-3


def _shared_case(api, d, dtype, tokens, seed):
    experts, hidden, inter, top_k = 16, 512, 256, 4
    fmt = api.QuantizationFormat(Q4_K)
    packed = {"win": synth.matrix(Q4_K, experts * 2 * inter, hidden, seed=seed),
              "wout": synth.matrix(Q4_K, experts * hidden, inter, seed=seed + 1),
              "sin": synth.matrix(Q4_K, 2 * inter, hidden, seed=seed + 2),
              "sout": synth.matrix(Q4_K, hidden, inter, seed=seed + 3)}
    w = {"win": api.QuantizedExpertMatrix.new(d, packed["win"], fmt, experts, 2 * inter, hidden),
         "wout": api.QuantizedExpertMatrix.new(d, packed["wout"], fmt, experts, hidden, inter),
         "sin": api.QuantizedMatrix.from_bytes(d, 2 * inter, hidden, fmt, packed["sin"]),
         "sout": api.QuantizedMatrix.from_bytes(d, hidden, inter, fmt, packed["sout"])}
    dt = getattr(api.DType, dtype)
    x = synth.activations(tokens, hidden, seed=seed + 4, f16=True) * np.float32(2.0 ** -6)
    logits = synth.rng(seed + 5).standard_normal((tokens, experts)).astype(np.float32)
    xt = api.Tensor.from_f32(d, x.shape, dt, x)
    lt = api.Tensor.from_f32(d, logits.shape, api.DType.F32, logits)
    return (experts, hidden, inter, top_k), packed, w, x, logits, xt, lt


@pytest.mark.parametrize("dtype", ["F32", "F16", "BF16"])
@pytest.mark.parametrize("tokens", [1, 3])
def test_shared_expert_rides_in_the_routed_launch(api, d, dtype, tokens):
    (experts, hidden, inter, top_k), _, w, _, _, xt, lt = _shared_case(api, d, dtype, tokens, 171)
    meta = d.moe_route(lt, None, api.MoeRoutingPolicy(experts, top_k))
    d.set_tuning("gemm_min_rows", 1000)  # the dense reference calls below take the per-row kernel too
    try:
        up, shared_up = d.expert_project_with_shared(xt, meta, w["win"], w["sin"], tokens, "gather")
        assert d.last_operation() == "expert_project_q4_k_factored"
        assert np.array_equal(up.raw(), d.expert_project_quantized(xt, meta, w["win"], hidden, experts,
                                                                   form="gather").raw())
        with fma_gemv(d):
            assert np.array_equal(shared_up.raw(), d.project_quantized(xt, w["sin"]).tensor.raw())
        down, shared_down = d.expert_project_with_shared(up, meta, w["wout"], w["sout"], tokens, "silu_mul",
                                                         shared_input=shared_up)
        assert np.array_equal(down.raw(), d.expert_project_quantized(up, meta, w["wout"], inter, experts,
                                                                     form="silu_mul").raw())
        assert np.array_equal(shared_down.raw(), d.project_quantized(shared_up, w["sout"], silu_mul=True).tensor.raw())
        assert np.abs(shared_down.to_f32()).max() > 1e-4 and np.abs(down.to_f32()).max() > 1e-4
    finally:
        d.set_tuning("gemm_min_rows", 2)


def test_shared_expert_projection_rejects_what_it_cannot_run(api, d):
    (experts, hidden, inter, top_k), packed, w, _, _, xt, lt = _shared_case(api, d, "F16", 2, 181)
    meta = d.moe_route(lt, None, api.MoeRoutingPolicy(experts, top_k))
    fmt = api.QuantizationFormat(Q4_K)
    with pytest.raises(api.ShapeError):   # a shared matrix of another shape
        d.expert_project_with_shared(xt, meta, w["win"], w["sout"], 2, "gather")
    with pytest.raises(api.ShapeError):   # the SiLU form needs the shared expert's own rows
        up, _ = d.expert_project_with_shared(xt, meta, w["win"], w["sin"], 2, "gather")
        d.expert_project_with_shared(up, meta, w["wout"], w["sout"], 2, "silu_mul")
    q6 = api.QuantizedMatrix.from_bytes(d, 2 * inter, hidden, api.QuantizationFormat(Q6_K),
                                        synth.matrix(Q6_K, 2 * inter, hidden, seed=182))
    with pytest.raises(api.ShapeError):   # another format
        d.expert_project_with_shared(xt, meta, w["win"], q6, 2, "gather")
    # the C entry point itself: the rows form has no shared variant, and outputs must not alias
    from ferrum_amd.api import _lib
    import ctypes
    up = api.Tensor.zeros(d, (2 * top_k, 2 * inter), api.DType.F16)
    sup = api.Tensor.zeros(d, (2, 2 * inter), api.DType.F16)
    xv, mv, ov, sv = xt._view(), meta._view(), up._view(), sup._view()
    call = lambda form, out, shared_out: _lib.fh_expert_project_with_shared(
        d._handle, w["win"]._handle, w["sin"]._handle, ctypes.byref(xv), 2, form, 2 * top_k, ctypes.byref(mv), None,
        ctypes.byref(out), ctypes.byref(shared_out))
    last_error = lambda: _lib.fh_last_error().decode()
    assert call(0, ov, sv) != 0 and "gathered or the SiLU" in last_error()
    assert call(1, ov, ov) != 0 and "aliases" in last_error()
    assert call(1, ov, sv) == 0


@pytest.mark.parametrize("tokens,gated", [(1, False), (3, True), (20, False), (300, True)])
def test_sparse_moe_with_a_shared_expert(api, d, tokens, gated):
    # one and three tokens: the shared expert's rows are batch entries of the per-assignment
    # launches; 20 and 300: token groups (of 16, then of 32) of the grouped kernel
    (experts, hidden, inter, top_k), packed, w, x, logits, xt, lt = _shared_case(api, d, "F16", tokens, 191)
    moe = api.SparseMoe(d, w["win"], w["wout"], api.MoeRoutingPolicy(experts, top_k),
                        shared_input=w["sin"], shared_output=w["sout"])
    gate = None
    gate_values = None
    if gated:
        gate_values = (0.25 + 0.5 * synth.rng(192).random(tokens)).astype(np.float32)
        gate = api.Tensor.from_f32(d, (tokens,), api.DType.F32, gate_values)
    got = moe.forward(xt, lt, shared_gate=gate)
    moe.fuse_inputs = False
    separate = moe.forward(xt, lt, shared_gate=gate)
    if tokens == 1:
        assert np.array_equal(got.raw(), separate.raw())   # every launch is the per-row kernel either way
    # the whole FFN against the host statement, f16 storage at every step
    code = oracle.F16
    xr = oracle.round_storage(x, code)
    meta = oracle.select_routes(logits, experts, top_k)
    up = oracle.round_storage(oracle.expert_project(Q4_K, packed["win"], experts, 2 * inter, hidden,
                                                    oracle.expert_assign(xr, meta), meta), code)
    down = oracle.round_storage(oracle.expert_project(Q4_K, packed["wout"], experts, hidden, inter,
                                                      oracle.expert_silu_mul(up, inter, code), meta), code)
    sup = oracle.round_storage(oracle.project(Q4_K, packed["sin"], 2 * inter, hidden, xr), code)
    sdown = oracle.round_storage(oracle.project(Q4_K, packed["sout"], hidden, inter,
                                                oracle.expert_silu_mul(sup, inter, code)), code)
    want = oracle.expert_combine_shared(down, meta, tokens, hidden, top_k, sdown, gate_values, dtype=code)
    assert np.isfinite(want).all() and np.abs(want).max() > 1e-3
    for result in (got, separate):
        assert rel_l2(result.to_f32(), want) <= 3e-3


@pytest.mark.parametrize("dtype,shared", [("F16", True), ("F16", False), ("F32", False)])
def test_chunked_forward_gives_the_bits_of_the_unchunked_one(api, d, dtype, shared):
    # the reference's chunk test (src/nn/moe.rs:467-520) compares two ways of assembling
    # the chunks; here every chunk's combine writes its rows of the one output, and the
    # comparison is with the pass that was not cut at all.  Chunks of 64 tokens leave a
    # last one of 44: every chunk has enough assignments for the kernels the whole batch
    # takes (grouped tiles for f16, the per-assignment GEMV for f32), whose rows do not
    # depend on their neighbours.
    tokens = 300
    (experts, hidden, inter, top_k), packed, w, x, logits, xt, lt = _shared_case(api, d, dtype, tokens, 201)
    kw = dict(shared_input=w["sin"], shared_output=w["sout"]) if shared else {}
    moe = api.SparseMoe(d, w["win"], w["wout"], api.MoeRoutingPolicy(experts, top_k), **kw)
    gate = api.Tensor.from_f32(d, (tokens,), api.DType.F32,
                               (0.25 + 0.5 * synth.rng(202).random(tokens)).astype(np.float32)) if shared else None
    before = d.moe_routing_temporary_limit()
    assert before == 128 << 20       # src/metal/legacy.rs:95
    whole = moe.forward(xt, lt, shared_gate=gate)
    stats = moe.take_stats()
    assert stats.assignments == tokens * top_k and not stats.active_experts_known
    assert stats.peak_temporary_bytes == moe.temporary_bytes(tokens, xt.dtype)
    per_token = moe.temporary_bytes(1, xt.dtype)
    assert per_token == ((2 * hidden + 3 * inter) * xt.dtype.size_bytes() + 12) * top_k \
        + (experts + hidden) * xt.dtype.size_bytes()
    try:
        d.set_moe_routing_temporary_limit(64 * per_token + per_token // 2)
        cut = moe.forward(xt, lt, shared_gate=gate)
        cut_stats = moe.take_stats()
        d.set_moe_routing_temporary_limit(1)          # one token per chunk: the per-assignment kernels
        single = moe.forward(xt, lt, shared_gate=gate)
        single_stats = moe.take_stats()
        with pytest.raises(api.ParameterError):
            d.set_moe_routing_temporary_limit(0)
        with d.execution():
            with pytest.raises(api.ParameterError):
                d.set_moe_routing_temporary_limit(1 << 20)
    finally:
        d.set_moe_routing_temporary_limit(before)
    assert np.array_equal(cut.raw(), whole.raw())
    assert cut_stats.assignments == tokens * top_k
    assert cut_stats.peak_temporary_bytes == 64 * per_token <= 64 * per_token + per_token // 2
    assert single_stats.peak_temporary_bytes == per_token and single_stats.assignments == tokens * top_k
    assert rel_l2(single.to_f32(), whole.to_f32()) <= (1e-6 if dtype == "F32" else 2e-3)
    assert moe.take_stats() == api.MoeStats()


@pytest.mark.parametrize("dtype,tokens,shared,gated", [("F16", 1, True, True), ("F16", 3, True, False), ("F16", 300, True, True),
                                                       ("F16", 20, False, False), ("F32", 5, True, True), ("F32", 40, True, False),
                                                       ("F32", 40, False, False), ("BF16", 70, True, False)])
def test_the_ffn_in_one_call_gives_the_bits_of_the_separate_calls(api, d, dtype, tokens, shared, gated):
    # fh_moe_ffn enqueues the steps SparseMoe.forward makes one by one (per-assignment and grouped
    # kernels, the shared expert riding or apart, f32 rows through assign / silu_mul launches of
    # their own), with its temporaries in the library's workspace; also cut into chunks, and
    # recorded into an execution once the workspace has its size
    (experts, hidden, inter, top_k), packed, w, x, logits, xt, lt = _shared_case(api, d, dtype, tokens, 301)
    kw = dict(shared_input=w["sin"], shared_output=w["sout"]) if shared else {}
    moe = api.SparseMoe(d, w["win"], w["wout"], api.MoeRoutingPolicy(experts, top_k), **kw)
    gate = api.Tensor.from_f32(d, (tokens,), api.DType.F32,
                               (0.25 + 0.5 * synth.rng(302).random(tokens)).astype(np.float32)) if gated else None
    want = moe.forward(xt, lt, shared_gate=gate)
    got = moe.forward_in_one_call(xt, lt, shared_gate=gate)
    assert np.abs(want.to_f32()).max() > 1e-3
    assert np.array_equal(got.raw(), want.raw())
    out = api.Tensor.zeros(d, (tokens, hidden), xt.dtype)
    with d.execution() as ex:
        moe.forward_in_one_call(xt, lt, shared_gate=gate, out=out)
    for _ in range(2):
        ex.graph.launch()
        d.synchronize()
        assert np.array_equal(out.raw(), want.raw())
        api._check(api._lib.fh_buffer_fill_zero(out.buffer._handle, 0, out.byte_size()))
        d.synchronize()
    if tokens >= 40:
        before = d.moe_routing_temporary_limit()
        try:
            d.set_moe_routing_temporary_limit(16 * moe.temporary_bytes(1, xt.dtype))
            cut = moe.forward_in_one_call(xt, lt, shared_gate=gate)
            stepwise = moe.forward(xt, lt, shared_gate=gate)
        finally:
            d.set_moe_routing_temporary_limit(before)
        assert np.array_equal(cut.raw(), stepwise.raw())
    with pytest.raises(api.ShapeError):
        moe.forward_in_one_call(xt, api.Tensor.zeros(d, (tokens, experts + 1), api.DType.F32))


@pytest.mark.parametrize("logit_dtype", ["BF16", "F16"])
def test_chunks_of_16_bit_logits_over_an_odd_number_of_experts(api, d, logit_dtype):
    # three tokens a chunk over 7 experts: the second chunk's logits start 42 bytes in, a
    # 2-byte boundary that is not a 4-byte one.  Both the chunked step-by-step pass and the
    # chunked single call give the bits of the pass that was not cut.
    experts, hidden, inter, top_k, tokens = 7, 512, 256, 2, 10
    fmt = api.QuantizationFormat(Q4_K)
    win = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * 2 * inter, hidden, seed=311), fmt,
                                        experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * hidden, inter, seed=312), fmt,
                                         experts, hidden, inter)
    moe = api.SparseMoe(d, win, wout, api.MoeRoutingPolicy(experts, top_k))
    x = synth.activations(tokens, hidden, seed=313, f16=True) * np.float32(2.0 ** -5)
    logits = synth.rng(314).standard_normal((tokens, experts)).astype(np.float32)
    xt = api.Tensor.from_f32(d, x.shape, api.DType.F16, x)
    lt = api.Tensor.from_f32(d, logits.shape, getattr(api.DType, logit_dtype), logits)
    whole = moe.forward(xt, lt)
    assert np.abs(whole.to_f32()).max() > 1e-3
    moe.take_stats()
    before = d.moe_routing_temporary_limit()
    try:
        d.set_moe_routing_temporary_limit(3 * moe.temporary_bytes(1, xt.dtype))
        cut = moe.forward(xt, lt)
        assert moe.take_stats().peak_temporary_bytes == 3 * moe.temporary_bytes(1, xt.dtype)
        cut_one_call = moe.forward_in_one_call(xt, lt)
    finally:
        d.set_moe_routing_temporary_limit(before)
    # fewer than 32 assignments either way: every row comes from the per-assignment kernel
    assert np.array_equal(cut.raw(), whole.raw())
    assert np.array_equal(cut_one_call.raw(), whole.raw())


@pytest.mark.parametrize("min_rows", [2, 1000])
def test_one_call_ffn_when_the_shared_expert_runs_apart_from_a_grouped_projection(api, d, min_rows):
    # 32 rows of 2816 halves do not fit the grouped kernel's LDS, so the shared expert's matrices
    # run as dense calls of their own after each grouped projection (on the tile kernel, or on
    # the per-row kernel under a high kernel-choice floor).  Those calls may use the scratch the
    # grouping lists lie in: the second projection groups the records again, and the single call
    # gives the bits of the separate calls.
    experts, hidden, inter, top_k, tokens = 4, 2816, 2816, 2, 40
    fmt = api.QuantizationFormat(Q4_K)
    win = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * 2 * inter, hidden, seed=321), fmt,
                                        experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * hidden, inter, seed=322), fmt,
                                         experts, hidden, inter)
    sin = api.QuantizedMatrix.from_bytes(d, 2 * inter, hidden, fmt, synth.matrix(Q4_K, 2 * inter, hidden, seed=323))
    sout = api.QuantizedMatrix.from_bytes(d, hidden, inter, fmt, synth.matrix(Q4_K, hidden, inter, seed=324))
    moe = api.SparseMoe(d, win, wout, api.MoeRoutingPolicy(experts, top_k), shared_input=sin, shared_output=sout)
    x = synth.activations(tokens, hidden, seed=325, f16=True) * np.float32(2.0 ** -5)
    logits = synth.rng(326).standard_normal((tokens, experts)).astype(np.float32)
    xt = api.Tensor.from_f32(d, x.shape, api.DType.F16, x)
    lt = api.Tensor.from_f32(d, logits.shape, api.DType.F32, logits)
    before = d.get_tuning("gemm_min_rows")
    d.set_tuning("gemm_min_rows", min_rows)
    try:
        want = moe.forward(xt, lt)
        got = moe.forward_in_one_call(xt, lt)
        again = moe.forward_in_one_call(xt, lt)
    finally:
        d.set_tuning("gemm_min_rows", before)
    assert np.abs(want.to_f32()).max() > 1e-3
    assert np.array_equal(got.raw(), want.raw())
    assert np.array_equal(again.raw(), want.raw())


@pytest.mark.parametrize("ggml,inter,top_k,tokens,shared,dtype", [
    (Q4_K, 512, 8, 1, True, "F16"), (Q4_K, 512, 8, 1, True, "BF16"), (Q4_K, 512, 8, 1, False, "F32"),
    (Q6_K, 768, 4, 1, True, "F16"), (Q6_K, 1024, 3, 1, False, "F16"), (synth.Q5_K, 1536, 2, 1, True, "F16"),
    (23, 2048, 2, 1, True, "F16"), (8, 512, 6, 1, True, "BF16"), (Q4_K, 256, 16, 1, True, "F16")])
def test_few_tokens_fold_the_weighted_sum_into_the_down_projection(api, d, ggml, inter, top_k, tokens, shared, dtype):
    # fh_moe_ffn with one token: route, gate|up, then one launch that multiplies every entry
    # of a token (top_k routed experts, the shared one) and adds them with expert_combine's
    # rounding.  Against the separate launches: the same bits, for every format, for rows of 1 - 8
    # super-blocks (all lane layouts of the kernel), with 17 entries (one wave takes two), without a
    # shared expert and with a gate on it.
    experts, hidden = 24, 512
    fmt_in, fmt_out = api.QuantizationFormat(Q4_K), api.QuantizationFormat(ggml)
    win = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * 2 * inter, hidden, seed=401), fmt_in,
                                        experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, synth.matrix(ggml, experts * hidden, inter, seed=402), fmt_out,
                                         experts, hidden, inter)
    kw = {}
    if shared:
        kw = dict(shared_input=api.QuantizedMatrix.from_bytes(d, 2 * inter, hidden, fmt_in,
                                                              synth.matrix(Q4_K, 2 * inter, hidden, seed=403)),
                  shared_output=api.QuantizedMatrix.from_bytes(d, hidden, inter, fmt_out,
                                                               synth.matrix(ggml, hidden, inter, seed=404)))
    moe = api.SparseMoe(d, win, wout, api.MoeRoutingPolicy(experts, top_k), **kw)
    dt = getattr(api.DType, dtype)
    x = synth.activations(tokens, hidden, seed=405, f16=True) * np.float32(2.0 ** -5)
    xt = api.Tensor.from_f32(d, x.shape, dt, x)
    lt = api.Tensor.from_f32(d, (tokens, experts), api.DType.F32,
                             synth.rng(406).standard_normal((tokens, experts)).astype(np.float32))
    gate = api.Tensor.from_f32(d, (tokens,), api.DType.F32,
                               (0.25 + 0.5 * synth.rng(407).random(tokens)).astype(np.float32)) if shared else None
    want = moe.forward(xt, lt, shared_gate=gate)
    got = moe.forward_in_one_call(xt, lt, shared_gate=gate)
    assert "combine" in d.last_operation() and "expert_project" in d.last_operation()
    assert np.abs(want.to_f32()).max() > 1e-4
    assert np.array_equal(got.raw(), want.raw())
    d.set_tuning("moe_fold_combine", 0)
    try:
        apart = moe.forward_in_one_call(xt, lt, shared_gate=gate)
        assert "expert_project" not in d.last_operation()
    finally:
        d.set_tuning("moe_fold_combine", 1)
    assert np.array_equal(apart.raw(), want.raw())


@pytest.mark.parametrize("ggml,hidden,experts,top_k,shared,dtype,policy", [
    (Q4_K, 2048, 256, 8, True, "F16", "softmax"), (Q4_K, 512, 24, 4, False, "F32", "softmax"),
    (Q6_K, 1024, 64, 6, True, "BF16", "sigmoid"), (synth.Q5_K, 256, 130, 2, True, "F16", "bias"),
    (23, 4096, 100, 8, False, "F16", "ties"), (8, 6144, 40, 16, True, "F16", "scaled"),
    (Q4_K, 2816, 7, 7, True, "F16", "softmax")])
def test_one_token_is_routed_by_its_gate_up_launch(api, d, ggml, hidden, experts, top_k, shared, dtype, policy):
    # fh_moe_ffn with one token: no moe_route launch; every workgroup of the gate|up launch routes
    # the token itself and workgroup 0 publishes the records the down projection reads.  The bits
    # of the three launches (tuning moe_fold_route 0) and of the separate calls, for every input
    # format and lane layout (rows of 1 - 24 super-blocks), routers of 7 - 256 experts, the sigmoid
    # policy, a selection bias, tied logits, a scaling factor and an epsilon.
    inter = 256
    fmt = api.QuantizationFormat(ggml)
    win = api.QuantizedExpertMatrix.new(d, synth.matrix(ggml, experts * 2 * inter, hidden, seed=501), fmt,
                                        experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, synth.matrix(ggml, experts * hidden, inter, seed=502), fmt,
                                         experts, hidden, inter)
    kw = {}
    if shared:
        kw = dict(shared_input=api.QuantizedMatrix.from_bytes(d, 2 * inter, hidden, fmt,
                                                              synth.matrix(ggml, 2 * inter, hidden, seed=503)),
                  shared_output=api.QuantizedMatrix.from_bytes(d, hidden, inter, fmt,
                                                               synth.matrix(ggml, hidden, inter, seed=504)))
    routing = api.MoeRoutingPolicy(experts, top_k)
    logits = synth.rng(506).standard_normal((1, experts)).astype(np.float32)
    if policy == "sigmoid":
        routing = api.MoeRoutingPolicy(experts, top_k, api.MoeScoringFunction.Sigmoid, True, 1e-6, 1.0)
    elif policy == "bias":
        routing = api.MoeRoutingPolicy(experts, top_k, api.MoeScoringFunction.Softmax, True, 0.0, 1.0, True)
        kw["selection_bias"] = api.Tensor.from_f32(d, (experts,), api.DType.F32,
                                                   synth.rng(508).standard_normal(experts).astype(np.float32) * 0.1)
    elif policy == "ties":
        logits = np.round(logits * 2) / 2   # many equal logits: the lower expert id wins
    elif policy == "scaled":
        routing = api.MoeRoutingPolicy(experts, top_k, api.MoeScoringFunction.Softmax, False, 0.0, 2.5)
    moe = api.SparseMoe(d, win, wout, routing, **kw)
    dt = getattr(api.DType, dtype)
    x = synth.activations(1, hidden, seed=505, f16=True) * np.float32(2.0 ** -5)
    xt = api.Tensor.from_f32(d, x.shape, dt, x)
    lt = api.Tensor.from_f32(d, (1, experts), api.DType.F32, logits)
    gate = api.Tensor.from_f32(d, (1,), api.DType.F32, np.array([0.625], np.float32)) if shared else None
    want = moe.forward(xt, lt, shared_gate=gate)
    assert np.abs(want.to_f32()).max() > 1e-5
    d.set_tuning("moe_fold_route", 1)
    got = moe.forward_in_one_call(xt, lt, shared_gate=gate)
    assert np.array_equal(got.raw(), want.raw())
    again = moe.forward_in_one_call(xt, lt, shared_gate=gate)
    assert np.array_equal(again.raw(), want.raw())
    d.set_tuning("moe_fold_route", 0)
    try:
        apart = moe.forward_in_one_call(xt, lt, shared_gate=gate)
    finally:
        d.set_tuning("moe_fold_route", 1)
    assert np.array_equal(apart.raw(), want.raw())


def test_shared_expert_runs_apart_when_an_experts_rows_do_not_fit_lds(api, d):
    # 32 rows of 2816 halves are more than the grouped kernel's LDS: the routed rows are staged and
    # the shared expert takes the dense kernels, which is what the separate calls do, bit for bit
    experts, hidden, inter, top_k, tokens = 4, 2816, 2816, 2, 40
    fmt = api.QuantizationFormat(Q4_K)
    win = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * 2 * inter, hidden, seed=85), fmt,
                                        experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * hidden, inter, seed=86), fmt,
                                         experts, hidden, inter)
    sin = api.QuantizedMatrix.from_bytes(d, 2 * inter, hidden, fmt, synth.matrix(Q4_K, 2 * inter, hidden, seed=89))
    sout = api.QuantizedMatrix.from_bytes(d, hidden, inter, fmt, synth.matrix(Q4_K, hidden, inter, seed=90))
    moe = api.SparseMoe(d, win, wout, api.MoeRoutingPolicy(experts, top_k), shared_input=sin, shared_output=sout)
    x = synth.activations(tokens, hidden, seed=87, f16=True) * np.float32(2.0 ** -5)
    logits = synth.rng(88).standard_normal((tokens, experts)).astype(np.float32)
    xt = api.Tensor.from_f32(d, x.shape, api.DType.F16, x)
    lt = api.Tensor.from_f32(d, logits.shape, api.DType.F32, logits)
    riding = moe.forward(xt, lt)
    moe.fuse_inputs = False
    apart = moe.forward(xt, lt)
    assert np.array_equal(riding.raw(), apart.raw())
    assert np.abs(riding.to_f32()).max() > 1e-3


# ------------------------------------------------- the hybrid engine's router and combine

@pytest.mark.parametrize("sigmoid,norm,shared_gate", [(True, True, False), (False, True, True), (True, False, True)])
def test_ranked_router_replays_the_hybrid_engines_test(api, d, sigmoid, norm, shared_gate):
    # src/hybrid/engine.rs:4949-5041: 256 experts, top-6, hidden 2048, three tokens; ids exact,
    # weights within 1e-5, gate within 1e-4 (the reference's tolerances)
    experts, top_k, hidden, tokens = 256, 6, 2048, 3
    rng = synth.rng(151)
    logits = (rng.standard_normal((tokens, experts)) * 3).astype(np.float32)
    x = rng.standard_normal((tokens, hidden)).astype(np.float32)
    w = rng.standard_normal(hidden).astype(np.float32)
    policy = api.MoeRoutingPolicy(experts, top_k, scoring_function=api.MoeScoringFunction.Sigmoid if sigmoid
                                  else api.MoeScoringFunction.Softmax, normalize_top_k_prob=norm)
    lt = api.Tensor.from_f32(d, logits.shape, api.DType.F32, logits)
    xt = api.Tensor.from_f32(d, x.shape, api.DType.F32, x)
    wt = api.Tensor.from_f32(d, w.shape, api.DType.F32, w)
    meta, gate = d.moe_route_ranked(lt, policy, xt if shared_gate else None, wt if shared_gate else None,
                                    want_gate=True)
    assert d.last_operation() == "h_moe_route"
    got = meta.to_f32()
    want = oracle.select_routes_ranked(logits, experts, top_k, sigmoid=sigmoid, normalize=norm)
    assert np.array_equal(bits(got[:, :2]), bits(want[:, :2]))
    assert np.abs(got[:, 2] - want[:, 2]).max() < 1e-5
    want_gate = oracle.shared_gate(x, w) if shared_gate else np.ones(tokens, np.float32)
    assert np.abs(gate.to_f32() - want_gate).max() < 1e-4


def test_hybrid_decode_chain_route_project_combine_with_shared_expert(api, d):
    # f32 model, one token: ranked route -> gate|up by gathered rows -> down with SiLU*up ->
    # combine + gate * shared expert, against the oracle's same chain
    experts, top_k, hidden, inter, tokens = 32, 4, 512, 256, 2
    fmt = api.QuantizationFormat(Q4_K)
    w_in = synth.matrix(Q4_K, experts * 2 * inter, hidden, seed=161)
    w_out = synth.matrix(Q4_K, experts * hidden, inter, seed=162)
    s_in = synth.matrix(Q4_K, 2 * inter, hidden, seed=163)
    s_out = synth.matrix(Q4_K, hidden, inter, seed=164)
    win = api.QuantizedExpertMatrix.new(d, w_in, fmt, experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(d, w_out, fmt, experts, hidden, inter)
    sin = api.QuantizedMatrix.from_bytes(d, 2 * inter, hidden, fmt, s_in)
    sout = api.QuantizedMatrix.from_bytes(d, hidden, inter, fmt, s_out)
    rng = synth.rng(165)
    x = (rng.standard_normal((tokens, hidden)) * 2.0 ** -6).astype(np.float32)
    logits = rng.standard_normal((tokens, experts)).astype(np.float32)
    gate_w = rng.standard_normal(hidden).astype(np.float32)
    f32 = api.DType.F32
    xt = api.Tensor.from_f32(d, x.shape, f32, x)
    policy = api.MoeRoutingPolicy(experts, top_k)
    meta, gate = d.moe_route_ranked(api.Tensor.from_f32(d, logits.shape, f32, logits), policy, xt,
                                    api.Tensor.from_f32(d, gate_w.shape, f32, gate_w))
    up = d.expert_project_quantized(xt, meta, win, hidden, experts, form="gather")
    down = d.expert_project_quantized(up, meta, wout, inter, experts, form="silu_mul")
    shared = d.project_quantized(d.project_quantized(xt, sin).tensor, sout, silu_mul=True).tensor
    out = d.expert_combine_shared(down, meta, tokens, hidden, top_k, shared, gate)
    assert d.last_operation() == "h_moe_combine"

    m = oracle.select_routes_ranked(logits, experts, top_k)
    assert np.array_equal(bits(meta.to_f32()[:, :2]), bits(m[:, :2]))
    o_up = oracle.expert_project(Q4_K, w_in, experts, 2 * inter, hidden, oracle.expert_assign(x, m), m, accumulate="f64")
    o_down = oracle.expert_project(Q4_K, w_out, experts, hidden, inter, oracle.expert_silu_mul(o_up, inter), m,
                                   accumulate="f64")
    o_sh = oracle.project(Q4_K, s_out, hidden, inter,
                          oracle.expert_silu_mul(oracle.project(Q4_K, s_in, 2 * inter, hidden, x, accumulate="f64"), inter),
                          accumulate="f64")
    want = oracle.expert_combine_shared(o_down, m, tokens, hidden, top_k, o_sh, oracle.shared_gate(x, gate_w))
    assert np.abs(want).max() > 1e-3
    assert rel_l2(out.to_f32(), want) <= 2e-5
    # without a gate tensor the shared expert is added whole
    whole = d.expert_combine_shared(down, meta, tokens, hidden, top_k, shared).to_f32()
    plain = d.expert_combine(down, meta, tokens, hidden, top_k).to_f32()
    assert np.allclose(whole, plain + shared.to_f32(), rtol=1e-6, atol=1e-7)


def test_f32_assignments_join_the_grouped_projection_on_request(api, d):
    # gemm_f32_min_rows opts f32 activations into the f16 tiles (the hybrid engine's prompt
    # path); without it every f32 assignment keeps exact f32 weights
    experts, rows, cols, a = 6, 64, 512, 48
    packed = synth.matrix(Q4_K, experts * rows, cols, seed=171)
    w = api.QuantizedExpertMatrix.new(d, packed, api.QuantizationFormat(Q4_K), experts, rows, cols)
    ids = synth.rng(172).integers(0, experts, a)
    meta = _routing_rows(ids)
    x = synth.activations(a, cols, seed=173)
    xt = api.Tensor.from_f32(d, x.shape, api.DType.F32, x)
    mt = api.Tensor.from_bits(d, meta.shape, meta)
    exact = d.expert_project_quantized(xt, mt, w, cols, experts)
    assert d.last_operation() == "expert_project_q4_k_factored"
    full = oracle.expert_project(Q4_K, packed, experts, rows, cols, x, meta.view(np.float32), accumulate="f64")
    assert_matmul_parity(exact.to_f32(), full, "exact f32 assignments")
    d.set_tuning("gemm_f32_min_rows", 5)
    try:
        tiled = d.expert_project_quantized(xt, mt, w, cols, experts)
        assert d.last_operation() == "expert_project_q4_k_grouped_mfma" and tiled.dtype == api.DType.F32
    finally:
        d.set_tuning("gemm_f32_min_rows", 0)
    want = oracle.expert_project(Q4_K, packed, experts, rows, cols, oracle.round_storage(x, oracle.F16).reshape(a, cols),
                                 meta.view(np.float32), weight_round=oracle.F16, accumulate="f64")
    assert_matmul_parity(tiled.to_f32(), want, "f32 assignments through the f16 tiles")
