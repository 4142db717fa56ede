"""GPU parity of the hybrid engine's routed FFN in its own data layout (ids and weights as
plain arrays; HybridModel::moe_ffn, src/hybrid/engine.rs:2881-3080), through the C ABI.

Integer stages (the route map) are bit-exact against the oracle's restatement of h_moe_map;
projections are held to the matmul bars; the reference's own expert tests use |err| <= 5e-3
max|ref| (src/hybrid/iq_tests.rs:1289-1298) and its router test 1e-5 / 1e-4
(src/hybrid/engine.rs:5025-5040).
"""
import numpy as np
import pytest

import oracle
from helpers import assert_matmul_parity, bits, fma_gemv, rel_l2
from ferrum_amd import synth

pytestmark = pytest.mark.gpu

Q4_K, IQ4_XS = 12, 23


@pytest.fixture(scope="module")
def api():
    from ferrum_amd import api as module
    return module


@pytest.fixture(scope="module")
def d(api):
    return api.Device.new()


def u32(t):
    return t.to_f32().view(np.uint32).reshape(-1)


def carrier(api, d, words):
    words = np.ascontiguousarray(words, dtype=np.uint32)
    return api.Tensor.from_bits(d, words.shape, words)


@pytest.mark.parametrize("experts,routes", [(4, 1), (8, 40), (256, 8), (256, 4096), (60, 1000), (1024, 5000), (1, 70)])
def test_route_map_is_bit_exact(api, d, experts, routes):
    rng = synth.rng(401, routes)
    ids = rng.integers(0, experts, routes).astype(np.uint32)
    if experts > 4 and routes > 10:
        ids[ids == 3] = 5                       # an empty expert
        ids[routes // 2] = experts + 7          # not an expert: left out of the map
    offsets, order, position = d.hybrid_moe_map(carrier(api, d, ids), experts)
    assert d.last_operation() == "h_moe_map"
    want_offsets, want_order, want_position = oracle.moe_map(ids, experts)
    assert np.array_equal(u32(offsets), want_offsets)
    placed = int(want_offsets[-1])
    assert np.array_equal(u32(order)[:placed], want_order[:placed])
    valid = ids < experts
    assert np.array_equal(u32(position)[valid], want_position[valid])


def test_router_writes_ids_weights_and_gate(api, d):
    # the reference's router test (src/hybrid/engine.rs:4949-5041) in the engine's own layout
    experts, top_k, hidden, tokens = 256, 6, 2048, 3
    rng = synth.rng(402)
    logits = (rng.standard_normal((tokens, experts)) * 3).astype(np.float32)
    x = rng.standard_normal((tokens, hidden)).astype(np.float32)
    w = rng.standard_normal(hidden).astype(np.float32)
    f32 = api.DType.F32
    policy = api.MoeRoutingPolicy(experts, top_k, normalize_top_k_prob=True)
    ids, weights, gate = d.hybrid_moe_route(api.Tensor.from_f32(d, logits.shape, f32, logits), policy,
                                            api.Tensor.from_f32(d, x.shape, f32, x), api.Tensor.from_f32(d, w.shape, f32, w))
    assert d.last_operation() == "h_moe_route"
    want = oracle.select_routes_ranked(logits, experts, top_k, normalize=True)
    assert np.array_equal(u32(ids), want[:, 0].view(np.uint32))
    assert np.abs(weights.to_f32().reshape(-1) - want[:, 2]).max() < 1e-5
    assert np.abs(gate.to_f32() - oracle.shared_gate(x, w)).max() < 1e-4
    # and it is the metadata form's columns
    meta, _ = d.moe_route_ranked(api.Tensor.from_f32(d, logits.shape, f32, logits), policy)
    assert np.array_equal(bits(meta.to_f32()[:, 0]), bits(ids.to_f32().reshape(-1)))
    assert np.array_equal(bits(meta.to_f32()[:, 2]), bits(weights.to_f32().reshape(-1)))


@pytest.mark.parametrize("ggml", [Q4_K, IQ4_XS])
def test_project_id_multiplies_each_route_by_its_expert(api, d, ggml):
    # iq_expert_projections_match_the_cpu_dequant (src/hybrid/iq_tests.rs:1398-1437):
    # x_div = 1 (a row per route) and x_div = used (the routes of a token share its row)
    experts, rows, cols = 3, 13, 1024
    packed = synth.matrix(ggml, experts * rows, cols, seed=411)
    w = api.QuantizedExpertMatrix.new(d, packed, api.QuantizationFormat(ggml), experts, rows, cols)
    ids = np.array([2, 0, 1, 1, 2, 0], dtype=np.uint32)
    routes = ids.size
    for x_div in (1, 3):
        x = synth.activations(routes // x_div, cols, seed=412 + x_div)
        y = d.hybrid_project_id(w, api.Tensor.from_f32(d, x.shape, api.DType.F32, x), carrier(api, d, ids), routes, x_div)
        assert d.last_operation().startswith("h_mv_id_")
        meta = np.zeros((routes, 3), dtype=np.uint32)
        meta[:, 0] = ids
        want = oracle.expert_project(ggml, packed, experts, rows, cols, np.repeat(x, x_div, axis=0),
                                     meta.view(np.float32), accumulate="f64")
        got = y.to_f32()
        assert np.abs(got - want).max() <= 5e-3 * np.abs(want).max()
        assert_matmul_parity(got, want, f"project_id x_div={x_div}")
    with pytest.raises(api.ShapeError):
        d.hybrid_project_id(w, api.Tensor.from_f32(d, (2, cols), api.DType.F32, x[:2]), carrier(api, d, ids[:5]), 5, 2)


@pytest.mark.parametrize("ggml", [Q4_K, IQ4_XS])
def test_project_id_carries_the_shared_expert(api, d, ggml):
    # moe_ffn's identity branch with its shared expert (src/hybrid/engine.rs:2925): the shared
    # rows ride in the routed launches and equal the separate one-row projections bit for bit
    experts, rows, cols, used, tokens = 4, 24, 512, 3, 2
    fmt = api.QuantizationFormat(ggml)
    w = api.QuantizedExpertMatrix.new(d, synth.matrix(ggml, experts * rows, cols, seed=421), fmt, experts, rows, cols)
    sw = api.QuantizedMatrix.from_bytes(d, rows, cols, fmt, synth.matrix(ggml, rows, cols, seed=422))
    ids = carrier(api, d, np.array([2, 0, 3, 1, 9, 0], dtype=np.uint32))   # 9 is not an expert: a zero row
    routes = tokens * used
    f32 = api.DType.F32
    x = api.Tensor.from_f32(d, (tokens, cols), f32, synth.activations(tokens, cols, seed=423))
    # gate / up: every route of a token and the shared expert read the token's row
    y, ys = d.hybrid_project_id_with_shared(w, sw, x, ids, routes, used, tokens)
    assert d.last_operation().startswith("h_mv_id_")
    assert np.array_equal(bits(y.to_f32()), bits(d.hybrid_project_id(w, x, ids, routes, used).to_f32()))
    with fma_gemv(d):
        assert np.array_equal(bits(ys.to_f32()), bits(d.hybrid_project(sw, x, exact=True).tensor.to_f32()))
    assert rel_l2(ys.to_f32(), d.hybrid_project(sw, x, exact=True).tensor.to_f32()) <= 1e-5
    assert np.abs(ys.to_f32()).max() > 1e-3 and not y.to_f32()[4].any()
    # down: a row per route, and the shared expert's own rows
    act = api.Tensor.from_f32(d, (routes, cols), f32, synth.activations(routes, cols, seed=424))
    shared_act = api.Tensor.from_f32(d, (tokens, cols), f32, synth.activations(tokens, cols, seed=425))
    y, ys = d.hybrid_project_id_with_shared(w, sw, act, ids, routes, 1, tokens, shared_x=shared_act)
    assert np.array_equal(bits(y.to_f32()), bits(d.hybrid_project_id(w, act, ids, routes, 1).to_f32()))
    with fma_gemv(d):
        assert np.array_equal(bits(ys.to_f32()), bits(d.hybrid_project(sw, shared_act, exact=True).tensor.to_f32()))
    with pytest.raises(api.ShapeError):   # without rows of its own the shared expert runs once per token row of x
        d.hybrid_project_id_with_shared(w, sw, act, ids, routes, 1, tokens)
    other = api.QuantizedMatrix.from_bytes(d, rows + 8, cols, fmt, synth.matrix(ggml, rows + 8, cols, seed=426))
    with pytest.raises(api.ShapeError):
        d.hybrid_project_id_with_shared(w, other, x, ids, routes, used, tokens)


@pytest.mark.parametrize("dtype,tokens", [("F32", 24), ("F16", 100), ("F32", 7)])
def test_project_mm_id_carries_the_shared_expert(api, d, dtype, tokens):
    # the prompt branch with its shared expert (src/hybrid/engine.rs:2925): routed rows are those of
    # project_mm_id bit for bit, shared rows are the dense projection of f16-rounded rows
    experts, used, rows, cols = 16, 4, 96, 512
    fmt = api.QuantizationFormat(Q4_K)
    packed_shared = synth.matrix(Q4_K, rows, cols, seed=432)
    w = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * rows, cols, seed=431), fmt, experts, rows, cols)
    sw = api.QuantizedMatrix.from_bytes(d, rows, cols, fmt, packed_shared)
    dt = getattr(api.DType, dtype)
    rng = synth.rng(433, tokens)
    routes = tokens * used
    ids = rng.integers(0, experts, routes).astype(np.uint32)
    offsets, order, _ = d.hybrid_moe_map(carrier(api, d, ids), experts)
    x = (rng.standard_normal((tokens, cols)) * 2.0 ** -3).astype(np.float32)
    xt = api.Tensor.from_f32(d, x.shape, dt, x)
    xg = d.hybrid_moe_gather(xt, order, used) if dtype == "F32" else \
        api.Tensor.from_f32(d, (routes, cols), dt, x[u32(order) // used])
    y, ys = d.hybrid_project_mm_id_with_shared(w, sw, xg, offsets, xt)
    assert d.last_operation() == "h_mm_id_q4_k"
    assert np.array_equal(y.raw(), d.hybrid_project_mm_id(w, xg, offsets).raw())
    want = oracle.project(Q4_K, packed_shared, rows, cols, oracle.round_storage(x, oracle.F16), accumulate="f64",
                          weight_round=oracle.F16)
    got = ys.to_f32()
    if dtype == "F32":
        assert_matmul_parity(got, want, "shared rows")
    else:   # the output itself is stored in f16
        assert_matmul_parity(got, want, "shared rows", max_rel_tol=2e-3, l2_tol=1e-3)
    with pytest.raises(api.ShapeError):
        other = api.QuantizedMatrix.from_bytes(d, rows, 2 * cols, fmt, synth.matrix(Q4_K, rows, 2 * cols, seed=434))
        d.hybrid_project_mm_id_with_shared(w, other, xg, offsets, xt)


@pytest.mark.parametrize("cols", [512, 6144])
def test_project_mm_id_keeps_inside_its_rows_whatever_the_offsets_say(api, d, cols):
    # offsets past the number of routes (a table made for another batch) are cut to it: the experts
    # before the damage give their usual rows, the damaged one takes what is left, none reads or
    # writes beyond the routes.  512 columns stay in LDS (the resident kernel), 6144 do not.
    experts, rows, routes = 8, 64, 200
    fmt = api.QuantizationFormat(Q4_K)
    w = api.QuantizedExpertMatrix.new(d, synth.matrix(Q4_K, experts * rows, cols, seed=441), fmt, experts, rows, cols)
    ids = synth.rng(442).integers(0, experts, routes).astype(np.uint32)
    offsets, order, _ = d.hybrid_moe_map(carrier(api, d, ids), experts)
    x = api.Tensor.from_f32(d, (routes, cols), api.DType.F16, synth.activations(routes, cols, seed=443, f16=True))
    good = d.hybrid_project_mm_id(w, x, offsets).to_f32()
    table = u32(offsets).copy()
    table[experts // 2 + 1:] = 0xFFFFFFF0
    damaged = d.hybrid_project_mm_id(w, x, carrier(api, d, table)).to_f32()
    intact = int(table[experts // 2])
    assert 0 < intact < routes
    assert np.array_equal(bits(damaged[:intact]), bits(good[:intact]))
    assert np.isfinite(damaged).all()
    table[1:] = table[:-1][::-1].copy()          # descending pairs are empty experts
    table[0] = 0
    assert np.isfinite(d.hybrid_project_mm_id(w, x, carrier(api, d, table)).to_f32()).all()


def test_prompt_chain_map_gather_mm_id_combine_matches_the_decode_chain_and_the_oracle(api, d):
    # HybridModel::moe_ffn's two branches (src/hybrid/engine.rs:3030-3075): per-route GEMVs with
    # `identity` rows, or map -> gather -> expert GEMM over sorted rows -> combine through position
    experts, used, hidden, inter, tokens = 16, 4, 512, 256, 24
    fmt = api.QuantizationFormat(Q4_K)
    w_gate = synth.matrix(Q4_K, experts * inter, hidden, seed=421)
    w_up = synth.matrix(Q4_K, experts * inter, hidden, seed=422)
    w_down = synth.matrix(Q4_K, experts * hidden, inter, seed=423)
    gate_e = api.QuantizedExpertMatrix.new(d, w_gate, fmt, experts, inter, hidden)
    up_e = api.QuantizedExpertMatrix.new(d, w_up, fmt, experts, inter, hidden)
    down_e = api.QuantizedExpertMatrix.new(d, w_down, fmt, experts, hidden, inter)
    rng = synth.rng(424)
    x = (rng.standard_normal((tokens, hidden)) * 2.0 ** -5).astype(np.float32)
    logits = rng.standard_normal((tokens, experts)).astype(np.float32)
    shared = (rng.standard_normal((tokens, hidden)) * 0.01).astype(np.float32)
    f32 = api.DType.F32
    xt = api.Tensor.from_f32(d, x.shape, f32, x)
    st = api.Tensor.from_f32(d, shared.shape, f32, shared)
    policy = api.MoeRoutingPolicy(experts, used, normalize_top_k_prob=True)
    ids, weights, gate = d.hybrid_moe_route(api.Tensor.from_f32(d, logits.shape, f32, logits), policy)
    routes = tokens * used

    def glu(g, u):                      # h_swiglu (hybrid.metal:1605-1612) on the host: the test's glue
        gv, uv = g.to_f32().astype(np.float64), u.to_f32().astype(np.float64)
        act = (gv / (1.0 + np.exp(-gv)) * uv).astype(np.float32)
        return api.Tensor.from_f32(d, act.shape, f32, act), act

    # decode branch: identity rows
    g1 = d.hybrid_project_id(gate_e, xt, ids, routes, used)
    u1 = d.hybrid_project_id(up_e, xt, ids, routes, used)
    a1, act1 = glu(g1, u1)
    d1 = d.hybrid_project_id(down_e, a1, ids, routes, 1)
    out1 = d.hybrid_moe_combine(d1, weights, None, st, gate, used).to_f32()
    assert d.last_operation() == "h_moe_combine"

    # prompt branch: expert-sorted rows
    offsets, order, position = d.hybrid_moe_map(ids, experts)
    xg = d.hybrid_moe_gather(xt, order, used)
    assert d.last_operation() == "h_moe_gather"
    assert np.array_equal(bits(xg.to_f32()), bits(x[u32(order) // used]))
    g2 = d.hybrid_project_mm_id(gate_e, xg, offsets)
    assert d.last_operation() == "h_mm_id_q4_k"
    u2 = d.hybrid_project_mm_id(up_e, xg, offsets)
    a2, act2 = glu(g2, u2)
    d2 = d.hybrid_project_mm_id(down_e, a2, offsets)
    out2 = d.hybrid_moe_combine(d2, weights, position, st, gate, used).to_f32()

    # oracle: exact-weight chain for the decode branch, f16-tile chain for the prompt branch
    id_words = u32(ids)
    meta = np.zeros((routes, 3), dtype=np.uint32)
    meta[:, 0] = id_words
    meta_f = meta.view(np.float32)
    xr = np.repeat(x, used, axis=0)
    og = oracle.expert_project(Q4_K, w_gate, experts, inter, hidden, xr, meta_f, accumulate="f64")
    ou = oracle.expert_project(Q4_K, w_up, experts, inter, hidden, xr, meta_f, accumulate="f64")
    assert_matmul_parity(g1.to_f32(), og, "gate by route")
    assert_matmul_parity(u1.to_f32(), ou, "up by route")
    od = oracle.expert_project(Q4_K, w_down, experts, hidden, inter, act1, meta_f, accumulate="f64")
    assert_matmul_parity(d1.to_f32(), od, "down by route")
    want1 = oracle.hybrid_combine(d1.to_f32(), weights.to_f32(), None, shared, gate.to_f32(), used)
    assert np.abs(out1 - want1).max() <= 1e-6 * max(1.0, np.abs(want1).max())

    pos = u32(position)
    sorted_meta = np.zeros((routes, 3), dtype=np.uint32)
    sorted_meta[pos, 0] = id_words
    xs16 = oracle.round_storage(x[u32(order) // used], oracle.F16).reshape(routes, hidden)
    og2 = oracle.expert_project(Q4_K, w_gate, experts, inter, hidden, xs16, sorted_meta.view(np.float32),
                                accumulate="f64", weight_round=oracle.F16)
    assert_matmul_parity(g2.to_f32(), og2, "gate over sorted rows")
    act16 = oracle.round_storage(act2, oracle.F16).reshape(routes, inter)
    od2 = oracle.expert_project(Q4_K, w_down, experts, hidden, inter, act16, sorted_meta.view(np.float32),
                                accumulate="f64", weight_round=oracle.F16)
    assert_matmul_parity(d2.to_f32(), od2, "down over sorted rows")
    want2 = oracle.hybrid_combine(d2.to_f32(), weights.to_f32(), pos, shared, gate.to_f32(), used)
    assert np.abs(out2 - want2).max() <= 1e-6 * max(1.0, np.abs(want2).max())
    # the two branches agree to the f16 tile rounding of the prompt branch
    assert rel_l2(out2, out1) <= 2e-3
    assert np.abs(out1).max() > 1e-4


@pytest.mark.parametrize("ggml", [Q4_K, IQ4_XS])
def test_project_tiers_follow_the_engine(api, d, ggml):
    # HybridModel::project (src/hybrid/engine.rs:3407-3500) and the cases of its format tests
    # (M = 1, 3, 16, 64: GEMV, batched GEMV, narrow tiles, tensor-op tiles; iq_tests.rs:1300-1337)
    n, k = 300, 1024
    packed = synth.matrix(ggml, n, k, seed=431)
    w = api.QuantizedMatrix.from_bytes(d, n, k, api.QuantizationFormat(ggml), packed)
    name = {Q4_K: "q4_k", IQ4_XS: "iq4_xs"}[ggml]
    for m, tier in ((1, "h_mv_"), (3, "h_mvb_"), (4, "h_mvb_"), (5, "h_mms_"), (16, "h_mms_"), (64, "h_mm_"), (200, "h_mm_")):
        x = synth.activations(m, k, seed=432 + m)
        out = d.hybrid_project(w, api.Tensor.from_f32(d, x.shape, api.DType.F32, x))
        assert out.operation == tier + name and out.tensor.dtype == api.DType.F32
        if m < 5:
            want = oracle.project(ggml, packed, n, k, x, accumulate="f64")
        else:
            want = oracle.project(ggml, packed, n, k, oracle.round_storage(x, oracle.F16).reshape(m, k),
                                  weight_round=oracle.F16, accumulate="f64")
        assert_matmul_parity(out.tensor.to_f32(), want, f"{tier}{name} m={m}")
        plain = oracle.project(ggml, packed, n, k, x, accumulate="f64")
        assert np.abs(out.tensor.to_f32() - plain).max() <= 5e-3 * np.abs(plain).max()      # the reference's bound
    x = synth.activations(16, k, seed=433)
    exact = d.hybrid_project(w, api.Tensor.from_f32(d, x.shape, api.DType.F32, x), exact=True)
    assert exact.operation == "h_mv_" + name
    assert_matmul_parity(exact.tensor.to_f32(), oracle.project(ggml, packed, n, k, x, accumulate="f64"), "exact")


def test_hybrid_entry_points_reject_bad_geometry(api, d):
    f32 = api.DType.F32
    ids = carrier(api, d, np.zeros(8, np.uint32))
    with pytest.raises(api.ShapeError):
        d.hybrid_moe_map(ids, 2000)                       # more than 1024 experts
    x = api.Tensor.zeros(d, (3, 64), f32)
    with pytest.raises(api.ShapeError):
        d.hybrid_moe_gather(x, ids, 2)                    # 8 routes are not 3 tokens x 2
    down = api.Tensor.zeros(d, (8, 64), api.DType.F16)
    with pytest.raises(api.DTypeError):
        d.hybrid_moe_combine(down, api.Tensor.zeros(d, (8,), f32), None, api.Tensor.zeros(d, (4, 64), f32),
                             api.Tensor.zeros(d, (4,), f32), 2)
