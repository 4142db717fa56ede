"""K-quant tensors read from a GGUF file reach the device verbatim and project
like the oracle: the loader side of the hot path (src/loader/gguf.rs:474-493
feeding src/quantization.rs:86-111)."""
import numpy as np
import pytest

import gguf_files as gf
import oracle
from helpers import assert_matmul_parity, bits
from ferrum_amd import gguf, synth

pytestmark = pytest.mark.gpu

Q4_K, Q6_K = 12, 14


def test_tensors_from_a_gguf_file_project_like_the_oracle(tmp_path):
    from ferrum_amd import api
    d = api.Device.new()
    n, k, experts, rows = 300, 1024, 4, 48
    q4 = synth.matrix(Q4_K, n, k, seed=31)
    q6 = synth.matrix(Q6_K, n, k, seed=32)
    ex = synth.matrix(Q4_K, experts * rows, k, seed=33)
    f32 = np.arange(8, dtype=np.float32)
    path = tmp_path / "layer.gguf"
    path.write_bytes(gf.build([("token_embd.weight", [8], 0, f32.view(np.uint8)),
                               ("blk.0.ffn_gate.weight", [k, n], Q4_K, q4),
                               ("output.weight", [k, n], Q6_K, q6),
                               ("blk.0.ffn_gate_exps.weight", [k, rows, experts], Q4_K, ex)]))
    f = gguf.GgufReader.open(str(path))

    x = synth.activations(3, k, seed=34)
    xt = api.Tensor.from_f32(d, x.shape, api.DType.F32, x)
    for name, ggml, packed in (("blk.0.ffn_gate.weight", Q4_K, q4), ("output.weight", Q6_K, q6)):
        w = f.quantized_matrix(d, name)
        assert (w.rows(), w.columns(), w.format().value) == (n, k, ggml)
        assert np.array_equal(bits(d.dequantize(w).to_f32()), bits(oracle.dequantize(ggml, packed, n, k)))
        got = d.project_quantized(xt, w).tensor.to_f32()
        assert_matmul_parity(got, oracle.project(ggml, packed, n, k, x, accumulate="f64"), name)

    w = f.quantized_expert_matrix(d, "blk.0.ffn_gate_exps.weight")
    assert (w.experts(), w.rows_per_expert(), w.columns()) == (experts, rows, k)
    meta = np.zeros((5, 3), dtype=np.uint32)
    meta[:, 0] = [3, 0, 2, 2, 1]
    meta[:, 1] = np.arange(5)
    meta[:, 2] = np.float32(1.0).view(np.uint32)
    xa = synth.activations(5, k, seed=35)
    got = d.expert_project_quantized(api.Tensor.from_f32(d, xa.shape, api.DType.F32, xa),
                                     api.Tensor.from_bits(d, meta.shape, meta), w, k, experts).to_f32()
    want = oracle.expert_project(Q4_K, ex, experts, rows, k, xa, meta.view(np.float32), accumulate="f64")
    assert_matmul_parity(got, want, "expert tensor from file")

    with pytest.raises(api.GgufError):
        f.quantized_matrix(d, "token_embd.weight")             # rank 1
    with pytest.raises(api.GgufError):
        f.quantized_matrix(d, "blk.0.ffn_gate_exps.weight")    # rank 3
    with pytest.raises(api.GgufError):
        f.quantized_expert_matrix(d, "output.weight")


def test_stacked_gate_up_experts_from_a_gguf_file_run_the_fused_decode_chain(tmp_path):
    from ferrum_amd import api
    d = api.Device.new()
    experts, inter, hidden, top_k, tokens = 4, 256, 512, 2, 2
    gate = synth.matrix(Q4_K, experts * inter, hidden, seed=41)
    up = synth.matrix(Q4_K, experts * inter, hidden, seed=42)
    down = synth.matrix(Q4_K, experts * hidden, inter, seed=43)
    path = tmp_path / "moe.gguf"
    path.write_bytes(gf.build([("blk.0.ffn_gate_exps.weight", [hidden, inter, experts], Q4_K, gate),
                               ("blk.0.ffn_up_exps.weight", [hidden, inter, experts], Q4_K, up),
                               ("blk.0.ffn_down_exps.weight", [inter, hidden, experts], Q4_K, down)]))
    f = gguf.GgufReader.open(str(path))
    win = f.quantized_input_experts(d, "blk.0.ffn_gate_exps.weight", "blk.0.ffn_up_exps.weight")
    wout = f.quantized_expert_matrix(d, "blk.0.ffn_down_exps.weight")
    assert (win.experts(), win.rows_per_expert(), win.columns()) == (experts, 2 * inter, hidden)
    moe = api.SparseMoe(d, win, wout, api.MoeRoutingPolicy(experts, top_k))
    rng = synth.rng(44)
    x = (rng.standard_normal((tokens, hidden)) * 2.0 ** -6).astype(np.float32)
    logits = rng.standard_normal((tokens, experts)).astype(np.float32)
    got = moe.forward(api.Tensor.from_f32(d, x.shape, api.DType.F32, x),
                      api.Tensor.from_f32(d, logits.shape, api.DType.F32, logits)).to_f32()
    row_bytes = hidden // 256 * 144
    stacked = np.concatenate([gate.reshape(experts, inter, row_bytes), up.reshape(experts, inter, row_bytes)],
                             axis=1).reshape(-1)
    m = oracle.select_routes(logits, experts, top_k)
    o_up = oracle.expert_project(Q4_K, stacked, experts, 2 * inter, hidden, oracle.expert_assign(x, m), m,
                                 accumulate="f64")
    o_down = oracle.expert_project(Q4_K, down, experts, hidden, inter, oracle.expert_silu_mul(o_up, inter), m,
                                   accumulate="f64")
    want = oracle.expert_combine(o_down, m, tokens, hidden, top_k)
    assert np.abs(want).max() > 1e-4
    l2 = float(np.linalg.norm(got - want) / np.linalg.norm(want))
    assert l2 <= 2e-5, l2


@pytest.mark.parametrize("ggml", [23, 8, 13], ids=["iq4_xs", "q8_0", "q5_k"])
def test_other_formats_load_from_a_gguf_file(tmp_path, ggml):
    # the file's bytes are the device payload unchanged, also for Q8_0 whose GGUF block is 32 weights
    from ferrum_amd import api
    d = api.Device.new()
    n, k, experts, rows = 70, 768, 3, 20
    dense = synth.matrix(ggml, n, k, seed=51)
    ex = synth.matrix(ggml, experts * rows, k, seed=52)
    path = tmp_path / "formats.gguf"
    path.write_bytes(gf.build([("blk.0.attn_q.weight", [k, n], ggml, dense),
                               ("blk.0.ffn_down_exps.weight", [k, rows, experts], ggml, ex)]))
    f = gguf.GgufReader.open(str(path))
    w = f.quantized_matrix(d, "blk.0.attn_q.weight")
    assert (w.rows(), w.columns(), w.format().value) == (n, k, ggml)
    assert np.array_equal(bits(d.dequantize(w).to_f32()), bits(oracle.dequantize(ggml, dense, n, k)))
    e = f.quantized_expert_matrix(d, "blk.0.ffn_down_exps.weight")
    assert (e.experts(), e.rows_per_expert(), e.columns()) == (experts, rows, k)
    assert np.array_equal(bits(d.dequantize(e.matrix_view()).to_f32()),
                          bits(oracle.dequantize(ggml, ex, experts * rows, k)))


def test_a_whole_lfm2_moe_file_binds_by_canonical_name_and_runs_a_sparse_layer(tmp_path):
    # the model-level adapter (src/model/lfm2_moe/gguf.rs:165-320, 434-574): every quantized tensor
    # of the file lands on the device under its canonical name, blocks verbatim, gate and up
    # experts interleaved; a sparse layer built from the bound matrices gives the host answer
    import test_gguf_models as files
    from ferrum_amd import api, gguf_models
    d = api.Device.new()
    tensors = files.lfm2_tensors()
    path = tmp_path / "lfm2moe.gguf"
    path.write_bytes(gf.build([(n, *v) for n, v in tensors.items()], files.lfm2_metadata()))
    f = gguf.GgufReader.open(str(path))
    plan = gguf_models.plan_lfm2_moe(f, gguf_models.lfm2_moe_shape(f))
    weights, quantized_bytes = gguf_models.bind_quantized(d, f, plan)
    assert sorted(weights) == sorted(b.canonical for b in plan.quantized())
    assert quantized_bytes == sum(np.asarray(v[2]).nbytes for v in tensors.values() if v[1] != 0)
    assert 0 < quantized_bytes <= plan.source_tensor_bytes
    H, I, E = files.H, files.MOE_INTER, files.EXPERTS
    q = weights["layers.1.q.weight"]
    assert (q.rows(), q.columns(), q.format().value) == (files.HEADS * files.HD, H, Q4_K)
    packed_q = np.asarray(tensors["blk.1.attn_q.weight"][2])
    assert np.array_equal(bits(d.dequantize(q).to_f32()), bits(oracle.dequantize(Q4_K, packed_q, q.rows(), H)))
    win, wout = weights["layers.2.moe.input.weight"], weights["layers.2.moe.output.weight"]
    assert (win.experts(), win.rows_per_expert(), win.columns()) == (E, 2 * I, H)
    assert (wout.experts(), wout.rows_per_expert(), wout.columns(), wout.format().value) == (E, H, I, Q6_K)
    gate = np.asarray(tensors["blk.2.ffn_gate_exps.weight"][2])
    up = np.asarray(tensors["blk.2.ffn_up_exps.weight"][2])
    down = np.asarray(tensors["blk.2.ffn_down_exps.weight"][2])
    row_bytes = H // 256 * 144
    stacked = np.concatenate([gate.reshape(E, I, row_bytes), up.reshape(E, I, row_bytes)], axis=1).reshape(-1)
    assert np.array_equal(bits(d.dequantize(win.matrix_view()).to_f32()), bits(oracle.dequantize(Q4_K, stacked, E * 2 * I, H)))
    top_k, tokens = 2, 3
    moe = api.SparseMoe(d, win, wout, api.MoeRoutingPolicy(E, top_k))
    rng = synth.rng(61)
    x = (rng.standard_normal((tokens, H)) * 2.0 ** -5).astype(np.float32)
    logits = rng.standard_normal((tokens, E)).astype(np.float32)
    got = moe.forward(api.Tensor.from_f32(d, x.shape, api.DType.F32, x),
                      api.Tensor.from_f32(d, logits.shape, api.DType.F32, logits)).to_f32()
    m = oracle.select_routes(logits, E, top_k)
    o_up = oracle.expert_project(Q4_K, stacked, E, 2 * I, H, oracle.expert_assign(x, m), m, accumulate="f64")
    o_down = oracle.expert_project(Q6_K, down, E, H, I, oracle.expert_silu_mul(o_up, I), m, accumulate="f64")
    want = oracle.expert_combine(o_down, m, tokens, H, top_k)
    assert np.abs(want).max() > 1e-4
    assert float(np.linalg.norm(got - want) / np.linalg.norm(want)) <= 2e-5
    # a Qwen file the same way: only the listed types are uploaded when asked
    qt = files.qwen_tensors("qwen3", tied=False)
    path = tmp_path / "qwen3.gguf"
    path.write_bytes(gf.build([(n, *v) for n, v in qt.items()], files.qwen_metadata("qwen3")))
    f = gguf.GgufReader.open(str(path))
    shape, plan = gguf_models.plan_qwen(f)
    only_q6, _ = gguf_models.bind_quantized(d, f, plan, only=(Q6_K,))
    assert sorted(only_q6) == sorted(["embedding.weight", "lm_head.weight"] + [f"layers.{l}.{n}.weight"
                                                                              for l in range(shape.num_layers) for n in ("v", "down")])
    head = only_q6["lm_head.weight"]
    xr = synth.activations(1, files.H, seed=62)
    got = d.project_quantized(api.Tensor.from_f32(d, xr.shape, api.DType.F32, xr), head).tensor.to_f32()
    assert_matmul_parity(got, oracle.project(Q6_K, np.asarray(qt["output.weight"][2]), files.VOCAB, files.H, xr, accumulate="f64"),
                         "lm_head bound by canonical name")
