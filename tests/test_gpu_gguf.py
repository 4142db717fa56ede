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
