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
