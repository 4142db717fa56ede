"""The model-level GGUF adapters on small files written here: the names and shapes of the
reference's tensor contract (src/model/qwen_gguf.rs:32-342, src/model/lfm2_moe/gguf.rs:165-405,
src/model/weights.rs:170-268) and every rejection it makes.  No device is needed: the plans
only read headers (and, for tied embeddings, compare payload bytes)."""
import numpy as np
import pytest

import gguf_files as gf
from ferrum_amd import api, gguf, gguf_models as gm, synth

F32, F16, Q4_0, Q8_0, Q4_K, Q6_K, IQ4_XS = 0, 1, 2, 8, 12, 14, 23


def dense(*dims, seed=0):
    """(GGUF dims fastest-first, F32, payload) for a logical shape."""
    values = synth.rng(seed).standard_normal(int(np.prod(dims))).astype(np.float32)
    return list(reversed(dims)), F32, values.view(np.uint8)


def packed(ggml, rows, cols, seed=0):
    return [cols, rows], ggml, synth.matrix(ggml, rows, cols, seed=seed)


# ---- Qwen --------------------------------------------------------------------------------

H, HEADS, KV, HD, INTER, VOCAB, LAYERS = 256, 2, 1, 128, 512, 512, 2


def qwen_metadata(arch):
    md = [("general.architecture", gf.STRING, arch), ("general.quantization_version", gf.U32, 2),
          (f"{arch}.embedding_length", gf.U32, H), (f"{arch}.attention.head_count", gf.U32, HEADS),
          (f"{arch}.attention.head_count_kv", gf.U32, KV), (f"{arch}.feed_forward_length", gf.U32, INTER),
          (f"{arch}.block_count", gf.U32, LAYERS), (f"{arch}.attention.layer_norm_rms_epsilon", gf.F32, 1e-6)]
    if arch == "qwen3":
        md += [("qwen3.attention.key_length", gf.U32, HD), ("qwen3.attention.value_length", gf.U32, HD)]
    return md


def qwen_tensors(arch, tied=True):
    t = {"token_embd.weight": packed(Q6_K, VOCAB, H, seed=1), "output_norm.weight": dense(H, seed=2)}
    if not tied:
        t["output.weight"] = packed(Q6_K, VOCAB, H, seed=3)
    for l in range(LAYERS):
        at = f"blk.{l}."
        t[at + "attn_norm.weight"] = dense(H)
        t[at + "ffn_norm.weight"] = dense(H)
        t[at + "attn_q.weight"] = packed(Q4_K, HEADS * HD, H, seed=10 + l)
        t[at + "attn_k.weight"] = packed(Q4_K, KV * HD, H, seed=20 + l)
        t[at + "attn_v.weight"] = packed(Q6_K, KV * HD, H, seed=30 + l)
        t[at + "attn_output.weight"] = packed(Q4_K, H, HEADS * HD, seed=40 + l)
        t[at + "ffn_gate.weight"] = packed(Q4_K, INTER, H, seed=50 + l)
        t[at + "ffn_up.weight"] = packed(Q4_K, INTER, H, seed=60 + l)
        t[at + "ffn_down.weight"] = packed(Q6_K, H, INTER, seed=70 + l)
        if arch == "qwen3":
            t[at + "attn_q_norm.weight"] = dense(HD)
            t[at + "attn_k_norm.weight"] = dense(HD)
        else:
            t[at + "attn_q.bias"] = dense(HEADS * HD)
            t[at + "attn_k.bias"] = dense(KV * HD)
            t[at + "attn_v.bias"] = dense(KV * HD)
    return t


def reader_of(tensors, metadata):
    return gguf.GgufReader.from_bytes(gf.build([(n, *v) for n, v in tensors.items()], metadata))


@pytest.mark.parametrize("arch", ["qwen2", "qwen3"])
@pytest.mark.parametrize("tied", [True, False])
def test_qwen_plan_names_every_tensor(arch, tied):
    tensors = qwen_tensors(arch, tied)
    shape, plan = gm.plan_qwen(reader_of(tensors, qwen_metadata(arch)))
    assert (shape.vocab_size, shape.hidden_size, shape.num_layers, shape.head_dim) == (VOCAB, H, LAYERS, HD)
    assert shape.tie_word_embeddings == tied and shape.qkv_bias == (arch == "qwen2")
    assert shape.qk_norm == ("per_head" if arch == "qwen3" else None)
    assert sorted(s for b in plan.bindings for s in b.sources) == sorted(tensors)
    assert plan.tensor_count == len(tensors) and not plan.redundant_output
    q = plan.binding("layers.1.q.weight")
    assert (q.sources, q.shape, q.kind, q.type_id) == (("blk.1.attn_q.weight",), [HEADS * HD, H], "quantized", Q4_K)
    down = plan.binding("layers.0.down.weight")
    assert (down.sources, down.shape, down.type_id) == (("blk.0.ffn_down.weight",), [H, INTER], Q6_K)
    assert plan.binding("embedding.weight").sources == ("token_embd.weight",)
    assert plan.binding("final_norm.weight").kind == "dense"
    if not tied:
        assert plan.binding("lm_head.weight").sources == ("output.weight",)
    else:
        with pytest.raises(api.WeightError):
            plan.binding("lm_head.weight")
    if arch == "qwen2":
        assert plan.binding("layers.0.k.bias").sources == ("blk.0.attn_k.bias",)
    else:
        assert plan.binding("layers.1.k_norm.weight").shape == [HD]
    elements = sum(int(np.prod(v[0])) for v in tensors.values())
    assert plan.parameter_count == elements
    assert plan.source_tensor_bytes == sum(len(np.asarray(v[2]).tobytes()) for v in tensors.values())
    assert [b.canonical for b in plan.quantized()] == [b.canonical for b in plan.bindings if b.type_id not in (0, 1, 30)]


def test_qwen_output_weight_that_repeats_the_embedding_is_tied_and_not_counted():
    tensors = qwen_tensors("qwen3")
    tensors["output.weight"] = tensors["token_embd.weight"]
    shape, plan = gm.plan_qwen(reader_of(tensors, qwen_metadata("qwen3")))
    assert shape.tie_word_embeddings and plan.redundant_output
    assert plan.tensor_count == len(tensors)
    assert plan.parameter_count == sum(int(np.prod(v[0])) for n, v in tensors.items() if n != "output.weight")
    assert all("output.weight" not in b.sources for b in plan.bindings)


def test_qwen2_head_dimension_comes_from_rope_metadata_when_present():
    md = qwen_metadata("qwen2") + [("qwen2.rope.dimension_count", gf.U32, HD)]
    shape, _ = gm.plan_qwen(reader_of(qwen_tensors("qwen2"), md))
    assert shape.head_dim == HD
    md[-1] = ("qwen2.rope.dimension_count", gf.U32, 64)      # then q is [128, 256] by contract, the file's is [256, 256]
    with pytest.raises(api.WeightError, match="expected shape"):
        gm.plan_qwen(reader_of(qwen_tensors("qwen2"), md))


def _changed(tensors, **changes):
    out = dict(tensors)
    for name, v in changes.items():
        name = name.replace("__", ".")
        if v is None:
            del out[name]
        else:
            out[name] = v
    return out


@pytest.mark.parametrize("change,error,text", [
    ({"blk__0__attn_rot__weight": dense(H)}, api.WeightError, "unexpected tensor"),
    ({"blk__1__ffn_up__weight": None}, api.GgufError, "missing tensor blk.1.ffn_up.weight"),
    ({"blk__0__ffn_gate__weight": packed(Q4_K, INTER + 8, H)}, api.WeightError, "expected shape"),
    ({"blk__0__attn_q__bias": dense(HD)}, api.WeightError, "unexpected tensor"),       # Qwen3 has no Q/K/V bias
    ({"output__bias": dense(VOCAB)}, api.WeightError, "no bias"),
    ({"blk__0__attn_q__weight": ([H, HEADS * HD], IQ4_XS, np.zeros(HEADS * HD * 136, np.uint8))}, api.WeightError,
     "unsupported GGML type 23"),
])
def test_qwen3_plan_rejections(change, error, text):
    with pytest.raises(error, match=text):
        gm.plan_qwen(reader_of(_changed(qwen_tensors("qwen3"), **change), qwen_metadata("qwen3")))


def test_qwen_metadata_rejections():
    with pytest.raises(api.ConfigError, match="unsupported"):
        gm.plan_qwen(reader_of(qwen_tensors("qwen3"), [("general.architecture", gf.STRING, "llama"),
                                                       ("general.quantization_version", gf.U32, 2)]))
    md = [m for m in qwen_metadata("qwen3") if m[0] != "qwen3.attention.value_length"]
    with pytest.raises(api.ConfigError, match="must match"):
        gm.plan_qwen(reader_of(qwen_tensors("qwen3"), md + [("qwen3.attention.value_length", gf.U32, 64)]))
    with pytest.raises(api.GgufError, match="missing metadata key"):
        gm.plan_qwen(reader_of(qwen_tensors("qwen3"), md))
    md = [m for m in qwen_metadata("qwen3") if m[0] != "qwen3.embedding_length"]
    with pytest.raises(api.ConfigError, match="differs from metadata"):
        gm.plan_qwen(reader_of(qwen_tensors("qwen3"), md + [("qwen3.embedding_length", gf.U32, 512)]))


def test_canonical_names_that_have_no_gguf_name():
    assert gm.qwen_source_name("layers.7.o.weight") == "blk.7.attn_output.weight"
    assert gm.qwen_source_name("layers.7.q.bias") == "blk.7.attn_q.bias"
    for bad in ("layers.0.conv.in_proj.weight", "layers.0.router.weight", "norm.weight"):
        with pytest.raises(api.WeightError):
            gm.qwen_source_name(bad)
    assert gm.lfm2_moe_source_names("layers.3.conv.depthwise.weight") == ["blk.3.shortconv.conv.weight"]
    assert gm.lfm2_moe_source_names("layers.3.moe.router_bias.weight") == ["blk.3.exp_probs_b.bias"]
    assert gm.lfm2_moe_source_names("final_norm.weight") == ["token_embd_norm.weight"]
    for bad in ("lm_head.weight", "layers.0.moe.gate.weight", "layers.0.q.bias", "layers.0.conv.bias"):
        with pytest.raises(api.WeightError):
            gm.lfm2_moe_source_names(bad)


# ---- LFM2-MoE ----------------------------------------------------------------------------

EXPERTS, MOE_INTER, TAPS = 4, 256, 3
KV_SCHEDULE = [0, 1, 0]          # layer 1 is attention, the others short convolutions
DENSE_LAYERS = 1


def lfm2_metadata():
    return [("general.architecture", gf.STRING, "lfm2moe"), ("general.quantization_version", gf.U32, 2),
            ("lfm2moe.vocab_size", gf.U32, VOCAB), ("lfm2moe.embedding_length", gf.U32, H),
            ("lfm2moe.feed_forward_length", gf.U32, INTER), ("lfm2moe.expert_feed_forward_length", gf.U32, MOE_INTER),
            ("lfm2moe.block_count", gf.U32, len(KV_SCHEDULE)), ("lfm2moe.attention.head_count", gf.U32, HEADS),
            ("lfm2moe.attention.head_count_kv", gf.ARRAY, KV_SCHEDULE, gf.I32), ("lfm2moe.expert_count", gf.U32, EXPERTS),
            ("lfm2moe.expert_used_count", gf.U32, 2), ("lfm2moe.leading_dense_block_count", gf.U32, DENSE_LAYERS),
            ("lfm2moe.shortconv.l_cache", gf.U32, TAPS), ("lfm2moe.expert_gating_func", gf.U32, 2)]


def experts_tensor(ggml, experts, rows, cols, seed):
    return [cols, rows, experts], ggml, synth.matrix(ggml, experts * rows, cols, seed=seed)


def lfm2_tensors():
    t = {"token_embd.weight": packed(Q6_K, VOCAB, H, seed=1), "token_embd_norm.weight": dense(H)}
    for l, kv in enumerate(KV_SCHEDULE):
        at = f"blk.{l}."
        t[at + "attn_norm.weight"] = dense(H)
        t[at + "ffn_norm.weight"] = dense(H)
        if kv:
            t[at + "attn_q.weight"] = packed(Q4_K, HEADS * HD, H, seed=10 + l)
            t[at + "attn_k.weight"] = packed(Q4_K, kv * HD, H, seed=20 + l)
            t[at + "attn_v.weight"] = packed(Q6_K, kv * HD, H, seed=30 + l)
            t[at + "attn_output.weight"] = packed(Q4_K, H, HEADS * HD, seed=40 + l)
            t[at + "attn_q_norm.weight"] = dense(HD)
            t[at + "attn_k_norm.weight"] = dense(HD)
        else:
            t[at + "shortconv.in_proj.weight"] = packed(Q4_K, 3 * H, H, seed=80 + l)
            t[at + "shortconv.conv.weight"] = ([TAPS, H], F32, np.zeros(TAPS * H, np.float32).view(np.uint8))
            t[at + "shortconv.out_proj.weight"] = packed(Q4_K, H, H, seed=90 + l)
        if l < DENSE_LAYERS:
            t[at + "ffn_gate.weight"] = packed(Q4_K, INTER, H, seed=50 + l)
            t[at + "ffn_up.weight"] = packed(Q4_K, INTER, H, seed=60 + l)
            t[at + "ffn_down.weight"] = packed(Q6_K, H, INTER, seed=70 + l)
        else:
            t[at + "ffn_gate_inp.weight"] = dense(EXPERTS, H)
            t[at + "exp_probs_b.bias"] = dense(EXPERTS)
            t[at + "ffn_gate_exps.weight"] = experts_tensor(Q4_K, EXPERTS, MOE_INTER, H, 100 + l)
            t[at + "ffn_up_exps.weight"] = experts_tensor(Q4_K, EXPERTS, MOE_INTER, H, 110 + l)
            t[at + "ffn_down_exps.weight"] = experts_tensor(Q6_K, EXPERTS, H, MOE_INTER, 120 + l)
    return t


def test_lfm2_moe_plan_names_every_tensor():
    tensors = lfm2_tensors()
    reader = reader_of(tensors, lfm2_metadata())
    shape = gm.lfm2_moe_shape(reader)
    assert [l.short_conv_kernel for l in shape.layers] == [TAPS, None, TAPS]
    assert [l.sparse is not None for l in shape.layers] == [False, True, True]
    assert (shape.num_key_value_heads, shape.head_dim, shape.qk_norm) == (1, HD, "per_head")
    plan = gm.plan_lfm2_moe(reader, shape)
    assert sorted(s for b in plan.bindings for s in b.sources) == sorted(tensors)
    stacked = plan.binding("layers.2.moe.input.weight")
    assert stacked.sources == ("blk.2.ffn_gate_exps.weight", "blk.2.ffn_up_exps.weight")
    assert (stacked.shape, stacked.kind, stacked.type_id) == ([EXPERTS, 2 * MOE_INTER, H], "stacked_experts", Q4_K)
    out = plan.binding("layers.1.moe.output.weight")
    assert (out.sources, out.shape, out.kind, out.type_id) == (("blk.1.ffn_down_exps.weight",), [EXPERTS, H, MOE_INTER],
                                                                "experts", Q6_K)
    assert plan.binding("layers.0.conv.depthwise.weight").shape == [H, 1, TAPS]
    assert plan.binding("layers.0.conv.in_proj.weight").shape == [3 * H, H]
    assert plan.binding("layers.1.moe.router_bias.weight").sources == ("blk.1.exp_probs_b.bias",)
    assert plan.binding("layers.1.moe.router.weight").kind == "dense"
    # the router's selection bias is not a parameter (src/model/lfm2_moe/gguf.rs:40-46)
    assert plan.parameter_count == sum(int(np.prod(v[0])) for n, v in tensors.items() if not n.endswith(".exp_probs_b.bias"))
    assert plan.tensor_count == len(tensors)
    # without the selection bias in the policy, the file's bias tensors are beyond the contract
    with pytest.raises(api.WeightError, match="unexpected tensor"):
        gm.plan_lfm2_moe(reader, gm.lfm2_moe_shape(reader, use_expert_bias=False))


@pytest.mark.parametrize("change,error,text", [
    ({"blk__1__ffn_up_exps__weight": experts_tensor(Q6_K, EXPERTS, MOE_INTER, H, 5)}, api.WeightError,
     "different quantization formats"),
    ({"blk__1__ffn_up_exps__weight": experts_tensor(Q4_K, EXPERTS, MOE_INTER + 8, H, 5)}, api.WeightError,
     "expected logical expert shape"),
    ({"blk__2__ffn_down_exps__weight": ([MOE_INTER, H, EXPERTS], Q8_0, np.zeros(EXPERTS * H * MOE_INTER // 32 * 34, np.uint8))},
     api.WeightError, "must use Q4_K, Q5_K, or Q6_K"),
    ({"blk__2__ffn_down_exps__weight": packed(Q6_K, EXPERTS * H, MOE_INTER)}, api.GgufError, "expected an expert matrix"),
    ({"blk__0__shortconv__conv__weight": ([TAPS + 1, H], F32, np.zeros((TAPS + 1) * H, np.float32).view(np.uint8))},
     api.WeightError, "expected logical shape"),
    ({"output__weight": packed(Q6_K, VOCAB, H, seed=9)}, api.WeightError, "differ from token embeddings"),
    ({"blk__1__ffn_gate__weight": packed(Q4_K, INTER, H)}, api.WeightError, "unexpected tensor"),
    ({"blk__1__attn_q__weight": ([H, HEADS * HD], IQ4_XS, np.zeros(HEADS * HD * 136, np.uint8))}, api.WeightError,
     "unsupported GGML tensor type 23"),
])
def test_lfm2_moe_plan_rejections(change, error, text):
    reader = reader_of(_changed(lfm2_tensors(), **change), lfm2_metadata())
    with pytest.raises(error, match=text):
        gm.plan_lfm2_moe(reader, gm.lfm2_moe_shape(reader))


def test_lfm2_moe_tied_output_copy_is_accepted_and_not_counted():
    tensors = lfm2_tensors()
    tensors["output.weight"] = tensors["token_embd.weight"]
    reader = reader_of(tensors, lfm2_metadata())
    plan = gm.plan_lfm2_moe(reader, gm.lfm2_moe_shape(reader))
    assert plan.redundant_output and plan.tensor_count == len(tensors)
    assert all("output.weight" not in b.sources for b in plan.bindings)


def test_lfm2_moe_metadata_rejections():
    tensors = lfm2_tensors()
    md = [m for m in lfm2_metadata() if m[0] != "lfm2moe.expert_gating_func"]
    with pytest.raises(api.ConfigError):
        gm.lfm2_moe_shape(reader_of(tensors, md + [("lfm2moe.expert_gating_func", gf.U32, 1)]))
    md = [m for m in lfm2_metadata() if m[0] != "lfm2moe.attention.head_count_kv"]
    with pytest.raises(api.ConfigError, match="schedule"):
        gm.lfm2_moe_shape(reader_of(tensors, md + [("lfm2moe.attention.head_count_kv", gf.ARRAY, [0, 1], gf.I32)]))
    with pytest.raises(api.ConfigError, match="schedule"):
        gm.lfm2_moe_shape(reader_of(tensors, md + [("lfm2moe.attention.head_count_kv", gf.ARRAY, [0, 1, 2], gf.I32)]))


def test_specifications_follow_the_reference_order():
    shape = gm.ModelShape(vocab_size=VOCAB, hidden_size=H, num_attention_heads=HEADS, num_key_value_heads=KV, head_dim=HD,
                          tie_word_embeddings=False, qk_norm="projection",
                          layers=[gm.LayerShape(INTER), gm.LayerShape(INTER, sparse=gm.SparseFeedForward(EXPERTS, MOE_INTER))])
    names = [n for n, _ in gm.specifications(shape)]
    assert names[:3] == ["embedding.weight", "final_norm.weight", "lm_head.weight"]
    assert names[3:14] == [f"layers.0.{n}.weight" for n in ("input_norm", "post_norm", "q", "k", "v", "o", "gate", "up", "down",
                                                             "q_norm", "k_norm")]
    assert dict(gm.specifications(shape))["layers.0.q_norm.weight"] == [HEADS * HD]     # the projection-wide layout
    assert dict(gm.specifications(shape))["layers.1.k_norm.weight"] == [KV * HD]
    assert "layers.1.moe.router_bias.weight" not in names and "layers.1.moe.input.weight" in names


# ---- the C++ adapter (include/ferrum_gguf_models.hpp) against the Python one ----------------

@pytest.fixture(scope="module")
def probe():
    from ferrum_amd import build
    return build.build_gguf_probe()


def _describe(shape, plan):
    kinds = {"dense": 0, "quantized": 1, "experts": 2, "stacked_experts": 3}
    norm = {None: 0, "per_head": 1, "projection": 2}[shape.qk_norm]
    lines = [f"shape {shape.architecture} vocab {shape.vocab_size} hidden {shape.hidden_size} heads {shape.num_attention_heads} "
             f"kv {shape.num_key_value_heads} head_dim {shape.head_dim} layers {shape.num_layers} "
             f"tied {int(shape.tie_word_embeddings)} bias {int(shape.qkv_bias)} qk_norm {norm}"]
    for b in plan.bindings:
        lines.append(f"bind {b.canonical} <- {' '.join(b.sources)} shape {' '.join(map(str, b.shape))} "
                     f"kind {kinds[b.kind]} type {b.type_id}")
    lines.append(f"totals {plan.tensor_count} tensors {plan.source_tensor_bytes} bytes {plan.parameter_count} parameters "
                 f"redundant {int(plan.redundant_output)}")
    return lines


def test_cpp_adapter_agrees_with_the_python_adapter(probe, tmp_path):
    import subprocess
    q3 = qwen_tensors("qwen3")
    redundant = dict(q3, **{"output.weight": q3["token_embd.weight"]})
    lfm = lfm2_tensors()
    cases = {
        "qwen2": ("qwen", qwen_tensors("qwen2", tied=False), qwen_metadata("qwen2"), None),
        "qwen3": ("qwen", q3, qwen_metadata("qwen3"), None),
        "redundant": ("qwen", redundant, qwen_metadata("qwen3"), None),
        "lfm2moe": ("lfm2moe", lfm, lfm2_metadata(), None),
        "extra": ("qwen", _changed(q3, blk__0__attn_rot__weight=dense(H)), qwen_metadata("qwen3"), api.WeightError),
        "shape": ("qwen", _changed(q3, blk__0__ffn_gate__weight=packed(Q4_K, INTER + 8, H)), qwen_metadata("qwen3"), api.WeightError),
        "missing": ("qwen", _changed(q3, blk__1__ffn_up__weight=None), qwen_metadata("qwen3"), api.GgufError),
        "arch": ("qwen", q3, lfm2_metadata(), api.ConfigError),
        "formats": ("lfm2moe", _changed(lfm, blk__1__ffn_up_exps__weight=experts_tensor(Q6_K, EXPERTS, MOE_INTER, H, 5)),
                    lfm2_metadata(), api.WeightError),
        "taps": ("lfm2moe", _changed(lfm, blk__0__shortconv__conv__weight=([TAPS + 1, H], F32,
                                                                            np.zeros((TAPS + 1) * H, np.float32).view(np.uint8))),
                 lfm2_metadata(), api.WeightError),
        "rank": ("lfm2moe", _changed(lfm, blk__2__ffn_down_exps__weight=packed(Q6_K, EXPERTS * H, MOE_INTER)), lfm2_metadata(),
                 api.GgufError),
        "nobias": ("lfm2moe nobias", lfm, lfm2_metadata(), api.WeightError),
    }
    for label, (family, tensors, metadata, error) in cases.items():
        path = tmp_path / f"{label}.gguf"
        path.write_bytes(gf.build([(n, *v) for n, v in tensors.items()], metadata))
        proc = subprocess.run([probe, str(path), "plan", *family.split()], capture_output=True, text=True, timeout=30)

        def python_side():
            reader = gguf.GgufReader.open(str(path))
            if family == "qwen":
                return gm.plan_qwen(reader)
            shape = gm.lfm2_moe_shape(reader, use_expert_bias="nobias" not in family)
            return shape, gm.plan_lfm2_moe(reader, shape)

        if error is None:
            assert proc.returncode == 0, (label, proc.stdout, proc.stderr)
            assert proc.stdout.splitlines() == _describe(*python_side()), label
        else:
            assert proc.returncode == (2 if error is api.GgufError else 3), (label, proc.stdout, proc.stderr)
            with pytest.raises(error) as caught:
                python_side()
            # the same rejection in both: the C++ message is the Python one without the kind prefix
            assert proc.stdout.strip() == "error: " + caught.value.message, label
