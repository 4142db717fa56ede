"""Model-level GGUF adapters: which tensor of a file is which weight of the model.

The reader (``gguf.GgufReader``) knows tensors by their GGUF names; the operators know
packed matrices.  These adapters are the step between: they restate the reference's
tensor contract for its two GGUF model families and bind every quantized tensor of a file
to a ``QuantizedMatrix`` / ``QuantizedExpertMatrix`` on the device, blocks verbatim.

* ``specifications`` lists the canonical weights of a model and their logical shapes
  (``specifications_with_policy``, src/model/weights.rs:170-268).
* ``qwen_source_name`` / ``lfm2_moe_source_names`` map a canonical name to the GGUF tensor
  name(s) that hold it (src/model/qwen_gguf.rs:304-342, src/model/lfm2_moe/gguf.rs:322-366).
* ``plan_qwen`` reads a Qwen2 / Qwen3 file's metadata into a ``ModelShape`` and checks the
  file against the contract (src/model/qwen_gguf.rs:32-222): every expected tensor present
  with its logical shape, no tensor beyond them, quantized types on matrices only.
* ``plan_lfm2_moe`` does the same for LFM2-MoE (``map_gguf_weights``,
  src/model/lfm2_moe/gguf.rs:165-320), whose routed experts are rank-3 tensors and whose
  gate and up experts become one ``[experts, 2 I, H]`` matrix.
* ``bind_quantized`` uploads the plan's quantized tensors (qwen_gguf.rs:236-268,
  lfm2_moe/gguf.rs:434-574).

Dense tensors (norms, biases, unquantized embeddings) are named and checked by the plan but
not uploaded here: they do not take the quantized-matmul path.  Every failure is one of the
``api`` error classes the reference's variant maps to (``WeightError``, ``ConfigError``,
``GgufError``).
"""
from __future__ import annotations

from dataclasses import dataclass, field

DENSE_TYPES = (0, 1, 30)                       # F32, F16, BF16
QWEN_QUANTIZED_TYPES = (2, 6, 7, 8, 12, 13, 14)    # src/model/qwen_gguf.rs:238
EXPERT_TYPES = (12, 13, 14)                    # Q4_K, Q5_K, Q6_K (lfm2_moe/gguf.rs:392-399)


def _api():
    from . import api
    return api


@dataclass(frozen=True)
class SparseFeedForward:
    """LayerFeedForwardPolicy::Sparse: `experts` routed experts of width `intermediate_size`."""
    experts: int
    intermediate_size: int
    use_expert_bias: bool = False


@dataclass(frozen=True)
class LayerShape:
    """One layer of the architecture policy: attention or a short convolution of
    `short_conv_kernel` taps, then a dense feed-forward of `intermediate_size` or a sparse one."""
    intermediate_size: int
    short_conv_kernel: int | None = None
    sparse: SparseFeedForward | None = None


@dataclass
class ModelShape:
    """The part of ModelConfig + ArchitecturePolicy the tensor contract depends on."""
    vocab_size: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    tie_word_embeddings: bool
    layers: list = field(default_factory=list)     # LayerShape per layer
    qk_norm: str | None = None                     # None, "per_head" or "projection"
    qkv_bias: bool = False                         # Qwen2's required Q/K/V biases
    architecture: str = ""

    @property
    def num_layers(self) -> int:
        return len(self.layers)


def specifications(shape: ModelShape) -> list[tuple[str, list[int]]]:
    """Canonical weight names and logical shapes, in the reference's order
    (src/model/weights.rs:170-268)."""
    h = shape.hidden_size
    q = shape.num_attention_heads * shape.head_dim
    k = shape.num_key_value_heads * shape.head_dim
    specs = [("embedding.weight", [shape.vocab_size, h]), ("final_norm.weight", [h])]
    if not shape.tie_word_embeddings:
        specs.append(("lm_head.weight", [shape.vocab_size, h]))
    for l, layer in enumerate(shape.layers):
        at = f"layers.{l}."
        specs += [(at + "input_norm.weight", [h]), (at + "post_norm.weight", [h])]
        if layer.short_conv_kernel is None:
            specs += [(at + "q.weight", [q, h]), (at + "k.weight", [k, h]), (at + "v.weight", [k, h]),
                      (at + "o.weight", [h, q])]
        else:
            specs += [(at + "conv.in_proj.weight", [3 * h, h]),
                      (at + "conv.depthwise.weight", [h, 1, layer.short_conv_kernel]),
                      (at + "conv.out_proj.weight", [h, h])]
        if layer.sparse is None:
            i = layer.intermediate_size
            specs += [(at + "gate.weight", [i, h]), (at + "up.weight", [i, h]), (at + "down.weight", [h, i])]
        else:
            s = layer.sparse
            specs += [(at + "moe.router.weight", [s.experts, h]),
                      (at + "moe.input.weight", [s.experts, 2 * s.intermediate_size, h]),
                      (at + "moe.output.weight", [s.experts, h, s.intermediate_size])]
            if s.use_expert_bias:
                specs.append((at + "moe.router_bias.weight", [s.experts]))
        if layer.short_conv_kernel is None and shape.qk_norm is not None:
            for name, heads in (("q_norm.weight", shape.num_attention_heads), ("k_norm.weight", shape.num_key_value_heads)):
                width = shape.head_dim if shape.qk_norm == "per_head" else heads * shape.head_dim
                specs.append((at + name, [width]))
    return specs


_COMPONENTS = {"input_norm": "attn_norm", "post_norm": "ffn_norm", "q": "attn_q", "k": "attn_k", "v": "attn_v",
               "o": "attn_output", "q_norm": "attn_q_norm", "k_norm": "attn_k_norm", "gate": "ffn_gate",
               "up": "ffn_up", "down": "ffn_down"}


def qwen_source_name(canonical: str) -> str:
    """GGUF name of a canonical Qwen weight (gguf_weight_name, src/model/qwen_gguf.rs:304-342)."""
    fixed = {"embedding.weight": "token_embd.weight", "final_norm.weight": "output_norm.weight",
             "lm_head.weight": "output.weight"}
    if canonical in fixed:
        return fixed[canonical]
    parts = canonical.split(".")
    if len(parts) != 4 or parts[0] != "layers":
        raise _api().WeightError(f"{canonical}: cannot map canonical Qwen weight")
    if parts[2] not in _COMPONENTS:
        raise _api().WeightError(f"{canonical}: unsupported Qwen weight component")
    return f"blk.{parts[1]}.{_COMPONENTS[parts[2]]}.{parts[3]}"


def lfm2_moe_source_names(canonical: str) -> list[str]:
    """GGUF name(s) of a canonical LFM2-MoE weight (source_names,
    src/model/lfm2_moe/gguf.rs:322-366): the routed input matrix comes from two tensors,
    gate experts first."""
    if canonical == "embedding.weight":
        return ["token_embd.weight"]
    if canonical == "final_norm.weight":
        return ["token_embd_norm.weight"]
    unmapped = _api().WeightError(f"{canonical}: unmapped LFM2-MoE GGUF tensor")
    parts = canonical.split(".")
    if len(parts) == 5 and parts[0] == "layers" and parts[2] == "moe":
        at = f"blk.{parts[1]}."
        table = {"router": [at + "ffn_gate_inp.weight"], "router_bias": [at + "exp_probs_b.bias"],
                 "input": [at + "ffn_gate_exps.weight", at + "ffn_up_exps.weight"],
                 "output": [at + "ffn_down_exps.weight"]}
        if parts[3] not in table:
            raise unmapped
        return table[parts[3]]
    if not parts or parts[0] != "layers":
        raise unmapped
    tail = tuple(parts[2:])
    if len(tail) == 2 and tail[1] == "weight" and tail[0] in _COMPONENTS:
        component = _COMPONENTS[tail[0]]
    elif tail in (("conv", "in_proj", "weight"), ("conv", "depthwise", "weight"), ("conv", "out_proj", "weight")):
        component = {"in_proj": "shortconv.in_proj", "depthwise": "shortconv.conv", "out_proj": "shortconv.out_proj"}[tail[1]]
    else:
        raise unmapped
    return [f"blk.{parts[1]}.{component}.weight"]


@dataclass
class Binding:
    """One canonical weight of the model and the tensor(s) of the file that hold it."""
    canonical: str
    sources: tuple
    shape: list               # logical: [rows, cols], [experts, rows, cols], [n] ...
    kind: str                 # "dense", "quantized", "experts" or "stacked_experts"
    type_id: int


@dataclass
class TensorPlan:
    bindings: list
    redundant_output: bool            # a tied model whose file also carries output.weight
    tensor_count: int
    source_tensor_bytes: int
    parameter_count: int

    def binding(self, canonical: str) -> Binding:
        for b in self.bindings:
            if b.canonical == canonical:
                return b
        raise _api().WeightError(f"{canonical}: missing mapped tensor")

    def quantized(self) -> list:
        return [b for b in self.bindings if b.kind != "dense"]


# ---- metadata ------------------------------------------------------------------------

def _meta(reader, key: str):
    value = reader.metadata_value(key)
    if value is None:
        raise _api().GgufError(f"missing metadata key {key}")
    return value


def _meta_string(reader, key: str) -> str:
    value = _meta(reader, key)
    if value.type_id != 8:
        raise _api().GgufError(f"metadata key {key} is not a string")
    return value.value


def _meta_usize(reader, key: str) -> int:
    value = _meta(reader, key)
    if value.type_id not in (0, 1, 2, 3, 4, 5, 10, 11) or value.value < 0:
        raise _api().GgufError(f"metadata key {key} is not a non-negative integer")
    return int(value.value)


def _meta_f32(reader, key: str) -> float:
    value = _meta(reader, key)
    if value.type_id not in (6, 12):
        raise _api().GgufError(f"metadata key {key} is not a float")
    return float(value.value)


def _logical_shape(info, depthwise: bool = False) -> list[int]:
    """GGUF dimensions are fastest-first (source_shape, qwen_gguf.rs:344-354 and
    lfm2_moe/gguf.rs:384-405)."""
    d = list(info.dimensions)
    if len(d) == 1:
        return d
    if len(d) == 2:
        return [d[1], 1, d[0]] if depthwise else [d[1], d[0]]
    if len(d) == 3:
        return [d[2], d[1], d[0]]
    raise _api().WeightError(f"{info.name}: unsupported GGUF tensor rank {len(d)}")


def _totals(reader, skip) -> tuple[int, int, int]:
    count = source_bytes = parameters = 0
    for name, info in reader.tensors.items():
        count += 1
        source_bytes += info.byte_len
        if not skip(name):
            elements = 1
            for d in info.dimensions:
                elements *= d
            parameters += elements
    return count, source_bytes, parameters


# ---- Qwen2 / Qwen3 -------------------------------------------------------------------

def plan_qwen(reader) -> tuple[ModelShape, TensorPlan]:
    """The model shape a Qwen2 / Qwen3 file declares and the binding of its tensors
    (src/model/qwen_gguf.rs:32-222)."""
    api = _api()
    architecture = _meta_string(reader, "general.architecture")
    if architecture not in ("qwen2", "qwen3"):
        raise api.ConfigError(f'GGUF architecture "{architecture}" is unsupported; expected qwen2 or qwen3')
    qwen3 = architecture == "qwen3"
    tied = reader.tensors_equal_payload("token_embd.weight", "output.weight") if "output.weight" in reader.tensors else True
    embedding = reader.tensor("token_embd.weight")
    vocab, width = embedding.logical_matrix_shape()
    hidden = _meta_usize(reader, f"{architecture}.embedding_length")
    if width != hidden:
        raise api.ConfigError(f"token_embd.weight hidden dimension {width} differs from metadata {hidden}")
    heads = _meta_usize(reader, f"{architecture}.attention.head_count")
    kv_heads = _meta_usize(reader, f"{architecture}.attention.head_count_kv")
    if qwen3:
        head_dim = _meta_usize(reader, "qwen3.attention.key_length")
        if _meta_usize(reader, "qwen3.attention.value_length") != head_dim:
            raise api.ConfigError("Qwen3 K/V head dimensions must match")
    elif reader.metadata_value("qwen2.rope.dimension_count") is not None:
        head_dim = _meta_usize(reader, "qwen2.rope.dimension_count")
    elif heads != 0 and hidden % heads == 0:
        head_dim = hidden // heads
    else:
        raise api.ConfigError("cannot infer head dimension from Qwen2 metadata")
    intermediate = _meta_usize(reader, f"{architecture}.feed_forward_length")
    layers = _meta_usize(reader, f"{architecture}.block_count")
    shape = ModelShape(vocab_size=vocab, hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=kv_heads,
                       head_dim=head_dim, tie_word_embeddings=tied,
                       layers=[LayerShape(intermediate_size=intermediate) for _ in range(layers)],
                       qk_norm="per_head" if qwen3 else None, qkv_bias=not qwen3, architecture=architecture)
    if min(vocab, hidden, heads, kv_heads, head_dim, intermediate, layers) == 0 or heads % kv_heads != 0:
        raise api.ConfigError("invalid Qwen model geometry")

    expected = [(qwen_source_name(c), c, dims) for c, dims in specifications(shape)]
    redundant_output = tied and "output.weight" in reader.tensors
    if shape.qkv_bias:
        for l in range(layers):
            for short, length in (("q", heads * head_dim), ("k", kv_heads * head_dim), ("v", kv_heads * head_dim)):
                expected.append((f"blk.{l}.attn_{short}.bias", f"layers.{l}.{short}.bias", [length]))
    if "output.bias" in reader.tensors:
        if qwen3:
            raise api.WeightError("output.bias: Qwen3 output projection has no bias")
        expected.append(("output.bias", "lm_head.bias", [vocab]))
    names = {source for source, _, _ in expected}
    bindings = []
    for source, canonical, dims in expected:
        info = reader.tensor(source)
        found = _logical_shape(info)
        if len(info.dimensions) > 2:
            raise api.WeightError(f"{source}: unsupported Qwen tensor rank {len(info.dimensions)}")
        if found != dims:
            raise api.WeightError(f"{source}: expected shape {dims}, found {found}")
        if info.type_id in DENSE_TYPES:
            kind = "dense"
        elif info.type_id in QWEN_QUANTIZED_TYPES and len(dims) == 2:
            kind = "quantized"
        else:
            raise api.WeightError(f"{source}: unsupported GGML type {info.type_id} for Qwen tensor")
        bindings.append(Binding(canonical, (source,), dims, kind, info.type_id))
    for name in reader.tensors:
        if name not in names and not (redundant_output and name == "output.weight"):
            raise api.WeightError(f"{name}: unexpected tensor for supported Qwen GGUF contract")
    count, source_bytes, parameters = _totals(reader, lambda n: redundant_output and n == "output.weight")
    return shape, TensorPlan(bindings, redundant_output, count, source_bytes, parameters)


# ---- LFM2-MoE ------------------------------------------------------------------------

def lfm2_moe_shape(reader, use_expert_bias: bool = True, tie_word_embeddings: bool = True) -> ModelShape:
    """The model shape an LFM2-MoE file's metadata declares: the keys validate_metadata
    compares with the companion config (src/model/lfm2_moe/gguf.rs:93-163).  Layers whose
    entry in the per-layer KV-head schedule is zero are short convolutions; the first
    `leading_dense_block_count` layers are dense, the rest sparse."""
    api = _api()
    if _meta_string(reader, "general.architecture") != "lfm2moe":
        raise api.ConfigError("LFM2-MoE GGUF metadata differs from the companion official config")
    if _meta_usize(reader, "lfm2moe.expert_gating_func") != 2:
        raise api.ConfigError("LFM2-MoE GGUF metadata differs from the companion official config")
    hidden = _meta_usize(reader, "lfm2moe.embedding_length")
    heads = _meta_usize(reader, "lfm2moe.attention.head_count")
    layers = _meta_usize(reader, "lfm2moe.block_count")
    schedule = _meta(reader, "lfm2moe.attention.head_count_kv")
    if schedule.type_id != 9 or len(schedule.value) != layers:
        raise api.ConfigError("LFM2-MoE GGUF per-layer KV-head schedule differs from config")
    kv = [int(v) for v in schedule.value]
    live = {v for v in kv if v != 0}
    if len(live) != 1 or heads == 0 or hidden % heads != 0:
        raise api.ConfigError("LFM2-MoE GGUF per-layer KV-head schedule differs from config")
    dense_layers = _meta_usize(reader, "lfm2moe.leading_dense_block_count")
    sparse = SparseFeedForward(_meta_usize(reader, "lfm2moe.expert_count"),
                               _meta_usize(reader, "lfm2moe.expert_feed_forward_length"), use_expert_bias)
    intermediate = _meta_usize(reader, "lfm2moe.feed_forward_length")
    taps = _meta_usize(reader, "lfm2moe.shortconv.l_cache")
    return ModelShape(
        vocab_size=_meta_usize(reader, "lfm2moe.vocab_size"), hidden_size=hidden, num_attention_heads=heads,
        num_key_value_heads=live.pop(), head_dim=hidden // heads, tie_word_embeddings=tie_word_embeddings,
        layers=[LayerShape(intermediate_size=intermediate, short_conv_kernel=None if kv[l] else taps,
                           sparse=None if l < dense_layers else sparse) for l in range(layers)],
        qk_norm="per_head", qkv_bias=False, architecture="lfm2moe")


def plan_lfm2_moe(reader, shape: ModelShape) -> TensorPlan:
    """Binding of an LFM2-MoE file's tensors (map_gguf_weights,
    src/model/lfm2_moe/gguf.rs:165-320)."""
    api = _api()
    redundant_output = shape.tie_word_embeddings and "output.weight" in reader.tensors
    if redundant_output and not reader.tensors_equal_payload("token_embd.weight", "output.weight"):
        raise api.WeightError("output.weight: tied GGUF output weights differ from token embeddings")
    specs = specifications(shape)
    expected = {source for canonical, _ in specs for source in lfm2_moe_source_names(canonical)}
    if redundant_output:
        expected.add("output.weight")
    for name in reader.tensors:
        if name not in expected:
            raise api.WeightError(f"{name}: unexpected tensor for the supported LFM2-MoE GGUF contract")

    def expert_component(name: str, want: list[int]):
        info = reader.tensor(name)
        if info.logical_expert_shape() != want:
            raise api.WeightError(f"{name}: expected logical expert shape {want}, found {info.logical_expert_shape()}")
        if info.type_id not in EXPERT_TYPES:
            raise api.WeightError(f"{name}: LFM2-MoE GGUF expert projections must use Q4_K, Q5_K, or Q6_K")
        return info

    bindings = []
    for canonical, dims in specs:
        sources = lfm2_moe_source_names(canonical)
        if canonical.endswith(".moe.input.weight") or canonical.endswith(".moe.output.weight"):
            sparse = shape.layers[int(canonical.split(".")[1])].sparse
            if sparse is None:
                raise api.ConfigError("GGUF expert tensor targets a dense layer")
            if canonical.endswith(".moe.input.weight"):
                want = [sparse.experts, sparse.intermediate_size, shape.hidden_size]
                gate, up = (expert_component(name, want) for name in sources)
                if gate.type_id != up.type_id:
                    raise api.WeightError(f"{canonical}: gate/up expert tensors use different quantization formats")
                bindings.append(Binding(canonical, tuple(sources), dims, "stacked_experts", gate.type_id))
            else:
                info = expert_component(sources[0], [sparse.experts, shape.hidden_size, sparse.intermediate_size])
                bindings.append(Binding(canonical, tuple(sources), dims, "experts", info.type_id))
            continue
        info = reader.tensor(sources[0])
        found = _logical_shape(info, depthwise=canonical.endswith(".conv.depthwise.weight"))
        if found != dims:
            raise api.WeightError(f"{sources[0]}: expected logical shape {dims}, found {found}")
        if info.type_id in DENSE_TYPES:
            kind = "dense"
        elif info.type_id in QWEN_QUANTIZED_TYPES:
            if len(dims) != 2:
                raise api.WeightError(f"{sources[0]}: quantized non-expert GGUF tensors must be matrices")
            kind = "quantized"
        else:
            raise api.WeightError(f"{sources[0]}: unsupported GGML tensor type {info.type_id}")
        bindings.append(Binding(canonical, tuple(sources), dims, kind, info.type_id))
    count, source_bytes, parameters = _totals(
        reader, lambda n: n.endswith(".exp_probs_b.bias") or (redundant_output and n == "output.weight"))
    return TensorPlan(bindings, redundant_output, count, source_bytes, parameters)


# ---- device -------------------------------------------------------------------------

def bind_quantized(device, reader, plan: TensorPlan, only: tuple | None = None):
    """Uploads the plan's quantized tensors, blocks verbatim (gate and up experts interleaved
    per expert): {canonical name: QuantizedMatrix | QuantizedExpertMatrix} and the bytes
    they hold on the device (`quantized_tensor_bytes` of the reference's loaders).  `only`
    restricts the upload to the given GGML type ids: formats this library has no kernels
    for (the legacy 32-weight formats other than Q8_0) are refused by the upload itself."""
    weights, total = {}, 0
    for b in plan.quantized():
        if only is not None and b.type_id not in only:
            continue
        if b.kind == "quantized":
            w = reader.quantized_matrix(device, b.sources[0])
            if [w.rows(), w.columns()] != b.shape:
                raise _api().WeightError(f"{b.canonical}: packed matrix shape differs from model policy")
        elif b.kind == "experts":
            w = reader.quantized_expert_matrix(device, b.sources[0])
        else:
            w = reader.quantized_input_experts(device, b.sources[0], b.sources[1])
        if b.kind != "quantized" and [w.experts(), w.rows_per_expert(), w.columns()] != b.shape:
            raise _api().WeightError(f"{b.canonical}: packed gate/up expert shape differs from model policy")
        weights[b.canonical] = w
        total += w.byte_size()
    return weights, total
