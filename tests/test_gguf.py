"""The GGUF reader against the cases of the reference's own reader tests
(src/loader/gguf.rs:750-979) plus K-quant files of the hot path's shapes."""
import numpy as np
import pytest

import gguf_files as gf
from ferrum_amd import api, gguf, synth


def read(data, **kw):
    return gguf.GgufReader.from_bytes(data, **kw)


def test_reads_aligned_q8_0_tensor_without_reordering_payload():
    f = read(gf.reference_fixture(8, [32, 2], [0], ["blk.0.attn_q.weight"]))
    t = f.tensor("blk.0.attn_q.weight")
    assert (t.type_id, t.byte_len) == (8, 68)
    assert t.logical_matrix_shape() == [2, 32]
    out = np.zeros(68, np.uint8)
    f.read_tensor_into("blk.0.attn_q.weight", out)
    assert (out == 1).all()
    with pytest.raises(api.GgufError):
        f.read_tensor_into("blk.0.attn_q.weight", np.zeros(67, np.uint8))
    with pytest.raises(api.GgufError, match="missing tensor"):
        f.tensor("absent")


def test_expert_tensor_shape_reverses_gguf_dimension_order():
    t = gguf.TensorInfo("blk.2.ffn_gate_exps.weight", [2048, 1792, 32], 12, 0, 0)
    assert t.logical_expert_shape() == [32, 1792, 2048]
    with pytest.raises(api.GgufError):
        t.logical_matrix_shape()
    with pytest.raises(api.GgufError):
        gguf.TensorInfo("m", [2048, 1792], 12, 0, 0).logical_expert_shape()


def test_compares_tensor_aliases_with_bounded_reads():
    data = bytearray(gf.reference_fixture(8, [32, 2], [0, 96], ["input.weight", "output.weight"]))
    start = read(bytes(data)).tensor_data_offset
    data[start + 96:start + 164] = data[start:start + 68]
    assert read(bytes(data)).tensors_equal_payload("input.weight", "output.weight")
    data[start + 120] ^= 1
    assert not read(bytes(data)).tensors_equal_payload("input.weight", "output.weight")


def test_rejects_bad_magic_and_truncated_header():
    bad = bytearray(gf.reference_fixture(8, [32, 2], [0], ["weight"]))
    bad[0] = ord("X")
    with pytest.raises(api.GgufError, match="magic"):
        read(bytes(bad))
    with pytest.raises(api.GgufError, match="end of file"):
        read(b"GGUF\x03\0")
    with pytest.raises(api.GgufError, match="version"):
        read(b"GGUF" + bytes([1, 0, 0, 0]) + bytes(16))


def test_rejects_unaligned_offsets_and_non_block_dimensions():
    with pytest.raises(api.GgufError, match="not aligned"):
        read(gf.reference_fixture(8, [32, 2], [1], ["weight"]))
    with pytest.raises(api.GgufError, match="block size"):
        read(gf.reference_fixture(8, [31, 2], [0], ["weight"]))


def test_rejects_unknown_quantization_and_overlapping_ranges():
    with pytest.raises(api.GgufError, match="unsupported GGML tensor type 99"):
        read(gf.reference_fixture(99, [32, 2], [0], ["weight"]))
    with pytest.raises(api.GgufError, match="ranges overlap"):
        read(gf.reference_fixture(8, [32, 2], [0, 0], ["weight.a", "weight.b"]))


def test_block_sizes_match_the_ggml_layouts():
    table = {8: (32, 34), 14: (256, 210), 13: (256, 176), 12: (256, 144), 18: (256, 98), 21: (256, 110),
             22: (256, 82), 0: (1, 4), 1: (1, 2), 30: (1, 2), 2: (32, 18), 10: (256, 84), 42: (64, 18)}
    for type_id, layout in table.items():
        assert gguf.block_layout(type_id) == layout, type_id
    for absent in (4, 5, 16, 17, 19, 24, 99):
        with pytest.raises(api.GgufError):
            gguf.block_layout(absent)


def test_an_untagged_file_opens_only_on_request():
    name = "model.diffusion_model.transformer_blocks.10.img_mlp.gate_up.weight"
    assert len(name) > 64
    data = gf.header([(name, [32, 1], 8, 0)], [])
    data += bytes(-len(data) % 32) + bytes(34)
    with pytest.raises(api.GgufError):
        read(bytes(data))
    assert read(bytes(data), require_architecture=False).tensor(name).dimensions == [32, 1]


def test_skipping_arrays_keeps_everything_else():
    metadata = [("general.architecture", gf.STRING, "qwen2"),
                ("tokenizer.ggml.tokens", gf.ARRAY, ["a", "bc", "def"], gf.STRING),
                ("tokenizer.ggml.token_type", gf.ARRAY, list(range(5)), gf.I32),
                ("qwen2.rope.dimension_sections", gf.ARRAY, [11, 12], gf.U32)]
    data = gf.header([("w", [4], 0, 0)], metadata)
    data += bytes(-len(data) % 32) + bytes([7]) * 16
    full, skim = read(bytes(data)), read(bytes(data), max_array_items=2)
    assert full.metadata_value("tokenizer.ggml.tokens").value == ["a", "bc", "def"]
    assert full.metadata_value("tokenizer.ggml.token_type").value == [0, 1, 2, 3, 4]
    assert skim.metadata_value("tokenizer.ggml.tokens").value == []
    assert skim.metadata_value("tokenizer.ggml.token_type").value == []
    assert skim.metadata_value("qwen2.rope.dimension_sections") == full.metadata_value("qwen2.rope.dimension_sections")
    assert skim.tensor("w") == full.tensor("w")
    out = np.zeros(16, np.uint8)
    skim.read_tensor_into("w", out)
    assert (out == 7).all()


def test_metadata_scalars_of_every_type_round_trip():
    metadata = gf.STANDARD + [("a.u8", gf.U8, 200), ("a.i8", gf.I8, -3), ("a.u16", gf.U16, 60000),
                              ("a.i16", gf.I16, -12345), ("a.i32", gf.I32, -7), ("a.f32", gf.F32, 0.5),
                              ("a.bool", gf.BOOL, 1), ("a.u64", gf.U64, 1 << 40), ("a.i64", gf.I64, -(1 << 40)),
                              ("a.f64", gf.F64, 1e-300), ("general.alignment", gf.U32, 64)]
    f = read(gf.build([("w", [256, 3], 12, synth.matrix(12, 3, 256, seed=5))], metadata, alignment=64))
    got = {k: v.value for k, v in f.metadata.items() if k.startswith("a.")}
    assert got == {"a.u8": 200, "a.i8": -3, "a.u16": 60000, "a.i16": -12345, "a.i32": -7, "a.f32": 0.5,
                   "a.bool": True, "a.u64": 1 << 40, "a.i64": -(1 << 40), "a.f64": 1e-300}
    assert f.alignment == 64 and f.tensor_data_offset % 64 == 0 and f.version == 3


def test_header_rules():
    q4 = synth.matrix(12, 2, 256, seed=1)
    ok = [("w", [256, 2], 12, q4)]
    with pytest.raises(api.GgufError, match="quantization_version"):
        read(gf.build(ok, [("general.architecture", gf.STRING, "qwen2")]))
    with pytest.raises(api.GgufError, match="architecture"):
        read(gf.build(ok, [("general.quantization_version", gf.U32, 2)]))
    with pytest.raises(api.GgufError, match="alignment"):
        read(gf.build(ok, gf.STANDARD + [("general.alignment", gf.U32, 12)], alignment=12))
    with pytest.raises(api.GgufError, match="uint32"):
        read(gf.build(ok, gf.STANDARD + [("general.alignment", gf.U64, 32)]))
    with pytest.raises(api.GgufError, match="duplicate metadata key"):
        read(gf.build(ok, gf.STANDARD + [("general.architecture", gf.STRING, "x")]))
    with pytest.raises(api.GgufError, match="duplicate tensor name"):
        read(gf.build(ok + ok))
    with pytest.raises(api.GgufError, match="rank"):
        read(gf.build([("w", [256, 1, 1, 1, 2], 12, q4)]))
    with pytest.raises(api.GgufError, match="empty dimension"):
        read(gf.build([("w", [256, 0], 12, np.zeros(0, np.uint8))]))
    with pytest.raises(api.GgufError, match="name exceeds"):
        read(gf.build([("n" * 65, [256, 2], 12, q4)]))
    with pytest.raises(api.GgufError, match="exceeds file length"):
        read(gf.build(ok)[:-1])
    with pytest.raises(api.GgufError, match="bool"):
        read(gf.build(ok, gf.STANDARD + [("flag", gf.BOOL, 2)]))
    nested = bytearray(gf.header([], [("general.architecture", gf.STRING, "q")]))
    nested[16:24] = (2).to_bytes(8, "little")
    nested += gf.string("k") + (9).to_bytes(4, "little") + (9).to_bytes(4, "little") + (0).to_bytes(8, "little")
    with pytest.raises(api.GgufError):
        read(bytes(nested))
    assert read(gf.build(ok, version=2)).version == 2


def test_k_quant_tensors_come_back_verbatim_and_streamed(tmp_path):
    q4 = synth.matrix(12, 7, 512, seed=11)
    q6 = synth.matrix(14, 5, 768, seed=12)
    ex = synth.matrix(12, 3 * 4, 256, seed=13)
    path = tmp_path / "weights.gguf"
    path.write_bytes(gf.build([("blk.0.ffn_up.weight", [512, 7], 12, q4), ("output.weight", [768, 5], 14, q6),
                               ("blk.0.ffn_up_exps.weight", [256, 4, 3], 12, ex)]))
    f = gguf.GgufReader.open(str(path))
    assert f.tensor("blk.0.ffn_up.weight").logical_matrix_shape() == [7, 512]
    assert f.tensor("blk.0.ffn_up_exps.weight").logical_expert_shape() == [3, 4, 256]
    for name, want in (("blk.0.ffn_up.weight", q4), ("output.weight", q6), ("blk.0.ffn_up_exps.weight", ex)):
        info = f.tensor(name)
        assert info.byte_len == want.size and (f.tensor_data_offset + info.offset) % 32 == 0
        out = np.zeros(info.byte_len, np.uint8)
        f.read_tensor_into(name, out)
        assert np.array_equal(out, want.reshape(-1))
        pieces = []
        f.stream_tensor(name, 1000, lambda offset, data: pieces.append((offset, data)))
        assert [o for o, _ in pieces] == list(range(0, want.size, 1000))
        assert b"".join(p for _, p in pieces) == want.tobytes()
    with pytest.raises(api.GgufError):
        f.stream_tensor("output.weight", 0, lambda *_: None)
    with pytest.raises(api.GgufError):
        gguf.GgufReader.open(str(tmp_path / "absent.gguf"))


# ---- the C++ reader (include/ferrum_gguf.hpp) against the Python one ----------------

@pytest.fixture(scope="module")
def probe():
    from ferrum_amd import build
    return build.build_gguf_probe()


def _describe(f):
    def show(v):
        if v.type_id == gf.ARRAY:
            return "[" + "".join(show(gguf.MetadataValue(v.element_type, item)) + "," for item in v.value) + "]"
        if v.type_id in (gf.F32, gf.F64):
            return "%.17g" % v.value
        return str(v.value)

    lines = [f"version {f.version} alignment {f.alignment} data {f.tensor_data_offset}"]
    lines += [f"meta {k} {v.type_id} {show(v)}" for k, v in sorted(f.metadata.items())]
    for name, t in sorted(f.tensors.items()):
        raw = np.zeros(t.byte_len, np.uint8)
        f.read_tensor_into(name, raw)
        h = 1469598103934665603
        for b in raw.tolist():
            h = ((h ^ b) * 1099511628211) & (2**64 - 1)
        dims = " ".join(str(x) for x in t.dimensions)
        lines.append(f"tensor {name} type {t.type_id} offset {t.offset} bytes {t.byte_len} dims {dims} "
                     f"fnv {h:016x} stream-ok")
    return lines


def test_cpp_reader_agrees_with_the_python_reader(probe, tmp_path):
    import subprocess
    metadata = gf.STANDARD + [("a.u8", gf.U8, 200), ("a.i8", gf.I8, -3), ("a.i16", gf.I16, -12345),
                              ("a.f32", gf.F32, 0.1), ("a.bool", gf.BOOL, 1), ("a.u64", gf.U64, 1 << 40),
                              ("a.i64", gf.I64, -(1 << 40)), ("a.f64", gf.F64, 1e-300),
                              ("tokenizer.ggml.tokens", gf.ARRAY, ["a", "bc", "déf"], gf.STRING),
                              ("tokenizer.ggml.token_type", gf.ARRAY, [1, -2, 3], gf.I32),
                              ("general.alignment", gf.U32, 64)]
    tensors = [("blk.0.ffn_up.weight", [512, 7], 12, synth.matrix(12, 7, 512, seed=11)),
               ("output.weight", [768, 5], 14, synth.matrix(14, 5, 768, seed=12)),
               ("blk.0.ffn_up_exps.weight", [256, 4, 3], 12, synth.matrix(12, 12, 256, seed=13)),
               ("norm.weight", [6], 0, np.arange(6, dtype=np.float32).view(np.uint8))]
    good = gf.build(tensors, metadata, alignment=64)
    cases = {"good": (good, [], 0), "skim": (good, ["2"], 0),
             "v2": (gf.build(tensors[:1], version=2), [], 0),
             "magic": (b"XGUF" + good[4:], [], 2), "short": (b"GGUF\x03\0", [], 2), "cut": (good[:-64], [], 2),
             "version": (b"GGUF\x07\0\0\0" + good[8:], [], 2),
             "unaligned": (gf.reference_fixture(8, [32, 2], [1], ["weight"]), [], 2),
             "tail": (gf.reference_fixture(8, [31, 2], [0], ["weight"]), [], 2),
             "type": (gf.reference_fixture(99, [32, 2], [0], ["weight"]), [], 2),
             "overlap": (gf.reference_fixture(8, [32, 2], [0, 0], ["weight.a", "weight.b"]), [], 2),
             "noversion": (gf.build(tensors[:1], [("general.architecture", gf.STRING, "q")]), [], 2),
             "noarch": (gf.build(tensors[3:], []), [], 2), "untagged": (gf.build(tensors[3:], []), ["0", "untagged"], 0),
             "dupkey": (gf.build(tensors[:1], gf.STANDARD + gf.STANDARD[:1]), [], 2),
             "dupname": (gf.build(tensors[:1] * 2), [], 2),
             "align12": (gf.build(tensors[:1], gf.STANDARD + [("general.alignment", gf.U32, 12)], alignment=12), [], 2),
             "bool": (gf.build(tensors[:1], gf.STANDARD + [("flag", gf.BOOL, 2)]), [], 2),
             "utf8": (gf.build(tensors[:1], gf.STANDARD + [("bad", gf.STRING, b"\xc3\x28")]), [], 2),
             "rank": (gf.build([("w", [256, 1, 1, 1, 2], 12, tensors[0][3][:288])]), [], 2),
             "longname": (gf.build([("n" * 65, [256, 2], 12, tensors[0][3][:288])]), [], 2)}
    for label, (data, args, code) in cases.items():
        path = tmp_path / f"{label}.gguf"
        path.write_bytes(data)
        proc = subprocess.run([probe, str(path), *args], capture_output=True, text=True, timeout=30)
        assert proc.returncode == code, (label, proc.stdout, proc.stderr)
        if code:
            with pytest.raises(api.GgufError):
                read(data)
            continue
        kw = {}
        if args:
            kw = {"max_array_items": int(args[0])} if len(args) == 1 else {"require_architecture": False}
        assert proc.stdout.splitlines() == _describe(read(data, **kw)), label


def test_both_readers_survive_truncated_and_corrupted_files(tmp_path):
    # an untrusted file may be cut anywhere or carry any byte: the C++ reader, built under
    # AddressSanitizer and UBSan, must either read it or refuse it (exit 0 or 2, never a report
    # or a crash), and the Python reader must do the same with GgufError
    import subprocess
    from ferrum_amd import build
    probe = build.build_gguf_probe(sanitize=True)
    metadata = gf.STANDARD + [("tokenizer.ggml.tokens", gf.ARRAY, ["a", "bc"], gf.STRING),
                              ("general.alignment", gf.U32, 32), ("x.f64", gf.F64, 2.5)]
    tensors = [("blk.0.ffn_up.weight", [256, 3], 12, synth.matrix(12, 3, 256, seed=21)),
               ("blk.0.ffn_up_exps.weight", [256, 2, 2], 23, synth.matrix(23, 4, 256, seed=22)),
               ("norm.weight", [4], 0, np.arange(4, dtype=np.float32).view(np.uint8))]
    good = gf.build(tensors, metadata)
    header = len(good) - 32 * -(-(3 * 144 + 4 * 136 + 16 + 64) // 32)      # at most: where the tensor data starts
    header = max(header, 200)
    rng = np.random.default_rng(7)
    variants = [good[:n] for n in range(0, min(len(good), header + 40), 5)]
    for _ in range(250):
        data = bytearray(good)
        at = int(rng.integers(0, header))
        data[at] = int(rng.integers(0, 256))
        variants.append(bytes(data))
    for _ in range(60):                                       # a huge count or length field
        data = bytearray(good)
        at = int(rng.integers(8, header - 8))
        data[at:at + 8] = int(rng.integers(1 << 40, 1 << 63)).to_bytes(8, "little")
        variants.append(bytes(data))
    path = tmp_path / "case.gguf"
    outcomes = {0: 0, 2: 0}
    for i, data in enumerate(variants):
        path.write_bytes(data)
        proc = subprocess.run([probe, str(path)], capture_output=True, text=True, timeout=30)
        assert proc.returncode in (0, 2), (i, len(data), proc.returncode, proc.stderr[-600:])
        outcomes[proc.returncode] += 1
        try:
            read(data)
            ok = True
        except api.GgufError:
            ok = False
        assert ok == (proc.returncode == 0), (i, len(data), proc.returncode)
    assert outcomes[0] > 0 and outcomes[2] > 100


def test_gate_and_up_expert_tensors_interleave_per_expert(probe, tmp_path):
    # load_quantized_input_experts (src/model/lfm2_moe/gguf.rs:466-534): [E, I, H] + [E, I, H] -> [E, 2I, H]
    import subprocess
    experts, inter, hidden = 3, 70, 512          # 70 rows per expert: chunks of 64 rows cross expert boundaries
    gate = synth.matrix(12, experts * inter, hidden, seed=31)
    up = synth.matrix(12, experts * inter, hidden, seed=32)
    path = tmp_path / "experts.gguf"
    path.write_bytes(gf.build([("blk.0.ffn_gate_exps.weight", [hidden, inter, experts], 12, gate),
                               ("blk.0.ffn_up_exps.weight", [hidden, inter, experts], 12, up),
                               ("blk.0.ffn_down_exps.weight", [inter * 0 + 256, hidden, experts], 12,
                                synth.matrix(12, experts * hidden, 256, seed=33))]))
    f = gguf.GgufReader.open(str(path))
    payload, fmt, e, rows, cols = f.read_stacked_experts("blk.0.ffn_gate_exps.weight", "blk.0.ffn_up_exps.weight")
    assert (fmt, e, rows, cols) == (api.QuantizationFormat.Q4_K, experts, 2 * inter, hidden)
    row_bytes = hidden // 256 * 144
    want = np.concatenate([gate.reshape(experts, inter, row_bytes), up.reshape(experts, inter, row_bytes)], axis=1)
    assert np.array_equal(payload.reshape(experts, 2 * inter, row_bytes), want)
    with pytest.raises(api.WeightError):
        f.read_stacked_experts("blk.0.ffn_gate_exps.weight", "blk.0.ffn_down_exps.weight")
    h = 1469598103934665603
    for b in payload.tolist():
        h = ((h ^ b) * 1099511628211) & (2**64 - 1)
    proc = subprocess.run([probe, str(path), "stack", "blk.0.ffn_gate_exps.weight", "blk.0.ffn_up_exps.weight"],
                          capture_output=True, text=True, timeout=30)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert proc.stdout.strip() == f"stacked {experts} {2 * inter} {hidden} fnv {h:016x}"
