"""The EXL3 checkpoint reader (libberth_exl3_reader.so through berth_amd.exl3) on the
reference's own reader tests, restated case by case:
  crates/berth-exl3/tests/synthetic.rs      (synthetic checkpoints written to a temp dir)
  crates/berth-exl3/src/config.rs:421-550   (config.json unit tests)
  crates/berth-exl3/src/signs.rs:48-92      (sign unpack known answers)
  crates/berth-exl3/tests/qwen38_27b.rs     (shapes and byte lengths of the real 27B
                                             checkpoint, rebuilt here as a sparse shard)
Host only: nothing here touches a GPU.
"""
import copy
import json
import os
import struct

import numpy as np
import pytest

from berth_amd import exl3
from berth_amd.exl3 import (FP16_NEG_ONE, FP16_ONE, Bitrate, Checkpoint, Codebook, DType, Error, ErrorKind, LayerType,
                            ModelConfig)

CONFIG = {
    "architectures": ["TestForCausalLM"],
    "ignored_top": True,
    "text_config": {
        "num_hidden_layers": 2, "hidden_size": 32, "intermediate_size": 64, "head_dim": 16,
        "num_attention_heads": 2, "num_key_value_heads": 1, "vocab_size": 128, "tie_word_embeddings": False,
        "layer_types": ["linear_attention", "full_attention"], "linear_conv_kernel_dim": 4,
        "linear_num_key_heads": 16, "linear_num_value_heads": 32, "linear_key_head_dim": 128,
        "linear_value_head_dim": 128, "attn_output_gate": False, "num_experts": 4, "num_experts_per_tok": 2,
        "moe_intermediate_size": 8, "shared_expert_intermediate_size": 16,
    },
    "quantization_config": {"quant_method": "exl3", "bits": 4, "head_bits": 6, "codebook": "mul1"},
}


def write_config(d, cfg=CONFIG):
    (d / "config.json").write_text(json.dumps(cfg))


def tensor(name, dtype, shape, data=None):
    n = int(np.prod(shape)) if shape else 1
    size = DType[dtype if dtype != "BF16" else "BF16"].size()
    return {"name": name, "dtype": dtype, "shape": list(shape), "data": data if data is not None else bytes(n * size)}


def words(*values):
    return b"".join(struct.pack("<H", v) for v in values)


def write_tensors(path, tensors, pad=0):
    data, entries = b"", []
    for t in tensors:
        start = len(data)
        data += t["data"]
        shape = ",".join(str(d) for d in t["shape"])
        entries.append(f'"{t["name"]}":{{"dtype":"{t["dtype"]}","shape":[{shape}],"data_offsets":[{start},{len(data)}]}}')
    header = ("{" + ",".join(entries) + "}" + " " * pad).encode()
    path.write_bytes(struct.pack("<Q", len(header)) + header + data)
    return len(header)


def write_raw(path, header: str, data: bytes):
    path.write_bytes(struct.pack("<Q", len(header)) + header.encode() + data)


def marker(name, dtype="I32"):
    return {"name": name, "dtype": dtype, "shape": [], "data": bytes([1, 0, 0, 0])}


def linear_parts(prefix, last, codebook, packed=False, bias=False, su_word=0, sv_word=0):
    parts = [tensor(f"{prefix}.trellis", "I16", [1, 1, last])]
    if packed:
        parts.append(tensor(f"{prefix}.su", "I16", [1], words(su_word)))
        parts.append(tensor(f"{prefix}.sv", "I16", [1], words(sv_word)))
    else:
        parts.append(tensor(f"{prefix}.suh", "F16", [4]))
        parts.append(tensor(f"{prefix}.svh", "F16", [4]))
    if codebook:
        parts.append(marker(f"{prefix}.{codebook}"))
    if bias:
        parts.append(tensor(f"{prefix}.bias", "F16", [2]))
    return parts


def others():
    return [tensor("model.norm.weight", "F16", [4]), tensor("model.norm.bias", "F16", [4]),
            tensor("model.layers.0.linear_attn.A_log", "F32", [2]),
            tensor("model.layers.0.linear_attn.dt_bias", "F32", [2]),
            tensor("model.layers.0.linear_attn.conv1d.weight", "BF16", [2, 1, 4]),
            tensor("model.embed.weight", "BF16", [2, 2])]


def demo_tensors():
    t = []
    t += linear_parts("block.0.down", 64, "mul1")
    t += linear_parts("block.1.q", 24, "mul1", packed=True, bias=True, su_word=0x0005, sv_word=0x8000)
    t += linear_parts("block.0.k", 64, "mcg")
    t += linear_parts("block.0.v", 64, None)
    t += linear_parts("wide.up", 128, "mul1")
    t += linear_parts("narrow.q", 16, "mul1")
    t += linear_parts("mid.o", 40, "mul1", packed=True)
    t += linear_parts("mid.down", 56, "mul1", packed=True)
    t += linear_parts("both.proj", 64, "mul1") + [tensor("both.proj.su", "I16", [1], words(0xFFFF))]
    t += others()
    return t


# ---- crates/berth-exl3/tests/synthetic.rs:318-424
def test_synthetic_checkpoint_groups_linears_and_unpacks_signs(tmp_path):
    write_config(tmp_path)
    shard = tmp_path / "model.safetensors"
    header = write_tensors(shard, demo_tensors())

    ckpt = Checkpoint.open(tmp_path)
    cfg = ckpt.config
    assert cfg.arch_string == "TestForCausalLM"
    assert cfg.hidden_size == 32
    assert cfg.intermediate_size == 64
    assert cfg.num_experts == 4
    assert cfg.shared_expert_intermediate_size == 16
    assert cfg.attn_output_gate is False
    assert sum(1 for kind, _ in cfg.layer_types if kind == LayerType.FULL_ATTENTION) == 1
    assert cfg.quantization.bits == 4.0

    assert len(ckpt.linears()) == 9
    by = {lin.prefix: lin for lin in ckpt.linears()}
    assert [lin.prefix for lin in ckpt.linears()] == sorted(by)
    assert by["block.0.down"].k == Bitrate.int(4)
    assert by["block.0.down"].codebook == Codebook.MUL1
    assert by["block.0.down"].bias is None
    assert not by["block.0.down"].input_scale.is_packed()

    half = by["block.1.q"]
    assert half.k == Bitrate.half(1)
    assert half.k.as_f64() == 1.5 and str(half.k) == "1.5"
    assert half.input_scale.is_packed()
    assert half.bias is not None and half.bias.dtype == DType.F16
    assert half.unpack_input_signs().tolist() == [FP16_NEG_ONE, FP16_ONE, FP16_NEG_ONE] + [FP16_ONE] * 13
    output = half.unpack_output_signs()
    assert output[15] == FP16_NEG_ONE and all(v == FP16_ONE for v in output[:15])

    assert by["block.0.k"].codebook == Codebook.MCG
    assert by["block.0.v"].codebook == Codebook.DEFAULT
    assert (by["block.0.k"].kernel_codebook, by["block.0.v"].kernel_codebook, by["wide.up"].kernel_codebook) == (1, 0, 2)
    assert by["wide.up"].k == Bitrate.int(8)
    assert by["narrow.q"].k == Bitrate.int(1)
    assert by["mid.o"].k == Bitrate.half(2)
    assert by["mid.down"].k == Bitrate.half(3)

    both = by["both.proj"]
    assert not both.input_scale.is_packed()
    with pytest.raises(Error, match="suh"):
        both.unpack_input_signs()
    assert ckpt.tensors.contains("both.proj.su")

    other_names = [t.name for t in ckpt.other_tensors()]
    for name in ("model.norm.weight", "model.norm.bias", "model.layers.0.linear_attn.A_log",
                 "model.layers.0.linear_attn.dt_bias", "model.layers.0.linear_attn.conv1d.weight",
                 "model.embed.weight"):
        assert name in other_names
    assert other_names == sorted(other_names)
    assert not any(n.endswith((".trellis", ".su", ".suh")) for n in other_names)

    trellis = ckpt.tensors.get("block.0.down.trellis")
    assert trellis.offset == 8 + header
    assert trellis.length == 128
    assert trellis.dtype == DType.I16
    assert trellis.shape == (1, 1, 64)
    suh = ckpt.tensors.get("block.0.down.suh")
    assert suh.offset == trellis.offset + trellis.length
    assert struct.unpack("<Q", shard.read_bytes()[:8])[0] == header
    assert [t.name for t in ckpt.tensors] == sorted(t["name"] for t in demo_tensors())
    assert len(ckpt.tensors) == len(demo_tensors())


# ---- synthetic.rs:426-437
def test_padded_header_still_locates_tensors(tmp_path):
    write_config(tmp_path)
    header = write_tensors(tmp_path / "model.safetensors", linear_parts("only.proj", 16, "mul1"), pad=7)
    ckpt = Checkpoint.open(tmp_path)
    assert ckpt.linears()[0].trellis.offset == 8 + header
    assert header > 7


# ---- synthetic.rs:439-493
def test_sharded_index_checks_total_size(tmp_path):
    write_config(tmp_path)
    shard_a = linear_parts("a.proj", 16, "mul1")
    shard_b = linear_parts("b.proj", 32, "mcg") + others()
    write_tensors(tmp_path / "model-00001-of-00002.safetensors", shard_a)
    write_tensors(tmp_path / "model-00002-of-00002.safetensors", shard_b)
    total = sum(len(t["data"]) for t in shard_a + shard_b)
    weight_map = {t["name"]: "model-00001-of-00002.safetensors" for t in shard_a}
    weight_map.update({t["name"]: "model-00002-of-00002.safetensors" for t in shard_b})
    (tmp_path / "model.safetensors.index.json").write_text(
        json.dumps({"metadata": {"total_size": total}, "weight_map": weight_map}))
    (tmp_path / "model.safetensors").write_bytes(b"not a checkpoint")     # a decoy that must be ignored

    ckpt = Checkpoint.open(tmp_path)
    assert len(ckpt.linears()) == 2
    assert ckpt.linears()[0].prefix == "a.proj"
    assert ckpt.linears()[1].codebook == Codebook.MCG
    assert ckpt.linears()[0].trellis.shard.endswith("model-00001-of-00002.safetensors")


def open_error(tmp_path, tensors):
    write_config(tmp_path)
    write_tensors(tmp_path / "model.safetensors", tensors)
    with pytest.raises(Error) as e:
        Checkpoint.open(tmp_path)
    return e.value


# ---- synthetic.rs:495-544
@pytest.mark.parametrize("tensors,needle", [
    (linear_parts("h.proj", 24, "mcg"), "mul1"),
    (linear_parts("h.proj", 64, "mul1") + [marker("h.proj.mcg")], "both mcg and mul1"),
    (linear_parts("h.proj", 144, "mul1"), "1..=8"),
    (linear_parts("h.proj", 72, "mul1"), "4.5"),
    (linear_parts("h.proj", 20, "mul1"), "16*K"),
    ([t for t in linear_parts("h.proj", 64, "mul1") if not t["name"].endswith((".suh", ".svh"))], "suh"),
])
def test_rejects_bad_linears(tmp_path, tensors, needle):
    err = open_error(tmp_path, tensors)
    assert needle in str(err)
    assert err.kind == ErrorKind.BAD_FIELD


def test_rejects_a_trellis_that_is_not_rank_3(tmp_path):
    bad = linear_parts("h.proj", 16, "mul1")
    bad[0] = tensor("h.proj.trellis", "I16", [16])
    assert "rank 3" in str(open_error(tmp_path, bad))


def test_exact_messages_follow_the_reference_text(tmp_path):
    # crates/berth-exl3/src/linear.rs:296-329, error.rs:12-14
    err = open_error(tmp_path, linear_parts("h.proj", 72, "mul1"))
    assert str(err) == ("field `h.proj.trellis`: half-integer bitrate 4.5 is not one of 1.5, 2.5, 3.5 (last dim 72)")
    assert err.field == "h.proj.trellis"


# ---- synthetic.rs:546-562
def test_rejects_a_mismatched_span_and_a_short_file(tmp_path):
    a, b = tmp_path / "a", tmp_path / "b"
    a.mkdir(), b.mkdir()
    write_config(a)
    write_raw(a / "model.safetensors", '{"h.proj.trellis":{"dtype":"I16","shape":[1],"data_offsets":[0,4]}}', bytes(4))
    with pytest.raises(Error, match="h.proj.trellis") as e:
        Checkpoint.open(a)
    assert "span 4 does not match I16 shape byte length 2" in str(e.value)
    write_config(b)
    write_raw(b / "model.safetensors", '{"h.proj.trellis":{"dtype":"I16","shape":[1],"data_offsets":[0,2]}}', b"")
    with pytest.raises(Error, match="h.proj.trellis") as e:
        Checkpoint.open(b)
    assert "but the shard is" in str(e.value)


# ---- synthetic.rs:564-601
def test_rejects_a_bad_index(tmp_path):
    write_config(tmp_path)
    parts = linear_parts("a.proj", 16, "mul1")
    shard = "model-00001-of-00002.safetensors"
    write_tensors(tmp_path / shard, parts)
    index = tmp_path / "model.safetensors.index.json"
    index.write_text(json.dumps({"metadata": {"total_size": 1}, "weight_map": {t["name"]: shard for t in parts}}))
    with pytest.raises(Error, match="total_size"):
        Checkpoint.open(tmp_path)

    index.write_text(json.dumps({"weight_map": {"missing.trellis": shard}}))
    with pytest.raises(Error) as e:
        Checkpoint.open(tmp_path)
    # header keys are visited in name order: the first tensor the index does not list is a.proj.mul1
    assert "a.proj.mul1" in str(e.value)

    index.write_text(json.dumps({"weight_map": {"a.proj.trellis": "../outside.safetensors"}}))
    with pytest.raises(Error, match="weight_map"):
        Checkpoint.open(tmp_path)
    index.write_text(json.dumps({"weight_map": {"a.proj.trellis": "/abs/outside.safetensors"}}))
    with pytest.raises(Error, match="weight_map"):
        Checkpoint.open(tmp_path)

    # a tensor the index lists but the shard does not hold
    wm = {t["name"]: shard for t in parts}
    wm["ghost.weight"] = shard
    index.write_text(json.dumps({"weight_map": wm}))
    with pytest.raises(Error, match="ghost.weight"):
        Checkpoint.open(tmp_path)


# ---- synthetic.rs:603-612
def test_missing_checkpoint_names_the_reason(tmp_path):
    write_config(tmp_path)
    with pytest.raises(Error, match="model.safetensors"):
        Checkpoint.open(tmp_path)
    with pytest.raises(Error) as e:
        Checkpoint.open(tmp_path / "nope")
    assert e.value.kind == ErrorKind.BAD_FIELD and "not a checkpoint directory" in str(e.value)


def test_missing_config_is_a_read_error(tmp_path):
    write_tensors(tmp_path / "model.safetensors", linear_parts("a.proj", 16, "mul1"))
    with pytest.raises(Error) as e:
        Checkpoint.open(tmp_path)
    assert e.value.kind == ErrorKind.READ
    assert "config.json" in str(e.value) and "(os error 2)" in str(e.value)


def test_header_limits_and_json_errors(tmp_path):
    write_config(tmp_path)
    shard = tmp_path / "model.safetensors"
    shard.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(Error, match="header length 1099511627776 is not usable in a 10-byte file"):
        Checkpoint.open(tmp_path)
    shard.write_bytes(struct.pack("<Q", 3))
    with pytest.raises(Error, match="is not usable in a 8-byte file"):
        Checkpoint.open(tmp_path)
    write_raw(shard, '{"a":', b"")
    with pytest.raises(Error) as e:
        Checkpoint.open(tmp_path)
    assert e.value.kind == ErrorKind.PARSE and "EOF while parsing" in str(e.value)
    write_raw(shard, "[1,2]", b"")
    with pytest.raises(Error, match="not a JSON object"):
        Checkpoint.open(tmp_path)
    shard.write_bytes(b"\x01\x02")
    with pytest.raises(Error) as e:
        Checkpoint.open(tmp_path)
    assert e.value.kind == ErrorKind.READ and "failed to fill whole buffer" in str(e.value)


@pytest.mark.parametrize("entry,needle", [
    ('{"shape":[1],"data_offsets":[0,2]}', "missing dtype"),
    ('{"dtype":5,"shape":[1],"data_offsets":[0,2]}', "expected a string"),
    ('{"dtype":"I17","shape":[1],"data_offsets":[0,2]}', "unknown safetensors dtype `I17`"),
    ('{"dtype":"I16","data_offsets":[0,2]}', "missing shape"),
    ('{"dtype":"I16","shape":"x","data_offsets":[0,2]}', "expected an array, got a string"),
    ('{"dtype":"I16","shape":[1.0],"data_offsets":[0,2]}', "expected an integer, got a number"),
    ('{"dtype":"I16","shape":[-1],"data_offsets":[0,2]}', "expected an integer, got a number"),
    ('{"dtype":"I16","shape":[1]}', "missing data_offsets"),
    ('{"dtype":"I16","shape":[1],"data_offsets":[0]}', "expected 2 offsets, got 1"),
    ('{"dtype":"I16","shape":[1],"data_offsets":[2,0]}', "end 0 is before start 2"),
    ('{"dtype":"I16","shape":[4294967296,4294967296,4294967296],"data_offsets":[0,2]}', "shape product overflows u64"),
    ('{"dtype":"I64","shape":[4294967296,1073741824],"data_offsets":[0,2]}', "byte length overflows u64"),
    ('7', "expected a tensor object, got a number"),
])
def test_header_entry_checks(tmp_path, entry, needle):
    # crates/berth-exl3/src/safetensors.rs:139-245
    write_config(tmp_path)
    write_raw(tmp_path / "model.safetensors", '{"t":' + entry + "}", bytes(2))
    with pytest.raises(Error) as e:
        Checkpoint.open(tmp_path)
    assert needle in str(e.value), str(e.value)


def test_metadata_entry_is_skipped_and_scalar_counts_one_element(tmp_path):
    write_config(tmp_path)
    header = ('{"__metadata__":{"format":"pt"},"s":{"dtype":"F32","shape":[],"data_offsets":[0,4]},'
              '"e":{"dtype":"F16","shape":[0,3],"data_offsets":[4,4]}}')
    write_raw(tmp_path / "model.safetensors", header, bytes(4))
    ckpt = Checkpoint.open(tmp_path)
    assert [t.name for t in ckpt.tensors] == ["e", "s"]
    assert ckpt.tensors.get("s").shape == () and ckpt.tensors.get("s").length == 4
    assert ckpt.tensors.get("e").length == 0 and ckpt.tensors.get("e").read() == b""
    assert ckpt.tensors.get("nope") is None
    assert len(ckpt.linears()) == 0 and len(ckpt.other_tensors()) == 2


def test_tensor_bodies_read_back(tmp_path):
    write_config(tmp_path)
    rng = np.random.default_rng(3)
    tr = rng.integers(0, 65536, size=(2, 2, 32), dtype=np.uint16)
    suh = rng.normal(size=32).astype(np.float16)
    svh = rng.normal(size=32).astype(np.float16)
    write_tensors(tmp_path / "model.safetensors", [
        tensor("l.trellis", "I16", tr.shape, tr.tobytes()), tensor("l.suh", "F16", [32], suh.tobytes()),
        tensor("l.svh", "F16", [32], svh.tobytes()), marker("l.mul1")])
    lin = Checkpoint.open(tmp_path).find_linear("l")
    assert lin.k == Bitrate.int(2)
    assert np.array_equal(lin.trellis.read_array(np.uint16), tr)
    assert np.array_equal(lin.input_scale.tensor.read_array(np.float16).view(np.uint16), suh.view(np.uint16))
    assert np.array_equal(lin.output_scale.tensor.read_array(np.float16).view(np.uint16), svh.view(np.uint16))
    with pytest.raises(Error, match="nope is not an EXL3 linear"):
        Checkpoint.open(tmp_path).find_linear("nope")


# ---- crates/berth-exl3/tests/qwen38_27b.rs:21-117: the real checkpoint is absent; a sparse
# shard with the same tensor shapes must yield the byte lengths and bit rates the test names
def test_27b_shapes_give_the_lengths_the_reference_test_names(tmp_path):
    write_config(tmp_path)
    specs = [("lm_head.trellis", "I16", [320, 15520, 96]), ("lm_head.suh", "F16", [5120]),
             ("lm_head.svh", "F16", [248320]), ("lm_head.mul1", "I32", []),
             ("model.language_model.layers.3.self_attn.q_proj.trellis", "I16", [320, 768, 64]),
             ("model.language_model.layers.3.self_attn.q_proj.suh", "F16", [5120]),
             ("model.language_model.layers.3.self_attn.q_proj.svh", "F16", [12288]),
             ("model.language_model.layers.3.self_attn.q_proj.mul1", "I32", []),
             ("model.language_model.embed_tokens.weight", "BF16", [248320, 5120])]
    entries, at = [], 0
    for name, dtype, shape in specs:
        n = int(np.prod(shape, dtype=np.int64)) if shape else 1
        size = n * DType[dtype].size()
        entries.append(f'"{name}":{{"dtype":"{dtype}","shape":{json.dumps(shape)},"data_offsets":[{at},{at + size}]}}')
        at += size
    header = ("{" + ",".join(entries) + "}").encode()
    shard = tmp_path / "model.safetensors"
    with open(shard, "wb") as f:
        f.write(struct.pack("<Q", len(header)) + header)
        f.truncate(8 + len(header) + at)          # sparse: the bodies are holes
    ckpt = Checkpoint.open(tmp_path)
    head = ckpt.find_linear("lm_head")
    assert head.k == Bitrate.int(6) and head.codebook == Codebook.MUL1
    assert head.trellis.length == 953_548_800
    q = ckpt.find_linear("model.language_model.layers.3.self_attn.q_proj")
    assert q.k == Bitrate.int(4) and q.bias is None
    assert q.trellis.length == 31_457_280
    assert q.input_scale.tensor.length == 10_240 and not q.input_scale.is_packed()
    embed = ckpt.tensors.get("model.language_model.embed_tokens.weight")
    assert embed.dtype == DType.BF16 and embed.length == 2_542_796_800
    assert [t.name for t in ckpt.other_tensors()] == ["model.language_model.embed_tokens.weight"]
    # one byte short: the last tensor no longer fits
    os.truncate(shard, 8 + len(header) + at - 1)
    with pytest.raises(Error, match="embed_tokens.weight"):
        Checkpoint.open(tmp_path)


# ---- crates/berth-exl3/src/config.rs:421-550
def sample():
    return {
        "architectures": ["Qwen3_5ForConditionalGeneration", "Ignored"],
        "unused_top": 1,
        "tie_word_embeddings": True,
        "text_config": {
            "num_hidden_layers": 2, "hidden_size": 32, "head_dim": 16, "num_attention_heads": 4,
            "num_key_value_heads": 2, "vocab_size": 128, "tie_word_embeddings": False,
            "layer_types": ["linear_attention", "full_attention"], "linear_conv_kernel_dim": 4,
            "linear_num_key_heads": 16, "linear_num_value_heads": 48, "linear_key_head_dim": 128,
            "linear_value_head_dim": 128, "attn_output_gate": True, "future_field": "ignored",
        },
        "quantization_config": {
            "quant_method": "exl3", "version": "1.5.0", "bits": 4.0, "head_bits": 6, "codebook": "mul1",
            "vision_bits": 6, "mtp_bits": 4, "out_scales": "always", "calibration": {"rows": 250, "cols": 2048},
            "original_quantization_config": {"quant_method": "other"},
        },
    }


def parse(value) -> ModelConfig:
    return ModelConfig.from_slice(json.dumps(value).encode())


def test_reads_text_config_ahead_of_the_top_level():
    cfg = parse(sample())
    assert cfg.arch_string == "Qwen3_5ForConditionalGeneration"
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.head_dim) == (2, 32, 16)
    assert cfg.tie_word_embeddings is False
    assert cfg.intermediate_size is None and cfg.num_experts is None
    assert [k for k, _ in cfg.layer_types] == [LayerType.LINEAR_ATTENTION, LayerType.FULL_ATTENTION]
    assert cfg.linear_num_value_heads == 48
    assert cfg.attn_output_gate is True
    q = cfg.quantization
    assert (q.quant_method, q.bits, q.head_bits, q.codebook, q.vision_bits, q.mtp_bits, q.version, q.out_scales) == \
        ("exl3", 4.0, 6, "mul1", 6, 4, "1.5.0", "always")
    assert q.calibration == exl3.Calibration(250, 2048)


def test_falls_back_to_the_top_level_per_field():
    value = sample()
    del value["text_config"]["tie_word_embeddings"]
    assert parse(value).tie_word_embeddings is True
    bare = sample()
    bare.update(bare.pop("text_config"))
    cfg = parse(bare)
    assert cfg.hidden_size == 32 and cfg.tie_word_embeddings is False


@pytest.mark.parametrize("key", ["head_dim", "attn_output_gate", "layer_types", "linear_conv_kernel_dim"])
def test_missing_required_field_names_the_field(key):
    value = sample()
    del value["text_config"][key]
    with pytest.raises(Error) as e:
        parse(value)
    assert e.value.kind == ErrorKind.MISSING_FIELD and e.value.field == key
    assert str(e.value) == f"missing field `{key}`"


def test_missing_quantization_config():
    value = sample()
    del value["quantization_config"]
    with pytest.raises(Error, match="quantization_config"):
        parse(value)


def test_optional_moe_and_other_layer_type():
    value = sample()
    value["text_config"].update({"intermediate_size": 17408, "num_experts": 256, "num_experts_per_tok": 8,
                                 "moe_intermediate_size": 512, "shared_expert_intermediate_size": 512,
                                 "layer_types": ["linear_attention", "qsa"]})
    cfg = parse(value)
    assert (cfg.intermediate_size, cfg.num_experts, cfg.num_experts_per_tok, cfg.moe_intermediate_size,
            cfg.shared_expert_intermediate_size) == (17408, 256, 8, 512, 512)
    assert cfg.layer_types[1] == (LayerType.OTHER, "qsa")


def test_layer_types_must_match_the_layer_count():
    value = sample()
    value["text_config"]["layer_types"] = ["full_attention"]
    with pytest.raises(Error) as e:
        parse(value)
    assert str(e.value) == "field `layer_types`: length 1 does not match num_hidden_layers 2"


def test_empty_architectures_names_the_field():
    value = sample()
    value["architectures"] = []
    with pytest.raises(Error, match="architectures"):
        parse(value)


def test_integer_valued_float_counts_as_an_integer():
    value = sample()
    value["quantization_config"]["head_bits"] = 6.0
    assert parse(value).quantization.head_bits == 6


@pytest.mark.parametrize("mutate,message", [
    (lambda v: v["text_config"].__setitem__("hidden_size", 1.5),
     "field `hidden_size`: expected a non-negative integer, got 1.5"),
    (lambda v: v["text_config"].__setitem__("hidden_size", -3),
     "field `hidden_size`: expected a non-negative integer, got -3"),
    (lambda v: v["text_config"].__setitem__("hidden_size", 4294967296),
     "field `hidden_size`: integer 4294967296 does not fit in u32"),
    (lambda v: v["text_config"].__setitem__("hidden_size", "32"),
     'field `hidden_size`: expected a non-negative integer, got string "32"'),
    (lambda v: v["text_config"].__setitem__("attn_output_gate", 1),
     "field `attn_output_gate`: expected a bool, got 1"),
    (lambda v: v.__setitem__("text_config", [1]), "field `text_config`: expected an object, got an array"),
    (lambda v: v.__setitem__("architectures", [""]), "field `architectures`: architecture string is empty"),
    (lambda v: v.__setitem__("architectures", [3]), "field `architectures`: expected a string, got 3"),
    (lambda v: v["text_config"].__setitem__("layer_types", ["full_attention", None]),
     "field `layer_types`: expected strings, got null"),
    (lambda v: v["quantization_config"].__setitem__("bits", "4"), 'field `bits`: expected a number, got string "4"'),
    (lambda v: v["quantization_config"].__setitem__("bits", -1.0),
     "field `bits`: expected a non-negative finite number, got -1.0"),
    (lambda v: v["quantization_config"].__setitem__("calibration", {"rows": 1}), "missing field `calibration.cols`"),
    (lambda v: v["quantization_config"].__setitem__("codebook", 7), "field `codebook`: expected a string, got 7"),
    (lambda v: v.__setitem__("quantization_config", "exl3"),
     'field `quantization_config`: expected an object, got string "exl3"'),
    (lambda v: v["quantization_config"].pop("quant_method"), "missing field `quant_method`"),
])
def test_config_type_errors_use_the_reference_text(mutate, message):
    # crates/berth-exl3/src/config.rs:113-127,178-260,352-418
    value = copy.deepcopy(sample())
    mutate(value)
    with pytest.raises(Error) as e:
        parse(value)
    assert str(e.value) == message


def test_config_that_is_not_json_or_not_an_object():
    with pytest.raises(Error) as e:
        ModelConfig.from_slice(b"{not json")
    assert e.value.kind == ErrorKind.PARSE and str(e.value).startswith("config.json: ")
    with pytest.raises(Error, match="expected a JSON object"):
        ModelConfig.from_slice(b"[]")


def test_json_reader_details():
    """What the reader relies on in its JSON layer: a repeated key keeps the last value,
    escapes decode to UTF-8, integers beyond 64 bits read as floats, nesting is limited."""
    value = sample()
    text = json.dumps(value)[:-1] + ',"architectures":["Last\\u00e9\\ud83d\\ude00"]}'
    assert ModelConfig.from_slice(text.encode()).arch_string == "Lasté😀"
    value["quantization_config"]["bits"] = 18446744073709551616        # 2^64: a float, fine for `bits`
    assert parse(value).quantization.bits == 2.0 ** 64
    # strings are UTF-8: a stray continuation byte, an overlong form and a surrogate are refused
    for bad in (b"\x80", b"\xc0\xaf", b"\xed\xa0\x80", b"\xf5\x80\x80\x80", b"\xe2\x82"):
        blob = json.dumps(sample()).encode().replace(b"Qwen3_5ForConditionalGeneration", b"Q" + bad + b"x")
        with pytest.raises(Error) as e:
            ModelConfig.from_slice(blob)
        assert e.value.kind == ErrorKind.PARSE and "invalid unicode code point" in str(e.value)
    ok = json.dumps(sample()).encode().replace(b"Qwen3_5ForConditionalGeneration", "Qé€😀".encode())
    assert ModelConfig.from_slice(ok).arch_string == "Qé€😀"
    deep = b"[" * 200 + b"]" * 200
    with pytest.raises(Error, match="recursion limit"):
        ModelConfig.from_slice(deep)
    with pytest.raises(Error, match="trailing characters"):
        ModelConfig.from_slice(json.dumps(sample()).encode() + b" x")


# ---- crates/berth-exl3/src/signs.rs:48-92
def test_unpack_signs_known_answers():
    s = exl3.unpack_signs((1).to_bytes(2, "little"))
    assert len(s) == 16 and s[0] == FP16_NEG_ONE and all(v == FP16_ONE for v in s[1:])
    s = exl3.unpack_signs((0x8000).to_bytes(2, "little"))
    assert all(v == FP16_ONE for v in s[:15]) and s[15] == FP16_NEG_ONE
    assert all(v == FP16_ONE for v in exl3.unpack_signs(bytes(2)))
    assert all(v == FP16_NEG_ONE for v in exl3.unpack_signs(b"\xff\xff"))
    s = exl3.unpack_signs((5).to_bytes(2, "little") + (1).to_bytes(2, "little"))
    assert len(s) == 32
    assert (s[0], s[1], s[2], s[16], s[17]) == (FP16_NEG_ONE, FP16_ONE, FP16_NEG_ONE, FP16_NEG_ONE, FP16_ONE)
    with pytest.raises(Error, match="su"):
        exl3.unpack_signs(b"\x01")


def test_dtype_table():
    # crates/berth-exl3/src/dtype.rs:27-78
    sizes = {"BOOL": 1, "U8": 1, "I8": 1, "I16": 2, "U16": 2, "I32": 4, "U32": 4, "I64": 8, "U64": 8, "F16": 2,
             "BF16": 2, "F32": 4, "F64": 8, "F8_E4M3": 1, "F8_E5M2": 1, "F8_E8M0": 1}
    for name, size in sizes.items():
        d = DType.parse(name)
        assert d is not None and d.as_str() == name and d.size() == size
    assert DType.parse("f16") is None and DType.parse("I128") is None


def test_cpp_host_layer_lists_a_checkpoint_without_a_device(tmp_path):
    """berth_host_check ckpt-info: the C++ reader used directly (no C interface, no GPU)."""
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "berth_amd", "lib", "berth_host_check")
    if not os.path.exists(exe):
        pytest.skip("berth_host_check is not built")
    write_config(tmp_path)
    write_tensors(tmp_path / "model.safetensors", demo_tensors())
    r = subprocess.run([exe, "ckpt-info", str(tmp_path)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert f"arch=TestForCausalLM layers=2 hidden=32 tensors={len(demo_tensors())} linears=9 other=6" in r.stdout
    assert "linear block.1.q k=1.5 codebook=1 packed=1/1 bias=1" in r.stdout
    assert "linear block.0.v k=4 codebook=2 packed=0/0 bias=0" in r.stdout
    r = subprocess.run([exe, "ckpt-info", str(tmp_path / "nope")], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "not a checkpoint directory" in r.stderr


def test_mutated_headers_and_configs_only_ever_raise_reader_errors(tmp_path):
    """Truncations and single-byte edits of a valid header / config either parse or fail with
    the reader's own error: never a crash, never another exception type."""
    rng = np.random.default_rng(11)
    write_config(tmp_path)
    shard = tmp_path / "model.safetensors"
    write_tensors(shard, demo_tensors())
    good = shard.read_bytes()
    header_len = struct.unpack("<Q", good[:8])[0]
    outcomes = {"ok": 0, "error": 0}

    def attempt():
        try:
            Checkpoint.open(tmp_path)
            outcomes["ok"] += 1
        except Error as e:
            assert e.kind in (ErrorKind.MISSING_FIELD, ErrorKind.BAD_FIELD, ErrorKind.READ, ErrorKind.PARSE)
            assert str(e)
            outcomes["error"] += 1

    for cut in list(range(0, 24)) + [int(v) for v in rng.integers(24, len(good), size=40)]:
        shard.write_bytes(good[:cut])
        attempt()
    for _ in range(200):
        pos = int(rng.integers(0, 8 + header_len))
        b = bytearray(good)
        b[pos] = int(rng.integers(0, 256))
        shard.write_bytes(bytes(b))
        attempt()
    shard.write_bytes(good)
    cfg = json.dumps(CONFIG).encode()
    for _ in range(200):
        b = bytearray(cfg)
        for _ in range(int(rng.integers(1, 4))):
            b[int(rng.integers(0, len(b)))] = int(rng.integers(0, 256))
        (tmp_path / "config.json").write_bytes(bytes(b))
        attempt()
        try:
            ModelConfig.from_slice(bytes(b[:int(rng.integers(0, len(b)))]))
        except Error:
            pass
    assert outcomes["error"] > 100 and outcomes["ok"] > 10, outcomes
