"""Writers of small EXL3 checkpoint directories for the tests: a safetensors shard
(8-byte little-endian header length, JSON header, tensor bodies back to back) and
the tensors of one EXL3 linear under a prefix."""
import json
import struct

import numpy as np

CONFIG = {
    "architectures": ["TestForCausalLM"],
    "text_config": {
        "num_hidden_layers": 2, "hidden_size": 256, "intermediate_size": 384, "head_dim": 16,
        "num_attention_heads": 2, "num_key_value_heads": 1, "vocab_size": 128, "tie_word_embeddings": False,
        "layer_types": ["linear_attention", "full_attention"], "linear_conv_kernel_dim": 4,
        "linear_num_key_heads": 16, "linear_num_value_heads": 32, "linear_key_head_dim": 128,
        "linear_value_head_dim": 128, "attn_output_gate": False,
    },
    "quantization_config": {"quant_method": "exl3", "bits": 4, "head_bits": 6, "codebook": "mul1"},
}


def write_shard(path, tensors):
    """tensors: list of (name, safetensors dtype, shape, bytes)."""
    data, header = b"", {}
    for name, dtype, shape, body in tensors:
        header[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [len(data), len(data) + len(body)]}
        data += body
    text = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)) + text + data)


def pack_signs(scale: np.ndarray) -> np.ndarray:
    """fp16 vector -> one bit per element (set = negative), element i in bit i % 16 of word i // 16."""
    neg = (scale.view(np.uint16) >> 15).astype(np.uint16).reshape(-1, 16)
    return (neg << np.arange(16, dtype=np.uint16)).sum(axis=1).astype(np.uint16)


def linear_tensors(prefix, trellis, suh, svh, codebook="mul1", packed=False, bias=None):
    """The tensors of one EXL3 linear.  packed: store su / sv sign words instead of suh / svh."""
    out = [(f"{prefix}.trellis", "I16", trellis.shape, trellis.tobytes())]
    if packed:
        su, sv = pack_signs(suh), pack_signs(svh)
        out += [(f"{prefix}.su", "I16", su.shape, su.tobytes()), (f"{prefix}.sv", "I16", sv.shape, sv.tobytes())]
    else:
        out += [(f"{prefix}.suh", "F16", suh.shape, suh.tobytes()), (f"{prefix}.svh", "F16", svh.shape, svh.tobytes())]
    if codebook:
        out.append((f"{prefix}.{codebook}", "I32", (), bytes([1, 0, 0, 0])))
    if bias is not None:
        out.append((f"{prefix}.bias", "F16", bias.shape, bias.tobytes()))
    return out


def write_checkpoint(directory, tensors, config=CONFIG):
    (directory / "config.json").write_text(json.dumps(config))
    write_shard(directory / "model.safetensors", tensors)
