"""ctypes binding of libberth_exl3_reader.so, shaped like the reference's
`berth_exl3` crate (crates/berth-exl3/src/lib.rs:16-30): `Checkpoint.open`,
`ModelConfig.from_slice`, `TensorInfo`, `LinearExl3`, `Bitrate`, `Codebook`,
`HadamardScale`, `unpack_signs`.  The parsing and every check run in the C++
library; this file only copies the records out.
"""
from __future__ import annotations

import ctypes as C
import dataclasses
import enum
import os
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libberth_exl3_reader.so")

FP16_ONE = 0x3C00        # crates/berth-exl3/src/signs.rs:4
FP16_NEG_ONE = 0xBC00    # crates/berth-exl3/src/signs.rs:7


class ErrorKind(enum.IntEnum):
    """crates/berth-exl3/src/error.rs:5-31."""
    MISSING_FIELD = 1
    BAD_FIELD = 2
    READ = 3
    PARSE = 4
    ARGUMENT = 5


class Error(Exception):
    """A failed checkpoint read: `kind`, the message text and the field or path it names."""

    def __init__(self, kind: ErrorKind, message: str, field: str):
        super().__init__(message)
        self.kind = kind
        self.field = field


class DType(enum.IntEnum):
    """crates/berth-exl3/src/dtype.rs:6-23."""
    BOOL = 0
    U8 = 1
    I8 = 2
    I16 = 3
    U16 = 4
    I32 = 5
    U32 = 6
    I64 = 7
    U64 = 8
    F16 = 9
    BF16 = 10
    F32 = 11
    F64 = 12
    F8_E4M3 = 13
    F8_E5M2 = 14
    F8_E8M0 = 15

    @classmethod
    def parse(cls, name: str) -> Optional["DType"]:
        v = _load().berth_ckpt_dtype_parse(name.encode())
        return None if v < 0 else cls(v)

    def as_str(self) -> str:
        return _load().berth_ckpt_dtype_name(int(self)).decode()

    def size(self) -> int:
        return int(_load().berth_ckpt_dtype_size(int(self)))


class Codebook(enum.IntEnum):
    """crates/berth-exl3/src/linear.rs:19-26 (the reader's order; `kernel_codebook` of a
    linear is the value the kernel entry points take)."""
    MCG = 0
    MUL1 = 1
    DEFAULT = 2


class LayerType(enum.IntEnum):
    """crates/berth-exl3/src/config.rs:6-13."""
    LINEAR_ATTENTION = 0
    FULL_ATTENTION = 1
    OTHER = 2


@dataclasses.dataclass(frozen=True)
class Bitrate:
    """crates/berth-exl3/src/linear.rs:43-60: `twice` is 2 K so that the half rates 1.5,
    2.5 and 3.5 stay integral."""
    twice: int

    @classmethod
    def int(cls, k: int) -> "Bitrate":
        return cls(2 * k)

    @classmethod
    def half(cls, floor: int) -> "Bitrate":
        return cls(2 * floor + 1)

    def is_half(self) -> bool:
        return bool(self.twice & 1)

    def as_f64(self) -> float:
        return self.twice / 2.0

    def __str__(self) -> str:
        return f"{self.twice // 2}.5" if self.is_half() else str(self.twice // 2)


@dataclasses.dataclass(frozen=True)
class TensorInfo:
    """crates/berth-exl3/src/safetensors.rs:14-33."""
    name: str
    shard: str
    dtype: DType
    shape: tuple
    offset: int
    length: int

    def read_array(self, dtype=np.uint8) -> np.ndarray:
        """The tensor's bytes (crates/berth-engine/src/device.rs:49-63) as a writable array of
        `dtype`, shaped like the tensor when the element sizes agree."""
        raw = np.empty(self.length, dtype=np.uint8)
        shape = (C.c_uint64 * max(1, len(self.shape)))(*self.shape)
        t = _Tensor(self.name.encode(), os.fsencode(self.shard), int(self.dtype), len(self.shape), shape, self.offset,
                    self.length)
        _check(_load().berth_ckpt_read_tensor(C.byref(t), raw.ctypes.data_as(C.c_void_p), self.length))
        out = raw.view(dtype)
        return out.reshape(self.shape) if np.dtype(dtype).itemsize == self.dtype.size() else out

    def read(self) -> bytes:
        return self.read_array().tobytes()


@dataclasses.dataclass(frozen=True)
class HadamardScale:
    """crates/berth-exl3/src/linear.rs:93-117."""
    tensor: TensorInfo
    packed: bool

    def is_packed(self) -> bool:
        return self.packed


@dataclasses.dataclass(frozen=True)
class Calibration:
    rows: int
    cols: int


@dataclasses.dataclass(frozen=True)
class QuantizationConfig:
    """crates/berth-exl3/src/config.rs:26-55."""
    quant_method: str
    bits: float
    head_bits: int
    codebook: Optional[str]
    version: Optional[str]
    vision_bits: Optional[int]
    mtp_bits: Optional[int]
    out_scales: Optional[str]
    calibration: Optional[Calibration]


@dataclasses.dataclass(frozen=True)
class ModelConfig:
    """crates/berth-exl3/src/config.rs:57-100."""
    arch_string: str
    num_hidden_layers: int
    hidden_size: int
    intermediate_size: Optional[int]
    head_dim: int
    num_attention_heads: int
    num_key_value_heads: int
    vocab_size: int
    tie_word_embeddings: bool
    layer_types: tuple          # of (LayerType, name as written)
    linear_conv_kernel_dim: int
    linear_num_key_heads: int
    linear_num_value_heads: int
    linear_key_head_dim: int
    linear_value_head_dim: int
    attn_output_gate: bool
    num_experts: Optional[int]
    num_experts_per_tok: Optional[int]
    moe_intermediate_size: Optional[int]
    shared_expert_intermediate_size: Optional[int]
    quantization: QuantizationConfig

    @classmethod
    def from_slice(cls, data: bytes) -> "ModelConfig":
        L = _load()
        handle = C.c_void_p()
        _check(L.berth_ckpt_config_parse(data, len(data), C.byref(handle)))
        try:
            return _config(handle)
        finally:
            L.berth_ckpt_config_free(handle)


class _Tensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("shard", C.c_char_p), ("dtype", C.c_int), ("rank", C.c_int),
                ("shape", C.POINTER(C.c_uint64)), ("offset", C.c_uint64), ("length", C.c_uint64)]


class _Linear(C.Structure):
    _fields_ = [("prefix", C.c_char_p), ("trellis", _Tensor), ("input_scale", _Tensor), ("output_scale", _Tensor),
                ("bias", _Tensor), ("input_packed", C.c_int), ("output_packed", C.c_int), ("has_bias", C.c_int),
                ("codebook", C.c_int), ("kernel_codebook", C.c_int), ("twice_k", C.c_int)]


_U32 = C.c_uint32


class _Config(C.Structure):
    _fields_ = ([("arch_string", C.c_char_p)]
                + [(n, _U32) for n in ("num_hidden_layers", "hidden_size", "head_dim", "num_attention_heads",
                                       "num_key_value_heads", "vocab_size", "linear_conv_kernel_dim",
                                       "linear_num_key_heads", "linear_num_value_heads", "linear_key_head_dim",
                                       "linear_value_head_dim")]
                + [(n, C.c_int) for n in ("tie_word_embeddings", "attn_output_gate", "has_intermediate_size",
                                          "has_num_experts", "has_num_experts_per_tok", "has_moe_intermediate_size",
                                          "has_shared_expert_intermediate_size")]
                + [(n, _U32) for n in ("intermediate_size", "num_experts", "num_experts_per_tok",
                                       "moe_intermediate_size", "shared_expert_intermediate_size")]
                + [("num_layer_types", C.c_size_t), ("layer_type_kinds", C.POINTER(C.c_int)),
                   ("layer_type_names", C.POINTER(C.c_char_p)),
                   ("quant_method", C.c_char_p), ("bits", C.c_double), ("head_bits", _U32),
                   ("codebook", C.c_char_p), ("version", C.c_char_p), ("out_scales", C.c_char_p)]
                + [(n, C.c_int) for n in ("has_vision_bits", "has_mtp_bits", "has_calibration")]
                + [(n, _U32) for n in ("vision_bits", "mtp_bits", "calibration_rows", "calibration_cols")])


_lib = None


def _load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m berth_amd.build`")
        L = C.CDLL(LIB_PATH)
        vp, sz = C.c_void_p, C.c_size_t
        L.berth_ckpt_last_error.restype = C.c_char_p
        L.berth_ckpt_last_error_field.restype = C.c_char_p
        L.berth_ckpt_dtype_name.restype = C.c_char_p
        L.berth_ckpt_dtype_name.argtypes = [C.c_int]
        L.berth_ckpt_dtype_parse.argtypes = [C.c_char_p]
        L.berth_ckpt_dtype_size.restype = C.c_uint64
        L.berth_ckpt_dtype_size.argtypes = [C.c_int]
        L.berth_ckpt_open.argtypes = [C.c_char_p, C.POINTER(vp)]
        L.berth_ckpt_free.argtypes = [vp]
        L.berth_ckpt_free.restype = None
        L.berth_ckpt_directory.argtypes = [vp]
        L.berth_ckpt_directory.restype = C.c_char_p
        L.berth_ckpt_config_of.argtypes = [vp]
        L.berth_ckpt_config_of.restype = vp
        L.berth_ckpt_config_parse.argtypes = [C.c_char_p, sz, C.POINTER(vp)]
        L.berth_ckpt_config_free.argtypes = [vp]
        L.berth_ckpt_config_free.restype = None
        L.berth_ckpt_config_get.argtypes = [vp, C.POINTER(_Config)]
        for name in ("tensor", "linear", "other"):
            getattr(L, f"berth_ckpt_{name}_count").argtypes = [vp]
            getattr(L, f"berth_ckpt_{name}_count").restype = sz
        L.berth_ckpt_tensor_at.argtypes = [vp, sz, C.POINTER(_Tensor)]
        L.berth_ckpt_other_at.argtypes = [vp, sz, C.POINTER(_Tensor)]
        L.berth_ckpt_tensor_find.argtypes = [vp, C.c_char_p, C.POINTER(_Tensor)]
        L.berth_ckpt_linear_at.argtypes = [vp, sz, C.POINTER(_Linear)]
        L.berth_ckpt_linear_find.argtypes = [vp, C.c_char_p, C.POINTER(_Linear)]
        L.berth_ckpt_linear_unpack_signs.argtypes = [vp, sz, C.c_int, vp, sz, C.POINTER(sz)]
        L.berth_ckpt_unpack_signs.argtypes = [C.c_char_p, sz, vp]
        L.berth_ckpt_read_tensor.argtypes = [C.POINTER(_Tensor), vp, sz]
        _lib = L
    return _lib


def _check(rc: int) -> None:
    if rc != 0:
        L = _load()
        raise Error(ErrorKind(L.berth_ckpt_last_error_kind()), L.berth_ckpt_last_error().decode("utf-8", "replace"),
                    L.berth_ckpt_last_error_field().decode("utf-8", "replace"))


def _str(b) -> Optional[str]:
    return None if b is None else b.decode("utf-8", "replace")


def _tensor(t: _Tensor) -> TensorInfo:
    return TensorInfo(t.name.decode("utf-8", "replace"), os.fsdecode(t.shard), DType(t.dtype), tuple(int(t.shape[i]) for i in range(t.rank)),
                      int(t.offset), int(t.length))


def _config(handle) -> ModelConfig:
    c = _Config()
    _check(_load().berth_ckpt_config_get(handle, C.byref(c)))

    def opt(name):
        return int(getattr(c, name)) if getattr(c, "has_" + name) else None

    q = QuantizationConfig(
        quant_method=_str(c.quant_method), bits=float(c.bits), head_bits=int(c.head_bits), codebook=_str(c.codebook),
        version=_str(c.version), vision_bits=opt("vision_bits"), mtp_bits=opt("mtp_bits"),
        out_scales=_str(c.out_scales),
        calibration=Calibration(int(c.calibration_rows), int(c.calibration_cols)) if c.has_calibration else None)
    layers = tuple((LayerType(c.layer_type_kinds[i]), c.layer_type_names[i].decode("utf-8", "replace"))
                   for i in range(c.num_layer_types))
    return ModelConfig(
        arch_string=_str(c.arch_string), num_hidden_layers=int(c.num_hidden_layers), hidden_size=int(c.hidden_size),
        intermediate_size=opt("intermediate_size"), head_dim=int(c.head_dim),
        num_attention_heads=int(c.num_attention_heads), num_key_value_heads=int(c.num_key_value_heads),
        vocab_size=int(c.vocab_size), tie_word_embeddings=bool(c.tie_word_embeddings), layer_types=layers,
        linear_conv_kernel_dim=int(c.linear_conv_kernel_dim), linear_num_key_heads=int(c.linear_num_key_heads),
        linear_num_value_heads=int(c.linear_num_value_heads), linear_key_head_dim=int(c.linear_key_head_dim),
        linear_value_head_dim=int(c.linear_value_head_dim), attn_output_gate=bool(c.attn_output_gate),
        num_experts=opt("num_experts"), num_experts_per_tok=opt("num_experts_per_tok"),
        moe_intermediate_size=opt("moe_intermediate_size"),
        shared_expert_intermediate_size=opt("shared_expert_intermediate_size"), quantization=q)


class LinearExl3:
    """crates/berth-exl3/src/linear.rs:119-151."""

    def __init__(self, owner: "Checkpoint", index: int, rec: _Linear):
        self._owner = owner
        self._index = index
        self.prefix = rec.prefix.decode("utf-8", "replace")
        self.trellis = _tensor(rec.trellis)
        self.input_scale = HadamardScale(_tensor(rec.input_scale), bool(rec.input_packed))
        self.output_scale = HadamardScale(_tensor(rec.output_scale), bool(rec.output_packed))
        self.bias = _tensor(rec.bias) if rec.has_bias else None
        self.codebook = Codebook(rec.codebook)
        self.kernel_codebook = int(rec.kernel_codebook)
        self.k = Bitrate(int(rec.twice_k))

    def _unpack(self, output_side: int) -> np.ndarray:
        L = _load()
        n = C.c_size_t(0)
        _check(L.berth_ckpt_linear_unpack_signs(self._owner._handle, self._index, output_side, None, 0, C.byref(n)))
        out = np.empty(n.value, dtype=np.uint16)
        _check(L.berth_ckpt_linear_unpack_signs(self._owner._handle, self._index, output_side,
                                                out.ctypes.data_as(C.c_void_p), n.value, C.byref(n)))
        return out

    def unpack_input_signs(self) -> np.ndarray:
        """fp16 +-1 bit patterns of packed `su`; an error when the linear stores `suh`."""
        return self._unpack(0)

    def unpack_output_signs(self) -> np.ndarray:
        return self._unpack(1)


class TensorIndex:
    """crates/berth-exl3/src/safetensors.rs:35-78."""

    def __init__(self, owner: "Checkpoint"):
        self._owner = owner

    def __len__(self) -> int:
        return int(_load().berth_ckpt_tensor_count(self._owner._handle))

    def get(self, name: str) -> Optional[TensorInfo]:
        t = _Tensor()
        rc = _load().berth_ckpt_tensor_find(self._owner._handle, name.encode(), C.byref(t))
        if rc < 0:
            _check(rc)
        return _tensor(t) if rc == 1 else None

    def contains(self, name: str) -> bool:
        return self.get(name) is not None

    def __iter__(self):
        L = _load()
        for i in range(len(self)):
            t = _Tensor()
            _check(L.berth_ckpt_tensor_at(self._owner._handle, i, C.byref(t)))
            yield _tensor(t)


class Checkpoint:
    """crates/berth-exl3/src/checkpoint.rs:21-84."""

    def __init__(self, handle):
        self._handle = handle
        L = _load()
        self.directory = os.fsdecode(L.berth_ckpt_directory(handle))
        self.config = _config(L.berth_ckpt_config_of(handle))
        self.tensors = TensorIndex(self)
        self._linears = []
        for i in range(L.berth_ckpt_linear_count(handle)):
            rec = _Linear()
            _check(L.berth_ckpt_linear_at(handle, i, C.byref(rec)))
            self._linears.append(LinearExl3(self, i, rec))
        self._other = []
        for i in range(L.berth_ckpt_other_count(handle)):
            t = _Tensor()
            _check(L.berth_ckpt_other_at(handle, i, C.byref(t)))
            self._other.append(_tensor(t))

    @classmethod
    def open(cls, directory) -> "Checkpoint":
        handle = C.c_void_p()
        _check(_load().berth_ckpt_open(os.fspath(directory).encode(), C.byref(handle)))
        return cls(handle)

    def linears(self) -> list:
        return self._linears

    def other_tensors(self) -> list:
        return self._other

    def find_linear(self, prefix: str) -> LinearExl3:
        """crates/berth-engine/src/device.rs:168-173."""
        for lin in self._linears:
            if lin.prefix == prefix:
                return lin
        raise Error(ErrorKind.ARGUMENT, f"{prefix} is not an EXL3 linear", prefix)

    def __del__(self):
        if getattr(self, "_handle", None) and _lib is not None:
            _lib.berth_ckpt_free(self._handle)
            self._handle = None


def unpack_signs(packed_le: bytes) -> np.ndarray:
    """crates/berth-exl3/src/signs.rs:25-46."""
    out = np.empty(16 * (len(packed_le) // 2), dtype=np.uint16)     # an odd length is refused before any write
    _check(_load().berth_ckpt_unpack_signs(packed_le, len(packed_le), out.ctypes.data_as(C.c_void_p)))
    return out
