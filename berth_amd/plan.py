"""ctypes binding of the model planner in libberth_exl3_reader.so, shaped like the
reference's `berth_plan` crate (crates/berth-plan/src/lib.rs): `ModelShape`,
`MoeDims`, `build_plan` -> `ModelPlan` with an `Ffn` per layer, `TensorBytes`,
`HbmBudget`, `place` -> `Placement` with `resident` and `bytes_moved` (one berth: the
reference's VRAM / pinned RAM / SSD tiers are collapsed into "resident in HBM"),
`is_routed_expert`, and the checkpoint adapters `model_shape` / `tensor_bytes`.
Every rule and check runs in the C++ library; this file copies records in and out.
"""
from __future__ import annotations

import ctypes as C
import dataclasses
import enum
from typing import Optional

from . import exl3

ARCH_QWEN3_5 = "Qwen3_5ForConditionalGeneration"             # crates/berth-plan/src/shape.rs:72
ARCH_QWEN3_5_MOE = "Qwen3_5MoeForConditionalGeneration"      # shape.rs:75
ARCH_MINICPM_V4_7 = "MiniCPMV4_7ForConditionalGeneration"    # shape.rs:78
ARCH_QWEN4_EXP = "Qwen4ExpForConditionalGeneration"          # shape.rs:81

MI355X_HBM_BYTES = 288 << 30


class ErrorKind(enum.IntEnum):
    """ShapeError (shape.rs:107-131), PlanError (plan.rs:115-125), PlaceError
    (place.rs:126-173), ConfigError (from_exl3/shape.rs:12-24)."""
    NO_LAYERS = 1
    LAYER_COUNT = 2
    UNKNOWN_LAYER_KIND = 3
    UNEXPECTED_MOE = 4
    MISSING_MOE = 5
    ZERO = 6
    EXPERTS_PER_TOK = 7
    NOT_YET = 20
    UNKNOWN_ARCH = 21
    EMPTY_NAME = 40
    DUPLICATE_TENSOR = 41
    OVERFLOW = 42
    RESERVATION_EXCEEDS_HBM = 43
    WEIGHTS_EXCEED_HBM = 44
    INCONSISTENT_MOE = 47
    INVALID_MOE = 48
    UNKNOWN_LAYER_TYPE = 60
    INCOMPLETE_MOE = 61
    ARGUMENT = 90


class PlanError(Exception):
    def __init__(self, kind: ErrorKind, message: str):
        super().__init__(message)
        self.kind = kind


class LayerKind(enum.IntEnum):
    """shape.rs:10-15."""
    LINEAR_ATTENTION = 0
    FULL_ATTENTION = 1

    @classmethod
    def from_config(cls, name: str) -> "LayerKind":
        """shape.rs:22-29."""
        v = _load().berth_plan_layer_kind_from_config(name.encode())
        if v < 0:
            _raise()
        return cls(v)

    def as_str(self) -> str:
        return "linear_attention" if self is LayerKind.LINEAR_ATTENTION else "full_attention"


class Mixer(enum.IntEnum):
    """plan.rs:10-17."""
    GDN = 0
    FULL_ATTN = 1
    QSA = 2


@dataclasses.dataclass(frozen=True)
class GdnDims:
    """shape.rs:51-57."""
    num_k_heads: int
    num_v_heads: int
    key_head_dim: int
    value_head_dim: int
    conv_kernel_dim: int


@dataclasses.dataclass(frozen=True)
class MoeDims:
    """shape.rs:64-69."""
    num_experts: int
    experts_per_tok: int
    moe_intermediate: int
    shared_intermediate: int


@dataclasses.dataclass
class ModelShape:
    """shape.rs:88-103."""
    arch_string: str
    num_layers: int
    layer_kinds: list
    hidden_size: int
    head_dim: int
    num_q_heads: int
    num_kv_heads: int
    gdn: GdnDims
    moe: Optional[MoeDims]
    vocab_size: int


@dataclasses.dataclass(frozen=True)
class Router:
    """plan.rs:24-27."""
    num_experts: int
    experts_per_tok: int


@dataclasses.dataclass(frozen=True)
class SharedExpert:
    """plan.rs:31-33."""
    intermediate_size: int


@dataclasses.dataclass(frozen=True)
class RoutedExperts:
    """plan.rs:37-41."""
    num_experts: int
    experts_per_tok: int
    intermediate_size: int


@dataclasses.dataclass(frozen=True)
class Ffn:
    """plan.rs:45-57: `DenseMlp` (the three records are None) or `Moe{router, shared, experts}`."""
    router: Optional[Router] = None
    shared: Optional[SharedExpert] = None
    experts: Optional[RoutedExperts] = None

    @property
    def is_moe(self) -> bool:
        return self.router is not None


DENSE_MLP = Ffn()


@dataclasses.dataclass(frozen=True)
class LayerPlan:
    """plan.rs:61-67."""
    index: int
    mixer: Mixer
    ffn: Ffn


@dataclasses.dataclass(frozen=True)
class HbmBudget:
    """What the weights may take of the device: its HBM less the caller's reservation (the
    role of MachineBudget, place.rs:39-61, with the pinned-RAM tier gone).  The default is one
    MI355X: 288 GiB."""
    hbm_bytes: int = MI355X_HBM_BYTES
    reserved_bytes: int = 0

    @classmethod
    def mi355x(cls, reserved_bytes: int = 0) -> "HbmBudget":
        b = _Budget()
        _load().berth_plan_budget_mi355x(reserved_bytes, C.byref(b))
        return cls(int(b.hbm_bytes), int(b.reserved_bytes))


@dataclasses.dataclass(frozen=True)
class Placement:
    """place.rs:111-122 with one berth: `resident` bytes held in HBM (every listed tensor),
    `bytes_moved` bytes one decoded token reads."""
    resident: int
    bytes_moved: int


class TensorBytes:
    """place.rs:71-79: (name, bytes) pairs in the caller's order."""

    def __init__(self, tensors):
        self.tensors = [(str(n), int(b)) for n, b in tensors]

    def total(self) -> int:
        return sum(b for _, b in self.tensors)


class _MoeDims(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("num_experts", "experts_per_tok", "moe_intermediate", "shared_intermediate")]


class _Shape(C.Structure):
    _fields_ = [("arch_string", C.c_char_p), ("num_layers", C.c_uint32), ("layer_kinds", C.POINTER(C.c_int)),
                ("num_layer_kinds", C.c_size_t)] + \
               [(n, C.c_uint32) for n in ("hidden_size", "head_dim", "num_q_heads", "num_kv_heads", "gdn_num_k_heads",
                                          "gdn_num_v_heads", "gdn_key_head_dim", "gdn_value_head_dim",
                                          "gdn_conv_kernel_dim")] + \
               [("has_moe", C.c_int), ("moe", _MoeDims), ("vocab_size", C.c_uint32)]


class _Layer(C.Structure):
    _fields_ = [("index", C.c_uint32), ("mixer", C.c_int), ("ffn_is_moe", C.c_int)] + \
               [(n, C.c_uint32) for n in ("router_num_experts", "router_experts_per_tok", "shared_intermediate_size",
                                          "experts_num_experts", "experts_experts_per_tok",
                                          "experts_intermediate_size")]


class _Summary(C.Structure):
    _fields_ = [("arch_string", C.c_char_p)] + \
               [(n, C.c_uint32) for n in ("hidden_size", "vocab_size", "head_dim", "num_q_heads", "num_kv_heads",
                                          "gdn_num_k_heads", "gdn_num_v_heads", "gdn_key_head_dim",
                                          "gdn_value_head_dim", "gdn_conv_kernel_dim")] + \
               [("num_layers", C.c_size_t)]


class _Budget(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("hbm_bytes", "reserved_bytes")]


_bound = False


def _load() -> C.CDLL:
    global _bound
    L = exl3._load()
    if not _bound:
        vp, sz, u64 = C.c_void_p, C.c_size_t, C.c_uint64
        L.berth_plan_last_error.restype = C.c_char_p
        L.berth_plan_layer_kind_from_config.argtypes = [C.c_char_p]
        L.berth_plan_shape_from_config.argtypes = [vp, C.POINTER(_Shape)]
        L.berth_plan_build.argtypes = [C.POINTER(_Shape), C.POINTER(vp)]
        L.berth_plan_from_config.argtypes = [vp, C.POINTER(vp)]
        L.berth_plan_free.argtypes = [vp]
        L.berth_plan_free.restype = None
        L.berth_plan_summary_of.argtypes = [vp, C.POINTER(_Summary)]
        L.berth_plan_layer_at.argtypes = [vp, sz, C.POINTER(_Layer)]
        L.berth_plan_is_routed_expert.argtypes = [C.c_char_p]
        L.berth_plan_budget_mi355x.argtypes = [u64, C.POINTER(_Budget)]
        L.berth_plan_budget_mi355x.restype = None
        L.berth_plan_place.argtypes = [vp, C.POINTER(C.c_char_p), C.POINTER(u64), sz, C.POINTER(_Budget),
                                       C.POINTER(u64), C.POINTER(u64)]
        L.berth_plan_tensor_bytes.argtypes = [vp, C.POINTER(vp)]
        L.berth_plan_bytes_free.argtypes = [vp]
        L.berth_plan_bytes_free.restype = None
        L.berth_plan_bytes_count.argtypes = [vp]
        L.berth_plan_bytes_count.restype = sz
        L.berth_plan_bytes_at.argtypes = [vp, sz, C.POINTER(C.c_char_p), C.POINTER(u64)]
        L.berth_plan_place_bytes.argtypes = [vp, vp, C.POINTER(_Budget), C.POINTER(u64), C.POINTER(u64)]
        _bound = True
    return L


def _raise():
    L = _load()
    raise PlanError(ErrorKind(L.berth_plan_last_error_kind()), L.berth_plan_last_error().decode("utf-8", "replace"))


def _check(rc: int) -> None:
    if rc != 0:
        _raise()


class ModelPlan:
    """plan.rs:99-111.  `embedding`, `final_norm` and `lm_head` (plan.rs:71-93) repeat
    `vocab_size` and `hidden_size`."""

    def __init__(self, handle):
        L = _load()
        try:
            s = _Summary()
            _check(L.berth_plan_summary_of(handle, C.byref(s)))
            self.arch_string = s.arch_string.decode("utf-8", "replace")
            self.hidden_size, self.vocab_size, self.head_dim = int(s.hidden_size), int(s.vocab_size), int(s.head_dim)
            self.num_q_heads, self.num_kv_heads = int(s.num_q_heads), int(s.num_kv_heads)
            self.gdn = GdnDims(int(s.gdn_num_k_heads), int(s.gdn_num_v_heads), int(s.gdn_key_head_dim),
                               int(s.gdn_value_head_dim), int(s.gdn_conv_kernel_dim))
            self.layers = []
            for i in range(s.num_layers):
                rec = _Layer()
                _check(L.berth_plan_layer_at(handle, i, C.byref(rec)))
                ffn = DENSE_MLP
                if rec.ffn_is_moe:
                    ffn = Ffn(Router(int(rec.router_num_experts), int(rec.router_experts_per_tok)),
                              SharedExpert(int(rec.shared_intermediate_size)),
                              RoutedExperts(int(rec.experts_num_experts), int(rec.experts_experts_per_tok),
                                            int(rec.experts_intermediate_size)))
                self.layers.append(LayerPlan(int(rec.index), Mixer(rec.mixer), ffn))
        except Exception:
            L.berth_plan_free(handle)
            raise
        self._handle = handle

    def __del__(self):
        if getattr(self, "_handle", None):
            _load().berth_plan_free(self._handle)
            self._handle = None


def _c_shape(shape: ModelShape):
    kinds = (C.c_int * max(1, len(shape.layer_kinds)))(*[int(k) for k in shape.layer_kinds])
    s = _Shape()
    s.arch_string = shape.arch_string.encode()
    s.num_layers = shape.num_layers
    s.layer_kinds = C.cast(kinds, C.POINTER(C.c_int))
    s.num_layer_kinds = len(shape.layer_kinds)
    for name in ("hidden_size", "head_dim", "num_q_heads", "num_kv_heads", "vocab_size"):
        setattr(s, name, getattr(shape, name))
    for name in ("num_k_heads", "num_v_heads", "key_head_dim", "value_head_dim", "conv_kernel_dim"):
        setattr(s, "gdn_" + name, getattr(shape.gdn, name))
    if shape.moe is not None:
        s.has_moe = 1
        s.moe = _MoeDims(shape.moe.num_experts, shape.moe.experts_per_tok, shape.moe.moe_intermediate,
                         shape.moe.shared_intermediate)
    return s, kinds


def build_plan(shape: ModelShape) -> ModelPlan:
    """plan.rs:133-163."""
    s, _keep = _c_shape(shape)
    handle = C.c_void_p()
    _check(_load().berth_plan_build(C.byref(s), C.byref(handle)))
    return ModelPlan(handle)


def _shape_from_handle(config_handle) -> ModelShape:
    s = _Shape()
    _check(_load().berth_plan_shape_from_config(config_handle, C.byref(s)))
    moe = None
    if s.has_moe:
        moe = MoeDims(int(s.moe.num_experts), int(s.moe.experts_per_tok), int(s.moe.moe_intermediate),
                      int(s.moe.shared_intermediate))
    return ModelShape(
        arch_string=s.arch_string.decode("utf-8", "replace"), num_layers=int(s.num_layers),
        layer_kinds=[LayerKind(s.layer_kinds[i]) for i in range(s.num_layer_kinds)], hidden_size=int(s.hidden_size),
        head_dim=int(s.head_dim), num_q_heads=int(s.num_q_heads), num_kv_heads=int(s.num_kv_heads),
        gdn=GdnDims(int(s.gdn_num_k_heads), int(s.gdn_num_v_heads), int(s.gdn_key_head_dim),
                    int(s.gdn_value_head_dim), int(s.gdn_conv_kernel_dim)),
        moe=moe, vocab_size=int(s.vocab_size))


def model_shape(source) -> ModelShape:
    """from_exl3/shape.rs:34-110.  `source`: an open `exl3.Checkpoint`, or the bytes of a
    config.json."""
    L = _load()
    if isinstance(source, exl3.Checkpoint):
        return _shape_from_handle(L.berth_ckpt_config_of(source._handle))
    handle = C.c_void_p()
    exl3._check(L.berth_ckpt_config_parse(bytes(source), len(source), C.byref(handle)))
    try:
        return _shape_from_handle(handle)
    finally:
        L.berth_ckpt_config_free(handle)


def tensor_bytes(ckpt: exl3.Checkpoint) -> TensorBytes:
    """from_exl3/bytes.rs:57-93."""
    L = _load()
    handle = C.c_void_p()
    _check(L.berth_plan_tensor_bytes(ckpt._handle, C.byref(handle)))
    try:
        out = []
        for i in range(L.berth_plan_bytes_count(handle)):
            name, size = C.c_char_p(), C.c_uint64()
            _check(L.berth_plan_bytes_at(handle, i, C.byref(name), C.byref(size)))
            out.append((name.value.decode("utf-8", "replace"), int(size.value)))
        return TensorBytes(out)
    finally:
        L.berth_plan_bytes_free(handle)


def is_routed_expert(name: str) -> bool:
    """place.rs:175-187."""
    return bool(_load().berth_plan_is_routed_expert(name.encode()))


def place(plan: ModelPlan, weights: TensorBytes, budget: HbmBudget = HbmBudget()) -> Placement:
    """place.rs:189-232 with one berth; `bytes_moved` follows place.rs:345-376."""
    n = len(weights.tensors)
    names = (C.c_char_p * max(1, n))(*[name.encode() for name, _ in weights.tensors])
    sizes = (C.c_uint64 * max(1, n))(*[size for _, size in weights.tensors])
    b = _Budget(budget.hbm_bytes, budget.reserved_bytes)
    resident, moved = C.c_uint64(), C.c_uint64()
    _check(_load().berth_plan_place(plan._handle, names, sizes, n, C.byref(b), C.byref(resident), C.byref(moved)))
    return Placement(int(resident.value), int(moved.value))
