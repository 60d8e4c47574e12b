"""The model planner (berth_amd/csrc/host/plan.hpp through include/berth_plan.h and
berth_amd/plan.py) against the cases and known answers of the reference's own tests:
crates/berth-plan/tests/plan.rs (27B dense, 35B MoE, one berth, errors, the expert name
rule), tests/from_exl3_shape.rs (config -> shape) and tests/from_exl3_bytes.rs
(checkpoint -> byte list).  Host only."""
import json
import os
import subprocess

import numpy as np
import pytest

from berth_amd import exl3, plan as P
from tests import ckpt_util as U

GIB = 1 << 30


def every_fourth_full(n):
    return [P.LayerKind.FULL_ATTENTION if (i + 1) % 4 == 0 else P.LayerKind.LINEAR_ATTENTION for i in range(n)]


def shape_27b():          # tests/plan.rs:32-45
    return P.ModelShape(P.ARCH_QWEN3_5, 64, every_fourth_full(64), 5120, 256, 24, 4,
                        P.GdnDims(16, 48, 128, 128, 4), None, 248_320)


def shape_35b():          # tests/plan.rs:47-75
    return P.ModelShape(P.ARCH_QWEN3_5_MOE, 40, every_fourth_full(40), 2048, 256, 16, 2,
                        P.GdnDims(16, 32, 128, 128, 4), P.MoeDims(256, 8, 512, 512), 248_320)


def bytes_35b():          # tests/plan.rs:96-120: 16.1 + 1.2 + 0.25 GB
    return P.TensorBytes([
        ("model.language_model.embed_tokens.weight", 400_000_000),
        ("model.language_model.layers.0.mlp.shared_expert.down_proj.trellis", 500_000_000),
        ("model.language_model.layers.0.mlp.shared_expert_gate.weight", 10_000),
        ("model.language_model.layers.0.mlp.gate.weight", 49_990_000),
        ("model.language_model.norm.weight", 10_000),
        ("lm_head.weight", 249_990_000),
        ("model.visual.patch_embed.proj.weight", 250_000_000),
        ("model.language_model.layers.0.mlp.experts.gate_up_proj.trellis", 10_000_000_000),
        ("model.language_model.layers.3.mlp.experts.down_proj.trellis", 6_100_000_000),
    ])


def this_machine(reserved):   # the VRAM of the reference's development box (place.rs:12-15): the known answers are quoted on it
    return P.HbmBudget(24 * GIB, reserved)


def mixers(plan):
    return [sum(1 for l in plan.layers if l.mixer == m) for m in (P.Mixer.GDN, P.Mixer.FULL_ATTN, P.Mixer.QSA)]


def test_27b_dense_plan_and_placement():
    """tests/plan.rs:135-197."""
    plan = P.build_plan(shape_27b())
    assert plan.arch_string == P.ARCH_QWEN3_5 and len(plan.layers) == 64 and mixers(plan) == [48, 16, 0]
    for layer in plan.layers:
        want = P.Mixer.FULL_ATTN if (layer.index + 1) % 4 == 0 else P.Mixer.GDN
        assert layer.mixer == want and layer.ffn == P.DENSE_MLP and not layer.ffn.is_moe
    assert plan.gdn == P.GdnDims(16, 48, 128, 128, 4)
    assert (plan.hidden_size, plan.head_dim, plan.num_q_heads, plan.num_kv_heads, plan.vocab_size) == \
        (5120, 256, 24, 4, 248_320)
    weights = P.TensorBytes([
        ("model.language_model.embed_tokens.weight", 2_000_000_000),
        ("model.language_model.layers.0.linear_attn.in_proj_qkv.trellis", 4_000_000_000),
        ("model.language_model.layers.3.self_attn.q_proj.trellis", 1_000_000_000),
        ("model.language_model.layers.0.mlp.down_proj.trellis", 3_000_000_000),
        ("model.language_model.norm.weight", 20_000),
        ("lm_head.weight", 3_199_980_000),
    ])
    assert weights.total() == 13_200_000_000
    placed = P.place(plan, weights, this_machine(4_600_000_000))
    assert placed == P.Placement(resident=13_200_000_000, bytes_moved=13_200_000_000)


def test_35b_moe_plan_and_bytes_moved():
    """tests/plan.rs:200-245: one decoded token reads the backbone plus 8/256 of the expert pool."""
    plan = P.build_plan(shape_35b())
    assert len(plan.layers) == 40 and mixers(plan) == [30, 10, 0]
    assert (plan.num_kv_heads, plan.head_dim, plan.hidden_size) == (2, 256, 2048)
    for layer in plan.layers:
        assert layer.ffn.is_moe
        assert layer.ffn.router == P.Router(256, 8)
        assert layer.ffn.shared == P.SharedExpert(512)
        assert layer.ffn.experts == P.RoutedExperts(256, 8, 512)
    weights = bytes_35b()
    assert weights.total() == 17_550_000_000
    for budget in (this_machine(2_500_000_000), P.HbmBudget.mi355x(2_500_000_000), P.HbmBudget()):
        placed = P.place(plan, weights, budget)
        assert 16_100_000_000 * 8 // 256 == 503_125_000
        assert placed == P.Placement(resident=17_550_000_000, bytes_moved=1_450_000_000 + 503_125_000)


def test_a_pool_that_does_not_fit_hbm_is_an_error_not_a_spill():
    """The budget of tests/plan.rs:248-282 (8 GB of device memory, where the reference moves the
    expert pool to pinned RAM): with one berth the same call fails and names the sizes."""
    plan = P.build_plan(shape_35b())
    with pytest.raises(P.PlanError) as e:
        P.place(plan, bytes_35b(), P.HbmBudget(8_000_000_000, 2_500_000_000))
    assert e.value.kind == P.ErrorKind.WEIGHTS_EXCEED_HBM
    assert str(e.value) == ("weights (17550000000 bytes) plus the HBM reservation (2500000000 bytes) exceed HBM "
                            "(8000000000 bytes); this build keeps every tensor resident")
    # the shared expert and the router are backbone: only `experts` names are scaled by k / E
    names = [n for n, _ in bytes_35b().tensors]
    assert not P.is_routed_expert("model.language_model.layers.0.mlp.shared_expert.down_proj.trellis")
    assert not P.is_routed_expert("model.language_model.layers.0.mlp.gate.weight")
    assert sum(P.is_routed_expert(n) for n in names) == 2


def test_later_and_unknown_architectures():
    """tests/plan.rs:285-307."""
    for arch in (P.ARCH_MINICPM_V4_7, P.ARCH_QWEN4_EXP):
        shape = shape_35b()
        shape.arch_string = arch
        with pytest.raises(P.PlanError, match=f"architecture `{arch}` is a later stage and is not planned yet") as e:
            P.build_plan(shape)
        assert e.value.kind == P.ErrorKind.NOT_YET
    for arch in ("Qwen3_5ForCausalLM", "Qwen3_5MoeForCausalLM", "LlamaForCausalLM", ""):
        shape = shape_27b()
        shape.arch_string = arch
        with pytest.raises(P.PlanError) as e:
            P.build_plan(shape)
        assert e.value.kind == P.ErrorKind.UNKNOWN_ARCH and str(e.value) == f"unknown architecture `{arch}`"


def _plan_error(shape):
    with pytest.raises(P.PlanError) as e:
        P.build_plan(shape)
    return e.value


def test_bad_shapes():
    """tests/plan.rs:310-362 plus every zero check of plan.rs:221-259."""
    dense = shape_27b()
    dense.layer_kinds.pop()
    err = _plan_error(dense)
    assert err.kind == P.ErrorKind.LAYER_COUNT and str(err) == "layer_kinds has 63 entries but num_layers is 64"
    with_moe = shape_27b()
    with_moe.moe = shape_35b().moe
    err = _plan_error(with_moe)
    assert err.kind == P.ErrorKind.UNEXPECTED_MOE and str(err) == f"{P.ARCH_QWEN3_5} is dense and does not take MoE dims"
    missing = shape_35b()
    missing.moe = None
    err = _plan_error(missing)
    assert err.kind == P.ErrorKind.MISSING_MOE and str(err) == f"{P.ARCH_QWEN3_5_MOE} requires MoE dims"
    for field in ("hidden_size", "head_dim", "num_q_heads", "num_kv_heads", "vocab_size"):
        zero = shape_27b()
        setattr(zero, field, 0)
        err = _plan_error(zero)
        assert err.kind == P.ErrorKind.ZERO and str(err) == f"{field} must be non-zero"
    for i, field in enumerate(("num_k_heads", "num_v_heads", "key_head_dim", "value_head_dim", "conv_kernel_dim")):
        zero = shape_27b()
        dims = [16, 48, 128, 128, 4]
        dims[i] = 0
        zero.gdn = P.GdnDims(*dims)
        assert str(_plan_error(zero)) == f"gdn.{field} must be non-zero"
        zero.layer_kinds = [P.LayerKind.FULL_ATTENTION] * 64       # the GDN widths only matter when a layer uses them
        assert len(P.build_plan(zero).layers) == 64
    for i, field in enumerate(("num_experts", "experts_per_tok", "moe_intermediate", "shared_intermediate")):
        zero = shape_35b()
        dims = [256, 8, 512, 512]
        dims[i] = 0
        zero.moe = P.MoeDims(*dims)
        assert str(_plan_error(zero)) == f"moe.{field} must be non-zero"
    too_many = shape_35b()
    too_many.moe = P.MoeDims(256, 300, 512, 512)
    err = _plan_error(too_many)
    assert err.kind == P.ErrorKind.EXPERTS_PER_TOK and str(err) == "experts_per_tok (300) exceeds num_experts (256)"
    none = shape_27b()
    none.num_layers, none.layer_kinds = 0, []
    assert _plan_error(none).kind == P.ErrorKind.NO_LAYERS
    with pytest.raises(P.PlanError, match="unknown layer kind `sliding_attention`") as e:
        P.LayerKind.from_config("sliding_attention")
    assert e.value.kind == P.ErrorKind.UNKNOWN_LAYER_KIND
    assert P.LayerKind.from_config("linear_attention") == P.LayerKind.LINEAR_ATTENTION
    assert P.LayerKind.from_config("full_attention") == P.LayerKind.FULL_ATTENTION
    assert P.LayerKind.FULL_ATTENTION.as_str() == "full_attention"


def test_overflowing_budgets():
    """tests/plan.rs:365-406 with one berth: what does not fit beside the reservation is refused."""
    dense = P.build_plan(shape_27b())
    with pytest.raises(P.PlanError) as e:
        P.place(dense, P.TensorBytes([("lm_head.weight", 13_200_000_000)]), P.HbmBudget(16_000_000_000, 4_600_000_000))
    assert e.value.kind == P.ErrorKind.WEIGHTS_EXCEED_HBM
    assert str(e.value) == ("weights (13200000000 bytes) plus the HBM reservation (4600000000 bytes) exceed HBM "
                            "(16000000000 bytes); this build keeps every tensor resident")
    moe, weights = P.build_plan(shape_35b()), bytes_35b()
    with pytest.raises(P.PlanError) as e:
        P.place(moe, weights, this_machine(24 * GIB + 1))
    assert e.value.kind == P.ErrorKind.RESERVATION_EXCEEDS_HBM
    assert str(e.value) == f"HBM reservation of {24 * GIB + 1} bytes exceeds the HBM budget of {24 * GIB} bytes"
    with pytest.raises(P.PlanError) as e:
        P.place(moe, weights, P.HbmBudget.mi355x(288 * GIB - 10_000_000_000))
    assert e.value.kind == P.ErrorKind.WEIGHTS_EXCEED_HBM
    # exactly full is placed
    placed = P.place(moe, weights, P.HbmBudget(17_550_000_000 + 7, 7))
    assert placed.resident == 17_550_000_000


def test_placement_input_checks_and_arithmetic():
    """place.rs:242-259 (names), :97-107 and :294-304 (sums), :367-376 (the slice is scaled once, in 128 bits)."""
    moe = P.build_plan(shape_35b())
    with pytest.raises(P.PlanError, match="tensor name is empty") as e:
        P.place(moe, P.TensorBytes([("", 1)]))
    assert e.value.kind == P.ErrorKind.EMPTY_NAME
    with pytest.raises(P.PlanError, match="duplicate tensor name `a.b`") as e:
        P.place(moe, P.TensorBytes([("a.b", 1), ("c", 2), ("a.b", 3)]))
    assert e.value.kind == P.ErrorKind.DUPLICATE_TENSOR
    big = (1 << 64) - 1
    with pytest.raises(P.PlanError, match="tensor byte sizes overflow u64") as e:
        P.place(moe, P.TensorBytes([("a", big), ("b", 1)]), P.HbmBudget(big, 0))
    assert e.value.kind == P.ErrorKind.OVERFLOW
    # bytes * 8 would not fit 64 bits; the quotient does
    placed = P.place(moe, P.TensorBytes([("x.experts.w", big - 5), ("y", 5)]), P.HbmBudget(big, 0))
    assert placed.bytes_moved == 5 + (big - 5) * 8 // 256
    # per-tensor truncation would lose a byte here: 3 tensors of 100 bytes -> 300 * 8 // 256 = 9, not 3 * 3
    placed = P.place(moe, P.TensorBytes([(f"l.{i}.experts.w", 100) for i in range(3)]))
    assert placed.bytes_moved == 9
    # an empty list is a valid placement
    assert P.place(moe, P.TensorBytes([])) == P.Placement(0, 0)


def test_routed_expert_name_rule():
    """tests/plan.rs:409-429."""
    L = "model.language_model.layers.0."
    assert P.is_routed_expert(L + "mlp.experts.gate_up_proj.trellis")
    assert P.is_routed_expert(L + "mlp.experts.12.down_proj.trellis")
    assert P.is_routed_expert("experts") and P.is_routed_expert("a.experts") and P.is_routed_expert("experts.b")
    for name in (L + "mlp.shared_expert.down_proj.trellis", L + "mlp.shared_expert_gate.weight", L + "mlp.gate.weight",
                 L + "linear_attn.out_proj.trellis", "lm_head.weight", "", "expert", "experts2.w", "my_experts.w"):
        assert not P.is_routed_expert(name), name


def test_mi355x_budget():
    """The counterpart of tests/plan.rs:432-443 for this build's default machine."""
    b = P.HbmBudget.mi355x(4)
    assert (b.hbm_bytes, b.reserved_bytes) == (288 << 30, 4)
    assert P.HbmBudget() == P.HbmBudget.mi355x(0)


# ---------------------------------------------------------------------------------------------
# config.json -> ModelShape (tests/from_exl3_shape.rs)

def config_json(arch=P.ARCH_QWEN3_5, num_layers=2, layer_types=("full_attention", "linear_attention"), hidden=96,
                head_dim=40, q_heads=6, kv_heads=3, vocab=12_345, gdn=(7, 11, 13, 17, 5), moe=None):
    text = {
        "num_hidden_layers": num_layers, "hidden_size": hidden, "head_dim": head_dim, "num_attention_heads": q_heads,
        "num_key_value_heads": kv_heads, "vocab_size": vocab, "tie_word_embeddings": False,
        "layer_types": list(layer_types), "linear_num_key_heads": gdn[0], "linear_num_value_heads": gdn[1],
        "linear_key_head_dim": gdn[2], "linear_value_head_dim": gdn[3], "linear_conv_kernel_dim": gdn[4],
        "attn_output_gate": True,
    }
    text.update(moe or {})
    return json.dumps({"architectures": [arch], "text_config": text,
                       "quantization_config": {"quant_method": "exl3", "bits": 4.0, "head_bits": 6}}).encode()


def test_dense_config_copies_widths_and_layer_order():
    """tests/from_exl3_shape.rs:94-120."""
    shape = P.model_shape(config_json())
    assert shape == P.ModelShape(P.ARCH_QWEN3_5, 2, [P.LayerKind.FULL_ATTENTION, P.LayerKind.LINEAR_ATTENTION], 96, 40,
                                 6, 3, P.GdnDims(7, 11, 13, 17, 5), None, 12_345)
    assert [l.mixer for l in P.build_plan(shape).layers] == [P.Mixer.FULL_ATTN, P.Mixer.GDN]


def test_moe_config_copies_all_four_expert_fields():
    """tests/from_exl3_shape.rs:122-168."""
    moe = {"num_experts": 256, "num_experts_per_tok": 8, "moe_intermediate_size": 512,
           "shared_expert_intermediate_size": 768}
    shape = P.model_shape(config_json(P.ARCH_QWEN3_5_MOE, 2, ("linear_attention", "full_attention"), 2048, 256, 16, 2,
                                      248_144, (16, 32, 128, 64, 4), moe))
    assert shape == P.ModelShape(P.ARCH_QWEN3_5_MOE, 2, [P.LayerKind.LINEAR_ATTENTION, P.LayerKind.FULL_ATTENTION],
                                 2048, 256, 16, 2, P.GdnDims(16, 32, 128, 64, 4), P.MoeDims(256, 8, 512, 768), 248_144)
    plan = P.build_plan(shape)
    assert [l.mixer for l in plan.layers] == [P.Mixer.GDN, P.Mixer.FULL_ATTN]
    assert plan.layers[0].ffn == P.Ffn(P.Router(256, 8), P.SharedExpert(768), P.RoutedExperts(256, 8, 512))


def test_unknown_layer_type_and_partial_moe():
    """tests/from_exl3_shape.rs:170-215."""
    with pytest.raises(P.PlanError) as e:
        P.model_shape(config_json(layer_types=("linear_attention", "qsa")))
    assert e.value.kind == P.ErrorKind.UNKNOWN_LAYER_TYPE and str(e.value) == "layer 1: unknown layer type `qsa`"
    with pytest.raises(P.PlanError) as e:
        P.model_shape(config_json(moe={"num_experts": 256, "moe_intermediate_size": 512}))
    assert e.value.kind == P.ErrorKind.INCOMPLETE_MOE
    assert str(e.value) == "incomplete MoE config, missing num_experts_per_tok, shared_expert_intermediate_size"
    with pytest.raises(P.PlanError) as e:
        P.model_shape(config_json(moe={"shared_expert_intermediate_size": 32}))
    assert str(e.value) == "incomplete MoE config, missing num_experts, num_experts_per_tok, moe_intermediate_size"


def test_moe_option_follows_the_four_fields_not_the_architecture():
    """tests/from_exl3_shape.rs:217-239."""
    moe = {"num_experts": 4, "num_experts_per_tok": 2, "moe_intermediate_size": 8, "shared_expert_intermediate_size": 16}
    shape = P.model_shape(config_json(moe=moe))
    assert shape.arch_string == P.ARCH_QWEN3_5 and shape.moe == P.MoeDims(4, 2, 8, 16)
    assert _plan_error(shape).kind == P.ErrorKind.UNEXPECTED_MOE
    bare = P.model_shape(config_json(arch=P.ARCH_QWEN3_5_MOE))
    assert bare.arch_string == P.ARCH_QWEN3_5_MOE and bare.moe is None
    assert _plan_error(bare).kind == P.ErrorKind.MISSING_MOE


# ---------------------------------------------------------------------------------------------
# checkpoint -> TensorBytes (tests/from_exl3_bytes.rs)

def _zeros(name, dtype, shape):
    size = {"I16": 2, "F16": 2, "BF16": 2, "I32": 4, "F32": 4}[dtype]
    n = 1
    for d in shape:
        n *= d
    return (name, dtype, shape, bytes(n * size))


def test_tensor_bytes_sums_owned_parts_keeps_expert_names_and_drops_vision_and_mtp(tmp_path):
    """tests/from_exl3_bytes.rs:278-412, the same tensor list."""
    expert = "model.language_model.layers.0.mlp.experts.3.gate_proj"
    fused = "model.language_model.layers.1.mlp.experts.down_proj"
    shared = "model.language_model.layers.0.mlp.shared_expert.down_proj"
    dense = "model.language_model.layers.0.mlp.down_proj"
    vision = "model.visual.blocks.0.attn.q_proj"
    mtp_fc = "mtp.fc"
    parts = {
        expert: [("trellis", "I16", (1, 1, 64)), ("suh", "F16", (4,)), ("svh", "F16", (4,)), ("su", "I16", (1,)),
                 ("mul1", "I32", ())],
        fused: [("trellis", "I16", (1, 1, 16)), ("suh", "F16", (2,)), ("svh", "F16", (2,)), ("mul1", "I32", ())],
        shared: [("trellis", "I16", (1, 1, 32)), ("su", "I16", (1,)), ("sv", "I16", (1,)), ("bias", "F16", (2,)),
                 ("mcg", "I32", ())],
        dense: [("trellis", "I16", (1, 1, 16)), ("suh", "F16", (2,)), ("svh", "F16", (2,))],
        vision: [("trellis", "I16", (1, 1, 16)), ("suh", "F16", (2,)), ("svh", "F16", (2,)), ("bias", "F16", (2,)),
                 ("mul1", "I32", ())],
        mtp_fc: [("trellis", "I16", (1, 1, 16)), ("suh", "F16", (2,)), ("svh", "F16", (2,)), ("mul1", "I32", ())],
    }
    tensors = [_zeros(f"{prefix}.{suffix}", dtype, shape) for prefix, items in parts.items()
               for suffix, dtype, shape in items]
    L0 = "model.language_model.layers.0."
    others = [
        _zeros("model.language_model.embed_tokens.weight", "BF16", (2, 2)),
        _zeros("model.language_model.norm.weight", "BF16", (4,)),
        _zeros(L0 + "input_layernorm.weight", "BF16", (4,)),
        _zeros(L0 + "linear_attn.A_log", "F32", (2,)),
        _zeros(L0 + "linear_attn.dt_bias", "F32", (2,)),
        _zeros(L0 + "linear_attn.conv1d.weight", "BF16", (2, 1, 4)),
        _zeros(L0 + "mlp.shared_expert_gate.weight", "F32", (4,)),
        _zeros("model.visual.pos_embed.weight", "BF16", (4,)),
        _zeros("mtp.norm.weight", "BF16", (4,)),
    ]
    tensors += others
    U.write_checkpoint(tmp_path, tensors)
    ckpt = exl3.Checkpoint.open(tmp_path)
    listed = P.tensor_bytes(ckpt)
    names = [n for n, _ in listed.tensors]
    assert names == sorted(names) and len(set(names)) == len(names)
    assert not any(n.startswith("model.visual.") or n.startswith("mtp.") for n in names)
    got = dict(listed.tensors)

    def part_len(prefix):
        return sum(len(body) for name, _, _, body in tensors
                   if name in {f"{prefix}.{s}" for s in ("trellis", "suh", "svh", "su", "sv", "bias", "mcg", "mul1")})

    for prefix in (expert, fused, shared, dense):
        assert got[prefix] == part_len(prefix), prefix
    assert part_len(expert) > 128 + 8 + 8
    assert P.is_routed_expert(expert) and P.is_routed_expert(fused) and not P.is_routed_expert(shared)
    for name, _, _, body in others[:7]:
        assert got[name] == len(body), name
    total = sum(len(body) for _, _, _, body in tensors)
    excluded = sum(len(body) for name, _, _, body in tensors if name.startswith(("model.visual.", "mtp.")))
    assert excluded > 0 and listed.total() + excluded == total
    assert len(listed.tensors) == 4 + 7
    # checkpoint -> plan -> placement: a dense plan moves every listed byte per token
    shape = P.model_shape(ckpt)
    shape.arch_string = P.ARCH_QWEN3_5
    placed = P.place(P.build_plan(shape), listed)
    assert placed.resident == placed.bytes_moved == listed.total()


# ---------------------------------------------------------------------------------------------
# the C++ layer used directly (berth_host_check, no device)

EXE = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "berth_amd", "lib", "berth_host_check")


def test_cpp_plan_of_a_moe_checkpoint(tmp_path):
    """config keys -> MoeDims -> Ffn::Moe on every layer -> bytes one token reads, in plan.hpp itself."""
    if not os.path.exists(EXE):
        pytest.skip("berth_host_check is not built")
    cfg = json.loads(json.dumps(U.CONFIG))
    cfg["architectures"] = [P.ARCH_QWEN3_5_MOE]
    cfg["text_config"].update(num_experts=4, num_experts_per_tok=2, moe_intermediate_size=128,
                              shared_expert_intermediate_size=256)
    mlp = "model.language_model.layers.0.mlp"
    tensors = [_zeros(f"{mlp}.gate.weight", "BF16", (4, 256))]                               # 2048 bytes of backbone
    for e in range(4):
        tensors += [_zeros(f"{mlp}.experts.{e}.down_proj.trellis", "I16", (8, 16, 32)),      # 8192
                    _zeros(f"{mlp}.experts.{e}.down_proj.suh", "F16", (128,)),               # 256
                    _zeros(f"{mlp}.experts.{e}.down_proj.svh", "F16", (256,))]               # 512
    tensors += [_zeros(f"{mlp}.shared_expert.down_proj.trellis", "I16", (16, 16, 32)),       # 16384
                _zeros(f"{mlp}.shared_expert.down_proj.suh", "F16", (256,)),
                _zeros(f"{mlp}.shared_expert.down_proj.svh", "F16", (256,)),
                _zeros("mtp.norm.weight", "BF16", (4,))]
    U.write_checkpoint(tmp_path, tensors, cfg)
    r = subprocess.run([EXE, "ckpt-plan", str(tmp_path)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    backbone, pool = 2048 + 16384 + 512 + 512, 4 * (8192 + 256 + 512)
    assert (f"plan arch={P.ARCH_QWEN3_5_MOE} layers=2 moe_layers=2 tensors=6 expert_tensors=4 "
            f"resident={backbone + pool} bytes_moved={backbone + pool * 2 // 4}") in r.stdout
    assert "ffn router=4/2 shared=256 experts=4/2/128" in r.stdout
    # the same through the C interface
    ckpt = exl3.Checkpoint.open(tmp_path)
    placed = P.place(P.build_plan(P.model_shape(ckpt)), P.tensor_bytes(ckpt))
    assert (placed.resident, placed.bytes_moved) == (backbone + pool, backbone + pool // 2)
    # a dense architecture string with MoE keys is refused by the plan, as in the reference
    cfg["architectures"] = [P.ARCH_QWEN3_5]
    U.write_checkpoint(tmp_path, tensors, cfg)
    r = subprocess.run([EXE, "ckpt-plan", str(tmp_path)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "is dense and does not take MoE dims" in r.stderr


def test_cpp_half_conversions_round_like_ieee(tmp_path):
    """The loaders' fp32 -> fp16 (router weights stored in BF16 / F32) against numpy's conversion."""
    if not os.path.exists(EXE):
        pytest.skip("berth_host_check is not built")
    rng = np.random.default_rng(5)
    special = np.array([0.0, -0.0, 1.0, -1.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, np.inf, -np.inf, 5.96e-8, 2.98e-8,
                        2.9802322e-8, 2.9802326e-8, 6.1e-5, 6.0975e-5, 6.103515625e-5, 1.0009765625, 1.00048828125,
                        1.00146484375, 0.33333334, 1e-10, -1e-10], dtype=np.float32)
    bits = rng.integers(0, 1 << 32, 200_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    near = (rng.standard_normal(100_000) * rng.choice([1e-6, 1e-4, 1e-2, 1.0, 100.0, 3e4], 100_000)).astype(np.float32)
    halves = np.arange(1 << 16, dtype=np.uint16).view(np.float16).astype(np.float32)          # every fp16 value
    with np.errstate(invalid="ignore"):
        ties = (halves[:-1].astype(np.float64) + halves[1:].astype(np.float64)) / 2           # exact midpoints
    x = np.concatenate([special, bits[~np.isnan(bits)], near, halves[~np.isnan(halves)],
                        ties[np.isfinite(ties)].astype(np.float32)])
    x.tofile(tmp_path / "x.f32")
    r = subprocess.run([EXE, "f16", str(tmp_path)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(tmp_path / "y.u16", dtype=np.uint16)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    assert np.array_equal(got, want.view(np.uint16))
    assert np.array_equal(np.fromfile(tmp_path / "y.f32", dtype=np.float32).view(np.uint32),
                          want.astype(np.float32).view(np.uint32))
