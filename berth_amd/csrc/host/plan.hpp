// Model shape -> per-layer plan -> placement, restated in C++ for the FFN half of the
// reference's planning crate:
//   ModelShape / MoeDims / LayerKind      crates/berth-plan/src/shape.rs:10-131
//   Router / SharedExpert / RoutedExperts / Ffn / LayerPlan / ModelPlan / build_plan
//                                         crates/berth-plan/src/plan.rs:10-267
//   is_routed_expert / place / bytes_moved crates/berth-plan/src/place.rs:175-376
//   model_shape / tensor_bytes            crates/berth-plan/src/from_exl3/{shape,bytes}.rs
// Same rules, same error texts for the shape and the plan.  The reference's placement over
// VRAM, pinned RAM and SSD is collapsed: one MI355X holds the whole weight set in its 288 GiB
// of HBM, so `place` only checks that it fits beside the reservation and does the accounting,
// above all bytes_moved, the bytes one decoded token reads, which is the algorithmic-bytes
// figure the MoE measurements are priced with.
// Header-only, host only.
#pragma once

#include "exl3_checkpoint.hpp"

#include <algorithm>
#include <cstdint>
#include <optional>
#include <stdexcept>
#include <string>
#include <unordered_set>
#include <utility>
#include <vector>

namespace berth::plan {

// one exception type; `kind` tells the reference's enum variant apart
class Error : public std::runtime_error {
public:
    enum class Kind : int {
        // shape.rs:107-131
        NoLayers = 1, LayerCount, UnknownLayerKind, UnexpectedMoe, MissingMoe, Zero, ExpertsPerTok,
        // plan.rs:115-125
        NotYet = 20, Unknown,
        // place.rs:126-173
        EmptyName = 40, DuplicateTensor, Overflow, ReservationExceedsHbm, WeightsExceedHbm,
        InconsistentMoe = 47, InvalidMoe,
        // from_exl3/shape.rs:12-24
        UnknownLayerType = 60, IncompleteMoe,
    };
    Kind kind;
    Error(Kind k, const std::string& what) : std::runtime_error(what), kind(k) {}
};

enum class LayerKind : int { LinearAttention = 0, FullAttention = 1 };      // shape.rs:10-15

inline LayerKind layer_kind_from_config(const std::string& name)            // shape.rs:22-29
{
    if (name == "linear_attention") return LayerKind::LinearAttention;
    if (name == "full_attention") return LayerKind::FullAttention;
    throw Error(Error::Kind::UnknownLayerKind, "unknown layer kind `" + name + "`");
}
inline const char* layer_kind_name(LayerKind k)                             // shape.rs:31-36
{
    return k == LayerKind::LinearAttention ? "linear_attention" : "full_attention";
}

struct GdnDims {                                                            // shape.rs:51-57
    uint32_t num_k_heads = 0, num_v_heads = 0, key_head_dim = 0, value_head_dim = 0, conv_kernel_dim = 0;
    bool operator==(const GdnDims& o) const
    {
        return num_k_heads == o.num_k_heads && num_v_heads == o.num_v_heads && key_head_dim == o.key_head_dim &&
               value_head_dim == o.value_head_dim && conv_kernel_dim == o.conv_kernel_dim;
    }
};

struct MoeDims {                                                            // shape.rs:64-69
    uint32_t num_experts = 0, experts_per_tok = 0, moe_intermediate = 0, shared_intermediate = 0;
    bool operator==(const MoeDims& o) const
    {
        return num_experts == o.num_experts && experts_per_tok == o.experts_per_tok &&
               moe_intermediate == o.moe_intermediate && shared_intermediate == o.shared_intermediate;
    }
};

// shape.rs:72-81
constexpr const char* kArchQwen35 = "Qwen3_5ForConditionalGeneration";
constexpr const char* kArchQwen35Moe = "Qwen3_5MoeForConditionalGeneration";
constexpr const char* kArchMiniCpmV47 = "MiniCPMV4_7ForConditionalGeneration";
constexpr const char* kArchQwen4Exp = "Qwen4ExpForConditionalGeneration";

struct ModelShape {                                                         // shape.rs:88-103
    std::string arch_string;
    uint32_t num_layers = 0;
    std::vector<LayerKind> layer_kinds;
    uint32_t hidden_size = 0, head_dim = 0, num_q_heads = 0, num_kv_heads = 0;
    GdnDims gdn;
    std::optional<MoeDims> moe;
    uint32_t vocab_size = 0;
};

enum class Mixer : int { Gdn = 0, FullAttn = 1, Qsa = 2 };                  // plan.rs:10-17

struct Router { uint32_t num_experts = 0, experts_per_tok = 0; };           // plan.rs:24-27
struct SharedExpert { uint32_t intermediate_size = 0; };                    // plan.rs:31-33
struct RoutedExperts { uint32_t num_experts = 0, experts_per_tok = 0, intermediate_size = 0; };   // plan.rs:37-41

struct Ffn {                                                                // plan.rs:45-57
    bool is_moe = false;            // false: DenseMlp; true: Moe{router, shared, experts}
    Router router;
    SharedExpert shared;
    RoutedExperts experts;
    static Ffn dense() { return Ffn{}; }
    static Ffn moe(const MoeDims& d)                                        // plan.rs:204-219
    {
        Ffn f;
        f.is_moe = true;
        f.router = Router{d.num_experts, d.experts_per_tok};
        f.shared = SharedExpert{d.shared_intermediate};
        f.experts = RoutedExperts{d.num_experts, d.experts_per_tok, d.moe_intermediate};
        return f;
    }
};

struct LayerPlan {                                                          // plan.rs:61-67
    uint32_t index = 0;
    Mixer mixer = Mixer::Gdn;
    Ffn ffn;
};

struct ModelPlan {                                                          // plan.rs:99-111
    std::string arch_string;
    uint32_t hidden_size = 0, vocab_size = 0, head_dim = 0, num_q_heads = 0, num_kv_heads = 0;
    GdnDims gdn;
    std::vector<LayerPlan> layers;
    // embedding {vocab_size, hidden_size}, final_norm {hidden_size} and lm_head {hidden_size, vocab_size}
    // repeat the two sizes above (plan.rs:71-93)
};

namespace detail {

inline void nonzero(uint32_t value, const char* field)                      // plan.rs:261-267
{
    if (value == 0) throw Error(Error::Kind::Zero, std::string(field) + " must be non-zero");
}

inline void validate_common(const ModelShape& s)                            // plan.rs:221-245
{
    if (s.layer_kinds.size() != (size_t)s.num_layers)
        throw Error(Error::Kind::LayerCount, "layer_kinds has " + std::to_string(s.layer_kinds.size()) +
                                                 " entries but num_layers is " + std::to_string(s.num_layers));
    if (s.num_layers == 0) throw Error(Error::Kind::NoLayers, "num_layers is 0");
    nonzero(s.hidden_size, "hidden_size");
    nonzero(s.head_dim, "head_dim");
    nonzero(s.num_q_heads, "num_q_heads");
    nonzero(s.num_kv_heads, "num_kv_heads");
    nonzero(s.vocab_size, "vocab_size");
    if (std::find(s.layer_kinds.begin(), s.layer_kinds.end(), LayerKind::LinearAttention) != s.layer_kinds.end()) {
        nonzero(s.gdn.num_k_heads, "gdn.num_k_heads");
        nonzero(s.gdn.num_v_heads, "gdn.num_v_heads");
        nonzero(s.gdn.key_head_dim, "gdn.key_head_dim");
        nonzero(s.gdn.value_head_dim, "gdn.value_head_dim");
        nonzero(s.gdn.conv_kernel_dim, "gdn.conv_kernel_dim");
    }
}

inline void validate_moe(const MoeDims& d)                                  // plan.rs:247-259
{
    nonzero(d.num_experts, "moe.num_experts");
    nonzero(d.experts_per_tok, "moe.experts_per_tok");
    nonzero(d.moe_intermediate, "moe.moe_intermediate");
    nonzero(d.shared_intermediate, "moe.shared_intermediate");
    if (d.experts_per_tok > d.num_experts)
        throw Error(Error::Kind::ExpertsPerTok, "experts_per_tok (" + std::to_string(d.experts_per_tok) +
                                                    ") exceeds num_experts (" + std::to_string(d.num_experts) + ")");
}

inline ModelPlan assemble(const ModelShape& s, const Ffn& ffn)              // plan.rs:165-202
{
    ModelPlan plan;
    plan.arch_string = s.arch_string;
    plan.hidden_size = s.hidden_size;
    plan.vocab_size = s.vocab_size;
    plan.head_dim = s.head_dim;
    plan.num_q_heads = s.num_q_heads;
    plan.num_kv_heads = s.num_kv_heads;
    plan.gdn = s.gdn;
    plan.layers.reserve(s.layer_kinds.size());
    for (size_t i = 0; i < s.layer_kinds.size(); ++i)
        plan.layers.push_back(LayerPlan{(uint32_t)i,
                                        s.layer_kinds[i] == LayerKind::LinearAttention ? Mixer::Gdn : Mixer::FullAttn, ffn});
    return plan;
}

}  // namespace detail

// plan.rs:133-163: the dense and the MoE Qwen3.5 family are planned; two named later
// architectures are NotYet; anything else is Unknown
inline ModelPlan build_plan(const ModelShape& shape)
{
    const std::string& arch = shape.arch_string;
    if (arch == kArchQwen35) {
        detail::validate_common(shape);
        if (shape.moe) throw Error(Error::Kind::UnexpectedMoe, arch + " is dense and does not take MoE dims");
        return detail::assemble(shape, Ffn::dense());
    }
    if (arch == kArchQwen35Moe) {
        detail::validate_common(shape);
        if (!shape.moe) throw Error(Error::Kind::MissingMoe, arch + " requires MoE dims");
        detail::validate_moe(*shape.moe);
        return detail::assemble(shape, Ffn::moe(*shape.moe));
    }
    if (arch == kArchMiniCpmV47 || arch == kArchQwen4Exp)
        throw Error(Error::Kind::NotYet, "architecture `" + arch + "` is a later stage and is not planned yet");
    throw Error(Error::Kind::Unknown, "unknown architecture `" + arch + "`");
}

// ------------------------------------------------------------------------------------------
// placement

constexpr uint64_t kMi355xHbmBytes = 288ull << 30;

// what the weights may take of the device: its HBM less what the caller keeps for the KV
// cache, activations and workspaces (the role of MachineBudget, place.rs:39-61, with its
// pinned-RAM tier gone)
struct HbmBudget {
    uint64_t hbm_bytes = kMi355xHbmBytes;
    uint64_t reserved_bytes = 0;
};

struct TensorBytes {                                                        // place.rs:71-79
    std::vector<std::pair<std::string, uint64_t>> tensors;
};

struct Placement {                                                          // place.rs:111-122, one berth
    uint64_t resident = 0;               // bytes held in HBM: every listed tensor
    uint64_t bytes_moved = 0;            // bytes one decoded token reads
};

// a tensor belongs to the routed expert pool when one dot-separated segment of its name is
// exactly "experts"; shared_expert, shared_expert_gate and the router (mlp.gate) are backbone
// (place.rs:175-187)
inline bool is_routed_expert(const std::string& name)
{
    size_t start = 0;
    while (start <= name.size()) {
        size_t end = name.find('.', start);
        if (end == std::string::npos) end = name.size();
        if (end - start == 7 && name.compare(start, 7, "experts") == 0) return true;
        start = end + 1;
    }
    return false;
}

namespace detail {

struct Classed {
    std::string name;
    uint64_t bytes;
    bool expert;
};

inline std::vector<Classed> classify(const TensorBytes& bytes)              // place.rs:242-259
{
    std::unordered_set<std::string> seen;
    std::vector<Classed> out;
    out.reserve(bytes.tensors.size());
    for (const auto& [name, size] : bytes.tensors) {
        if (name.empty()) throw Error(Error::Kind::EmptyName, "tensor name is empty");
        if (!seen.insert(name).second) throw Error(Error::Kind::DuplicateTensor, "duplicate tensor name `" + name + "`");
        out.push_back(Classed{name, size, is_routed_expert(name)});
    }
    return out;
}

inline std::string invalid_moe(uint32_t per_tok, uint32_t num_experts)
{
    return "invalid MoE routing: experts_per_tok=" + std::to_string(per_tok) + " num_experts=" + std::to_string(num_experts);
}

// (experts_per_tok, num_experts) every MoE layer agrees on, or nothing for a dense plan (place.rs:261-292)
inline std::optional<std::pair<uint32_t, uint32_t>> moe_ratio(const ModelPlan& plan)
{
    std::optional<std::pair<uint32_t, uint32_t>> found;
    for (const LayerPlan& layer : plan.layers) {
        if (!layer.ffn.is_moe) continue;
        const RoutedExperts& ex = layer.ffn.experts;
        const Router& router = layer.ffn.router;
        if (ex.num_experts == 0 || ex.experts_per_tok == 0 || ex.experts_per_tok > ex.num_experts)
            throw Error(Error::Kind::InvalidMoe, invalid_moe(ex.experts_per_tok, ex.num_experts));
        if (router.num_experts != ex.num_experts || router.experts_per_tok != ex.experts_per_tok)
            throw Error(Error::Kind::InconsistentMoe, "MoE layers disagree on the expert pool");
        const std::pair<uint32_t, uint32_t> ratio{ex.experts_per_tok, ex.num_experts};
        if (found && *found != ratio) throw Error(Error::Kind::InconsistentMoe, "MoE layers disagree on the expert pool");
        found = ratio;
    }
    return found;
}

template <typename Keep>
uint64_t sum_bytes(const std::vector<Classed>& classed, Keep keep)          // place.rs:294-304
{
    uint64_t total = 0;
    for (const Classed& t : classed)
        if (keep(t) && __builtin_add_overflow(total, t.bytes, &total))
            throw Error(Error::Kind::Overflow, "tensor byte sizes overflow u64");
    return total;
}

// bytes * per_tok / num_experts in 128 bits, truncated once (place.rs:367-376)
inline uint64_t portion(uint64_t bytes, uint32_t per_tok, uint32_t num_experts)
{
    if (num_experts == 0 || per_tok > num_experts) throw Error(Error::Kind::InvalidMoe, invalid_moe(per_tok, num_experts));
    const unsigned __int128 moved = (unsigned __int128)bytes * per_tok / num_experts;
    if (moved > (unsigned __int128)UINT64_MAX) throw Error(Error::Kind::Overflow, "tensor byte sizes overflow u64");
    return (uint64_t)moved;
}

}  // namespace detail

// place.rs:189-232 with one berth: everything is resident in HBM or the call fails.
// bytes_moved (place.rs:345-365): a dense plan reads every listed tensor once per token; a MoE
// plan reads the backbone plus experts_per_tok / num_experts of the routed-expert pool.
inline Placement place(const ModelPlan& plan, const TensorBytes& bytes, const HbmBudget& budget = HbmBudget{})
{
    using K = Error::Kind;
    auto n = [](uint64_t v) { return std::to_string(v); };
    if (budget.reserved_bytes > budget.hbm_bytes)
        throw Error(K::ReservationExceedsHbm, "HBM reservation of " + n(budget.reserved_bytes) +
                                                  " bytes exceeds the HBM budget of " + n(budget.hbm_bytes) + " bytes");
    const std::vector<detail::Classed> classed = detail::classify(bytes);
    const auto ratio = detail::moe_ratio(plan);
    const uint64_t backbone = detail::sum_bytes(classed, [](const detail::Classed& t) { return !t.expert; });
    const uint64_t experts = detail::sum_bytes(classed, [](const detail::Classed& t) { return t.expert; });
    uint64_t total = 0;
    if (__builtin_add_overflow(backbone, experts, &total)) throw Error(K::Overflow, "tensor byte sizes overflow u64");
    if (total > budget.hbm_bytes - budget.reserved_bytes)
        throw Error(K::WeightsExceedHbm, "weights (" + n(total) + " bytes) plus the HBM reservation (" +
                                             n(budget.reserved_bytes) + " bytes) exceed HBM (" + n(budget.hbm_bytes) +
                                             " bytes); this build keeps every tensor resident");
    Placement p;
    p.resident = total;
    p.bytes_moved = total;
    if (ratio) {
        p.bytes_moved = backbone;
        if (__builtin_add_overflow(p.bytes_moved, detail::portion(experts, ratio->first, ratio->second), &p.bytes_moved))
            throw Error(K::Overflow, "tensor byte sizes overflow u64");
    }
    return p;
}

// ------------------------------------------------------------------------------------------
// checkpoint -> shape and byte list

// from_exl3/shape.rs:34-110.  MoE dims are present when all four config keys are, absent when
// none is; a partial set names the missing keys in field order.
inline ModelShape model_shape(const exl3::ModelConfig& config)
{
    ModelShape s;
    s.arch_string = config.arch_string;
    s.num_layers = config.num_hidden_layers;
    for (size_t i = 0; i < config.layer_types.size(); ++i) {
        const exl3::LayerType& t = config.layer_types[i];
        if (t.kind == exl3::LayerType::Kind::Other)
            throw Error(Error::Kind::UnknownLayerType, "layer " + std::to_string(i) + ": unknown layer type `" + t.name + "`");
        s.layer_kinds.push_back(t.kind == exl3::LayerType::Kind::LinearAttention ? LayerKind::LinearAttention
                                                                                 : LayerKind::FullAttention);
    }
    s.hidden_size = config.hidden_size;
    s.head_dim = config.head_dim;
    s.num_q_heads = config.num_attention_heads;
    s.num_kv_heads = config.num_key_value_heads;
    s.gdn = GdnDims{config.linear_num_key_heads, config.linear_num_value_heads, config.linear_key_head_dim,
                    config.linear_value_head_dim, config.linear_conv_kernel_dim};
    const auto &e = config.num_experts, &k = config.num_experts_per_tok, &i = config.moe_intermediate_size,
               &sh = config.shared_expert_intermediate_size;
    if (e && k && i && sh) {
        s.moe = MoeDims{*e, *k, *i, *sh};
    } else if (e || k || i || sh) {
        std::string missing;
        auto add = [&](bool absent, const char* key) {
            if (absent) missing += (missing.empty() ? "" : ", ") + std::string(key);
        };
        add(!e, "num_experts");
        add(!k, "num_experts_per_tok");
        add(!i, "moe_intermediate_size");
        add(!sh, "shared_expert_intermediate_size");
        throw Error(Error::Kind::IncompleteMoe, "incomplete MoE config, missing " + missing);
    }
    s.vocab_size = config.vocab_size;
    return s;
}

// from_exl3/bytes.rs:18-93: one entry per quantized linear (all of its parts), one per tensor
// outside a linear; the vision tower and the MTP head are not on the text decode path
inline TensorBytes tensor_bytes(const exl3::Checkpoint& ckpt)
{
    auto off_decode_path = [](const std::string& name) {
        return name.rfind("model.visual.", 0) == 0 || name.rfind("mtp.", 0) == 0;
    };
    static const char* const parts[] = {"trellis", "suh", "svh", "su", "sv", "bias", "mcg", "mul1"};
    TensorBytes out;
    for (const exl3::LinearExl3& linear : ckpt.linears()) {
        if (off_decode_path(linear.prefix)) continue;
        uint64_t total = 0;
        for (const char* part : parts)
            if (const exl3::TensorInfo* info = ckpt.tensors.get(linear.prefix + "." + part)) total += info->length;
        out.tensors.emplace_back(linear.prefix, total);
    }
    for (const exl3::TensorInfo& info : ckpt.other_tensors()) {
        if (off_decode_path(info.name)) continue;
        out.tensors.emplace_back(info.name, info.length);
    }
    std::sort(out.tensors.begin(), out.tensors.end(),
              [](const auto& a, const auto& b) { return a.first < b.first; });
    return out;
}

}  // namespace berth::plan
