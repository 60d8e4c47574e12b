// C interface of the model planner (include/berth_plan.h) over plan.hpp.  Host only.
// Exceptions stop here: every entry returns a status and leaves the message in a
// thread-local string.
#include "../../../include/berth_plan.h"
#include "plan.hpp"
#include "reader_handles.hpp"

#include <memory>
#include <new>

using namespace berth::plan;

struct berth_plan {
    ModelPlan plan;
};
struct berth_plan_bytes {
    TensorBytes list;
};

namespace {

thread_local std::string g_error;
thread_local int g_kind = BERTH_PLAN_OK;

int ok()
{
    g_error.clear();
    g_kind = BERTH_PLAN_OK;
    return 0;
}
int fail(int kind, const std::string& what)
{
    g_error = what;
    g_kind = kind;
    return -1;
}

template <typename F>
int guarded(F&& body)
{
    try {
        body();
        return ok();
    } catch (const Error& e) {
        return fail((int)e.kind, e.what());
    } catch (const std::exception& e) {
        return fail(BERTH_PLAN_ARGUMENT, e.what());
    }
}

ModelShape shape_of(const berth_plan_shape& in)
{
    ModelShape s;
    s.arch_string = in.arch_string ? in.arch_string : "";
    s.num_layers = in.num_layers;
    for (size_t i = 0; i < in.num_layer_kinds; ++i) {
        if (in.layer_kinds[i] != 0 && in.layer_kinds[i] != 1)
            throw std::invalid_argument("layer_kinds[" + std::to_string(i) + "] is neither 0 nor 1");
        s.layer_kinds.push_back((LayerKind)in.layer_kinds[i]);
    }
    s.hidden_size = in.hidden_size;
    s.head_dim = in.head_dim;
    s.num_q_heads = in.num_q_heads;
    s.num_kv_heads = in.num_kv_heads;
    s.gdn = GdnDims{in.gdn_num_k_heads, in.gdn_num_v_heads, in.gdn_key_head_dim, in.gdn_value_head_dim,
                    in.gdn_conv_kernel_dim};
    if (in.has_moe)
        s.moe = MoeDims{in.moe.num_experts, in.moe.experts_per_tok, in.moe.moe_intermediate, in.moe.shared_intermediate};
    s.vocab_size = in.vocab_size;
    return s;
}

int place_list(const berth_plan* plan, const TensorBytes& list, const berth_plan_budget* budget, uint64_t* resident,
               uint64_t* bytes_moved)
{
    return guarded([&] {
        HbmBudget b;
        if (budget) b = HbmBudget{budget->hbm_bytes, budget->reserved_bytes};
        const Placement placed = place(plan->plan, list, b);
        if (resident) *resident = placed.resident;
        if (bytes_moved) *bytes_moved = placed.bytes_moved;
    });
}

}  // namespace

extern "C" {

const char* berth_plan_last_error(void) { return g_error.c_str(); }
int berth_plan_last_error_kind(void) { return g_kind; }

int berth_plan_layer_kind_from_config(const char* name)
{
    if (!name) {
        fail(BERTH_PLAN_ARGUMENT, "berth_plan_layer_kind_from_config: null argument");
        return -1;
    }
    int kind = -1;
    if (guarded([&] { kind = (int)layer_kind_from_config(name); }) != 0) return -1;
    return kind;
}

int berth_plan_shape_from_config(const berth_ckpt_config* config, berth_plan_shape* out)
{
    if (!config || !out) return fail(BERTH_PLAN_ARGUMENT, "berth_plan_shape_from_config: null argument");
    return guarded([&] {
        const ModelShape s = model_shape(config->cfg);      // the checks; the arrays come from the handle
        *out = berth_plan_shape{};
        out->arch_string = config->cfg.arch_string.c_str();
        out->num_layers = s.num_layers;
        out->layer_kinds = config->kinds.data();            // 0 / 1 as in LayerKind: "other" was refused above
        out->num_layer_kinds = config->kinds.size();
        out->hidden_size = s.hidden_size;
        out->head_dim = s.head_dim;
        out->num_q_heads = s.num_q_heads;
        out->num_kv_heads = s.num_kv_heads;
        out->gdn_num_k_heads = s.gdn.num_k_heads;
        out->gdn_num_v_heads = s.gdn.num_v_heads;
        out->gdn_key_head_dim = s.gdn.key_head_dim;
        out->gdn_value_head_dim = s.gdn.value_head_dim;
        out->gdn_conv_kernel_dim = s.gdn.conv_kernel_dim;
        out->has_moe = s.moe ? 1 : 0;
        if (s.moe)
            out->moe = berth_plan_moe_dims{s.moe->num_experts, s.moe->experts_per_tok, s.moe->moe_intermediate,
                                           s.moe->shared_intermediate};
        out->vocab_size = s.vocab_size;
    });
}

int berth_plan_build(const berth_plan_shape* shape, berth_plan** out)
{
    if (!shape || !out || (shape->num_layer_kinds && !shape->layer_kinds))
        return fail(BERTH_PLAN_ARGUMENT, "berth_plan_build: null argument");
    *out = nullptr;
    return guarded([&] {
        auto handle = std::make_unique<berth_plan>();
        handle->plan = build_plan(shape_of(*shape));
        *out = handle.release();
    });
}

int berth_plan_from_config(const berth_ckpt_config* config, berth_plan** out)
{
    if (!config || !out) return fail(BERTH_PLAN_ARGUMENT, "berth_plan_from_config: null argument");
    *out = nullptr;
    return guarded([&] {
        auto handle = std::make_unique<berth_plan>();
        handle->plan = build_plan(model_shape(config->cfg));
        *out = handle.release();
    });
}

void berth_plan_free(berth_plan* plan) { delete plan; }

int berth_plan_summary_of(const berth_plan* plan, berth_plan_summary* out)
{
    if (!plan || !out) return fail(BERTH_PLAN_ARGUMENT, "berth_plan_summary_of: null argument");
    const ModelPlan& p = plan->plan;
    *out = berth_plan_summary{p.arch_string.c_str(), p.hidden_size,       p.vocab_size,         p.head_dim,
                              p.num_q_heads,         p.num_kv_heads,      p.gdn.num_k_heads,    p.gdn.num_v_heads,
                              p.gdn.key_head_dim,    p.gdn.value_head_dim, p.gdn.conv_kernel_dim, p.layers.size()};
    return ok();
}

int berth_plan_layer_at(const berth_plan* plan, size_t i, berth_plan_layer* out)
{
    if (!plan || !out) return fail(BERTH_PLAN_ARGUMENT, "berth_plan_layer_at: null argument");
    if (i >= plan->plan.layers.size()) return fail(BERTH_PLAN_ARGUMENT, "berth_plan_layer_at: index out of range");
    const LayerPlan& l = plan->plan.layers[i];
    *out = berth_plan_layer{};
    out->index = l.index;
    out->mixer = (int)l.mixer;
    out->ffn_is_moe = l.ffn.is_moe ? 1 : 0;
    if (l.ffn.is_moe) {
        out->router_num_experts = l.ffn.router.num_experts;
        out->router_experts_per_tok = l.ffn.router.experts_per_tok;
        out->shared_intermediate_size = l.ffn.shared.intermediate_size;
        out->experts_num_experts = l.ffn.experts.num_experts;
        out->experts_experts_per_tok = l.ffn.experts.experts_per_tok;
        out->experts_intermediate_size = l.ffn.experts.intermediate_size;
    }
    return ok();
}

int berth_plan_is_routed_expert(const char* name) { return name && is_routed_expert(name) ? 1 : 0; }

void berth_plan_budget_mi355x(uint64_t reserved_bytes, berth_plan_budget* out)
{
    if (out) *out = berth_plan_budget{kMi355xHbmBytes, reserved_bytes};
}

int berth_plan_place(const berth_plan* plan, const char* const* names, const uint64_t* bytes, size_t n,
                     const berth_plan_budget* budget, uint64_t* resident, uint64_t* bytes_moved)
{
    if (!plan || (n && (!names || !bytes))) return fail(BERTH_PLAN_ARGUMENT, "berth_plan_place: null argument");
    TensorBytes list;
    for (size_t i = 0; i < n; ++i) {
        if (!names[i]) return fail(BERTH_PLAN_ARGUMENT, "berth_plan_place: null tensor name");
        list.tensors.emplace_back(names[i], bytes[i]);
    }
    return place_list(plan, list, budget, resident, bytes_moved);
}

int berth_plan_tensor_bytes(const berth_ckpt* ckpt, berth_plan_bytes** out)
{
    if (!ckpt || !out) return fail(BERTH_PLAN_ARGUMENT, "berth_plan_tensor_bytes: null argument");
    *out = nullptr;
    return guarded([&] {
        auto handle = std::make_unique<berth_plan_bytes>();
        handle->list = tensor_bytes(ckpt->ckpt);
        *out = handle.release();
    });
}

void berth_plan_bytes_free(berth_plan_bytes* list) { delete list; }
size_t berth_plan_bytes_count(const berth_plan_bytes* list) { return list ? list->list.tensors.size() : 0; }

int berth_plan_bytes_at(const berth_plan_bytes* list, size_t i, const char** name, uint64_t* bytes)
{
    if (!list || i >= list->list.tensors.size()) return fail(BERTH_PLAN_ARGUMENT, "berth_plan_bytes_at: index out of range");
    if (name) *name = list->list.tensors[i].first.c_str();
    if (bytes) *bytes = list->list.tensors[i].second;
    return ok();
}

int berth_plan_place_bytes(const berth_plan* plan, const berth_plan_bytes* list, const berth_plan_budget* budget,
                           uint64_t* resident, uint64_t* bytes_moved)
{
    if (!plan || !list) return fail(BERTH_PLAN_ARGUMENT, "berth_plan_place_bytes: null argument");
    return place_list(plan, list->list, budget, resident, bytes_moved);
}

}  // extern "C"
