/*
 * berth_plan.h — C ABI of the model planner in libberth_exl3_reader.so: model
 * shape -> per-layer plan (which layers carry a dense MLP, which a MoE block of
 * router + shared expert + routed experts) -> the bytes resident in HBM and the
 * bytes one decoded token reads.  The reference's three-tier placement (VRAM,
 * pinned RAM, SSD) is collapsed: one MI355X keeps the whole weight set in HBM.
 * Host only; no device call is made.
 *
 * The reference plans with a Rust crate (crates/berth-plan) that has no foreign
 * interface; this header is the surface a non-Rust host uses for the same
 * records.  Each entry cites the reference item it corresponds to.  Conventions:
 *   - return 0 on success, -1 on error; `berth_plan_last_error` is a
 *     thread-local C string with the reference's message text and
 *     `berth_plan_last_error_kind` one of the BERTH_PLAN_* values;
 *   - strings and arrays inside a handle live until the handle is freed.
 */
#ifndef BERTH_PLAN_H
#define BERTH_PLAN_H

#include <stddef.h>
#include <stdint.h>

#include "berth_exl3_reader.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ShapeError (shape.rs:107-131), PlanError (plan.rs:115-125), PlaceError (place.rs:126-173),
 * ConfigError (from_exl3/shape.rs:12-24) */
enum {
    BERTH_PLAN_OK = 0,
    BERTH_PLAN_NO_LAYERS = 1, BERTH_PLAN_LAYER_COUNT = 2, BERTH_PLAN_UNKNOWN_LAYER_KIND = 3,
    BERTH_PLAN_UNEXPECTED_MOE = 4, BERTH_PLAN_MISSING_MOE = 5, BERTH_PLAN_ZERO = 6, BERTH_PLAN_EXPERTS_PER_TOK = 7,
    BERTH_PLAN_NOT_YET = 20, BERTH_PLAN_UNKNOWN_ARCH = 21,
    BERTH_PLAN_EMPTY_NAME = 40, BERTH_PLAN_DUPLICATE_TENSOR = 41, BERTH_PLAN_OVERFLOW = 42,
    BERTH_PLAN_RESERVATION_EXCEEDS_HBM = 43, BERTH_PLAN_WEIGHTS_EXCEED_HBM = 44,
    BERTH_PLAN_INCONSISTENT_MOE = 47, BERTH_PLAN_INVALID_MOE = 48,
    BERTH_PLAN_UNKNOWN_LAYER_TYPE = 60, BERTH_PLAN_INCOMPLETE_MOE = 61,
    BERTH_PLAN_ARGUMENT = 90
};
const char* berth_plan_last_error(void);
int berth_plan_last_error_kind(void);

/* MoeDims (crates/berth-plan/src/shape.rs:64-69) */
typedef struct {
    uint32_t num_experts, experts_per_tok, moe_intermediate, shared_intermediate;
} berth_plan_moe_dims;

/* ModelShape (shape.rs:88-103).  layer_kinds: 0 linear_attention, 1 full_attention (shape.rs:10-15). */
typedef struct {
    const char* arch_string;
    uint32_t num_layers;
    const int* layer_kinds;
    size_t num_layer_kinds;
    uint32_t hidden_size, head_dim, num_q_heads, num_kv_heads;
    uint32_t gdn_num_k_heads, gdn_num_v_heads, gdn_key_head_dim, gdn_value_head_dim, gdn_conv_kernel_dim;
    int has_moe;
    berth_plan_moe_dims moe;
    uint32_t vocab_size;
} berth_plan_shape;

/* LayerKind::from_config (shape.rs:22-29): 0 / 1, or -1 with BERTH_PLAN_UNKNOWN_LAYER_KIND */
int berth_plan_layer_kind_from_config(const char* name);

typedef struct berth_plan berth_plan;   /* ModelPlan (plan.rs:99-111) */

/* model_shape (from_exl3/shape.rs:34-110).  arch_string and layer_kinds are borrowed from
 * `config` and live as long as it does.  MoE dims are present when all four config keys are
 * (num_experts, num_experts_per_tok, moe_intermediate_size, shared_expert_intermediate_size),
 * absent when none is; a partial set is BERTH_PLAN_INCOMPLETE_MOE naming the missing keys. */
int berth_plan_shape_from_config(const berth_ckpt_config* config, berth_plan_shape* out);

/* build_plan (plan.rs:133-163) */
int berth_plan_build(const berth_plan_shape* shape, berth_plan** out);
/* model_shape (from_exl3/shape.rs:34-110), then build_plan */
int berth_plan_from_config(const berth_ckpt_config* config, berth_plan** out);
void berth_plan_free(berth_plan* plan);

/* LayerPlan (plan.rs:61-67) with its Ffn (plan.rs:45-57) flattened.  mixer: 0 gdn, 1 full
 * attention (plan.rs:10-17).  ffn_is_moe 0: DenseMlp, the remaining fields are zero.
 * ffn_is_moe 1: router {num_experts, experts_per_tok} (plan.rs:24-27), shared expert
 * {intermediate_size} (plan.rs:31-33), routed experts {num_experts, experts_per_tok,
 * intermediate_size} (plan.rs:37-41). */
typedef struct {
    uint32_t index;
    int mixer;
    int ffn_is_moe;
    uint32_t router_num_experts, router_experts_per_tok;
    uint32_t shared_intermediate_size;
    uint32_t experts_num_experts, experts_experts_per_tok, experts_intermediate_size;
} berth_plan_layer;

typedef struct {
    const char* arch_string;
    uint32_t hidden_size, vocab_size, head_dim, num_q_heads, num_kv_heads;
    uint32_t gdn_num_k_heads, gdn_num_v_heads, gdn_key_head_dim, gdn_value_head_dim, gdn_conv_kernel_dim;
    size_t num_layers;
} berth_plan_summary;
int berth_plan_summary_of(const berth_plan* plan, berth_plan_summary* out);
int berth_plan_layer_at(const berth_plan* plan, size_t i, berth_plan_layer* out);

/* is_routed_expert (place.rs:175-187): 1 when a dot-separated segment of the name is "experts" */
int berth_plan_is_routed_expert(const char* name);

/* What the weights may take of the device (the role of MachineBudget, place.rs:39-61, with
 * its pinned-RAM tier gone).  berth_plan_budget_mi355x: 288 GiB of HBM. */
typedef struct {
    uint64_t hbm_bytes, reserved_bytes;
} berth_plan_budget;
void berth_plan_budget_mi355x(uint64_t reserved_bytes, berth_plan_budget* out);

/* place (place.rs:189-232, one berth) over n (name, bytes) pairs: every tensor is resident in
 * HBM, or the call fails with BERTH_PLAN_WEIGHTS_EXCEED_HBM.  `resident`: the bytes held;
 * `bytes_moved`: the bytes one decoded token reads (place.rs:345-376: every tensor for a dense
 * plan; for a MoE plan the backbone plus experts_per_tok / num_experts of the expert pool,
 * scaled once in 128-bit arithmetic).  budget NULL: one MI355X, nothing reserved. */
int berth_plan_place(const berth_plan* plan, const char* const* names, const uint64_t* bytes, size_t n,
                     const berth_plan_budget* budget, uint64_t* resident, uint64_t* bytes_moved);

/* tensor_bytes (from_exl3/bytes.rs:57-93): one entry per EXL3 linear (all its parts) and one per
 * other tensor, sorted by name, without the vision tower and the MTP head. */
typedef struct berth_plan_bytes berth_plan_bytes;
int berth_plan_tensor_bytes(const berth_ckpt* ckpt, berth_plan_bytes** out);
void berth_plan_bytes_free(berth_plan_bytes* list);
size_t berth_plan_bytes_count(const berth_plan_bytes* list);
int berth_plan_bytes_at(const berth_plan_bytes* list, size_t i, const char** name, uint64_t* bytes);
/* place() on a list from berth_plan_tensor_bytes */
int berth_plan_place_bytes(const berth_plan* plan, const berth_plan_bytes* list, const berth_plan_budget* budget,
                           uint64_t* resident, uint64_t* bytes_moved);

#ifdef __cplusplus
}
#endif
#endif
