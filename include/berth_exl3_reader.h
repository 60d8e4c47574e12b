/*
 * berth_exl3_reader.h — C ABI of libberth_exl3_reader.so: the EXL3 checkpoint
 * reader (host only; no device call is made).
 *
 * The reference reads checkpoints with a Rust crate that has no foreign
 * interface; this header is the surface a non-Rust host (and this build's C++
 * engine layer and tests) uses for the same records.  Each entry cites the
 * reference item it corresponds to.  Conventions:
 *   - return 0 on success, -1 on error; `berth_ckpt_last_error` is a
 *     thread-local C string with the reference's message text
 *     (crates/berth-exl3/src/error.rs:5-31), `berth_ckpt_last_error_kind` its
 *     kind, `berth_ckpt_last_error_field` the field or path it names;
 *   - every `const char*` and array inside a returned struct is owned by the
 *     handle it came from and lives until that handle is freed;
 *   - tensor bodies are never read, except packed `su` / `sv` sign words by
 *     `berth_ckpt_linear_unpack_signs`.
 */
#ifndef BERTH_EXL3_READER_H
#define BERTH_EXL3_READER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct berth_ckpt berth_ckpt;                 /* crates/berth-exl3/src/checkpoint.rs:21-31 */
typedef struct berth_ckpt_config berth_ckpt_config;   /* crates/berth-exl3/src/config.rs:57-100 */

/* error.rs:5-31 */
enum { BERTH_CKPT_OK = 0, BERTH_CKPT_MISSING_FIELD = 1, BERTH_CKPT_BAD_FIELD = 2, BERTH_CKPT_READ = 3,
       BERTH_CKPT_PARSE = 4, BERTH_CKPT_ARGUMENT = 5 };
const char* berth_ckpt_last_error(void);
int berth_ckpt_last_error_kind(void);
const char* berth_ckpt_last_error_field(void);

/* dtype.rs:6-23, in that order: BOOL U8 I8 I16 U16 I32 U32 I64 U64 F16 BF16 F32 F64 F8_E4M3 F8_E5M2 F8_E8M0 */
const char* berth_ckpt_dtype_name(int dtype);   /* dtype.rs:49-68; NULL if out of range */
int berth_ckpt_dtype_parse(const char* name);   /* dtype.rs:27-47; -1 if unknown */
uint64_t berth_ckpt_dtype_size(int dtype);      /* dtype.rs:71-78; 0 if out of range */

/* safetensors.rs:14-33 */
typedef struct {
    const char* name;
    const char* shard;
    int dtype;
    int rank;
    const uint64_t* shape;
    uint64_t offset;   /* absolute byte offset in `shard` */
    uint64_t length;   /* byte length of the body */
} berth_ckpt_tensor;

/* linear.rs:12-151.  codebook: 0 mcg, 1 mul1, 2 default (3INST) — note this is the
 * reader's enumeration order, not the kernel ABI's; `kernel_codebook` is the value
 * berth_exl3_linear takes (0 default, 1 mcg, 2 mul1).  twice_k = 2 * bits per weight
 * (3, 5, 7 are the half rates 1.5, 2.5, 3.5). */
typedef struct {
    const char* prefix;
    berth_ckpt_tensor trellis;
    berth_ckpt_tensor input_scale;
    berth_ckpt_tensor output_scale;
    berth_ckpt_tensor bias;   /* valid when has_bias */
    int input_packed;
    int output_packed;
    int has_bias;
    int codebook;
    int kernel_codebook;
    int twice_k;
} berth_ckpt_linear;

/* config.rs:16-100.  Optional integers come with a has_ flag; optional strings are NULL
 * when absent.  layer_type_kinds: 0 linear_attention, 1 full_attention, 2 other. */
typedef struct {
    const char* arch_string;
    uint32_t num_hidden_layers, hidden_size, head_dim, num_attention_heads, num_key_value_heads, vocab_size;
    uint32_t linear_conv_kernel_dim, linear_num_key_heads, linear_num_value_heads;
    uint32_t linear_key_head_dim, linear_value_head_dim;
    int tie_word_embeddings, attn_output_gate;
    int has_intermediate_size, has_num_experts, has_num_experts_per_tok, has_moe_intermediate_size,
        has_shared_expert_intermediate_size;
    uint32_t intermediate_size, num_experts, num_experts_per_tok, moe_intermediate_size,
        shared_expert_intermediate_size;
    size_t num_layer_types;
    const int* layer_type_kinds;
    const char* const* layer_type_names;
    /* quantization_config (config.rs:26-55) */
    const char* quant_method;
    double bits;
    uint32_t head_bits;
    const char* codebook;
    const char* version;
    const char* out_scales;
    int has_vision_bits, has_mtp_bits, has_calibration;
    uint32_t vision_bits, mtp_bits, calibration_rows, calibration_cols;
} berth_ckpt_model_config;

/* Checkpoint::open (checkpoint.rs:38-72): config.json, the shard index when present, and
 * every shard header. */
int berth_ckpt_open(const char* dir, berth_ckpt** out);
void berth_ckpt_free(berth_ckpt* ckpt);
const char* berth_ckpt_directory(const berth_ckpt* ckpt);
const berth_ckpt_config* berth_ckpt_config_of(const berth_ckpt* ckpt);   /* borrowed from ckpt */

/* ModelConfig::from_slice (config.rs:104-108) on bytes the caller holds */
int berth_ckpt_config_parse(const char* json, size_t len, berth_ckpt_config** out);
void berth_ckpt_config_free(berth_ckpt_config* cfg);
int berth_ckpt_config_get(const berth_ckpt_config* cfg, berth_ckpt_model_config* out);

/* TensorIndex (safetensors.rs:35-78): sorted by name */
size_t berth_ckpt_tensor_count(const berth_ckpt* ckpt);
int berth_ckpt_tensor_at(const berth_ckpt* ckpt, size_t i, berth_ckpt_tensor* out);
int berth_ckpt_tensor_find(const berth_ckpt* ckpt, const char* name, berth_ckpt_tensor* out);   /* 1 found, 0 absent */

/* Checkpoint::linears (checkpoint.rs:74-77), sorted by prefix; other_tensors (:79-83) */
size_t berth_ckpt_linear_count(const berth_ckpt* ckpt);
int berth_ckpt_linear_at(const berth_ckpt* ckpt, size_t i, berth_ckpt_linear* out);
int berth_ckpt_linear_find(const berth_ckpt* ckpt, const char* prefix, berth_ckpt_linear* out);  /* index, or -1 */
size_t berth_ckpt_other_count(const berth_ckpt* ckpt);
int berth_ckpt_other_at(const berth_ckpt* ckpt, size_t i, berth_ckpt_tensor* out);

/* LinearExl3::unpack_input_signs / unpack_output_signs (linear.rs:139-151): reads the packed
 * tensor's own byte range and expands it to fp16 +-1 bit patterns.  `*written` is the number
 * of values the tensor holds; nothing is written when `capacity` is smaller. */
int berth_ckpt_linear_unpack_signs(const berth_ckpt* ckpt, size_t linear, int output_side, uint16_t* out,
                                   size_t capacity, size_t* written);
/* unpack_signs (signs.rs:25-46) on bytes the caller holds; out has 8 * nbytes entries */
int berth_ckpt_unpack_signs(const uint8_t* packed_le, size_t nbytes, uint16_t* out);

/* read_tensor (crates/berth-engine/src/device.rs:49-63): the tensor's bytes into dst[length] */
int berth_ckpt_read_tensor(const berth_ckpt_tensor* tensor, void* dst, size_t capacity);

#ifdef __cplusplus
}
#endif
#endif
