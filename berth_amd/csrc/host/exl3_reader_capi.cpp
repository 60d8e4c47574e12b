// C interface of the EXL3 checkpoint reader (include/berth_exl3_reader.h) over
// exl3_checkpoint.hpp.  Host only.  Exceptions stop here: every entry returns a
// status and leaves the message in a thread-local string.
#include "../../../include/berth_exl3_reader.h"
#include "exl3_checkpoint.hpp"
#include "reader_handles.hpp"

#include <algorithm>
#include <new>

using namespace berth::exl3;

namespace {

thread_local std::string g_error, g_field;
thread_local int g_kind = BERTH_CKPT_OK;

int ok()
{
    g_error.clear();
    g_field.clear();
    g_kind = BERTH_CKPT_OK;
    return 0;
}
int fail(int kind, const std::string& what, const std::string& field = "")
{
    g_error = what;
    g_field = field;
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
        return fail((int)e.kind, e.what(), e.field.empty() ? e.path : e.field);
    } catch (const std::bad_alloc&) {
        return fail(BERTH_CKPT_READ, "out of memory");
    } catch (const std::exception& e) {
        return fail(BERTH_CKPT_ARGUMENT, e.what());
    }
}

void view(const TensorInfo& t, berth_ckpt_tensor* out)
{
    out->name = t.name.c_str();
    out->shard = t.shard.c_str();
    out->dtype = (int)t.dtype;
    out->rank = (int)t.shape.size();
    out->shape = t.shape.data();
    out->offset = t.offset;
    out->length = t.length;
}

void view(const LinearExl3& l, berth_ckpt_linear* out)
{
    *out = berth_ckpt_linear{};
    out->prefix = l.prefix.c_str();
    view(l.trellis, &out->trellis);
    view(l.input_scale.tensor, &out->input_scale);
    view(l.output_scale.tensor, &out->output_scale);
    out->input_packed = l.input_scale.packed ? 1 : 0;
    out->output_packed = l.output_scale.packed ? 1 : 0;
    out->has_bias = l.bias ? 1 : 0;
    if (l.bias) view(*l.bias, &out->bias);
    out->codebook = (int)l.codebook;
    out->kernel_codebook = l.codebook == Codebook::Default ? 0 : l.codebook == Codebook::Mcg ? 1 : 2;
    out->twice_k = l.k.twice;
}

}  // namespace

extern "C" {

const char* berth_ckpt_last_error(void) { return g_error.c_str(); }
int berth_ckpt_last_error_kind(void) { return g_kind; }
const char* berth_ckpt_last_error_field(void) { return g_field.c_str(); }

const char* berth_ckpt_dtype_name(int dtype) { return dtype >= 0 && dtype < 16 ? dtype_name((DType)dtype) : nullptr; }
int berth_ckpt_dtype_parse(const char* name)
{
    DType d;
    return name && dtype_parse(name, &d) ? (int)d : -1;
}
uint64_t berth_ckpt_dtype_size(int dtype) { return dtype >= 0 && dtype < 16 ? dtype_size((DType)dtype) : 0; }

int berth_ckpt_open(const char* dir, berth_ckpt** out)
{
    if (!dir || !out) return fail(BERTH_CKPT_ARGUMENT, "berth_ckpt_open: null argument");
    *out = nullptr;
    return guarded([&] {
        auto handle = std::make_unique<berth_ckpt>();
        handle->ckpt = Checkpoint::open(dir);
        handle->config.cfg = handle->ckpt.config;
        handle->config.index();
        for (const auto& [name, info] : handle->ckpt.tensors) {
            (void)name;
            handle->tensors.push_back(&info);
        }
        *out = handle.release();
    });
}

void berth_ckpt_free(berth_ckpt* ckpt) { delete ckpt; }
const char* berth_ckpt_directory(const berth_ckpt* ckpt) { return ckpt ? ckpt->ckpt.directory.c_str() : nullptr; }
const berth_ckpt_config* berth_ckpt_config_of(const berth_ckpt* ckpt) { return ckpt ? &ckpt->config : nullptr; }

int berth_ckpt_config_parse(const char* json, size_t len, berth_ckpt_config** out)
{
    if ((!json && len) || !out) return fail(BERTH_CKPT_ARGUMENT, "berth_ckpt_config_parse: null argument");
    *out = nullptr;
    return guarded([&] {
        auto handle = std::make_unique<berth_ckpt_config>();
        handle->cfg = ModelConfig::from_slice(json ? json : "", len);
        handle->index();
        *out = handle.release();
    });
}

void berth_ckpt_config_free(berth_ckpt_config* cfg) { delete cfg; }

int berth_ckpt_config_get(const berth_ckpt_config* handle, berth_ckpt_model_config* o)
{
    if (!handle || !o) return fail(BERTH_CKPT_ARGUMENT, "berth_ckpt_config_get: null argument");
    const ModelConfig& c = handle->cfg;
    *o = berth_ckpt_model_config{};
    o->arch_string = c.arch_string.c_str();
    o->num_hidden_layers = c.num_hidden_layers;
    o->hidden_size = c.hidden_size;
    o->head_dim = c.head_dim;
    o->num_attention_heads = c.num_attention_heads;
    o->num_key_value_heads = c.num_key_value_heads;
    o->vocab_size = c.vocab_size;
    o->linear_conv_kernel_dim = c.linear_conv_kernel_dim;
    o->linear_num_key_heads = c.linear_num_key_heads;
    o->linear_num_value_heads = c.linear_num_value_heads;
    o->linear_key_head_dim = c.linear_key_head_dim;
    o->linear_value_head_dim = c.linear_value_head_dim;
    o->tie_word_embeddings = c.tie_word_embeddings;
    o->attn_output_gate = c.attn_output_gate;
    auto opt = [](const std::optional<uint32_t>& v, int* has, uint32_t* val) {
        *has = v ? 1 : 0;
        *val = v ? *v : 0;
    };
    opt(c.intermediate_size, &o->has_intermediate_size, &o->intermediate_size);
    opt(c.num_experts, &o->has_num_experts, &o->num_experts);
    opt(c.num_experts_per_tok, &o->has_num_experts_per_tok, &o->num_experts_per_tok);
    opt(c.moe_intermediate_size, &o->has_moe_intermediate_size, &o->moe_intermediate_size);
    opt(c.shared_expert_intermediate_size, &o->has_shared_expert_intermediate_size, &o->shared_expert_intermediate_size);
    o->num_layer_types = handle->kinds.size();
    o->layer_type_kinds = handle->kinds.data();
    o->layer_type_names = handle->names.data();
    const QuantizationConfig& q = c.quantization;
    o->quant_method = q.quant_method.c_str();
    o->bits = q.bits;
    o->head_bits = q.head_bits;
    o->codebook = q.codebook ? q.codebook->c_str() : nullptr;
    o->version = q.version ? q.version->c_str() : nullptr;
    o->out_scales = q.out_scales ? q.out_scales->c_str() : nullptr;
    opt(q.vision_bits, &o->has_vision_bits, &o->vision_bits);
    opt(q.mtp_bits, &o->has_mtp_bits, &o->mtp_bits);
    o->has_calibration = q.calibration ? 1 : 0;
    if (q.calibration) {
        o->calibration_rows = q.calibration->rows;
        o->calibration_cols = q.calibration->cols;
    }
    return ok();
}

size_t berth_ckpt_tensor_count(const berth_ckpt* ckpt) { return ckpt ? ckpt->tensors.size() : 0; }
int berth_ckpt_tensor_at(const berth_ckpt* ckpt, size_t i, berth_ckpt_tensor* out)
{
    if (!ckpt || !out || i >= ckpt->tensors.size()) return fail(BERTH_CKPT_ARGUMENT, "berth_ckpt_tensor_at: out of range");
    view(*ckpt->tensors[i], out);
    return ok();
}
int berth_ckpt_tensor_find(const berth_ckpt* ckpt, const char* name, berth_ckpt_tensor* out)
{
    if (!ckpt || !name) return fail(BERTH_CKPT_ARGUMENT, "berth_ckpt_tensor_find: null argument");
    const TensorInfo* t = ckpt->ckpt.tensors.get(name);
    ok();
    if (!t) return 0;
    if (out) view(*t, out);
    return 1;
}

size_t berth_ckpt_linear_count(const berth_ckpt* ckpt) { return ckpt ? ckpt->ckpt.linears().size() : 0; }
int berth_ckpt_linear_at(const berth_ckpt* ckpt, size_t i, berth_ckpt_linear* out)
{
    if (!ckpt || !out || i >= ckpt->ckpt.linears().size())
        return fail(BERTH_CKPT_ARGUMENT, "berth_ckpt_linear_at: out of range");
    view(ckpt->ckpt.linears()[i], out);
    return ok();
}
int berth_ckpt_linear_find(const berth_ckpt* ckpt, const char* prefix, berth_ckpt_linear* out)
{
    if (!ckpt || !prefix) return fail(BERTH_CKPT_ARGUMENT, "berth_ckpt_linear_find: null argument");
    const auto& ls = ckpt->ckpt.linears();
    for (size_t i = 0; i < ls.size(); ++i)
        if (ls[i].prefix == prefix) {
            if (out) view(ls[i], out);
            ok();
            return (int)i;
        }
    // crates/berth-engine/src/device.rs:168-173
    fail(BERTH_CKPT_ARGUMENT, std::string(prefix) + " is not an EXL3 linear", prefix);
    return -1;
}
size_t berth_ckpt_other_count(const berth_ckpt* ckpt) { return ckpt ? ckpt->ckpt.other_tensors().size() : 0; }
int berth_ckpt_other_at(const berth_ckpt* ckpt, size_t i, berth_ckpt_tensor* out)
{
    if (!ckpt || !out || i >= ckpt->ckpt.other_tensors().size())
        return fail(BERTH_CKPT_ARGUMENT, "berth_ckpt_other_at: out of range");
    view(ckpt->ckpt.other_tensors()[i], out);
    return ok();
}

int berth_ckpt_linear_unpack_signs(const berth_ckpt* ckpt, size_t linear, int output_side, uint16_t* out,
                                   size_t capacity, size_t* written)
{
    if (!ckpt || linear >= ckpt->ckpt.linears().size() || !written)
        return fail(BERTH_CKPT_ARGUMENT, "berth_ckpt_linear_unpack_signs: bad argument");
    return guarded([&] {
        const LinearExl3& l = ckpt->ckpt.linears()[linear];
        const std::vector<uint16_t> signs = output_side ? l.unpack_output_signs() : l.unpack_input_signs();
        *written = signs.size();
        if (out && capacity >= signs.size()) std::copy(signs.begin(), signs.end(), out);
    });
}

int berth_ckpt_unpack_signs(const uint8_t* packed_le, size_t nbytes, uint16_t* out)
{
    if ((!packed_le && nbytes) || (!out && nbytes >= 2))
        return fail(BERTH_CKPT_ARGUMENT, "berth_ckpt_unpack_signs: null argument");
    return guarded([&] {
        const std::vector<uint16_t> signs = unpack_signs(packed_le, nbytes);
        std::copy(signs.begin(), signs.end(), out);
    });
}

int berth_ckpt_read_tensor(const berth_ckpt_tensor* tensor, void* dst, size_t capacity)
{
    if (!tensor || !tensor->shard || (!dst && tensor->length))
        return fail(BERTH_CKPT_ARGUMENT, "berth_ckpt_read_tensor: null argument");
    if (capacity < tensor->length)
        return fail(BERTH_CKPT_ARGUMENT, std::string(tensor->name ? tensor->name : "tensor") + ": buffer too small");
    return guarded([&] {
        const std::string path = tensor->shard;
        detail::Fd f(path);
        if (f.fd < 0) throw Error::read(path, errno);
        if (tensor->length) detail::read_exact_at(path, f.fd, tensor->offset, dst, (size_t)tensor->length);
    });
}

}  // extern "C"
