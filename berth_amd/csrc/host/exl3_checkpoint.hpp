// EXL3 checkpoint reader: config.json, the safetensors shard headers and one
// LinearExl3 record per quantized linear (trellis, Hadamard scales suh/svh or
// packed su/sv, optional bias, codebook marker, bit rate).  Tensor bodies stay on
// disk; only packed sign words are read, and only on request.
//
// Same records, checks, error kinds and messages as the reference's reader crate:
//   dtype names and sizes          crates/berth-exl3/src/dtype.rs:6-85
//   error kinds and their text     crates/berth-exl3/src/error.rs:5-31
//   shard header parsing           crates/berth-exl3/src/safetensors.rs:79-257
//   config.json                    crates/berth-exl3/src/config.rs:102-419
//   linears, bit rates, signs      crates/berth-exl3/src/linear.rs:139-361, signs.rs:25-46
//   directory layout, shard index  crates/berth-exl3/src/checkpoint.rs:38-208
// Header-only C++17; the C interface over it is exl3_reader_capi.cpp.
#pragma once

#include "json.hpp"

#include <algorithm>
#include <cerrno>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <optional>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

namespace berth::exl3 {

// ---- errors (error.rs:5-31)
class Error : public std::runtime_error {
public:
    enum class Kind : int { MissingField = 1, BadField = 2, Read = 3, Parse = 4 };
    Kind kind;
    std::string field;   // MissingField / BadField: the config key or tensor name
    std::string path;    // Read / Parse: the file

    static Error missing(const std::string& field)
    {
        return Error(Kind::MissingField, "missing field `" + field + "`", field, "");
    }
    static Error bad(const std::string& field, const std::string& detail)
    {
        return Error(Kind::BadField, "field `" + field + "`: " + detail, field, "");
    }
    static Error read(const std::string& path, int err)
    {
        return Error(Kind::Read, path + ": " + std::strerror(err) + " (os error " + std::to_string(err) + ")", "", path);
    }
    static Error short_read(const std::string& path)
    {
        return Error(Kind::Read, path + ": failed to fill whole buffer", "", path);
    }
    static Error parse(const std::string& path, const std::string& why)
    {
        return Error(Kind::Parse, path + ": " + why, "", path);
    }

private:
    Error(Kind k, const std::string& what, std::string f, std::string p)
        : std::runtime_error(what), kind(k), field(std::move(f)), path(std::move(p)) {}
};

// ---- dtypes (dtype.rs:6-85)
enum class DType : int { Bool, U8, I8, I16, U16, I32, U32, I64, U64, F16, Bf16, F32, F64, F8E4M3, F8E5M2, F8E8M0 };

inline const char* dtype_name(DType d)
{
    static const char* names[] = {"BOOL", "U8", "I8", "I16", "U16", "I32", "U32", "I64", "U64", "F16", "BF16",
                                  "F32", "F64", "F8_E4M3", "F8_E5M2", "F8_E8M0"};
    return names[(int)d];
}
inline bool dtype_parse(const std::string& name, DType* out)
{
    for (int i = 0; i < 16; ++i)
        if (name == dtype_name((DType)i)) { *out = (DType)i; return true; }
    return false;
}
inline uint64_t dtype_size(DType d)
{
    switch (d) {
    case DType::Bool: case DType::U8: case DType::I8: case DType::F8E4M3: case DType::F8E5M2: case DType::F8E8M0: return 1;
    case DType::I16: case DType::U16: case DType::F16: case DType::Bf16: return 2;
    case DType::I32: case DType::U32: case DType::F32: return 4;
    default: return 8;
    }
}

// ---- one tensor, located but not loaded (safetensors.rs:14-33)
struct TensorInfo {
    std::string name;
    std::string shard;             // file that holds the bytes
    DType dtype = DType::U8;
    std::vector<uint64_t> shape;   // empty = scalar (one element)
    uint64_t offset = 0;           // absolute offset of the first byte in `shard`
    uint64_t length = 0;           // byte length of the body
    bool operator==(const TensorInfo& o) const
    {
        return name == o.name && shard == o.shard && dtype == o.dtype && shape == o.shape && offset == o.offset &&
               length == o.length;
    }
};

// every tensor of the checkpoint, sorted by name (safetensors.rs:35-78)
class TensorIndex {
public:
    const TensorInfo* get(const std::string& name) const
    {
        auto it = by_name_.find(name);
        return it == by_name_.end() ? nullptr : &it->second;
    }
    bool contains(const std::string& name) const { return by_name_.count(name) != 0; }
    size_t len() const { return by_name_.size(); }
    bool is_empty() const { return by_name_.empty(); }
    auto begin() const { return by_name_.begin(); }
    auto end() const { return by_name_.end(); }
    void insert(TensorInfo info)
    {
        const std::string name = info.name;
        if (!by_name_.emplace(name, std::move(info)).second) throw Error::bad(name, "tensor name appears more than once");
    }

private:
    std::map<std::string, TensorInfo> by_name_;
};

namespace detail {

constexpr uint64_t kMaxHeaderBytes = 64ull << 20;        // safetensors.rs:11-12
constexpr uint64_t kMaxConfigBytes = 32ull << 20;        // checkpoint.rs:11-12
constexpr uint64_t kMaxPackedSignBytes = 64ull << 20;    // linear.rs:8-10

inline bool mul_overflows(uint64_t a, uint64_t b, uint64_t* out) { return __builtin_mul_overflow(a, b, out); }
inline bool add_overflows(uint64_t a, uint64_t b, uint64_t* out) { return __builtin_add_overflow(a, b, out); }

inline const char* json_kind(const json::Value& v)      // safetensors.rs:247-256
{
    switch (v.kind) {
    case json::Value::Kind::Null: return "null";
    case json::Value::Kind::Bool: return "a bool";
    case json::Value::Kind::Number: return "a number";
    case json::Value::Kind::String: return "a string";
    case json::Value::Kind::Array: return "an array";
    default: return "an object";
    }
}

inline std::string quoted(const std::string& s)          // Rust's {:?} of a str, for the common cases
{
    std::string out = "\"";
    for (unsigned char c : s) {
        if (c == '"') out += "\\\"";
        else if (c == '\\') out += "\\\\";
        else if (c == '\n') out += "\\n";
        else if (c == '\r') out += "\\r";
        else if (c == '\t') out += "\\t";
        else out += (char)c;
    }
    return out + "\"";
}

inline std::string describe(const json::Value& v)        // config.rs:408-418
{
    switch (v.kind) {
    case json::Value::Kind::Null: return "null";
    case json::Value::Kind::Bool: return v.boolean ? "true" : "false";
    case json::Value::Kind::Number: return v.number_text();
    case json::Value::Kind::String: return v.text.size() < 64 ? "string " + quoted(v.text) : "a long string";
    case json::Value::Kind::Array: return "an array";
    default: return "an object";
    }
}

struct Fd {
    int fd = -1;
    explicit Fd(const std::string& path) { fd = ::open(path.c_str(), O_RDONLY | O_CLOEXEC); }
    ~Fd() { if (fd >= 0) ::close(fd); }
    Fd(const Fd&) = delete;
    Fd& operator=(const Fd&) = delete;
};

// exactly `len` bytes at `offset`
inline void read_exact_at(const std::string& path, int fd, uint64_t offset, void* dst, size_t len)
{
    char* p = (char*)dst;
    while (len) {
        const ssize_t got = ::pread(fd, p, len, (off_t)offset);
        if (got < 0) {
            if (errno == EINTR) continue;
            throw Error::read(path, errno);
        }
        if (got == 0) throw Error::short_read(path);
        p += got;
        offset += (uint64_t)got;
        len -= (size_t)got;
    }
}

inline std::string read_file(const std::string& path)
{
    Fd f(path);
    if (f.fd < 0) throw Error::read(path, errno);
    struct stat st;
    if (::fstat(f.fd, &st) != 0) throw Error::read(path, errno);
    if (S_ISDIR(st.st_mode)) throw Error::read(path, EISDIR);
    std::string out((size_t)st.st_size, '\0');
    if (!out.empty()) read_exact_at(path, f.fd, 0, out.data(), out.size());
    return out;
}

inline bool is_dir(const std::string& p)
{
    struct stat st;
    return ::stat(p.c_str(), &st) == 0 && S_ISDIR(st.st_mode);
}
inline bool is_file(const std::string& p)
{
    struct stat st;
    return ::stat(p.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}
inline std::string join(const std::string& dir, const std::string& rel)
{
    if (dir.empty()) return rel;
    return dir.back() == '/' ? dir + rel : dir + "/" + rel;
}

inline uint64_t expect_u64(const std::string& field, const json::Value& v)    // safetensors.rs:238-245
{
    uint64_t x;
    if (!v.as_u64(&x)) throw Error::bad(field, std::string("expected an integer, got ") + json_kind(v));
    return x;
}

}  // namespace detail

// ---- shard headers (safetensors.rs:79-236)
inline TensorInfo parse_tensor(const std::string& path, const std::string& name, const json::Value& entry,
                               uint64_t data_start, uint64_t file_len)
{
    using namespace detail;
    if (!entry.is_object())
        throw Error::bad(name, std::string("expected a tensor object, got ") + json_kind(entry));
    const json::Value* dtype_value = entry.get("dtype");
    if (!dtype_value) throw Error::bad(name + ".dtype", "missing dtype");
    if (!dtype_value->is_string()) throw Error::bad(name + ".dtype", "expected a string");
    DType dtype;
    if (!dtype_parse(dtype_value->text, &dtype))
        throw Error::bad(name + ".dtype", "unknown safetensors dtype `" + dtype_value->text + "`");
    const json::Value* shape_value = entry.get("shape");
    if (!shape_value) throw Error::bad(name + ".shape", "missing shape");
    if (!shape_value->is_array())
        throw Error::bad(name + ".shape", std::string("expected an array, got ") + json_kind(*shape_value));
    std::vector<uint64_t> shape;
    for (const auto& dim : shape_value->items) shape.push_back(expect_u64(name + ".shape", *dim));
    const json::Value* offsets = entry.get("data_offsets");
    const std::string off_field = name + ".data_offsets";
    if (!offsets) throw Error::bad(off_field, "missing data_offsets");
    if (!offsets->is_array()) throw Error::bad(off_field, std::string("expected an array, got ") + json_kind(*offsets));
    if (offsets->items.size() != 2)
        throw Error::bad(off_field, "expected 2 offsets, got " + std::to_string(offsets->items.size()));
    const uint64_t start = expect_u64(off_field, *offsets->items[0]);
    const uint64_t end = expect_u64(off_field, *offsets->items[1]);
    if (end < start)
        throw Error::bad(off_field, "end " + std::to_string(end) + " is before start " + std::to_string(start));
    const uint64_t span = end - start;
    uint64_t numel = 1;
    for (uint64_t dim : shape)
        if (mul_overflows(numel, dim, &numel)) throw Error::bad(name, "shape product overflows u64");
    uint64_t nbytes;
    if (mul_overflows(numel, dtype_size(dtype), &nbytes)) throw Error::bad(name, "byte length overflows u64");
    if (span != nbytes)
        throw Error::bad(name, "data_offsets span " + std::to_string(span) + " does not match " + dtype_name(dtype) +
                                   " shape byte length " + std::to_string(nbytes));
    uint64_t offset, end_abs;
    if (add_overflows(data_start, start, &offset)) throw Error::bad(name, "byte offset overflows u64");
    if (add_overflows(offset, span, &end_abs)) throw Error::bad(name, "tensor end overflows u64");
    if (end_abs > file_len)
        throw Error::bad(name, "tensor extends to byte " + std::to_string(end_abs) + " but the shard is " +
                                   std::to_string(file_len) + " bytes");
    TensorInfo info;
    info.name = name;
    info.shard = path;
    info.dtype = dtype;
    info.shape = std::move(shape);
    info.offset = offset;
    info.length = span;
    return info;
}

// one shard's header; tensor bodies are not read.  Records come back in name order.
inline std::vector<TensorInfo> read_shard(const std::string& path)
{
    using namespace detail;
    Fd f(path);
    if (f.fd < 0) throw Error::read(path, errno);
    struct stat st;
    if (::fstat(f.fd, &st) != 0) throw Error::read(path, errno);
    const uint64_t file_len = (uint64_t)st.st_size;
    unsigned char len_buf[8];
    read_exact_at(path, f.fd, 0, len_buf, 8);
    uint64_t header_len = 0;
    for (int i = 7; i >= 0; --i) header_len = (header_len << 8) | len_buf[i];
    if (header_len > kMaxHeaderBytes || header_len > (file_len >= 8 ? file_len - 8 : 0))
        throw Error::bad(path, "safetensors header length " + std::to_string(header_len) + " is not usable in a " +
                                   std::to_string(file_len) + "-byte file");
    std::string header((size_t)header_len, '\0');
    if (header_len) read_exact_at(path, f.fd, 8, header.data(), header.size());
    json::Value value;
    try {
        value = json::parse(header);
    } catch (const json::ParseError& e) {
        throw Error::parse(path, e.what());
    }
    if (!value.is_object()) throw Error::bad(path, "safetensors header is not a JSON object");
    const uint64_t data_start = 8 + header_len;
    std::vector<TensorInfo> tensors;
    for (const auto& [name, entry] : value.members) {
        if (name == "__metadata__") continue;
        tensors.push_back(parse_tensor(path, name, *entry, data_start, file_len));
    }
    return tensors;
}

// ---- config.json (config.rs:5-419)
struct LayerType {
    enum class Kind : int { LinearAttention = 0, FullAttention = 1, Other = 2 };
    Kind kind = Kind::Other;
    std::string name;    // the string as written
    bool operator==(const LayerType& o) const { return kind == o.kind && (kind != Kind::Other || name == o.name); }
};

struct Calibration {
    uint32_t rows = 0, cols = 0;
};

struct QuantizationConfig {
    std::string quant_method;
    double bits = 0.0;
    uint32_t head_bits = 0;
    std::optional<std::string> codebook, version, out_scales;
    std::optional<uint32_t> vision_bits, mtp_bits;
    std::optional<Calibration> calibration;
};

struct ModelConfig {
    std::string arch_string;
    uint32_t num_hidden_layers = 0, hidden_size = 0;
    std::optional<uint32_t> intermediate_size;
    uint32_t head_dim = 0, num_attention_heads = 0, num_key_value_heads = 0, vocab_size = 0;
    bool tie_word_embeddings = false;
    std::vector<LayerType> layer_types;
    uint32_t linear_conv_kernel_dim = 0, linear_num_key_heads = 0, linear_num_value_heads = 0;
    uint32_t linear_key_head_dim = 0, linear_value_head_dim = 0;
    bool attn_output_gate = false;
    std::optional<uint32_t> num_experts, num_experts_per_tok, moe_intermediate_size, shared_expert_intermediate_size;
    QuantizationConfig quantization;

    static ModelConfig from_slice(const char* bytes, size_t len)
    {
        json::Value value;
        try {
            value = json::parse(bytes, len);
        } catch (const json::ParseError& e) {
            throw Error::parse("config.json", e.what());
        }
        return from_value(value);
    }

    // text fields come from `text_config` when that object has the key, else from the top level
    static ModelConfig from_value(const json::Value& value)
    {
        using detail::describe;
        if (!value.is_object()) throw Error::bad("config.json", "expected a JSON object");
        const json::Value* text = value.get("text_config");
        if (text && !text->is_object())
            throw Error::bad("text_config", "expected an object, got " + describe(*text));

        auto lookup = [&](const char* key) -> const json::Value* {
            if (text)
                if (const json::Value* v = text->get(key)) return v;
            return value.get(key);
        };
        auto require = [&](const char* key) -> const json::Value& {
            const json::Value* v = lookup(key);
            if (!v) throw Error::missing(key);
            return *v;
        };
        auto require_u32 = [&](const char* key) { return expect_u32(require(key), key); };
        auto optional_u32 = [&](const char* key) -> std::optional<uint32_t> {
            const json::Value* v = lookup(key);
            if (!v) return std::nullopt;
            return expect_u32(*v, key);
        };
        auto require_bool = [&](const char* key) {
            const json::Value& v = require(key);
            if (!v.is_bool()) throw Error::bad(key, "expected a bool, got " + describe(v));
            return v.boolean;
        };

        ModelConfig cfg;
        cfg.arch_string = arch(value);
        cfg.num_hidden_layers = require_u32("num_hidden_layers");
        cfg.layer_types = parse_layer_types(require("layer_types"));
        if (cfg.layer_types.size() != cfg.num_hidden_layers)
            throw Error::bad("layer_types", "length " + std::to_string(cfg.layer_types.size()) +
                                                " does not match num_hidden_layers " +
                                                std::to_string(cfg.num_hidden_layers));
        const json::Value* quant = value.get("quantization_config");
        if (!quant) throw Error::missing("quantization_config");
        cfg.hidden_size = require_u32("hidden_size");
        cfg.intermediate_size = optional_u32("intermediate_size");
        cfg.head_dim = require_u32("head_dim");
        cfg.num_attention_heads = require_u32("num_attention_heads");
        cfg.num_key_value_heads = require_u32("num_key_value_heads");
        cfg.vocab_size = require_u32("vocab_size");
        cfg.tie_word_embeddings = require_bool("tie_word_embeddings");
        cfg.linear_conv_kernel_dim = require_u32("linear_conv_kernel_dim");
        cfg.linear_num_key_heads = require_u32("linear_num_key_heads");
        cfg.linear_num_value_heads = require_u32("linear_num_value_heads");
        cfg.linear_key_head_dim = require_u32("linear_key_head_dim");
        cfg.linear_value_head_dim = require_u32("linear_value_head_dim");
        cfg.attn_output_gate = require_bool("attn_output_gate");
        cfg.num_experts = optional_u32("num_experts");
        cfg.num_experts_per_tok = optional_u32("num_experts_per_tok");
        cfg.moe_intermediate_size = optional_u32("moe_intermediate_size");
        cfg.shared_expert_intermediate_size = optional_u32("shared_expert_intermediate_size");
        cfg.quantization = parse_quant(*quant);
        return cfg;
    }

private:
    // integers, or floats that are exactly an integer ("6.0"): config writers emit both
    static uint32_t expect_u32(const json::Value& v, const std::string& field)
    {
        uint64_t n;
        if (v.as_u64(&n)) {
            if (n > 0xFFFFFFFFull) throw Error::bad(field, "integer " + std::to_string(n) + " does not fit in u32");
            return (uint32_t)n;
        }
        double d;
        if (v.as_f64(&d) && std::isfinite(d) && d >= 0.0 && d == std::floor(d) && d <= 4294967295.0) return (uint32_t)d;
        throw Error::bad(field, "expected a non-negative integer, got " + detail::describe(v));
    }
    static std::string expect_string(const json::Value& v, const std::string& field)
    {
        if (!v.is_string()) throw Error::bad(field, "expected a string, got " + detail::describe(v));
        return v.text;
    }
    static std::string arch(const json::Value& root)
    {
        using detail::describe;
        const json::Value* v = root.get("architectures");
        if (!v) throw Error::missing("architectures");
        if (!v->is_array()) throw Error::bad("architectures", "expected an array, got " + describe(*v));
        if (v->items.empty()) throw Error::bad("architectures", "expected a non-empty array");
        const json::Value& first = *v->items[0];
        if (!first.is_string()) throw Error::bad("architectures", "expected a string, got " + describe(first));
        if (first.text.empty()) throw Error::bad("architectures", "architecture string is empty");
        return first.text;
    }
    static std::vector<LayerType> parse_layer_types(const json::Value& v)
    {
        using detail::describe;
        if (!v.is_array()) throw Error::bad("layer_types", "expected an array, got " + describe(v));
        std::vector<LayerType> out;
        for (const auto& item : v.items) {
            if (!item->is_string()) throw Error::bad("layer_types", "expected strings, got " + describe(*item));
            LayerType t;
            t.name = item->text;
            t.kind = t.name == "linear_attention" ? LayerType::Kind::LinearAttention
                     : t.name == "full_attention" ? LayerType::Kind::FullAttention
                                                  : LayerType::Kind::Other;
            out.push_back(std::move(t));
        }
        return out;
    }
    static QuantizationConfig parse_quant(const json::Value& v)
    {
        using detail::describe;
        if (!v.is_object()) throw Error::bad("quantization_config", "expected an object, got " + describe(v));
        QuantizationConfig q;
        if (const json::Value* raw = v.get("calibration")) {
            if (!raw->is_object()) throw Error::bad("calibration", "expected an object, got " + describe(*raw));
            Calibration c;
            const json::Value* rows = raw->get("rows");
            if (!rows) throw Error::missing("calibration.rows");
            c.rows = expect_u32(*rows, "calibration.rows");
            const json::Value* cols = raw->get("cols");
            if (!cols) throw Error::missing("calibration.cols");
            c.cols = expect_u32(*cols, "calibration.cols");
            q.calibration = c;
        }
        auto req = [&](const char* key) -> const json::Value& {
            const json::Value* x = v.get(key);
            if (!x) throw Error::missing(key);
            return *x;
        };
        auto opt_string = [&](const char* key) -> std::optional<std::string> {
            const json::Value* x = v.get(key);
            if (!x) return std::nullopt;
            return expect_string(*x, key);
        };
        auto opt_u32 = [&](const char* key) -> std::optional<uint32_t> {
            const json::Value* x = v.get(key);
            if (!x) return std::nullopt;
            return expect_u32(*x, key);
        };
        q.quant_method = expect_string(req("quant_method"), "quant_method");
        const json::Value& bits = req("bits");
        double number;
        if (!bits.as_f64(&number)) throw Error::bad("bits", "expected a number, got " + describe(bits));
        if (!std::isfinite(number) || number < 0.0)
            throw Error::bad("bits", "expected a non-negative finite number, got " + bits.number_text());
        q.bits = number;
        q.head_bits = expect_u32(req("head_bits"), "head_bits");
        q.codebook = opt_string("codebook");
        q.version = opt_string("version");
        q.vision_bits = opt_u32("vision_bits");
        q.mtp_bits = opt_u32("mtp_bits");
        q.out_scales = opt_string("out_scales");
        return q;
    }
};

// ---- packed signs (signs.rs:3-46)
constexpr uint16_t kFp16One = 0x3C00;
constexpr uint16_t kFp16NegOne = 0xBC00;

// bit 0 of each little-endian 16-bit word is the first sign; a set bit is -1
inline std::vector<uint16_t> unpack_signs(const uint8_t* packed_le, size_t nbytes)
{
    if (nbytes % 2 != 0)
        throw Error::bad("su", "packed sign bytes " + std::to_string(nbytes) + " are not a multiple of 2");
    std::vector<uint16_t> out;
    out.reserve(nbytes * 8);
    for (size_t w = 0; w < nbytes / 2; ++w) {
        const unsigned word = (unsigned)packed_le[2 * w] | ((unsigned)packed_le[2 * w + 1] << 8);
        for (int bit = 0; bit < 16; ++bit) out.push_back(((word >> bit) & 1u) ? kFp16NegOne : kFp16One);
    }
    return out;
}

// ---- linears (linear.rs:12-361)
enum class Codebook : int { Mcg = 0, Mul1 = 1, Default = 2 };

// bits per weight from trellis.shape[-1]: 16*K words, or 16*floor(K)+8 for K = 1.5, 2.5, 3.5
struct Bitrate {
    int twice = 0;                                    // 2 * K, so that half rates stay integral
    bool is_half() const { return (twice & 1) != 0; }
    int whole() const { return twice / 2; }           // K for an integer rate
    double as_f64() const { return twice / 2.0; }
    std::string to_string() const { return is_half() ? std::to_string(twice / 2) + ".5" : std::to_string(twice / 2); }
    bool operator==(const Bitrate& o) const { return twice == o.twice; }
};

struct HadamardScale {
    bool packed = false;    // true: I16 sign words (su / sv); false: fp16 vector (suh / svh)
    TensorInfo tensor;
    bool is_packed() const { return packed; }
};

struct LinearExl3 {
    std::string prefix;                 // tensor prefix without ".trellis"
    TensorInfo trellis;                 // I16, rank 3
    HadamardScale input_scale, output_scale;
    std::optional<TensorInfo> bias;     // F16, BF16 or F32, as stored
    Codebook codebook = Codebook::Default;
    Bitrate k;

    std::vector<uint16_t> unpack_input_signs() const { return unpack_scale(input_scale, "su", "suh"); }
    std::vector<uint16_t> unpack_output_signs() const { return unpack_scale(output_scale, "sv", "svh"); }

private:
    static std::vector<uint16_t> unpack_scale(const HadamardScale& scale, const char* packed, const char* unpacked)
    {
        const TensorInfo& info = scale.tensor;
        if (!scale.packed)
            throw Error::bad(info.name, std::string("scale is unpacked `") + unpacked + "` fp16, not packed `" + packed + "`");
        if (info.dtype != DType::I16) throw Error::bad(info.name, std::string("expected I16, got ") + dtype_name(info.dtype));
        if (info.length > detail::kMaxPackedSignBytes)
            throw Error::bad(info.name, "refusing to read " + std::to_string(info.length) +
                                            " bytes; packed sign reads are capped at " +
                                            std::to_string(detail::kMaxPackedSignBytes));
        detail::Fd f(info.shard);
        if (f.fd < 0) throw Error::read(info.shard, errno);
        std::vector<uint8_t> bytes((size_t)info.length);
        if (!bytes.empty()) detail::read_exact_at(info.shard, f.fd, info.offset, bytes.data(), bytes.size());
        return unpack_signs(bytes.data(), bytes.size());
    }
};

inline Bitrate bitrate(const std::string& tensor, uint64_t last, Codebook codebook)     // linear.rs:295-330
{
    const std::string l = std::to_string(last);
    if (last % 16 == 0) {
        const uint64_t k = last / 16;
        if (k >= 1 && k <= 8) return Bitrate{(int)(2 * k)};
        throw Error::bad(tensor, "integer bitrate " + std::to_string(k) + " is outside 1..=8 (last dim " + l + ")");
    }
    if (last % 16 == 8) {
        const uint64_t floor = last / 16;
        if (floor < 1 || floor > 3)
            throw Error::bad(tensor, "half-integer bitrate " + std::to_string(floor) +
                                         ".5 is not one of 1.5, 2.5, 3.5 (last dim " + l + ")");
        const Bitrate half{(int)(2 * floor + 1)};
        if (codebook != Codebook::Mul1)
            throw Error::bad(tensor, "half-integer bitrate " + half.to_string() + " requires mul1 (last dim " + l + ")");
        return half;
    }
    throw Error::bad(tensor, "last dim " + l + " is not 16*K or 16*K+8");
}

namespace detail {

inline HadamardScale scale_of(const TensorIndex& index, const std::string& prefix, const char* unpacked_suffix,
                              const char* packed_suffix)                                 // linear.rs:243-283
{
    const TensorInfo* unpacked = index.get(prefix + "." + unpacked_suffix);
    const TensorInfo* packed = index.get(prefix + "." + packed_suffix);
    if (unpacked && unpacked->dtype != DType::F16)
        throw Error::bad(unpacked->name, std::string("expected F16, got ") + dtype_name(unpacked->dtype));
    if (packed && packed->dtype != DType::I16)
        throw Error::bad(packed->name, std::string("expected I16, got ") + dtype_name(packed->dtype));
    if (unpacked) return HadamardScale{false, *unpacked};
    if (packed) return HadamardScale{true, *packed};
    throw Error::bad(prefix + "." + unpacked_suffix, std::string("missing ") + unpacked_suffix + " or " + packed_suffix);
}

inline LinearExl3 build_linear(const TensorIndex& index, const std::string& prefix)     // linear.rs:187-241
{
    const TensorInfo* trellis = index.get(prefix + ".trellis");
    if (!trellis) throw Error::bad(prefix + ".trellis", "missing trellis");
    if (trellis->dtype != DType::I16)
        throw Error::bad(trellis->name, std::string("expected I16, got ") + dtype_name(trellis->dtype));
    if (trellis->shape.size() != 3)
        throw Error::bad(trellis->name, "expected rank 3, got rank " + std::to_string(trellis->shape.size()));
    const bool mcg = index.contains(prefix + ".mcg"), mul1 = index.contains(prefix + ".mul1");
    if (mcg && mul1) throw Error::bad(prefix + ".mcg", "both mcg and mul1 are present");
    LinearExl3 lin;
    lin.prefix = prefix;
    lin.trellis = *trellis;
    lin.codebook = mcg ? Codebook::Mcg : mul1 ? Codebook::Mul1 : Codebook::Default;
    lin.k = bitrate(trellis->name, trellis->shape[2], lin.codebook);
    lin.input_scale = scale_of(index, prefix, "suh", "su");
    lin.output_scale = scale_of(index, prefix, "svh", "sv");
    if (const TensorInfo* bias = index.get(prefix + ".bias")) {
        if (bias->dtype != DType::F16 && bias->dtype != DType::Bf16 && bias->dtype != DType::F32)
            throw Error::bad(bias->name, std::string("expected a float bias, got ") + dtype_name(bias->dtype));
        lin.bias = *bias;
    }
    return lin;
}

}  // namespace detail

// linears sorted by prefix, and the tensors that belong to none (linear.rs:153-185)
inline void group_linears(const TensorIndex& index, std::vector<LinearExl3>* linears, std::vector<TensorInfo>* other)
{
    static const char* parts[] = {"trellis", "suh", "svh", "su", "sv", "bias", "mcg", "mul1"};
    const std::string suffix = ".trellis";
    std::set<std::string> consumed;
    for (const auto& [name, info] : index) {
        (void)info;
        if (name.size() < suffix.size() || name.compare(name.size() - suffix.size(), suffix.size(), suffix) != 0) continue;
        const std::string prefix = name.substr(0, name.size() - suffix.size());
        if (prefix.empty()) throw Error::bad(name, "trellis tensor has an empty linear prefix");
        linears->push_back(detail::build_linear(index, prefix));
        for (const char* part : parts) {
            const std::string sibling = prefix + "." + part;
            if (index.contains(sibling)) consumed.insert(sibling);
        }
    }
    std::stable_sort(linears->begin(), linears->end(),
                     [](const LinearExl3& a, const LinearExl3& b) { return a.prefix < b.prefix; });
    for (const auto& [name, info] : index)
        if (!consumed.count(name)) other->push_back(info);
}

// ---- the checkpoint directory (checkpoint.rs:14-208)
class Checkpoint {
public:
    std::string directory;
    ModelConfig config;
    TensorIndex tensors;

    // a sharded model is the shards named by model.safetensors.index.json; an unsharded one is model.safetensors
    static Checkpoint open(const std::string& dir)
    {
        using namespace detail;
        if (!is_dir(dir)) throw Error::bad(dir, "not a checkpoint directory");
        Checkpoint c;
        c.directory = dir;
        c.config = read_config(join(dir, "config.json"));
        std::optional<uint64_t> total_size;
        c.tensors = read_tensors(dir, &total_size);
        if (total_size) {
            uint64_t sum = 0;
            for (const auto& [name, info] : c.tensors) {
                (void)name;
                if (add_overflows(sum, info.length, &sum))
                    throw Error::bad("metadata.total_size", "tensor byte sum overflows u64");
            }
            if (sum != *total_size)
                throw Error::bad("metadata.total_size", "index says " + std::to_string(*total_size) +
                                                            ", tensor bytes sum to " + std::to_string(sum));
        }
        group_linears(c.tensors, &c.linears_, &c.other_);
        return c;
    }

    const std::vector<LinearExl3>& linears() const { return linears_; }          // sorted by prefix
    const std::vector<TensorInfo>& other_tensors() const { return other_; }      // sorted by name
    const LinearExl3* find_linear(const std::string& prefix) const
    {
        for (const LinearExl3& l : linears_)
            if (l.prefix == prefix) return &l;
        return nullptr;
    }

private:
    std::vector<LinearExl3> linears_;
    std::vector<TensorInfo> other_;

    static ModelConfig read_config(const std::string& path)
    {
        struct stat st;
        if (::stat(path.c_str(), &st) != 0) throw Error::read(path, errno);
        if ((uint64_t)st.st_size > detail::kMaxConfigBytes)
            throw Error::bad("config.json", "config is " + std::to_string((uint64_t)st.st_size) + " bytes");
        const std::string bytes = detail::read_file(path);
        json::Value value;
        try {
            value = json::parse(bytes);
        } catch (const json::ParseError& e) {
            throw Error::parse(path, e.what());
        }
        return ModelConfig::from_value(value);
    }

    static TensorIndex read_tensors(const std::string& dir, std::optional<uint64_t>* total_size)
    {
        using namespace detail;
        const std::string index_path = join(dir, "model.safetensors.index.json");
        if (is_file(index_path)) {
            std::map<std::string, std::string> weight_map = read_weight_map(index_path, total_size);
            return read_sharded(dir, weight_map);
        }
        const std::string single = join(dir, "model.safetensors");
        if (is_file(single)) {
            TensorIndex index;
            for (TensorInfo& info : read_shard(single)) index.insert(std::move(info));
            return index;
        }
        throw Error::bad("model.safetensors", "no model.safetensors.index.json and no model.safetensors");
    }

    static std::map<std::string, std::string> read_weight_map(const std::string& path, std::optional<uint64_t>* total_size)
    {
        const std::string bytes = detail::read_file(path);
        json::Value value;
        try {
            value = json::parse(bytes);
        } catch (const json::ParseError& e) {
            throw Error::parse(path, e.what());
        }
        if (!value.is_object()) throw Error::bad("model.safetensors.index.json", "expected a JSON object");
        const json::Value* map = value.get("weight_map");
        if (!map) throw Error::missing("weight_map");
        if (!map->is_object()) throw Error::bad("weight_map", "expected an object");
        std::map<std::string, std::string> weight_map;
        for (const auto& [name, shard] : map->members) {
            if (!shard->is_string()) throw Error::bad("weight_map." + name, "expected a shard filename");
            if (shard->text.empty()) throw Error::bad("weight_map." + name, "empty shard path");
            weight_map[name] = shard->text;
        }
        if (const json::Value* meta = value.get("metadata")) {
            if (!meta->is_object()) throw Error::bad("metadata", "expected an object");
            if (const json::Value* total = meta->get("total_size")) {
                uint64_t n;
                if (!total->as_u64(&n)) throw Error::bad("metadata.total_size", "expected an integer");
                *total_size = n;
            }
        }
        return weight_map;
    }

    // a shard path must stay inside the checkpoint directory
    static std::string shard_path(const std::string& dir, const std::string& rel)
    {
        bool escapes = !rel.empty() && rel[0] == '/';
        size_t start = 0;
        while (!escapes && start <= rel.size()) {
            const size_t slash = rel.find('/', start);
            const std::string part = rel.substr(start, slash == std::string::npos ? std::string::npos : slash - start);
            if (part == "..") escapes = true;
            if (slash == std::string::npos) break;
            start = slash + 1;
        }
        if (escapes)
            throw Error::bad("weight_map", "shard `" + rel + "` is not a path inside the checkpoint directory");
        return detail::join(dir, rel);
    }

    static TensorIndex read_sharded(const std::string& dir, const std::map<std::string, std::string>& weight_map)
    {
        std::map<std::string, std::set<std::string>> by_shard;
        for (const auto& [name, shard] : weight_map) by_shard[shard_path(dir, shard)].insert(name);
        TensorIndex index;
        for (const auto& [path, expected] : by_shard) {
            std::set<std::string> saw;
            for (TensorInfo& info : read_shard(path)) {
                if (!expected.count(info.name))
                    throw Error::bad(info.name, "present in " + path + " but not in model.safetensors.index.json");
                if (!saw.insert(info.name).second) throw Error::bad(info.name, "duplicated inside one shard header");
                index.insert(std::move(info));
            }
            for (const std::string& name : expected)
                if (!saw.count(name))
                    throw Error::bad(name, "weight_map lists it in " + path + " but the shard header does not");
        }
        return index;
    }
};

// one tensor's bytes from its shard (crates/berth-engine/src/device.rs:49-63)
inline std::vector<uint8_t> read_tensor(const TensorInfo& info)
{
    detail::Fd f(info.shard);
    if (f.fd < 0) throw Error::read(info.shard, errno);
    std::vector<uint8_t> bytes((size_t)info.length);
    if (!bytes.empty()) detail::read_exact_at(info.shard, f.fd, info.offset, bytes.data(), bytes.size());
    return bytes;
}

}  // namespace berth::exl3
