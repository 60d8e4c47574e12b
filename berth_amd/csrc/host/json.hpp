// A small JSON reader for checkpoint metadata (config.json, the shard index and
// safetensors headers).  It keeps what the checkpoint reader relies on in the
// reference's JSON library (serde_json as used by crates/berth-exl3):
//   * object members iterate in key order, a repeated key keeps the last value;
//   * a number is an unsigned integer, a negative integer or a float, decided by
//     its spelling ("6" is an integer, "6.0" and "6e0" are floats), and integers
//     that do not fit 64 bits become floats;
//   * strings must be valid UTF-8;
//   * nesting is limited to 128 levels;
//   * errors carry "<reason> at line L column C".
// Header-only, no dependencies beyond the standard library.
#pragma once

#include <cerrno>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace berth::json {

struct ParseError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

class Value;
using Object = std::map<std::string, std::shared_ptr<Value>>;
using Array = std::vector<std::shared_ptr<Value>>;

class Value {
public:
    enum class Kind { Null, Bool, Number, String, Array, Object };
    enum class Num { Unsigned, Negative, Float };

    Kind kind = Kind::Null;
    bool boolean = false;
    Num num = Num::Float;
    uint64_t u = 0;      // Num::Unsigned
    int64_t i = 0;       // Num::Negative
    double f = 0.0;      // every number, as a double
    std::string text;    // Kind::String
    Array items;         // Kind::Array
    Object members;      // Kind::Object

    bool is_object() const { return kind == Kind::Object; }
    bool is_array() const { return kind == Kind::Array; }
    bool is_string() const { return kind == Kind::String; }
    bool is_bool() const { return kind == Kind::Bool; }
    // true only for a number spelled as a non-negative integer that fits 64 bits
    bool as_u64(uint64_t* out) const
    {
        if (kind != Kind::Number || num != Num::Unsigned) return false;
        *out = u;
        return true;
    }
    bool as_f64(double* out) const
    {
        if (kind != Kind::Number) return false;
        *out = f;
        return true;
    }
    const Value* get(const std::string& key) const
    {
        if (kind != Kind::Object) return nullptr;
        auto it = members.find(key);
        return it == members.end() ? nullptr : it->second.get();
    }
    // how a number reads when echoed in a message: integers as written, floats in the
    // shortest form that reads back to the same double, always with a fraction or exponent
    std::string number_text() const
    {
        if (num == Num::Unsigned) return std::to_string(u);
        if (num == Num::Negative) return std::to_string(i);
        char buf[40];
        for (int prec = 1; prec <= 17; ++prec) {
            std::snprintf(buf, sizeof buf, "%.*g", prec, f);
            if (std::strtod(buf, nullptr) == f) break;
        }
        std::string s(buf);
        if (s.find_first_of(".en") == std::string::npos) s += ".0";
        return s;
    }
};

class Parser {
public:
    Parser(const char* data, size_t len) : p_(data), end_(data + len), begin_(data) {}

    Value parse_document()
    {
        Value v = parse_value(0);
        skip_ws();
        if (p_ != end_) fail("trailing characters");
        return v;
    }

private:
    const char* p_;
    const char* end_;
    const char* begin_;

    [[noreturn]] void fail(const std::string& why) const
    {
        size_t line = 1, col = 0;
        for (const char* q = begin_; q < p_ && q < end_; ++q) {
            if (*q == '\n') { ++line; col = 0; }
            else ++col;
        }
        throw ParseError(why + " at line " + std::to_string(line) + " column " + std::to_string(col));
    }
    void skip_ws()
    {
        while (p_ < end_ && (*p_ == ' ' || *p_ == '\t' || *p_ == '\n' || *p_ == '\r')) ++p_;
    }
    bool literal(const char* word)
    {
        const char* q = p_;
        for (const char* w = word; *w; ++w, ++q)
            if (q >= end_ || *q != *w) return false;
        p_ = q;
        return true;
    }

    Value parse_value(int depth)
    {
        if (depth > 128) fail("recursion limit exceeded");
        skip_ws();
        if (p_ == end_) fail("EOF while parsing a value");
        Value v;
        switch (*p_) {
        case 'n':
            if (!literal("null")) { ++p_; fail("expected ident"); }
            return v;
        case 't':
            if (!literal("true")) { ++p_; fail("expected ident"); }
            v.kind = Value::Kind::Bool; v.boolean = true;
            return v;
        case 'f':
            if (!literal("false")) { ++p_; fail("expected ident"); }
            v.kind = Value::Kind::Bool; v.boolean = false;
            return v;
        case '"':
            v.kind = Value::Kind::String;
            v.text = parse_string();
            return v;
        case '[': {
            ++p_;
            v.kind = Value::Kind::Array;
            skip_ws();
            if (p_ < end_ && *p_ == ']') { ++p_; return v; }
            for (;;) {
                v.items.push_back(std::make_shared<Value>(parse_value(depth + 1)));
                skip_ws();
                if (p_ == end_) fail("EOF while parsing a list");
                if (*p_ == ',') { ++p_; skip_ws(); if (p_ < end_ && *p_ == ']') fail("trailing comma"); continue; }
                if (*p_ == ']') { ++p_; return v; }
                fail("expected `,` or `]`");
            }
        }
        case '{': {
            ++p_;
            v.kind = Value::Kind::Object;
            skip_ws();
            if (p_ < end_ && *p_ == '}') { ++p_; return v; }
            for (;;) {
                skip_ws();
                if (p_ == end_) fail("EOF while parsing an object");
                if (*p_ != '"') fail("key must be a string");
                std::string key = parse_string();
                skip_ws();
                if (p_ == end_) fail("EOF while parsing an object");
                if (*p_ != ':') fail("expected `:`");
                ++p_;
                v.members[key] = std::make_shared<Value>(parse_value(depth + 1));
                skip_ws();
                if (p_ == end_) fail("EOF while parsing an object");
                if (*p_ == ',') { ++p_; skip_ws(); if (p_ < end_ && *p_ == '}') fail("trailing comma"); continue; }
                if (*p_ == '}') { ++p_; return v; }
                fail("expected `,` or `}`");
            }
        }
        default:
            if (*p_ == '-' || (*p_ >= '0' && *p_ <= '9')) return parse_number();
            ++p_;
            fail("expected value");
        }
    }

    static void put_utf8(std::string& out, uint32_t cp)
    {
        if (cp < 0x80) out += (char)cp;
        else if (cp < 0x800) { out += (char)(0xC0 | (cp >> 6)); out += (char)(0x80 | (cp & 0x3F)); }
        else if (cp < 0x10000) {
            out += (char)(0xE0 | (cp >> 12)); out += (char)(0x80 | ((cp >> 6) & 0x3F)); out += (char)(0x80 | (cp & 0x3F));
        } else {
            out += (char)(0xF0 | (cp >> 18)); out += (char)(0x80 | ((cp >> 12) & 0x3F));
            out += (char)(0x80 | ((cp >> 6) & 0x3F)); out += (char)(0x80 | (cp & 0x3F));
        }
    }
    uint32_t hex4()
    {
        if (end_ - p_ < 4) { p_ = end_; fail("EOF while parsing a string"); }
        uint32_t v = 0;
        for (int k = 0; k < 4; ++k, ++p_) {
            const char c = *p_;
            v <<= 4;
            if (c >= '0' && c <= '9') v |= (uint32_t)(c - '0');
            else if (c >= 'a' && c <= 'f') v |= (uint32_t)(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F') v |= (uint32_t)(c - 'A' + 10);
            else { ++p_; fail("invalid escape"); }
        }
        return v;
    }
    std::string parse_string()
    {
        ++p_;   // opening quote
        std::string out;
        for (;;) {
            if (p_ == end_) fail("EOF while parsing a string");
            const unsigned char c = (unsigned char)*p_++;
            if (c == '"') return out;
            if (c < 0x20) fail("control character (\\u0000-\\u001F) found while parsing a string");
            if (c >= 0x80) {
                // a string is UTF-8: check the sequence (no overlong forms, no surrogates, <= U+10FFFF)
                int more = c >= 0xF0 ? 3 : c >= 0xE0 ? 2 : c >= 0xC2 ? 1 : -1;
                if (c > 0xF4) more = -1;
                if (more < 0 || end_ - p_ < more) fail("invalid unicode code point");
                const unsigned char c1 = (unsigned char)p_[0];
                bool okay = (c1 & 0xC0) == 0x80;
                if (c == 0xE0) okay = okay && c1 >= 0xA0;
                if (c == 0xED) okay = okay && c1 < 0xA0;
                if (c == 0xF0) okay = okay && c1 >= 0x90;
                if (c == 0xF4) okay = okay && c1 < 0x90;
                for (int k = 1; k < more; ++k) okay = okay && ((unsigned char)p_[k] & 0xC0) == 0x80;
                if (!okay) fail("invalid unicode code point");
                out += (char)c;
                out.append(p_, (size_t)more);
                p_ += more;
                continue;
            }
            if (c != '\\') { out += (char)c; continue; }
            if (p_ == end_) fail("EOF while parsing a string");
            const char e = *p_++;
            switch (e) {
            case '"': out += '"'; break;
            case '\\': out += '\\'; break;
            case '/': out += '/'; break;
            case 'b': out += '\b'; break;
            case 'f': out += '\f'; break;
            case 'n': out += '\n'; break;
            case 'r': out += '\r'; break;
            case 't': out += '\t'; break;
            case 'u': {
                uint32_t cp = hex4();
                if (cp >= 0xDC00 && cp <= 0xDFFF) fail("lone leading surrogate in hex escape");
                if (cp >= 0xD800 && cp <= 0xDBFF) {
                    if (end_ - p_ < 2 || p_[0] != '\\' || p_[1] != 'u') fail("unexpected end of hex escape");
                    p_ += 2;
                    const uint32_t lo = hex4();
                    if (lo < 0xDC00 || lo > 0xDFFF) fail("lone leading surrogate in hex escape");
                    cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                }
                put_utf8(out, cp);
                break;
            }
            default: fail("invalid escape");
            }
        }
    }

    Value parse_number()
    {
        const char* start = p_;
        bool negative = false, integral = true;
        if (*p_ == '-') { negative = true; ++p_; }
        if (p_ == end_) fail("EOF while parsing a value");
        if (*p_ == '0') {
            ++p_;
            if (p_ < end_ && *p_ >= '0' && *p_ <= '9') fail("invalid number");
        } else if (*p_ >= '1' && *p_ <= '9') {
            while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_;
        } else {
            ++p_;
            fail("invalid number");
        }
        if (p_ < end_ && *p_ == '.') {
            integral = false;
            ++p_;
            if (p_ == end_) fail("EOF while parsing a value");
            if (*p_ < '0' || *p_ > '9') { ++p_; fail("invalid number"); }
            while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_;
        }
        if (p_ < end_ && (*p_ == 'e' || *p_ == 'E')) {
            integral = false;
            ++p_;
            if (p_ < end_ && (*p_ == '+' || *p_ == '-')) ++p_;
            if (p_ == end_) fail("EOF while parsing a value");
            if (*p_ < '0' || *p_ > '9') { ++p_; fail("invalid number"); }
            while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_;
        }
        const std::string spelled(start, p_);
        Value v;
        v.kind = Value::Kind::Number;
        v.f = std::strtod(spelled.c_str(), nullptr);
        v.num = Value::Num::Float;
        if (integral) {
            errno = 0;
            if (!negative) {
                const unsigned long long x = std::strtoull(spelled.c_str(), nullptr, 10);
                if (errno == 0) { v.num = Value::Num::Unsigned; v.u = x; }
            } else {
                const long long x = std::strtoll(spelled.c_str(), nullptr, 10);
                // "-0" is the float negative zero
                if (errno == 0 && x != 0) { v.num = Value::Num::Negative; v.i = x; }
            }
        } else if (!std::isfinite(v.f)) {
            fail("number out of range");
        }
        return v;
    }
};

inline Value parse(const char* data, size_t len) { return Parser(data, len).parse_document(); }
inline Value parse(const std::string& s) { return parse(s.data(), s.size()); }

}  // namespace berth::json
