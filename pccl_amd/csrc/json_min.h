// Minimal JSON reader for the JSON v2 graph documents (objects, arrays, strings, numbers, bools, null).
// Dependency-free replacement for the reference's use of nlohmann::json in
// csrc/engine/graph_builder.cc:12-107 — only what that loader needs: ordered object lookup,
// array iteration, integer and string extraction, with precise error positions.
#pragma once

#include <cerrno>
#include <cstdint>
#include <cstdlib>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace pccl_hip::json {

struct ParseError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct Value {
    enum Kind { Null, Bool, Int, Real, String, Array, Object } kind = Null;
    bool b = false;
    int64_t i = 0;
    double d = 0.0;
    std::string s;
    std::vector<Value> arr;
    std::vector<std::pair<std::string, Value>> obj;  // insertion order kept

    bool is_object() const { return kind == Object; }
    bool is_array() const { return kind == Array; }
    bool is_string() const { return kind == String; }
    bool is_int() const { return kind == Int; }

    const Value* find(const std::string& key) const {
        if (kind != Object) return nullptr;
        for (auto& kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
    bool contains(const std::string& key) const { return find(key) != nullptr; }

    const Value& at(const std::string& key) const {
        const Value* v = find(key);
        if (!v) throw ParseError("missing key '" + key + "'");
        return *v;
    }
    int64_t as_int(const char* what) const {
        if (kind == Int) return i;
        if (kind == Real && d == (double)(int64_t)d) return (int64_t)d;
        throw ParseError(std::string("expected an integer for ") + what);
    }
    const std::string& as_string(const char* what) const {
        if (kind != String) throw ParseError(std::string("expected a string for ") + what);
        return s;
    }
    int64_t int_or(const std::string& key, int64_t dflt) const {
        const Value* v = find(key);
        return v ? v->as_int(key.c_str()) : dflt;
    }
};

class Parser {
   public:
    Parser(const char* text, size_t len) : p_(text), end_(text + len), begin_(text) {}

    Value parse_document() {
        Value v = parse_value(0);
        skip_ws();
        if (p_ != end_) fail("trailing characters after the document");
        return v;
    }

   private:
    const char* p_;
    const char* end_;
    const char* begin_;
    static constexpr int kMaxDepth = 64;

    [[noreturn]] void fail(const std::string& msg) const {
        throw ParseError("JSON: " + msg + " at byte " + std::to_string(p_ - begin_));
    }
    void skip_ws() {
        while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r')) ++p_;
    }
    bool consume(char c) {
        skip_ws();
        if (p_ < end_ && *p_ == c) { ++p_; return true; }
        return false;
    }
    void expect_word(const char* w) {
        for (const char* q = w; *q; ++q, ++p_)
            if (p_ >= end_ || *p_ != *q) fail(std::string("bad literal, expected '") + w + "'");
    }

    Value parse_value(int depth) {
        if (depth > kMaxDepth) fail("nesting too deep");
        skip_ws();
        if (p_ >= end_) fail("unexpected end of input");
        Value v;
        switch (*p_) {
            case '{': {
                ++p_;
                v.kind = Value::Object;
                if (consume('}')) return v;
                do {
                    skip_ws();
                    if (p_ >= end_ || *p_ != '"') fail("expected a string key");
                    std::string key = parse_string();
                    if (!consume(':')) fail("expected ':'");
                    v.obj.emplace_back(std::move(key), parse_value(depth + 1));
                } while (consume(','));
                if (!consume('}')) fail("expected ',' or '}'");
                return v;
            }
            case '[': {
                ++p_;
                v.kind = Value::Array;
                if (consume(']')) return v;
                do { v.arr.push_back(parse_value(depth + 1)); } while (consume(','));
                if (!consume(']')) fail("expected ',' or ']'");
                return v;
            }
            case '"':
                v.kind = Value::String;
                v.s = parse_string();
                return v;
            case 't': expect_word("true"); v.kind = Value::Bool; v.b = true; return v;
            case 'f': expect_word("false"); v.kind = Value::Bool; v.b = false; return v;
            case 'n': expect_word("null"); v.kind = Value::Null; return v;
            default: return parse_number();
        }
    }

    std::string parse_string() {
        ++p_;  // opening quote
        std::string out;
        while (true) {
            if (p_ >= end_) fail("unterminated string");
            char c = *p_++;
            if (c == '"') return out;
            if ((unsigned char)c < 0x20) fail("control character in string");
            if (c != '\\') { out.push_back(c); continue; }
            if (p_ >= end_) fail("unterminated escape");
            char e = *p_++;
            switch (e) {
                case '"': out.push_back('"'); break;
                case '\\': out.push_back('\\'); break;
                case '/': out.push_back('/'); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'n': out.push_back('\n'); break;
                case 'r': out.push_back('\r'); break;
                case 't': out.push_back('\t'); break;
                case 'u': {
                    if (end_ - p_ < 4) fail("short \\u escape");
                    unsigned cp = 0;
                    for (int k = 0; k < 4; ++k) {
                        char h = *p_++;
                        cp <<= 4;
                        if (h >= '0' && h <= '9') cp |= h - '0';
                        else if (h >= 'a' && h <= 'f') cp |= h - 'a' + 10;
                        else if (h >= 'A' && h <= 'F') cp |= h - 'A' + 10;
                        else fail("bad hex digit in \\u escape");
                    }
                    // UTF-8 encode (surrogate pairs are passed through as two 3-byte sequences;
                    // graph documents are ASCII)
                    if (cp < 0x80) out.push_back((char)cp);
                    else if (cp < 0x800) { out.push_back((char)(0xC0 | (cp >> 6))); out.push_back((char)(0x80 | (cp & 0x3F))); }
                    else { out.push_back((char)(0xE0 | (cp >> 12))); out.push_back((char)(0x80 | ((cp >> 6) & 0x3F))); out.push_back((char)(0x80 | (cp & 0x3F))); }
                    break;
                }
                default: fail("bad escape character");
            }
        }
    }

    Value parse_number() {
        const char* start = p_;
        bool real = false;
        if (p_ < end_ && *p_ == '-') ++p_;
        if (p_ >= end_ || *p_ < '0' || *p_ > '9') fail("unexpected character");
        while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_;
        if (p_ < end_ && *p_ == '.') { real = true; ++p_; while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_; }
        if (p_ < end_ && (*p_ == 'e' || *p_ == 'E')) {
            real = true; ++p_;
            if (p_ < end_ && (*p_ == '+' || *p_ == '-')) ++p_;
            while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_;
        }
        std::string tok(start, p_);
        Value v;
        if (real) { v.kind = Value::Real; v.d = std::strtod(tok.c_str(), nullptr); }
        else {
            errno = 0;
            v.kind = Value::Int; v.i = std::strtoll(tok.c_str(), nullptr, 10);
            if (errno == ERANGE) { v.kind = Value::Real; v.d = std::strtod(tok.c_str(), nullptr); }
        }
        return v;
    }
};

inline Value parse(const char* text, size_t len) { return Parser(text, len).parse_document(); }

}  // namespace pccl_hip::json
