// Minimal strict JSON reader for PTIR program text (serde_json output of
// crates/gpt-rs/src/backend/spec.rs `Program`).  DOM with ordered object members.
#pragma once
#include <cerrno>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace gptrs {

struct JsonError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct Json {
    enum Kind { Null, Bool, Int, Float, String, Array, Object } kind = Null;
    bool b = false;
    int64_t i = 0;
    double d = 0.0;
    std::string s;
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj;

    bool is_null() const { return kind == Null; }
    bool is_string() const { return kind == String; }
    bool is_object() const { return kind == Object; }
    bool is_array() const { return kind == Array; }
    bool is_number() const { return kind == Int || kind == Float; }

    const Json* find(const char* key) const {
        if (kind != Object) return nullptr;
        for (auto& kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
    const Json& at(const char* key) const {
        const Json* j = find(key);
        if (!j) throw JsonError(std::string("missing field `") + key + "`");
        return *j;
    }
    int64_t as_int() const {
        if (kind == Int) return i;
        if (kind == Float && d == (double)(int64_t)d) return (int64_t)d;
        throw JsonError("expected integer");
    }
    double as_double() const {
        if (kind == Int) return (double)i;
        if (kind == Float) return d;
        throw JsonError("expected number");
    }
    const std::string& as_string() const {
        if (kind != String) throw JsonError("expected string");
        return s;
    }
    bool as_bool() const {
        if (kind != Bool) throw JsonError("expected bool");
        return b;
    }
    const std::vector<Json>& as_array() const {
        if (kind != Array) throw JsonError("expected array");
        return arr;
    }
};

class JsonParser {
  public:
    JsonParser(const char* p, size_t n) : p_(p), end_(p + n) {}
    Json parse() {
        Json v = value(0);
        ws();
        if (p_ != end_) fail("trailing characters");
        return v;
    }

  private:
    const char* p_;
    const char* end_;
    [[noreturn]] void fail(const char* m) { throw JsonError(std::string("json error: ") + m); }
    void ws() {
        while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r')) ++p_;
    }
    Json value(int depth) {
        if (depth > 64) fail("nesting too deep");
        ws();
        if (p_ >= end_) fail("unexpected end");
        char c = *p_;
        Json v;
        if (c == '{') {
            ++p_;
            v.kind = Json::Object;
            ws();
            if (p_ < end_ && *p_ == '}') { ++p_; return v; }
            for (;;) {
                ws();
                if (p_ >= end_ || *p_ != '"') fail("expected object key");
                std::string k = str();
                ws();
                if (p_ >= end_ || *p_ != ':') fail("expected ':'");
                ++p_;
                v.obj.emplace_back(std::move(k), value(depth + 1));
                ws();
                if (p_ < end_ && *p_ == ',') { ++p_; continue; }
                if (p_ < end_ && *p_ == '}') { ++p_; break; }
                fail("expected ',' or '}'");
            }
        } else if (c == '[') {
            ++p_;
            v.kind = Json::Array;
            ws();
            if (p_ < end_ && *p_ == ']') { ++p_; return v; }
            for (;;) {
                v.arr.push_back(value(depth + 1));
                ws();
                if (p_ < end_ && *p_ == ',') { ++p_; continue; }
                if (p_ < end_ && *p_ == ']') { ++p_; break; }
                fail("expected ',' or ']'");
            }
        } else if (c == '"') {
            v.kind = Json::String;
            v.s = str();
        } else if (c == 't' && end_ - p_ >= 4 && !memcmp(p_, "true", 4)) {
            p_ += 4; v.kind = Json::Bool; v.b = true;
        } else if (c == 'f' && end_ - p_ >= 5 && !memcmp(p_, "false", 5)) {
            p_ += 5; v.kind = Json::Bool; v.b = false;
        } else if (c == 'n' && end_ - p_ >= 4 && !memcmp(p_, "null", 4)) {
            p_ += 4; v.kind = Json::Null;
        } else if (c == '-' || (c >= '0' && c <= '9')) {
            const char* s = p_;
            bool is_float = false;
            if (*p_ == '-') ++p_;
            while (p_ < end_ && ((*p_ >= '0' && *p_ <= '9') || *p_ == '.' || *p_ == 'e' || *p_ == 'E' || *p_ == '+' || *p_ == '-')) {
                if (*p_ == '.' || *p_ == 'e' || *p_ == 'E') is_float = true;
                ++p_;
            }
            std::string tok(s, p_);
            if (is_float) {
                v.kind = Json::Float;
                v.d = strtod(tok.c_str(), nullptr);
            } else {
                v.kind = Json::Int;
                errno = 0;
                v.i = strtoll(tok.c_str(), nullptr, 10);
                if (errno) { v.kind = Json::Float; v.d = strtod(tok.c_str(), nullptr); }
            }
        } else {
            fail("unexpected character");
        }
        return v;
    }
    std::string str() {
        ++p_;  // opening quote
        std::string out;
        while (p_ < end_ && *p_ != '"') {
            if (*p_ == '\\') {
                ++p_;
                if (p_ >= end_) fail("bad escape");
                switch (*p_) {
                    case 'n': out.push_back('\n'); break;
                    case 't': out.push_back('\t'); break;
                    case 'r': out.push_back('\r'); break;
                    case 'b': out.push_back('\b'); break;
                    case 'f': out.push_back('\f'); break;
                    case 'u': {
                        if (end_ - p_ < 5) fail("bad \\u escape");
                        unsigned cp = (unsigned)strtoul(std::string(p_ + 1, p_ + 5).c_str(), nullptr, 16);
                        p_ += 4;
                        if (cp < 0x80) out.push_back((char)cp);
                        else if (cp < 0x800) { out.push_back((char)(0xC0 | (cp >> 6))); out.push_back((char)(0x80 | (cp & 0x3F))); }
                        else { out.push_back((char)(0xE0 | (cp >> 12))); out.push_back((char)(0x80 | ((cp >> 6) & 0x3F))); out.push_back((char)(0x80 | (cp & 0x3F))); }
                        break;
                    }
                    default: out.push_back(*p_);
                }
                ++p_;
            } else {
                out.push_back(*p_++);
            }
        }
        if (p_ >= end_) fail("unterminated string");
        ++p_;
        return out;
    }
};

}  // namespace gptrs
