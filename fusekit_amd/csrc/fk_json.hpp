// Minimal JSON reader for the artifact files (task_graph.json, manifest.json).
// Parses into a small tree; numbers are doubles, objects keep insertion order.
#pragma once
#include <cstdlib>
#include <cstring>
#include <memory>
#include <string>
#include <utility>
#include <vector>

namespace fk {
namespace json {

struct Value {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    bool b = false;
    double num = 0.0;
    std::string str;
    std::vector<Value> arr;
    std::vector<std::pair<std::string, Value>> obj;

    const Value* get(const char* key) const {
        if (kind != Object) return nullptr;
        for (const auto& kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
    bool is_number() const { return kind == Number; }
    bool is_string() const { return kind == String; }
    bool is_array() const { return kind == Array; }
    bool is_object() const { return kind == Object; }
};

class Parser {
   public:
    explicit Parser(const std::string& text) : s_(text) {}
    bool parse(Value* out, std::string* err) {
        skip();
        if (!value(out)) {
            *err = err_ + " at byte " + std::to_string(i_);
            return false;
        }
        skip();
        if (i_ != s_.size()) {
            *err = "trailing characters at byte " + std::to_string(i_);
            return false;
        }
        return true;
    }

   private:
    const std::string& s_;
    size_t i_ = 0;
    std::string err_;
    int depth_ = 0;

    void skip() {
        while (i_ < s_.size() && (s_[i_] == ' ' || s_[i_] == '\n' || s_[i_] == '\t' || s_[i_] == '\r')) ++i_;
    }
    bool fail(const char* m) {
        err_ = m;
        return false;
    }
    bool literal(const char* lit) {
        const size_t n = strlen(lit);
        if (s_.compare(i_, n, lit) != 0) return fail("bad literal");
        i_ += n;
        return true;
    }
    bool string(std::string* out) {
        if (i_ >= s_.size() || s_[i_] != '"') return fail("expected string");
        ++i_;
        out->clear();
        while (i_ < s_.size() && s_[i_] != '"') {
            char c = s_[i_++];
            if (c == '\\') {
                if (i_ >= s_.size()) return fail("bad escape");
                char e = s_[i_++];
                switch (e) {
                    case 'n': out->push_back('\n'); break;
                    case 't': out->push_back('\t'); break;
                    case 'r': out->push_back('\r'); break;
                    case 'b': out->push_back('\b'); break;
                    case 'f': out->push_back('\f'); break;
                    case 'u': {
                        if (i_ + 4 > s_.size()) return fail("bad \\u escape");
                        unsigned cp = (unsigned)strtoul(s_.substr(i_, 4).c_str(), nullptr, 16);
                        i_ += 4;
                        if (cp < 0x80) {
                            out->push_back((char)cp);
                        } else if (cp < 0x800) {
                            out->push_back((char)(0xC0 | (cp >> 6)));
                            out->push_back((char)(0x80 | (cp & 0x3F)));
                        } else {
                            out->push_back((char)(0xE0 | (cp >> 12)));
                            out->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
                            out->push_back((char)(0x80 | (cp & 0x3F)));
                        }
                        break;
                    }
                    default: out->push_back(e);
                }
            } else {
                out->push_back(c);
            }
        }
        if (i_ >= s_.size()) return fail("unterminated string");
        ++i_;
        return true;
    }
    bool value(Value* v) {
        if (++depth_ > 256) return fail("nesting too deep");
        bool ok = value_inner(v);
        --depth_;
        return ok;
    }
    bool value_inner(Value* v) {
        skip();
        if (i_ >= s_.size()) return fail("unexpected end");
        const char c = s_[i_];
        if (c == '{') {
            v->kind = Value::Object;
            ++i_;
            skip();
            if (i_ < s_.size() && s_[i_] == '}') {
                ++i_;
                return true;
            }
            while (true) {
                skip();
                std::string key;
                if (!string(&key)) return false;
                skip();
                if (i_ >= s_.size() || s_[i_] != ':') return fail("expected ':'");
                ++i_;
                Value child;
                if (!value(&child)) return false;
                v->obj.emplace_back(std::move(key), std::move(child));
                skip();
                if (i_ < s_.size() && s_[i_] == ',') {
                    ++i_;
                    continue;
                }
                if (i_ < s_.size() && s_[i_] == '}') {
                    ++i_;
                    return true;
                }
                return fail("expected ',' or '}'");
            }
        }
        if (c == '[') {
            v->kind = Value::Array;
            ++i_;
            skip();
            if (i_ < s_.size() && s_[i_] == ']') {
                ++i_;
                return true;
            }
            while (true) {
                Value child;
                if (!value(&child)) return false;
                v->arr.push_back(std::move(child));
                skip();
                if (i_ < s_.size() && s_[i_] == ',') {
                    ++i_;
                    continue;
                }
                if (i_ < s_.size() && s_[i_] == ']') {
                    ++i_;
                    return true;
                }
                return fail("expected ',' or ']'");
            }
        }
        if (c == '"') {
            v->kind = Value::String;
            return string(&v->str);
        }
        if (c == 't') {
            v->kind = Value::Bool;
            v->b = true;
            return literal("true");
        }
        if (c == 'f') {
            v->kind = Value::Bool;
            v->b = false;
            return literal("false");
        }
        if (c == 'n') {
            v->kind = Value::Null;
            return literal("null");
        }
        if (c == '-' || (c >= '0' && c <= '9')) {
            char* end = nullptr;
            v->kind = Value::Number;
            v->num = strtod(s_.c_str() + i_, &end);
            if (end == s_.c_str() + i_) return fail("bad number");
            i_ = (size_t)(end - s_.c_str());
            return true;
        }
        return fail("unexpected character");
    }
};

}  // namespace json
}  // namespace fk
