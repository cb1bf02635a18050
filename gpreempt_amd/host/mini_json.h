// A small JSON value with parser and writer (the reference links jsoncpp for its config and
// report files; this build has no external dependency).
#pragma once
#include <cstdio>
#include <cstdlib>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace foo {
namespace json {

struct Value {
    enum Type { Null, Bool, Number, String, Array, Object } type = Null;
    bool b = false;
    double num = 0;
    std::string str;
    std::vector<Value> arr;
    std::vector<std::pair<std::string, Value>> obj;  // insertion order kept for readable reports

    Value() {}
    Value(double v) : type(Number), num(v) {}
    Value(int v) : type(Number), num(v) {}
    Value(long v) : type(Number), num((double)v) {}
    Value(size_t v) : type(Number), num((double)v) {}
    Value(bool v) : type(Bool), b(v) {}
    Value(const char *s) : type(String), str(s) {}
    Value(const std::string &s) : type(String), str(s) {}
    static Value array() { Value v; v.type = Array; return v; }
    static Value object() { Value v; v.type = Object; return v; }

    bool has(const std::string &k) const {
        for (auto &kv : obj) if (kv.first == k) return true;
        return false;
    }
    const Value &operator[](const std::string &k) const {
        static const Value null_value;
        for (auto &kv : obj) if (kv.first == k) return kv.second;
        return null_value;
    }
    Value &set(const std::string &k) {
        if (type != Object) { type = Object; }
        for (auto &kv : obj) if (kv.first == k) return kv.second;
        obj.emplace_back(k, Value());
        return obj.back().second;
    }
    void push(const Value &v) { type = Array; arr.push_back(v); }
    double number(double d = 0) const { return type == Number ? num : (type == Bool ? (b ? 1 : 0) : d); }
    std::string string(const std::string &d = "") const { return type == String ? str : d; }
    bool boolean(bool d = false) const { return type == Bool ? b : (type == Number ? num != 0 : d); }

    std::string dump() const {
        std::string out;
        write(out);
        return out;
    }
    void write(std::string &out) const {
        char buf[64];
        switch (type) {
            case Null: out += "null"; break;
            case Bool: out += b ? "true" : "false"; break;
            case Number:
                if (num == (double)(long long)num && num > -1e15 && num < 1e15) std::snprintf(buf, sizeof buf, "%lld", (long long)num);
                else std::snprintf(buf, sizeof buf, "%.9g", num);
                out += buf;
                break;
            case String:
                out += '"';
                for (char c : str) {
                    if (c == '"' || c == '\\') { out += '\\'; out += c; }
                    else if (c == '\n') out += "\\n";
                    else if ((unsigned char)c < 0x20) { std::snprintf(buf, sizeof buf, "\\u%04x", c); out += buf; }
                    else out += c;
                }
                out += '"';
                break;
            case Array:
                out += '[';
                for (size_t i = 0; i < arr.size(); ++i) { if (i) out += ','; arr[i].write(out); }
                out += ']';
                break;
            case Object:
                out += '{';
                for (size_t i = 0; i < obj.size(); ++i) {
                    if (i) out += ',';
                    Value(obj[i].first).write(out);
                    out += ':';
                    obj[i].second.write(out);
                }
                out += '}';
                break;
        }
    }
};

class Parser {
public:
    explicit Parser(const std::string &s) : s_(s) {}
    bool parse(Value &out) {
        ok_ = true;
        out = value();
        ws();
        return ok_ && i_ == s_.size();
    }

private:
    const std::string &s_;
    size_t i_ = 0;
    bool ok_ = true;
    int depth_ = 0;
    static constexpr int kMaxDepth = 64;  // nesting beyond this is refused instead of recursed into
    void ws() { while (i_ < s_.size() && (s_[i_] == ' ' || s_[i_] == '\n' || s_[i_] == '\t' || s_[i_] == '\r')) ++i_; }
    bool eat(char c) { ws(); if (i_ < s_.size() && s_[i_] == c) { ++i_; return true; } return false; }
    Value value() {
        ws();
        if (i_ >= s_.size()) { ok_ = false; return Value(); }
        char c = s_[i_];
        if ((c == '{' || c == '[') && depth_ >= kMaxDepth) { ok_ = false; return Value(); }
        if (c == '{') {
            ++i_;
            ++depth_;
            Value v = Value::object();
            if (eat('}')) { --depth_; return v; }
            do {
                ws();
                Value k = value();
                if (k.type != Value::String || !eat(':')) { ok_ = false; --depth_; return v; }
                v.set(k.str) = value();
            } while (ok_ && eat(','));
            if (!eat('}')) ok_ = false;
            --depth_;
            return v;
        }
        if (c == '[') {
            ++i_;
            ++depth_;
            Value v = Value::array();
            if (eat(']')) { --depth_; return v; }
            do { v.arr.push_back(value()); } while (ok_ && eat(','));
            if (!eat(']')) ok_ = false;
            --depth_;
            return v;
        }
        if (c == '"') {
            ++i_;
            Value v("");
            while (i_ < s_.size() && s_[i_] != '"') {
                if (s_[i_] == '\\' && i_ + 1 < s_.size()) {
                    char e = s_[++i_];
                    v.str += e == 'n' ? '\n' : e == 't' ? '\t' : e;
                } else v.str += s_[i_];
                ++i_;
            }
            if (i_ >= s_.size()) ok_ = false; else ++i_;
            return v;
        }
        if (s_.compare(i_, 4, "true") == 0) { i_ += 4; return Value(true); }
        if (s_.compare(i_, 5, "false") == 0) { i_ += 5; return Value(false); }
        if (s_.compare(i_, 4, "null") == 0) { i_ += 4; return Value(); }
        char *end = nullptr;
        double d = std::strtod(s_.c_str() + i_, &end);
        if (end == s_.c_str() + i_) { ok_ = false; return Value(); }
        i_ = end - s_.c_str();
        return Value(d);
    }
};

inline bool parse(const std::string &text, Value &out) { return Parser(text).parse(out); }

}  // namespace json
}  // namespace foo
