// Minimal JSON reader for symmetrix model files.
//
// The model file (keys read at libsymmetrix/source/mace.cpp:912-1029) uses only
// objects, arrays, numbers, booleans and strings; the bulk is deeply nested
// arrays of numbers (spline tables).  Arrays whose elements are all numbers are
// stored flat as doubles, which keeps an 80 MB file at one allocation per row.
#pragma once

#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace smx {

struct JsonError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct Json {
    enum Type { Null, Bool, Number, String, Array, NumArray, Object } type = Null;
    bool b = false;
    double num = 0.0;
    std::string str;
    std::vector<Json> arr;
    std::vector<double> nums;  // NumArray payload
    std::map<std::string, Json> obj;

    bool has(const std::string& k) const { return type == Object && obj.count(k); }
    const Json& at(const std::string& k) const
    {
        if (type != Object) throw JsonError("model file: expected an object while looking up '" + k + "'");
        auto it = obj.find(k);
        if (it == obj.end()) throw JsonError("model file: missing key '" + k + "'");
        return it->second;
    }
    size_t size() const
    {
        if (type == NumArray) return nums.size();
        if (type == Array) return arr.size();
        throw JsonError("model file: expected an array");
    }
    double as_double() const
    {
        if (type != Number) throw JsonError("model file: expected a number");
        return num;
    }
    int as_int() const { return (int)as_double(); }
    bool as_bool() const
    {
        if (type != Bool) throw JsonError("model file: expected a boolean");
        return b;
    }
    // flat vector of doubles from a (possibly empty) 1-d array
    std::vector<double> as_doubles() const
    {
        if (type == NumArray) return nums;
        if (type == Array && arr.empty()) return {};
        if (type == Array) {  // numbers nested one level deeper are flattened
            std::vector<double> out;
            for (const auto& e : arr) {
                auto v = e.as_doubles();
                out.insert(out.end(), v.begin(), v.end());
            }
            return out;
        }
        throw JsonError("model file: expected an array of numbers");
    }
    std::vector<int> as_ints() const
    {
        auto d = as_doubles();
        std::vector<int> out(d.size());
        for (size_t i = 0; i < d.size(); ++i) out[i] = (int)d[i];
        return out;
    }
    const Json& operator[](size_t i) const
    {
        if (type != Array || i >= arr.size()) throw JsonError("model file: array index out of range");
        return arr[i];
    }
};

class JsonParser {
public:
    explicit JsonParser(const std::string& text) : p_(text.data()), end_(text.data() + text.size()) {}
    Json parse()
    {
        Json v = value();
        ws();
        if (p_ != end_) fail("trailing characters");
        return v;
    }

private:
    const char* p_;
    const char* end_;
    [[noreturn]] void fail(const char* what) { throw JsonError(std::string("model file: JSON parse error: ") + what); }
    void ws()
    {
        while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r')) ++p_;
    }
    Json value()
    {
        ws();
        if (p_ >= end_) fail("unexpected end of input");
        switch (*p_) {
        case '{': return object();
        case '[': return array();
        case '"': { Json j; j.type = Json::String; j.str = string(); return j; }
        case 't': lit("true"); { Json j; j.type = Json::Bool; j.b = true; return j; }
        case 'f': lit("false"); { Json j; j.type = Json::Bool; j.b = false; return j; }
        case 'n': lit("null"); return Json();
        default: { Json j; j.type = Json::Number; j.num = number(); return j; }
        }
    }
    void lit(const char* s)
    {
        size_t n = strlen(s);
        if ((size_t)(end_ - p_) < n || strncmp(p_, s, n)) fail("bad literal");
        p_ += n;
    }
    double number()
    {
        char* e = nullptr;
        double v = strtod(p_, &e);
        if (e == p_) {
            // python's json writes these for non-finite floats
            if (end_ - p_ >= 3 && !strncmp(p_, "NaN", 3)) { p_ += 3; return std::strtod("nan", nullptr); }
            if (end_ - p_ >= 8 && !strncmp(p_, "Infinity", 8)) { p_ += 8; return HUGE_VAL; }
            if (end_ - p_ >= 9 && !strncmp(p_, "-Infinity", 9)) { p_ += 9; return -HUGE_VAL; }
            fail("bad number");
        }
        p_ = e;
        return v;
    }
    std::string string()
    {
        ++p_;  // opening quote
        std::string s;
        while (p_ < end_ && *p_ != '"') {
            if (*p_ == '\\') {
                ++p_;
                if (p_ >= end_) fail("bad escape");
                switch (*p_) {
                case 'n': s += '\n'; break;
                case 't': s += '\t'; break;
                case 'r': s += '\r'; break;
                case 'b': s += '\b'; break;
                case 'f': s += '\f'; break;
                case 'u': p_ += 4; s += '?'; break;
                default: s += *p_;
                }
                ++p_;
            } else {
                s += *p_++;
            }
        }
        if (p_ >= end_) fail("unterminated string");
        ++p_;
        return s;
    }
    Json array()
    {
        ++p_;
        Json j;
        ws();
        if (p_ < end_ && *p_ == ']') { ++p_; j.type = Json::Array; return j; }
        // fast path: run of numbers
        ws();
        if (p_ < end_ && (*p_ == '-' || (*p_ >= '0' && *p_ <= '9') || *p_ == 'N' || *p_ == 'I')) {
            j.type = Json::NumArray;
            for (;;) {
                ws();
                j.nums.push_back(number());
                ws();
                if (p_ >= end_) fail("unterminated array");
                if (*p_ == ',') { ++p_; continue; }
                if (*p_ == ']') { ++p_; return j; }
                fail("mixed array of numbers and other values");
            }
        }
        j.type = Json::Array;
        for (;;) {
            j.arr.push_back(value());
            ws();
            if (p_ >= end_) fail("unterminated array");
            if (*p_ == ',') { ++p_; continue; }
            if (*p_ == ']') { ++p_; return j; }
            fail("expected ',' or ']'");
        }
    }
    Json object()
    {
        ++p_;
        Json j;
        j.type = Json::Object;
        ws();
        if (p_ < end_ && *p_ == '}') { ++p_; return j; }
        for (;;) {
            ws();
            if (p_ >= end_ || *p_ != '"') fail("expected a string key");
            std::string k = string();
            ws();
            if (p_ >= end_ || *p_ != ':') fail("expected ':'");
            ++p_;
            j.obj.emplace(std::move(k), value());
            ws();
            if (p_ >= end_) fail("unterminated object");
            if (*p_ == ',') { ++p_; continue; }
            if (*p_ == '}') { ++p_; return j; }
            fail("expected ',' or '}'");
        }
    }
};

}  // namespace smx
