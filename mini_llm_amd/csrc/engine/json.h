// A small JSON reader and writer: what config.json and the header of a safetensors file need
// (objects, arrays, strings with the common escapes, numbers, true/false/null).
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace minillm {

class JsonError : public std::runtime_error {
public:
    explicit JsonError(const std::string& what) : std::runtime_error(what) {}
};

class Json {
public:
    enum Kind { Null, Bool, Number, String, Array, Object };

    Json() = default;
    static Json parse(const std::string& text);
    std::string dump() const;

    Kind kind() const { return kind_; }
    bool is_null() const { return kind_ == Null; }
    bool is_number() const { return kind_ == Number; }
    bool is_integer() const { return kind_ == Number && integral_; }
    bool is_string() const { return kind_ == String; }
    bool is_bool() const { return kind_ == Bool; }
    bool is_array() const { return kind_ == Array; }
    bool is_object() const { return kind_ == Object; }

    double number() const { need(Number, "a number"); return num_; }
    int64_t integer() const { need(Number, "an integer"); if (!integral_) throw JsonError("expected an integer"); return static_cast<int64_t>(num_); }
    bool boolean() const { need(Bool, "true or false"); return bool_; }
    const std::string& string() const { need(String, "a string"); return str_; }
    const std::vector<Json>& array() const { need(Array, "an array"); return arr_; }
    // object members in the order they were read or added
    const std::vector<std::pair<std::string, Json>>& members() const { need(Object, "an object"); return obj_; }
    bool has(const std::string& key) const;
    const Json& at(const std::string& key) const;          // throws if absent
    const Json* find(const std::string& key) const;        // nullptr if absent

    static Json of(double v) { Json j; j.kind_ = Number; j.num_ = v; j.integral_ = false; return j; }
    static Json of(int64_t v) { Json j; j.kind_ = Number; j.num_ = static_cast<double>(v); j.integral_ = true; return j; }
    static Json of(int v) { return of(static_cast<int64_t>(v)); }
    static Json of(bool v) { Json j; j.kind_ = Bool; j.bool_ = v; return j; }
    static Json of(const std::string& v) { Json j; j.kind_ = String; j.str_ = v; return j; }
    static Json of(const char* v) { return of(std::string(v)); }
    static Json array_of(std::vector<Json> v) { Json j; j.kind_ = Array; j.arr_ = std::move(v); return j; }
    static Json object() { Json j; j.kind_ = Object; return j; }
    void set(const std::string& key, Json v);

private:
    void need(Kind k, const char* what) const {
        if (kind_ != k) throw JsonError(std::string("expected ") + what);
    }
    Kind kind_ = Null;
    bool bool_ = false, integral_ = false;
    double num_ = 0.0;
    std::string str_;
    std::vector<Json> arr_;
    std::vector<std::pair<std::string, Json>> obj_;
    friend class JsonParser;
};

}  // namespace minillm
