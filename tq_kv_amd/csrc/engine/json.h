// A small JSON value: enough to read config.json, generation_config.json, tokenizer.json and
// safetensors headers, and to carry part parameters across the C boundary.  Objects keep
// the order of their keys.  Numbers remember whether they were written as integers.
#pragma once
#include <stdint.h>

#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace tq {

struct JsonError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

class Json {
public:
    enum Kind { Null, Bool, Int, Float, String, Array, Object };
    using Member = std::pair<std::string, Json>;

    Json() : kind_(Null) {}
    Json(std::nullptr_t) : kind_(Null) {}
    Json(bool b) : kind_(Bool), int_(b) {}
    Json(int v) : kind_(Int), int_(v) {}
    Json(long v) : kind_(Int), int_(v) {}
    Json(long long v) : kind_(Int), int_(v) {}
    Json(unsigned long v) : kind_(Int), int_((long long)v) {}
    Json(double v) : kind_(Float), num_(v) {}
    Json(const char* s) : kind_(String), str_(s) {}
    Json(std::string s) : kind_(String), str_(std::move(s)) {}
    static Json array() { Json j; j.kind_ = Array; return j; }
    static Json object() { Json j; j.kind_ = Object; return j; }

    Kind kind() const { return kind_; }
    bool is_null() const { return kind_ == Null; }
    bool is_bool() const { return kind_ == Bool; }
    bool is_int() const { return kind_ == Int; }
    bool is_number() const { return kind_ == Int || kind_ == Float; }
    bool is_string() const { return kind_ == String; }
    bool is_array() const { return kind_ == Array; }
    bool is_object() const { return kind_ == Object; }

    bool as_bool() const { return int_ != 0; }
    long long as_int() const { return kind_ == Float ? (long long)num_ : int_; }
    double as_number() const { return kind_ == Int ? (double)int_ : num_; }
    const std::string& as_string() const { return str_; }
    const std::vector<Json>& items() const { return arr_; }
    std::vector<Json>& items() { return arr_; }
    const std::vector<Member>& members() const { return obj_; }

    // object access: a pointer to the member or nullptr
    const Json* find(const std::string& key) const {
        if (kind_ != Object) return nullptr;
        for (const Member& m : obj_)
            if (m.first == key) return &m.second;
        return nullptr;
    }
    // the member, or a null value where there is none
    const Json& operator[](const std::string& key) const {
        static const Json none;
        const Json* j = find(key);
        return j ? *j : none;
    }
    void set(const std::string& key, Json value) {
        if (kind_ != Object) { *this = object(); }
        for (Member& m : obj_)
            if (m.first == key) { m.second = std::move(value); return; }
        obj_.emplace_back(key, std::move(value));
    }
    // adds a member without looking for an earlier one of the same key (what the parser does: a
    // tokenizer's vocabulary has 150k keys)
    void append(std::string key, Json value) {
        if (kind_ != Object) { *this = object(); }
        obj_.emplace_back(std::move(key), std::move(value));
    }
    void push(Json value) {
        if (kind_ != Array) { *this = array(); }
        arr_.push_back(std::move(value));
    }

    static Json parse(const std::string& text);          // throws JsonError
    static Json parse(const char* text, size_t n);
    std::string dump() const;

private:
    Kind kind_;
    long long int_ = 0;
    double num_ = 0.0;
    std::string str_;
    std::vector<Json> arr_;
    std::vector<Member> obj_;
    void dump_to(std::string& out) const;
};

}  // namespace tq
