// Minimal JSON value, parser and writer for the SDFG interchange format.
// (The reference serialises SDFGs with nlohmann::json,
// sdfg/src/serializer/json_serializer.cpp:56-176; only the value model is
// needed here.)
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace sdfg::json {

class Value;
using Array = std::vector<Value>;
// insertion-ordered object: argument order and connector order matter
using Object = std::vector<std::pair<std::string, Value>>;

class ParseError : public std::runtime_error {
public:
    using std::runtime_error::runtime_error;
};

class Value {
public:
    enum class Kind { Null, Bool, Int, Double, String, Array, Object };

    Value() : kind_(Kind::Null) {}
    Value(std::nullptr_t) : kind_(Kind::Null) {}
    Value(bool b) : kind_(Kind::Bool), b_(b) {}
    Value(int v) : kind_(Kind::Int), i_(v) {}
    Value(int64_t v) : kind_(Kind::Int), i_(v) {}
    Value(size_t v) : kind_(Kind::Int), i_((int64_t) v) {}
    Value(double v) : kind_(Kind::Double), d_(v) {}
    Value(const char* s) : kind_(Kind::String), s_(s) {}
    Value(std::string s) : kind_(Kind::String), s_(std::move(s)) {}
    Value(Array a) : kind_(Kind::Array), a_(std::make_shared<Array>(std::move(a))) {}
    Value(Object o) : kind_(Kind::Object), o_(std::make_shared<Object>(std::move(o))) {}

    Kind kind() const { return kind_; }
    bool is_null() const { return kind_ == Kind::Null; }
    bool is_string() const { return kind_ == Kind::String; }
    bool is_number() const { return kind_ == Kind::Int || kind_ == Kind::Double; }
    bool is_array() const { return kind_ == Kind::Array; }
    bool is_object() const { return kind_ == Kind::Object; }
    bool is_bool() const { return kind_ == Kind::Bool; }

    bool as_bool() const;
    int64_t as_int() const;
    double as_double() const;
    const std::string& as_string() const;
    const Array& as_array() const;
    const Object& as_object() const;
    Array& as_array();
    Object& as_object();

    // object access; `at` throws when the key is missing
    bool contains(const std::string& key) const;
    const Value& at(const std::string& key) const;
    const Value* find(const std::string& key) const;
    void set(const std::string& key, Value v);

    // a number or a string holding an expression -> expression text
    std::string as_expression() const;

    std::string dump(int indent = -1) const;
    static Value parse(const std::string& text);

private:
    void dump_to(std::string& out, int indent, int depth) const;

    Kind kind_;
    bool b_ = false;
    int64_t i_ = 0;
    double d_ = 0.0;
    std::string s_;
    std::shared_ptr<Array> a_;
    std::shared_ptr<Object> o_;
};

} // namespace sdfg::json
