// A small JSON value with the three things the backend configurations need: parsing (with //
// line comments, which the configuration files use), RFC 7396 merge-patch, and object iteration
// in key order.  The reference uses nlohmann::json for this (configs/json_repository.h).
#pragma once

#include <map>
#include <memory>
#include <string>
#include <vector>

namespace chainer_compiler {

class Json {
public:
    enum class Kind { kNull, kBool, kNumber, kString, kArray, kObject };

    Json() = default;
    static Json Parse(const std::string& text);

    Kind kind() const { return kind_; }
    bool is_null() const { return kind_ == Kind::kNull; }
    bool is_boolean() const { return kind_ == Kind::kBool; }
    bool is_number() const { return kind_ == Kind::kNumber; }
    bool is_string() const { return kind_ == Kind::kString; }
    bool is_array() const { return kind_ == Kind::kArray; }
    bool is_object() const { return kind_ == Kind::kObject; }

    bool boolean() const { return bool_; }
    double number() const { return number_; }
    const std::string& string() const { return string_; }
    const std::vector<Json>& array() const { return array_; }
    const std::map<std::string, Json>& items() const { return object_; }

    const Json* find(const std::string& key) const;
    void erase(const std::string& key) { object_.erase(key); }

    // RFC 7396: objects merge member by member, null deletes, anything else replaces.
    void merge_patch(const Json& patch);

    std::string dump() const;

private:
    friend class JsonParser;
    Kind kind_ = Kind::kNull;
    bool bool_ = false;
    double number_ = 0;
    std::string string_;
    std::vector<Json> array_;
    std::map<std::string, Json> object_;
};

}  // namespace chainer_compiler
