// Json.h — a small JSON document reader for network definition files.
// The reference reads those files with the jsoncpp library (engine/NNNetwork.cpp:2792-2812, Json::Reader with comments
// allowed); only reading is needed here: objects, arrays, strings with escapes, numbers, booleans, null, and // or /* */ comments.
// Object members keep the order of the file.
#ifndef DSSTNE_AMD_JSON_H
#define DSSTNE_AMD_JSON_H

#include <cstdint>
#include <string>
#include <utility>
#include <vector>

namespace json {

class Value {
public:
    enum Type { Null, Bool, Number, String, Array, Object };

    Value() : _type(Null), _number(0.0), _bool(false) {}

    Type type() const { return _type; }
    bool isNull() const { return _type == Null; }
    bool isBool() const { return _type == Bool; }
    bool isNumber() const { return _type == Number; }
    bool isString() const { return _type == String; }
    bool isArray() const { return _type == Array; }
    bool isObject() const { return _type == Object; }

    // Conversions follow what callers of a lenient reader expect: numbers from numeric strings are not converted, a
    // wrong kind throws std::runtime_error naming the kind found.
    double asDouble() const;
    float asFloat() const { return (float)asDouble(); }
    int64_t asInt() const;
    bool asBool() const;
    const std::string& asString() const;

    // Elements of an array; a scalar counts as an array of one (the definition files allow "Source": "a" and
    // "Source": ["a", "b"] alike).
    size_t size() const { return _type == Array ? _items.size() : (_type == Null ? 0 : 1); }
    const Value& operator[](size_t i) const { return _type == Array ? _items.at(i) : *this; }

    const std::vector<std::pair<std::string, Value>>& members() const { return _members; }
    const Value* find(const std::string& key) const;

private:
    friend class Parser;
    Type _type;
    double _number;
    bool _bool;
    std::string _string;
    std::vector<Value> _items;
    std::vector<std::pair<std::string, Value>> _members;
};

// Parses a whole document.  On failure returns false and sets error to "line L, column C: what".
bool parse(const std::string& text, Value& root, std::string& error);
bool parseFile(const std::string& path, Value& root, std::string& error);

// ASCII lower-case copy (keys and enumerated values of definition files are matched without regard to case).
std::string lower(const std::string& s);

}  // namespace json

#endif
