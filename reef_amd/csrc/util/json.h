// Minimal JSON reader for the model resource files.
// Accepts what the reference's parser accepts (src/reef/util/json.cpp: strings
// in " or ', integers, plain decimals, lists, dicts) and, as a superset, what
// standard JSON adds (true/false/null, exponents, escapes), so files written by
// either side load.  Parse errors are reported, not fatal.
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace reef {
namespace util {

class JsonValue {
public:
    enum Type { Null, Bool, Int, Float, String, List, Dict };
    Type type = Null;
    bool bval = false;
    int64_t ival = 0;
    double fval = 0.0;
    std::string sval;
    std::vector<std::unique_ptr<JsonValue>> lval;
    std::map<std::string, std::unique_ptr<JsonValue>> mval;

    bool has(const std::string& key) const { return type == Dict && mval.count(key) != 0; }
    const JsonValue* get(const std::string& key) const;  // nullptr when absent
    int64_t as_int() const { return type == Float ? (int64_t)fval : ival; }
};

// Returns nullptr and fills `err` on malformed input.
std::unique_ptr<JsonValue> parse_json(const std::string& text, std::string* err);
std::unique_ptr<JsonValue> parse_json_file(const char* path, std::string* err);

}  // namespace util
}  // namespace reef
