#include "util/json.h"

#include <cstdlib>
#include <fstream>
#include <sstream>

namespace reef {
namespace util {

const JsonValue* JsonValue::get(const std::string& key) const {
    if (type != Dict) return nullptr;
    auto it = mval.find(key);
    return it == mval.end() ? nullptr : it->second.get();
}

namespace {

struct Cursor {
    const std::string& s;
    size_t p = 0;
    std::string err;
    explicit Cursor(const std::string& str) : s(str) {}

    void skip_ws() {
        while (p < s.size() && (s[p] == ' ' || s[p] == '\n' || s[p] == '\t' || s[p] == '\r')) ++p;
    }
    bool fail(const std::string& what) {
        if (err.empty()) err = what + " at offset " + std::to_string(p);
        return false;
    }

    bool parse_string(std::string& out) {
        const char q = s[p++];
        out.clear();
        while (p < s.size() && s[p] != q) {
            char c = s[p++];
            if (c == '\\' && p < s.size()) {
                char e = s[p++];
                switch (e) {
                    case 'n': out += '\n'; break;
                    case 't': out += '\t'; break;
                    case 'r': out += '\r'; break;
                    case 'b': out += '\b'; break;
                    case 'f': out += '\f'; break;
                    case 'u':  // keep the escape verbatim: names here are ASCII
                        out += "\\u";
                        break;
                    default: out += e; break;
                }
            } else {
                out += c;
            }
        }
        if (p >= s.size()) return fail("unterminated string");
        ++p;
        return true;
    }

    bool parse_number(JsonValue& v) {
        const size_t b = p;
        bool is_float = false;
        if (s[p] == '-' || s[p] == '+') ++p;
        while (p < s.size()) {
            char c = s[p];
            if (c >= '0' && c <= '9') { ++p; continue; }
            if (c == '.' || c == 'e' || c == 'E') { is_float = true; ++p; continue; }
            if ((c == '-' || c == '+') && (s[p - 1] == 'e' || s[p - 1] == 'E')) { ++p; continue; }
            break;
        }
        if (p == b) return fail("bad number");
        const std::string tok = s.substr(b, p - b);
        if (is_float) {
            v.type = JsonValue::Float;
            v.fval = std::strtod(tok.c_str(), nullptr);
            v.ival = (int64_t)v.fval;
        } else {
            v.type = JsonValue::Int;
            v.ival = std::strtoll(tok.c_str(), nullptr, 10);
            v.fval = (double)v.ival;
        }
        return true;
    }

    bool parse_value(JsonValue& v, int depth) {
        if (depth > 64) return fail("nesting too deep");
        skip_ws();
        if (p >= s.size()) return fail("unexpected end");
        const char c = s[p];
        if (c == '{') {
            ++p;
            v.type = JsonValue::Dict;
            skip_ws();
            while (p < s.size() && s[p] != '}') {
                skip_ws();
                if (p >= s.size() || (s[p] != '"' && s[p] != '\'')) return fail("expected key");
                std::string key;
                if (!parse_string(key)) return false;
                skip_ws();
                if (p >= s.size() || s[p] != ':') return fail("expected ':'");
                ++p;
                std::unique_ptr<JsonValue> child(new JsonValue);
                if (!parse_value(*child, depth + 1)) return false;
                v.mval[key] = std::move(child);
                skip_ws();
                if (p < s.size() && s[p] == ',') ++p;
                skip_ws();
            }
            if (p >= s.size()) return fail("unterminated object");
            ++p;
            return true;
        }
        if (c == '[') {
            ++p;
            v.type = JsonValue::List;
            skip_ws();
            while (p < s.size() && s[p] != ']') {
                std::unique_ptr<JsonValue> child(new JsonValue);
                if (!parse_value(*child, depth + 1)) return false;
                v.lval.push_back(std::move(child));
                skip_ws();
                if (p < s.size() && s[p] == ',') ++p;
                skip_ws();
            }
            if (p >= s.size()) return fail("unterminated list");
            ++p;
            return true;
        }
        if (c == '"' || c == '\'') {
            v.type = JsonValue::String;
            return parse_string(v.sval);
        }
        if (c == '-' || c == '+' || (c >= '0' && c <= '9')) return parse_number(v);
        if (s.compare(p, 4, "true") == 0) { v.type = JsonValue::Bool; v.bval = true; v.ival = 1; p += 4; return true; }
        if (s.compare(p, 5, "false") == 0) { v.type = JsonValue::Bool; p += 5; return true; }
        if (s.compare(p, 4, "null") == 0) { v.type = JsonValue::Null; p += 4; return true; }
        return fail("unrecognizable token");
    }
};

}  // namespace

std::unique_ptr<JsonValue> parse_json(const std::string& text, std::string* err) {
    Cursor c(text);
    std::unique_ptr<JsonValue> root(new JsonValue);
    if (!c.parse_value(*root, 0)) {
        if (err) *err = c.err;
        return nullptr;
    }
    c.skip_ws();
    if (c.p != text.size()) {
        if (err) *err = "trailing characters at offset " + std::to_string(c.p);
        return nullptr;
    }
    return root;
}

std::unique_ptr<JsonValue> parse_json_file(const char* path, std::string* err) {
    std::ifstream fs(path, std::ios::binary);
    if (!fs) {
        if (err) *err = std::string("cannot open ") + path;
        return nullptr;
    }
    std::stringstream ss;
    ss << fs.rdbuf();
    return parse_json(ss.str(), err);
}

}  // namespace util
}  // namespace reef
