// Minimal JSON reader for the index / search parameter strings (objects, arrays, strings, numbers, booleans,
// null).  The reference parses the same strings with nlohmann::json (src/json_wrapper.*); only what the
// brute_force / ivf parameter contract needs is implemented here.
#pragma once

#include <cstdlib>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace vsag_host {

class Json {
public:
    enum class Type { Null, Bool, Number, String, Object, Array };

    Type type = Type::Null;
    bool boolean = false;
    double number = 0.0;
    bool is_integer = false;
    std::string string;
    std::vector<std::pair<std::string, Json>> members;  // insertion order kept
    std::vector<Json> elements;

    static Json
    Parse(const std::string& text) {
        size_t pos = 0;
        Json value = parse_value(text, pos);
        skip_space(text, pos);
        if (pos != text.size()) {
            throw std::invalid_argument("trailing characters after JSON value");
        }
        return value;
    }

    bool
    IsObject() const {
        return type == Type::Object;
    }
    bool
    Contains(const std::string& key) const {
        return find(key) != nullptr;
    }
    const Json&
    operator[](const std::string& key) const {
        const Json* v = find(key);
        if (v == nullptr) {
            throw std::invalid_argument("missing key: " + key);
        }
        return *v;
    }
    const Json*
    find(const std::string& key) const {
        for (const auto& m : members) {
            if (m.first == key) {
                return &m.second;
            }
        }
        return nullptr;
    }
    int64_t
    GetInt() const {
        if (type != Type::Number) {
            throw std::invalid_argument("expected a number");
        }
        return static_cast<int64_t>(number);
    }
    bool
    IsNumberInteger() const {
        return type == Type::Number && number == static_cast<double>(static_cast<int64_t>(number));
    }
    double
    GetFloat() const {
        if (type != Type::Number) {
            throw std::invalid_argument("expected a number");
        }
        return number;
    }
    bool
    GetBool() const {
        if (type != Type::Bool) {
            throw std::invalid_argument("expected a boolean");
        }
        return boolean;
    }
    const std::string&
    GetString() const {
        if (type != Type::String) {
            throw std::invalid_argument("expected a string");
        }
        return string;
    }

private:
    static void
    skip_space(const std::string& s, size_t& p) {
        while (p < s.size() && (s[p] == ' ' || s[p] == '\t' || s[p] == '\n' || s[p] == '\r')) {
            ++p;
        }
    }

    static Json
    parse_value(const std::string& s, size_t& p) {
        skip_space(s, p);
        if (p >= s.size()) {
            throw std::invalid_argument("unexpected end of JSON");
        }
        char c = s[p];
        if (c == '{') {
            return parse_object(s, p);
        }
        if (c == '[') {
            return parse_array(s, p);
        }
        if (c == '"') {
            Json v;
            v.type = Type::String;
            v.string = parse_string(s, p);
            return v;
        }
        if (s.compare(p, 4, "true") == 0) {
            p += 4;
            Json v;
            v.type = Type::Bool;
            v.boolean = true;
            return v;
        }
        if (s.compare(p, 5, "false") == 0) {
            p += 5;
            Json v;
            v.type = Type::Bool;
            return v;
        }
        if (s.compare(p, 4, "null") == 0) {
            p += 4;
            return Json();
        }
        return parse_number(s, p);
    }

    static Json
    parse_number(const std::string& s, size_t& p) {
        size_t start = p;
        bool integer = true;
        if (p < s.size() && (s[p] == '-' || s[p] == '+')) {
            ++p;
        }
        while (p < s.size() && ((s[p] >= '0' && s[p] <= '9') || s[p] == '.' || s[p] == 'e' || s[p] == 'E' ||
                                s[p] == '-' || s[p] == '+')) {
            if (s[p] == '.' || s[p] == 'e' || s[p] == 'E') {
                integer = false;
            }
            ++p;
        }
        if (p == start) {
            throw std::invalid_argument("invalid JSON value at offset " + std::to_string(start));
        }
        std::string tok = s.substr(start, p - start);
        char* end = nullptr;
        double value = std::strtod(tok.c_str(), &end);
        if (end == nullptr || *end != '\0') {
            throw std::invalid_argument("invalid number: " + tok);
        }
        Json v;
        v.type = Type::Number;
        v.number = value;
        v.is_integer = integer;
        return v;
    }

    static std::string
    parse_string(const std::string& s, size_t& p) {
        ++p;  // opening quote
        std::string out;
        while (p < s.size() && s[p] != '"') {
            if (s[p] == '\\') {
                ++p;
                if (p >= s.size()) {
                    break;
                }
                switch (s[p]) {
                    case 'n':
                        out.push_back('\n');
                        break;
                    case 't':
                        out.push_back('\t');
                        break;
                    case 'r':
                        out.push_back('\r');
                        break;
                    case 'b':
                        out.push_back('\b');
                        break;
                    case 'f':
                        out.push_back('\f');
                        break;
                    case 'u': {
                        if (p + 4 >= s.size()) {
                            throw std::invalid_argument("truncated \\u escape");
                        }
                        unsigned code = static_cast<unsigned>(std::strtoul(s.substr(p + 1, 4).c_str(), nullptr, 16));
                        p += 4;
                        if (code < 0x80) {
                            out.push_back(static_cast<char>(code));
                        } else if (code < 0x800) {
                            out.push_back(static_cast<char>(0xC0 | (code >> 6)));
                            out.push_back(static_cast<char>(0x80 | (code & 0x3F)));
                        } else {
                            out.push_back(static_cast<char>(0xE0 | (code >> 12)));
                            out.push_back(static_cast<char>(0x80 | ((code >> 6) & 0x3F)));
                            out.push_back(static_cast<char>(0x80 | (code & 0x3F)));
                        }
                        break;
                    }
                    default:
                        out.push_back(s[p]);
                }
                ++p;
            } else {
                out.push_back(s[p++]);
            }
        }
        if (p >= s.size()) {
            throw std::invalid_argument("unterminated string");
        }
        ++p;  // closing quote
        return out;
    }

    static Json
    parse_object(const std::string& s, size_t& p) {
        Json v;
        v.type = Type::Object;
        ++p;
        skip_space(s, p);
        if (p < s.size() && s[p] == '}') {
            ++p;
            return v;
        }
        while (true) {
            skip_space(s, p);
            if (p >= s.size() || s[p] != '"') {
                throw std::invalid_argument("expected a key string at offset " + std::to_string(p));
            }
            std::string key = parse_string(s, p);
            skip_space(s, p);
            if (p >= s.size() || s[p] != ':') {
                throw std::invalid_argument("expected ':' after key " + key);
            }
            ++p;
            Json value = parse_value(s, p);
            bool replaced = false;
            for (auto& m : v.members) {
                if (m.first == key) {
                    m.second = value;
                    replaced = true;
                }
            }
            if (!replaced) {
                v.members.emplace_back(key, value);
            }
            skip_space(s, p);
            if (p < s.size() && s[p] == ',') {
                ++p;
                continue;
            }
            if (p < s.size() && s[p] == '}') {
                ++p;
                return v;
            }
            throw std::invalid_argument("expected ',' or '}' at offset " + std::to_string(p));
        }
    }

    static Json
    parse_array(const std::string& s, size_t& p) {
        Json v;
        v.type = Type::Array;
        ++p;
        skip_space(s, p);
        if (p < s.size() && s[p] == ']') {
            ++p;
            return v;
        }
        while (true) {
            v.elements.push_back(parse_value(s, p));
            skip_space(s, p);
            if (p < s.size() && s[p] == ',') {
                ++p;
                continue;
            }
            if (p < s.size() && s[p] == ']') {
                ++p;
                return v;
            }
            throw std::invalid_argument("expected ',' or ']' at offset " + std::to_string(p));
        }
    }
};

}  // namespace vsag_host
