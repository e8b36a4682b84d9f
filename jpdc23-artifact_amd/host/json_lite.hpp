// Reader for the per-algorithm argument files: one flat JSON object whose values are
// numbers, strings or booleans (what benchmark/benchmark.py:112-153 writes and the
// reference reads with nlohmann's args.value(key, default), e.g. one_to_one.hpp:739-741).
#pragma once

#include <cctype>
#include <cstdlib>
#include <istream>
#include <map>
#include <sstream>
#include <stdexcept>
#include <string>

namespace cross {

class json_args {
public:
    enum class kind { number, string, boolean, null };
    struct entry {
        kind k;
        double number;
        std::string text;
        bool flag;
    };

    json_args() = default;

    static json_args parse(std::istream &in) {
        std::stringstream ss;
        ss << in.rdbuf();
        return parse(ss.str());
    }

    static json_args parse(const std::string &text) {
        json_args out;
        std::size_t i = 0;
        skip_ws(text, i);
        if (i >= text.size()) return out; // empty file = no arguments
        expect(text, i, '{');
        skip_ws(text, i);
        if (peek(text, i) == '}') {
            ++i;
        } else {
            for (;;) {
                skip_ws(text, i);
                std::string key = parse_string(text, i);
                skip_ws(text, i);
                expect(text, i, ':');
                skip_ws(text, i);
                out.values_[key] = parse_value(text, i);
                skip_ws(text, i);
                char c = peek(text, i);
                ++i;
                if (c == ',') continue;
                if (c == '}') break;
                throw std::runtime_error("JSON arguments: expected ',' or '}' at offset " + std::to_string(i - 1));
            }
        }
        skip_ws(text, i);
        if (i != text.size()) throw std::runtime_error("JSON arguments: trailing characters after the object");
        return out;
    }

    bool contains(const std::string &key) const { return values_.count(key) != 0; }

    // args.value(key, default) for the three value types the algorithms read
    long long value(const std::string &key, long long def) const {
        auto it = values_.find(key);
        if (it == values_.end()) return def;
        if (it->second.k == kind::number) return static_cast<long long>(it->second.number);
        if (it->second.k == kind::boolean) return it->second.flag ? 1 : 0;
        throw std::runtime_error("JSON arguments: \"" + key + "\" must be a number");
    }
    unsigned value(const std::string &key, unsigned def) const {
        long long v = value(key, static_cast<long long>(def));
        if (v < 0) throw std::runtime_error("JSON arguments: \"" + key + "\" must not be negative");
        return static_cast<unsigned>(v);
    }
    unsigned value(const std::string &key, int def) const { return value(key, static_cast<unsigned>(def)); }
    bool value(const std::string &key, bool def) const {
        auto it = values_.find(key);
        if (it == values_.end()) return def;
        if (it->second.k == kind::boolean) return it->second.flag;
        if (it->second.k == kind::number) return it->second.number != 0;
        throw std::runtime_error("JSON arguments: \"" + key + "\" must be a boolean");
    }
    std::string value(const std::string &key, const char *def) const {
        auto it = values_.find(key);
        if (it == values_.end()) return def;
        if (it->second.k == kind::string) return it->second.text;
        throw std::runtime_error("JSON arguments: \"" + key + "\" must be a string");
    }

private:
    std::map<std::string, entry> values_;

    static char peek(const std::string &t, std::size_t i) {
        if (i >= t.size()) throw std::runtime_error("JSON arguments: unexpected end of input");
        return t[i];
    }
    static void skip_ws(const std::string &t, std::size_t &i) {
        while (i < t.size() && std::isspace(static_cast<unsigned char>(t[i]))) ++i;
    }
    static void expect(const std::string &t, std::size_t &i, char c) {
        if (peek(t, i) != c) throw std::runtime_error(std::string("JSON arguments: expected '") + c + "' at offset " + std::to_string(i));
        ++i;
    }
    static std::string parse_string(const std::string &t, std::size_t &i) {
        expect(t, i, '"');
        std::string out;
        for (;;) {
            char c = peek(t, i++);
            if (c == '"') break;
            if (c == '\\') {
                char e = peek(t, i++);
                switch (e) {
                case 'n': out += '\n'; break;
                case 't': out += '\t'; break;
                case 'r': out += '\r'; break;
                case 'b': out += '\b'; break;
                case 'f': out += '\f'; break;
                case 'u': throw std::runtime_error("JSON arguments: \\u escapes are not supported");
                default: out += e; break;
                }
            } else {
                out += c;
            }
        }
        return out;
    }
    static entry parse_value(const std::string &t, std::size_t &i) {
        char c = peek(t, i);
        entry e{kind::null, 0.0, "", false};
        if (c == '"') {
            e.k = kind::string;
            e.text = parse_string(t, i);
        } else if (t.compare(i, 4, "true") == 0) {
            e.k = kind::boolean;
            e.flag = true;
            i += 4;
        } else if (t.compare(i, 5, "false") == 0) {
            e.k = kind::boolean;
            i += 5;
        } else if (t.compare(i, 4, "null") == 0) {
            i += 4;
        } else if (c == '-' || std::isdigit(static_cast<unsigned char>(c))) {
            const char *begin = t.c_str() + i;
            char *end = nullptr;
            e.k = kind::number;
            e.number = std::strtod(begin, &end);
            if (end == begin) throw std::runtime_error("JSON arguments: bad number at offset " + std::to_string(i));
            i += static_cast<std::size_t>(end - begin);
        } else {
            throw std::runtime_error("JSON arguments: only numbers, strings and booleans are supported (offset " + std::to_string(i) + ")");
        }
        return e;
    }
};

} // namespace cross
