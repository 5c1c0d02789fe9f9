// A small JSON value for network descriptions and weight-file headers.
//
// dlprimitives reads its network format (docs/network_json_format.md) and the header of its
// DLPW weight files through dlprim::json::value (include/dlprim/json.hpp, src/json.cpp); this is
// an independent implementation of the part the network loader needs: parse, typed access with
// defaults (`get<T>(key, default)`), arrays, objects (insertion-ordered), and serialisation.
#pragma once
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <istream>
#include <map>
#include <memory>
#include <sstream>
#include <string>
#include <utility>
#include <vector>

#include "definitions.hpp"

namespace dlprim {
namespace json {

enum json_type { is_undefined, is_null, is_boolean, is_number, is_string, is_array, is_object };

class value;
typedef std::vector<value> array;
// objects keep the order of their keys (a weight file lists its tensors in file order)
typedef std::vector<std::pair<std::string, value>> object;

class value {
public:
    value() {}
    value(std::nullptr_t) : type_(json::is_null) {}
    value(bool b) : type_(is_boolean), num_(b ? 1.0 : 0.0) {}
    value(int v) : type_(is_number), num_(v) {}
    value(long long v) : type_(is_number), num_((double)v) {}
    value(size_t v) : type_(is_number), num_((double)v) {}
    value(double v) : type_(is_number), num_(v) {}
    value(float v) : type_(is_number), num_(v) {}
    value(char const *s) : type_(is_string), str_(s) {}
    value(std::string const &s) : type_(is_string), str_(s) {}
    value(json::array const &a) : type_(is_array), arr_(std::make_shared<json::array>(a)) {}
    value(json::object const &o) : type_(is_object), obj_(std::make_shared<json::object>(o)) {}

    json_type type() const { return type_; }
    bool is_undefined() const { return type_ == json::is_undefined; }
    bool is_null() const { return type_ == json::is_null; }

    bool boolean() const
    {
        if (type_ == is_boolean || type_ == is_number) // the reference's files use 0 / 1 for flags as well
            return num_ != 0.0;
        throw ValidationError("json: not a boolean");
    }
    double number() const
    {
        if (type_ != is_number && type_ != is_boolean)
            throw ValidationError("json: not a number");
        return num_;
    }
    std::string const &str() const
    {
        if (type_ != is_string)
            throw ValidationError("json: not a string");
        return str_;
    }
    json::array const &array() const
    {
        if (type_ != is_array)
            throw ValidationError("json: not an array");
        return *arr_;
    }
    json::array &array()
    {
        if (type_ == json::is_undefined) {
            type_ = is_array;
            arr_ = std::make_shared<json::array>();
        }
        if (type_ != is_array)
            throw ValidationError("json: not an array");
        return *arr_;
    }
    json::object const &object() const
    {
        if (type_ != is_object)
            throw ValidationError("json: not an object");
        return *obj_;
    }
    json::object &object()
    {
        if (type_ == json::is_undefined) {
            type_ = is_object;
            obj_ = std::make_shared<json::object>();
        }
        if (type_ != is_object)
            throw ValidationError("json: not an object");
        return *obj_;
    }

    // member of an object, or an undefined value
    value const &find(std::string const &key) const
    {
        static const value undefined;
        if (type_ != is_object)
            return undefined;
        for (auto const &kv : *obj_)
            if (kv.first == key)
                return kv.second;
        return undefined;
    }
    value const &operator[](std::string const &key) const
    {
        value const &v = find(key);
        if (v.is_undefined())
            throw ValidationError("json: no member '" + key + "'");
        return v;
    }
    value &operator[](std::string const &key)
    {
        json::object &o = object();
        for (auto &kv : o)
            if (kv.first == key)
                return kv.second;
        o.push_back(std::make_pair(key, value()));
        return o.back().second;
    }
    value const &operator[](size_t i) const { return array().at(i); }
    value &operator[](size_t i)
    {
        json::array &a = array();
        if (a.size() <= i)
            a.resize(i + 1);
        return a[i];
    }
    size_t size() const { return type_ == is_array ? arr_->size() : type_ == is_object ? obj_->size() : 0; }

    template <typename T>
    T get_value() const;
    // typed member access: throws when the member is missing / returns the default
    template <typename T>
    T get(std::string const &key) const
    {
        return (*this)[key].template get_value<T>();
    }
    template <typename T>
    T get(std::string const &key, T const &def) const
    {
        value const &v = find(key);
        return v.is_undefined() ? def : v.template get_value<T>();
    }
    std::string get(std::string const &key, char const *def) const
    {
        value const &v = find(key);
        return v.is_undefined() ? std::string(def) : v.str();
    }

    // ---- text ----
    std::string save() const
    {
        std::string out;
        write(out);
        return out;
    }
    static value parse(std::string const &text)
    {
        size_t pos = 0;
        value v = parse_value(text, pos);
        skip_space(text, pos);
        if (pos != text.size())
            fail(text, pos, "trailing characters");
        return v;
    }
    static value load(std::istream &in)
    {
        std::ostringstream ss;
        ss << in.rdbuf();
        return parse(ss.str());
    }

private:
    static void fail(std::string const &t, size_t pos, char const *what)
    {
        size_t line = 1;
        for (size_t i = 0; i < pos && i < t.size(); i++)
            if (t[i] == '\n')
                line++;
        throw ValidationError(std::string("json: ") + what + " at line " + std::to_string(line));
    }
    static void skip_space(std::string const &t, size_t &pos)
    {
        while (pos < t.size() && (t[pos] == ' ' || t[pos] == '\t' || t[pos] == '\n' || t[pos] == '\r'))
            pos++;
    }
    static void append_utf8(std::string &s, unsigned cp)
    {
        if (cp < 0x80)
            s += (char)cp;
        else if (cp < 0x800) {
            s += (char)(0xC0 | (cp >> 6));
            s += (char)(0x80 | (cp & 0x3F));
        } else if (cp < 0x10000) {
            s += (char)(0xE0 | (cp >> 12));
            s += (char)(0x80 | ((cp >> 6) & 0x3F));
            s += (char)(0x80 | (cp & 0x3F));
        } else {
            s += (char)(0xF0 | (cp >> 18));
            s += (char)(0x80 | ((cp >> 12) & 0x3F));
            s += (char)(0x80 | ((cp >> 6) & 0x3F));
            s += (char)(0x80 | (cp & 0x3F));
        }
    }
    static unsigned parse_hex4(std::string const &t, size_t &pos)
    {
        if (pos + 4 > t.size())
            fail(t, pos, "short \\u escape");
        unsigned v = 0;
        for (int i = 0; i < 4; i++) {
            char c = t[pos++];
            v <<= 4;
            if (c >= '0' && c <= '9')
                v |= (unsigned)(c - '0');
            else if (c >= 'a' && c <= 'f')
                v |= (unsigned)(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F')
                v |= (unsigned)(c - 'A' + 10);
            else
                fail(t, pos, "bad \\u escape");
        }
        return v;
    }
    static std::string parse_string(std::string const &t, size_t &pos)
    {
        std::string s;
        pos++; // opening quote
        while (true) {
            if (pos >= t.size())
                fail(t, pos, "unterminated string");
            char c = t[pos++];
            if (c == '"')
                return s;
            if (c != '\\') {
                s += c;
                continue;
            }
            if (pos >= t.size())
                fail(t, pos, "unterminated escape");
            char e = t[pos++];
            switch (e) {
            case '"': s += '"'; break;
            case '\\': s += '\\'; break;
            case '/': s += '/'; break;
            case 'b': s += '\b'; break;
            case 'f': s += '\f'; break;
            case 'n': s += '\n'; break;
            case 'r': s += '\r'; break;
            case 't': s += '\t'; break;
            case 'u': {
                unsigned cp = parse_hex4(t, pos);
                if (cp >= 0xD800 && cp < 0xDC00) { // a high surrogate must be followed by a low one (the reference's utf16 decoder, src/json.cpp:215-229)
                    if (!(pos + 1 < t.size() && t[pos] == '\\' && t[pos + 1] == 'u'))
                        fail(t, pos, "unpaired surrogate");
                    pos += 2;
                    unsigned lo = parse_hex4(t, pos);
                    if (lo < 0xDC00 || lo > 0xDFFF)
                        fail(t, pos, "unpaired surrogate");
                    cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                } else if (cp >= 0xDC00 && cp <= 0xDFFF)
                    fail(t, pos, "unpaired surrogate");
                append_utf8(s, cp);
                break;
            }
            default: fail(t, pos, "bad escape");
            }
        }
    }
    static value parse_value(std::string const &t, size_t &pos)
    {
        skip_space(t, pos);
        if (pos >= t.size())
            fail(t, pos, "unexpected end");
        char c = t[pos];
        if (c == '{') {
            value v;
            json::object &o = v.object();
            pos++;
            skip_space(t, pos);
            if (pos < t.size() && t[pos] == '}') {
                pos++;
                return v;
            }
            while (true) {
                skip_space(t, pos);
                if (pos >= t.size() || t[pos] != '"')
                    fail(t, pos, "member name expected");
                std::string key = parse_string(t, pos);
                skip_space(t, pos);
                if (pos >= t.size() || t[pos] != ':')
                    fail(t, pos, "':' expected");
                pos++;
                o.push_back(std::make_pair(key, parse_value(t, pos)));
                skip_space(t, pos);
                if (pos < t.size() && t[pos] == ',') {
                    pos++;
                    continue;
                }
                if (pos < t.size() && t[pos] == '}') {
                    pos++;
                    return v;
                }
                fail(t, pos, "',' or '}' expected");
            }
        }
        if (c == '[') {
            value v;
            json::array &a = v.array();
            pos++;
            skip_space(t, pos);
            if (pos < t.size() && t[pos] == ']') {
                pos++;
                return v;
            }
            while (true) {
                a.push_back(parse_value(t, pos));
                skip_space(t, pos);
                if (pos < t.size() && t[pos] == ',') {
                    pos++;
                    continue;
                }
                if (pos < t.size() && t[pos] == ']') {
                    pos++;
                    return v;
                }
                fail(t, pos, "',' or ']' expected");
            }
        }
        if (c == '"')
            return value(parse_string(t, pos));
        if (t.compare(pos, 4, "true") == 0) {
            pos += 4;
            return value(true);
        }
        if (t.compare(pos, 5, "false") == 0) {
            pos += 5;
            return value(false);
        }
        if (t.compare(pos, 4, "null") == 0) {
            pos += 4;
            return value(nullptr);
        }
        if (c == '-' || (c >= '0' && c <= '9')) {
            char const *begin = t.c_str() + pos;
            char *end = nullptr;
            double d = std::strtod(begin, &end);
            if (end == begin)
                fail(t, pos, "bad number");
            pos += (size_t)(end - begin);
            return value(d);
        }
        fail(t, pos, "unexpected character");
        return value();
    }
    static void write_string(std::string &out, std::string const &s)
    {
        out += '"';
        for (unsigned char c : s) {
            switch (c) {
            case '"': out += "\\\""; break;
            case '\\': out += "\\\\"; break;
            case '\n': out += "\\n"; break;
            case '\r': out += "\\r"; break;
            case '\t': out += "\\t"; break;
            default:
                if (c < 0x20) {
                    char buf[8];
                    std::snprintf(buf, sizeof(buf), "\\u%04x", c);
                    out += buf;
                } else
                    out += (char)c;
            }
        }
        out += '"';
    }
    void write(std::string &out) const
    {
        switch (type_) {
        case json::is_undefined:
        case json::is_null: out += "null"; break;
        case is_boolean: out += num_ != 0.0 ? "true" : "false"; break;
        case is_number: {
            char buf[40];
            if (num_ == std::floor(num_) && std::fabs(num_) < 1e15)
                std::snprintf(buf, sizeof(buf), "%lld", (long long)num_);
            else
                std::snprintf(buf, sizeof(buf), "%.17g", num_);
            out += buf;
            break;
        }
        case is_string: write_string(out, str_); break;
        case is_array: {
            out += '[';
            bool first = true;
            for (auto const &v : *arr_) {
                if (!first)
                    out += ',';
                first = false;
                v.write(out);
            }
            out += ']';
            break;
        }
        case is_object: {
            out += '{';
            bool first = true;
            for (auto const &kv : *obj_) {
                if (!first)
                    out += ',';
                first = false;
                write_string(out, kv.first);
                out += ':';
                kv.second.write(out);
            }
            out += '}';
            break;
        }
        }
    }

    json_type type_ = json::is_undefined;
    double num_ = 0.0;
    std::string str_;
    std::shared_ptr<json::array> arr_;
    std::shared_ptr<json::object> obj_;
};

template <>
inline bool value::get_value<bool>() const
{
    return boolean();
}
template <>
inline int value::get_value<int>() const
{
    return (int)number();
}
template <>
inline long long value::get_value<long long>() const
{
    return (long long)number();
}
template <>
inline size_t value::get_value<size_t>() const
{
    return (size_t)number();
}
template <>
inline float value::get_value<float>() const
{
    return (float)number();
}
template <>
inline double value::get_value<double>() const
{
    return number();
}
template <>
inline std::string value::get_value<std::string>() const
{
    return str();
}
template <>
inline std::vector<int> value::get_value<std::vector<int>>() const
{
    std::vector<int> r;
    for (auto const &v : array())
        r.push_back((int)v.number());
    return r;
}
template <>
inline std::vector<std::string> value::get_value<std::vector<std::string>>() const
{
    std::vector<std::string> r;
    for (auto const &v : array())
        r.push_back(v.str());
    return r;
}

} // namespace json
} // namespace dlprim
