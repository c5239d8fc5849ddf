// A small JSON value with a parser and a writer: what config.json, safetensors headers,
// model descriptions and the structured arguments of the C API need.  Objects keep the
// order of their keys; a duplicate key is an error (safetensors forbids duplicate names).
#pragma once
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace celeg {

struct JsonError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

class Json {
public:
    enum Kind { Null, Bool, Int, Float, String, Array, Object };
    using Member = std::pair<std::string, Json>;

    Json() = default;
    Json(std::nullptr_t) {}
    Json(bool b) : kind_(Bool), b_(b) {}
    Json(int v) : kind_(Int), i_(v) {}
    Json(long v) : kind_(Int), i_(v) {}
    Json(long long v) : kind_(Int), i_(v) {}
    Json(unsigned v) : kind_(Int), i_(v) {}
    Json(unsigned long v) : kind_(Int), i_(static_cast<long long>(v)) {}
    Json(double v) : kind_(Float), f_(v) {}
    Json(const char* s) : kind_(String), s_(s) {}
    Json(std::string s) : kind_(String), s_(std::move(s)) {}
    static Json array() { Json j; j.kind_ = Array; return j; }
    static Json object() { Json j; j.kind_ = Object; return j; }
    template <typename T>
    static Json array_of(const std::vector<T>& values) {
        Json j = array();
        for (const auto& v : values) j.push(Json(v));
        return j;
    }

    Kind kind() const { return kind_; }
    bool is_null() const { return kind_ == Null; }
    bool is_bool() const { return kind_ == Bool; }
    bool is_int() const { return kind_ == Int; }
    bool is_number() const { return kind_ == Int || kind_ == Float; }
    bool is_string() const { return kind_ == String; }
    bool is_array() const { return kind_ == Array; }
    bool is_object() const { return kind_ == Object; }

    bool as_bool() const { need(Bool, "a boolean"); return b_; }
    long long as_int() const {
        if (kind_ == Float && std::floor(f_) == f_ && std::fabs(f_) < 9.0e18) return static_cast<long long>(f_);
        need(Int, "an integer");
        return i_;
    }
    double as_double() const {
        if (kind_ == Int) return static_cast<double>(i_);
        need(Float, "a number");
        return f_;
    }
    const std::string& as_string() const { need(String, "a string"); return s_; }
    const std::vector<Json>& items() const { need(Array, "an array"); return a_; }
    const std::vector<Member>& members() const { need(Object, "an object"); return o_; }

    size_t size() const { return kind_ == Array ? a_.size() : kind_ == Object ? o_.size() : 0; }
    const Json& operator[](size_t i) const { need(Array, "an array"); return a_.at(i); }
    const Json& operator[](int i) const { return (*this)[static_cast<size_t>(i)]; }
    // a member of an object, or a shared null value
    const Json& operator[](const std::string& key) const {
        static const Json null_value;
        if (kind_ != Object) return null_value;
        for (const auto& m : o_)
            if (m.first == key) return m.second;
        return null_value;
    }
    const Json& operator[](const char* key) const { return (*this)[std::string(key)]; }
    bool contains(const std::string& key) const {
        if (kind_ != Object) return false;
        for (const auto& m : o_)
            if (m.first == key) return true;
        return false;
    }
    void push(Json v) { need(Array, "an array"); a_.push_back(std::move(v)); }
    // sets or replaces a member
    Json& set(const std::string& key, Json v) {
        need(Object, "an object");
        for (auto& m : o_)
            if (m.first == key) { m.second = std::move(v); return *this; }
        o_.emplace_back(key, std::move(v));
        return *this;
    }
    void erase(const std::string& key) {
        need(Object, "an object");
        for (size_t i = 0; i < o_.size(); ++i)
            if (o_[i].first == key) { o_.erase(o_.begin() + static_cast<long>(i)); return; }
    }

    // typed reads with defaults, for parameters of parts
    long long get_int(const std::string& key, long long fallback) const {
        const Json& v = (*this)[key];
        return v.is_null() ? fallback : v.as_int();
    }
    double get_double(const std::string& key, double fallback) const {
        const Json& v = (*this)[key];
        return v.is_null() ? fallback : v.as_double();
    }
    bool get_bool(const std::string& key, bool fallback) const {
        const Json& v = (*this)[key];
        return v.is_null() ? fallback : v.as_bool();
    }
    std::string get_string(const std::string& key, const std::string& fallback) const {
        const Json& v = (*this)[key];
        return v.is_null() ? fallback : v.as_string();
    }

    bool operator==(const Json& other) const {
        if (is_number() && other.is_number()) return as_double() == other.as_double();
        if (kind_ != other.kind_) return false;
        switch (kind_) {
            case Null: return true;
            case Bool: return b_ == other.b_;
            case String: return s_ == other.s_;
            case Array: return a_ == other.a_;
            case Object: return o_ == other.o_;
            default: return false;
        }
    }
    bool operator!=(const Json& other) const { return !(*this == other); }

    static Json parse(const std::string& text) {
        Parser p{text.data(), text.data() + text.size()};
        p.skip();
        Json v = p.value(0);
        p.skip();
        if (p.at != p.end) p.fail("text after the value");
        return v;
    }

    std::string dump() const {
        std::string out;
        write(out);
        return out;
    }

private:
    Kind kind_ = Null;
    bool b_ = false;
    long long i_ = 0;
    double f_ = 0.0;
    std::string s_;
    std::vector<Json> a_;
    std::vector<Member> o_;

    void need(Kind k, const char* what) const {
        if (kind_ != k) throw JsonError(std::string("JSON value is not ") + what);
    }

    static void write_string(std::string& out, const std::string& s) {
        out.push_back('"');
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
                        std::snprintf(buf, sizeof buf, "\\u%04x", c);
                        out += buf;
                    } else {
                        out.push_back(static_cast<char>(c));
                    }
            }
        }
        out.push_back('"');
    }

    void write(std::string& out) const {
        switch (kind_) {
            case Null: out += "null"; break;
            case Bool: out += b_ ? "true" : "false"; break;
            case Int: out += std::to_string(i_); break;
            case Float: {
                if (!std::isfinite(f_)) { out += "null"; break; }
                char buf[40];
                std::snprintf(buf, sizeof buf, "%.17g", f_);
                out += buf;
                bool plain = true;
                for (const char* p = buf; *p; ++p)
                    if (*p == '.' || *p == 'e' || *p == 'E' || *p == 'n' || *p == 'i') plain = false;
                if (plain) out += ".0";
                break;
            }
            case String: write_string(out, s_); break;
            case Array:
                out.push_back('[');
                for (size_t i = 0; i < a_.size(); ++i) {
                    if (i) out.push_back(',');
                    a_[i].write(out);
                }
                out.push_back(']');
                break;
            case Object:
                out.push_back('{');
                for (size_t i = 0; i < o_.size(); ++i) {
                    if (i) out.push_back(',');
                    write_string(out, o_[i].first);
                    out.push_back(':');
                    o_[i].second.write(out);
                }
                out.push_back('}');
                break;
        }
    }

    struct Parser {
        const char* at;
        const char* end;
        const char* begin = at;

        [[noreturn]] void fail(const std::string& what) const {
            throw JsonError("invalid JSON at byte " + std::to_string(at - begin) + ": " + what);
        }
        void skip() {
            while (at != end && (*at == ' ' || *at == '\n' || *at == '\t' || *at == '\r')) ++at;
        }
        bool take(const char* word) {
            const char* p = at;
            for (const char* w = word; *w; ++w, ++p)
                if (p == end || *p != *w) return false;
            at = p;
            return true;
        }
        Json value(int depth) {
            if (depth > 200) fail("nested too deeply");
            if (at == end) fail("unexpected end");
            switch (*at) {
                case '{': return object(depth);
                case '[': return array(depth);
                case '"': return Json(string());
                case 't': if (take("true")) return Json(true); fail("unknown word");
                case 'f': if (take("false")) return Json(false); fail("unknown word");
                case 'n': if (take("null")) return Json(); fail("unknown word");
                // what Python's writer emits for non-finite floats
                case 'N': if (take("NaN")) return Json(std::nan("")); fail("unknown word");
                case 'I': if (take("Infinity")) return Json(HUGE_VAL); fail("unknown word");
                default: return number();
            }
        }
        Json number() {
            const char* start = at;
            if (at != end && *at == '-') {
                ++at;
                if (take("Infinity")) return Json(-HUGE_VAL);
            }
            bool integral = true;
            while (at != end && ((*at >= '0' && *at <= '9') || *at == '.' || *at == 'e' || *at == 'E' ||
                                 *at == '+' || *at == '-')) {
                if (*at == '.' || *at == 'e' || *at == 'E') integral = false;
                ++at;
            }
            if (at == start || (at - start == 1 && *start == '-')) fail("a value was expected");
            const std::string text(start, at);
            char* stop = nullptr;
            if (integral && text.size() < 19) {
                const long long v = std::strtoll(text.c_str(), &stop, 10);
                if (*stop) fail("malformed number");
                return Json(v);
            }
            const double v = std::strtod(text.c_str(), &stop);
            if (*stop) fail("malformed number");
            return Json(v);
        }
        static void utf8(std::string& out, unsigned cp) {
            if (cp < 0x80) out.push_back(static_cast<char>(cp));
            else if (cp < 0x800) { out.push_back(static_cast<char>(0xC0 | (cp >> 6))); out.push_back(static_cast<char>(0x80 | (cp & 0x3F))); }
            else if (cp < 0x10000) {
                out.push_back(static_cast<char>(0xE0 | (cp >> 12)));
                out.push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
                out.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
            } else {
                out.push_back(static_cast<char>(0xF0 | (cp >> 18)));
                out.push_back(static_cast<char>(0x80 | ((cp >> 12) & 0x3F)));
                out.push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
                out.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
            }
        }
        unsigned hex4() {
            unsigned v = 0;
            for (int i = 0; i < 4; ++i) {
                if (at == end) fail("unfinished escape");
                const char c = *at++;
                v <<= 4;
                if (c >= '0' && c <= '9') v |= static_cast<unsigned>(c - '0');
                else if (c >= 'a' && c <= 'f') v |= static_cast<unsigned>(c - 'a' + 10);
                else if (c >= 'A' && c <= 'F') v |= static_cast<unsigned>(c - 'A' + 10);
                else fail("malformed escape");
            }
            return v;
        }
        std::string string() {
            ++at;  // the opening quote
            std::string out;
            for (;;) {
                if (at == end) fail("unfinished string");
                const char c = *at++;
                if (c == '"') return out;
                if (c != '\\') { out.push_back(c); continue; }
                if (at == end) fail("unfinished escape");
                const char e = *at++;
                switch (e) {
                    case '"': out.push_back('"'); break;
                    case '\\': out.push_back('\\'); break;
                    case '/': out.push_back('/'); break;
                    case 'b': out.push_back('\b'); break;
                    case 'f': out.push_back('\f'); break;
                    case 'n': out.push_back('\n'); break;
                    case 'r': out.push_back('\r'); break;
                    case 't': out.push_back('\t'); break;
                    case 'u': {
                        unsigned cp = hex4();
                        if (cp >= 0xD800 && cp < 0xDC00 && at + 1 < end && at[0] == '\\' && at[1] == 'u') {
                            at += 2;
                            const unsigned low = hex4();
                            cp = 0x10000 + ((cp - 0xD800) << 10) + (low - 0xDC00);
                        }
                        utf8(out, cp);
                        break;
                    }
                    default: fail("unknown escape");
                }
            }
        }
        Json array(int depth) {
            ++at;
            Json out = Json::array();
            skip();
            if (at != end && *at == ']') { ++at; return out; }
            for (;;) {
                skip();
                out.push(value(depth + 1));
                skip();
                if (at == end) fail("unfinished array");
                if (*at == ',') { ++at; continue; }
                if (*at == ']') { ++at; return out; }
                fail("',' or ']' was expected");
            }
        }
        Json object(int depth) {
            ++at;
            Json out = Json::object();
            skip();
            if (at != end && *at == '}') { ++at; return out; }
            for (;;) {
                skip();
                if (at == end || *at != '"') fail("a member name was expected");
                std::string key = string();
                skip();
                if (at == end || *at != ':') fail("':' was expected");
                ++at;
                skip();
                if (out.contains(key)) throw JsonError("duplicate name: " + key);
                Json v = value(depth + 1);
                out.o_.emplace_back(std::move(key), std::move(v));
                skip();
                if (at == end) fail("unfinished object");
                if (*at == ',') { ++at; continue; }
                if (*at == '}') { ++at; return out; }
                fail("',' or '}' was expected");
            }
        }
    };
};

}  // namespace celeg
