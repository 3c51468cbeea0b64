// A small JSON value type, enough for the encoding and network configurations. The reference configures its
// encodings through nlohmann::json (include/encodings/encoding.h:25, include/common/io.h:41-79); this class
// offers the part of that interface the configuration code uses: contains, operator[], value(key, default),
// get<T>, is_string, items, parse (with // and /* */ comments skipped, as the reference asks of its parser).
#pragma once

#include <cctype>
#include <cstdint>
#include <cstdlib>
#include <map>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

namespace tnn {

class Json {
  public:
    enum class Kind { Null, Bool, Int, Float, String, Object, Array };
    using object_t = std::map<std::string, Json>;
    using array_t = std::vector<Json>;

    Json() = default;
    Json(std::nullptr_t) {}
    Json(bool b) : kind_(Kind::Bool), int_(b) {}
    Json(const char *s) : kind_(Kind::String), str_(s) {}
    Json(const std::string &s) : kind_(Kind::String), str_(s) {}
    template <typename N, typename std::enable_if<std::is_integral<N>::value && !std::is_same<N, bool>::value, int>::type = 0>
    Json(N v) : kind_(Kind::Int), int_((int64_t)v) {}
    template <typename N, typename std::enable_if<std::is_floating_point<N>::value, int>::type = 0>
    Json(N v) : kind_(Kind::Float), num_((double)v) {}
    template <typename E, typename std::enable_if<std::is_enum<E>::value, int>::type = 0>
    Json(E v) : kind_(Kind::Int), int_((int64_t)v) {}
    Json(std::initializer_list<std::pair<const std::string, Json>> init) : kind_(Kind::Object), obj_(init) {}

    static Json object() {
        Json j;
        j.kind_ = Kind::Object;
        return j;
    }
    static Json array() {
        Json j;
        j.kind_ = Kind::Array;
        return j;
    }

    Kind kind() const { return kind_; }
    bool is_null() const { return kind_ == Kind::Null; }
    bool is_boolean() const { return kind_ == Kind::Bool; }
    bool is_number() const { return kind_ == Kind::Int || kind_ == Kind::Float; }
    bool is_number_integer() const { return kind_ == Kind::Int; }
    bool is_string() const { return kind_ == Kind::String; }
    bool is_object() const { return kind_ == Kind::Object; }
    bool is_array() const { return kind_ == Kind::Array; }

    bool contains(const std::string &key) const { return kind_ == Kind::Object && obj_.count(key) != 0; }
    size_t size() const { return kind_ == Kind::Object ? obj_.size() : kind_ == Kind::Array ? arr_.size() : (kind_ == Kind::Null ? 0 : 1); }

    const Json &operator[](const std::string &key) const {
        if (kind_ != Kind::Object) throw std::invalid_argument("json: not an object");
        const auto it = obj_.find(key);
        if (it == obj_.end()) throw std::out_of_range("json: key '" + key + "' not found");
        return it->second;
    }
    Json &operator[](const std::string &key) {
        if (kind_ == Kind::Null) kind_ = Kind::Object;
        if (kind_ != Kind::Object) throw std::invalid_argument("json: not an object");
        return obj_[key];
    }
    const Json &operator[](const char *key) const { return (*this)[std::string(key)]; }
    Json &operator[](const char *key) { return (*this)[std::string(key)]; }
    template <typename I, typename std::enable_if<std::is_integral<I>::value, int>::type = 0> const Json &operator[](I i) const {
        if (kind_ != Kind::Array) throw std::invalid_argument("json: not an array");
        return arr_.at((size_t)i);
    }
    void push_back(const Json &v) {
        if (kind_ == Kind::Null) kind_ = Kind::Array;
        if (kind_ != Kind::Array) throw std::invalid_argument("json: not an array");
        arr_.push_back(v);
    }

    const object_t &items() const { return obj_; }
    const array_t &elements() const { return arr_; }

    template <typename V> V get() const {
        if constexpr (std::is_same<V, std::string>::value) {
            if (kind_ != Kind::String) throw std::invalid_argument("json: value is not a string");
            return str_;
        } else if constexpr (std::is_same<V, bool>::value) {
            if (kind_ == Kind::Bool || kind_ == Kind::Int) return int_ != 0;
            throw std::invalid_argument("json: value is not a boolean");
        } else if constexpr (std::is_enum<V>::value) {
            if (kind_ != Kind::Int) throw std::invalid_argument("json: value is not an enum ordinal");
            return static_cast<V>(int_);
        } else {
            static_assert(std::is_arithmetic<V>::value, "unsupported json::get type");
            if (kind_ == Kind::Int || kind_ == Kind::Bool) return static_cast<V>(int_);
            if (kind_ == Kind::Float) return static_cast<V>(num_);
            throw std::invalid_argument("json: value is not a number");
        }
    }
    template <typename V, typename std::enable_if<std::is_arithmetic<V>::value || std::is_enum<V>::value || std::is_same<V, std::string>::value, int>::type = 0>
    operator V() const {
        return get<V>();
    }

    template <typename V> V value(const std::string &key, const V &default_value) const {
        if (!contains(key)) return default_value;
        return obj_.at(key).template get<V>();
    }
    std::string value(const std::string &key, const char *default_value) const {
        if (!contains(key)) return default_value;
        return obj_.at(key).template get<std::string>();
    }

    bool operator==(const Json &o) const {
        if (is_number() && o.is_number()) return get<double>() == o.get<double>();
        if (kind_ != o.kind_) return false;
        switch (kind_) {
        case Kind::Null: return true;
        case Kind::Bool: return int_ == o.int_;
        case Kind::String: return str_ == o.str_;
        case Kind::Object: return obj_ == o.obj_;
        case Kind::Array: return arr_ == o.arr_;
        default: return false;
        }
    }
    bool operator!=(const Json &o) const { return !(*this == o); }

    static Json parse(const std::string &text) {
        Parser p{text, 0};
        Json j = p.value();
        p.skip();
        if (p.pos != text.size()) p.error("trailing characters");
        return j;
    }

    std::string dump() const {
        switch (kind_) {
        case Kind::Null: return "null";
        case Kind::Bool: return int_ ? "true" : "false";
        case Kind::Int: return std::to_string(int_);
        case Kind::Float: return std::to_string(num_);
        case Kind::String: return "\"" + str_ + "\"";
        case Kind::Object: {
            std::string s = "{";
            bool first = true;
            for (const auto &kv : obj_) {
                s += (first ? "\"" : ",\"") + kv.first + "\":" + kv.second.dump();
                first = false;
            }
            return s + "}";
        }
        case Kind::Array: {
            std::string s = "[";
            for (size_t i = 0; i < arr_.size(); ++i) s += (i ? "," : "") + arr_[i].dump();
            return s + "]";
        }
        }
        return "";
    }

  private:
    struct Parser {
        const std::string &s;
        size_t pos;

        [[noreturn]] void error(const std::string &what) const {
            throw std::invalid_argument("json parse error at offset " + std::to_string(pos) + ": " + what);
        }
        void skip() {
            for (;;) {
                while (pos < s.size() && std::isspace((unsigned char)s[pos])) ++pos;
                if (pos + 1 < s.size() && s[pos] == '/' && s[pos + 1] == '/') {
                    while (pos < s.size() && s[pos] != '\n') ++pos;
                } else if (pos + 1 < s.size() && s[pos] == '/' && s[pos + 1] == '*') {
                    const size_t end = s.find("*/", pos + 2);
                    if (end == std::string::npos) error("unterminated comment");
                    pos = end + 2;
                } else {
                    return;
                }
            }
        }
        bool literal(const char *lit) {
            const size_t n = std::char_traits<char>::length(lit);
            if (s.compare(pos, n, lit) == 0) {
                pos += n;
                return true;
            }
            return false;
        }
        std::string string() {
            ++pos; // opening quote
            std::string out;
            while (pos < s.size() && s[pos] != '"') {
                char c = s[pos++];
                if (c == '\\') {
                    if (pos >= s.size()) error("bad escape");
                    const char e = s[pos++];
                    switch (e) {
                    case 'n': c = '\n'; break;
                    case 't': c = '\t'; break;
                    case 'r': c = '\r'; break;
                    case 'b': c = '\b'; break;
                    case 'f': c = '\f'; break;
                    case '"': case '\\': case '/': c = e; break;
                    default: error("unsupported escape");
                    }
                }
                out.push_back(c);
            }
            if (pos >= s.size()) error("unterminated string");
            ++pos;
            return out;
        }
        Json value() {
            skip();
            if (pos >= s.size()) error("unexpected end");
            const char c = s[pos];
            if (c == '{') {
                ++pos;
                Json j = Json::object();
                skip();
                if (pos < s.size() && s[pos] == '}') {
                    ++pos;
                    return j;
                }
                for (;;) {
                    skip();
                    if (pos >= s.size() || s[pos] != '"') error("expected a key");
                    const std::string key = string();
                    skip();
                    if (pos >= s.size() || s[pos] != ':') error("expected ':'");
                    ++pos;
                    j.obj_[key] = value();
                    skip();
                    if (pos < s.size() && s[pos] == ',') {
                        ++pos;
                        continue;
                    }
                    if (pos < s.size() && s[pos] == '}') {
                        ++pos;
                        return j;
                    }
                    error("expected ',' or '}'");
                }
            }
            if (c == '[') {
                ++pos;
                Json j = Json::array();
                skip();
                if (pos < s.size() && s[pos] == ']') {
                    ++pos;
                    return j;
                }
                for (;;) {
                    j.arr_.push_back(value());
                    skip();
                    if (pos < s.size() && s[pos] == ',') {
                        ++pos;
                        continue;
                    }
                    if (pos < s.size() && s[pos] == ']') {
                        ++pos;
                        return j;
                    }
                    error("expected ',' or ']'");
                }
            }
            if (c == '"') return Json(string());
            if (literal("true")) return Json(true);
            if (literal("false")) return Json(false);
            if (literal("null")) return Json();
            const char *begin = s.c_str() + pos;
            char *end = nullptr;
            const double d = std::strtod(begin, &end);
            if (end == begin) error("unexpected character");
            bool integral = true;
            for (const char *p = begin; p < end; ++p)
                if (*p == '.' || *p == 'e' || *p == 'E') integral = false;
            pos += (size_t)(end - begin);
            if (integral) return Json((int64_t)std::strtoll(begin, nullptr, 10));
            return Json(d);
        }
    };

    Kind kind_ = Kind::Null;
    int64_t int_ = 0;
    double num_ = 0.0;
    std::string str_;
    object_t obj_;
    array_t arr_;
};

} // namespace tnn

using json = tnn::Json;
