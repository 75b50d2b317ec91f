// Minimal JSON reader for converted-JSON model files (hundreds of MB of base64 text).
// Strings are kept as views into the caller's buffer; escapes are resolved on demand.
// Also holds the base64 decoder for the weight chunks.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace fdx {
namespace json {

    struct Value;
    using Member = std::pair<std::string, Value>;

    struct Value {
        enum Type { Null, Bool, Number, String, Array, Object } type = Null;
        bool b = false;
        double num = 0;
        const char* s = nullptr; // String: raw body (still escaped); Object: the object's own text, braces included
        size_t slen = 0;
        bool has_escape = false;
        std::vector<Value> arr;
        std::vector<Member> obj;

        bool is_null() const { return type == Null; }
        bool is_array() const { return type == Array; }
        bool is_object() const { return type == Object; }
        bool is_string() const { return type == String; }
        bool is_number() const { return type == Number; }
        bool is_bool() const { return type == Bool; }

        const Value* find(const char* key) const
        {
            if (type != Object)
                return nullptr;
            for (const auto& m : obj)
                if (m.first == key)
                    return &m.second;
            return nullptr;
        }
        bool has(const char* key) const { return find(key) != nullptr; }
        const Value& at(const char* key) const
        {
            const Value* v = find(key);
            if (!v)
                throw std::runtime_error(std::string("missing JSON member: ") + key);
            return *v;
        }
        const Value& at(size_t i) const
        {
            if (type != Array || i >= arr.size())
                throw std::runtime_error("JSON array index out of range");
            return arr[i];
        }
        size_t size() const { return type == Array ? arr.size() : (type == Object ? obj.size() : 0); }

        std::string str() const
        {
            if (type != String)
                throw std::runtime_error("JSON value is not a string");
            if (!has_escape)
                return std::string(s, slen);
            std::string out;
            out.reserve(slen);
            for (size_t i = 0; i < slen; ++i) {
                char c = s[i];
                if (c != '\\') {
                    out.push_back(c);
                    continue;
                }
                if (++i >= slen)
                    break;
                switch (s[i]) {
                case 'n': out.push_back('\n'); break;
                case 't': out.push_back('\t'); break;
                case 'r': out.push_back('\r'); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'u': { // only the BMP code points Keras emits in names; encode as UTF-8
                    unsigned cp = 0;
                    for (int k = 0; k < 4 && i + 1 < slen; ++k) {
                        char h = s[++i];
                        cp = cp * 16 + (h <= '9' ? h - '0' : (h | 32) - 'a' + 10);
                    }
                    if (cp < 0x80)
                        out.push_back((char)cp);
                    else if (cp < 0x800) {
                        out.push_back((char)(0xC0 | (cp >> 6)));
                        out.push_back((char)(0x80 | (cp & 63)));
                    } else {
                        out.push_back((char)(0xE0 | (cp >> 12)));
                        out.push_back((char)(0x80 | ((cp >> 6) & 63)));
                        out.push_back((char)(0x80 | (cp & 63)));
                    }
                    break;
                }
                default: out.push_back(s[i]);
                }
            }
            return out;
        }
        double number() const
        {
            if (type != Number)
                throw std::runtime_error("JSON value is not a number");
            return num;
        }
        int64_t integer() const { return (int64_t)std::llround(number()); }
        bool boolean() const
        {
            if (type != Bool)
                throw std::runtime_error("JSON value is not a boolean");
            return b;
        }
    };

    class Parser {
    public:
        Parser(const char* p, size_t n)
            : p_(p)
            , end_(p + n)
        {
        }
        Value parse()
        {
            Value v = value(0);
            ws();
            if (p_ != end_)
                fail("trailing characters after JSON document");
            return v;
        }

    private:
        const char* p_;
        const char* end_;
        [[noreturn]] void fail(const char* what) { throw std::runtime_error(std::string("JSON parse error: ") + what); }
        void ws()
        {
            while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r'))
                ++p_;
        }
        Value value(int depth)
        {
            if (depth > 200)
                fail("nesting too deep");
            ws();
            if (p_ >= end_)
                fail("unexpected end");
            Value v;
            const char c = *p_;
            if (c == '{') {
                v.s = p_;
                ++p_;
                v.type = Value::Object;
                ws();
                if (p_ < end_ && *p_ == '}') {
                    ++p_;
                    v.slen = (size_t)(p_ - v.s);
                    return v;
                }
                for (;;) {
                    ws();
                    if (p_ >= end_ || *p_ != '"')
                        fail("expected member name");
                    Value k = string();
                    ws();
                    if (p_ >= end_ || *p_ != ':')
                        fail("expected ':'");
                    ++p_;
                    v.obj.emplace_back(k.str(), value(depth + 1));
                    ws();
                    if (p_ < end_ && *p_ == ',') {
                        ++p_;
                        continue;
                    }
                    if (p_ < end_ && *p_ == '}') {
                        ++p_;
                        v.slen = (size_t)(p_ - v.s);
                        return v;
                    }
                    fail("expected ',' or '}'");
                }
            }
            if (c == '[') {
                ++p_;
                v.type = Value::Array;
                ws();
                if (p_ < end_ && *p_ == ']') {
                    ++p_;
                    return v;
                }
                for (;;) {
                    v.arr.push_back(value(depth + 1));
                    ws();
                    if (p_ < end_ && *p_ == ',') {
                        ++p_;
                        continue;
                    }
                    if (p_ < end_ && *p_ == ']') {
                        ++p_;
                        return v;
                    }
                    fail("expected ',' or ']'");
                }
            }
            if (c == '"')
                return string();
            if (c == 't' && end_ - p_ >= 4 && !std::memcmp(p_, "true", 4)) {
                p_ += 4;
                v.type = Value::Bool;
                v.b = true;
                return v;
            }
            if (c == 'f' && end_ - p_ >= 5 && !std::memcmp(p_, "false", 5)) {
                p_ += 5;
                v.type = Value::Bool;
                return v;
            }
            if (c == 'n' && end_ - p_ >= 4 && !std::memcmp(p_, "null", 4)) {
                p_ += 4;
                return v;
            }
            if (c == 'N' && end_ - p_ >= 3 && !std::memcmp(p_, "NaN", 3)) { // Python's json writes bare NaN
                p_ += 3;
                v.type = Value::Number;
                v.num = std::nan("");
                return v;
            }
            if (c == '-' || (c >= '0' && c <= '9') || c == 'I') {
                if (c == 'I' || (c == '-' && p_ + 1 < end_ && p_[1] == 'I')) {
                    const bool neg = c == '-';
                    p_ += neg ? 9 : 8; // [-]Infinity
                    if (p_ > end_)
                        fail("bad number");
                    v.type = Value::Number;
                    v.num = neg ? -INFINITY : INFINITY;
                    return v;
                }
                char buf[64];
                size_t n = 0;
                while (p_ < end_ && n < sizeof(buf) - 1
                    && ((*p_ >= '0' && *p_ <= '9') || *p_ == '-' || *p_ == '+' || *p_ == '.' || *p_ == 'e' || *p_ == 'E'))
                    buf[n++] = *p_++;
                buf[n] = 0;
                char* e = nullptr;
                v.num = std::strtod(buf, &e);
                if (e == buf)
                    fail("bad number");
                v.type = Value::Number;
                return v;
            }
            fail("unexpected character");
        }
        Value string()
        {
            ++p_; // opening quote
            Value v;
            v.type = Value::String;
            v.s = p_;
            for (;;) {
                const char* q = static_cast<const char*>(std::memchr(p_, '"', (size_t)(end_ - p_)));
                if (!q)
                    fail("unterminated string");
                // a quote preceded by an odd number of backslashes is escaped
                size_t bs = 0;
                while (q - 1 - bs >= v.s && *(q - 1 - bs) == '\\')
                    ++bs;
                p_ = q + 1;
                if (bs % 2 == 0) {
                    v.slen = (size_t)(q - v.s);
                    break;
                }
            }
            v.has_escape = std::memchr(v.s, '\\', v.slen) != nullptr;
            return v;
        }
    };

} // namespace json

// Standard and URL-safe base64 alphabets, '=' padding optional (include/fdeep/base64.hpp:65-108).
// Appends decoded bytes to out; returns false on an invalid character.
inline bool base64_decode_append(const char* s, size_t n, std::vector<uint8_t>& out)
{
    static int8_t table[256];
    static bool init = false;
    if (!init) {
        std::memset(table, -1, sizeof table);
        const char* abc = "ABCDEFGHIJKLMNOPQRSTUVWXYZabcdefghijklmnopqrstuvwxyz0123456789+/";
        for (int i = 0; i < 64; ++i)
            table[(uint8_t)abc[i]] = (int8_t)i;
        table[(uint8_t)'-'] = 62;
        table[(uint8_t)'_'] = 63;
        init = true;
    }
    while (n > 0 && s[n - 1] == '=')
        --n;
    const size_t old = out.size();
    out.resize(old + n / 4 * 3 + 3);
    uint8_t* w = out.data() + old;
    size_t i = 0;
    for (; i + 4 <= n; i += 4) { // whole quanta: 4 characters -> 3 bytes
        const int a = table[(uint8_t)s[i]], b = table[(uint8_t)s[i + 1]], c = table[(uint8_t)s[i + 2]],
                  d = table[(uint8_t)s[i + 3]];
        if ((a | b | c | d) < 0)
            return false;
        const uint32_t v = ((uint32_t)a << 18) | ((uint32_t)b << 12) | ((uint32_t)c << 6) | (uint32_t)d;
        w[0] = (uint8_t)(v >> 16);
        w[1] = (uint8_t)(v >> 8);
        w[2] = (uint8_t)v;
        w += 3;
    }
    uint32_t acc = 0;
    int bits = 0;
    for (; i < n; ++i) { // unpadded tail
        const int8_t v = table[(uint8_t)s[i]];
        if (v < 0)
            return false;
        acc = (acc << 6) | (uint32_t)v;
        bits += 6;
        if (bits >= 8) {
            bits -= 8;
            *w++ = (uint8_t)((acc >> bits) & 0xFF);
        }
    }
    out.resize((size_t)(w - out.data()));
    return true;
}

} // namespace fdx
