// Minimal JSON document reader for the graph / block / stage documents that cross the C ABI.
// Supports objects, arrays, strings (with escapes), numbers, true / false / null.  Object members keep
// their document order.  Errors are reported by throwing std::runtime_error with the byte offset.
#pragma once

#include <cstdlib>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace ios {

class Json {
public:
    enum Kind { Null, Bool, Number, String, Array, Object };

    Json() = default;

    static Json parse(const char *text) {
        if (text == nullptr) throw std::runtime_error("json: null document");
        Reader r{text, text, 0};
        Json v = r.value();
        r.skip_ws();
        if (*r.p != '\0') r.fail("trailing characters");
        return v;
    }

    Kind kind() const { return kind_; }
    bool is_null() const { return kind_ == Null; }
    bool is_array() const { return kind_ == Array; }
    bool is_object() const { return kind_ == Object; }
    bool is_string() const { return kind_ == String; }

    size_t size() const { return kind_ == Array ? items_.size() : (kind_ == Object ? members_.size() : 0); }

    const Json &operator[](size_t i) const {
        if (kind_ != Array || i >= items_.size()) throw std::runtime_error("json: array index out of range");
        return items_[i];
    }

    bool has(const std::string &key) const {
        if (kind_ != Object) return false;
        for (const auto &m : members_)
            if (m.first == key) return true;
        return false;
    }

    const Json &operator[](const std::string &key) const {
        if (kind_ != Object) throw std::runtime_error("json: member '" + key + "' requested from a non-object");
        for (const auto &m : members_)
            if (m.first == key) return m.second;
        throw std::runtime_error("json: missing member '" + key + "'");
    }

    const std::vector<std::pair<std::string, Json>> &members() const { return members_; }
    const std::vector<Json> &items() const { return items_; }

    int as_int() const {
        if (kind_ != Number) throw std::runtime_error("json: expected a number");
        // NaN fails both comparisons; a value outside int cannot be converted without undefined behaviour
        if (!(number_ >= -2147483648.0 && number_ <= 2147483647.0)) throw std::runtime_error("json: number out of integer range");
        return static_cast<int>(number_);
    }
    double as_double() const {
        if (kind_ != Number) throw std::runtime_error("json: expected a number");
        return number_;
    }
    bool as_bool() const {
        if (kind_ == Bool) return bool_;
        if (kind_ == Number) return number_ != 0.0;
        throw std::runtime_error("json: expected a boolean");
    }
    const std::string &as_string() const {
        if (kind_ != String) throw std::runtime_error("json: expected a string");
        return string_;
    }

private:
    struct Reader {
        const char *begin;
        const char *p;
        int depth;   // open arrays / objects around the value being read
        // graph documents nest a handful of levels (graph > blocks > nodes > inputs > term > value); a bound keeps a
        // hostile document from exhausting the stack, which no exception handler could report
        static constexpr int kMaxDepth = 64;
        struct Nest {
            Reader &r;
            explicit Nest(Reader &reader) : r(reader) {
                if (++r.depth > kMaxDepth) r.fail("nesting deeper than 64 levels");
            }
            ~Nest() { --r.depth; }
        };

        [[noreturn]] void fail(const std::string &what) const {
            throw std::runtime_error("json: " + what + " at byte " + std::to_string(p - begin));
        }
        void skip_ws() {
            while (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r') ++p;
        }
        bool consume(char c) {
            skip_ws();
            if (*p != c) return false;
            ++p;
            return true;
        }
        void expect(char c) {
            if (!consume(c)) fail(std::string("expected '") + c + "'");
        }
        Json value() {
            skip_ws();
            Json v;
            switch (*p) {
                case '{': {
                    Nest nest(*this);
                    ++p;
                    v.kind_ = Object;
                    if (consume('}')) return v;
                    do {
                        skip_ws();
                        if (*p != '"') fail("expected a member name");
                        std::string key = string();
                        expect(':');
                        v.members_.emplace_back(std::move(key), value());
                    } while (consume(','));
                    expect('}');
                    return v;
                }
                case '[': {
                    Nest nest(*this);
                    ++p;
                    v.kind_ = Array;
                    if (consume(']')) return v;
                    do {
                        v.items_.push_back(value());
                    } while (consume(','));
                    expect(']');
                    return v;
                }
                case '"':
                    v.kind_ = String;
                    v.string_ = string();
                    return v;
                case 't':
                    literal("true");
                    v.kind_ = Bool;
                    v.bool_ = true;
                    return v;
                case 'f':
                    literal("false");
                    v.kind_ = Bool;
                    v.bool_ = false;
                    return v;
                case 'n':
                    literal("null");
                    return v;
                default: {
                    char *end = nullptr;
                    double d = std::strtod(p, &end);
                    if (end == p) fail("unexpected character");
                    p = end;
                    v.kind_ = Number;
                    v.number_ = d;
                    return v;
                }
            }
        }
        void literal(const char *word) {
            size_t n = std::strlen(word);
            if (std::strncmp(p, word, n) != 0) fail("bad literal");
            p += n;
        }
        std::string string() {
            std::string out;
            ++p;  // opening quote
            while (*p != '"') {
                if (*p == '\0') fail("unterminated string");
                if (*p == '\\') {
                    ++p;
                    switch (*p) {
                        case 'n': out += '\n'; break;
                        case 't': out += '\t'; break;
                        case 'r': out += '\r'; break;
                        case 'b': out += '\b'; break;
                        case 'f': out += '\f'; break;
                        case 'u': {
                            unsigned code = 0;
                            for (int i = 1; i <= 4; i++) {
                                char c = p[i];
                                code <<= 4;
                                if (c >= '0' && c <= '9') code |= c - '0';
                                else if (c >= 'a' && c <= 'f') code |= c - 'a' + 10;
                                else if (c >= 'A' && c <= 'F') code |= c - 'A' + 10;
                                else fail("bad \\u escape");
                            }
                            p += 4;
                            // names in graph documents are ASCII; encode the rest as UTF-8 without surrogates
                            if (code < 0x80) out += static_cast<char>(code);
                            else if (code < 0x800) {
                                out += static_cast<char>(0xC0 | (code >> 6));
                                out += static_cast<char>(0x80 | (code & 0x3F));
                            } else {
                                out += static_cast<char>(0xE0 | (code >> 12));
                                out += static_cast<char>(0x80 | ((code >> 6) & 0x3F));
                                out += static_cast<char>(0x80 | (code & 0x3F));
                            }
                            break;
                        }
                        case '\0': fail("unterminated string");   // a backslash was the last byte of the document
                        default: out += *p;  // \" \\ \/
                    }
                    ++p;
                } else {
                    out += *p++;
                }
            }
            ++p;  // closing quote
            return out;
        }
    };

    Kind kind_ = Null;
    bool bool_ = false;
    double number_ = 0.0;
    std::string string_;
    std::vector<Json> items_;
    std::vector<std::pair<std::string, Json>> members_;
};

}  // namespace ios
