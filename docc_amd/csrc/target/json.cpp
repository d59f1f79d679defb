#include "json.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <cctype>

namespace sdfg::json {

namespace {

[[noreturn]] void type_error(const char* want) { throw std::runtime_error(std::string("json: value is not ") + want); }

struct Parser {
    const std::string& t;
    size_t p = 0;

    explicit Parser(const std::string& text) : t(text) {}

    [[noreturn]] void fail(const std::string& msg) const {
        throw ParseError("json parse error at offset " + std::to_string(p) + ": " + msg);
    }
    void ws() {
        while (p < t.size() && (t[p] == ' ' || t[p] == '\n' || t[p] == '\t' || t[p] == '\r')) p++;
    }
    bool consume(char c) {
        ws();
        if (p < t.size() && t[p] == c) {
            p++;
            return true;
        }
        return false;
    }
    void expect(char c) {
        if (!consume(c)) fail(std::string("expected '") + c + "'");
    }
    std::string string() {
        expect('"');
        std::string out;
        while (true) {
            if (p >= t.size()) fail("unterminated string");
            char c = t[p++];
            if (c == '"') break;
            if (c != '\\') {
                out.push_back(c);
                continue;
            }
            if (p >= t.size()) fail("bad escape");
            char e = t[p++];
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
                    if (p + 4 > t.size()) fail("bad \\u escape");
                    unsigned cp = (unsigned) std::strtoul(t.substr(p, 4).c_str(), nullptr, 16);
                    p += 4;
                    if (cp < 0x80) {
                        out.push_back((char) cp);
                    } else if (cp < 0x800) {
                        out.push_back((char) (0xC0 | (cp >> 6)));
                        out.push_back((char) (0x80 | (cp & 0x3F)));
                    } else {
                        out.push_back((char) (0xE0 | (cp >> 12)));
                        out.push_back((char) (0x80 | ((cp >> 6) & 0x3F)));
                        out.push_back((char) (0x80 | (cp & 0x3F)));
                    }
                    break;
                }
                default: fail("unknown escape");
            }
        }
        return out;
    }
    Value value() {
        ws();
        if (p >= t.size()) fail("unexpected end");
        char c = t[p];
        if (c == '{') {
            p++;
            Object o;
            if (consume('}')) return Value(std::move(o));
            do {
                ws();
                std::string k = string();
                expect(':');
                o.emplace_back(std::move(k), value());
            } while (consume(','));
            expect('}');
            return Value(std::move(o));
        }
        if (c == '[') {
            p++;
            Array a;
            if (consume(']')) return Value(std::move(a));
            do {
                a.push_back(value());
            } while (consume(','));
            expect(']');
            return Value(std::move(a));
        }
        if (c == '"') return Value(string());
        if (t.compare(p, 4, "true") == 0) {
            p += 4;
            return Value(true);
        }
        if (t.compare(p, 5, "false") == 0) {
            p += 5;
            return Value(false);
        }
        if (t.compare(p, 4, "null") == 0) {
            p += 4;
            return Value(nullptr);
        }
        size_t start = p;
        bool is_double = false;
        if (t[p] == '-' || t[p] == '+') p++;
        while (p < t.size() && (std::isdigit((unsigned char) t[p]) || t[p] == '.' || t[p] == 'e' || t[p] == 'E' || t[p] == '-' || t[p] == '+')) {
            if (t[p] == '.' || t[p] == 'e' || t[p] == 'E') is_double = true;
            p++;
        }
        if (start == p) fail("unexpected character");
        std::string num = t.substr(start, p - start);
        if (is_double) return Value(std::strtod(num.c_str(), nullptr));
        return Value((int64_t) std::strtoll(num.c_str(), nullptr, 10));
    }
};

void escape_to(std::string& out, const std::string& s) {
    out.push_back('"');
    for (char c : s) {
        switch (c) {
            case '"': out += "\\\""; break;
            case '\\': out += "\\\\"; break;
            case '\n': out += "\\n"; break;
            case '\r': out += "\\r"; break;
            case '\t': out += "\\t"; break;
            default:
                if ((unsigned char) c < 0x20) {
                    char buf[8];
                    std::snprintf(buf, sizeof(buf), "\\u%04x", c);
                    out += buf;
                } else {
                    out.push_back(c);
                }
        }
    }
    out.push_back('"');
}

} // namespace

bool Value::as_bool() const {
    if (kind_ != Kind::Bool) type_error("a bool");
    return b_;
}
int64_t Value::as_int() const {
    if (kind_ == Kind::Int) return i_;
    if (kind_ == Kind::Double && std::floor(d_) == d_) return (int64_t) d_;
    type_error("an integer");
}
double Value::as_double() const {
    if (kind_ == Kind::Double) return d_;
    if (kind_ == Kind::Int) return (double) i_;
    type_error("a number");
}
const std::string& Value::as_string() const {
    if (kind_ != Kind::String) type_error("a string");
    return s_;
}
const Array& Value::as_array() const {
    if (kind_ != Kind::Array) type_error("an array");
    return *a_;
}
const Object& Value::as_object() const {
    if (kind_ != Kind::Object) type_error("an object");
    return *o_;
}
Array& Value::as_array() {
    if (kind_ != Kind::Array) type_error("an array");
    return *a_;
}
Object& Value::as_object() {
    if (kind_ != Kind::Object) type_error("an object");
    return *o_;
}

bool Value::contains(const std::string& key) const { return find(key) != nullptr; }

const Value* Value::find(const std::string& key) const {
    if (kind_ != Kind::Object) return nullptr;
    for (auto& kv : *o_)
        if (kv.first == key) return &kv.second;
    return nullptr;
}

const Value& Value::at(const std::string& key) const {
    const Value* v = find(key);
    if (!v) throw std::runtime_error("json: missing key '" + key + "'");
    return *v;
}

void Value::set(const std::string& key, Value v) {
    if (kind_ == Kind::Null) {
        kind_ = Kind::Object;
        o_ = std::make_shared<Object>();
    }
    if (kind_ != Kind::Object) type_error("an object");
    for (auto& kv : *o_)
        if (kv.first == key) {
            kv.second = std::move(v);
            return;
        }
    o_->emplace_back(key, std::move(v));
}

std::string Value::as_expression() const {
    if (kind_ == Kind::String) return s_;
    if (kind_ == Kind::Int) return std::to_string(i_);
    if (kind_ == Kind::Double) {
        char buf[64];
        std::snprintf(buf, sizeof(buf), "%.17g", d_);
        return buf;
    }
    type_error("an expression (string or number)");
}

void Value::dump_to(std::string& out, int indent, int depth) const {
    auto newline = [&](int d) {
        if (indent < 0) return;
        out.push_back('\n');
        out.append((size_t) (indent * d), ' ');
    };
    switch (kind_) {
        case Kind::Null: out += "null"; break;
        case Kind::Bool: out += b_ ? "true" : "false"; break;
        case Kind::Int: out += std::to_string(i_); break;
        case Kind::Double: {
            char buf[64];
            std::snprintf(buf, sizeof(buf), "%.17g", d_);
            out += buf;
            if (!std::strpbrk(buf, ".eEn")) out += ".0";
            break;
        }
        case Kind::String: escape_to(out, s_); break;
        case Kind::Array:
            out.push_back('[');
            for (size_t i = 0; i < a_->size(); i++) {
                if (i) out.push_back(',');
                newline(depth + 1);
                (*a_)[i].dump_to(out, indent, depth + 1);
            }
            if (!a_->empty()) newline(depth);
            out.push_back(']');
            break;
        case Kind::Object:
            out.push_back('{');
            for (size_t i = 0; i < o_->size(); i++) {
                if (i) out.push_back(',');
                newline(depth + 1);
                escape_to(out, (*o_)[i].first);
                out += indent < 0 ? ":" : ": ";
                (*o_)[i].second.dump_to(out, indent, depth + 1);
            }
            if (!o_->empty()) newline(depth);
            out.push_back('}');
            break;
    }
}

std::string Value::dump(int indent) const {
    std::string out;
    dump_to(out, indent, 0);
    return out;
}

Value Value::parse(const std::string& text) {
    Parser ps(text);
    Value v = ps.value();
    ps.ws();
    if (ps.p != text.size()) ps.fail("trailing characters");
    return v;
}

} // namespace sdfg::json
