#include "json.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

namespace tq {
namespace {

struct Parser {
    const char* p;
    const char* end;
    const char* begin;
    int depth = 0;

    [[noreturn]] void fail(const char* what) const {
        char msg[160];
        snprintf(msg, sizeof(msg), "%s at byte %ld", what, (long)(p - begin));
        throw JsonError(msg);
    }
    void skip() {
        while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) ++p;
    }
    static void put_utf8(std::string& out, unsigned cp) {
        if (cp < 0x80) out.push_back((char)cp);
        else if (cp < 0x800) { out.push_back((char)(0xC0 | (cp >> 6))); out.push_back((char)(0x80 | (cp & 0x3F))); }
        else if (cp < 0x10000) {
            out.push_back((char)(0xE0 | (cp >> 12))); out.push_back((char)(0x80 | ((cp >> 6) & 0x3F))); out.push_back((char)(0x80 | (cp & 0x3F)));
        } else {
            out.push_back((char)(0xF0 | (cp >> 18))); out.push_back((char)(0x80 | ((cp >> 12) & 0x3F)));
            out.push_back((char)(0x80 | ((cp >> 6) & 0x3F))); out.push_back((char)(0x80 | (cp & 0x3F)));
        }
    }
    unsigned hex4() {
        if (end - p < 4) fail("short \\u escape");
        unsigned v = 0;
        for (int i = 0; i < 4; ++i, ++p) {
            const char c = *p;
            v <<= 4;
            if (c >= '0' && c <= '9') v |= (unsigned)(c - '0');
            else if (c >= 'a' && c <= 'f') v |= (unsigned)(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F') v |= (unsigned)(c - 'A' + 10);
            else fail("bad \\u escape");
        }
        return v;
    }
    std::string string() {
        if (p >= end || *p != '"') fail("expected a string");
        ++p;
        std::string out;
        while (true) {
            if (p >= end) fail("unterminated string");
            const char c = *p++;
            if (c == '"') break;
            if (c != '\\') { out.push_back(c); continue; }
            if (p >= end) fail("unterminated escape");
            const char e = *p++;
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
                    if (cp >= 0xD800 && cp < 0xDC00 && end - p >= 6 && p[0] == '\\' && p[1] == 'u') {
                        p += 2;
                        const unsigned lo = hex4();
                        if (lo >= 0xDC00 && lo < 0xE000) cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                        else { put_utf8(out, 0xFFFD); cp = lo; }
                    }
                    put_utf8(out, cp);
                    break;
                }
                default: fail("unknown escape");
            }
        }
        return out;
    }
    Json number() {
        const char* s = p;
        bool integral = true;
        if (p < end && *p == '-') ++p;
        if (p >= end || !((*p >= '0' && *p <= '9'))) {
            // Infinity / NaN as Python's json module writes them
            if (end - p >= 8 && !strncmp(p, "Infinity", 8)) { p += 8; return Json(*s == '-' ? -INFINITY : INFINITY); }
            fail("expected a number");
        }
        while (p < end && *p >= '0' && *p <= '9') ++p;
        if (p < end && *p == '.') { integral = false; ++p; while (p < end && *p >= '0' && *p <= '9') ++p; }
        if (p < end && (*p == 'e' || *p == 'E')) {
            integral = false;
            ++p;
            if (p < end && (*p == '+' || *p == '-')) ++p;
            while (p < end && *p >= '0' && *p <= '9') ++p;
        }
        std::string text(s, p);
        if (integral && text.size() <= 18) return Json((long long)strtoll(text.c_str(), nullptr, 10));
        return Json(strtod(text.c_str(), nullptr));
    }
    Json value() {
        skip();
        if (p >= end) fail("unexpected end");
        if (++depth > 200) fail("nested too deeply");
        Json out;
        const char c = *p;
        if (c == '{') {
            ++p;
            out = Json::object();
            skip();
            if (p < end && *p == '}') { ++p; }
            else
                while (true) {
                    skip();
                    std::string key = string();
                    skip();
                    if (p >= end || *p != ':') fail("expected ':'");
                    ++p;
                    out.append(std::move(key), value());
                    skip();
                    if (p < end && *p == ',') { ++p; continue; }
                    if (p < end && *p == '}') { ++p; break; }
                    fail("expected ',' or '}'");
                }
        } else if (c == '[') {
            ++p;
            out = Json::array();
            skip();
            if (p < end && *p == ']') { ++p; }
            else
                while (true) {
                    out.push(value());
                    skip();
                    if (p < end && *p == ',') { ++p; continue; }
                    if (p < end && *p == ']') { ++p; break; }
                    fail("expected ',' or ']'");
                }
        } else if (c == '"') {
            out = Json(string());
        } else if (end - p >= 4 && !strncmp(p, "true", 4)) { p += 4; out = Json(true); }
        else if (end - p >= 5 && !strncmp(p, "false", 5)) { p += 5; out = Json(false); }
        else if (end - p >= 4 && !strncmp(p, "null", 4)) { p += 4; out = Json(); }
        else if (end - p >= 3 && !strncmp(p, "NaN", 3)) { p += 3; out = Json((double)NAN); }
        else out = number();
        --depth;
        return out;
    }
};

void dump_string(std::string& out, const std::string& s) {
    out.push_back('"');
    for (unsigned char c : s) {
        switch (c) {
            case '"': out += "\\\""; break;
            case '\\': out += "\\\\"; break;
            case '\n': out += "\\n"; break;
            case '\r': out += "\\r"; break;
            case '\t': out += "\\t"; break;
            default:
                if (c < 0x20) { char b[8]; snprintf(b, sizeof(b), "\\u%04x", c); out += b; }
                else out.push_back((char)c);
        }
    }
    out.push_back('"');
}

}  // namespace

Json Json::parse(const char* text, size_t n) {
    Parser ps{text, text + n, text};
    Json v = ps.value();
    ps.skip();
    if (ps.p != ps.end) ps.fail("trailing characters");
    return v;
}

Json Json::parse(const std::string& text) { return parse(text.data(), text.size()); }

void Json::dump_to(std::string& out) const {
    char b[40];
    switch (kind_) {
        case Null: out += "null"; break;
        case Bool: out += int_ ? "true" : "false"; break;
        case Int: snprintf(b, sizeof(b), "%lld", int_); out += b; break;
        case Float:
            if (isnan(num_)) out += "NaN";
            else if (isinf(num_)) out += num_ < 0 ? "-Infinity" : "Infinity";
            else { snprintf(b, sizeof(b), "%.17g", num_); out += b; if (!strpbrk(b, ".eE")) out += ".0"; }
            break;
        case String: dump_string(out, str_); break;
        case Array:
            out.push_back('[');
            for (size_t i = 0; i < arr_.size(); ++i) { if (i) out.push_back(','); arr_[i].dump_to(out); }
            out.push_back(']');
            break;
        case Object:
            out.push_back('{');
            for (size_t i = 0; i < obj_.size(); ++i) {
                if (i) out.push_back(',');
                dump_string(out, obj_[i].first);
                out.push_back(':');
                obj_[i].second.dump_to(out);
            }
            out.push_back('}');
            break;
    }
}

std::string Json::dump() const {
    std::string out;
    dump_to(out);
    return out;
}

}  // namespace tq
