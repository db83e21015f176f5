// JSON reading and writing shared by the line protocol of `generate --jsonl-session` and the HTTP
// server: a cursor over one text with the value kinds those requests use (strings, numbers,
// booleans, null, arrays of numbers, anything else skipped), and writers for the value kinds of
// the answers.
#pragma once
#include <errno.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

namespace rustane {
namespace json {

// ---- a reader for the flat objects of the protocol: strings, numbers, booleans, null, arrays of numbers
struct Reader {
    const std::string &s;
    size_t i = 0;
    std::string err;

    explicit Reader(const std::string &str) : s(str) {}
    void ws() { while (i < s.size() && (s[i] == ' ' || s[i] == '\t' || s[i] == '\r' || s[i] == '\n')) ++i; }
    bool fail(const std::string &m) { if (err.empty()) err = m + " at column " + std::to_string(i + 1); return false; }
    bool lit(const char *w) {
        const size_t n = strlen(w);
        if (s.compare(i, n, w) == 0) { i += n; return true; }
        return false;
    }
    bool string(std::string *out) {
        if (i >= s.size() || s[i] != '"') return fail("expected a string");
        ++i;
        out->clear();
        while (i < s.size() && s[i] != '"') {
            char c = s[i++];
            if (c == '\\') {
                if (i >= s.size()) return fail("unterminated escape");
                const char e = s[i++];
                switch (e) {
                    case '"': c = '"'; break;
                    case '\\': c = '\\'; break;
                    case '/': c = '/'; break;
                    case 'b': c = '\b'; break;
                    case 'f': c = '\f'; break;
                    case 'n': c = '\n'; break;
                    case 'r': c = '\r'; break;
                    case 't': c = '\t'; break;
                    case 'u': {
                        if (i + 4 > s.size()) return fail("short \\u escape");
                        unsigned v = 0;
                        for (int k = 0; k < 4; ++k) {
                            const char h = s[i++];
                            v <<= 4;
                            if (h >= '0' && h <= '9') v |= (unsigned)(h - '0');
                            else if (h >= 'a' && h <= 'f') v |= (unsigned)(h - 'a' + 10);
                            else if (h >= 'A' && h <= 'F') v |= (unsigned)(h - 'A' + 10);
                            else return fail("bad \\u escape");
                        }
                        // UTF-8 of the code unit (surrogate pairs are not joined: no field here needs them)
                        if (v < 0x80) out->push_back((char)v);
                        else if (v < 0x800) { out->push_back((char)(0xC0 | (v >> 6))); out->push_back((char)(0x80 | (v & 0x3F))); }
                        else { out->push_back((char)(0xE0 | (v >> 12))); out->push_back((char)(0x80 | ((v >> 6) & 0x3F))); out->push_back((char)(0x80 | (v & 0x3F))); }
                        continue;
                    }
                    default: return fail("bad escape");
                }
            }
            out->push_back(c);
        }
        if (i >= s.size()) return fail("unterminated string");
        ++i;
        return true;
    }
    // the characters of a JSON number
    bool number_text(std::string *out) {
        const size_t b = i;
        if (i < s.size() && s[i] == '-') ++i;
        while (i < s.size() && ((s[i] >= '0' && s[i] <= '9') || s[i] == '.' || s[i] == 'e' || s[i] == 'E' || s[i] == '+' || s[i] == '-')) ++i;
        if (i == b) return fail("expected a number");
        *out = s.substr(b, i - b);
        return true;
    }
    bool unsigned_int(uint64_t *v, uint64_t max, const char *what) {
        std::string t;
        if (!number_text(&t)) return false;
        if (t.empty() || t.find_first_not_of("0123456789") != std::string::npos) return fail(std::string("expected ") + what);
        errno = 0;
        char *end = nullptr;
        const unsigned long long x = strtoull(t.c_str(), &end, 10);
        if (errno || *end || x > max) return fail(std::string("number out of range for ") + what);
        *v = x;
        return true;
    }
    bool real(double *v) {
        std::string t;
        if (!number_text(&t)) return false;
        char *end = nullptr;
        *v = strtod(t.c_str(), &end);
        if (*end) return fail("malformed number");
        return true;
    }
    // skips any value (fields the protocol does not know); nesting is bounded, so that a request made of
    // brackets cannot run the stack out
    int depth = 0;
    bool skip() {
        struct Level { int &d; explicit Level(int &x) : d(x) { ++d; } ~Level() { --d; } } level(depth);
        if (depth > 128) return fail("value nested too deeply");
        ws();
        if (i >= s.size()) return fail("unexpected end of input");
        std::string tmp;
        if (s[i] == '"') return string(&tmp);
        if (s[i] == '{' || s[i] == '[') {
            const char close = s[i] == '{' ? '}' : ']';
            const bool obj = s[i] == '{';
            ++i; ws();
            if (i < s.size() && s[i] == close) { ++i; return true; }
            for (;;) {
                ws();
                if (obj) { if (!string(&tmp)) return false; ws(); if (i >= s.size() || s[i] != ':') return fail("expected ':'"); ++i; }
                if (!skip()) return false;
                ws();
                if (i < s.size() && s[i] == ',') { ++i; continue; }
                if (i < s.size() && s[i] == close) { ++i; return true; }
                return fail("expected ',' or a closing bracket");
            }
        }
        if (lit("true") || lit("false") || lit("null")) return true;
        return number_text(&tmp);
    }
};

// shortest decimal form that reads back as the same double, always with a fraction or exponent
inline std::string json_f64(double v) {
    if (!isfinite(v)) return "null";
    char buf[40];
    for (int p = 1; p <= 17; ++p) {
        snprintf(buf, sizeof buf, "%.*g", p, v);
        if (strtod(buf, nullptr) == v) break;
    }
    if (!strpbrk(buf, ".eEn")) strcat(buf, ".0");
    return buf;
}
inline std::string json_str(const std::string &s) {
    std::string o = "\"";
    for (unsigned char c : s) {
        switch (c) {
            case '"': o += "\\\""; break;
            case '\\': o += "\\\\"; break;
            case '\n': o += "\\n"; break;
            case '\r': o += "\\r"; break;
            case '\t': o += "\\t"; break;
            default:
                if (c < 0x20) { char b[8]; snprintf(b, sizeof b, "\\u%04x", c); o += b; }
                else o.push_back((char)c);
        }
    }
    return o + "\"";
}
inline std::string json_opt(const char *s) { return s ? json_str(s) : "null"; }
inline std::string json_ids(const std::vector<uint32_t> &ids) {
    std::string o = "[";
    for (size_t i = 0; i < ids.size(); ++i) { if (i) o += ","; o += std::to_string(ids[i]); }
    return o + "]";
}

}  // namespace json
}  // namespace rustane
