#include "json.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

namespace mll {

const Json* Json::get(const std::string& key) const {
    if (type != Object) return nullptr;
    for (const auto& kv : obj)
        if (kv.first == key) return &kv.second;
    return nullptr;
}

namespace {

struct Parser {
    const char* s;
    size_t n;
    size_t i = 0;
    std::string err;

    bool fail(const char* what) {
        if (err.empty()) err = std::string(what) + " at byte " + std::to_string(i);
        return false;
    }
    void ws() {
        while (i < n && (s[i] == ' ' || s[i] == '\t' || s[i] == '\n' || s[i] == '\r')) i++;
    }
    static void appendUtf8(std::string& o, unsigned cp) {
        if (cp < 0x80) o += (char)cp;
        else if (cp < 0x800) { o += (char)(0xC0 | (cp >> 6)); o += (char)(0x80 | (cp & 0x3F)); }
        else if (cp < 0x10000) {
            o += (char)(0xE0 | (cp >> 12)); o += (char)(0x80 | ((cp >> 6) & 0x3F)); o += (char)(0x80 | (cp & 0x3F));
        } else {
            o += (char)(0xF0 | (cp >> 18)); o += (char)(0x80 | ((cp >> 12) & 0x3F));
            o += (char)(0x80 | ((cp >> 6) & 0x3F)); o += (char)(0x80 | (cp & 0x3F));
        }
    }
    bool hex4(unsigned& v) {
        if (i + 4 > n) return fail("truncated \\u escape");
        v = 0;
        for (int k = 0; k < 4; k++) {
            char c = s[i++];
            v <<= 4;
            if (c >= '0' && c <= '9') v |= (unsigned)(c - '0');
            else if (c >= 'a' && c <= 'f') v |= (unsigned)(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F') v |= (unsigned)(c - 'A' + 10);
            else return fail("bad hex digit in \\u escape");
        }
        return true;
    }
    bool string(std::string& out) {
        if (i >= n || s[i] != '"') return fail("expected string");
        i++;
        out.clear();
        while (i < n) {
            unsigned char c = (unsigned char)s[i++];
            if (c == '"') return true;
            if (c == '\\') {
                if (i >= n) return fail("truncated escape");
                char e = s[i++];
                switch (e) {
                    case '"': out += '"'; break;
                    case '\\': out += '\\'; break;
                    case '/': out += '/'; break;
                    case 'b': out += '\b'; break;
                    case 'f': out += '\f'; break;
                    case 'n': out += '\n'; break;
                    case 'r': out += '\r'; break;
                    case 't': out += '\t'; break;
                    case 'u': {
                        unsigned cp;
                        if (!hex4(cp)) return false;
                        if (cp >= 0xD800 && cp <= 0xDBFF) { // surrogate pair
                            if (i + 2 <= n && s[i] == '\\' && s[i + 1] == 'u') {
                                i += 2;
                                unsigned lo;
                                if (!hex4(lo)) return false;
                                if (lo < 0xDC00 || lo > 0xDFFF) return fail("bad low surrogate");
                                cp = 0x10000 + (((cp - 0xD800) << 10) | (lo - 0xDC00));
                            } else return fail("lone high surrogate");
                        } else if (cp >= 0xDC00 && cp <= 0xDFFF) return fail("lone low surrogate");
                        appendUtf8(out, cp);
                        break;
                    }
                    default: return fail("unknown escape");
                }
            } else {
                out += (char)c;
            }
        }
        return fail("unterminated string");
    }
    bool number(Json& out) {
        size_t st = i;
        if (i < n && (s[i] == '-' || s[i] == '+')) i++;
        bool digits = false;
        while (i < n && s[i] >= '0' && s[i] <= '9') { i++; digits = true; }
        if (i < n && s[i] == '.') { i++; while (i < n && s[i] >= '0' && s[i] <= '9') { i++; digits = true; } }
        if (digits && i < n && (s[i] == 'e' || s[i] == 'E')) {
            i++;
            if (i < n && (s[i] == '-' || s[i] == '+')) i++;
            while (i < n && s[i] >= '0' && s[i] <= '9') i++;
        }
        if (!digits) { i = st; return fail("expected value"); }
        std::string t(s + st, i - st);
        out.type = Json::Number;
        out.num = strtod(t.c_str(), nullptr);
        return true;
    }
    bool value(Json& out, int depth) {
        if (depth > 256) return fail("nesting too deep");
        ws();
        if (i >= n) return fail("unexpected end of document");
        char c = s[i];
        if (c == '{') {
            i++;
            out.type = Json::Object;
            ws();
            if (i < n && s[i] == '}') { i++; return true; }
            while (true) {
                ws();
                std::string k;
                if (!string(k)) return false;
                ws();
                if (i >= n || s[i] != ':') return fail("expected ':'");
                i++;
                Json v;
                if (!value(v, depth + 1)) return false;
                out.obj.emplace_back(std::move(k), std::move(v));
                ws();
                if (i < n && s[i] == ',') { i++; continue; }
                if (i < n && s[i] == '}') { i++; return true; }
                return fail("expected ',' or '}'");
            }
        }
        if (c == '[') {
            i++;
            out.type = Json::Array;
            ws();
            if (i < n && s[i] == ']') { i++; return true; }
            while (true) {
                Json v;
                if (!value(v, depth + 1)) return false;
                out.arr.push_back(std::move(v));
                ws();
                if (i < n && s[i] == ',') { i++; continue; }
                if (i < n && s[i] == ']') { i++; return true; }
                return fail("expected ',' or ']'");
            }
        }
        if (c == '"') { out.type = Json::String; return string(out.str); }
        if (n - i >= 4 && !strncmp(s + i, "true", 4)) { i += 4; out.type = Json::Bool; out.b = true; return true; }
        if (n - i >= 5 && !strncmp(s + i, "false", 5)) { i += 5; out.type = Json::Bool; out.b = false; return true; }
        if (n - i >= 4 && !strncmp(s + i, "null", 4)) { i += 4; out.type = Json::Null; return true; }
        return number(out);
    }
};

void dumpString(const std::string& s, std::string& o) {
    o += '"';
    for (unsigned char c : s) {
        switch (c) {
            case '"': o += "\\\""; break;
            case '\\': o += "\\\\"; break;
            case '\n': o += "\\n"; break;
            case '\r': o += "\\r"; break;
            case '\t': o += "\\t"; break;
            case '\b': o += "\\b"; break;
            case '\f': o += "\\f"; break;
            default:
                if (c < 0x20) { char b[8]; snprintf(b, sizeof b, "\\u%04x", c); o += b; }
                else o += (char)c;
        }
    }
    o += '"';
}

void dump(const Json& j, std::string& o) {
    switch (j.type) {
        case Json::Null: o += "null"; break;
        case Json::Bool: o += j.b ? "true" : "false"; break;
        case Json::Number: {
            char b[40];
            if (j.num == floor(j.num) && fabs(j.num) < 1e15) snprintf(b, sizeof b, "%.0f", j.num);
            else snprintf(b, sizeof b, "%.17g", j.num);
            o += b;
            break;
        }
        case Json::String: dumpString(j.str, o); break;
        case Json::Array:
            o += '[';
            for (size_t k = 0; k < j.arr.size(); k++) { if (k) o += ','; dump(j.arr[k], o); }
            o += ']';
            break;
        case Json::Object:
            o += '{';
            for (size_t k = 0; k < j.obj.size(); k++) {
                if (k) o += ',';
                dumpString(j.obj[k].first, o);
                o += ':';
                dump(j.obj[k].second, o);
            }
            o += '}';
            break;
    }
}

} // namespace

bool parseJson(const char* text, size_t len, Json& out, std::string& err) {
    Parser p{text, len};
    out = Json();
    if (!p.value(out, 0)) { err = p.err; return false; }
    p.ws();
    // cJSON_Parse does not require the document to end here; a NUL-padded or
    // newline-terminated header therefore still parses.  Other trailing bytes are an error.
    while (p.i < p.n && p.s[p.i] == '\0') p.i++;
    if (p.i != p.n) { err = "trailing characters at byte " + std::to_string(p.i); return false; }
    return true;
}

std::string dumpJson(const Json& j) {
    std::string o;
    dump(j, o);
    return o;
}

Json jsonNumber(double v) { Json j; j.type = Json::Number; j.num = v; return j; }
Json jsonString(const std::string& s) { Json j; j.type = Json::String; j.str = s; return j; }
Json jsonIntArray(const std::vector<int>& v) {
    Json j;
    j.type = Json::Array;
    for (int x : v) j.arr.push_back(jsonNumber(x));
    return j;
}

} // namespace mll
