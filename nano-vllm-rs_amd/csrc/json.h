// json.h — a small JSON reader for model configuration files (objects, arrays, strings, numbers, true / false / null).  Host only.
#pragma once
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace nvr {

struct Json {
    enum Kind { Null, Bool, Num, Str, Arr, Obj } kind = Null;
    bool b = false; double num = 0; std::string str;
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj;

    const Json *get(const char *key) const {
        if (kind != Obj) return nullptr;
        for (const auto &kv : obj) if (kv.first == key) return &kv.second;
        return nullptr;
    }
    bool is_null() const { return kind == Null; }

    // parse(text, err): false with a message in *err on malformed input
    static bool parse(const char *text, Json *out, std::string *err) {
        const char *p = text;
        if (!value(p, *out, err, 0)) return false;
        skip(p);
        if (*p) { *err = "trailing characters after the JSON value"; return false; }
        return true;
    }

private:
    static void skip(const char *&p) { while (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r') ++p; }
    static bool string(const char *&p, std::string &s, std::string *err) {
        ++p;                                                          // opening quote
        while (*p && *p != '"') {
            if (*p == '\\') {
                ++p;
                switch (*p) {
                    case 'n': s += '\n'; break; case 't': s += '\t'; break; case 'r': s += '\r'; break; case 'b': s += '\b'; break; case 'f': s += '\f'; break;
                    case 'u': {
                        unsigned cp = 0;
                        for (int i = 0; i < 4; ++i) {
                            ++p; char c = *p; cp <<= 4;
                            if (c >= '0' && c <= '9') cp |= (unsigned)(c - '0'); else if (c >= 'a' && c <= 'f') cp |= (unsigned)(c - 'a' + 10);
                            else if (c >= 'A' && c <= 'F') cp |= (unsigned)(c - 'A' + 10); else { *err = "bad \\u escape"; return false; }
                        }
                        if (cp < 0x80) s += (char)cp;
                        else if (cp < 0x800) { s += (char)(0xC0 | (cp >> 6)); s += (char)(0x80 | (cp & 0x3F)); }
                        else { s += (char)(0xE0 | (cp >> 12)); s += (char)(0x80 | ((cp >> 6) & 0x3F)); s += (char)(0x80 | (cp & 0x3F)); }
                        break;
                    }
                    case 0: *err = "unterminated string"; return false;
                    default: s += *p;
                }
                ++p;
            } else s += *p++;
        }
        if (*p != '"') { *err = "unterminated string"; return false; }
        ++p;
        return true;
    }
    static bool value(const char *&p, Json &v, std::string *err, int depth) {
        if (depth > 64) { *err = "nesting too deep"; return false; }
        skip(p);
        if (*p == '{') {
            v.kind = Obj; ++p; skip(p);
            if (*p == '}') { ++p; return true; }
            for (;;) {
                skip(p);
                if (*p != '"') { *err = "object key expected"; return false; }
                std::string key;
                if (!string(p, key, err)) return false;
                skip(p);
                if (*p != ':') { *err = "':' expected"; return false; }
                ++p;
                v.obj.emplace_back(key, Json());
                if (!value(p, v.obj.back().second, err, depth + 1)) return false;
                skip(p);
                if (*p == ',') { ++p; continue; }
                if (*p == '}') { ++p; return true; }
                *err = "',' or '}' expected"; return false;
            }
        }
        if (*p == '[') {
            v.kind = Arr; ++p; skip(p);
            if (*p == ']') { ++p; return true; }
            for (;;) {
                v.arr.emplace_back();
                if (!value(p, v.arr.back(), err, depth + 1)) return false;
                skip(p);
                if (*p == ',') { ++p; continue; }
                if (*p == ']') { ++p; return true; }
                *err = "',' or ']' expected"; return false;
            }
        }
        if (*p == '"') { v.kind = Str; return string(p, v.str, err); }
        if (!std::strncmp(p, "true", 4)) { v.kind = Bool; v.b = true; p += 4; return true; }
        if (!std::strncmp(p, "false", 5)) { v.kind = Bool; v.b = false; p += 5; return true; }
        if (!std::strncmp(p, "null", 4)) { v.kind = Null; p += 4; return true; }
        char *end = nullptr;
        const double d = std::strtod(p, &end);
        if (end == p) { *err = "value expected"; return false; }
        v.kind = Num; v.num = d; p = end;
        return true;
    }
};

}  // namespace nvr
