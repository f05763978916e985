// engine/json.h -- a small JSON reader (objects, arrays, strings, numbers, true / false / null) for config.json and the safetensors header.
// Header only; values are a tree of nt::Json.  Malformed input sets ok() to false instead of throwing.
#pragma once
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

namespace nt {

class Json {
public:
    enum Kind { NUL, BOOL, NUM, STR, ARR, OBJ };
    Kind kind = NUL;
    bool b = false;
    double num = 0.0;
    std::string str;
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj;   // in file order

    bool is_null() const { return kind == NUL; }
    bool is_object() const { return kind == OBJ; }
    bool is_array() const { return kind == ARR; }
    bool is_number() const { return kind == NUM; }
    bool is_string() const { return kind == STR; }
    const Json* find(const std::string& key) const {
        if (kind != OBJ) return nullptr;
        for (const auto& kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
    bool has(const std::string& key) const { const Json* j = find(key); return j && !j->is_null(); }
    const Json& at(const std::string& key) const { static const Json none; const Json* j = find(key); return j ? *j : none; }
    double number(double dflt = 0.0) const { return kind == NUM ? num : dflt; }
    long long integer(long long dflt = 0) const { return kind == NUM ? (long long)num : dflt; }
    bool truth(bool dflt = false) const { return kind == BOOL ? b : kind == NUM ? num != 0.0 : dflt; }   // true / false (or a number that is not zero)

    // parse `n` bytes; on failure returns false and leaves *this null
    bool parse(const char* s, size_t n) {
        const char* p = s;
        const char* e = s + n;
        Json v;
        if (!value(p, e, v, 0)) return false;
        ws(p, e);
        if (p != e) return false;
        *this = std::move(v);
        return true;
    }

private:
    static void ws(const char*& p, const char* e) { while (p < e && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p; }
    static bool text(const char*& p, const char* e, std::string& out) {
        if (p >= e || *p != '"') return false;
        ++p;
        out.clear();
        while (p < e && *p != '"') {
            if (*p == '\\') {
                if (++p >= e) return false;
                switch (*p) {
                    case 'n': out += '\n'; break;
                    case 't': out += '\t'; break;
                    case 'r': out += '\r'; break;
                    case 'b': out += '\b'; break;
                    case 'f': out += '\f'; break;
                    case 'u': {
                        if (e - p < 5) return false;
                        char hex[5] = {p[1], p[2], p[3], p[4], 0};
                        const unsigned c = (unsigned)strtoul(hex, nullptr, 16);
                        if (c < 0x80) out += (char)c;
                        else if (c < 0x800) { out += (char)(0xC0 | (c >> 6)); out += (char)(0x80 | (c & 0x3F)); }
                        else { out += (char)(0xE0 | (c >> 12)); out += (char)(0x80 | ((c >> 6) & 0x3F)); out += (char)(0x80 | (c & 0x3F)); }
                        p += 4;
                        break;
                    }
                    default: out += *p;
                }
                ++p;
            } else {
                out += *p++;
            }
        }
        if (p >= e) return false;
        ++p;
        return true;
    }
    static bool value(const char*& p, const char* e, Json& v, int depth) {
        if (depth > 64) return false;
        ws(p, e);
        if (p >= e) return false;
        if (*p == '{') {
            v.kind = OBJ;
            ++p;
            ws(p, e);
            if (p < e && *p == '}') { ++p; return true; }
            for (;;) {
                ws(p, e);
                std::string k;
                if (!text(p, e, k)) return false;
                ws(p, e);
                if (p >= e || *p != ':') return false;
                ++p;
                Json c;
                if (!value(p, e, c, depth + 1)) return false;
                v.obj.emplace_back(std::move(k), std::move(c));
                ws(p, e);
                if (p < e && *p == ',') { ++p; continue; }
                if (p < e && *p == '}') { ++p; return true; }
                return false;
            }
        }
        if (*p == '[') {
            v.kind = ARR;
            ++p;
            ws(p, e);
            if (p < e && *p == ']') { ++p; return true; }
            for (;;) {
                Json c;
                if (!value(p, e, c, depth + 1)) return false;
                v.arr.push_back(std::move(c));
                ws(p, e);
                if (p < e && *p == ',') { ++p; continue; }
                if (p < e && *p == ']') { ++p; return true; }
                return false;
            }
        }
        if (*p == '"') { v.kind = STR; return text(p, e, v.str); }
        if (e - p >= 4 && !strncmp(p, "true", 4)) { v.kind = BOOL; v.b = true; p += 4; return true; }
        if (e - p >= 5 && !strncmp(p, "false", 5)) { v.kind = BOOL; v.b = false; p += 5; return true; }
        if (e - p >= 4 && !strncmp(p, "null", 4)) { v.kind = NUL; p += 4; return true; }
        // number
        const char* q = p;
        while (q < e && (strchr("+-0123456789.eE", *q) != nullptr)) ++q;
        if (q == p) return false;
        const std::string t(p, q);
        char* end = nullptr;
        v.num = strtod(t.c_str(), &end);
        if (!end || *end) return false;
        v.kind = NUM;
        p = q;
        return true;
    }
};

}  // namespace nt
