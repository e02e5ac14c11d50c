// A small JSON reader for model descriptions (config.json, the header of a safetensors file): objects, arrays, strings, numbers, true / false / null.
#pragma once

#include <cstdlib>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace pi {

struct json {
    enum kind_t { NUL, BOOL, NUM, STR, ARR, OBJ } kind = NUL;
    bool b = false; double num = 0.0; std::string str;
    std::vector<json> arr;
    std::vector<std::pair<std::string, json>> obj;            // (file order is kept)

    bool is_null() const { return kind == NUL; }
    bool is_obj() const { return kind == OBJ; }
    bool is_arr() const { return kind == ARR; }
    bool is_num() const { return kind == NUM; }
    bool is_str() const { return kind == STR; }
    const json * find(const std::string & key) const { for (const auto & kv : obj) if (kv.first == key) return &kv.second; return nullptr; }
    bool has(const std::string & key) const { const json * j = find(key); return j && !j->is_null(); }
    // a.b.c path lookup; nullptr when any step is missing
    const json * at(const std::string & path) const {
        const json * j = this; size_t p = 0;
        while (j && p <= path.size()) { const size_t q = path.find('.', p); const std::string key = path.substr(p, q == std::string::npos ? q : q - p); j = j->find(key); if (q == std::string::npos) break; p = q + 1; }
        return j;
    }

    static bool parse(const std::string & text, json & out, std::string & err) {
        size_t p = 0;
        if (!value(text, p, out, err, 0)) return false;
        ws(text, p);
        if (p != text.size()) { err = "trailing characters after the JSON value at byte " + std::to_string(p); return false; }
        return true;
    }

private:
    static void ws(const std::string & s, size_t & p) { while (p < s.size() && (s[p] == ' ' || s[p] == '\n' || s[p] == '\t' || s[p] == '\r')) p++; }
    static bool fail(std::string & err, const char * what, size_t p) { err = std::string(what) + " at byte " + std::to_string(p); return false; }
    static bool string(const std::string & s, size_t & p, std::string & out, std::string & err) {
        if (s[p] != '"') return fail(err, "expected a string", p);
        p++; out.clear();
        while (p < s.size() && s[p] != '"') {
            if (s[p] == '\\') {
                if (++p >= s.size()) break;
                switch (s[p]) {
                    case 'n': out += '\n'; break; case 't': out += '\t'; break; case 'r': out += '\r'; break; case 'b': out += '\b'; break; case 'f': out += '\f'; break;
                    case 'u': {
                        if (p + 4 >= s.size()) return fail(err, "short \\u escape", p);
                        const unsigned c = (unsigned) strtoul(s.substr(p + 1, 4).c_str(), nullptr, 16); p += 4;
                        if (c < 0x80) out += (char) c; else if (c < 0x800) { out += (char) (0xC0 | (c >> 6)); out += (char) (0x80 | (c & 63)); } else { out += (char) (0xE0 | (c >> 12)); out += (char) (0x80 | ((c >> 6) & 63)); out += (char) (0x80 | (c & 63)); }
                        break;
                    }
                    default: out += s[p];
                }
                p++;
            } else out += s[p++];
        }
        if (p >= s.size()) return fail(err, "unterminated string", p);
        p++;
        return true;
    }
    static bool value(const std::string & s, size_t & p, json & out, std::string & err, int depth) {
        if (depth > 64) return fail(err, "nesting too deep", p);
        ws(s, p);
        if (p >= s.size()) return fail(err, "unexpected end", p);
        const char c = s[p];
        if (c == '{') {
            out.kind = OBJ; p++; ws(s, p);
            if (p < s.size() && s[p] == '}') { p++; return true; }
            while (true) {
                ws(s, p);
                std::string key;
                if (p >= s.size() || !string(s, p, key, err)) return err.empty() ? fail(err, "expected a key", p) : false;
                ws(s, p);
                if (p >= s.size() || s[p] != ':') return fail(err, "expected ':'", p);
                p++;
                json v;
                if (!value(s, p, v, err, depth + 1)) return false;
                out.obj.emplace_back(std::move(key), std::move(v));
                ws(s, p);
                if (p < s.size() && s[p] == ',') { p++; continue; }
                if (p < s.size() && s[p] == '}') { p++; return true; }
                return fail(err, "expected ',' or '}'", p);
            }
        }
        if (c == '[') {
            out.kind = ARR; p++; ws(s, p);
            if (p < s.size() && s[p] == ']') { p++; return true; }
            while (true) {
                json v;
                if (!value(s, p, v, err, depth + 1)) return false;
                out.arr.push_back(std::move(v));
                ws(s, p);
                if (p < s.size() && s[p] == ',') { p++; continue; }
                if (p < s.size() && s[p] == ']') { p++; return true; }
                return fail(err, "expected ',' or ']'", p);
            }
        }
        if (c == '"') { out.kind = STR; return string(s, p, out.str, err); }
        if (s.compare(p, 4, "true") == 0) { out.kind = BOOL; out.b = true; p += 4; return true; }
        if (s.compare(p, 5, "false") == 0) { out.kind = BOOL; out.b = false; p += 5; return true; }
        if (s.compare(p, 4, "null") == 0) { out.kind = NUL; p += 4; return true; }
        {
            const char * b = s.c_str() + p; char * e = nullptr;
            const double v = strtod(b, &e);
            if (e == b) return fail(err, "unexpected character", p);
            out.kind = NUM; out.num = v; p += (size_t) (e - b);
            return true;
        }
    }
};

}  // namespace pi
