// json_lite.h — a small JSON reader (objects, arrays, strings, numbers, true / false / null) for model descriptions
// (a checkpoint folder's config.json, the header of a safetensors file).  Header-only; parse errors return false.
#ifndef JSON_LITE_H
#define JSON_LITE_H
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

struct json_value {
    enum kind_t { NUL, BOOL, NUM, STR, ARR, OBJ } kind = NUL;
    bool b = false;
    double num = 0.0;
    std::string str;
    std::vector<json_value> arr;
    std::vector<std::pair<std::string, json_value>> obj;  // in file order

    const json_value * get(const char * key) const {
        if (kind != OBJ) return nullptr;
        for (auto & kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
    bool is_null() const { return kind == NUL; }
    double number(double dflt) const { return kind == NUM ? num : (kind == BOOL ? (b ? 1.0 : 0.0) : dflt); }
    // obj.path("a", "b"): nested lookup, nullptr when a step is missing or null
    const json_value * path(const char * k0, const char * k1 = nullptr, const char * k2 = nullptr) const {
        const json_value * v = get(k0);
        if (v && k1) v = v->get(k1);
        if (v && k2) v = v->get(k2);
        return (v && v->kind != NUL) ? v : nullptr;
    }
};

class json_parser {
  public:
    static bool parse(const char * text, size_t n, json_value & out) {
        json_parser p(text, n);
        p.ws();
        if (!p.value(out, 0)) return false;
        p.ws();
        return p.at == p.n;
    }

  private:
    const char * s;
    size_t n, at = 0;
    json_parser(const char * text, size_t len) : s(text), n(len) {}
    void ws() {
        while (at < n && (s[at] == ' ' || s[at] == '\t' || s[at] == '\n' || s[at] == '\r')) ++at;
    }
    bool lit(const char * w) {
        const size_t l = strlen(w);
        if (at + l > n || memcmp(s + at, w, l) != 0) return false;
        at += l;
        return true;
    }
    bool string(std::string & out) {
        if (at >= n || s[at] != '"') return false;
        ++at;
        out.clear();
        while (at < n && s[at] != '"') {
            char c = s[at++];
            if (c == '\\') {
                if (at >= n) return false;
                const char e = s[at++];
                switch (e) {
                    case 'n': out += '\n'; break;
                    case 't': out += '\t'; break;
                    case 'r': out += '\r'; break;
                    case 'b': out += '\b'; break;
                    case 'f': out += '\f'; break;
                    case 'u': {
                        if (at + 4 > n) return false;
                        const unsigned cp = (unsigned) strtoul(std::string(s + at, 4).c_str(), nullptr, 16);
                        at += 4;
                        if (cp < 0x80) out += (char) cp;
                        else if (cp < 0x800) { out += (char) (0xC0 | (cp >> 6)); out += (char) (0x80 | (cp & 0x3F)); }
                        else { out += (char) (0xE0 | (cp >> 12)); out += (char) (0x80 | ((cp >> 6) & 0x3F)); out += (char) (0x80 | (cp & 0x3F)); }
                    } break;
                    default: out += e;
                }
            } else out += c;
        }
        if (at >= n) return false;
        ++at;
        return true;
    }
    bool value(json_value & v, int depth) {
        if (depth > 64 || at >= n) return false;
        const char c = s[at];
        if (c == '{') {
            v.kind = json_value::OBJ;
            ++at;
            ws();
            if (at < n && s[at] == '}') { ++at; return true; }
            for (;;) {
                ws();
                std::string k;
                if (!string(k)) return false;
                ws();
                if (at >= n || s[at] != ':') return false;
                ++at;
                ws();
                v.obj.emplace_back(k, json_value());
                if (!value(v.obj.back().second, depth + 1)) return false;
                ws();
                if (at < n && s[at] == ',') { ++at; continue; }
                if (at < n && s[at] == '}') { ++at; return true; }
                return false;
            }
        }
        if (c == '[') {
            v.kind = json_value::ARR;
            ++at;
            ws();
            if (at < n && s[at] == ']') { ++at; return true; }
            for (;;) {
                ws();
                v.arr.emplace_back();
                if (!value(v.arr.back(), depth + 1)) return false;
                ws();
                if (at < n && s[at] == ',') { ++at; continue; }
                if (at < n && s[at] == ']') { ++at; return true; }
                return false;
            }
        }
        if (c == '"') { v.kind = json_value::STR; return string(v.str); }
        if (lit("true")) { v.kind = json_value::BOOL; v.b = true; return true; }
        if (lit("false")) { v.kind = json_value::BOOL; v.b = false; return true; }
        if (lit("null")) { v.kind = json_value::NUL; return true; }
        // number (also the non-standard NaN / Infinity spellings some writers emit are refused)
        size_t e = at;
        while (e < n && (strchr("+-0123456789.eE", s[e]) != nullptr)) ++e;
        if (e == at) return false;
        const std::string t(s + at, e - at);
        char * endp = nullptr;
        v.num = strtod(t.c_str(), &endp);
        if (!endp || *endp) return false;
        v.kind = json_value::NUM;
        at = e;
        return true;
    }
};
#endif
