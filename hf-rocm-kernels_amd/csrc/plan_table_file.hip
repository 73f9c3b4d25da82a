// hfrk_plan_table_load: install a plan-table file (the JSON that hf_rocm_kernels/plan_table.py and the grid-search
// tool write) from a host that has no Python -- the C counterpart of plan_table.load.  Host code only.
//
// The file is one JSON object {"format": "hfrk-plan-table-1", "entries": [{"m", "n", "k", "packed", "plan": {the
// eight fields of hfrk_gemm_plan}, ...}, ...]}; members this loader does not know (measurements, provenance) are
// skipped.  Every entry goes through hfrk_plan_table_set, which validates the plan for its shape.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <utility>
#include <vector>

#include "hfrk_internal.h"

namespace hfrk {
namespace {

struct Json {
    enum Kind { kNull, kBool, kNumber, kString, kArray, kObject } kind = kNull;
    bool boolean = false;
    double number = 0.0;
    std::string text;
    std::vector<Json> items;
    std::vector<std::pair<std::string, Json>> members;

    const Json* get(const char* key) const {
        if (kind != kObject) return nullptr;
        for (const auto& m : members)
            if (m.first == key) return &m.second;
        return nullptr;
    }
};

// Recursive-descent reader for the JSON grammar (RFC 8259); \u escapes above 0x7f are kept as '?', which no key or
// value this loader looks at contains.
class JsonReader {
  public:
    JsonReader(const char* begin, const char* end) : p_(begin), end_(end) {}

    bool parse(Json* out) {
        if (!value(out, 0)) return false;
        skip_space();
        return p_ == end_;
    }

  private:
    static constexpr int kMaxDepth = 32;
    const char* p_;
    const char* end_;

    void skip_space() {
        while (p_ < end_ && (*p_ == ' ' || *p_ == '\t' || *p_ == '\n' || *p_ == '\r')) ++p_;
    }
    bool literal(const char* word) {
        const size_t len = strlen(word);
        if ((size_t)(end_ - p_) < len || memcmp(p_, word, len) != 0) return false;
        p_ += len;
        return true;
    }
    bool string(std::string* out) {
        if (p_ >= end_ || *p_ != '"') return false;
        ++p_;
        while (p_ < end_ && *p_ != '"') {
            char c = *p_++;
            if ((unsigned char)c < 0x20) return false;
            if (c == '\\') {
                if (p_ >= end_) return false;
                const char e = *p_++;
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
                        if (end_ - p_ < 4) return false;
                        unsigned code = 0;
                        for (int i = 0; i < 4; ++i) {
                            const char h = *p_++;
                            code <<= 4;
                            if (h >= '0' && h <= '9') code |= (unsigned)(h - '0');
                            else if (h >= 'a' && h <= 'f') code |= (unsigned)(h - 'a' + 10);
                            else if (h >= 'A' && h <= 'F') code |= (unsigned)(h - 'A' + 10);
                            else return false;
                        }
                        c = code < 0x80 ? (char)code : '?';
                        break;
                    }
                    default: return false;
                }
            }
            out->push_back(c);
        }
        if (p_ >= end_) return false;
        ++p_;  // closing quote
        return true;
    }
    bool number(double* out) {
        const char* start = p_;
        if (p_ < end_ && *p_ == '-') ++p_;
        if (p_ >= end_ || *p_ < '0' || *p_ > '9') return false;
        if (*p_ == '0') ++p_;
        else while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_;
        if (p_ < end_ && *p_ == '.') {
            ++p_;
            if (p_ >= end_ || *p_ < '0' || *p_ > '9') return false;
            while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_;
        }
        if (p_ < end_ && (*p_ == 'e' || *p_ == 'E')) {
            ++p_;
            if (p_ < end_ && (*p_ == '+' || *p_ == '-')) ++p_;
            if (p_ >= end_ || *p_ < '0' || *p_ > '9') return false;
            while (p_ < end_ && *p_ >= '0' && *p_ <= '9') ++p_;
        }
        *out = strtod(std::string(start, p_).c_str(), nullptr);
        return true;
    }
    bool value(Json* out, int depth) {
        if (depth > kMaxDepth) return false;
        skip_space();
        if (p_ >= end_) return false;
        switch (*p_) {
            case '{': {
                out->kind = Json::kObject;
                ++p_;
                skip_space();
                if (p_ < end_ && *p_ == '}') { ++p_; return true; }
                for (;;) {
                    skip_space();
                    std::string key;
                    if (!string(&key)) return false;
                    skip_space();
                    if (p_ >= end_ || *p_++ != ':') return false;
                    Json member;
                    if (!value(&member, depth + 1)) return false;
                    out->members.emplace_back(std::move(key), std::move(member));
                    skip_space();
                    if (p_ >= end_) return false;
                    if (*p_ == ',') { ++p_; continue; }
                    if (*p_ == '}') { ++p_; return true; }
                    return false;
                }
            }
            case '[': {
                out->kind = Json::kArray;
                ++p_;
                skip_space();
                if (p_ < end_ && *p_ == ']') { ++p_; return true; }
                for (;;) {
                    Json item;
                    if (!value(&item, depth + 1)) return false;
                    out->items.push_back(std::move(item));
                    skip_space();
                    if (p_ >= end_) return false;
                    if (*p_ == ',') { ++p_; continue; }
                    if (*p_ == ']') { ++p_; return true; }
                    return false;
                }
            }
            case '"': out->kind = Json::kString; return string(&out->text);
            case 't': out->kind = Json::kBool; out->boolean = true; return literal("true");
            case 'f': out->kind = Json::kBool; out->boolean = false; return literal("false");
            case 'n': out->kind = Json::kNull; return literal("null");
            default: out->kind = Json::kNumber; return number(&out->number);
        }
    }
};

// an integer member that fits an int, exactly
bool int_member(const Json& object, const char* key, int* out) {
    const Json* v = object.get(key);
    if (!v || v->kind != Json::kNumber) return false;
    if (!(v->number >= -2147483648.0 && v->number <= 2147483647.0) || v->number != (double)(long long)v->number) return false;
    *out = (int)v->number;
    return true;
}

bool read_file(const char* path, std::string* out) {
    constexpr long kMaxBytes = 16L << 20;
    FILE* f = fopen(path, "rb");
    if (!f) return false;
    bool ok = false;
    if (fseek(f, 0, SEEK_END) == 0) {
        const long size = ftell(f);
        if (size >= 0 && size <= kMaxBytes && fseek(f, 0, SEEK_SET) == 0) {
            out->resize((size_t)size);
            ok = size == 0 || fread(&(*out)[0], 1, (size_t)size, f) == (size_t)size;
        }
    }
    fclose(f);
    return ok;
}

}  // namespace
}  // namespace hfrk

extern "C" int hfrk_plan_table_load(const char* path, int strict, int* installed) {
    using namespace hfrk;
    if (installed) *installed = 0;
    if (!path) return HFRK_BAD_SHAPE;
    std::string text;
    if (!read_file(path, &text)) return HFRK_BAD_FILE;
    Json root;
    if (!JsonReader(text.data(), text.data() + text.size()).parse(&root) || root.kind != Json::kObject) return HFRK_BAD_FILE;
    const Json* format = root.get("format");
    if (!format || format->kind != Json::kString || format->text != "hfrk-plan-table-1") return HFRK_BAD_FILE;
    const Json* entries = root.get("entries");
    if (!entries || entries->kind != Json::kArray) return HFRK_BAD_FILE;
    int count = 0;
    for (const Json& e : entries->items) {
        int m, n, k, packed = 0;
        hfrk_gemm_plan plan;
        const Json* p = e.get("plan");
        const Json* pk = e.get("packed");
        bool ok = e.kind == Json::kObject && p && p->kind == Json::kObject && int_member(e, "m", &m) && int_member(e, "n", &n) &&
                  int_member(e, "k", &k) && int_member(*p, "m_tiles", &plan.m_tiles) && int_member(*p, "wn", &plan.wn) &&
                  int_member(*p, "wk", &plan.wk) && int_member(*p, "ch", &plan.ch) && int_member(*p, "grid", &plan.grid) &&
                  int_member(*p, "panels", &plan.panels) && int_member(*p, "slabs", &plan.slabs) &&
                  int_member(*p, "lds_bytes", &plan.lds_bytes);
        if (ok && pk) {
            if (pk->kind == Json::kBool) packed = pk->boolean ? 1 : 0;
            else if (pk->kind == Json::kNumber) packed = pk->number != 0.0 ? 1 : 0;
            else ok = false;
        }
        if (!ok) {
            if (strict) return HFRK_BAD_FILE;
            continue;
        }
        const int rc = hfrk_plan_table_set(m, n, k, packed, &plan);
        if (rc == HFRK_SUCCESS) ++count;
        else if (strict) return rc;
        if (installed) *installed = count;
    }
    return HFRK_SUCCESS;
}
