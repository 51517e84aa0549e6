// The quant-table semantics of turboexl3 (table/config.zig, table/table.zig) behind the C ABI, free of any array
// library: which blocks of a pack's config the table claims, what validation names, the bill, the checks a trunk
// linear and a routed bank pass when they load, and `matmul` / `moe` / `swiglu` over the loaded weights.

#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "t3_host.hpp"

namespace t3 {
namespace {

// ---- a small JSON reader: objects, strings, numbers (whole or not, as the reference's parser tells them apart),
// arrays, true / false / null. Anything malformed parses as "not an object".
struct Json {
    enum Kind { kNull, kBool, kInt, kFloat, kString, kArray, kObject } kind = kNull;
    bool b = false;
    int64_t i = 0;
    double f = 0.0;
    std::string s;
    std::vector<Json> items;
    std::map<std::string, Json> fields;

    const Json* get(const char* key) const {
        if (kind != kObject) return nullptr;
        const auto it = fields.find(key);
        return it == fields.end() ? nullptr : &it->second;
    }
};

struct Parser {
    const char* p;
    const char* end;
    int depth = 0;

    void ws() {
        while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) ++p;
    }
    bool lit(const char* word) {
        const size_t n = std::strlen(word);
        if (static_cast<size_t>(end - p) < n || std::strncmp(p, word, n) != 0) return false;
        p += n;
        return true;
    }
    bool string(std::string* out) {
        if (p >= end || *p != '"') return false;
        ++p;
        while (p < end && *p != '"') {
            if (*p == '\\') {
                if (++p >= end) return false;
                switch (*p) {
                    case 'n': out->push_back('\n'); break;
                    case 't': out->push_back('\t'); break;
                    case 'r': out->push_back('\r'); break;
                    case 'b': out->push_back('\b'); break;
                    case 'f': out->push_back('\f'); break;
                    case 'u':  // kept as written: no key or value this table reads has an escape
                        out->append("\\u");
                        break;
                    default: out->push_back(*p); break;
                }
                ++p;
            } else {
                out->push_back(*p++);
            }
        }
        if (p >= end) return false;
        ++p;
        return true;
    }
    bool number(Json* out) {
        const char* s = p;
        bool whole = true;
        if (p < end && *p == '-') ++p;
        if (p >= end || *p < '0' || *p > '9') return false;
        while (p < end && *p >= '0' && *p <= '9') ++p;
        if (p < end && *p == '.') {
            whole = false;
            ++p;
            if (p >= end || *p < '0' || *p > '9') return false;
            while (p < end && *p >= '0' && *p <= '9') ++p;
        }
        if (p < end && (*p == 'e' || *p == 'E')) {
            whole = false;
            ++p;
            if (p < end && (*p == '+' || *p == '-')) ++p;
            if (p >= end || *p < '0' || *p > '9') return false;
            while (p < end && *p >= '0' && *p <= '9') ++p;
        }
        const std::string text(s, p);
        if (whole && text.size() <= 18) {
            out->kind = Json::kInt;
            out->i = std::strtoll(text.c_str(), nullptr, 10);
        } else {
            out->kind = Json::kFloat;
            out->f = std::strtod(text.c_str(), nullptr);
        }
        return true;
    }
    bool value(Json* out) {
        if (++depth > 64) return false;
        ws();
        if (p >= end) return false;
        bool ok = false;
        if (*p == '{') {
            ++p;
            out->kind = Json::kObject;
            ws();
            if (p < end && *p == '}') {
                ++p;
                ok = true;
            } else {
                for (;;) {
                    ws();
                    std::string key;
                    if (!string(&key)) break;
                    ws();
                    if (p >= end || *p != ':') break;
                    ++p;
                    Json v;
                    if (!value(&v)) break;
                    out->fields[key] = std::move(v);  // a repeated key keeps its last value
                    ws();
                    if (p < end && *p == ',') {
                        ++p;
                        continue;
                    }
                    if (p < end && *p == '}') {
                        ++p;
                        ok = true;
                    }
                    break;
                }
            }
        } else if (*p == '[') {
            ++p;
            out->kind = Json::kArray;
            ws();
            if (p < end && *p == ']') {
                ++p;
                ok = true;
            } else {
                for (;;) {
                    Json v;
                    if (!value(&v)) break;
                    out->items.push_back(std::move(v));
                    ws();
                    if (p < end && *p == ',') {
                        ++p;
                        continue;
                    }
                    if (p < end && *p == ']') {
                        ++p;
                        ok = true;
                    }
                    break;
                }
            }
        } else if (*p == '"') {
            out->kind = Json::kString;
            ok = string(&out->s);
        } else if (lit("true")) {
            out->kind = Json::kBool;
            out->b = true;
            ok = true;
        } else if (lit("false")) {
            out->kind = Json::kBool;
            ok = true;
        } else if (lit("null")) {
            ok = true;
        } else {
            ok = number(out);
        }
        --depth;
        return ok;
    }
};

// the text parsed as one JSON object, or null
std::unique_ptr<Json> parse_object(const char* text) {
    if (!text) return nullptr;
    Parser ps{text, text + std::strlen(text)};
    auto root = std::make_unique<Json>();
    if (!ps.value(root.get())) return nullptr;
    ps.ws();
    if (ps.p != ps.end || root->kind != Json::kObject) return nullptr;
    return root;
}

// table/config.zig:88-93: a routed bank set's block declares its rate `k`; a dense trunk's does not
int kind_of(const Json& o) {
    const Json* f = o.get("format");
    if (!f || f->kind != Json::kString || f->s != "exl3") return -1;
    return o.get("k") ? T3_BLOCK_BANK : T3_BLOCK_TRUNK;
}

// table/config.zig:95-106: `k` as halfwords a tile: an even whole number in 16..128 (fractional k included)
bool rate_of(const Json& k, uint32_t* n) {
    double scaled;
    if (k.kind == Json::kInt) scaled = static_cast<double>(k.i) * 16.0;
    else if (k.kind == Json::kFloat) scaled = k.f * 16.0;
    else return false;
    const double whole = std::round(scaled);
    if (std::fabs(scaled - whole) > 1e-6 || whole < 16 || whole > 128) return false;
    const uint32_t v = static_cast<uint32_t>(whole);
    if (v % 2u != 0u) return false;
    *n = v;
    return true;
}

// table/config.zig:36-52
int32_t parse_block(const char* json, t3_block* out) {
    const auto o = parse_object(json);
    if (!o) return T3_NotExl3;
    t3_block b = {0, 0, 16, 0};
    b.kind = kind_of(*o);
    if (b.kind < 0) return T3_NotExl3;
    if (const Json* c = o->get("codebook")) {
        if (c->kind != Json::kString) return T3_Exl3CodebookUnsupported;
        if (c->s == "mul1") b.codebook = 0;
        else if (c->s == "mcg") b.codebook = 1;
        else return T3_Exl3CodebookUnsupported;
    } else if (b.kind == T3_BLOCK_BANK) {
        return T3_Exl3CodebookUnsupported;
    }
    if (const Json* w = o->get("window")) {
        if (w->kind != Json::kInt || w->i < 8 || w->i > 16) return T3_Exl3WindowUnsupported;
        b.window_bits = static_cast<int32_t>(w->i);
    }
    if (b.kind == T3_BLOCK_BANK) {
        uint32_t n = 0;
        if (!rate_of(*o->get("k"), &n)) return T3_Exl3RateUnsupported;
        b.n = static_cast<int32_t>(n);
    }
    *out = b;
    return T3_OK;
}

// the text config of a config root: `text_config` when it nests one, else the root (table/config.zig:141-146)
const Json* text_of(const Json* cfg) {
    if (!cfg) return nullptr;
    const Json* t = cfg->get("text_config");
    return t && t->kind == Json::kObject ? t : cfg;
}

// table/config.zig:110-117: a fully EXL3 Qwen3.8 pack
bool profile(const Json* cfg) {
    if (!cfg || !cfg->get("trunk_quant")) return false;
    for (const Json* o : {cfg, text_of(cfg)}) {
        const Json* mt = o ? o->get("model_type") : nullptr;
        if (mt && mt->kind == Json::kString && (mt->s == "qwen4_exp" || mt->s == "qwen4_exp_text")) return true;
    }
    return false;
}

// table/config.zig:121-132: a clamped SwiGLU
bool clamped(const Json* cfg) {
    for (const Json* o : {cfg, text_of(cfg)}) {
        const Json* v = o ? o->get("swiglu_limit") : nullptr;
        if (!v) continue;
        if ((v->kind == Json::kInt && v->i > 0) || (v->kind == Json::kFloat && v->f > 0)) return true;
    }
    return false;
}

void put_why(char* why, size_t cap, const char* text) {
    if (why && cap > 0) std::snprintf(why, cap, "%s", text);
}

int32_t refuse(int32_t kind, char* why, size_t cap, const char* text) {
    put_why(why, cap, text);
    return kind;
}

// table/table.zig:591-593: a missing tensor failed; everything else is unsupported
int32_t verdict_of(int32_t status, char* why, size_t cap) {
    if (status == T3_OK) {
        put_why(why, cap, "");
        return T3_VERDICT_OK;
    }
    put_why(why, cap, t3_error_name(status));
    return status == T3_MissingWeight || status == T3_HipFailed ? T3_VERDICT_FAILED : T3_VERDICT_UNSUPPORTED;
}

bool shape_is(const t3_array& a, std::initializer_list<int64_t> dims) {
    if (a.ndim != static_cast<int32_t>(dims.size())) return false;
    int i = 0;
    for (const int64_t d : dims)
        if (a.shape[i++] != d) return false;
    return true;
}

void fill(t3_weight* out, const t3_array& t, const t3_array& suh, const t3_array& svh, const t3_block& b, int64_t n) {
    out->w = t;
    out->scales = suh;
    out->biases = svh;
    out->layout = b.codebook;
    out->flags = b.window_bits;
    out->block = static_cast<int32_t>(n);
}

bool decode_of(const t3_weight* w, t3_decode* dec) {
    if (!w || !w->w.data || (w->layout != 0 && w->layout != 1) || w->flags < 8 || w->flags > 16) return false;
    dec->codebook = w->layout;
    dec->window_bits = w->flags;
    return true;
}

t3_proj proj_of(const t3_weight* w) { return t3_proj{w->w, w->scales, w->biases}; }

}  // namespace
}  // namespace t3

extern "C" {

int32_t t3_table_parse_block(const char* block_json, t3_block* out) {
    if (!out) return T3_BadArgs;
    return t3::parse_block(block_json, out);
}

int32_t t3_table_claims(const char* block_json, const char* config_json, int32_t matrix_gate) {
    const auto o = t3::parse_object(block_json);
    if (!o) return T3_CLAIM_NO;
    const int kind = t3::kind_of(*o);
    if (kind < 0) return T3_CLAIM_NO;
    // a trunk block is this table's alone; validation names what it lacks (table/config.zig:64-67)
    if (kind == T3_BLOCK_TRUNK) return T3_CLAIM_BY_MARKER;
    t3_block b;
    if (t3::parse_block(block_json, &b) != T3_OK) return T3_CLAIM_NO;
    const auto cfg = t3::parse_object(config_json);
    if (!t3::profile(cfg.get()) || !matrix_gate || t3::clamped(cfg.get())) return T3_CLAIM_NO;
    return T3_CLAIM_BY_MARKER;
}

int32_t t3_table_validate(const char* block_json, const char* config_json, char* why, size_t why_bytes) {
    t3_block b;
    if (const int32_t st = t3::parse_block(block_json, &b); st != T3_OK)
        return t3::refuse(T3_VERDICT_UNSUPPORTED, why, why_bytes, t3_error_name(st));
    if (b.kind == T3_BLOCK_BANK) {
        const auto cfg = t3::parse_object(config_json);
        const t3::Json* text = t3::text_of(cfg.get());
        const t3::Json* k = text ? text->get("num_experts_per_tok") : nullptr;
        if (k && k->kind == t3::Json::kInt && k->i > T3_REDUCE_MAX_TOPK)
            return t3::refuse(T3_VERDICT_UNSUPPORTED, why, why_bytes, "Exl3TopKExceedsReduceBank");
    }
    t3::put_why(why, why_bytes, "");
    return T3_VERDICT_OK;
}

uint64_t t3_table_bill(const char* block_json, const char* model_dir, uint64_t stored) {
    (void)block_json;
    (void)model_dir;
    return stored;
}

int32_t t3_table_load_tensor(const t3_block* block, const t3_array* weight, const t3_array* scales,
                             const t3_array* biases, uint32_t in_dim, t3_weight* out, char* why, size_t why_bytes) {
    if (!block || !out) return t3::refuse(T3_VERDICT_FAILED, why, why_bytes, "turboexl3: the format is not open");
    if (block->kind != T3_BLOCK_TRUNK)
        return t3::refuse(T3_VERDICT_UNSUPPORTED, why, why_bytes, "turboexl3: dense linears load under the trunk_quant block");
    // table/table.zig:128-145
    const auto check = [&]() -> int32_t {
        if (!t3::array_ok(weight) || !t3::array_ok(scales) || !t3::array_ok(biases)) return T3_MissingWeight;
        const t3_array& t = *weight;
        if (t.ndim != 3 || (t.dtype != T3_U16 && t.dtype != T3_I16) || t.shape[0] <= 0 || t.shape[1] <= 0)
            return T3_Exl3TrellisGeometry;
        if (!t3::rate_ok(t.shape[2])) return T3_Exl3RateUnsupported;
        const int64_t in = t.shape[0] * 16, width = t.shape[1] * 16;
        if (in % 128 != 0 || width % 128 != 0) return T3_Exl3WidthNotMultipleOf128;
        if (in_dim != 0 && in_dim != in) return T3_Exl3TrellisGeometry;
        if (!t3::shape_is(*scales, {in}) || !t3::shape_is(*biases, {width})) return T3_Exl3SideGeometry;
        if (scales->dtype != T3_F16 || biases->dtype != T3_F16) return T3_Exl3SideDtype;
        t3::fill(out, t, *scales, *biases, *block, t.shape[2]);
        return T3_OK;
    };
    return t3::verdict_of(check(), why, why_bytes);
}

int32_t t3_table_load_bank(const t3_block* block, const t3_array* trellis, const t3_array* suh, const t3_array* svh,
                           uint32_t in_dim, t3_weight* out, char* why, size_t why_bytes) {
    if (!block || !out) return t3::refuse(T3_VERDICT_FAILED, why, why_bytes, "turboexl3: the format is not open");
    if (block->kind != T3_BLOCK_BANK)
        return t3::refuse(T3_VERDICT_UNSUPPORTED, why, why_bytes, "turboexl3: routed banks load under the expert_quant block");
    // table/table.zig:157-174
    const auto check = [&]() -> int32_t {
        if (!t3::array_ok(trellis) || !t3::array_ok(suh) || !t3::array_ok(svh)) return T3_MissingWeight;
        const t3_array& t = *trellis;
        if (t.ndim != 4 || t.shape[0] <= 0 || t.shape[1] <= 0 || t.shape[2] <= 0) return T3_Exl3TrellisGeometry;
        const int64_t experts = t.shape[0], in = t.shape[1] * 16, width = t.shape[2] * 16;
        if (in_dim != 0 && in_dim != in) return T3_Exl3TrellisGeometry;
        if (!t3::rate_ok(block->n)) return T3_Exl3RateUnsupported;
        if (t.dtype != T3_U16 || !t3_trellis_admitted(t.shape, t.ndim, experts, in, width, block->n))
            return T3_Exl3TrellisGeometry;
        if (!t3::shape_is(*suh, {experts, in}) || !t3::shape_is(*svh, {experts, width})) return T3_Exl3SideGeometry;
        if (suh->dtype != T3_F16 || svh->dtype != T3_F16) return T3_Exl3SideDtype;
        t3::fill(out, t, *suh, *svh, *block, t.shape[3]);
        return T3_OK;
    };
    return t3::verdict_of(check(), why, why_bytes);
}

int32_t t3_table_matmul(t3_stream stream, const t3_weight* w, const t3_array* x, t3_array* y, void* workspace,
                        size_t workspace_bytes, char* why, size_t why_bytes) {
    const t3::ConfigScope one_config;
    t3_decode dec;
    if (!t3::decode_of(w, &dec)) return t3::refuse(T3_VERDICT_FAILED, why, why_bytes, "turboexl3: a weight without its decode");
    return t3::verdict_of(t3_linear(stream, x, &w->w, &w->scales, &w->biases, dec, y, workspace, workspace_bytes), why,
                          why_bytes);
}

int32_t t3_table_matmul_workspace_bytes(const t3_weight* w, const t3_array* x, size_t* bytes) {
    const t3::ConfigScope one_config;
    t3_decode dec;
    if (!t3::decode_of(w, &dec)) return T3_BadArgs;
    return t3_linear_workspace_bytes(x, &w->w, dec, bytes);
}

int32_t t3_table_moe(char* why, size_t why_bytes) {
    // table/table.zig:203-205
    return t3::refuse(T3_VERDICT_UNSUPPORTED, why, why_bytes, "turboexl3: a layer's banks run as one routed SwiGLU (swiglu)");
}

int32_t t3_table_swiglu(t3_stream stream, const t3_weight* gate, const t3_weight* up, const t3_weight* down,
                        const t3_array* x, const t3_array* inds, const t3_array* scores, int32_t limit,
                        int32_t verify_rows, t3_array* y, void* workspace, size_t workspace_bytes, char* why,
                        size_t why_bytes) {
    const t3::ConfigScope one_config;
    // table/table.zig:210-222
    t3_decode dec, du, dd;
    if (!t3::decode_of(gate, &dec)) return t3::refuse(T3_VERDICT_FAILED, why, why_bytes, "turboexl3: a bank without its decode");
    if (!t3::decode_of(up, &du) || !t3::decode_of(down, &dd) || du.codebook != dec.codebook ||
        du.window_bits != dec.window_bits || dd.codebook != dec.codebook || dd.window_bits != dec.window_bits)
        return t3::refuse(T3_VERDICT_UNSUPPORTED, why, why_bytes, "turboexl3: a layer's banks decode differently");
    const t3_bank bank = {t3::proj_of(gate), t3::proj_of(up), t3::proj_of(down)};
    const int32_t st = limit > 0 ? t3_moe_clamped(stream, x, &bank, inds, scores, dec, limit, y, workspace, workspace_bytes)
                                 : t3_moe(stream, x, &bank, inds, scores, dec, verify_rows, y, workspace, workspace_bytes);
    return t3::verdict_of(st, why, why_bytes);
}

int32_t t3_table_swiglu_workspace_bytes(const t3_weight* gate, const t3_weight* up, const t3_weight* down,
                                        const t3_array* x, const t3_array* inds, size_t* bytes) {
    const t3::ConfigScope one_config;
    if (!gate || !up || !down) return T3_BadArgs;
    const t3_bank bank = {t3::proj_of(gate), t3::proj_of(up), t3::proj_of(down)};
    return t3_moe_workspace_bytes(x, &bank, inds, nullptr, bytes);
}

}  // extern "C"
