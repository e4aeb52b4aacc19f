// Run-time loader and validator for the operator's knob file.
//
// The reference reads aristos_config.json with CMake's string(JSON ... GET) and turns each key into a
// compile definition (CMakeLists.txt:167-216); nothing validates the file against
// aristos_config.schema.json.  Here the same keys are read at run time and checked against the schema's
// domains (aristos_config.schema.json:5-71), relaxed only where moe355.h says so.
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>

#include "../../include/moe355.h"

namespace {

void set_err(char* err, size_t n, const char* fmt, ...) {
    if (!err || n == 0) return;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(err, n, fmt, ap);
    va_end(ap);
}

// A flat JSON object whose values are numbers or booleans; that is all the schema admits.
struct FlatJson {
    std::map<std::string, double> num;
    std::map<std::string, bool> integral;   // value was written without fraction or exponent
    std::string error;

    const char* p = nullptr;

    void ws() { while (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r') ++p; }

    bool parse_string(std::string& out) {
        if (*p != '"') { error = "expected '\"'"; return false; }
        ++p;
        out.clear();
        while (*p && *p != '"') {
            if (*p == '\\') {
                ++p;
                if (!*p) break;
                switch (*p) {
                    case 'n': out.push_back('\n'); break;
                    case 't': out.push_back('\t'); break;
                    case 'u': error = "\\u escapes are not supported in keys"; return false;
                    default: out.push_back(*p);
                }
                ++p;
            } else {
                out.push_back(*p++);
            }
        }
        if (*p != '"') { error = "unterminated string"; return false; }
        ++p;
        return true;
    }

    // skips any JSON value we do not interpret (strings, arrays, nested objects, null)
    bool skip_value() {
        ws();
        if (*p == '"') { std::string s; return parse_string(s); }
        if (*p == '{' || *p == '[') {
            const char open = *p, close = (*p == '{') ? '}' : ']';
            int depth = 0;
            while (*p) {
                if (*p == '"') { std::string s; if (!parse_string(s)) return false; continue; }
                if (*p == open) ++depth;
                if (*p == close) { --depth; if (depth == 0) { ++p; return true; } }
                ++p;
            }
            error = "unterminated container";
            return false;
        }
        if (!strncmp(p, "null", 4)) { p += 4; return true; }
        error = "unexpected token";
        return false;
    }

    bool parse(const char* text) {
        p = text;
        ws();
        if (*p != '{') { error = "top level must be an object"; return false; }
        ++p;
        ws();
        if (*p == '}') { ++p; return true; }
        for (;;) {
            ws();
            std::string key;
            if (!parse_string(key)) return false;
            ws();
            if (*p != ':') { error = "expected ':' after key \"" + key + "\""; return false; }
            ++p;
            ws();
            if (*p == '-' || (*p >= '0' && *p <= '9')) {
                char* end = nullptr;
                const double v = strtod(p, &end);
                if (end == p) { error = "bad number for \"" + key + "\""; return false; }
                bool integral_text = true;
                for (const char* q = p; q < end; ++q)
                    if (*q == '.' || *q == 'e' || *q == 'E') integral_text = false;
                if (num.count(key)) { error = "duplicate key \"" + key + "\""; return false; }
                num[key] = v;
                integral[key] = integral_text || (std::floor(v) == v);
                p = end;
            } else if (!strncmp(p, "true", 4)) {
                num[key] = 1; integral[key] = true; p += 4;
            } else if (!strncmp(p, "false", 5)) {
                num[key] = 0; integral[key] = true; p += 5;
            } else {
                if (!skip_value()) return false;   // "$schema", "$comment", ... are legal and ignored
            }
            ws();
            if (*p == ',') { ++p; continue; }
            if (*p == '}') { ++p; break; }
            error = "expected ',' or '}'";
            return false;
        }
        ws();
        if (*p) { error = "trailing characters after object"; return false; }
        return true;
    }
};

bool get_int(const FlatJson& j, const char* key, bool required, int32_t* out, char* err, size_t n, bool* present) {
    auto it = j.num.find(key);
    if (present) *present = it != j.num.end();
    if (it == j.num.end()) {
        if (required) { set_err(err, n, "missing required key \"%s\"", key); return false; }
        return true;
    }
    if (!j.integral.at(key) || std::fabs(it->second) > 2147483647.0) {
        set_err(err, n, "\"%s\" must be an integer", key);
        return false;
    }
    *out = (int32_t)it->second;
    return true;
}

}  // namespace

extern "C" {

int moe_config_default(moe_config* c) {
    if (!c) return MOE_ERR_BAD_ARGUMENT;
    // the values of the reference's own aristos_config.json:1-13
    c->capacity_factor = 1.0;
    c->drop_tokens = 0;
    c->expert_top_k = 1;
    c->is_training = 0;
    c->hidden_act = MOE_ACT_RELU;
    c->hidden_size = 1024;
    c->intermediate_size = 4096;
    c->micro_batch = 4;
    c->num_experts = 1;
    c->sequence_len = 2048;
    c->torch_dtype = MOE_DTYPE_F32;
    c->gate_fn = MOE_GATE_SOFTMAX;
    c->norm_topk_prob = 0;
    return MOE_OK;
}

int moe_config_validate(const moe_config* c, char* err, size_t n) {
    if (!c) return MOE_ERR_BAD_ARGUMENT;
    if (!(c->capacity_factor > 0.0) || !std::isfinite(c->capacity_factor)) {
        set_err(err, n, "capacity_factor must be a finite number > 0"); return MOE_ERR_BAD_CONFIG; }
    if (c->drop_tokens != 0 && c->drop_tokens != 1) { set_err(err, n, "drop_tokens must be 0 or 1"); return MOE_ERR_BAD_CONFIG; }
    if (c->is_training != 0 && c->is_training != 1) { set_err(err, n, "is_training must be 0 or 1"); return MOE_ERR_BAD_CONFIG; }
    if (c->expert_top_k < 1) { set_err(err, n, "expert_top_k must be >= 1"); return MOE_ERR_BAD_CONFIG; }
    if (c->num_experts < 1) { set_err(err, n, "num_experts must be >= 1"); return MOE_ERR_BAD_CONFIG; }
    if (c->expert_top_k > c->num_experts) { set_err(err, n, "expert_top_k exceeds num_experts"); return MOE_ERR_BAD_CONFIG; }
    if (c->hidden_act < 0 || c->hidden_act > 2) { set_err(err, n, "hidden_act must be 0 (relu), 1 (gelu) or 2 (swiglu)"); return MOE_ERR_BAD_CONFIG; }
    if (c->hidden_size < 64 || c->hidden_size % 64) { set_err(err, n, "hidden_size must be a positive multiple of 64"); return MOE_ERR_BAD_CONFIG; }
    if (c->intermediate_size < 64 || c->intermediate_size % 64) { set_err(err, n, "intermediate_size must be a positive multiple of 64"); return MOE_ERR_BAD_CONFIG; }
    if (c->micro_batch < 1) { set_err(err, n, "micro_batch must be >= 1"); return MOE_ERR_BAD_CONFIG; }
    if (c->sequence_len < 1) { set_err(err, n, "sequence_len must be >= 1"); return MOE_ERR_BAD_CONFIG; }
    if (c->torch_dtype < 0 || c->torch_dtype > 4) { set_err(err, n, "torch_dtype must be 0..4"); return MOE_ERR_BAD_CONFIG; }
    if (c->gate_fn != MOE_GATE_SOFTMAX && c->gate_fn != MOE_GATE_SIGMOID) { set_err(err, n, "gate_fn must be 0 (softmax) or 1 (sigmoid)"); return MOE_ERR_BAD_CONFIG; }
    if (c->norm_topk_prob != 0 && c->norm_topk_prob != 1) { set_err(err, n, "norm_topk_prob must be 0 or 1"); return MOE_ERR_BAD_CONFIG; }
    const int64_t S = (int64_t)c->micro_batch * c->sequence_len;
    // S * k against 2^30, without forming a product that could overflow
    if (S > ((int64_t)1 << 30) / c->expert_top_k) { set_err(err, n, "micro_batch*sequence_len*expert_top_k exceeds 2^30"); return MOE_ERR_BAD_CONFIG; }
    return MOE_OK;
}

int moe_config_from_json_string(const char* json, moe_config* c, char* err, size_t n) {
    if (!json || !c) return MOE_ERR_BAD_ARGUMENT;
    FlatJson j;
    if (!j.parse(json)) { set_err(err, n, "JSON: %s", j.error.c_str()); return MOE_ERR_BAD_CONFIG; }
    moe_config_default(c);
    // required keys: aristos_config.schema.json:60-71
    auto cf = j.num.find("capacity_factor");
    if (cf == j.num.end()) { set_err(err, n, "missing required key \"capacity_factor\""); return MOE_ERR_BAD_CONFIG; }
    c->capacity_factor = cf->second;
    bool has = false;
    if (!get_int(j, "drop_tokens", true, &c->drop_tokens, err, n, nullptr)) return MOE_ERR_BAD_CONFIG;
    // the schema types expert_top_k as "number" (schema:15-19); a fractional k has no meaning
    if (!get_int(j, "expert_top_k", true, &c->expert_top_k, err, n, nullptr)) return MOE_ERR_BAD_CONFIG;
    if (!get_int(j, "is_training", false, &c->is_training, err, n, nullptr)) return MOE_ERR_BAD_CONFIG;
    if (!get_int(j, "hidden_act", true, &c->hidden_act, err, n, nullptr)) return MOE_ERR_BAD_CONFIG;
    if (!get_int(j, "hidden_size", true, &c->hidden_size, err, n, nullptr)) return MOE_ERR_BAD_CONFIG;
    if (!get_int(j, "intermediate_size", true, &c->intermediate_size, err, n, nullptr)) return MOE_ERR_BAD_CONFIG;
    if (!get_int(j, "micro_batch", true, &c->micro_batch, err, n, nullptr)) return MOE_ERR_BAD_CONFIG;
    if (!get_int(j, "num_experts", true, &c->num_experts, err, n, nullptr)) return MOE_ERR_BAD_CONFIG;
    if (!get_int(j, "sequence_len", true, &c->sequence_len, err, n, nullptr)) return MOE_ERR_BAD_CONFIG;
    if (!get_int(j, "torch_dtype", true, &c->torch_dtype, err, n, nullptr)) return MOE_ERR_BAD_CONFIG;
    if (!get_int(j, "gate_fn", false, &c->gate_fn, err, n, nullptr)) return MOE_ERR_BAD_CONFIG;
    c->norm_topk_prob = c->expert_top_k > 1 ? 1 : 0;
    if (!get_int(j, "norm_topk_prob", false, &c->norm_topk_prob, err, n, &has)) return MOE_ERR_BAD_CONFIG;
    return moe_config_validate(c, err, n);
}

int moe_config_from_json_file(const char* path, moe_config* c, char* err, size_t n) {
    if (!path || !c) return MOE_ERR_BAD_ARGUMENT;
    FILE* f = fopen(path, "rb");
    if (!f) { set_err(err, n, "cannot open %s", path); return MOE_ERR_BAD_CONFIG; }
    std::string text;
    char buf[4096];
    size_t got;
    while ((got = fread(buf, 1, sizeof buf, f)) > 0) text.append(buf, got);
    fclose(f);
    return moe_config_from_json_string(text.c_str(), c, err, n);
}

int64_t moe_config_tokens(const moe_config* c) {
    return c ? (int64_t)c->micro_batch * c->sequence_len : 0;
}

// C = ceil(capacity_factor * S * k / E) in double precision; the reference defines CAP_FACTOR
// (CMakeLists.txt:204) and never reads it, so the formula is this library's.
int moe_config_capacity(const moe_config* c, int64_t* capacity) {
    if (!c || !capacity) return MOE_ERR_BAD_ARGUMENT;
    if (c->num_experts < 1 || c->expert_top_k < 1 || !(c->capacity_factor > 0.0)) return MOE_ERR_BAD_CONFIG;
    const int64_t S = moe_config_tokens(c);
    double v = std::ceil(c->capacity_factor * ((double)S * (double)c->expert_top_k) / (double)c->num_experts);
    if (!(v >= 1.0)) v = 1.0;
    if (v > 9.0e18) v = 9.0e18;   // beyond any row count; keeps the conversion defined
    *capacity = (int64_t)v;
    return MOE_OK;
}

const char* moe_status_string(int s) {
    switch (s) {
        case MOE_OK: return "ok";
        case MOE_ERR_BAD_CONFIG: return "bad config";
        case MOE_ERR_UNSUPPORTED: return "unsupported configuration";
        case MOE_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case MOE_ERR_BAD_ARGUMENT: return "bad argument";
        case MOE_ERR_HIP: return "HIP error";
        case MOE_ERR_NO_DEVICE: return "no gfx950 device";
        case MOE_ERR_QUEUE_STALL: return "task queue dependency wait expired";
        default: return "unknown status";
    }
}

int moe_version(void) { return MOE355_VERSION; }

}  // extern "C"
