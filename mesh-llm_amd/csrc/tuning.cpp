// The tuning table: names, ranges, parsing.  Host code only.
#include "tuning.hpp"

#include <cctype>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "mesh_common.hpp"

namespace mesh {

const TuningField *tuning_fields() {
    static const TuningField table[] = {
        {"gemm_layout", &Tuning::gemm_layout, 0, 1, TUNE_STAGE},
        {"gemm_min_tokens", &Tuning::gemm_min_tokens, 1, 1 << 20, TUNE_STAGE},
        {"skinny_min_tokens", &Tuning::skinny_min_tokens, 0, 1 << 20, TUNE_STAGE},
        {"gemm_splitk", &Tuning::gemm_splitk, 0, 1, TUNE_SESSION},
        {"chunk_kv16", &Tuning::chunk_kv16, 0, 1, TUNE_SESSION},
        {"gemv_rope", &Tuning::gemv_rope, 0, 1, TUNE_SESSION},
        {"xq_handover", &Tuning::xq_handover, 0, 1, TUNE_SESSION},
        {"skinny_f16", &Tuning::skinny_f16, 0, 1, TUNE_SESSION},
        {"skinny_norm_fused", &Tuning::skinny_norm_fused, 0, 1, TUNE_SESSION},
        {"skinny_pair", &Tuning::skinny_pair, 0, 1, TUNE_SESSION},
        {"skinny_f16_wide", &Tuning::skinny_f16_wide, 0, 1, TUNE_SESSION},
        {"gemm_fused", &Tuning::gemm_fused, 0, 1, TUNE_SESSION},
        {"gemm_xdirect", &Tuning::gemm_xdirect, 0, 1, TUNE_SESSION},
        {"gemm_big", &Tuning::gemm_big, 0, 1, TUNE_SESSION},
        {"gemm_narrow", &Tuning::gemm_narrow, 0, 1, TUNE_SESSION},
        {"attn_chunk_ksplit", &Tuning::attn_chunk_ksplit, 0, 1, TUNE_SESSION},
        {"attn_mma_min_tokens", &Tuning::attn_mma_min_tokens, 1, 1 << 20, TUNE_SESSION},
        {"attn_split_target", &Tuning::attn_split_target, 0, 1 << 16, TUNE_SESSION},
        {"moe_group", &Tuning::moe_group, 0, 1, TUNE_SESSION},
        {"moe_router_tail", &Tuning::moe_router_tail, 0, 1, TUNE_SESSION},
        {"moe_fuse_quant", &Tuning::moe_fuse_quant, 0, 1, TUNE_SESSION},
        {"moe_gemm", &Tuning::moe_gemm, 0, 1, TUNE_SESSION},
        {"moe_gemm_min_pairs", &Tuning::moe_gemm_min_pairs, 1, 1 << 20, TUNE_SESSION},
        {"grouped_oversub", &Tuning::grouped_oversub, 1, 64, TUNE_SESSION},
        {"graphs", &Tuning::graphs, 0, 1, TUNE_SESSION},
        {nullptr, nullptr, 0, 0, TUNE_STAGE},
    };
    return table;
}

static const TuningField *find_field(const char *name) {
    if (!name) return nullptr;
    for (const TuningField *f = tuning_fields(); f->name; ++f)
        if (!strcmp(f->name, name)) return f;
    return nullptr;
}

int tuning_set(Tuning &t, const char *name, int value, bool session_only) {
    const TuningField *f = find_field(name);
    if (!f) return fail(MESH_ERR_INVALID, "tuning: no switch named '%s'", name ? name : "(null)");
    if (session_only && f->level != TUNE_SESSION)
        return fail(MESH_ERR_INVALID, "tuning: '%s' is fixed when the stage is opened (mesh_stage_opts.tuning)", name);
    if (value < f->lo || value > f->hi) return fail(MESH_ERR_INVALID, "tuning: %s=%d outside [%d, %d]", name, value, f->lo, f->hi);
    t.*(f->field) = value;
    return MESH_OK;
}

int tuning_get(const Tuning &t, const char *name, int *value) {
    const TuningField *f = find_field(name);
    if (!f || !value) return fail(MESH_ERR_INVALID, "tuning: no switch named '%s'", name ? name : "(null)");
    *value = t.*(f->field);
    return MESH_OK;
}

int tuning_parse(Tuning &t, const char *text, const char *what) {
    if (!text) return MESH_OK;
    std::string s;
    for (const char *p = text; *p; ++p)
        if (!isspace((unsigned char)*p)) s.push_back(*p);
    size_t at = 0;
    while (at < s.size()) {
        size_t end = s.find(',', at);
        if (end == std::string::npos) end = s.size();
        const std::string item = s.substr(at, end - at);
        at = end + 1;
        if (item.empty()) continue;
        const size_t eq = item.find('=');
        char *rest = nullptr;
        const long v = eq == std::string::npos ? 0 : strtol(item.c_str() + eq + 1, &rest, 10);
        if (eq == std::string::npos || eq == 0 || eq + 1 == item.size() || (rest && *rest) || v < -(1L << 30) || v > (1L << 30))
            return fail(MESH_ERR_INVALID, "%s: '%s' is not name=integer", what, item.c_str());
        const int rc = tuning_set(t, item.substr(0, eq).c_str(), (int)v, false);
        if (rc != MESH_OK) {
            const std::string inner = last_error_slot();
            return fail(rc, "%s: %s", what, inner.c_str());
        }
    }
    return MESH_OK;
}

int tuning_process_default(Tuning &out) {
    static std::once_flag once;
    static Tuning def;
    static int rc = MESH_OK;
    static std::string err;
    std::call_once(once, [] {
        rc = tuning_parse(def, getenv("MESH_TUNING"), "MESH_TUNING");
        if (rc != MESH_OK) err = last_error_slot();
    });
    if (rc != MESH_OK) return fail(rc, "%s", err.c_str());
    out = def;
    return MESH_OK;
}

std::string tuning_describe(const Tuning &t) {
    std::string s;
    for (const TuningField *f = tuning_fields(); f->name; ++f) {
        if (!s.empty()) s += ",";
        s += f->name;
        s += "=" + std::to_string(t.*(f->field));
    }
    return s;
}

}  // namespace mesh
