// C ABI of the host tools (libcogent_mi355.so); see include/cogent_mi355.h.
#include "tc_ir.hpp"
#include "../../include/cogent_mi355.h"
#include <cstdint>
#include <cstring>
#include <fstream>
#include <sstream>

using namespace cogent;

struct cogent_plan {
    Contraction c;
    DType t;
    Mapping m;
    std::string json, cand_json;
};

static thread_local std::string g_err;
static int fail(int code, const std::string& msg) { g_err = msg; return code; }

static std::string json_escape(const std::string& s)
{
    std::string o;
    for (char ch : s) { if (ch == '"' || ch == '\\') o.push_back('\\'); o.push_back(ch); }
    return o;
}

static std::string plan_json(const cogent_plan& p)
{
    std::ostringstream o;
    auto names = [&](const std::vector<int>& ids) {
        std::string s = "[";
        for (size_t i = 0; i < ids.size(); i++) s += std::string(i ? ", " : "") + "\"" + p.c.indices[ids[i]].name + "\"";
        return s + "]";
    };
    o << "{\"expression\": \"" << json_escape(p.c.text) << "\", \"out\": \"" << p.c.out_name << "\", \"a\": \"" << p.c.a_name
      << "\", \"b\": \"" << p.c.b_name << "\", \"op\": \"" << p.c.op << "\", \"out_idx\": " << names(p.c.out_idx)
      << ", \"sum_idx\": " << names(p.c.int_idx) << ", \"a_idx\": " << names(p.c.a_idx) << ", \"b_idx\": " << names(p.c.b_idx)
      << ", \"rep_sizes\": [";
    for (int i = 0; i < p.c.n_idx(); i++) o << (i ? ", " : "") << p.c.indices[i].rep_size;
    o << "], \"mapping\": " << mapping_json(p.c, p.t, p.m) << "}";
    return o.str();
}

extern "C" {

int cogent_plan_create(const char* text, const char* dtype, int config_rank, const char* mapping_spec, cogent_plan** out)
{
    if (!text || !dtype || !out) return fail(1, "null argument");
    *out = nullptr;
    DType t;
    if (!strcmp(dtype, "DOUBLE")) t = DType::F64;
    else if (!strcmp(dtype, "FLOAT")) t = DType::F32;
    else return fail(2, std::string("data type must be DOUBLE or FLOAT, got '") + dtype + "'");
    std::vector<Contraction> cs;
    std::string err;
    if (!parse_expression_text(text, cs, err)) return fail(1, err);
    if (cs.size() != 1) return fail(4, "exactly one expression per plan (several expressions with one output form a fused group: cogent_group_emit)");
    cogent_plan* p = new cogent_plan();
    p->c = cs[0];
    p->t = t;
    ArchGfx950 arch;
    bool ok = (mapping_spec && *mapping_spec) ? mapping_from_spec(p->c, t, arch, mapping_spec, p->m, err)
                                              : select_mapping(p->c, t, arch, config_rank, p->m, err);
    if (!ok) { delete p; return fail(3, err); }
    p->json = plan_json(*p);
    *out = p;
    return 0;
}

void cogent_plan_destroy(cogent_plan* plan) { delete plan; }
const char* cogent_plan_json(const cogent_plan* plan) { return plan ? plan->json.c_str() : ""; }
int cogent_plan_num_indices(const cogent_plan* plan) { return plan ? plan->c.n_idx() : 0; }
long long cogent_plan_flops(const cogent_plan* plan, const int* sizes) { return contraction_flops(plan->c, sizes); }
long long cogent_plan_bytes(const cogent_plan* plan, const int* sizes) { return contraction_bytes(plan->c, plan->t, sizes); }

const char* cogent_plan_candidates_json(cogent_plan* plan, int k)
{
    ArchGfx950 arch;
    std::vector<Mapping> all = enumerate_mappings(plan->c, plan->t, arch);
    std::ostringstream o;
    o << "[";
    for (int i = 0; i < (int)all.size() && i < k; i++) o << (i ? ", " : "") << mapping_json(plan->c, plan->t, all[i]);
    o << "]";
    plan->cand_json = o.str();
    return plan->cand_json.c_str();
}

int cogent_plan_emit(const cogent_plan* plan, const char* unique_name, const char* out_path)
{
    if (!plan || !unique_name || !out_path) return fail(1, "null argument");
    std::ofstream f(out_path);
    if (!f) return fail(5, std::string("cannot write '") + out_path + "'");
    f << emit_hip_source(plan->c, plan->t, plan->m, unique_name);
    return f.good() ? 0 : fail(5, std::string("cannot write '") + out_path + "'");
}

static thread_local std::string g_group_json;   // per thread, like the error message: concurrent callers do not share it

int cogent_group_emit(const char* text, const char* dtype, const char* tile_spec, const char* unique_name, const char* out_path)
{
    if (!text || !dtype || !unique_name) return fail(1, "null argument");
    DType t;
    if (!strcmp(dtype, "DOUBLE")) t = DType::F64;
    else if (!strcmp(dtype, "FLOAT")) t = DType::F32;
    else return fail(2, std::string("data type must be DOUBLE or FLOAT, got '") + dtype + "'");
    std::vector<Contraction> cs;
    std::string err;
    if (!parse_expression_text(text, cs, err)) return fail(1, err);
    ArchGfx950 arch;
    GroupPlan g;
    if (!plan_group(cs, t, arch, tile_spec ? tile_spec : "", g, err)) return fail(3, err);
    g_group_json = group_json(g);
    if (!out_path || !*out_path) return 0;
    std::ofstream f(out_path);
    if (!f) return fail(5, std::string("cannot write '") + out_path + "'");
    f << emit_group_source(g, unique_name);
    return f.good() ? 0 : fail(5, std::string("cannot write '") + out_path + "'");
}

const char* cogent_group_last_json(void) { return g_group_json.c_str(); }

const char* cogent_host_last_error(void) { return g_err.c_str(); }

static inline uint64_t mix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

void cogent_fill_uniform_f64(double* dst, long long n, unsigned long long seed)
{
    #pragma omp parallel for schedule(static)
    for (long long i = 0; i < n; i++) {
        const uint64_t z = mix64((uint64_t)seed + (uint64_t)(i + 1) * 0x9E3779B97F4A7C15ULL);
        dst[i] = 2.0 * ((double)(z >> 11) * (1.0 / 9007199254740992.0)) - 1.0;
    }
}

void cogent_fill_uniform_f32(float* dst, long long n, unsigned long long seed)
{
    #pragma omp parallel for schedule(static)
    for (long long i = 0; i < n; i++) {
        const uint64_t z = mix64((uint64_t)seed + (uint64_t)(i + 1) * 0x9E3779B97F4A7C15ULL);
        dst[i] = 2.0f * ((float)(z >> 40) * (1.0f / 16777216.0f)) - 1.0f;
    }
}

}  // extern "C"
