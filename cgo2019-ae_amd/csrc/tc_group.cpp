// Fused groups: several contractions with one and the same output index list, emitted as ONE kernel
// that keeps the output tile on chip across the terms (kernels/tc_group.hpp).
//
// The reference groups expressions by identical output index list
// (cogent/src/algs/bases/tc_gen_inputs.py:113-123) and gives the fused entry point one pair of input
// pointers and one `cond_kernel_N` flag per term
// (cogent/src/codes/kernels/tc_interface.py:1494-1511).  Here the group shares a tile of C -- one tile
// size per output index -- and every term derives its own X/Y roles from it: X = the externals of the
// input that holds C's fastest index, in C order.
#include "tc_ir.hpp"
#include <algorithm>
#include <cmath>
#include <set>
#include <sstream>

namespace cogent {

void emit_cfg_members(std::ostringstream& o, const Contraction& c, DType t, const Mapping& m);   // tc_emit.cpp

static int esize(DType t) { return t == DType::F64 ? 8 : 4; }
static int ceil_div(int a, int b) { return (a + b - 1) / b; }
static int pos_in(const std::vector<int>& v, int id)
{
    for (int i = 0; i < (int)v.size(); i++) if (v[i] == id) return i;
    return -1;
}

static std::string c_escape(const std::string& s)
{
    std::string o;
    for (char ch : s) {
        if (ch == '"' || ch == '\\') { o.push_back('\\'); o.push_back(ch); }
        else if (ch == '\n') o += "\\n";
        else o.push_back(ch);
    }
    return o;
}

// The mapping of one term for a given tile of C.  Returns false when the term cannot be laid out
// (accumulators or LDS out of budget).
static bool term_mapping(const Contraction& c, DType t, const ArchGfx950& arch, const std::vector<int>& c_tile, int NW, int k_room,
                         Mapping& m, std::string& err)
{
    m = Mapping();
    m.x_is_a = c.in_a(c.out_idx[0]);
    m.MI = (t == DType::F64) ? 0 : 1;
    const std::vector<int>& xop = m.x_is_a ? c.a_idx : c.b_idx;
    const std::vector<int>& yop = m.x_is_a ? c.b_idx : c.a_idx;
    for (size_t j = 0; j < c.out_idx.size(); j++) {
        const int id = c.out_idx[j];
        if (pos_in(xop, id) >= 0) { m.x_ids.push_back(id); m.x_tiles.push_back(c_tile[j]); }
        else                      { m.y_ids.push_back(id); m.y_tiles.push_back(c_tile[j]); }
    }
    // contracted indices in the X input's order, at most k_room deep per K block
    int room = k_room;
    for (int id : xop) {
        if (!c.indices[id].internal) continue;
        const int rep = c.indices[id].rep_size;
        int tl = std::min(rep, room);
        if (tl < rep && tl >= 4) tl -= tl % 4;
        tl = std::max(tl, 1);
        m.k_ids.push_back(id); m.k_tiles.push_back(tl);
        room = std::max(1, room / tl);
    }
    int BX = 1, BY = 1;
    for (int v : m.x_tiles) BX *= v;
    for (int v : m.y_tiles) BY *= v;
    const int MT = 16, nx = ceil_div(BX, MT), ny = ceil_div(BY, MT);
    int best = 1 << 30;
    for (int wx = 1; wx <= NW; wx++) {
        if (NW % wx) continue;
        const int wy = NW / wx, tx = ceil_div(nx, wx), ty = ceil_div(ny, wy);
        if (tx * ty < best) { best = tx * ty; m.WX = wx; m.WY = wy; m.TX = tx; m.TY = ty; }
    }
    auto fvi = [](const std::vector<int>& v) { return v.empty() ? -1 : v[0]; };
    m.layx = (!m.k_ids.empty() && m.k_ids[0] == fvi(xop) && m.k_tiles[0] >= 4) ? 1 : 0;
    m.layy = (!m.k_ids.empty() && m.k_ids[0] == fvi(yop) && m.k_tiles[0] >= 4) ? 1 : 0;
    m.VL = 1;                              // 16-byte slice loads wherever a call's tiles are whole (the pipelined kernel's variant without predicates)
    finish_geometry(c, t, m);
    if (!check_mapping(c, t, arch, m, err)) return false;
    return true;
}

static std::vector<int> divisors_up_to(int n, int cap)
{
    std::vector<int> v;
    for (int d = 1; d <= n && d <= cap; d++) if (n % d == 0) v.push_back(d);
    if (n <= cap && (v.empty() || v.back() != n)) v.push_back(n);
    return v;
}

bool plan_group(const std::vector<Contraction>& cs, DType t, const ArchGfx950& arch, const std::string& spec,
                GroupPlan& g, std::string& err)
{
    g = GroupPlan();
    if (cs.size() < 2) { err = "a fused group needs at least two expressions"; return false; }
    if (cs.size() > 16) { err = "a fused group holds at most 16 expressions"; return false; }
    const Contraction& c0 = cs[0];
    for (const Contraction& c : cs) {
        bool same = c.out_name == c0.out_name && c.out_idx == c0.out_idx && c.int_idx == c0.int_idx && c.n_idx() == c0.n_idx();
        for (int i = 0; same && i < c.n_idx(); i++)
            same = c.indices[i].name == c0.indices[i].name && c.indices[i].rep_size == c0.indices[i].rep_size;
        if (!same) { err = "the expressions of a fused group must share the output tensor, its index list, the summed indices and all sizes"; return false; }
    }
    g.terms = cs;
    g.t = t;
    const int s = esize(t);
    const int CR = (int)c0.out_idx.size();
    const int vol_max = 32768 / s;

    std::string why;
    auto evaluate = [&](const std::vector<int>& tile, std::vector<Mapping>& maps, double& score) -> bool {
        long long vol = 1;
        for (int v : tile) vol *= v;
        if (vol > 2 * vol_max) { why = "the tile of the output exceeds 64 KB"; return false; }
        maps.assign(cs.size(), Mapping());
        double mfma_eff = 0, op_eff = 0, slice_eff = 0;
        int lds_ops = 0;
        for (size_t k = 0; k < cs.size(); k++) {
            std::string e;
            if (!term_mapping(cs[k], t, arch, tile, g.NW, g.k_room, maps[k], e)) { why = "term " + std::to_string(k + 1) + ": " + e; return false; }
            const Mapping& m = maps[k];
            if (m.lds_bytes > 65536) { why = "term " + std::to_string(k + 1) + ": input slices exceed 64 KB"; return false; }
            if (vol * s + m.lds_bytes > 160 * 1024) { why = "term " + std::to_string(k + 1) + ": the tile of the output and the input slices exceed the 160 KB of LDS"; return false; }
            lds_ops = std::max(lds_ops, m.lds_bytes);
            mfma_eff += (double)(m.BX * m.BY) / (double)(m.BXP * m.BYP);
            // rows of slices a term stages per element of the tile, against the square split of the same volume: a
            // 16x256 split moves 1.7 times the slice bytes (L2 and LDS traffic) of 128x32
            slice_eff += 2.0 * std::sqrt((double)m.BX * m.BY) / (double)(m.BX + m.BY);
            for (int side = 0; side < 2; side++) {
                const std::vector<int>& op = (side == 0) == m.x_is_a ? cs[k].a_idx : cs[k].b_idx;
                const int f = op[0];
                int p, tl = 1;
                if ((p = pos_in(m.x_ids, f)) >= 0) tl = m.x_tiles[p];
                else if ((p = pos_in(m.y_ids, f)) >= 0) tl = m.y_tiles[p];
                else if ((p = pos_in(m.k_ids, f)) >= 0) tl = m.k_tiles[p];
                op_eff += std::min(1.0, tl * s / 64.0);
            }
        }
        mfma_eff /= cs.size();
        slice_eff /= cs.size();
        op_eff /= 2.0 * cs.size();
        const double c_eff = std::min(1.0, tile[0] * s / 128.0);
        // contiguous run of the tile in C's memory order, in lines
        double run = 1;
        for (int j = 0; j < CR; j++) { run *= tile[j]; if (tile[j] != c0.indices[c0.out_idx[j]].rep_size) break; }
        const double run_eff = std::min(1.0, 0.75 + 0.25 * std::log2(std::max(1.0, run * s / 128.0)) / 4.0);
        score = c_eff * (0.5 + 0.5 * op_eff) * (0.3 + 0.7 * mfma_eff) * (0.4 + 0.6 * slice_eff) * (0.5 + 0.5 * std::min(1.0, (double)vol / vol_max)) * run_eff;
        (void)lds_ops;
        return true;
    };

    std::vector<int> tile(CR, 1);
    std::string ct_spec;
    bool nw_given = false;
    {
        // fields separated by ';': ct=<tile>,<tile>,... (one per output index), kt=<K depth per block>, nw=<wavefronts>
        std::istringstream fs(spec);
        std::string field;
        while (std::getline(fs, field, ';')) {
            if (field.empty()) continue;
            if (field.compare(0, 3, "ct=") == 0) ct_spec = field.substr(3);
            else if (field.compare(0, 3, "kt=") == 0) g.k_room = std::max(4, std::min(64, atoi(field.c_str() + 3)));
            else if (field.compare(0, 3, "nw=") == 0) { g.NW = std::max(1, std::min(8, atoi(field.c_str() + 3))); nw_given = true; }
            else if (field.compare(0, 3, "nr=") == 0) g.nregion = std::max(0, std::min(2, atoi(field.c_str() + 3)));
            else if (field.compare(0, 3, "ps=") == 0) g.persist = atoi(field.c_str() + 3) ? 1 : 0;
            else { err = "group mapping spec: fields are ct=<tile>,... kt=<n> nw=<n> nr=<0|1|2> ps=<0|1>"; return false; }
        }
    }
    if (!ct_spec.empty()) {
        std::istringstream is(ct_spec);
        std::string item;
        int j = 0;
        while (std::getline(is, item, ',')) { if (j < CR) tile[j] = atoi(item.c_str()); j++; }
        if (j != CR) { err = "group mapping spec: one tile per output index"; return false; }
        for (int v : tile) if (v < 1) { err = "group mapping spec: tiles must be positive"; return false; }
        double sc;
        if (!evaluate(tile, g.maps, sc)) { err = "group mapping spec: tile does not fit: " + why; return false; }
        g.c_tile = tile;
    } else {
        std::vector<std::vector<int>> opts(CR);
        for (int j = 0; j < CR; j++) opts[j] = divisors_up_to(c0.indices[c0.out_idx[j]].rep_size, 64);
        double best = -1;
        std::vector<int> idx(CR, 0);
        std::vector<Mapping> maps;
        while (true) {
            long long vol = 1;
            for (int j = 0; j < CR; j++) { tile[j] = opts[j][idx[j]]; vol *= tile[j]; }
            double sc;
            if (vol >= 256 && vol <= vol_max && evaluate(tile, maps, sc) && sc > best) { best = sc; g.c_tile = tile; g.maps = maps; }
            int j = 0;
            while (j < CR && ++idx[j] == (int)opts[j].size()) { idx[j] = 0; j++; }
            if (j == CR) break;
        }
        if (best < 0) { err = "no admissible tile for this group"; return false; }
    }
    // wavefronts: eight on tiles of 4096 elements or more (measured on the chosen tiles of the two CCSD(T) groups:
    // 162 -> 149 us fp64, 96 -> 88 us fp32), four below; a spec's nw= stands
    if (!nw_given) {
        long long vol = 1;
        for (int v : g.c_tile) vol *= v;
        const int nw = vol >= 4096 ? 8 : 4;
        if (nw != g.NW) {
            const int keep = g.NW;
            g.NW = nw;
            std::vector<Mapping> maps;
            double sc;
            if (evaluate(g.c_tile, maps, sc)) g.maps = maps; else g.NW = keep;
        }
    }
    g.vol = 1;
    for (int v : g.c_tile) g.vol *= v;
    g.lds_ops = 0;
    for (const Mapping& m : g.maps) g.lds_ops = std::max(g.lds_ops, m.lds_bytes / s);
    return true;
}

std::string group_json(const GroupPlan& g)
{
    std::ostringstream o;
    const Contraction& c0 = g.terms[0];
    o << "{\"dtype\": \"" << (g.t == DType::F64 ? "f64" : "f32") << "\", \"group\": true, \"n_terms\": " << g.terms.size()
      << ", \"out\": \"" << c0.out_name << "\", \"out_idx\": [";
    for (size_t j = 0; j < c0.out_idx.size(); j++) o << (j ? ", " : "") << "\"" << c0.indices[c0.out_idx[j]].name << "\"";
    o << "], \"sum_idx\": [";
    for (size_t j = 0; j < c0.int_idx.size(); j++) o << (j ? ", " : "") << "\"" << c0.indices[c0.int_idx[j]].name << "\"";
    o << "], \"c_tile\": [";
    for (size_t j = 0; j < g.c_tile.size(); j++) o << (j ? ", " : "") << g.c_tile[j];
    o << "], \"threads\": " << 64 * g.NW << ", \"lds_bytes\": " << (g.vol + g.lds_ops) * esize(g.t) << ", \"spec\": \"ct=";
    for (size_t j = 0; j < g.c_tile.size(); j++) o << (j ? "," : "") << g.c_tile[j];
    o << ";kt=" << g.k_room << ";nw=" << g.NW << ";nr=" << g.nregion << (g.persist ? ";ps=1" : "") << "\", \"terms\": [";
    for (size_t k = 0; k < g.terms.size(); k++)
        o << (k ? ", " : "") << "{\"text\": \"" << c_escape(g.terms[k].text) << "\", \"mapping\": " << mapping_json(g.terms[k], g.t, g.maps[k]) << "}";
    o << "]}";
    return o.str();
}

std::string emit_group_source(const GroupPlan& g, const std::string& unique_name)
{
    std::ostringstream o;
    const char* T = g.t == DType::F64 ? "double" : "float";
    const Contraction& c0 = g.terms[0];
    const int N = (int)g.terms.size();
    o << "// Emitted by cogent-mi355 for gfx950.  Do not edit: regenerate from the expressions.\n";
    o << "// Fused group of " << N << " contractions into " << c0.out_name << ":\n";
    for (const Contraction& c : g.terms) o << "//   " << c.text << "\n";
    o << "#include \"tc_group.hpp\"\n\nnamespace {\n";
    auto table = [&](const char* name, const std::vector<int>& v) {
        o << "    static constexpr __host__ __device__ int " << name << "(int i) { constexpr int v[" << (v.empty() ? 1 : v.size()) << "] = {";
        if (v.empty()) o << "0";
        for (size_t i = 0; i < v.size(); i++) o << (i ? ", " : "") << v[i];
        o << "}; return v[i]; }\n";
    };
    o << "struct G {\n    typedef " << T << " T;\n";
    o << "    static constexpr int NIDX = " << c0.n_idx() << ", CR = " << c0.out_idx.size() << ", NTERM = " << N << ", NT = " << 64 * g.NW
      << ", TILE_VOL = " << g.vol << ", LDS_OPS = " << g.lds_ops << ", NREGION = " << g.nregion << ", PERSIST = " << g.persist << ";\n";
    table("c_id", c0.out_idx);
    table("c_tile", g.c_tile);
    o << "};\n";
    for (int k = 0; k < N; k++) {
        o << "struct Term" << k << " {   // " << g.terms[k].text << "\n";
        emit_cfg_members(o, g.terms[k], g.t, g.maps[k]);
        o << "};\n";
    }
    o << "}  // namespace\n\n";

    // unique parameter names for the inputs
    std::vector<std::string> names;
    std::set<std::string> used = {c0.out_name};
    for (int k = 0; k < N; k++)
        for (const std::string& base : {g.terms[k].a_name, g.terms[k].b_name}) {
            std::string nm = base;
            if (used.count(nm)) nm = base + "_" + std::to_string(k + 1);
            while (used.count(nm)) nm += "_";
            used.insert(nm);
            names.push_back(nm);
        }
    std::ostringstream params, sizes, ptrs, conds, terms;
    for (int i = 0; i < c0.n_idx(); i++) {
        params << "int size_" << c0.indices[i].name << ", ";
        sizes << (i ? ", " : "") << "size_" << c0.indices[i].name;
    }
    params << T << "* " << c0.out_name;
    for (size_t i = 0; i < names.size(); i++) { params << ", " << T << "* " << names[i]; ptrs << (i ? ", " : "") << names[i]; }
    for (int k = 0; k < N; k++) { params << ", int cond_kernel_" << k + 1; conds << (k ? ", " : "") << "cond_kernel_" << k + 1; }
    params << ", int opt_register_transpose";
    for (int k = 0; k < N; k++) terms << ", Term" << k;

    o << "extern \"C\" {\n\n";
    o << "// Public entry point of the group, in the reference's shape: extents, the output, one pair of inputs per\n";
    o << "// term, one flag per term (0 leaves that term out), the register-transpose option (accepted, unused).\n";
    o << "// DEVICE pointers; default stream; returns without synchronising.  Returns 0 on success.\n";
    o << "int sd_t_d2_fusion_(" << params.str() << ")\n{\n    (void)opt_register_transpose;\n";
    o << "    const int sizes[" << c0.n_idx() << "] = {" << sizes.str() << "};\n";
    o << "    const void* inputs[" << 2 * N << "] = {" << ptrs.str() << "};\n";
    o << "    const int enabled[" << N << "] = {" << conds.str() << "};\n";
    o << "    return cogent::tc_group_run<G" << terms.str() << ">(sizes, " << c0.out_name << ", inputs, enabled, 0);\n}\n\n";
    o << "// Host-pointer form with the reference's behaviour: allocate, copy in, run every term, copy the output back, free.\n";
    o << "int sd_t_d2_fusion_host_(" << params.str() << ")\n{\n    (void)opt_register_transpose;";
    for (int k = 0; k < N; k++) o << " (void)cond_kernel_" << k + 1 << ";";
    o << "\n    const int sizes[" << c0.n_idx() << "] = {" << sizes.str() << "};\n";
    o << "    const void* inputs[" << 2 * N << "] = {" << ptrs.str() << "};\n";
    o << "    return cogent::tc_group_run_host<G" << terms.str() << ">(sizes, " << c0.out_name << ", inputs);\n}\n\n";
    o << "// Array form: sizes[] in entry-point order, inputs[] = A of term 1, B of term 1, A of term 2, ...;\n";
    o << "// enabled[] may be null (every term).\n";
    o << "int cogent_run_group(const int* sizes, int n_sizes, void* C, const void* const* inputs, int n_inputs, const int* enabled, void* stream)\n{\n";
    o << "    if (!sizes || n_sizes != G::NIDX) return cogent::tc_fail(cogent::TC_ERR_NULL_POINTER, \"sizes[] must hold one extent per index\");\n";
    o << "    if (n_inputs != " << 2 * N << ") return cogent::tc_fail(cogent::TC_ERR_NULL_POINTER, \"inputs[] must hold two pointers per term\");\n";
    o << "    return cogent::tc_group_run<G" << terms.str() << ">(sizes, C, inputs, enabled, (hipStream_t)stream);\n}\n\n";
    o << "int cogent_" << unique_name << "_run_group(const int* sizes, int n_sizes, void* C, const void* const* inputs, int n_inputs, const int* enabled, void* stream)\n{\n";
    o << "    return cogent_run_group(sizes, n_sizes, C, inputs, n_inputs, enabled, stream);\n}\n\n";
    o << "int cogent_num_indices(void) { return G::NIDX; }\n";
    o << "int cogent_num_terms(void) { return G::NTERM; }\n";
    o << "const char* cogent_last_error(void) { return cogent::tc_error_buffer(); }\n";
    std::string all;
    for (int k = 0; k < N; k++) all += (k ? "\n" : "") + g.terms[k].text;
    o << "const char* cogent_expression(void) { return \"" << c_escape(all) << "\"; }\n";
    o << "const char* cogent_info(void) { return \"" << c_escape(group_json(g)) << "\"; }\n";
    o << "\n}  // extern \"C\"\n";
    return o.str();
}

}  // namespace cogent
