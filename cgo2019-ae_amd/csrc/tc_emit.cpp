// HIP source emitter: one translation unit per contraction expression.
//
// Counterpart of cogent/src/codes/tc_gen_code.py:22-447, which writes
// `temp__NN.cu` with #defines, four kernels, the host caller and the public
// interface.  Here the per-expression text is a configuration struct (index
// roles, tiles, wavefront layout, LDS layouts chosen by the mapping pass) that
// instantiates the hand-written gfx950 kernel templates, plus the same public
// entry point: `sd_t_d2_fusion_(int size_<idx>..., T* out, T* a, T* b, int, int)`
// (cogent/src/codes/kernels/tc_interface.py:1444-1516) -- taking DEVICE pointers.
#include "tc_ir.hpp"
#include <sstream>

namespace cogent {

static std::string table(const char* name, const std::vector<int>& v)
{
    std::ostringstream o;
    o << "    static constexpr __host__ __device__ int " << name << "(int i) { constexpr int v[" << (v.empty() ? 1 : v.size()) << "] = {";
    if (v.empty()) o << "0";
    for (size_t i = 0; i < v.size(); i++) o << (i ? ", " : "") << v[i];
    o << "}; return v[i]; }\n";
    return o.str();
}

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

// The members every kernel helper expects of a configuration struct (the whole of `Cfg` of a single
// expression; one `TermN` per contraction of a fused group).
void emit_cfg_members(std::ostringstream& o, const Contraction& c, DType t, const Mapping& m)
{
    const char* T = t == DType::F64 ? "double" : "float";
    const std::vector<int> xop = operand_order(c, m, true), yop = operand_order(c, m, false);
    o << "    typedef " << T << " T;\n";
    o << "    static constexpr int NIDX = " << c.n_idx() << ", SIGN = " << c.sign << ";\n";
    o << "    static constexpr bool X_IS_A = " << (m.x_is_a ? "true" : "false") << ";\n";
    o << "    // tensors in memory order (index ids, fastest first)\n";
    o << "    static constexpr int CR = " << c.out_idx.size() << ", AR = " << c.a_idx.size() << ", BR = " << c.b_idx.size() << ";\n";
    o << table("c_id", c.out_idx) << table("a_id", c.a_idx) << table("b_id", c.b_idx) << table("sum_id", c.int_idx);
    o << "    // composite tiles (fastest first): X side = externals of the input that holds C's fastest index\n";
    o << "    static constexpr int NX = " << m.x_ids.size() << ", NY = " << m.y_ids.size() << ", NK = " << m.k_ids.size() << ";\n";
    o << table("x_id", m.x_ids) << table("x_tile", m.x_tiles);
    o << table("y_id", m.y_ids) << table("y_tile", m.y_tiles);
    o << table("k_id", m.k_ids) << table("k_tile", m.k_tiles);
    {
        // the C tile as a dense block in C's own index order: tile per C index, stride per index id
        std::vector<int> ct, cls(c.n_idx(), 0);
        int run = 1;
        for (int id : c.out_idx) {
            int p, tl = 1;
            if ((p = pos_in(m.x_ids, id)) >= 0) tl = m.x_tiles[p];
            else if ((p = pos_in(m.y_ids, id)) >= 0) tl = m.y_tiles[p];
            ct.push_back(tl);
            cls[id] = run;
            run *= tl;
        }
        o << table("c_tile", ct) << table("cl_stride", cls);
    }
    o << "    static constexpr int BX = " << m.BX << ", BY = " << m.BY << ", BK = " << m.BK << ";\n";
    o << "    static constexpr int BXP = " << m.BXP << ", BYP = " << m.BYP << ", BKP = " << m.BKP << ";\n";

    auto operand = [&](const char* p, const std::vector<int>& op, const std::vector<int>& e_ids, const std::vector<int>& e_tiles) {
        std::vector<int> ids, tiles, isk, mul;
        for (int id : op) {
            ids.push_back(id);
            int q;
            if ((q = pos_in(m.k_ids, id)) >= 0) {
                tiles.push_back(m.k_tiles[q]); isk.push_back(1);
                int mm = 1; for (int j = 0; j < q; j++) mm *= m.k_tiles[j];
                mul.push_back(mm);
            } else {
                q = pos_in(e_ids, id);
                tiles.push_back(e_tiles[q]); isk.push_back(0);
                int mm = 1; for (int j = 0; j < q; j++) mm *= e_tiles[j];
                mul.push_back(mm);
            }
        }
        o << "    static constexpr int " << p << "R = " << op.size() << ";\n";
        // elements per slice load: as many as 16 bytes hold, when the tile of the operand's fastest index is a multiple
        const int vmax = (t == DType::F64) ? 2 : 4;
        const int t0 = tiles.empty() ? 1 : tiles[0];
        const bool on = m.VL == 1 || (m.VL == 2 && p[0] == 'X') || (m.VL == 3 && p[0] == 'Y');      // vl=1 both inputs, 2 the X side only, 3 the Y side only
        const int vw = !on ? 1 : (t0 % vmax == 0 ? vmax : (t0 % 2 == 0 ? 2 : 1));
        o << "    static constexpr int VW" << p << " = " << vw << ";\n";
        std::string s(1, (char)tolower(p[0]));
        o << table((s + "o_id").c_str(), ids) << table((s + "o_tile").c_str(), tiles)
          << table((s + "o_isk").c_str(), isk) << table((s + "o_mul").c_str(), mul);
    };
    o << "    // the X- and Y-side operands in the memory order the kernel reads: id, tile, contracted?, weight in the composite coordinate\n";
    operand("X", xop, m.x_ids, m.x_tiles);
    operand("Y", yop, m.y_ids, m.y_tiles);
    o << "    static constexpr int WX = " << m.WX << ", WY = " << m.WY << ", TX = " << m.TX << ", TY = " << m.TY << ", NT = " << 64 * m.WX * m.WY << ";\n";
    o << "    static constexpr int MI = " << m.MI << ", SK = " << m.SK << ", SKO = " << m.SKO << ", MINW = " << m.MINW << ", LATEC = " << m.LATEC << ", NTC = " << m.NTC << ", SWAP = " << m.SWAP << ", PD = " << m.PD << ", RPX = " << m.RPX << ", RPY = " << m.RPY << ", CLDS = " << m.CLDS << ", NTO = " << m.NTO << ";\n";
    o << "    static constexpr int STREAM = " << m.STREAM << ", SPD = " << m.SPD << ", SMW = " << m.SMW << ", SRES = " << m.SRES << ", SOV = " << m.SOV << ", SCD = " << m.SCD << ", SIL = " << m.SIL << ", TORD = " << m.TORD << ", DBUF = " << m.DBUF << ", ESL = " << m.ESL << ", OKP = " << m.OKP << ";\n";
    o << "    static constexpr int LAYX = " << m.layx << ", LDX = " << m.ldx << ", LAYY = " << m.layy << ", LDY = " << m.ldy << ";\n";
}

std::string emit_hip_source(const Contraction& c, DType t, const Mapping& m, const std::string& unique_name)
{
    std::ostringstream o;
    const char* T = t == DType::F64 ? "double" : "float";
    // the inputs in the memory order the kernel reads them in (tile order for a repacked input)
    const std::vector<int> xop = operand_order(c, m, true), yop = operand_order(c, m, false);

    o << "// Emitted by cogent-mi355 for gfx950.  Do not edit: regenerate from the expression.\n";
    o << "//   " << c.text << "\n";
    o << "//   element type " << T << ", mapping " << m.spec() << "\n";
    o << "#include \"tc_launch.hpp\"\n\n";
    o << "namespace {\n";
    o << "struct Cfg {\n";
    emit_cfg_members(o, c, t, m);
    o << "};\n";
    o << "}  // namespace\n\n";
    const bool uses_scratch = m.RPX || m.RPY;
    if (uses_scratch) {
        o << "// Scratch of the allocation-free entry point (cogent_run_noalloc): the repacked copies of the inputs.\n";
        o << "// Every GPU this object runs on holds its own copy of the array until the process ends.\n";
        o << "#define COGENT_SCRATCH_BYTES (16u << 20)\n";
        o << "static __device__ __align__(256) unsigned char scratch[COGENT_SCRATCH_BYTES];\n\n";
        o << "// In host code the array's name is only a stand-in, not a device address: the address is asked of the\n";
        o << "// runtime once per device, with that device current, and kept.\n";
        o << "static int scratch_address(void** out)\n{\n";
        o << "    static std::atomic<void*> addr[64];\n";
        o << "    int dev = 0;\n";
        o << "    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void)hipGetLastError(); return cogent::tc_fail(cogent::TC_ERR_LAUNCH, \"no current device\"); }\n";
        o << "    void* p = addr[dev].load(std::memory_order_acquire);\n";
        o << "    if (!p) {\n";
        o << "        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) { (void)hipGetLastError(); return cogent::tc_fail(cogent::TC_ERR_LAUNCH, \"hipGetSymbolAddress(scratch) failed\"); }\n";
        o << "        addr[dev].store(p, std::memory_order_release);\n";
        o << "    }\n";
        o << "    *out = p;\n    return 0;\n}\n\n";
    }

    // parameter lists
    std::ostringstream params, sizes;
    for (int i = 0; i < c.n_idx(); i++) {
        params << "int size_" << c.indices[i].name << ", ";
        sizes << (i ? ", " : "") << "size_" << c.indices[i].name;
    }
    params << T << "* " << c.out_name << ", " << T << "* " << c.a_name << ", " << T << "* " << c.b_name
           << ", int cond_kernel_1, int opt_register_transpose";

    o << "extern \"C\" {\n\n";
    o << "// Public entry point, same name and argument order as the reference's generated interface;\n";
    o << "// the three pointers are DEVICE pointers, the launch goes to the default stream and the call\n";
    o << "// returns without synchronising.  Computes " << c.out_name << " " << c.op << " sum(" << c.a_name << " * " << c.b_name << ").  Returns 0 on success.\n";
    o << "int sd_t_d2_fusion_(" << params.str() << ")\n{\n";
    o << "    (void)cond_kernel_1; (void)opt_register_transpose;\n";
    o << "    const int sizes[" << c.n_idx() << "] = {" << sizes.str() << "};\n";
    o << "    return cogent::tc_run<Cfg>(sizes, " << c.out_name << ", " << c.a_name << ", " << c.b_name << ", 0, cogent::TC_VARIANT_AUTO);\n}\n\n";
    o << "// Host-pointer form with the reference's behaviour: allocate, copy in (C included), run, copy C back, free.\n";
    o << "int sd_t_d2_fusion_host_(" << params.str() << ")\n{\n";
    o << "    (void)cond_kernel_1; (void)opt_register_transpose;\n";
    o << "    const int sizes[" << c.n_idx() << "] = {" << sizes.str() << "};\n";
    o << "    return cogent::tc_run_host<Cfg>(sizes, " << c.out_name << ", " << c.a_name << ", " << c.b_name << ");\n}\n\n";
    o << "// Array form for drivers that load several expressions: sizes[] in entry-point order.\n";
    o << "int cogent_run(const int* sizes, int n_sizes, void* C, const void* A, const void* B, void* stream, int variant)\n{\n";
    o << "    if (!sizes || n_sizes != Cfg::NIDX) return cogent::tc_fail(cogent::TC_ERR_NULL_POINTER, \"sizes[] must hold one extent per index\");\n";
    o << "    return cogent::tc_run<Cfg>(sizes, C, A, B, (hipStream_t)stream, variant);\n}\n\n";
    o << "// The same call for callers that cannot allocate (code under graph capture, serving loops): no hipMalloc,\n";
    o << "// hipFree or allocating library routine on any path.  ";
    if (uses_scratch) {
        o << "This mapping repacks inputs: the copies go into the\n";
        o << "// static device array `scratch` (COGENT_SCRATCH_BYTES); inputs that do not fit it are refused with status 3.\n";
        o << "// Calls that overlap on one GPU share the array and race: one call at a time per device.\n";
    } else {
        o << "This mapping needs no scratch memory, so the call\n// is cogent_run itself.\n";
    }
    o << "int cogent_run_noalloc(const int* sizes, int n_sizes, void* C, const void* A, const void* B, void* stream, int variant)\n{\n";
    o << "    if (!sizes || n_sizes != Cfg::NIDX) return cogent::tc_fail(cogent::TC_ERR_NULL_POINTER, \"sizes[] must hold one extent per index\");\n";
    if (uses_scratch) {
        o << "    void* ws = nullptr;\n";
        o << "    if (const int rc = scratch_address(&ws)) return rc;\n";
        o << "    return cogent::tc_run<Cfg>(sizes, C, A, B, (hipStream_t)stream, variant, ws, (size_t)COGENT_SCRATCH_BYTES, true);\n}\n\n";
    } else {
        o << "    return cogent::tc_run<Cfg>(sizes, C, A, B, (hipStream_t)stream, variant, nullptr, 0, true);\n}\n\n";
    }
    o << "int cogent_" << unique_name << "_run(const int* sizes, int n_sizes, void* C, const void* A, const void* B, void* stream, int variant)\n{\n";
    o << "    return cogent_run(sizes, n_sizes, C, A, B, stream, variant);\n}\n\n";
    o << "int cogent_num_indices(void) { return Cfg::NIDX; }\n";
    o << "const char* cogent_last_error(void) { return cogent::tc_error_buffer(); }\n";
    o << "int cogent_last_kernel(void) { return cogent::tc_last_kernel(); }\n";
    o << "const char* cogent_expression(void) { return \"" << c_escape(c.text) << "\"; }\n";
    o << "const char* cogent_info(void) { return \"" << c_escape(mapping_json(c, t, m)) << "\"; }\n";
    o << "\n}  // extern \"C\"\n";
    return o.str();
}

}  // namespace cogent
