// Intermediate representation shared by the parser, the mapping pass and the emitter.
#pragma once
#include <string>
#include <vector>

namespace cogent {

// One index of a contraction.  Ids are dense: output indices in output order
// first, then the contracted ("internal") indices in sum() order -- the order
// in which the generated entry point takes its `int size_*` arguments
// (cogent/src/codes/kernels/tc_interface.py:1459-1492).
struct Index {
    std::string name;
    int rep_size = 0;        // representative problem size from the expression (mapping only)
    bool internal = false;   // summed over
};

// `out [..] op sum(..) * a [..] * b [..];`, the record of
// cogent/src/algs/bases/tc_gen_inputs.py:108.  Index lists hold ids, FASTEST
// index first (the reference's tensors are column-major).
struct Contraction {
    std::string text;
    std::string out_name, a_name, b_name;
    std::string op;          // "+=" or "-="
    int sign = 1;
    std::vector<Index> indices;
    std::vector<int> out_idx, int_idx, a_idx, b_idx;

    int n_idx() const { return (int)indices.size(); }
    bool in_a(int id) const { for (int v : a_idx) if (v == id) return true; return false; }
    bool in_b(int id) const { for (int v : b_idx) if (v == id) return true; return false; }
};

enum class DType { F64, F32 };

// gfx950 (MI355X) figures the mapping pass sizes tiles against.
struct ArchGfx950 {
    int wave = 64;
    int n_cu = 256;
    int simd_per_cu = 4;
    int lds_bytes_per_cu = 160 * 1024;
    int lds_bytes_per_block = 64 * 1024;     // static __shared__ limit
    int max_threads_per_block = 1024;
    int max_waves_per_cu = 32;
    int vgpr_per_lane = 512;                 // unified VGPR+AGPR file at one wave per SIMD
    double clock_hz = 2.4e9;
    double hbm_bytes_per_s = 8.0e12;         // published peak
    double hbm_sustained_fraction = 0.66;    // what a plain read-modify-write kernel reaches on the part
    double l2_bytes_per_s = 10.0e12;         // aggregate L2/Infinity-Cache rate for re-read operand slices
    double lds_bytes_per_clk_cu = 128.0;
    double mfma_f64_flops = 78.6e12;
    double mfma_f32_flops = 157.3e12;
};

// One index-to-tile mapping for gfx950: the counterpart of the reference's
// Config record (cogent/src/algs/bases/class_configuration.py:4-65), with
// wave / MFMA tiling and LDS layouts in place of TB_X/TB_Y/REG_X/REG_Y.
struct Mapping {
    bool x_is_a = true;                       // X side = the input that holds the output's fastest index
    std::vector<int> x_ids, x_tiles;          // composite order, fastest first
    std::vector<int> y_ids, y_tiles;
    std::vector<int> k_ids, k_tiles;
    int BX = 0, BY = 0, BK = 0;               // tile products
    int BXP = 0, BYP = 0, BKP = 0;            // padded to MFMA granularity
    int WX = 1, WY = 1, TX = 1, TY = 1;       // wavefront grid and MFMA tiles per wavefront
    int MI = 0;                               // 0 f64 16x16x4, 1 f32 16x16x4, 2 f32 32x32x2
    int MINW = 1;                             // resident wavefronts per SIMD asked of the register allocator
    bool from_spec = false;                   // written by hand or by the tuner (not enumerated): the register check trusts it further
    int SKO = 0;                              // 1 (split K, so=1): the K shares are the grid's outermost level, so the tiles of one share run on one XCD
    int LATEC = 0;                            // 1: load the C tile during the first K block instead of before the loop
    int ntc_forced = -1;                      // -1: decide from the tile shape; 0..3: pinned by a mapping spec (nt=)
    int NTC = 0;                              // non-temporal C accesses: bit 0 loads, bit 1 stores (both when rows are whole 128-byte lines)
    int SWAP = 0;                             // 1 (fp32): C's fastest index on the MFMA rows, 128-bit C accesses
    int swap_forced = -1;
    int PD = 1;                               // K blocks requested ahead of the one being contracted (register stages)
    int pd_forced = -1;
    int RPX = 0, RPY = 0;                     // 1 (mapping spec rx=/ry= only): that input is first copied into tile order, see operand_order()
    int CLDS = 0;                             // 1: full C tiles pass through LDS in C's memory order (16-byte, whole-line global accesses)
    int clds_forced = -1;
    int NTO = 0, nto_forced = -1;             // non-temporal input loads: bit 0 X side, bit 1 Y side (an input every element of which is read once)
    int st_forced = 0;                        // mapping spec st=<depth>: ask for the panel-resident streaming kernel with that many Y slices requested ahead
    int STREAM = 0, SPD = 1, SMW = 1;         // streaming kernel: its compile-time K-block count (0: none), prefetch depth, wavefronts per SIMD to leave room for
    int SRES = 0;                             // ... and which side's panel stays in LDS: 0 X (default), 1 Y (mapping spec sy=1)
    int SOV = 0;                              // 1 (mapping spec ov=1, streaming kernel): only the first slice of the resident panel is loaded before the first tile, the rest behind it
    int TORD = 0;                             // 1 (mapping spec to=1, per-tile kernel): workgroups take the tiles in the order of their origins in C's memory, no XCD-contiguous ranges
    int OKP = 1;                              // 0 (mapping spec ok=0, no split K): calls whose contracted extents fit one K block take the K-loop kernels unless all their tiles are whole; the one-K-block kernel then serves whole tiles only
    int ESL = 0;                              // 1 (mapping spec es=1, per-tile kernel with the C tile through LDS): the first K block's slices are requested before the C tile is staged
    int SIL = 0;                              // 1 (mapping spec il=1, streaming kernel): the runs of the workgroups are interleaved (tile rn, rn + nruns, ..) instead of contiguous
    int SCD = 1;                              // (mapping spec cd=2, streaming kernel): C is read that many tiles ahead (1 or 2), in register tiles of its own
    int VL = 0;                               // mapping spec vl=1 (both inputs), 2 (X side only), 3 (Y side only): slice loads of 8/16 bytes per lane along the operand's fastest index
    int DBUF = 0;                             // 1 (mapping spec db=1): two LDS stages in dynamic LDS when they exceed the 64 KB a static array may have
    int SK = 1;                               // split-K factor: SK workgroups per output tile, atomic accumulate
    int layx = 0, ldx = 0, layy = 0, ldy = 0; // LDS layout per operand
    // model outputs
    double t_hbm = 0, t_l2 = 0, t_mfma = 0, t_lds = 0, tail_eff = 1, cost = 0;
    long long n_blocks = 0; int lds_bytes = 0; int blocks_per_cu = 0;
    int steps_main_loop = 0;
    std::string spec() const;                 // compact text form, parseable by mapping_from_spec
};

// ---- parser (tc_parse.cpp)
// Reads an expression file the way the reference does: lines starting with '#'
// are skipped, every other line is one expression.  Returns false and sets err
// on the inputs the reference cannot process.
bool parse_expression_line(const std::string& line, Contraction& out, std::string& err);
bool parse_expression_file(const std::string& path, std::vector<Contraction>& out, std::string& err);
bool parse_expression_text(const std::string& text, std::vector<Contraction>& out, std::string& err);

// ---- mapping (tc_mapping.cpp)
std::vector<Mapping> enumerate_mappings(const Contraction& c, DType t, const ArchGfx950& arch);
void cost_model(const Contraction& c, DType t, const ArchGfx950& arch, Mapping& m);
// rank < 0: cheapest by the model; otherwise the rank-th of the sorted list
bool select_mapping(const Contraction& c, DType t, const ArchGfx950& arch, int rank, Mapping& out, std::string& err);
bool mapping_from_spec(const Contraction& c, DType t, const ArchGfx950& arch, const std::string& spec, Mapping& out, std::string& err);
bool check_mapping(const Contraction& c, DType t, const ArchGfx950& arch, const Mapping& m, std::string& err);
std::string mapping_json(const Contraction& c, DType t, const Mapping& m);
// Index ids of the X-side (or Y-side) input in the memory order the kernel reads it in, fastest first:
// the tensor's own order, or for a repacked input its externals in tile order followed by the K indices.
std::vector<int> operand_order(const Contraction& c, const Mapping& m, bool x_side);

void finish_geometry(const Contraction& c, DType t, Mapping& m);      // tile products, padding, LDS leading dimensions

// ---- fused groups (tc_group.cpp): expressions with one output index list, one kernel
struct GroupPlan {
    std::vector<Contraction> terms;
    DType t = DType::F64;
    std::vector<int> c_tile;          // tile per output index, in output order
    std::vector<Mapping> maps;        // per term: roles and tiles derived from c_tile
    int NW = 4;                       // wavefronts per workgroup
    int k_room = 32;                  // contracted depth per K block
    int persist = 0;                  // spec ps=1: for whole-tile calls, workgroups persistent over several tiles with the term pipeline running across tile boundaries (measured 6-10 % slower than one workgroup per tile: off)
    int nregion = 1;                  // operand regions in LDS of the pipelined kernel (spec nr=): 1 = more workgroups per CU, 2 = one barrier per term
    int vol = 0, lds_ops = 0;         // elements of the C tile; elements of the largest pair of operand slices
};
// spec: empty (search) or fields "ct=<tile>,<tile>,..." (one per output index), "kt=<K depth>", "nw=<wavefronts>" joined by ';'
bool plan_group(const std::vector<Contraction>& cs, DType t, const ArchGfx950& arch, const std::string& spec,
                GroupPlan& g, std::string& err);
std::string group_json(const GroupPlan& g);
std::string emit_group_source(const GroupPlan& g, const std::string& unique_name);

// ---- emitter (tc_emit.cpp)
std::string emit_hip_source(const Contraction& c, DType t, const Mapping& m, const std::string& unique_name);

// ---- accounting
long long contraction_flops(const Contraction& c, const int* sizes);                 // 2 * prod(all extents)
long long contraction_bytes(const Contraction& c, DType t, const int* sizes);        // sizeof(T) * (|A| + |B| + 2|C|)

}  // namespace cogent
