// Index-to-tile mapping pass for gfx950.
//
// Plays the part of the reference's enumeration + pruning
// (cogent/src/algs/bases/enumeration.py:15-278), cost model
// (cogent/src/algs/bases/cost_models.py:11-631) and selection
// (cogent/src/generators/configurations.py:254-289), re-derived for CDNA4:
//
//   reference (warp-32, 48 KB smem)            here (wave-64, MFMA, 160 KB LDS)
//   ---------------------------------------    ----------------------------------------
//   TB_X / TB_Y thread-block index lists       X / Y composite tiles, X = side of C's
//   ("left" = input with the output FVI,         fastest index (same rule, enumeration.py:72-99)
//    enumeration.py:72-99)
//   REG_X / REG_Y per-thread register tile     TX x TY MFMA accumulator tiles per wavefront
//   tile menus TB {4,8,16}, REG {1,2,4,6,8}    any divisor / power of two per index, tile
//                                                products up to 512, padded to 16 or 32
//   greedy prefix over consecutive indices     the same greedy prefix (full extents, then
//   (enumeration.py:352-374)                     one partial index, then 1s), tried in C
//                                                order and in operand order
//   cost = DRAM transactions x thread blocks   time = max(HBM, L2 re-reads, MFMA, LDS) with
//                                                coalescing, tail and latency-hiding terms
//   limits: 64..1024 threads, 6144 elements    64..1024 threads, 64 KB LDS per block,
//   of smem (tc_gen.py:167-196)                  accumulators within the VGPR file
//
// A single external index of an input may be given a tile smaller than its
// extent, so the reference's x -> x1,x2 split (configurations.py:93-230) is not
// needed: the grid takes the quotient.  The entry point keeps the un-split arity.
#include "tc_ir.hpp"
#include <algorithm>
#include <array>
#include <cmath>
#include <cstdio>
#include <map>
#include <set>
#include <sstream>

namespace cogent {

static int esize(DType t) { return t == DType::F64 ? 8 : 4; }
static int ceil_div(int a, int b) { return (a + b - 1) / b; }
static int round_up(int a, int b) { return ceil_div(a, b) * b; }

struct MiInfo { int MT, KSTEP, NREG; double cycles; };
static MiInfo mi_info(int mi)
{
    // cycles per instruction per SIMD implied by the published matrix peaks
    // (78.6 TFLOP/s fp64, 157.3 TFLOP/s fp32 over 256 CUs x 4 SIMDs at 2.4 GHz)
    if (mi == 0) return {16, 4, 4, 64.0};
    if (mi == 1) return {16, 4, 4, 32.0};
    return {32, 2, 16, 64.0};
}

std::string Mapping::spec() const
{
    std::ostringstream o;
    auto side = [&](const char* tag, const std::vector<int>& ids, const std::vector<int>& tiles) {
        o << tag << "=";
        for (size_t i = 0; i < ids.size(); i++) o << (i ? "," : "") << ids[i] << ":" << tiles[i];
        o << ";";
    };
    side("x", x_ids, x_tiles);
    side("y", y_ids, y_tiles);
    side("k", k_ids, k_tiles);
    o << "w=" << WX << "x" << WY << ";t=" << TX << "x" << TY << ";mi=" << MI
      << ";lx=" << layx << ";ly=" << layy;
    if (SK > 1) o << ";sk=" << SK;
    if (SKO) o << ";so=1";
    if (MINW > 1) o << ";mw=" << MINW;
    if (LATEC) o << ";lc=1";
    if (ntc_forced >= 0) o << ";nt=" << ntc_forced;
    if (swap_forced >= 0) o << ";sw=" << swap_forced;
    if (pd_forced >= 1) o << ";pd=" << pd_forced;
    if (clds_forced >= 0) o << ";cl=" << clds_forced;
    if (nto_forced >= 0) o << ";no=" << nto_forced;
    if (st_forced > 0) o << ";st=" << st_forced;
    if (SRES) o << ";sy=1";
    if (SOV) o << ";ov=1";
    if (TORD) o << ";to=1";
    if (ESL) o << ";es=1";
    if (!OKP) o << ";ok=0";
    if (SIL) o << ";il=1";
    if (SCD > 1) o << ";cd=" << SCD;
    if (DBUF) o << ";db=1";
    if (VL) o << ";vl=" << VL;
    if (RPX) o << ";rx=1";
    if (RPY) o << ";ry=1";
    return o.str();
}

static std::vector<int> tile_options(int ext, int cap)
{
    std::set<int> s;
    for (int t = 1; t <= ext && t <= cap; t++) if (ext % t == 0) s.insert(t);
    for (int t = 1; t < ext && t <= cap; t *= 2) s.insert(t);
    if (ext <= cap) s.insert(ext);
    return std::vector<int>(s.begin(), s.end());
}

struct SideCand { std::vector<int> ids, tiles; int B; };

// Tile lists for one side.  The reference's greedy prefix (leading indices at their full extent,
// one index with a partial tile, the rest 1; enumeration.py:352-374) plus one generalisation:
// the index after the partial one may carry a tile too, e.g. d:24,c:4 of extents 72,72, which
// gives 96 = 6 MFMA tiles where the prefix rule only offers 72 (4.5 tiles) or 144.
static void prefix_candidates(const Contraction& c, const std::vector<int>& order, int maxB,
                              std::vector<SideCand>& out)
{
    std::set<std::vector<int>> seen;
    const int n = (int)order.size();
    long long P = 1;
    for (int p = 0; p < n; p++) {
        const int ext = c.indices[order[p]].rep_size;
        for (int t : tile_options(ext, maxB)) {
            if (P * t > maxB) break;
            std::vector<int> second = {1};
            if (p + 1 < n && t < ext && t >= 8) second = tile_options(c.indices[order[p + 1]].rep_size, maxB);
            for (int t2 : second) {
                if (P * t * t2 > maxB) break;
                SideCand sc;
                sc.ids = order;
                sc.tiles.assign(n, 1);
                for (int j = 0; j < p; j++) sc.tiles[j] = c.indices[order[j]].rep_size;
                sc.tiles[p] = t;
                if (p + 1 < n) sc.tiles[p + 1] = t2;
                sc.B = (int)(P * t * t2);
                std::vector<int> key = sc.ids;
                key.insert(key.end(), sc.tiles.begin(), sc.tiles.end());
                if (seen.insert(key).second) out.push_back(sc);
            }
        }
        P *= ext;
        if (P > maxB) break;
    }
}

static int pos_in(const std::vector<int>& v, int id)
{
    for (int i = 0; i < (int)v.size(); i++) if (v[i] == id) return i;
    return -1;
}

// LDS leading dimension (elements) that keeps the MFMA operand reads free of bank conflicts.
//   k-major (addr = k*LD + e): the rows read together by one half-wave must land in
//   different bank groups: LD = 16 mod 32 for 8-byte elements; 16 mod 64 (16-wide tiles)
//   or 32 mod 64 (32-wide tiles) for 4-byte elements.
//   e-major (addr = e*LD + k): LD = BKP + 2 (8-byte, or 32-wide 4-byte tiles) or
//   BKP + 4 (16-wide 4-byte tiles), bumped until LD/2 (resp. LD/4) is odd.
static int lds_ld(int lay, int bep, int bkp, DType t, int mi)
{
    if (lay == 0) {
        int mod = (t == DType::F64) ? 32 : 64;
        int want = (t == DType::F64) ? 16 : (mi == 2 ? 32 : 16);
        int ld = bep;
        while (ld % mod != want) ld++;
        return ld;
    }
    if (t == DType::F64 || mi == 2) {
        int ld = bkp + 2;
        while ((ld % 2) || ((ld / 2) % 2 == 0)) ld++;
        return ld;
    }
    int ld = bkp + 4;
    while ((ld % 4) || ((ld / 4) % 2 == 0)) ld++;
    return ld;
}

static int fvi(const std::vector<int>& idx) { return idx.empty() ? -1 : idx[0]; }

void finish_geometry(const Contraction& c, DType t, Mapping& m)
{
    const MiInfo mi = mi_info(m.MI);
    m.BX = 1; for (int v : m.x_tiles) m.BX *= v;
    m.BY = 1; for (int v : m.y_tiles) m.BY *= v;
    m.BK = 1; for (int v : m.k_tiles) m.BK *= v;
    m.BXP = m.WX * m.TX * mi.MT;
    m.BYP = m.WY * m.TY * mi.MT;
    m.BKP = round_up(m.BK, mi.KSTEP);
    m.ldx = lds_ld(m.layx, m.BXP, m.BKP, t, m.MI);
    m.ldy = lds_ld(m.layy, m.BYP, m.BKP, t, m.MI);
    const int ex = m.layx == 0 ? m.BKP * m.ldx : m.BXP * m.ldx;
    const int ey = m.layy == 0 ? m.BKP * m.ldy : m.BYP * m.ldy;
    m.lds_bytes = (ex + ey) * esize(t);
    // fp32: put C's fastest index on the MFMA rows when its tile is a multiple of 4 (128-bit C accesses)
    const bool can_swap = t == DType::F32 && !m.x_tiles.empty() && m.x_ids[0] == c.out_idx[0] && m.x_tiles[0] % 4 == 0;
    m.SWAP = can_swap && (m.swap_forced != 0) ? 1 : 0;
}

std::vector<int> operand_order(const Contraction& c, const Mapping& m, bool x_side)
{
    const bool is_a = x_side ? m.x_is_a : !m.x_is_a;
    if (!(x_side ? m.RPX : m.RPY)) return is_a ? c.a_idx : c.b_idx;
    std::vector<int> o = x_side ? m.x_ids : m.y_ids;
    o.insert(o.end(), m.k_ids.begin(), m.k_ids.end());
    return o;
}

bool check_mapping(const Contraction& c, DType t, const ArchGfx950& arch, const Mapping& m, std::string& err)
{
    const MiInfo mi = mi_info(m.MI);
    if ((t == DType::F64) != (m.MI == 0)) { err = "matrix instruction does not match the element type"; return false; }
    const std::vector<int>& xop = m.x_is_a ? c.a_idx : c.b_idx;
    const std::vector<int>& yop = m.x_is_a ? c.b_idx : c.a_idx;
    std::vector<int> seen(c.n_idx(), 0);
    auto side = [&](const std::vector<int>& ids, const std::vector<int>& tiles, const std::vector<int>& op, bool internal, const char* what) -> bool {
        if (ids.size() != tiles.size()) { err = std::string(what) + ": ids and tiles differ in length"; return false; }
        for (size_t i = 0; i < ids.size(); i++) {
            int id = ids[i];
            if (id < 0 || id >= c.n_idx()) { err = std::string(what) + ": unknown index id"; return false; }
            if (c.indices[id].internal != internal) { err = std::string(what) + ": index '" + c.indices[id].name + "' is on the wrong side"; return false; }
            if (pos_in(op, id) < 0) { err = std::string(what) + ": index '" + c.indices[id].name + "' is not in that operand"; return false; }
            if (tiles[i] < 1) { err = std::string(what) + ": tile must be positive"; return false; }
            seen[id]++;
        }
        return true;
    };
    if (!side(m.x_ids, m.x_tiles, xop, false, "x") || !side(m.y_ids, m.y_tiles, yop, false, "y")) return false;
    if (!side(m.k_ids, m.k_tiles, xop, true, "k")) return false;
    for (int i = 0; i < c.n_idx(); i++)
        if (seen[i] != 1) { err = "index '" + c.indices[i].name + "' must be mapped exactly once"; return false; }
    if (m.x_ids.empty()) { err = "the input holding the output's fastest index needs an external index"; return false; }
    const int threads = 64 * m.WX * m.WY;
    if (threads < 64 || threads > arch.max_threads_per_block) { err = "threads per block outside 64..1024"; return false; }
    if (m.BXP < m.BX || m.BYP < m.BY) { err = "wavefront tiling does not cover the block tile"; return false; }
    if (m.lds_bytes > (m.DBUF ? arch.lds_bytes_per_cu : arch.lds_bytes_per_block)) {
        err = m.DBUF ? "LDS slices exceed the 160 KB of a CU" : "LDS slices exceed 64 KB per block";
        return false;
    }
    const int acc_regs = m.TX * m.TY * mi.NREG * (esize(t) / 4);
    // 512 registers per lane and SIMD are shared by the block's wavefronts on that SIMD;
    // the accumulators may take half of a wavefront's share.  A mapping given as a spec may take all but
    // the ~56 registers the rest of the kernel needs at least (whether it then spills is for its author,
    // or the tuner's clock, to find out).
    const int waves_per_simd = ceil_div(m.WX * m.WY, arch.simd_per_cu);
    const int reg_budget = std::min(512, arch.vgpr_per_lane / waves_per_simd);
    if (acc_regs > 256 || (m.from_spec ? acc_regs + 56 > reg_budget : acc_regs * 2 > reg_budget)) { err = "accumulator tiles exceed the register budget per lane"; return false; }
    if (m.layx < 0 || m.layx > 1 || m.layy < 0 || m.layy > 1) { err = "unknown LDS layout"; return false; }
    if (m.SK < 1 || m.SK > 64) { err = "split-K factor outside 1..64"; return false; }
    if (m.MINW < 1 || m.MINW > 8) { err = "wavefronts per SIMD outside 1..8"; return false; }
    return true;
}

// LDS of the streaming kernel: the resident panel over all K blocks and two slices of the other side
static long long stream_lds_bytes(DType t, const Mapping& m, long long nkb)
{
    const long long lds_x = (m.layx == 0 ? (long long)m.BKP * m.ldx : (long long)m.BXP * m.ldx);
    const long long lds_y = (m.layy == 0 ? (long long)m.BKP * m.ldy : (long long)m.BYP * m.ldy);
    return (long long)esize(t) * (m.SRES ? nkb * lds_y + 2 * lds_x : nkb * lds_x + 2 * lds_y);
}

void cost_model(const Contraction& c, DType t, const ArchGfx950& arch, Mapping& m)
{
    const MiInfo mi = mi_info(m.MI);
    const double s = esize(t);
    auto ext = [&](int id) { return (double)c.indices[id].rep_size; };
    auto tile_of = [&](int id) -> int {
        int p;
        if ((p = pos_in(m.x_ids, id)) >= 0) return m.x_tiles[p];
        if ((p = pos_in(m.y_ids, id)) >= 0) return m.y_tiles[p];
        if ((p = pos_in(m.k_ids, id)) >= 0) return m.k_tiles[p];
        return 1;
    };
    double nC = 1, nA = 1, nB = 1;
    for (int id : c.out_idx) nC *= ext(id);
    for (int id : c.a_idx) nA *= ext(id);
    for (int id : c.b_idx) nB *= ext(id);

    long long nblocks = 1;
    for (size_t i = 0; i < m.x_ids.size(); i++) nblocks *= ceil_div(c.indices[m.x_ids[i]].rep_size, m.x_tiles[i]);
    for (size_t i = 0; i < m.y_ids.size(); i++) nblocks *= ceil_div(c.indices[m.y_ids[i]].rep_size, m.y_tiles[i]);
    long long nkb = 1;
    for (size_t i = 0; i < m.k_ids.size(); i++) nkb *= ceil_div(c.indices[m.k_ids[i]].rep_size, m.k_tiles[i]);
    // non-temporal input loads (mapping spec no= only: bit 0 X side, bit 1 Y side), meant for an input
    // every element of which is read once.  Measured: config 1's 134 MB input, read once in 128-byte
    // pieces, got 6 % slower with the hint; TCCG-15 6 % faster.  Never chosen automatically.
    m.NTO = m.nto_forced >= 0 ? m.nto_forced : 0;
    // split K: SK workgroups per tile, each a share of the K blocks, accumulated with atomics
    const int sk = (nkb > 1) ? std::max(1, m.SK) : 1;
    const double c_passes = sk > 1 ? (double)sk : 1.0;
    nblocks *= sk;
    nkb = (nkb + sk - 1) / sk;
    m.n_blocks = nblocks;
    m.steps_main_loop = (int)nkb;

    // contiguous run of C covered by neighbouring lanes (elements)
    double run = 1;
    if (!m.x_ids.empty() && m.x_ids[0] == c.out_idx[0]) {
        run = m.x_tiles[0];
        size_t j = 0;
        while (j + 1 < m.x_ids.size() && m.x_tiles[j] == c.indices[m.x_ids[j]].rep_size &&
               pos_in(c.out_idx, m.x_ids[j + 1]) == pos_in(c.out_idx, m.x_ids[j]) + 1) {
            run *= m.x_tiles[j + 1];
            j++;
        }
    }
    const double seg_bytes = std::min(run, (double)mi.MT) * s;
    // whole aligned 128-byte lines per lane group: the first X tile is a multiple of a line and the
    // index's full extent keeps every row start on a line boundary at the representative sizes
    m.NTC = (m.ntc_forced >= 0) ? m.ntc_forced
          : (seg_bytes >= 128.0 && ((long long)(m.x_tiles[0] * s) % 128 == 0) && ((long long)(ext(m.x_ids[0]) * s) % 128 == 0)) ? 3 : 0;
    const double c_l1_eff = std::min(1.0, seg_bytes / 128.0);
    // contiguous chunk of C owned by one block (bytes): whole 128-byte lines or not
    double chunk = 1;
    for (int id : c.out_idx) {
        const int tl = tile_of(id);
        chunk *= tl;
        if (tl != c.indices[id].rep_size) break;
    }
    // C through LDS (mapping spec cl=1 only): possible for 16-byte multiples along C's fastest index,
    // tiles of at most 64 KB, no split K.  The tile is then moved in its own memory order with 16-byte
    // accesses, a contiguous kilobyte per wavefront instruction, non-temporal when it is made of whole
    // lines.  Measured on config 4 (96-byte rows, 2304-byte planes) and on the TCCG 6-D shapes it
    // changed nothing (+-2 %), on config 5 it cost 12 %: never chosen automatically.
    {
        const double tile_bytes = (double)m.BX * m.BY * s;
        const bool possible = ((long long)(tile_of(c.out_idx[0]) * s) % 16 == 0) && tile_bytes <= 65536.0 && m.SK == 1 &&
                              !(m.LATEC && nkb > 1);
        const bool whole_lines = chunk * s >= 256.0 && std::fmod(chunk * s, 128.0) == 0.0;
        m.CLDS = (m.clds_forced == 1 && possible) ? 1 : 0;
        if (m.CLDS && m.ntc_forced < 0) m.NTC = whole_lines ? 3 : 0;
    }
    // 128-byte lines a contiguous chunk of the tile touches, relative to the bytes it holds: chunks start at multiples
    // of g bytes (their own size, and C's row pitch when a chunk is part of a row), so a chunk touches
    // bytes / 128 + 1 - gcd(g, 128) / 128 lines on average; the lines it only partly owns are shared with a neighbouring
    // tile and move twice (config 2: 128-byte chunks at a 576-byte row pitch measured 196 us, 192-byte chunks 118,
    // whole 1152-byte chunks 98)
    double c_hbm_eff;
    {
        const long long chunk_b = (long long)(chunk * s), row_b = (long long)(ext(c.out_idx[0]) * s);
        const bool within_row = tile_of(c.out_idx[0]) != c.indices[c.out_idx[0]].rep_size;
        long long g = within_row ? std::__gcd(chunk_b, row_b) : chunk_b;
        g = std::__gcd(g, 128LL);
        const double lines = (double)chunk_b / 128.0 + 1.0 - (double)g / 128.0;
        c_hbm_eff = ((double)chunk_b / 128.0) / lines;
    }
    // address span of the block's C tile relative to its volume: compact tiles keep DRAM pages and
    // TLB entries busy with fewer blocks (measured: tiling the Y side in C's own index order beats
    // the operand's order by 20-40% on the 6-D contractions)
    double span = 1, vol = 1, strideC = 1;
    for (int id : c.out_idx) {
        const int tl = tile_of(id);
        span += (tl - 1) * strideC;
        vol *= tl;
        strideC *= ext(id);
    }
    const double spread = 1.0 + 0.012 * std::log2(std::max(1.0, span / vol));

    // ---- registers per lane, calibrated on hipcc's reports for this kernel: accumulators, one
    // value register set per staged slice element, C offsets, MFMA operands and ~40 of
    // bookkeeping; with a K loop the per-element addresses are hoisted out of it (two more each)
    const int W = m.WX * m.WY;
    const int r4 = (int)(s / 4);
    const int acc_regs = m.TX * m.TY * mi.NREG * r4;
    const int slots = (int)(std::ceil((double)m.BK * m.BX / (64.0 * W)) + std::ceil((double)m.BK * m.BY / (64.0 * W)));
    int regs = acc_regs + 40 + slots * r4 + (m.TX + m.TY * mi.NREG) + (m.TX + m.TY) * r4;
    if (nkb > 1) regs += 2 * slots;
    if (m.STREAM > 0) regs += acc_regs;                 // the streaming kernel holds the next tile's C values next to the accumulators
    // prefetch depth: one K block ahead unless a mapping spec asks for more (pd=); each extra stage
    // holds one slice share in registers, and on the shapes measured so far the registers were worth
    // more as a resident wavefront
    m.PD = 1;
    if (nkb > 1 && m.pd_forced >= 1) m.PD = m.pd_forced;
    regs += (m.PD - 1) * slots * (r4 + 1);
    const int reg_cap = std::min(512, arch.vgpr_per_lane / ceil_div(W, arch.simd_per_cu));
    const double spill_penalty = regs > reg_cap ? 1.0 + 2.0 * (double)(regs - reg_cap) / reg_cap : 1.0;
    int waves_per_simd = std::max(1, std::min(8, arch.vgpr_per_lane / std::max(regs, 64)));
    const bool two_stage = nkb > 1 && (2 * m.lds_bytes <= arch.lds_bytes_per_block || (m.DBUF && 2 * m.lds_bytes <= arch.lds_bytes_per_cu));
    int lds_block = std::max(m.lds_bytes * (two_stage ? 2 : 1), m.CLDS ? (int)(m.BX * m.BY * s) : 0);
    if (m.STREAM > 0) lds_block = (int)std::min<long long>(arch.lds_bytes_per_cu, stream_lds_bytes(t, m, m.STREAM));
    int r = std::min(arch.lds_bytes_per_cu / std::max(lds_block, 1), arch.max_waves_per_cu / W);
    r = std::min(r, std::max(1, waves_per_simd * arch.simd_per_cu / W));
    r = std::max(r, 1);
    r = (int)std::min<long long>(r, std::max<long long>(1, ceil_div((int)std::min<long long>(nblocks, 1 << 30), arch.n_cu)));
    m.blocks_per_cu = r;
    const double waves_simd = (double)(r * W) / arch.simd_per_cu;      // resident wavefronts per SIMD

    const std::vector<int> xop = operand_order(c, m, true), yop = operand_order(c, m, false);
    // ---- HBM: a streaming kernel reaches the sustained rate only with about four resident
    // wavefronts per SIMD in different phases (load C / contract / store C); measured 0.75 at two
    const double bw = arch.hbm_bytes_per_s * arch.hbm_sustained_fraction;
    // (wavefronts of one block move in lock-step between barriers, so blocks count too)
    const double occ_eff = std::min(1.0, 0.5 + 0.125 * waves_simd) * (r >= 3 ? 1.0 : r == 2 ? 0.93 : 0.85);
    // an input whose tile is shorter than a 64-byte sector along its fastest index is fetched with waste
    const double nX = m.x_is_a ? nA : nB, nY = m.x_is_a ? nB : nA;
    auto sector_eff = [&](const std::vector<int>& op) { return std::min(1.0, tile_of(op[0]) * s / 64.0); };
    m.t_hbm = (nX * s / sector_eff(xop) + nY * s / sector_eff(yop) + 2.0 * nC * s * c_passes * spread / c_hbm_eff) / (bw * occ_eff);
    // a K loop in a memory-bound kernel: the variant without one requests its slices and its C tile together and has
    // nothing else to wait for; with a loop a tile spends about a microsecond more in which it requests nothing from
    // memory, and only the other workgroups of the CU keep the memory pipe busy meanwhile.  How MANY K blocks the loop
    // has matters little (4-D shapes measured best with 18 blocks of 4).  The 6-D shapes with a 24-deep contracted
    // index: one K block 107-129 us, blocks of 4 137-154 us.
    // Likewise the first slices of a tile: until they are in LDS the tile computes nothing, and the wait grows with
    // their size at about a CU's share of the memory bandwidth (one 55 KB slice pair per tile measured 1.3-1.4 times
    // slower than 8-deep K blocks on the 5-D shapes; 41 KB against 7 KB 1.2 times on the 4-D shapes).
    // (The variant without a K loop requests its slices together with its C tile and waits for both at once: no such
    // term there, as long as the slices are no larger than the kernel was measured with, see the end of this function.)
    if (m.STREAM == 0 && nkb > 1) {
        const double fill = (double)m.BK * (m.BX + m.BY) * s / (arch.hbm_bytes_per_s / arch.n_cu);
        m.t_hbm += (double)nblocks * (fill + 1.0e-6) / ((double)arch.n_cu * r);
    }
    const double l1_bw = 64.0 * arch.n_cu * arch.clock_hz;
    const double t_l1 = 2.0 * nC * s * c_passes / (l1_bw * c_l1_eff);

    // ---- operand slices are re-read by every block that needs them; they mostly hit in L2 / Infinity Cache
    auto op_eff = [&](const std::vector<int>& op) {
        double rn = tile_of(op[0]);
        size_t j = 0;
        while (j + 1 < op.size() && tile_of(op[j]) == c.indices[op[j]].rep_size) { rn *= tile_of(op[j + 1]); j++; }
        // an input of at most 2 MB stays in the L2 of every XCD (4 MB) and its lines are shared by neighbouring lanes and
        // tiles: short runs then waste 32-byte requests, not 128-byte lines (config 4: 16-byte runs of a 1.3 MB input
        // measured FASTER than 32-byte runs with twice the slice volume)
        double total = s;
        for (int id : op) total *= ext(id);
        return std::min(1.0, rn * s / (total <= 2.0e6 ? 32.0 : 128.0));
    };
    double stage_x = (double)nblocks * nkb * m.BK * m.BX * s;
    double stage_y = (double)nblocks * nkb * m.BK * m.BY * s;
    if (m.STREAM > 0) {
        // panel-resident streaming kernel: a workgroup fetches the resident side once for its whole run of tiles,
        // and its reads of the next tile's C are in flight while the current one is contracted, so that the
        // memory pipe does not wait for co-resident workgroups in other phases (measured 0.55-0.75 of the HBM
        // peak with ONE workgroup per CU, where the per-tile kernel needs three)
        const double wgs = (double)std::min<long long>(nblocks, (long long)arch.n_cu * std::max(1, m.blocks_per_cu));
        (m.SRES ? stage_y : stage_x) *= wgs / (double)nblocks;
        m.t_hbm *= occ_eff / std::min(0.95, 0.55 + 0.05 * r * W);
    }
    m.t_l2 = stage_x / (arch.l2_bytes_per_s * op_eff(xop)) + stage_y / (arch.l2_bytes_per_s * op_eff(yop));

    // ---- matrix cores: wavefronts of the resident blocks spread over 4 SIMDs (9 wavefronts leave
    // three SIMDs idle a third of the time); every wavefront also pays about 700 issue cycles of
    // address arithmetic, staging and barrier per K block next to its MFMAs
    // (a block's wavefronts are dealt to the SIMDs starting at SIMD 0: 6 or 9 of them load the SIMDs unevenly;
    // measured: 6-wavefront blocks run 40% slower than 4-wavefront ones on the same tile volume)
    const double per_block = W >= arch.simd_per_cu ? ((double)W / arch.simd_per_cu) / std::ceil((double)W / arch.simd_per_cu) : 1.0;
    const double simd_busy = waves_simd / std::ceil(waves_simd);          // (uneven wavefront counts per workgroup: priced on the total below)
    const double n_mfma = (double)nblocks * nkb * (m.BKP / mi.KSTEP) * (m.BXP / mi.MT) * (m.BYP / mi.MT);
    const double simd_hz = (double)arch.n_cu * arch.simd_per_cu * arch.clock_hz;
    // issue cycles next to the MFMAs, per wavefront and K block: loop, barrier and LDS operand reads
    // (~250) plus load, address and LDS-store instructions for every slice element the lane stages
    // (~10 each).  Calibrated on TCCG-22: 96x96x8 tiles on 4 wavefronts measured 72 % of MFMA peak
    // (6 elements per lane), 48x96x48 tiles on 2 wavefronts 59 % (54 per lane and one wavefront per SIMD).
    const double t_overhead = (double)nblocks * nkb * W * (250.0 + 10.0 * slots) / simd_hz;
    // an LDS-fed MFMA loop needs co-resident wavefronts to cover LDS and MFMA latency: measured 68 % of
    // peak with one wavefront per SIMD, 84 % with two, little more beyond
    // (the wavefronts of ONE workgroup meet at every barrier and so stall together: what counts is the number of
    // workgroups on the CU -- twelve wavefronts of one workgroup measured 64 % on config 3, where two workgroups
    // of four reached 77 % with a second K block requested ahead)
    // Both counts matter: one-wavefront workgroups, however many of them, leave every SIMD with a single wavefront that
    // stages its slices alone (the DGEMM on 48x80 tiles of one wavefront measured 1.34 times its four-wavefront mapping).
    // With a second K block in flight in registers the global loads are never exposed and a lone large workgroup keeps
    // its matrix cores fed (4-D x 4-D shapes, 192x192 tiles on twelve wavefronts, 8-deep K blocks, pd=2: 78-84 % of
    // peak).  Not with split K: there a workgroup ends with an atomic pass over its tile that only another workgroup
    // of the CU can overlap (config 3, 144x192 tiles on twelve wavefronts, pd=2: 64 %); there it is worth five points.
    const double by_groups = r >= 3 ? 0.92 : r == 2 ? 0.84 : 0.70;
    const double by_waves = waves_simd >= 3.0 ? 0.92 : waves_simd >= 2.0 ? 0.84 : 0.68;
    const double mfma_occ = (m.PD >= 2 && sk == 1) ? std::min(0.92, std::max(by_waves, by_groups + 0.05))
                                                   : std::min(0.92, std::min(by_groups, by_waves) + (m.PD >= 2 ? 0.05 : 0.0));
    m.t_mfma = (n_mfma * mi.cycles / simd_hz / mfma_occ + t_overhead) / simd_busy;

    const double lds_reads = (double)nblocks * nkb * (m.BKP / mi.KSTEP) * W * (m.TX + m.TY) * 64.0 * s;
    m.t_lds = (lds_reads + stage_x + stage_y) / (arch.lds_bytes_per_clk_cu * arch.n_cu * arch.clock_hz);

    // ---- tail: blocks are handed out as slots free up, so the last CU finishes at most one block late
    const double per_cu = (double)nblocks / arch.n_cu;
    m.tail_eff = per_cu / std::ceil(per_cu);
    if (per_cu > 1.0) m.tail_eff = std::max(m.tail_eff, per_cu / (std::floor(per_cu) + 1.0));

    const double parts[4] = {m.t_hbm, m.t_l2, m.t_mfma, m.t_lds};
    double mx = t_l1, sum = t_l1;
    for (double p : parts) { mx = std::max(mx, p); sum += p; }
    // the slowest pipe sets the pace; the others overlap imperfectly
    // (where HBM sets the pace the slice traffic weighs more than the rest: the slices come through the same L2 and
    // fabric as C, and the mappings measured best on the 6-D shapes were those with the least of it among near-equal
    // HBM terms)
    m.cost = (mx + 0.15 * (sum - mx) + (std::max(m.t_hbm, m.t_l2) >= mx ? 0.25 * std::min(m.t_l2, m.t_hbm) : 0.0)) * spill_penalty / std::max(m.tail_eff, 0.05) + 2.0e-6;
    // one K block with more than 32 KB of slices: measured 1.3-1.4 times slower than an 8-deep K loop (5-D shapes, 55 KB);
    // 16 and 25 KB are where the one-block kernel wins (6-D shapes)
    if (nkb == 1 && (double)m.BK * (m.BX + m.BY) * s > 32768.0) m.cost *= 1.3;
    // workgroups whose wavefronts load the SIMDs unevenly are slow whatever binds (6 wavefronts: +40 % measured on an
    // HBM-bound shape), and a tile that does not divide its representative extent sends every call at those extents to
    // the predicated kernel variant (no vector accesses, edge tests in every access)
    m.cost /= std::max(0.6, per_block);
    {
        bool ragged = false;
        for (size_t i = 0; i < m.x_ids.size(); i++) ragged = ragged || (c.indices[m.x_ids[i]].rep_size % m.x_tiles[i]) != 0;
        for (size_t i = 0; i < m.y_ids.size(); i++) ragged = ragged || (c.indices[m.y_ids[i]].rep_size % m.y_tiles[i]) != 0;
        for (size_t i = 0; i < m.k_ids.size(); i++) ragged = ragged || (c.indices[m.k_ids[i]].rep_size % m.k_tiles[i]) != 0;
        if (ragged) m.cost *= 1.10;
    }
    // the streaming kernel must win clearly: on the 6-D shapes it measured level with the per-tile kernel for most
    // index orders and a third slower for some, which nothing above tells apart
    if (m.STREAM > 0) m.cost *= 1.05;
    // a repacked input is read and written once more by a kernel of its own, which the contraction waits for
    if (m.RPX) m.cost += 2.0 * nX * s / bw + 4.0e-6;
    if (m.RPY) m.cost += 2.0 * nY * s / bw + 4.0e-6;
}

static bool plan_stream(const Contraction& c, DType t, const ArchGfx950& arch, Mapping& m, std::string& err);

static long long k_blocks(const Contraction& c, const Mapping& m)
{
    long long nkb = 1;
    for (size_t i = 0; i < m.k_ids.size(); i++) nkb *= ceil_div(c.indices[m.k_ids[i]].rep_size, m.k_tiles[i]);
    return nkb;
}

// 16-byte slice loads (vl=) for the inputs whose tile along their fastest index spans at least half a line
static int vector_sides(const Contraction& c, DType t, const Mapping& m)
{
    auto tile_of = [&](int id) -> int {
        int p;
        if ((p = pos_in(m.x_ids, id)) >= 0) return m.x_tiles[p];
        if ((p = pos_in(m.y_ids, id)) >= 0) return m.y_tiles[p];
        if ((p = pos_in(m.k_ids, id)) >= 0) return m.k_tiles[p];
        return 1;
    };
    const std::vector<int> xop = operand_order(c, m, true), yop = operand_order(c, m, false);
    const bool vx = !xop.empty() && tile_of(xop[0]) * esize(t) >= 64, vy = !yop.empty() && tile_of(yop[0]) * esize(t) >= 64;
    return vx && vy ? 1 : vx ? 2 : vy ? 3 : 0;
}

// Options that the cost terms do not separate, set the way they measured best on the part.  (A mapping spec sets
// them itself; these rules only act on the mappings the pass enumerates.)
//   One K block (the many-index shapes whose cost is the traffic of C): tiles handed out in the order of their
//   origins in C's memory, -7 to -12 % on the 6-D shapes of the benchmark set; C through LDS when C's rows are not
//   whole 128-byte lines (96-byte fp32 rows, 192-byte fp64 rows: -5 % and -3 to -5 %), not otherwise (+12 % on
//   128-byte rows).
//   With or without a K loop: 16-byte slice loads for the inputs whose tile along their fastest index spans half a
//   line or more (config 1: -5 %; figures for one K block at the rule itself).
static void measured_rules(const Contraction& c, DType t, Mapping& m)
{
    // C through LDS in memory order, with non-temporal accesses, when C's rows are not whole 128-byte lines (96-byte
    // fp32 rows -5 %, 192-byte fp64 rows -3 to -5 % with one K block; the 3-D and 4-D shapes with 192-byte rows and a K
    // loop 89 -> 70 us); not on whole-line rows (+12 %).  The cost model drops it where the tile exceeds 64 KB.
    {
        const long long row = (long long)m.x_tiles[0] * esize(t);
        const bool fits = (long long)m.BX * m.BY * esize(t) <= 65536;
        if (row % 128 != 0 && row % 16 == 0 && m.SK == 1 && fits) { m.clds_forced = 1; m.ntc_forced = 3; }
        // ... in fp32 with the first slices requested before the tile is staged (nine 6-D shapes at extents 24/16
        // -5 to -11 %, config 4 at 24s -3 %; fp64 shapes 0 to +7 %: the slices held in registers through the staging
        // cost a resident wavefront there)
        if (m.clds_forced == 1 && t == DType::F32) m.ESL = 1;
    }
    if (k_blocks(c, m) != 1) {
        m.VL = vector_sides(c, t, m);
        // a long K loop: a second K block in flight in registers (config 3 +12-17 %, the DGEMM and the 4-D x 4-D shapes
        // +4-10 %), which pays where the register budget takes it: small slice shares per lane
        const int W = m.WX * m.WY;
        const int slots = (m.BK * m.BX + 64 * W - 1) / (64 * W) + (m.BK * m.BY + 64 * W - 1) / (64 * W);
        if (k_blocks(c, m) / std::max(1, m.SK) >= 8 && slots <= 8) m.pd_forced = 2;
        return;
    }
    if (m.SK > 1) return;
    m.TORD = 1;
    // 16-byte slice loads by the same 64-byte rule as with a K loop.  Runs of 128 bytes on both sides: -1 to -2 % on the
    // 6-D shapes at extent 16.  A side with 32-byte runs loaded that way: +6 % on the 6-D shapes at extents 24/16.  The
    // long side alone there: -5 % on the picks with four wavefronts in a row and on config 4 at 24s, +3 % on the picks
    // with two by two (no vector loads at all would suit those, and cost the others 2 to 7 %).
    // ... and only where the vectors fill the workgroup's lanes well enough to save instructions: a side is loaded in
    // ceil(elements / lanes) rounds of 8-byte loads or ceil(vectors / lanes) rounds of 16-byte ones, and a 16-byte
    // round costs about one and a half 8-byte rounds (a 32x24 fp64 slice on 256 lanes: 3 rounds against 2, the second
    // half empty, measured +3 %; 48x24: 5 against 3, -2 to -5 %; 128x16: 8 against 4, -1 to -2 %)
    {
        const int side = vector_sides(c, t, m);
        const int lanes = 64 * m.WX * m.WY, v = 16 / esize(t);
        auto pays = [&](int ext_tile) {
            const int elems = m.BK * ext_tile;
            return 3 * ceil_div(ceil_div(elems, v), lanes) < 2 * ceil_div(elems, lanes);
        };
        const bool vx = (side == 1 || side == 2) && pays(m.BX), vy = (side == 1 || side == 3) && pays(m.BY);
        m.VL = vx && vy ? 1 : vx ? 2 : vy ? 3 : 0;
    }
}

// The streaming kernel for an enumerated mapping: depth 3 for three K blocks, else 2; C non-temporal; runs of the
// workgroups interleaved (-1 to -4 % wherever it was measured); the resident panel loaded behind the first tile when
// it is larger than 64 KB (config 2: -4 %).
static bool stream_variant(const Contraction& c, DType t, const ArchGfx950& arch, Mapping& m)
{
    const long long nkb = k_blocks(c, m);
    // three K blocks or more: with two, the kernel measured level with the per-tile kernel at best (config 4 with 16s,
    // some 6-D shapes) and a third to two thirds slower on others (config 4, config 5 #9), which nothing here tells apart
    // (and no more: its design point is a handful of K blocks per tile; every win of this kernel that came out of these
    // candidates had three.  On config 1 one tile shape with 16 K blocks measured 28 us, another, which the model
    // priced lower, 52 us, and one with four 33 us against 30 us for the per-tile pick)
    if (nkb != 3 || m.SK > 1) return false;
    if (t != DType::F64) return false;       // fp32: its one measured win had two K blocks; the six-index fp32 shape ran 1.7 to 2 times slower with it
    // every measured win of this kernel had eight or more wavefronts with at most three accumulator tiles each (its one
    // workgroup per CU is all that hides the memory latency; two wavefronts with 18 tiles each ran at half the
    // per-tile kernel's speed on config 4)
    if (m.WX * m.WY < 8 || m.TX * m.TY > 3) return false;
    // ... and contiguous chunks of C made of whole 128-byte lines, which its non-temporal accesses need (on partial
    // lines they defeat write combining: +35 % on 96-byte fp32 rows)
    {
        long long chunk = esize(t);
        for (int id : c.out_idx) {
            int p, tl = 1;
            if ((p = pos_in(m.x_ids, id)) >= 0) tl = m.x_tiles[p];
            else if ((p = pos_in(m.y_ids, id)) >= 0) tl = m.y_tiles[p];
            chunk *= tl;
            if (tl != c.indices[id].rep_size) break;
        }
        if (chunk % 128) return false;
    }
    // the panel is worth keeping only if several tiles of the other side pass by it (with one, "resident" means an
    // exposed panel load per tile: 167 against 126 us on the 4-D shapes whose second input is a 72x72 matrix)
    {
        long long streamed = 1;
        const std::vector<int>& ids = m.SRES ? m.x_ids : m.y_ids;
        const std::vector<int>& tiles = m.SRES ? m.x_tiles : m.y_tiles;
        for (size_t i = 0; i < ids.size(); i++) streamed *= ceil_div(c.indices[ids[i]].rep_size, tiles[i]);
        if (streamed < 4) return false;
    }
    m.st_forced = nkb == 3 ? 3 : nkb % 2 == 0 ? 2 : nkb % 3 == 0 ? 3 : 0;
    if (m.st_forced == 0) return false;
    std::string err;
    if (!plan_stream(c, t, arch, m, err)) return false;
    m.ntc_forced = 3;
    m.SIL = 1;
    const long long panel = (long long)esize(t) * nkb * (m.SRES ? (m.layy == 0 ? (long long)m.BKP * m.ldy : (long long)m.BYP * m.ldy)
                                                                : (m.layx == 0 ? (long long)m.BKP * m.ldx : (long long)m.BXP * m.ldx));
    m.SOV = panel > 65536 ? 1 : 0;
    m.VL = vector_sides(c, t, m);
    return true;
}

static void wave_layouts(int nx, int ny, int max_acc_tiles, std::vector<std::array<int, 4>>& out)
{
    for (int wx = 1; wx <= nx && wx <= 16; wx++) {
        if (nx % wx) continue;
        for (int wy = 1; wy <= ny && wx * wy <= 16; wy++) {
            if (ny % wy) continue;
            const int tx = nx / wx, ty = ny / wy;
            if (tx * ty > max_acc_tiles) continue;
            out.push_back({wx, wy, tx, ty});
        }
    }
}

std::vector<Mapping> enumerate_mappings(const Contraction& c, DType t, const ArchGfx950& arch)
{
    std::vector<Mapping> out;
    if (c.out_idx.empty()) return out;
    const bool x_is_a = c.in_a(c.out_idx[0]);
    const std::vector<int>& xop = x_is_a ? c.a_idx : c.b_idx;
    const std::vector<int>& yop = x_is_a ? c.b_idx : c.a_idx;

    auto externals_in = [&](const std::vector<int>& op, bool by_c_order) {
        std::vector<int> v;
        if (by_c_order) { for (int id : c.out_idx) if (pos_in(op, id) >= 0) v.push_back(id); }
        else            { for (int id : op) if (!c.indices[id].internal) v.push_back(id); }
        return v;
    };
    std::vector<std::vector<int>> x_orders, y_orders, k_orders;
    x_orders.push_back(externals_in(xop, true));          // X must start at C's fastest index
    {
        // ... and may continue in the operand's own order, so that the operand's fastest external
        // index can take a tile even when it is late in C (TCCG-3: C [a,b,c,d], input [d,b,e,a])
        std::vector<int> o = {c.out_idx[0]};
        for (int id : xop) if (!c.indices[id].internal && id != c.out_idx[0]) o.push_back(id);
        if (o != x_orders[0]) x_orders.push_back(o);
    }
    for (int by_c = 1; by_c >= 0; by_c--) {
        std::vector<int> o = externals_in(yop, by_c != 0);
        if (std::find(y_orders.begin(), y_orders.end(), o) == y_orders.end()) y_orders.push_back(o);
    }
    // K composite order: an index that is the fastest one of an operand goes first
    {
        std::vector<int> base = c.int_idx, o1, o2;
        auto order_with_first = [&](int first) {
            std::vector<int> o;
            if (first >= 0 && c.indices[first].internal) o.push_back(first);
            for (int id : xop) if (c.indices[id].internal && pos_in(o, id) < 0) o.push_back(id);
            return o;
        };
        std::vector<std::vector<int>> cand = {order_with_first(fvi(xop)), order_with_first(fvi(yop)), base};
        std::vector<int> by_y;
        for (int id : yop) if (c.indices[id].internal) by_y.push_back(id);
        cand.push_back(by_y);
        for (auto& o : cand)
            if (o.size() == c.int_idx.size() && std::find(k_orders.begin(), k_orders.end(), o) == k_orders.end()) k_orders.push_back(o);
    }

    std::vector<SideCand> xc, yc, kc;
    for (auto& o : x_orders) prefix_candidates(c, o, 256, xc);
    for (auto& o : y_orders) prefix_candidates(c, o, 256, yc);
    for (auto& o : k_orders) prefix_candidates(c, o, 64, kc);
    // an input without external indices (matrix-vector shapes) or without a summed index: one empty tile
    if (yc.empty()) yc.push_back(SideCand{{}, {}, 1});
    if (kc.empty()) kc.push_back(SideCand{{}, {}, 1});
    int max_bx = 1, max_by = 1, max_bk = 1;
    for (auto& s : xc) max_bx = std::max(max_bx, s.B);
    for (auto& s : yc) max_by = std::max(max_by, s.B);
    for (auto& s : kc) max_bk = std::max(max_bk, s.B);
    // external tile products that are whole MFMA tiles (or the whole side when it is small),
    // K tiles that are whole MFMA steps
    auto keep_whole = [](std::vector<SideCand>& v, int gran, int mx) {
        std::vector<SideCand> o;
        for (auto& s : v) if (s.B % gran == 0 || s.B == mx) o.push_back(s);
        if (!o.empty()) v.swap(o);
    };
    keep_whole(xc, 16, max_bx);
    keep_whole(yc, 16, max_by);
    keep_whole(kc, 4, max_bk);

    const std::vector<int> mis = (t == DType::F64) ? std::vector<int>{0} : std::vector<int>{1, 2};
    for (int miv : mis) {
        const MiInfo mi = mi_info(miv);
        const int max_acc_tiles = 128 / (mi.NREG * (esize(t) / 4));     // 128 accumulator registers per lane
        for (const SideCand& kx : kc) {
            if (kx.B < std::min(4, max_bk)) continue;
            for (const SideCand& sx : xc) {
                if (sx.B < std::min(8, max_bx)) continue;
                const int nx = ceil_div(sx.B, mi.MT);
                if ((double)sx.B / (nx * mi.MT) < 0.8 && sx.B != max_bx) continue;
                for (const SideCand& sy : yc) {
                    if (sy.B < std::min(8, max_by)) continue;
                    const int ny = ceil_div(sy.B, mi.MT);
                    if ((double)sy.B / (ny * mi.MT) < 0.8 && sy.B != max_by) continue;
                    std::vector<std::array<int, 4>> wl;
                    wave_layouts(nx, ny, max_acc_tiles, wl);
                    for (auto& w : wl) {
                        Mapping m;
                        m.x_is_a = x_is_a;
                        m.x_ids = sx.ids; m.x_tiles = sx.tiles;
                        m.y_ids = sy.ids; m.y_tiles = sy.tiles;
                        m.k_ids = kx.ids; m.k_tiles = kx.tiles;
                        m.WX = w[0]; m.WY = w[1]; m.TX = w[2]; m.TY = w[3];
                        m.MI = miv;
                        // k-fast LDS layout when the operand's fastest index is the leading K index with a real tile
                        m.layx = (!kx.ids.empty() && kx.ids[0] == fvi(xop) && kx.tiles[0] >= 4) ? 1 : 0;
                        m.layy = (!kx.ids.empty() && kx.ids[0] == fvi(yop) && kx.tiles[0] >= 4) ? 1 : 0;
                        finish_geometry(c, t, m);
                        std::string err;
                        if (!check_mapping(c, t, arch, m, err)) continue;
                        measured_rules(c, t, m);
                        cost_model(c, t, arch, m);
                        out.push_back(m);
                        // the streaming kernel wherever it can run with this tile
                        for (int resident_y = 0; resident_y < 2; resident_y++) {
                            Mapping mv = m;
                            mv.SRES = resident_y;          // either side's panel can be the resident one: the cost terms choose
                            if (stream_variant(c, t, arch, mv)) { cost_model(c, t, arch, mv); out.push_back(mv); }
                        }
                        // few output tiles and a long K loop: also try splitting K over 2, 4, 8 workgroups
                        const long long tiles = m.n_blocks;
                        const int ksteps = m.steps_main_loop;
                        for (int sk = 2; sk <= 64 && tiles * (sk / 2) < 4LL * arch.n_cu && ksteps >= 8 * sk; sk *= 2) {
                            Mapping ms = m;
                            ms.SK = sk;
                            ms.SKO = 1;       // shares outermost: measured ahead of innermost on every split-K shape tried (1-4 %)
                            cost_model(c, t, arch, ms);
                            out.push_back(ms);
                        }
                    }
                }
            }
        }
    }
    // cheapest first; ties go to fewer main-loop steps (configurations.py:260-283)
    std::stable_sort(out.begin(), out.end(), [](const Mapping& a, const Mapping& b) {
        if (a.cost != b.cost) return a.cost < b.cost;
        return a.steps_main_loop < b.steps_main_loop;
    });
    return out;
}

// The pass's own pick with a long K loop and one K block requested ahead: the same tile with 8-deep K blocks and two of
// them in flight, when the smaller slices bring the staged elements per lane within the budget of that option.  The
// cost terms prefer deep K blocks (fewer barriers and loop trips) and do not see that a single block's matrix steps
// are too short to cover the load latency.  Measured, same tile both ways (fp64): 3-D x 2-D shapes with K = 296,
// 16- or 24-deep against 8-deep with two ahead 388 -> 336 us and 362 -> 340 us; the 2-D output with K = 92,000,
// 32-deep 440 -> 8-deep 360 us; config 3, 24-deep 407 -> 398 us.
static void deepen_prefetch(const Contraction& c, DType t, const ArchGfx950& arch, Mapping& pick)
{
    if (t != DType::F64 || pick.STREAM != 0 || pick.PD >= 2 || pick.k_ids.empty()) return;
    if (pick.BK <= 8 || pick.k_tiles[0] < 8 || c.indices[pick.k_ids[0]].rep_size % 8 != 0) return;
    // only where the matrix cores set the pace (a memory-bound 4-D shape lost 6 % with it) ...
    if (pick.t_mfma < std::max(pick.t_hbm, pick.t_l2)) return;
    Mapping m = pick;
    m.k_tiles[0] = 8;
    // ... and no input may lose the tile along its fastest index (4-D x 4-D and 3-D x 3-D shapes whose second
    // contracted index is an input's fastest one: 1.1 to 2.6 times slower with that tile at 1)
    for (size_t i = 1; i < m.k_tiles.size(); i++) {
        if (m.k_tiles[i] > 1 && (m.k_ids[i] == c.a_idx[0] || m.k_ids[i] == c.b_idx[0])) return;
        m.k_tiles[i] = 1;
    }
    finish_geometry(c, t, m);
    std::string err;
    if (!check_mapping(c, t, arch, m, err)) return;
    m.pd_forced = -1;
    measured_rules(c, t, m);
    if (m.pd_forced != 2) return;               // still too many staged elements per lane, or too few K blocks
    cost_model(c, t, arch, m);
    if (m.PD != 2) return;
    pick = m;
}

bool select_mapping(const Contraction& c, DType t, const ArchGfx950& arch, int rank, Mapping& out, std::string& err)
{
    std::vector<Mapping> all = enumerate_mappings(c, t, arch);
    if (all.empty()) { err = "no admissible mapping for this expression"; return false; }
    if (rank >= 0 && rank < (int)all.size()) out = all[rank];   // manual pick, configurations.py:285-289
    else { out = all[0]; deepen_prefetch(c, t, arch, out); }
    return true;
}

// spec grammar: x=<id>:<tile>,...;y=...;k=...;w=<WX>x<WY>;t=<TX>x<TY>;mi=<n>;lx=<0|1>;ly=<0|1>
// index ids may also be given by name.

// The panel-resident streaming kernel for this mapping (spec st=<slices requested ahead>, sy=1 to keep the
// Y panel instead of the X panel): possible when, at the representative extents, every extent is a multiple
// of its tile, there are at least two K blocks, the depth divides their number, and the resident tile over
// the whole contracted range plus two slices of the other operand fit the LDS of a CU.  The K-block count
// becomes a compile-time constant of the emitted object.
static bool plan_stream(const Contraction& c, DType t, const ArchGfx950& arch, Mapping& m, std::string& err)
{
    auto full = [&](const std::vector<int>& ids, const std::vector<int>& tiles) {
        for (size_t i = 0; i < ids.size(); i++) if (c.indices[ids[i]].rep_size % tiles[i]) return false;
        return true;
    };
    if (!full(m.x_ids, m.x_tiles) || !full(m.y_ids, m.y_tiles) || !full(m.k_ids, m.k_tiles)) {
        err = "streaming kernel (st=): tiles must divide the representative extents";
        return false;
    }
    long long nkb = 1;
    for (size_t i = 0; i < m.k_ids.size(); i++) nkb *= c.indices[m.k_ids[i]].rep_size / m.k_tiles[i];
    if (nkb < 2 || nkb > 64 || nkb % m.st_forced) {
        err = "streaming kernel (st=): needs 2..64 K blocks and a prefetch depth that divides their number (K blocks here: " + std::to_string(nkb) + ")";
        return false;
    }
    const long long bytes = stream_lds_bytes(t, m, nkb);
    if (bytes > arch.lds_bytes_per_cu) {
        err = "streaming kernel (st=): the resident panel needs " + std::to_string(bytes) + " bytes of LDS";
        return false;
    }
    m.STREAM = (int)nkb;
    m.SPD = m.st_forced;
    const int waves = m.WX * m.WY;
    const int bpc = std::max(1, std::min((int)(arch.lds_bytes_per_cu / bytes), arch.max_waves_per_cu / 2 / waves));
    m.SMW = std::max(1, std::min(4, (bpc * waves + arch.simd_per_cu - 1) / arch.simd_per_cu));
    // mw= asks for more resident wavefronts per SIMD (fewer registers each, more workgroups per CU): for the
    // HBM-bound shapes with small accumulator tiles the memory system wants as many wavefronts in flight as fit
    if (m.MINW > 1) m.SMW = std::min(8, m.MINW);
    return true;
}

bool mapping_from_spec(const Contraction& c, DType t, const ArchGfx950& arch, const std::string& spec, Mapping& m, std::string& err)
{
    m = Mapping();
    m.x_is_a = c.in_a(c.out_idx[0]);
    m.MI = (t == DType::F64) ? 0 : 1;
    int lx = -1, ly = -1;
    std::istringstream is(spec);
    std::string field;
    auto index_of = [&](const std::string& s) -> int {
        for (int i = 0; i < c.n_idx(); i++) if (c.indices[i].name == s) return i;
        bool digits = !s.empty();
        for (char ch : s) if (ch < '0' || ch > '9') digits = false;
        if (digits) { int v = atoi(s.c_str()); if (v < c.n_idx()) return v; }
        return -1;
    };
    while (std::getline(is, field, ';')) {
        if (field.empty()) continue;
        size_t eq = field.find('=');
        if (eq == std::string::npos) { err = "mapping spec field without '=': " + field; return false; }
        std::string key = field.substr(0, eq), val = field.substr(eq + 1);
        if (key == "x" || key == "y" || key == "k") {
            std::vector<int>& ids = key == "x" ? m.x_ids : key == "y" ? m.y_ids : m.k_ids;
            std::vector<int>& tiles = key == "x" ? m.x_tiles : key == "y" ? m.y_tiles : m.k_tiles;
            std::istringstream vs(val);
            std::string item;
            while (std::getline(vs, item, ',')) {
                size_t colon = item.find(':');
                if (colon == std::string::npos) { err = "mapping spec item without ':': " + item; return false; }
                int id = index_of(item.substr(0, colon));
                if (id < 0) { err = "mapping spec names an unknown index: " + item; return false; }
                ids.push_back(id);
                tiles.push_back(atoi(item.substr(colon + 1).c_str()));
            }
        } else if (key == "w" || key == "t") {
            int a = 0, b = 0;
            if (sscanf(val.c_str(), "%dx%d", &a, &b) != 2 || a < 1 || b < 1) { err = "mapping spec: bad " + key; return false; }
            if (key == "w") { m.WX = a; m.WY = b; } else { m.TX = a; m.TY = b; }
        } else if (key == "mi") m.MI = atoi(val.c_str());
        else if (key == "sk") m.SK = atoi(val.c_str());
        else if (key == "so") m.SKO = atoi(val.c_str()) ? 1 : 0;
        else if (key == "mw") m.MINW = atoi(val.c_str());
        else if (key == "lc") m.LATEC = atoi(val.c_str()) ? 1 : 0;
        else if (key == "nt") m.ntc_forced = std::max(0, std::min(3, atoi(val.c_str())));
        else if (key == "sw") m.swap_forced = atoi(val.c_str()) ? 1 : 0;
        else if (key == "pd") m.pd_forced = std::max(1, std::min(8, atoi(val.c_str())));
        else if (key == "cl") m.clds_forced = atoi(val.c_str()) ? 1 : 0;
        else if (key == "no") m.nto_forced = std::max(0, std::min(3, atoi(val.c_str())));
        else if (key == "st") m.st_forced = std::max(0, std::min(64, atoi(val.c_str())));
        else if (key == "vl") m.VL = std::max(0, std::min(3, atoi(val.c_str())));
        else if (key == "db") m.DBUF = atoi(val.c_str()) ? 1 : 0;
        else if (key == "sy") m.SRES = atoi(val.c_str()) ? 1 : 0;
        else if (key == "ov") m.SOV = atoi(val.c_str()) ? 1 : 0;
        else if (key == "to") m.TORD = atoi(val.c_str()) ? 1 : 0;
        else if (key == "es") m.ESL = atoi(val.c_str()) ? 1 : 0;
        else if (key == "ok") m.OKP = atoi(val.c_str()) ? 1 : 0;
        else if (key == "il") m.SIL = atoi(val.c_str()) ? 1 : 0;
        else if (key == "cd") m.SCD = std::max(1, std::min(2, atoi(val.c_str())));
        else if (key == "rx") m.RPX = atoi(val.c_str()) ? 1 : 0;
        else if (key == "ry") m.RPY = atoi(val.c_str()) ? 1 : 0;
        else if (key == "lx") lx = atoi(val.c_str());
        else if (key == "ly") ly = atoi(val.c_str());
        else { err = "mapping spec: unknown key " + key; return false; }
    }
    if (m.MI < 0 || m.MI > 2) { err = "mapping spec: unknown matrix instruction"; return false; }
    if (m.x_ids.empty()) { err = "mapping spec must give x"; return false; }
    // ranges first: everything below multiplies these numbers
    {
        long long vol = 1;
        for (const std::vector<int>* tl : {&m.x_tiles, &m.y_tiles, &m.k_tiles})
            for (int v : *tl) {
                if (v < 1 || v > 65536) { err = "mapping spec: a tile outside 1..65536"; return false; }
                vol *= v;
                if (vol > (1LL << 24)) { err = "mapping spec: tile volume too large"; return false; }
            }
        if (m.WX < 1 || m.WY < 1 || m.TX < 1 || m.TY < 1 || m.WX > 16 || m.WY > 16 || m.TX > 64 || m.TY > 64) { err = "mapping spec: wavefront grid or MFMA tile count out of range"; return false; }
    }
    const std::vector<int> xop = operand_order(c, m, true), yop = operand_order(c, m, false);
    m.layx = lx >= 0 ? lx : ((!m.k_ids.empty() && m.k_ids[0] == fvi(xop) && m.k_tiles[0] >= 4) ? 1 : 0);
    m.layy = ly >= 0 ? ly : ((!m.k_ids.empty() && m.k_ids[0] == fvi(yop) && m.k_tiles[0] >= 4) ? 1 : 0);
    finish_geometry(c, t, m);
    m.from_spec = true;
    if (!check_mapping(c, t, arch, m, err)) return false;
    // the streaming kernel gives every output tile to exactly one workgroup: K shares cannot be combined with it
    if (m.st_forced > 0 && m.SK > 1) { err = "mapping spec: st= (streaming kernel) and sk= (split K) exclude each other"; return false; }
    if (!m.OKP && m.SK > 1) { err = "mapping spec: ok=0 (ragged single K blocks through the K-loop kernels) and sk= (split K) exclude each other"; return false; }
    if (m.st_forced > 0 && !plan_stream(c, t, arch, m, err)) return false;
    cost_model(c, t, arch, m);
    return true;
}

std::string mapping_json(const Contraction& c, DType t, const Mapping& m)
{
    std::ostringstream o;
    auto side = [&](const char* tag, const std::vector<int>& ids, const std::vector<int>& tiles) {
        o << "\"" << tag << "\": [";
        for (size_t i = 0; i < ids.size(); i++)
            o << (i ? ", " : "") << "[\"" << c.indices[ids[i]].name << "\", " << tiles[i] << "]";
        o << "]";
    };
    o << "{\"dtype\": \"" << (t == DType::F64 ? "f64" : "f32") << "\", \"x_operand\": \"" << (m.x_is_a ? c.a_name : c.b_name) << "\", ";
    side("x", m.x_ids, m.x_tiles); o << ", ";
    side("y", m.y_ids, m.y_tiles); o << ", ";
    side("k", m.k_ids, m.k_tiles); o << ", ";
    const char* names[3] = {"v_mfma_f64_16x16x4_f64", "v_mfma_f32_16x16x4_f32", "v_mfma_f32_32x32x2_f32"};
    o << "\"block_tile\": [" << m.BX << ", " << m.BY << ", " << m.BK << "], \"padded\": [" << m.BXP << ", " << m.BYP << ", " << m.BKP << "], "
      << "\"waves\": [" << m.WX << ", " << m.WY << "], \"mfma_tiles_per_wave\": [" << m.TX << ", " << m.TY << "], "
      << "\"mfma\": \"" << names[m.MI] << "\", \"split_k\": " << m.SK << ", \"split_k_outermost\": " << m.SKO << ", \"min_waves_per_simd\": " << m.MINW << ", \"late_c\": " << m.LATEC << ", \"nontemporal_c\": " << m.NTC << ", \"swapped_roles\": " << m.SWAP << ", \"prefetch_depth\": " << m.PD << ", \"nontemporal_inputs\": " << m.NTO << ", \"stream\": [" << m.STREAM << ", " << m.SPD << "], \"stream_resident\": \"" << (m.SRES ? "y" : "x") << "\", \"stream_panel_overlap\": " << m.SOV << ", \"stream_c_distance\": " << m.SCD << ", \"stream_interleaved_runs\": " << m.SIL << ", \"tile_order_c_memory\": " << m.TORD << ", \"early_slices\": " << m.ESL << ", \"one_block_ragged\": " << m.OKP << ", \"dynamic_lds_stages\": " << m.DBUF << ", \"vector_slice_loads\": " << m.VL << ", \"c_through_lds\": " << m.CLDS << ", \"repack\": [" << m.RPX << ", " << m.RPY << "], \"threads\": " << 64 * m.WX * m.WY << ", "
      << "\"lds_layout\": [" << m.layx << ", " << m.layy << "], \"lds_ld\": [" << m.ldx << ", " << m.ldy << "], \"lds_bytes\": " << m.lds_bytes << ", "
      << "\"model\": {\"blocks\": " << m.n_blocks << ", \"k_steps\": " << m.steps_main_loop << ", \"blocks_per_cu\": " << m.blocks_per_cu
      << ", \"t_hbm_us\": " << m.t_hbm * 1e6 << ", \"t_l2_us\": " << m.t_l2 * 1e6 << ", \"t_mfma_us\": " << m.t_mfma * 1e6
      << ", \"t_lds_us\": " << m.t_lds * 1e6 << ", \"tail_eff\": " << m.tail_eff << ", \"cost_us\": " << m.cost * 1e6 << "}, "
      << "\"spec\": \"" << m.spec() << "\"}";
    return o.str();
}

}  // namespace cogent
