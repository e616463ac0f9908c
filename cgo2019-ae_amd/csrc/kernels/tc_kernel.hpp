// Device-side building blocks of the gfx950 tensor-contraction engine.
//
// The emitter writes, per contraction expression, a small configuration struct
// (`Cfg`) and instantiates the templates below with it.  They take the place of
// the CUDA kernel text the reference generator writes out
// (cogent/src/codes/kernels/tc_code_kernel.py:20-135: shared-memory slices of
// both inputs, a per-thread register tile, a K loop of {load, sync, outer
// product, sync}, then the store), re-designed for CDNA4:
//
//   * one wavefront = 64 lanes; a block is WY x WX wavefronts;
//   * the inner product runs on the matrix cores (v_mfma_f64_16x16x4_f64,
//     v_mfma_f32_16x16x4_f32 or v_mfma_f32_32x32x2_f32); every wavefront owns
//     TY x TX accumulator tiles;
//   * the output tile is READ into the accumulators before the K loop, so the
//     kernel computes C <- C +/- sum(A*B) (the reference kernel overwrites C,
//     cogent/src/codes/kernels/tc_code_kernel_store_output.py:78) and the C
//     loads overlap the staging of the first input slices;
//   * both input slices are staged global -> registers -> LDS in the operand's
//     own memory order (coalesced along its fastest index) and scattered into
//     an LDS layout chosen per operand so that MFMA operand reads are
//     bank-conflict free:
//        LAY 0  "k-major"  addr = k * LD + e   (operand fastest index external)
//        LAY 1  "e-major"  addr = e * LD + k   (operand fastest index contracted)
//
// Naming: the "X side" is the input that holds the output's fastest index; its
// external indices run along the MFMA column (lane % 16) so that stores to C
// are contiguous.  The "Y side" is the other input.  Composite coordinates:
// x = x0 + tx0*(x1 + tx1*(...)) over the X-side external tiles, likewise y, k.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace cogent {

constexpr int TC_MAXI = 12;   // most distinct indices in one expression

// Run-time geometry handed to every kernel (by value, in kernel-argument space).
struct TcDims {
    int ext[TC_MAXI];    // extent of every index id
    int nblk[TC_MAXI];   // tiles along the index (grid factor for externals, K blocks for contracted)
    int sC[TC_MAXI];     // element stride inside C  (0 when the index is absent)
    int sX[TC_MAXI];     // element stride inside the X-side operand
    int sY[TC_MAXI];     // element stride inside the Y-side operand
    int nkb;             // number of K blocks = product of nblk over contracted ids
    unsigned nblocks;    // number of output tiles = grid size
    unsigned nxt;        // number of tiles along the composite X coordinate (product of nblk over X ids)
};

typedef double v4f64 __attribute__((ext_vector_type(4)));
typedef float  v4f32 __attribute__((ext_vector_type(4)));
typedef float  v16f32 __attribute__((ext_vector_type(16)));

// Matrix-instruction traits.  Lane l of a wavefront supplies A[i = l % MT][k = l / MT]
// and B[k = l / MT][j = l % MT]; row() gives the D row held in accumulator register r.
template <int MI> struct Mfma;
template <> struct Mfma<0> {   // v_mfma_f64_16x16x4_f64
    typedef double T; typedef v4f64 Acc;
    static constexpr int MT = 16, KSTEP = 4, NREG = 4;
    __device__ static __forceinline__ int row(int r, int lane) { return 4 * r + lane / 16; }
    __device__ static __forceinline__ Acc mma(T a, T b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
};
template <> struct Mfma<1> {   // v_mfma_f32_16x16x4_f32
    typedef float T; typedef v4f32 Acc;
    static constexpr int MT = 16, KSTEP = 4, NREG = 4;
    __device__ static __forceinline__ int row(int r, int lane) { return 4 * (lane / 16) + r; }
    __device__ static __forceinline__ Acc mma(T a, T b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
};
template <> struct Mfma<2> {   // v_mfma_f32_32x32x2_f32
    typedef float T; typedef v16f32 Acc;
    static constexpr int MT = 32, KSTEP = 2, NREG = 16;
    __device__ static __forceinline__ int row(int r, int lane) { return 8 * (r / 4) + 4 * (lane / 32) + (r % 4); }
    __device__ static __forceinline__ Acc mma(T a, T b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
};

// View of one input operand of a Cfg (SIDE 0 = X, 1 = Y).
template <class Cfg, int SIDE> struct Operand;
template <class Cfg> struct Operand<Cfg, 0> {
    static constexpr int R = Cfg::XR, LAY = Cfg::LAYX, LD = Cfg::LDX, BE = Cfg::BX, BEP = Cfg::BXP;
    static constexpr bool NTL = (Cfg::NTO & 1) != 0;      // this input is read once: non-temporal loads
    static constexpr int VW = Cfg::VWX;                   // elements per global load when the slice's fastest run allows (1: scalar)
    __device__ static __forceinline__ constexpr int id(int j)   { return Cfg::xo_id(j); }
    __device__ static __forceinline__ constexpr int tile(int j) { return Cfg::xo_tile(j); }
    __device__ static __forceinline__ constexpr int isk(int j)  { return Cfg::xo_isk(j); }
    __device__ static __forceinline__ constexpr int mul(int j)  { return Cfg::xo_mul(j); }
    __device__ static __forceinline__ int stride(const TcDims& d, int id) { return d.sX[id]; }
};
template <class Cfg> struct Operand<Cfg, 1> {
    static constexpr int R = Cfg::YR, LAY = Cfg::LAYY, LD = Cfg::LDY, BE = Cfg::BY, BEP = Cfg::BYP;
    static constexpr bool NTL = (Cfg::NTO & 2) != 0;
    static constexpr int VW = Cfg::VWY;
    __device__ static __forceinline__ constexpr int id(int j)   { return Cfg::yo_id(j); }
    __device__ static __forceinline__ constexpr int tile(int j) { return Cfg::yo_tile(j); }
    __device__ static __forceinline__ constexpr int isk(int j)  { return Cfg::yo_isk(j); }
    __device__ static __forceinline__ constexpr int mul(int j)  { return Cfg::yo_mul(j); }
    __device__ static __forceinline__ int stride(const TcDims& d, int id) { return d.sY[id]; }
};

// A value that is the same in every lane, moved into scalar registers.  64-bit products of
// uniform values are computed on the vector ALU (the scalar ALU has no 64-bit multiply) and would
// otherwise stay in vector registers, which turns every address built from them into vector adds.
__device__ __forceinline__ int64_t uniform64(int64_t v)
{
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)(uint64_t)v);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// C is read once and written once.  When every row segment a wavefront touches is a whole, aligned
// 128-byte line (NT), the accesses are marked non-temporal so that C does not displace the operand
// panels in L2 / Infinity Cache (measured +8-12% on the fp64 6-D contractions); with partial lines
// (fp32 rows of 64 or 96 bytes) the same hint defeats write combining and costs 35%, so it is off.
template <bool NT, class T> __device__ __forceinline__ T c_load(const T* p) { return NT ? __builtin_nontemporal_load(p) : *p; }
template <bool NT, class T> __device__ __forceinline__ void c_store(T v, T* p) { if (NT) __builtin_nontemporal_store(v, p); else *p = v; }

template <class Op, int BKP>
constexpr int lds_elems() { return Op::LAY == 0 ? BKP * Op::LD : Op::BEP * Op::LD; }

template <class Op>
__device__ __forceinline__ int lds_addr(int k, int e) { return Op::LAY == 0 ? k * Op::LD + e : e * Op::LD + k; }

// Element q of an operand's slice, enumerated in the operand's memory order
// (fastest index first, each index restricted to its tile): gives the element
// offset relative to the slice origin, the LDS address and whether the element
// lies inside the tensor.  rem[id] = extent[id] - tile origin along id.
template <class Op, bool EXT_FULL, bool INT_FULL>
__device__ __forceinline__ void slice_element(unsigned q, const TcDims& d, const int* rem,
                                              unsigned& goff, int& loff, bool& valid)
{
    int e = 0, k = 0;
    goff = 0u;
    valid = true;
#pragma unroll
    for (int j = 0; j < Op::R; j++) {
        const unsigned t = (unsigned)Op::tile(j);
        const int i = (int)(q % t);
        q /= t;
        const int id = Op::id(j);
        goff += (unsigned)i * (unsigned)Op::stride(d, id);
        if (Op::isk(j)) {
            k += i * Op::mul(j);
            if (!INT_FULL) valid = valid && (i < rem[id]);
        } else {
            e += i * Op::mul(j);
            if (!EXT_FULL) valid = valid && (i < rem[id]);
        }
    }
    loff = lds_addr<Op>(k, e);
}

// Vector width of an operand's slice loads in a kernel variant: Op::VW consecutive elements of the operand's
// fastest index per lane (one 8- or 16-byte load) when that index's tile is a multiple of it and the tiles of
// its class are full in this variant (so that a vector never straddles the edge of the tensor); 1 otherwise.
template <class Op, bool EXT_FULL, bool INT_FULL>
constexpr int slice_vw() { return (Op::VW > 1 && Op::tile(0) % Op::VW == 0 && (Op::isk(0) ? INT_FULL : EXT_FULL)) ? Op::VW : 1; }
// Registers per lane that hold its share of a slice
template <class Cfg, class Op, int V>
constexpr int slice_slots() { return V * ((Cfg::BK * Op::BE / V + Cfg::NT - 1) / Cfg::NT); }

template <class Cfg, class Op, bool EXT_FULL, bool INT_FULL, int SLOTS>
__device__ __forceinline__ void slice_load(typename Cfg::T (&reg)[SLOTS], const typename Cfg::T* __restrict__ src,
                                           const TcDims& d, const int* rem, int tid)
{
    typedef typename Cfg::T T;
    constexpr int V = slice_vw<Op, EXT_FULL, INT_FULL>();
    static_assert(SLOTS == slice_slots<Cfg, Op, V>(), "register count of a slice does not match its vector width");
    // element alignment only: the vector may start at any element of the tensor
    typedef T TVec __attribute__((ext_vector_type(V), aligned(sizeof(T))));
    constexpr unsigned E = (unsigned)(Cfg::BK * Op::BE);
#pragma unroll
    for (int s = 0; s < SLOTS / V; s++) {
        const unsigned q = ((unsigned)tid + (unsigned)s * Cfg::NT) * V;
        unsigned goff; int loff; bool valid;
        slice_element<Op, EXT_FULL, INT_FULL>(q, d, rem, goff, loff, valid);
        const bool take = ((E / V) % Cfg::NT == 0 || q < E) && valid;
        if constexpr (V == 1) {
            T v = (T)0;
            if (take) v = c_load<Op::NTL>((const T*)((const char*)src + goff * (unsigned)sizeof(T)));
            reg[s] = v;
        } else {
            TVec v;
#pragma unroll
            for (int e = 0; e < V; e++) v[e] = (T)0;
            if (take) {
                const TVec* p = (const TVec*)((const char*)src + goff * (unsigned)sizeof(T));
                v = Op::NTL ? __builtin_nontemporal_load(p) : *p;
            }
#pragma unroll
            for (int e = 0; e < V; e++) reg[s * V + e] = v[e];
        }
    }
}

// LDS distance between two elements that are neighbours along the operand's fastest index
template <class Op>
constexpr int slice_lds_step() { return Op::isk(0) ? (Op::LAY == 0 ? Op::mul(0) * Op::LD : Op::mul(0)) : (Op::LAY == 0 ? Op::mul(0) : Op::mul(0) * Op::LD); }

template <class Cfg, class Op, bool NEGATE, int V = 1, int SLOTS>
__device__ __forceinline__ void slice_store(const typename Cfg::T (&reg)[SLOTS], typename Cfg::T* lds,
                                            const TcDims& d, int tid)
{
    constexpr unsigned E = (unsigned)(Cfg::BK * Op::BE);
    constexpr int STEP = slice_lds_step<Op>();
#pragma unroll
    for (int s = 0; s < SLOTS / V; s++) {
        const unsigned q = ((unsigned)tid + (unsigned)s * Cfg::NT) * V;
        unsigned goff; int loff; bool valid;
        slice_element<Op, true, true>(q, d, nullptr, goff, loff, valid);
        if ((E / V) % Cfg::NT == 0 || q < E) {
#pragma unroll
            for (int e = 0; e < V; e++) lds[loff + e * STEP] = NEGATE ? -reg[s * V + e] : reg[s * V + e];
        }
    }
}

// Element offsets, relative to the block's C tile origin, of the accumulator elements a lane holds.
// Normal roles (X along MFMA columns): cx[tj][0] for the lane's column in tile column tj, cy[ti][r] for
// the row of register r in tile row ti.  Swapped roles (SWP, X along MFMA rows): cx[tj][r], cy[ti][0].
// -1 marks positions outside the tensor (ragged tiles, padding).
// LOCAL: the offsets are positions in a dense copy of the tile alone, kept in C's index order (the
// layout of the tile when it is staged through LDS), instead of offsets into the tensor.
template <class Cfg, bool EXT_FULL, bool SWP, bool LOCAL>
__device__ __forceinline__ void c_tile_offsets(int lane, int wx, int wy, const int* rem, const TcDims& d,
                                               int (&cx)[Cfg::TX][SWP ? Mfma<Cfg::MI>::NREG : 1],
                                               int (&cy)[Cfg::TY][SWP ? 1 : Mfma<Cfg::MI>::NREG])
{
    typedef Mfma<Cfg::MI> MM;
    constexpr int MT = MM::MT, NREG = MM::NREG, TX = Cfg::TX, TY = Cfg::TY;
#pragma unroll
    for (int tj = 0; tj < TX; tj++) {
#pragma unroll
        for (int r = 0; r < (SWP ? NREG : 1); r++) {
            const int x = (wx * TX + tj) * MT + (SWP ? MM::row(r, lane) : lane % MT);
            unsigned q = (unsigned)x;
            int off = 0; bool ok = (Cfg::BXP == Cfg::BX) || (x < Cfg::BX);
#pragma unroll
            for (int i = 0; i < Cfg::NX; i++) {
                const int c = (int)(q % (unsigned)Cfg::x_tile(i));
                q /= (unsigned)Cfg::x_tile(i);
                off += c * (LOCAL ? Cfg::cl_stride(Cfg::x_id(i)) : d.sC[Cfg::x_id(i)]);
                if (!EXT_FULL) ok = ok && (c < rem[Cfg::x_id(i)]);
            }
            cx[tj][r] = ok ? off : -1;
        }
    }
#pragma unroll
    for (int ti = 0; ti < TY; ti++) {
#pragma unroll
        for (int r = 0; r < (SWP ? 1 : NREG); r++) {
            const int y = (wy * TY + ti) * MT + (SWP ? lane % MT : MM::row(r, lane));
            unsigned q = (unsigned)y;
            int off = 0; bool ok = (Cfg::BYP == Cfg::BY) || (y < Cfg::BY);
#pragma unroll
            for (int i = 0; i < Cfg::NY; i++) {
                const int c = (int)(q % (unsigned)Cfg::y_tile(i));
                q /= (unsigned)Cfg::y_tile(i);
                off += c * (LOCAL ? Cfg::cl_stride(Cfg::y_id(i)) : d.sC[Cfg::y_id(i)]);
                if (!EXT_FULL) ok = ok && (c < rem[Cfg::y_id(i)]);
            }
            cy[ti][r] = ok ? off : -1;
        }
    }
}

extern __shared__ __attribute__((aligned(16))) unsigned char tc_dynamic_lds[];

// Bytes of dynamic LDS a variant of the contraction kernel needs (0: its buffers are static): with Cfg::DBUF,
// whenever two stages do not fit a static array -- two stages if they fit the CU's 160 KB, else the one.
template <class Cfg, bool ONE_KB>
constexpr size_t tc_mfma_dynamic_lds()
{
    typedef typename Cfg::T T;
    constexpr size_t one = (size_t)(lds_elems<Operand<Cfg, 0>, Cfg::BKP>() + lds_elems<Operand<Cfg, 1>, Cfg::BKP>()) * sizeof(T);
    if (ONE_KB || Cfg::DBUF == 0 || 2 * one <= 65536) return 0;
    return 2 * one <= 160 * 1024 ? 2 * one : one;
}

// The contraction kernel.  EXT_FULL: every external extent is a multiple of its
// tile and the tile products need no padding; INT_FULL: the same for the
// contracted indices.  (The reference picks among four kernels by the same two
// tests, cogent/src/codes/kernels/tc_interface.py:1150-1175.)
//
// ONE_KB: the whole contracted range fits one K block (every contracted extent <= its tile), the
// shape of the HBM-bound many-index contractions.  The K loop, its odometer and the register
// prefetch of the next slices disappear, which frees registers for more resident wavefronts.
//
// SWP (fp32 only): the X side runs along the MFMA ROWS instead of the columns.  In the fp32 MFMA
// layouts a lane holds 4 consecutive rows per register group, so with C's fastest index on the rows
// each lane owns 16 contiguous bytes of C and the tile is read and written with one 128-bit access
// per group -- a wavefront covers a contiguous kilobyte per instruction where the column layout
// gives 64-byte pieces.  The launcher uses it when the fastest extent is a multiple of 4 and C is
// 16-byte aligned.
// f(integral_constant<int, 0>), .., f(integral_constant<int, N - 1>), unconditionally
template <int N, int I = 0, class F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) { f(std::integral_constant<int, I>()); static_for<N, I + 1>(f); }
}
// f(0), f(1), .. while the index is below both N and n: every call sits inside the branch of the one
// before it, so control reaches call I only from call I - 1
template <int N, int I = 0, class F>
__device__ __forceinline__ void static_chain(int n, F&& f)
{
    if constexpr (I < N) { if (I < n) { f(std::integral_constant<int, I>()); static_chain<N, I + 1>(n, f); } }
}

template <class Cfg, bool EXT_FULL, bool INT_FULL, bool ONE_KB, bool SWP>
__global__ __launch_bounds__(Cfg::NT, Cfg::MINW)     // MINW: wavefronts per SIMD the register allocator must leave room for
void tc_mfma_kernel(typename Cfg::T* __restrict__ C, const typename Cfg::T* __restrict__ X,
                    const typename Cfg::T* __restrict__ Y, const TcDims d)
{
    typedef typename Cfg::T T;
    typedef Mfma<Cfg::MI> MM;
    typedef typename MM::Acc Acc;
    typedef Operand<Cfg, 0> OX;
    typedef Operand<Cfg, 1> OY;
    constexpr int MT = MM::MT, NREG = MM::NREG, KSTEP = MM::KSTEP;
    constexpr int TX = Cfg::TX, TY = Cfg::TY, NT = Cfg::NT;
    constexpr int VX = slice_vw<OX, EXT_FULL, INT_FULL>(), VY = slice_vw<OY, EXT_FULL, INT_FULL>();
    constexpr int SLOTS_X = slice_slots<Cfg, OX, VX>();
    constexpr int SLOTS_Y = slice_slots<Cfg, OY, VY>();
    constexpr int LDS_X = lds_elems<OX, Cfg::BKP>();
    constexpr int LDS_Y = lds_elems<OY, Cfg::BKP>();
    constexpr bool PADDED = (Cfg::BKP != Cfg::BK) || (Cfg::BXP != Cfg::BX) || (Cfg::BYP != Cfg::BY);
    // two LDS stages when there is a K loop and both fit the static 64 KB: the next slices are
    // written while other wavefronts still read the current ones, one barrier per K block
    // Cfg::DBUF: the two stages live in dynamic LDS, which can be larger than the 64 KB a static array may have
    // (large tiles with deep K blocks, one workgroup per CU anyway): the launcher passes the size.
    // With Cfg::DBUF a single stage of more than 64 KB (a deep K block of a wide tile) is allowed too, up to the
    // CU's 160 KB; two stages are used whenever both fit.
    constexpr int ONE_STAGE = (LDS_X + LDS_Y) * (int)sizeof(T);
    constexpr bool BIG = tc_mfma_dynamic_lds<Cfg, ONE_KB>() > 0;
    constexpr int NBUF = (!ONE_KB && (BIG ? 2 * ONE_STAGE <= 160 * 1024 : 2 * ONE_STAGE <= 65536)) ? 2 : 1;

    // C tile through LDS (CL): the tile is read from and written to global memory in C's own memory
    // order, 16 bytes per lane and whole lines per wavefront whatever the MFMA lane layout is, and
    // changes hands with the accumulators through a dense copy in LDS that shares the operand buffers.
    // Full tiles without split K only; the other variants of the same object use the direct path.
    constexpr int SK0 = ONE_KB ? 1 : Cfg::SK;
    constexpr bool CL = (Cfg::CLDS != 0) && EXT_FULL && SK0 == 1 && (ONE_KB || Cfg::LATEC == 0) && !BIG;
    constexpr int TILE_VOL = Cfg::BX * Cfg::BY;
    constexpr int LDS_OPS = NBUF * (LDS_X + LDS_Y);
    constexpr int LDS_ALL = (CL && TILE_VOL > LDS_OPS) ? TILE_VOL : LDS_OPS;
    __shared__ __attribute__((aligned(16))) T lds_static[BIG ? 4 : LDS_ALL];
    T* const lds_all = BIG ? (T*)tc_dynamic_lds : lds_static;
    T* const lds_x_all = lds_all;
    T* const lds_y_all = lds_all + NBUF * LDS_X;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wx = wave % Cfg::WX;
    const int wy = wave / Cfg::WX;

    // ---- which output tile: X-side tiles vary fastest over the grid
    constexpr int SK = ONE_KB ? 1 : Cfg::SK;
    unsigned ks = 0;
    int rem[Cfg::NIDX];
    int64_t baseC = 0, baseX = 0, baseY = 0;
    {
        if constexpr (Cfg::TORD != 0) {
            // Tile order = the order of the tile origins in C's memory, workgroup b = blockIdx.x: the workgroups in
            // flight chip-wide (consecutive ones go to different XCDs) then cover ONE compact window of C that moves
            // linearly through the tensor, the access pattern of a plain streaming kernel.  For outputs much larger
            // than the inputs (which then sit in every XCD's L2 anyway) this is what the memory system likes best.
            unsigned b = blockIdx.x;
            if (SK > 1) {
                if (Cfg::SKO != 0) { const unsigned nt = d.nblocks / (unsigned)SK; ks = b / nt; b %= nt; }
                else               { ks = b % (unsigned)SK; b /= (unsigned)SK; }
            }
#pragma unroll
            for (int j = 0; j < Cfg::CR; j++) {
                const int id = Cfg::c_id(j);
                const unsigned nb = (unsigned)d.nblk[id];
                const int o = (int)(b % nb) * Cfg::c_tile(j);
                b /= nb;
                rem[id] = d.ext[id] - o;
                baseC += (int64_t)o * d.sC[id];
                baseX += (int64_t)o * d.sX[id];         // (the stride is zero in the operand that does not hold the index)
                baseY += (int64_t)o * d.sY[id];
            }
        } else {
            // Workgroups are handed to the 8 XCDs round-robin and every XCD has its own L2: give XCD x
            // a CONTIGUOUS range of output tiles, so that the tiles resident on one XCD share their
            // operand panels in that L2.
            unsigned b;
            {
                const unsigned n = d.nblocks, xcd = blockIdx.x % 8u, idx = blockIdx.x / 8u;
                const unsigned q = n / 8u, r = n % 8u;
                b = xcd * q + (xcd < r ? xcd : r) + idx;
            }
            // split K: SK consecutive workgroups share one output tile, each takes a share of the K blocks.
            // SKO: the shares are the outermost level instead, so an XCD's range holds ALL tiles of a few
            // shares and the operand slices those tiles have in common meet in that XCD's L2.
            if (SK > 1) {
                if (Cfg::SKO != 0) { const unsigned nt = d.nblocks / (unsigned)SK; ks = b / nt; b %= nt; }
                else               { ks = b % (unsigned)SK; b /= (unsigned)SK; }
            }
            // Within that range walk the tile grid in bands of TILE_GROUP X-tiles (X fastest inside a
            // band, then Y): the ~100 tiles in flight on an XCD then touch a dozen X panels and a dozen
            // Y panels instead of every X panel, and the panels stay in the 4 MB L2 while C streams by.
            {
                constexpr unsigned GX = 8;
                const unsigned nyt = (d.nblocks / (unsigned)SK) / d.nxt;
                const unsigned G = GX * nyt;
                const unsigned g = b / G, r = b % G;
                const unsigned first = g * GX;
                const unsigned gx = (d.nxt - first) < GX ? (d.nxt - first) : GX;
                b = (first + r % gx) + (r / gx) * d.nxt;
            }
#pragma unroll
            for (int i = 0; i < Cfg::NX; i++) {
                const int id = Cfg::x_id(i);
                const unsigned nb = (unsigned)d.nblk[id];
                const int o = (int)(b % nb) * Cfg::x_tile(i);
                b /= nb;
                rem[id] = d.ext[id] - o;
                baseC += (int64_t)o * d.sC[id];
                baseX += (int64_t)o * d.sX[id];
            }
#pragma unroll
            for (int i = 0; i < Cfg::NY; i++) {
                const int id = Cfg::y_id(i);
                const unsigned nb = (unsigned)d.nblk[id];
                const int o = (int)(b % nb) * Cfg::y_tile(i);
                b /= nb;
                rem[id] = d.ext[id] - o;
                baseC += (int64_t)o * d.sC[id];
                baseY += (int64_t)o * d.sY[id];
            }
        }
#pragma unroll
        for (int i = 0; i < Cfg::NK; i++) rem[Cfg::k_id(i)] = d.ext[Cfg::k_id(i)];
    }
    T* __restrict__ Cb = C + uniform64(baseC);
    const T* __restrict__ Xb = X + uniform64(baseX);
    const T* __restrict__ Yb = Y + uniform64(baseY);

    // ---- where this lane's accumulator elements live in C (-1: outside)
    int cx[TX][SWP ? NREG : 1];
    int cy[TY][SWP ? 1 : NREG];
    c_tile_offsets<Cfg, EXT_FULL, SWP, CL>(lane, wx, wy, rem, d, cx, cy);
    // offset of accumulator element (ti, tj, r) (CL: its place in the LDS copy) and whether it is inside the tensor
    auto c_off = [&](int ti, int tj, int r) -> int { return cx[tj][SWP ? r : 0] + cy[ti][SWP ? 0 : r]; };
    auto c_ok = [&](int ti, int tj, int r) -> bool {
        return (EXT_FULL && !PADDED) || (cx[tj][SWP ? r : 0] >= 0 && cy[ti][SWP ? 0 : r] >= 0);
    };
    typedef T T4 __attribute__((ext_vector_type(4)));
    constexpr bool VEC4 = SWP;      // 4 consecutive registers = 4 consecutive elements of C's fastest index

    // ---- accumulators start from the C tile: C_in + sum, summed in k order.
    // LATE_C: they start from zero instead and the C tile is loaded into registers of its own during
    // the first trip of the K loop, AFTER that trip's prefetch was issued (loads return in order, so
    // the wait for the prefetch does not wait for C): the block starts contracting one L2 latency
    // after launch instead of one HBM latency, and the C read hides behind its own K loop.
    constexpr bool LATE_C = !ONE_KB && SK == 1 && (Cfg::LATEC != 0);
    Acc cpre[LATE_C ? TY : 1][LATE_C ? TX : 1];
    Acc acc[TY][TX];
    // the tile in C's memory order: element q of it, as an offset from the tile origin
    constexpr int CV = 16 / (int)sizeof(T);
    typedef T TV __attribute__((ext_vector_type(CV)));
    // the same vector in global memory: element alignment only, so that C may start at any element of a larger
    // buffer (the LDS copy is always 16-byte aligned)
    typedef T TVG __attribute__((ext_vector_type(CV), aligned(sizeof(T))));
    constexpr int NVEC = CL ? (TILE_VOL / CV + NT - 1) / NT : 1;
    auto c_linear = [&](unsigned q) -> unsigned {
        unsigned off = 0;
#pragma unroll
        for (int j = 0; j < Cfg::CR; j++) {
            const unsigned t = (unsigned)Cfg::c_tile(j);
            off += (q % t) * (unsigned)d.sC[Cfg::c_id(j)];
            q /= t;
        }
        return off;
    };
    // Slices of the first K block.  Cfg::ESL with the C tile through LDS: they are requested BEFORE the tile is staged
    // (two barriers that no load may cross stand between the staging and the K loop: requested behind them, the
    // slices' round trip to L2 follows the tile's round trip to HBM instead of overlapping it).  The slices then sit
    // in registers through the staging, which can cost a resident wavefront: measured -11 % on a 96x64 fp32 tile of a
    // 6-D shape, +3 to +7 % on three other tiles, hence an option.  CL implies no split K, so the first block is at
    // the origin of both slices.
    constexpr int PD = ONE_KB ? 1 : Cfg::PD;
    T rx[PD][SLOTS_X], ry[PD][SLOTS_Y];
    constexpr bool EARLY = CL && (Cfg::ESL != 0);
    if (EARLY) {
        slice_load<Cfg, OX, EXT_FULL, INT_FULL>(rx[0], Xb, d, rem, tid);
        slice_load<Cfg, OY, EXT_FULL, INT_FULL>(ry[0], Yb, d, rem, tid);
    }
    if (CL) {
        TV cv[NVEC];
#pragma unroll
        for (int i = 0; i < NVEC; i++) {
            const unsigned q = (unsigned)(tid + i * NT) * CV;
            if (TILE_VOL % (NT * CV) == 0 || q < (unsigned)TILE_VOL)
            {
                // (not through c_load<>: template deduction would drop the reduced alignment of TVG)
                const TVG* src = (const TVG*)(Cb + c_linear(q));
                if ((Cfg::NTC & 1) != 0) cv[i] = __builtin_nontemporal_load(src); else cv[i] = *src;
            }
        }
#pragma unroll
        for (int i = 0; i < NVEC; i++) {
            const unsigned q = (unsigned)(tid + i * NT) * CV;
            if (TILE_VOL % (NT * CV) == 0 || q < (unsigned)TILE_VOL) *(TV*)&lds_all[q] = cv[i];
        }
        __syncthreads();
    }
#pragma unroll
    for (int ti = 0; ti < TY; ti++)
#pragma unroll
        for (int tj = 0; tj < TX; tj++) {
            if (VEC4) {
#pragma unroll
                for (int g = 0; g < NREG / 4; g++) {
                    T4 v = {(T)0, (T)0, (T)0, (T)0};
                    if (SK == 1 && !LATE_C && c_ok(ti, tj, 4 * g)) {
                        if (CL) v = *(const T4*)&lds_all[c_off(ti, tj, 4 * g)];
                        else v = c_load<(Cfg::NTC & 1) != 0>((const T4*)((const char*)Cb + (unsigned)c_off(ti, tj, 4 * g) * (unsigned)sizeof(T)));
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[ti][tj][4 * g + e] = v[e];
                }
            } else {
#pragma unroll
                for (int r = 0; r < NREG; r++) {
                    T v = (T)0;
                    if (SK == 1 && !LATE_C && c_ok(ti, tj, r)) {
                        if (CL) v = lds_all[c_off(ti, tj, r)];
                        else v = c_load<(Cfg::NTC & 1) != 0>((const T*)((const char*)Cb + (unsigned)c_off(ti, tj, r) * (unsigned)sizeof(T)));
                    }
                    acc[ti][tj][r] = v;
                }
            }
        }
    if (CL) __syncthreads();        // the copy has been read: the operand slices may take its place

    // ---- padding rows/columns of the LDS slices are never written by the staging: clear once
    if (PADDED) {
        for (int i = tid; i < NBUF * LDS_X; i += NT) lds_x_all[i] = (T)0;
        for (int i = tid; i < NBUF * LDS_Y; i += NT) lds_y_all[i] = (T)0;
        __syncthreads();
    }

    // ---- K loop
    int kbc[Cfg::NK > 0 ? Cfg::NK : 1];
#pragma unroll
    for (int i = 0; i < Cfg::NK; i++) kbc[i] = 0;
    // this workgroup's share of the K blocks: [kb0, kb0 + nkb)
    int kb0 = 0, nkb = ONE_KB ? 1 : d.nkb;
    int64_t kx0 = 0, ky0 = 0;
    if (SK > 1) {
        kb0 = (int)(((int64_t)ks * d.nkb) / SK);
        nkb = (int)(((int64_t)(ks + 1) * d.nkb) / SK) - kb0;
        if (nkb <= 0) return;                      // more splits than K blocks: uniform for the block
        unsigned q = (unsigned)kb0;
#pragma unroll
        for (int i = 0; i < Cfg::NK; i++) {
            const int id = Cfg::k_id(i);
            kbc[i] = (int)(q % (unsigned)d.nblk[id]);
            q /= (unsigned)d.nblk[id];
            const int o = kbc[i] * Cfg::k_tile(i);
            rem[id] = d.ext[id] - o;
            kx0 += (int64_t)o * d.sX[id];
            ky0 += (int64_t)o * d.sY[id];
        }
    }

    // Prefetch depth PD: the slices of K block kb + PD are requested while block kb is contracted,
    // each depth in registers of its own (stage kb % PD, a compile-time index in every copy of the
    // trip below).  One trip of MFMA work is a fraction of a microsecond; a slice gathered through a
    // busy L2 takes several times that, so one stage of look-ahead leaves the loop waiting on loads.
    int64_t kxh = kx0, kyh = ky0;                  // slice origin of the newest K block requested
    int head = 0;                                  // ... and its number within this workgroup's share
    // Move the head one K block on (first composite K index fastest) -- unless it is at the last one:
    // then the same block is requested again and never used.  Every trip thus issues the same loads
    // whatever the trip count, which keeps the outstanding-load count known at compile time: the wait
    // before a stage is stored to LDS then leaves the PD - 1 newer stages in flight.
    auto advance_head = [&]() {
        if (head + 1 < nkb) {
            head++;
            kxh = 0; kyh = 0;
            bool carry = true;
#pragma unroll
            for (int i = 0; i < Cfg::NK; i++) {
                const int id = Cfg::k_id(i);
                if (carry) { kbc[i]++; carry = false; if (kbc[i] == d.nblk[id]) { kbc[i] = 0; carry = true; } }
                const int o = kbc[i] * Cfg::k_tile(i);
                rem[id] = d.ext[id] - o;
                kxh += (int64_t)o * d.sX[id];
                kyh += (int64_t)o * d.sY[id];
            }
        }
    };
    if (!EARLY) {
        slice_load<Cfg, OX, EXT_FULL, INT_FULL>(rx[0], Xb + uniform64(kxh), d, rem, tid);
        slice_load<Cfg, OY, EXT_FULL, INT_FULL>(ry[0], Yb + uniform64(kyh), d, rem, tid);
    }
#pragma unroll
    for (int s = 1; s < PD; s++) {
        advance_head();
        slice_load<Cfg, OX, EXT_FULL, INT_FULL>(rx[s], Xb + uniform64(kxh), d, rem, tid);
        slice_load<Cfg, OY, EXT_FULL, INT_FULL>(ry[s], Yb + uniform64(kyh), d, rem, tid);
    }

    if (!ONE_KB) {
        // Drain the C-tile and first-slice loads BEFORE the K loop.  Otherwise the compiler has to
        // assume, on every trip, that the accumulators may still be in flight, and its wait for
        // them (an in-order counter) also waits for the prefetch issued at the top of the trip,
        // which takes the prefetch's whole latency out of hiding.  s_waitcnt vmcnt(0).
        __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    if (NBUF == 2) {
        slice_store<Cfg, OX, false, VX>(rx[0], lds_x_all, d, tid);
        slice_store<Cfg, OY, (Cfg::SIGN < 0), VY>(ry[0], lds_y_all, d, tid);
        __syncthreads();
    }
    // One trip: contract K block kb, whose slices are (NBUF == 2) already in LDS or (NBUF == 1) in
    // stage S = kb % PD.
    auto k_block = [&](const int kb, auto stage, auto first_trip) {
        constexpr int S = decltype(stage)::value, SN = (S + 1) % PD;
        T* lds_x = lds_x_all + (NBUF == 2 ? (kb & 1) * LDS_X : 0);
        T* lds_y = lds_y_all + (NBUF == 2 ? (kb & 1) * LDS_Y : 0);
        if (NBUF == 1) {
            if (!ONE_KB) __syncthreads();      // previous slices fully consumed
            slice_store<Cfg, OX, false, VX>(rx[S], lds_x, d, tid);
            slice_store<Cfg, OY, (Cfg::SIGN < 0), VY>(ry[S], lds_y, d, tid);
            __syncthreads();
        }

        // with one stage nothing newer is in flight, so the last trip can simply skip the request
        const bool more = PD > 1 || kb + 1 < nkb;
        if (!ONE_KB && more) {
            // stage S is free (its slices are in LDS): request K block kb + PD into it
            advance_head();
            slice_load<Cfg, OX, EXT_FULL, INT_FULL>(rx[S], Xb + uniform64(kxh), d, rem, tid);
            slice_load<Cfg, OY, EXT_FULL, INT_FULL>(ry[S], Yb + uniform64(kyh), d, rem, tid);
        }
        if (LATE_C && decltype(first_trip)::value) {
#pragma unroll
            for (int ti = 0; ti < TY; ti++)
#pragma unroll
                for (int tj = 0; tj < TX; tj++)
#pragma unroll
                    for (int r = 0; r < NREG; r++) {
                        T v = (T)0;
                        if (c_ok(ti, tj, r))
                            v = c_load<(Cfg::NTC & 1) != 0>((const T*)((const char*)Cb + (unsigned)c_off(ti, tj, r) * (unsigned)sizeof(T)));
                        cpre[LATE_C ? ti : 0][LATE_C ? tj : 0][r] = v;
                    }
        }

#pragma unroll
        for (int k4 = 0; k4 < Cfg::BKP / KSTEP; k4++) {
            const int kk = k4 * KSTEP + lane / MT;
            T a[TY], b[TX];
#pragma unroll
            for (int ti = 0; ti < TY; ti++) a[ti] = lds_y[lds_addr<OY>(kk, (wy * TY + ti) * MT + lane % MT)];
#pragma unroll
            for (int tj = 0; tj < TX; tj++) b[tj] = lds_x[lds_addr<OX>(kk, (wx * TX + tj) * MT + lane % MT)];
#pragma unroll
            for (int ti = 0; ti < TY; ti++)
#pragma unroll
                for (int tj = 0; tj < TX; tj++) acc[ti][tj] = SWP ? MM::mma(b[tj], a[ti], acc[ti][tj]) : MM::mma(a[ti], b[tj], acc[ti][tj]);
        }

        if (NBUF == 2) {
            // the slices of K block kb + 1 go to the other LDS buffer (after the last block: the
            // unused repeat of it, harmless)
            if (more) {
                slice_store<Cfg, OX, false, VX>(rx[SN], lds_x_all + ((kb + 1) & 1) * LDS_X, d, tid);
                slice_store<Cfg, OY, (Cfg::SIGN < 0), VY>(ry[SN], lds_y_all + ((kb + 1) & 1) * LDS_Y, d, tid);
            }
            __syncthreads();
        }
    };
    // The first trip is a copy of its own so that what is in flight during it is known exactly; then
    // whole groups of PD trips (stage indices 1, 2, .., 0), then the at most PD - 1 trips left over,
    // each entered only from the one before it so that no two load histories meet.
    k_block(0, std::integral_constant<int, 0>(), std::true_type());
    if (!ONE_KB) {
        int kb = 1;
        for (; kb + PD <= nkb; kb += PD)
            static_for<PD>([&](auto s) { k_block(kb + decltype(s)::value, std::integral_constant<int, (1 + decltype(s)::value) % PD>(), std::false_type()); });
        const int left = nkb - kb;
        static_chain<PD - 1>(left, [&](auto s) { k_block(kb + decltype(s)::value, std::integral_constant<int, (1 + decltype(s)::value) % PD>(), std::false_type()); });
    }

    // ---- write the tile back.  With a K loop the offsets are derived again here from an opaque
    // copy of the lane id instead of being kept in registers across the loop (one register per
    // accumulator element otherwise, which costs a resident wavefront per SIMD).
    if (!ONE_KB) {
        int lane2 = lane;
        asm volatile("" : "+v"(lane2));
        c_tile_offsets<Cfg, EXT_FULL, SWP, CL>(lane2, wx, wy, rem, d, cx, cy);
    }
    if (CL) {
        __syncthreads();            // every wavefront is done with the operand slices
#pragma unroll
        for (int ti = 0; ti < TY; ti++)
#pragma unroll
            for (int tj = 0; tj < TX; tj++) {
                if (VEC4) {
#pragma unroll
                    for (int g = 0; g < NREG / 4; g++)
                        if (c_ok(ti, tj, 4 * g)) {
                            T4 v;
#pragma unroll
                            for (int e = 0; e < 4; e++) v[e] = acc[ti][tj][4 * g + e];
                            *(T4*)&lds_all[c_off(ti, tj, 4 * g)] = v;
                        }
                } else {
#pragma unroll
                    for (int r = 0; r < NREG; r++)
                        if (c_ok(ti, tj, r)) lds_all[c_off(ti, tj, r)] = acc[ti][tj][r];
                }
            }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NVEC; i++) {
            const unsigned q = (unsigned)(tid + i * NT) * CV;
            if (TILE_VOL % (NT * CV) == 0 || q < (unsigned)TILE_VOL)
            {
                TVG* dst = (TVG*)(Cb + c_linear(q));
                const TVG v = *(const TV*)&lds_all[q];
                if ((Cfg::NTC & 2) != 0) __builtin_nontemporal_store(v, dst); else *dst = v;
            }
        }
        return;
    }
#pragma unroll
    for (int ti = 0; ti < TY; ti++)
#pragma unroll
        for (int tj = 0; tj < TX; tj++) {
            if (VEC4 && SK == 1) {
#pragma unroll
                for (int g = 0; g < NREG / 4; g++)
                    if (c_ok(ti, tj, 4 * g)) {
                        T4 v;
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            v[e] = LATE_C ? cpre[LATE_C ? ti : 0][LATE_C ? tj : 0][4 * g + e] + acc[ti][tj][4 * g + e] : acc[ti][tj][4 * g + e];
                        c_store<(Cfg::NTC & 2) != 0>(v, (T4*)((char*)Cb + (unsigned)c_off(ti, tj, 4 * g) * (unsigned)sizeof(T)));
                    }
            } else {
#pragma unroll
                for (int r = 0; r < NREG; r++)
                    if (c_ok(ti, tj, r)) {
                        T* dst = (T*)((char*)Cb + (unsigned)c_off(ti, tj, r) * (unsigned)sizeof(T));
                        if (SK == 1) c_store<(Cfg::NTC & 2) != 0>(LATE_C ? cpre[LATE_C ? ti : 0][LATE_C ? tj : 0][r] + acc[ti][tj][r] : acc[ti][tj][r], dst);
                        else unsafeAtomicAdd(dst, acc[ti][tj][r]);   // hardware global_atomic_add, device scope
                    }
            }
        }
}

// ---------------------------------------------------------------------------
// Repack kernel: out = the input with its indices permuted, dense, ext[]/sin[]
// listed in the OUTPUT order (fastest first).  One lane per element, writes
// coalesced; the reads are a gather, which is fine for the inputs this is used
// on: a few megabytes next to an output of hundreds, mostly served from L2.
struct TcRepackDims {
    int n;
    int ext[TC_MAXI], sin[TC_MAXI];
    long long total;
};

template <class T>
__global__ __launch_bounds__(256)
void tc_repack_kernel(const T* __restrict__ in, T* __restrict__ out, const TcRepackDims p)
{
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= p.total) return;
    unsigned q = (unsigned)i;
    unsigned off = 0;
    for (int j = 0; j < p.n; j++) {
        const unsigned e = (unsigned)p.ext[j];
        off += (q % e) * (unsigned)p.sin[j];
        q /= e;
    }
    out[i] = in[off];
}

// ---------------------------------------------------------------------------
// Plain kernel: one lane per output element, contracted indices walked in
// sum() order with separately rounded multiply and add, i.e. the summation
// order of the reference's host check (cogent/drivers/tccg/code_main_tccg_01.c:117-133).
// Used as the fallback for shapes the tiled kernel does not cover and as an
// on-device cross-check of it.
struct TcPlainDims {
    int n_out, n_int;
    int ext_out[TC_MAXI], sA_out[TC_MAXI], sB_out[TC_MAXI];
    int ext_k[TC_MAXI], sA_k[TC_MAXI], sB_k[TC_MAXI];
    int sign;
    long long total;    // elements of C
    long long ktotal;   // product of contracted extents
};

__device__ __forceinline__ double tc_mul_rn(double a, double b) { return __dmul_rn(a, b); }
__device__ __forceinline__ float  tc_mul_rn(float a, float b)   { return __fmul_rn(a, b); }
__device__ __forceinline__ double tc_add_rn(double a, double b) { return __dadd_rn(a, b); }
__device__ __forceinline__ float  tc_add_rn(float a, float b)   { return __fadd_rn(a, b); }

template <class T>
__global__ __launch_bounds__(256)
void tc_plain_kernel(T* __restrict__ C, const T* __restrict__ A, const T* __restrict__ B, const TcPlainDims p)
{
    const long long lin = (long long)blockIdx.x * 256 + threadIdx.x;
    if (lin >= p.total) return;
    long long r = lin;
    long long oa = 0, ob = 0;
    for (int i = 0; i < p.n_out; i++) {
        const int e = (int)(r % p.ext_out[i]);
        r /= p.ext_out[i];
        oa += (long long)e * p.sA_out[i];
        ob += (long long)e * p.sB_out[i];
    }
    T acc = C[lin];
    int k[TC_MAXI];
    for (int i = 0; i < p.n_int; i++) k[i] = 0;
    for (long long kk = 0; kk < p.ktotal; kk++) {
        long long ka = oa, kb = ob;
        for (int i = 0; i < p.n_int; i++) { ka += (long long)k[i] * p.sA_k[i]; kb += (long long)k[i] * p.sB_k[i]; }
        const T prod = tc_mul_rn(A[ka], B[kb]);
        acc = tc_add_rn(acc, p.sign < 0 ? -prod : prod);
        for (int j = p.n_int - 1; j >= 0; j--) { if (++k[j] < p.ext_k[j]) break; k[j] = 0; }
    }
    C[lin] = acc;
}

// ---------------------------------------------------------------------------
// VALU streaming kernel, written for contracted ranges too short to fill one step of a matrix instruction (fewer than
// 4 terms per output element: the fp64 and fp32 MFMAs are 4 deep).  Such a contraction is a read-modify-write stream of
// C with two or three multiply-adds per element attached.  Measured, the tiled kernel with its slices zero-padded to
// one matrix step is still the faster one there (see tc_launch.hpp), so this kernel runs only on request
// (variant 3): as a second bit-exact check kernel, 2 to 5 times faster than the plain one.  Every lane owns V
// consecutive elements of C's fastest index (one 16-byte access), U such vectors in flight, blocks walk C in its
// memory order like a plain copy kernel, and the few input elements an output element needs are read straight
// through L1/L2 (the inputs of such a shape are tiny next to C).  The terms are added in sum() order with separately
// rounded multiply and add, which is the reference host loop's arithmetic
// (cogent/drivers/tccg/code_main_tccg_01.c:117-133): the result is bit-exact with the oracle.  No cross-lane
// reduction is needed, the whole contracted range sits in one lane.
// The reference's register-tile FMA loop is the counterpart: cogent/src/codes/kernels/tc_code_kernel_compute.py:4-204.
struct TcValuDims {
    int n_out, n_int;
    int ext_out[TC_MAXI], sA_out[TC_MAXI], sB_out[TC_MAXI];     // C's indices in memory order: extent, stride in A, in B
    int ext_k[TC_MAXI], sA_k[TC_MAXI], sB_k[TC_MAXI];           // contracted indices in sum() order
    int sign;
    unsigned plane;        // elements of C's three fastest indices together: what a lane decodes for itself
    unsigned chunks;       // blocks per plane
    unsigned nplanes;      // product of the remaining output extents
    int ktotal;
};

template <class T, int V, int U>
__global__ __launch_bounds__(256)
void tc_valu_kernel(T* __restrict__ C, const T* __restrict__ A, const T* __restrict__ B, const TcValuDims p)
{
    typedef T TV __attribute__((ext_vector_type(V), aligned(sizeof(T) * V)));
    const unsigned pl = blockIdx.x / p.chunks, ch = blockIdx.x % p.chunks;
    // the block's plane: indices 3.. are the same for all its lanes
    long long baseA = 0, baseB = 0;
    {
        unsigned r = pl;
        for (int i = 3; i < p.n_out; i++) {
            const unsigned e = (unsigned)p.ext_out[i], q = r % e;
            r /= e;
            baseA += (long long)q * p.sA_out[i];
            baseB += (long long)q * p.sB_out[i];
        }
    }
    T* const Cp = C + (long long)pl * p.plane;
    const T* const Ap = A + uniform64(baseA);
    const T* const Bp = B + uniform64(baseB);
    const unsigned e0 = (unsigned)p.ext_out[0], e1 = p.n_out > 1 ? (unsigned)p.ext_out[1] : 1u;
    const int sA0 = p.sA_out[0], sB0 = p.sB_out[0];
    const int sA1 = p.n_out > 1 ? p.sA_out[1] : 0, sB1 = p.n_out > 1 ? p.sB_out[1] : 0;
    const int sA2 = p.n_out > 2 ? p.sA_out[2] : 0, sB2 = p.n_out > 2 ? p.sB_out[2] : 0;
    TV c[U];
    unsigned pos[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        pos[u] = ((ch * U + u) * 256u + threadIdx.x) * V;
        if (pos[u] < p.plane) c[u] = __builtin_nontemporal_load((const TV*)(Cp + pos[u]));
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        if (pos[u] >= p.plane) continue;
        const unsigned i0 = pos[u] % e0, t = pos[u] / e0, i1 = t % e1, i2 = t / e1;
        const int oa = (int)i0 * sA0 + (int)i1 * sA1 + (int)i2 * sA2;
        const int ob = (int)i0 * sB0 + (int)i1 * sB1 + (int)i2 * sB2;
        int k[TC_MAXI];
        for (int i = 0; i < p.n_int; i++) k[i] = 0;
        for (int kk = 0; kk < p.ktotal; kk++) {
            int ka = oa, kb = ob;
            for (int i = 0; i < p.n_int; i++) { ka += k[i] * p.sA_k[i]; kb += k[i] * p.sB_k[i]; }
#pragma unroll
            for (int v = 0; v < V; v++) {
                const T prod = tc_mul_rn(Ap[ka + v * sA0], Bp[kb + v * sB0]);
                c[u][v] = tc_add_rn(c[u][v], p.sign < 0 ? -prod : prod);
            }
            for (int j = p.n_int - 1; j >= 0; j--) { if (++k[j] < p.ext_k[j]) break; k[j] = 0; }
        }
        __builtin_nontemporal_store(c[u], (TV*)(Cp + pos[u]));
    }
}

}  // namespace cogent
