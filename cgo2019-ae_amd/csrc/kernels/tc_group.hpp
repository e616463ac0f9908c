// Fused group of contractions that accumulate into ONE output tensor:
//
//     C ±= sum A1*B1;  C ±= sum A2*B2;  ...  (same output index list, any input index orders)
//
// -- the reference's "outer group" of expressions with an identical output
// (cogent/src/algs/bases/tc_gen_inputs.py:113-123), of which the CCSD(T) triples
// terms are the use: nine contractions into one t3
// (cogent/drivers/ccsd_t/code_main_sd2_1.c:573-606).  Run one after the other
// they read and write C nine times; for these 6-D shapes that traffic is the
// whole cost.  Here a workgroup owns one tile of C for the whole group:
//
//   1. the tile is read from global memory once, in C's memory order, into LDS;
//   2. for every term: both input slices are staged to LDS, contracted on the
//      matrix cores into zero-initialised accumulators, and the result is added
//      into the LDS copy.  Which input holds C's fastest index, hence which
//      side runs along MFMA columns, differs from term to term -- the copy in
//      LDS is what lets every term use its own lane layout;
//   3. the tile is written back once.
//
// G is the group configuration (C tile, block size), Terms... one Cfg-like
// struct per term with the members the helpers of tc_kernel.hpp expect.  All
// tiles are predicated: any extents.
#pragma once
#include "tc_launch.hpp"

namespace cogent {

constexpr int TC_MAXTERMS = 16;

// per-term run-time data: the two input pointers and their element strides per index id
struct TcTermArgs {
    const void* x;
    const void* y;
    int sX[TC_MAXI], sY[TC_MAXI];
    int enabled;
};

template <int N>
struct TcGroupArgs {
    int ext[TC_MAXI], nblk[TC_MAXI], sC[TC_MAXI];
    unsigned nblocks;
    TcTermArgs term[N];
};

template <class Term> struct TermSlots {
    static constexpr int X = (Term::BK * Term::BX + Term::NT - 1) / Term::NT;
    static constexpr int Y = (Term::BK * Term::BY + Term::NT - 1) / Term::NT;
};

// Geometry of one term for the block's C tile, in the shape the helpers of tc_kernel.hpp take.
template <class Term>
struct TermGeom {
    TcDims d;
    int rem[Term::NIDX];
    const typename Term::T* Xb;
    const typename Term::T* Yb;
    int nkb;
};

template <class Term, int NARGS>
__device__ __forceinline__ void term_setup(TermGeom<Term>& g, const TcGroupArgs<NARGS>& ga, const TcTermArgs& ta, const int* origin)
{
    typedef typename Term::T T;
    // element offsets of the slices' origins: the host refuses inputs of 2^31 elements or more, so 32 bits hold them
    unsigned baseX = 0, baseY = 0;
#pragma unroll
    for (int i = 0; i < Term::NIDX; i++) {
        g.d.ext[i] = ga.ext[i]; g.d.nblk[i] = ga.nblk[i]; g.d.sC[i] = ga.sC[i]; g.d.sX[i] = ta.sX[i]; g.d.sY[i] = ta.sY[i];
        g.rem[i] = ga.ext[i] - origin[i];                     // contracted ids: origin 0
        baseX += (unsigned)origin[i] * (unsigned)ta.sX[i];
        baseY += (unsigned)origin[i] * (unsigned)ta.sY[i];
    }
    g.nkb = 1;
#pragma unroll
    for (int i = 0; i < Term::NK; i++) g.nkb *= (ga.ext[Term::k_id(i)] + Term::k_tile(i) - 1) / Term::k_tile(i);
    g.Xb = (const T*)ta.x + (size_t)(unsigned)__builtin_amdgcn_readfirstlane(baseX);
    g.Yb = (const T*)ta.y + (size_t)(unsigned)__builtin_amdgcn_readfirstlane(baseY);
}

// One term: contract its slices for the block's C tile and add the result into the LDS copy of the tile.
// (Requesting the next term's first slices while this one is contracted was tried and was 14 % slower.)
template <class G, class Term, int NARGS>
__device__ __forceinline__ void group_term(typename G::T* lds_c, typename G::T* lds_ops, const TcGroupArgs<NARGS>& ga,
                                           const TcTermArgs& ta, const int* origin, int tid)
{
    typedef typename G::T T;
    typedef Mfma<Term::MI> MM;
    typedef typename MM::Acc Acc;
    typedef Operand<Term, 0> OX;
    typedef Operand<Term, 1> OY;
    constexpr int MT = MM::MT, NREG = MM::NREG, KSTEP = MM::KSTEP, TX = Term::TX, TY = Term::TY, NT = Term::NT;
    constexpr int LDS_X = lds_elems<OX, Term::BKP>();
    constexpr int LDS_Y = lds_elems<OY, Term::BKP>();
    constexpr bool PADDED = (Term::BKP != Term::BK) || (Term::BXP != Term::BX) || (Term::BYP != Term::BY);
    static_assert(LDS_X + LDS_Y <= G::LDS_OPS, "operand slices exceed the group's LDS share");

    const int lane = tid & 63, wave = tid >> 6;
    const int wx = wave % Term::WX, wy = wave / Term::WX;
    T* lds_x = lds_ops;
    T* lds_y = lds_ops + LDS_X;

    TermGeom<Term> g;
    term_setup<Term>(g, ga, ta, origin);
    const TcDims& d = g.d;
    int* rem = g.rem;
    const int nkb = g.nkb;

    Acc acc[TY][TX];
#pragma unroll
    for (int ti = 0; ti < TY; ti++)
#pragma unroll
        for (int tj = 0; tj < TX; tj++)
#pragma unroll
            for (int r = 0; r < NREG; r++) acc[ti][tj][r] = (T)0;

    __syncthreads();                       // the previous term is done with the operand region
    if (PADDED) {
        for (int i = tid; i < LDS_X + LDS_Y; i += NT) lds_ops[i] = (T)0;
        __syncthreads();
    }

    int kbc[Term::NK > 0 ? Term::NK : 1];
#pragma unroll
    for (int i = 0; i < Term::NK; i++) kbc[i] = 0;
    for (int kb = 0; kb < nkb; kb++) {
        int64_t kx = 0, ky = 0;
#pragma unroll
        for (int i = 0; i < Term::NK; i++) {
            const int id = Term::k_id(i);
            const int o = kbc[i] * Term::k_tile(i);
            rem[id] = ga.ext[id] - o;
            kx += (int64_t)o * ta.sX[id];
            ky += (int64_t)o * ta.sY[id];
        }
        typename Term::T rx[TermSlots<Term>::X], ry[TermSlots<Term>::Y];
        slice_load<Term, OX, false, false>(rx, g.Xb + uniform64(kx), d, rem, tid);
        slice_load<Term, OY, false, false>(ry, g.Yb + uniform64(ky), d, rem, tid);
        if (kb > 0) __syncthreads();       // the previous K block's slices have been consumed
        slice_store<Term, OX, false>(rx, lds_x, d, tid);
        slice_store<Term, OY, (Term::SIGN < 0)>(ry, lds_y, d, tid);
        __syncthreads();
#pragma unroll
        for (int k4 = 0; k4 < Term::BKP / KSTEP; k4++) {
            const int kk = k4 * KSTEP + lane / MT;
            T a[TY], b[TX];
#pragma unroll
            for (int ti = 0; ti < TY; ti++) a[ti] = lds_y[lds_addr<OY>(kk, (wy * TY + ti) * MT + lane % MT)];
#pragma unroll
            for (int tj = 0; tj < TX; tj++) b[tj] = lds_x[lds_addr<OX>(kk, (wx * TX + tj) * MT + lane % MT)];
#pragma unroll
            for (int ti = 0; ti < TY; ti++)
#pragma unroll
                for (int tj = 0; tj < TX; tj++) acc[ti][tj] = MM::mma(a[ti], b[tj], acc[ti][tj]);
        }
        // next K block (first composite K index fastest)
        bool carry = true;
#pragma unroll
        for (int i = 0; i < Term::NK; i++) {
            const int id = Term::k_id(i);
            const int nb = (ga.ext[id] + Term::k_tile(i) - 1) / Term::k_tile(i);
            if (carry) { kbc[i]++; carry = false; if (kbc[i] == nb) { kbc[i] = 0; carry = true; } }
        }
    }

    // add into the LDS copy of the C tile: every element of the tile belongs to exactly one lane of
    // this term, and the barriers at the head of the next term order the terms
#pragma unroll
    for (int i = 0; i < Term::NK; i++) rem[Term::k_id(i)] = ga.ext[Term::k_id(i)];
    int cx[TX][1], cy[TY][NREG];
    c_tile_offsets<Term, false, false, true>(lane, wx, wy, rem, d, cx, cy);
#pragma unroll
    for (int ti = 0; ti < TY; ti++)
#pragma unroll
        for (int tj = 0; tj < TX; tj++)
#pragma unroll
            for (int r = 0; r < NREG; r++)
                if (cx[tj][0] >= 0 && cy[ti][r] >= 0) lds_c[cx[tj][0] + cy[ti][r]] += acc[ti][tj][r];
}

template <class G, class... Terms>
__global__ __launch_bounds__(G::NT)
void tc_group_kernel(typename G::T* __restrict__ C, const TcGroupArgs<(int)sizeof...(Terms)> ga)
{
    typedef typename G::T T;
    constexpr int NT = G::NT, VOL = G::TILE_VOL;
    T* const lds_c = (T*)tc_dynamic_lds;                     // the copy of the C tile, then one operand region
    T* const lds_ops = lds_c + VOL;
    const int tid = threadIdx.x;

    // which C tile: C's indices in C order, fastest first; XCD-contiguous ranges as in the single kernel
    int origin[G::NIDX];
#pragma unroll
    for (int i = 0; i < G::NIDX; i++) origin[i] = 0;
    int64_t baseC = 0;
    {
        const unsigned n = ga.nblocks, xcd = blockIdx.x % 8u, idx = blockIdx.x / 8u;
        const unsigned q = n / 8u, r = n % 8u;
        unsigned b = xcd * q + (xcd < r ? xcd : r) + idx;
#pragma unroll
        for (int j = 0; j < G::CR; j++) {
            const int id = G::c_id(j);
            const unsigned nb = (unsigned)ga.nblk[id];
            origin[id] = (int)(b % nb) * G::c_tile(j);
            b /= nb;
            baseC += (int64_t)origin[id] * ga.sC[id];
        }
    }
    T* __restrict__ Cb = C + uniform64(baseC);

    // element q of the tile in C's memory order: offset in the tensor, inside or outside
    auto c_element = [&](unsigned q, unsigned& off) -> bool {
        bool ok = true;
        off = 0;
#pragma unroll
        for (int j = 0; j < G::CR; j++) {
            const unsigned t = (unsigned)G::c_tile(j);
            const int c = (int)(q % t);
            q /= t;
            const int id = G::c_id(j);
            off += (unsigned)c * (unsigned)ga.sC[id];
            ok = ok && (origin[id] + c < ga.ext[id]);
        }
        return ok;
    };
    constexpr int NEL = (VOL + NT - 1) / NT;
    {
        T v[NEL];
#pragma unroll
        for (int i = 0; i < NEL; i++) {
            const unsigned q = (unsigned)(tid + i * NT);
            unsigned off;
            v[i] = (T)0;
            if ((VOL % NT == 0 || q < (unsigned)VOL) && c_element(q, off)) v[i] = Cb[off];
        }
#pragma unroll
        for (int i = 0; i < NEL; i++) {
            const unsigned q = (unsigned)(tid + i * NT);
            if (VOL % NT == 0 || q < (unsigned)VOL) lds_c[q] = v[i];
        }
    }

    // the terms, in the order of the expression file
    int t = 0;
    ((ga.term[t].enabled ? group_term<G, Terms>(lds_c, lds_ops, ga, ga.term[t], origin, tid) : (void)0, t++), ...);

    __syncthreads();
#pragma unroll
    for (int i = 0; i < NEL; i++) {
        const unsigned q = (unsigned)(tid + i * NT);
        unsigned off;
        if ((VOL % NT == 0 || q < (unsigned)VOL) && c_element(q, off)) Cb[off] = lds_c[q];
    }
}

// ---------------------------------------------------------------------------------------------------------
// Pipelined form of the group kernel, for the common call: every term enabled and every term's contracted range in
// one K block.  The serial form above pays, per term, an exposed gather of the two slices (an L2 round trip that
// nothing overlaps) and three barriers for a fraction of a microsecond of matrix work.  Here the slices of term
// t + 1 are requested BEFORE term t is contracted and go to a second operand region of the LDS after it, so that
// a term costs one barrier and its gather hides behind the previous term's matrix instructions:
//
//     load(0); load(1); store(0 -> region 0); barrier
//     for t: load(t + 2) | contract(t, region t % 2) | add into the LDS copy of C | store(t + 1 -> region (t + 1) % 2) | barrier
//
// (two register sets alternate, so a gather has two terms' time to arrive before its slices are needed in LDS)
// The one barrier per term orders three things at once: region (t + 1) % 2 is complete before term t + 1 reads it,
// term t's additions to the copy of C are visible before term t + 1 adds to other lanes' elements, and region
// t % 2 has been read by everybody before term t + 2's slices overwrite it.
// Registers per lane for a term's two slices in the pipelined kernel.  FULL: every tile of the call is whole (no
// predicates), which also lets a lane fetch Operand::VW consecutive elements of the input's fastest index at once.
// *p += v in LDS.  fp64: ONE instruction (the LDS unit adds; no value comes back) instead of read, add, write
// (5 to 15 % faster for the group of nine fp64 terms, measured side by side on several tiles).  fp32: read, add, write -- the single-instruction form
// measured 2.2 times SLOWER there (787 against 351 us for the nine fp32 terms, whatever the tile).  Every element of
// the tile is added to by exactly one lane per term and barriers separate the terms, so the sum is deterministic.
__device__ __forceinline__ void lds_accumulate(double* p, double v)
{
    (void)__hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void lds_accumulate(float* p, float v) { *p += v; }

template <class Term, bool FULL> struct PipeSlots {
    static constexpr int VX = slice_vw<Operand<Term, 0>, FULL, FULL>(), VY = slice_vw<Operand<Term, 1>, FULL, FULL>();
    static constexpr int X = slice_slots<Term, Operand<Term, 0>, VX>(), Y = slice_slots<Term, Operand<Term, 1>, VY>();
};

template <class Term, bool FULL, int MAXX, int MAXY, int NARGS>
__device__ __forceinline__ void group_load(typename Term::T (&px)[MAXX], typename Term::T (&py)[MAXY], const TcGroupArgs<NARGS>& ga,
                                           const TcTermArgs& ta, const int* origin, int tid)
{
    TermGeom<Term> g;
    term_setup<Term>(g, ga, ta, origin);
    typedef PipeSlots<Term, FULL> S;
    typename Term::T rx[S::X], ry[S::Y];
    slice_load<Term, Operand<Term, 0>, FULL, FULL>(rx, g.Xb, g.d, g.rem, tid);
    slice_load<Term, Operand<Term, 1>, FULL, FULL>(ry, g.Yb, g.d, g.rem, tid);
#pragma unroll
    for (int i = 0; i < S::X; i++) px[i] = rx[i];
#pragma unroll
    for (int i = 0; i < S::Y; i++) py[i] = ry[i];
}

template <class G, class Term, bool FULL, int MAXX, int MAXY, int NARGS>
__device__ __forceinline__ void group_store(const typename Term::T (&px)[MAXX], const typename Term::T (&py)[MAXY], typename G::T* region,
                                            const TcGroupArgs<NARGS>& ga, const TcTermArgs& ta, const int* origin, int tid)
{
    typedef typename G::T T;
    typedef Operand<Term, 0> OX;
    typedef Operand<Term, 1> OY;
    constexpr int LDS_X = lds_elems<OX, Term::BKP>(), LDS_Y = lds_elems<OY, Term::BKP>();
    constexpr bool PADDED = (Term::BKP != Term::BK) || (Term::BXP != Term::BX) || (Term::BYP != Term::BY);
    static_assert(LDS_X + LDS_Y <= G::LDS_OPS, "operand slices exceed the group's LDS share");
    TermGeom<Term> g;
    term_setup<Term>(g, ga, ta, origin);
    // the staging never writes the padding rows and columns: clear them (disjoint from what the staging writes)
    if (PADDED) {
        constexpr bool PX = (Term::BKP != Term::BK) || (Term::BXP != Term::BX), PY = (Term::BKP != Term::BK) || (Term::BYP != Term::BY);
        if (PX) for (int i = tid; i < LDS_X; i += Term::NT) region[i] = (T)0;
        if (PY) for (int i = tid; i < LDS_Y; i += Term::NT) region[LDS_X + i] = (T)0;
        if (PX || PY) __syncthreads();
    }
    typedef PipeSlots<Term, FULL> S;
    typename Term::T rx[S::X], ry[S::Y];
#pragma unroll
    for (int i = 0; i < S::X; i++) rx[i] = px[i];
#pragma unroll
    for (int i = 0; i < S::Y; i++) ry[i] = py[i];
    slice_store<Term, OX, false, S::VX>(rx, region, g.d, tid);
    slice_store<Term, OY, (Term::SIGN < 0), S::VY>(ry, region + LDS_X, g.d, tid);
}

template <class G, class Term, bool FULL, int NARGS>
__device__ __forceinline__ void group_contract(typename G::T* lds_c, const typename G::T* region, const TcGroupArgs<NARGS>& ga,
                                               const TcTermArgs& ta, const int* origin, int tid)
{
    typedef typename G::T T;
    typedef Mfma<Term::MI> MM;
    typedef typename MM::Acc Acc;
    typedef Operand<Term, 0> OX;
    typedef Operand<Term, 1> OY;
    constexpr int MT = MM::MT, NREG = MM::NREG, KSTEP = MM::KSTEP, TX = Term::TX, TY = Term::TY;
    constexpr int LDS_X = lds_elems<OX, Term::BKP>();
    const int lane = tid & 63, wave = tid >> 6;
    const int wx = wave % Term::WX, wy = wave / Term::WX;
    const T* lds_x = region;
    const T* lds_y = region + LDS_X;
    Acc acc[TY][TX];
#pragma unroll
    for (int ti = 0; ti < TY; ti++)
#pragma unroll
        for (int tj = 0; tj < TX; tj++)
#pragma unroll
            for (int r = 0; r < NREG; r++) acc[ti][tj][r] = (T)0;
#pragma unroll
    for (int k4 = 0; k4 < Term::BKP / KSTEP; k4++) {
        const int kk = k4 * KSTEP + lane / MT;
        T a[TY], b[TX];
#pragma unroll
        for (int ti = 0; ti < TY; ti++) a[ti] = lds_y[lds_addr<OY>(kk, (wy * TY + ti) * MT + lane % MT)];
#pragma unroll
        for (int tj = 0; tj < TX; tj++) b[tj] = lds_x[lds_addr<OX>(kk, (wx * TX + tj) * MT + lane % MT)];
#pragma unroll
        for (int ti = 0; ti < TY; ti++)
#pragma unroll
            for (int tj = 0; tj < TX; tj++) acc[ti][tj] = MM::mma(a[ti], b[tj], acc[ti][tj]);
    }
    TermGeom<Term> g;
    term_setup<Term>(g, ga, ta, origin);
    int cx[TX][1], cy[TY][NREG];
    c_tile_offsets<Term, FULL, false, true>(lane, wx, wy, g.rem, g.d, cx, cy);
    constexpr bool ALL = FULL && Term::BXP == Term::BX && Term::BYP == Term::BY;     // no lane holds a position outside the tile
#pragma unroll
    for (int ti = 0; ti < TY; ti++)
#pragma unroll
        for (int tj = 0; tj < TX; tj++)
#pragma unroll
            for (int r = 0; r < NREG; r++)
                if (ALL || (cx[tj][0] >= 0 && cy[ti][r] >= 0)) lds_accumulate(lds_c + cx[tj][0] + cy[ti][r], (T)acc[ti][tj][r]);
}

template <class... Terms> struct TermList {};
template <int I, class First, class... Rest> struct TermAt { typedef typename TermAt<I - 1, Rest...>::type type; };
template <class First, class... Rest> struct TermAt<0, First, Rest...> { typedef First type; };
constexpr int tc_max_of() { return 0; }
template <class... R> constexpr int tc_max_of(int a, R... r) { return a > tc_max_of(r...) ? a : tc_max_of(r...); }

// NREGION = 2: as above.  NREGION = 1: one operand region; the slices of term t + 1 wait in registers until everybody
// has finished term t (a second barrier per term), which halves the operand LDS and so lets twice as many workgroups
// share a CU -- the kernel is bound by latency, not by bandwidth, so resident wavefronts are what it wants.
// FULL: every extent is a whole number of tiles, so nothing is predicated.
template <int NREGION, bool FULL, class G, class... Terms>
__global__ __launch_bounds__(G::NT)
void tc_group_pipe_kernel(typename G::T* __restrict__ C, const TcGroupArgs<(int)sizeof...(Terms)> ga)
{
    typedef typename G::T T;
    constexpr int N = (int)sizeof...(Terms);
    constexpr int NT = G::NT, VOL = G::TILE_VOL;
    constexpr int MAXX = tc_max_of(PipeSlots<Terms, FULL>::X...), MAXY = tc_max_of(PipeSlots<Terms, FULL>::Y...);
    T* const lds_c = (T*)tc_dynamic_lds;
    T* const lds_ops = lds_c + VOL;                          // two regions of G::LDS_OPS elements
    const int tid = threadIdx.x;

    int origin[G::NIDX];
#pragma unroll
    for (int i = 0; i < G::NIDX; i++) origin[i] = 0;
    int64_t baseC = 0;
    {
        // tiles in the order of their origins in C's memory: the tiles in flight chip-wide form one compact window
        unsigned b = blockIdx.x;
#pragma unroll
        for (int j = 0; j < G::CR; j++) {
            const int id = G::c_id(j);
            const unsigned nb = (unsigned)ga.nblk[id];
            origin[id] = (int)(b % nb) * G::c_tile(j);
            b /= nb;
            baseC += (int64_t)origin[id] * ga.sC[id];
        }
    }
    T* __restrict__ Cb = C + uniform64(baseC);
    auto c_element = [&](unsigned q, unsigned& off) -> bool {
        bool ok = true;
        off = 0;
#pragma unroll
        for (int j = 0; j < G::CR; j++) {
            const unsigned t = (unsigned)G::c_tile(j);
            const int c = (int)(q % t);
            q /= t;
            const int id = G::c_id(j);
            off += (unsigned)c * (unsigned)ga.sC[id];
            if (!FULL) ok = ok && (origin[id] + c < ga.ext[id]);
        }
        return ok;
    };
    // whole tiles: CV consecutive elements of C's fastest index per lane and access (C's fastest stride is 1)
    constexpr int CV = (FULL && G::c_tile(0) % (16 / (int)sizeof(T)) == 0 && VOL % (NT * (16 / (int)sizeof(T))) == 0) ? 16 / (int)sizeof(T) : 1;
    typedef T TCV __attribute__((ext_vector_type(CV), aligned(sizeof(T))));
    typedef T TLV __attribute__((ext_vector_type(CV)));
    constexpr int NEL = (VOL / CV + NT - 1) / NT;
    T px[2][MAXX], py[2][MAXY];
    {
        // the first two terms' slices are requested before the C tile: they come from L2, the tile from HBM
        typedef typename TermAt<0, Terms...>::type Term0;
        typedef typename TermAt<(N > 1 ? 1 : 0), Terms...>::type Term1;
        group_load<Term0, FULL, MAXX, MAXY>(px[0], py[0], ga, ga.term[0], origin, tid);
        if constexpr (N > 1) group_load<Term1, FULL, MAXX, MAXY>(px[1], py[1], ga, ga.term[1], origin, tid);
        TLV v[NEL];
#pragma unroll
        for (int i = 0; i < NEL; i++) {
            const unsigned q = (unsigned)(tid + i * NT) * CV;
            unsigned off;
#pragma unroll
            for (int e = 0; e < CV; e++) v[i][e] = (T)0;
            if ((VOL % (NT * CV) == 0 || q < (unsigned)VOL) && c_element(q, off)) {
                const TCV w = __builtin_nontemporal_load((const TCV*)(Cb + off));
#pragma unroll
                for (int e = 0; e < CV; e++) v[i][e] = w[e];
            }
        }
        group_store<G, Term0, FULL, MAXX, MAXY>(px[0], py[0], lds_ops, ga, ga.term[0], origin, tid);
#pragma unroll
        for (int i = 0; i < NEL; i++) {
            const unsigned q = (unsigned)(tid + i * NT) * CV;
            if (VOL % (NT * CV) == 0 || q < (unsigned)VOL) *(TLV*)(lds_c + q) = v[i];
        }
        __syncthreads();
    }
    static_for<N>([&](auto tt) {
        constexpr int t = decltype(tt)::value;
        typedef typename TermAt<t, Terms...>::type Term;
        typedef typename TermAt<(t + 1 < N ? t + 1 : t), Terms...>::type Next;
        typedef typename TermAt<(t + 2 < N ? t + 2 : t), Terms...>::type Far;
        if constexpr (t + 2 < N) group_load<Far, FULL, MAXX, MAXY>(px[t & 1], py[t & 1], ga, ga.term[t + 2], origin, tid);
        group_contract<G, Term, FULL>(lds_c, lds_ops + (NREGION == 2 ? (t & 1) : 0) * G::LDS_OPS, ga, ga.term[t], origin, tid);
        if constexpr (NREGION == 1 && t + 1 < N) __syncthreads();          // everybody is done reading the one region
        if constexpr (t + 1 < N) group_store<G, Next, FULL, MAXX, MAXY>(px[(t + 1) & 1], py[(t + 1) & 1], lds_ops + (NREGION == 2 ? ((t + 1) & 1) : 0) * G::LDS_OPS, ga, ga.term[t + 1], origin, tid);
        __syncthreads();
    });
#pragma unroll
    for (int i = 0; i < NEL; i++) {
        const unsigned q = (unsigned)(tid + i * NT) * CV;
        unsigned off;
        if ((VOL % (NT * CV) == 0 || q < (unsigned)VOL) && c_element(q, off)) {
            const TLV w = *(const TLV*)(lds_c + q);
            TCV o;
#pragma unroll
            for (int e = 0; e < CV; e++) o[e] = w[e];
            __builtin_nontemporal_store(o, (TCV*)(Cb + off));
        }
    }
}

// Persistent form of the pipelined kernel for whole tiles: a workgroup takes tiles blockIdx.x, + gridDim.x, ... and the
// pipeline of the terms runs ACROSS tile boundaries -- during the last two terms of a tile the slices of the next
// tile's first two terms are requested, during the last term its C tile, so that no tile but a workgroup's first
// starts with an exposed round trip to memory.  Opt-in (spec ps=1): measured 169 against 160 us (fp64) and 100 against
// 90 us (fp32) for the nine CCSD(T) terms -- two to six workgroups per CU in different phases already hide a tile's
// start, and this kernel needs 40 more registers.  With an odd number of terms the two register sets (and, with two
// operand regions, the regions) change roles from tile to tile: the tile body exists once per parity P, a term t of
// the tile living in set (t + P) % 2.
template <int NREGION, class G, class... Terms>
__global__ __launch_bounds__(G::NT)
void tc_group_persist_kernel(typename G::T* __restrict__ C, const TcGroupArgs<(int)sizeof...(Terms)> ga)
{
    typedef typename G::T T;
    constexpr bool FULL = true;
    constexpr int N = (int)sizeof...(Terms);
    static_assert(N >= 2, "a group has two terms or more");
    constexpr int NT = G::NT, VOL = G::TILE_VOL;
    constexpr int MAXX = tc_max_of(PipeSlots<Terms, FULL>::X...), MAXY = tc_max_of(PipeSlots<Terms, FULL>::Y...);
    T* const lds_c = (T*)tc_dynamic_lds;
    T* const lds_ops = lds_c + VOL;
    // (not const: every tile re-reads it through an empty asm, so that the per-lane offsets of all terms' slice
    // elements, which do not change from tile to tile, are recomputed per tile instead of being kept in ~200
    // registers across the tile loop, which is what the compiler otherwise does)
    int tid = threadIdx.x;
    constexpr int CV = (G::c_tile(0) % (16 / (int)sizeof(T)) == 0 && VOL % (NT * (16 / (int)sizeof(T))) == 0) ? 16 / (int)sizeof(T) : 1;
    typedef T TCV __attribute__((ext_vector_type(CV), aligned(sizeof(T))));
    typedef T TLV __attribute__((ext_vector_type(CV)));
    constexpr int NEL = (VOL / CV + NT - 1) / NT;

    // origin of tile b (tiles in the order of their origins in C's memory) and the address of its first element
    auto decode = [&](unsigned b, int (&org)[G::NIDX]) -> T* {
        int64_t baseC = 0;
#pragma unroll
        for (int i = 0; i < G::NIDX; i++) org[i] = 0;
#pragma unroll
        for (int j = 0; j < G::CR; j++) {
            const int id = G::c_id(j);
            const unsigned nb = (unsigned)ga.nblk[id];
            org[id] = (int)(b % nb) * G::c_tile(j);
            b /= nb;
            baseC += (int64_t)org[id] * ga.sC[id];
        }
        return C + uniform64(baseC);
    };
    // element q of a tile in C's memory order: its offset from the tile's first element (the same for every tile)
    auto c_offset = [&](unsigned q) -> unsigned {
        unsigned off = 0;
#pragma unroll
        for (int j = 0; j < G::CR; j++) {
            const unsigned t = (unsigned)G::c_tile(j);
            off += (q % t) * (unsigned)ga.sC[G::c_id(j)];
            q /= t;
        }
        return off;
    };
    auto c_read = [&](TLV (&v)[NEL], const T* Cb) {
#pragma unroll
        for (int i = 0; i < NEL; i++) {
            const unsigned q = (unsigned)(tid + i * NT) * CV;
            if (VOL % (NT * CV) == 0 || q < (unsigned)VOL) {
                const TCV w = __builtin_nontemporal_load((const TCV*)(Cb + c_offset(q)));
#pragma unroll
                for (int e = 0; e < CV; e++) v[i][e] = w[e];
            }
        }
    };
    auto c_to_lds = [&](const TLV (&v)[NEL]) {
#pragma unroll
        for (int i = 0; i < NEL; i++) {
            const unsigned q = (unsigned)(tid + i * NT) * CV;
            if (VOL % (NT * CV) == 0 || q < (unsigned)VOL) *(TLV*)(lds_c + q) = v[i];
        }
    };
    auto c_write = [&](T* Cb) {
#pragma unroll
        for (int i = 0; i < NEL; i++) {
            const unsigned q = (unsigned)(tid + i * NT) * CV;
            if (VOL % (NT * CV) == 0 || q < (unsigned)VOL) {
                const TLV w = *(const TLV*)(lds_c + q);
                TCV o;
#pragma unroll
                for (int e = 0; e < CV; e++) o[e] = w[e];
                __builtin_nontemporal_store(o, (TCV*)(Cb + c_offset(q)));
            }
        }
    };

    typedef typename TermAt<0, Terms...>::type Term0;
    typedef typename TermAt<(N > 1 ? 1 : 0), Terms...>::type Term1;
    T px[2][MAXX], py[2][MAXY];
    TLV v[NEL];
    int org[G::NIDX], org_n[G::NIDX];
    unsigned tile = blockIdx.x;
    T* Cb = decode(tile, org);
    T* Cb_n = Cb;
    group_load<Term0, FULL, MAXX, MAXY>(px[0], py[0], ga, ga.term[0], org, tid);
    if constexpr (N > 1) group_load<Term1, FULL, MAXX, MAXY>(px[1], py[1], ga, ga.term[1], org, tid);
    c_read(v, Cb);
    group_store<G, Term0, FULL, MAXX, MAXY>(px[0], py[0], lds_ops, ga, ga.term[0], org, tid);
    c_to_lds(v);
    __syncthreads();

    // one tile.  HAS_NEXT is a template parameter, not a run-time test, so that a tile body holds no branch: the
    // compiler's counts of outstanding loads stay exact at every wait (a branch around a load makes every later wait
    // in the body a wait for everything).
    auto body = [&](auto par, auto more) {
        constexpr int P = decltype(par)::value;
        constexpr bool HAS_NEXT = decltype(more)::value;
        asm volatile("" : "+v"(tid));
        static_for<N>([&](auto tt) {
            constexpr int t = decltype(tt)::value;
            constexpr int S = (t + P) & 1;                       // the set term t came from: free now
            typedef typename TermAt<t, Terms...>::type Term;
            typedef typename TermAt<(t + 1) % N, Terms...>::type Next;
            typedef typename TermAt<(t + 2) % N, Terms...>::type Far;
            if constexpr (t + 2 < N) group_load<Far, FULL, MAXX, MAXY>(px[S], py[S], ga, ga.term[t + 2], org, tid);
            else if constexpr (HAS_NEXT) group_load<Far, FULL, MAXX, MAXY>(px[S], py[S], ga, ga.term[(t + 2) % N], org_n, tid);
            if constexpr (t == N - 1 && HAS_NEXT) c_read(v, Cb_n);
            group_contract<G, Term, FULL>(lds_c, lds_ops + (NREGION == 2 ? S : 0) * G::LDS_OPS, ga, ga.term[t], org, tid);
            if constexpr (t + 1 < N || HAS_NEXT) {
                if constexpr (NREGION == 1) __syncthreads();     // everybody is done reading the one region
                group_store<G, Next, FULL, MAXX, MAXY>(px[S ^ 1], py[S ^ 1], lds_ops + (NREGION == 2 ? (S ^ 1) : 0) * G::LDS_OPS, ga,
                                                       ga.term[(t + 1) % N], t + 1 < N ? org : org_n, tid);
            }
            __syncthreads();
        });
        c_write(Cb);
        if constexpr (HAS_NEXT) {
            // a lane overwrites exactly the elements it has just read; the barrier is for the other lanes' additions
            c_to_lds(v);
            __syncthreads();
        }
    };
    const std::true_type yes;
    const std::false_type no;
    auto advance = [&](unsigned next) {
        tile = next;
        Cb = Cb_n;
#pragma unroll
        for (int i = 0; i < G::NIDX; i++) org[i] = org_n[i];
    };
    // two tiles per trip: with an odd number of terms the second one runs with the register sets exchanged
    for (;;) {
        unsigned next = tile + gridDim.x;
        if (next >= ga.nblocks) { body(std::integral_constant<int, 0>(), no); break; }
        Cb_n = decode(next, org_n);
        body(std::integral_constant<int, 0>(), yes);
        advance(next);
        next = tile + gridDim.x;
        if (next >= ga.nblocks) { body(std::integral_constant<int, N & 1>(), no); break; }
        Cb_n = decode(next, org_n);
        body(std::integral_constant<int, N & 1>(), yes);
        advance(next);
    }
}

// Host side.  inputs[] holds the 2 * NTERM input pointers in expression order (A of term 1, B of term 1,
// A of term 2, ...); enabled[] (may be null: all) says which terms to apply; sizes[] as for tc_run.
template <class G, class... Terms>
int tc_group_run(const int* sizes, void* C, const void* const* inputs, const int* enabled, hipStream_t stream)
{
    typedef typename G::T T;
    constexpr int N = (int)sizeof...(Terms);
    static_assert(N >= 1 && N <= TC_MAXTERMS, "number of fused terms");
    tc_error_buffer()[0] = 0;
    for (int i = 0; i < G::NIDX; i++)
        if (sizes[i] < 0) return tc_fail(TC_ERR_NEGATIVE_EXTENT, "negative extent");
    for (int i = 0; i < G::NIDX; i++)
        if (sizes[i] == 0) return TC_OK;
    if (!C || !inputs) return tc_fail(TC_ERR_NULL_POINTER, "null tensor pointer");
    for (int i = 0; i < 2 * N; i++)
        if (!inputs[i] && (!enabled || enabled[i / 2])) return tc_fail(TC_ERR_NULL_POINTER, "null tensor pointer");

    TcGroupArgs<N> ga;
    memset(&ga, 0, sizeof(ga));
    const int64_t lim = ((int64_t)1 << 31) - 1;
    int64_t nC = 1, grid = 1;
    for (int i = 0; i < G::NIDX; i++) { ga.ext[i] = sizes[i]; ga.nblk[i] = 1; }
    for (int j = 0; j < G::CR; j++) {
        const int id = G::c_id(j);
        ga.sC[id] = (int)nC;
        nC *= sizes[id];
        if (nC > lim) return tc_fail(TC_ERR_TOO_LARGE, "a tensor has more than 2^31-1 elements");
        ga.nblk[id] = (sizes[id] + G::c_tile(j) - 1) / G::c_tile(j);
        grid *= ga.nblk[id];
        if (grid > lim) return tc_fail(TC_ERR_TOO_LARGE, "grid too large");
    }
    ga.nblocks = (unsigned)grid;
    bool too_large = false, too_far = false;
    const int64_t far = ((int64_t)1 << 32) / (int64_t)sizeof(T) - 4;   // 32-bit byte offsets inside a tile and a slice
    {
        int64_t span = 0;
        for (int j = 0; j < G::CR; j++) {
            const int id = G::c_id(j);
            span += (int64_t)((sizes[id] < G::c_tile(j) ? sizes[id] : G::c_tile(j)) - 1) * ga.sC[id];
        }
        if (span >= far) too_far = true;
    }
    int t = 0;
    auto fill = [&](auto term) {
        typedef decltype(term) Term;
        TcTermArgs& ta = ga.term[t];
        ta.x = inputs[2 * t + (Term::X_IS_A ? 0 : 1)];
        ta.y = inputs[2 * t + (Term::X_IS_A ? 1 : 0)];
        ta.enabled = enabled ? (enabled[t] != 0) : 1;
        int64_t n = 1;
        for (int j = 0; j < Term::XR; j++) { ta.sX[Term::xo_id(j)] = (int)n; n *= sizes[Term::xo_id(j)]; if (n > lim) too_large = true; }
        n = 1;
        for (int j = 0; j < Term::YR; j++) { ta.sY[Term::yo_id(j)] = (int)n; n *= sizes[Term::yo_id(j)]; if (n > lim) too_large = true; }
        if (!too_large) {
            int64_t sx = 0, sy = 0;
            for (int j = 0; j < Term::XR; j++) { const int id = Term::xo_id(j); sx += (int64_t)((sizes[id] < Term::xo_tile(j) ? sizes[id] : Term::xo_tile(j)) - 1) * ta.sX[id]; }
            for (int j = 0; j < Term::YR; j++) { const int id = Term::yo_id(j); sy += (int64_t)((sizes[id] < Term::yo_tile(j) ? sizes[id] : Term::yo_tile(j)) - 1) * ta.sY[id]; }
            if (sx >= far || sy >= far) too_far = true;
        }
        t++;
    };
    (fill(Terms()), ...);
    if (too_large) return tc_fail(TC_ERR_TOO_LARGE, "a tensor has more than 2^31-1 elements");
    if (too_far) return tc_fail(TC_ERR_TOO_LARGE, "a tile of this mapping spans 4 GB or more of a tensor (byte offsets inside a tile are 32-bit)");

    tc_clear_hip_error();
    // every term enabled, every contracted range within one K block: the pipelined kernel
    bool pipe = true;
    for (int i = 0; i < N; i++) pipe = pipe && ga.term[i].enabled;
    auto one_kb = [&](auto term) {
        typedef decltype(term) Term;
        for (int i = 0; i < Term::NK; i++) if (sizes[Term::k_id(i)] > Term::k_tile(i)) pipe = false;
    };
    (one_kb(Terms()), ...);
    // whole tiles everywhere (the contracted extents then equal their tiles): the variant without predicates
    bool full = true;
    for (int j = 0; j < G::CR; j++) if (sizes[G::c_id(j)] % G::c_tile(j)) full = false;
    auto whole_k = [&](auto term) {
        typedef decltype(term) Term;
        for (int i = 0; i < Term::NK; i++) if (sizes[Term::k_id(i)] != Term::k_tile(i)) full = false;
    };
    (whole_k(Terms()), ...);
    constexpr int NREGION = G::NREGION > 0 ? G::NREGION : 1;
    if (G::NREGION == 0) pipe = false;                 // nr=0: the kernel with one load-store-contract pass per term
    constexpr size_t pipe_lds = sizeof(T) * ((size_t)G::TILE_VOL + NREGION * (size_t)G::LDS_OPS);
    constexpr size_t serial_lds = sizeof(T) * ((size_t)G::TILE_VOL + (size_t)G::LDS_OPS);
    static_assert(serial_lds <= 160 * 1024, "the C tile and one operand region exceed the LDS of a CU");
    if (pipe_lds > 160 * 1024) pipe = false;
    if (pipe_lds > 65536 || serial_lds > 65536) {
        // more than the 64 KB a kernel may use unasked: raise the limit once per device
        static std::atomic<bool> configured[64];
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return tc_fail(TC_ERR_LAUNCH, "no current device for the fused group kernel");
        if (!configured[dev].load(std::memory_order_acquire)) {
            bool ok = hipFuncSetAttribute((const void*)&tc_group_kernel<G, Terms...>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)serial_lds) == hipSuccess;
            if (pipe_lds <= 160 * 1024) {
                ok = ok && hipFuncSetAttribute((const void*)&tc_group_pipe_kernel<NREGION, false, G, Terms...>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)pipe_lds) == hipSuccess;
                ok = ok && hipFuncSetAttribute((const void*)&tc_group_pipe_kernel<NREGION, true, G, Terms...>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)pipe_lds) == hipSuccess;
                ok = ok && hipFuncSetAttribute((const void*)&tc_group_persist_kernel<NREGION, G, Terms...>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)pipe_lds) == hipSuccess;
            }
            if (!ok) { (void)hipGetLastError(); return tc_fail(TC_ERR_LAUNCH, "the fused group kernel's LDS size was refused"); }
            configured[dev].store(true, std::memory_order_release);
        }
    }
    if (pipe && full && G::PERSIST) {
        // as many workgroups as the chip holds at once, each walking tiles blockIdx.x, + gridDim.x, ...
        static std::atomic<int> slots[64];
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return tc_fail(TC_ERR_LAUNCH, "no current device for the fused group kernel");
        int n_slots = slots[dev].load(std::memory_order_acquire);
        if (n_slots == 0) {
            int per_cu = 0, cus = 0;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)&tc_group_persist_kernel<NREGION, G, Terms...>, G::NT, pipe_lds) != hipSuccess ||
                hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || per_cu < 1 || cus < 1) {
                (void)hipGetLastError();
                n_slots = -1;                          // no answer: the kernel with one workgroup per tile
            } else {
                n_slots = per_cu * cus;
            }
            slots[dev].store(n_slots, std::memory_order_release);
        }
        if (n_slots > 0) {
            const unsigned g = (unsigned)std::min<int64_t>(grid, n_slots);
            hipLaunchKernelGGL((tc_group_persist_kernel<NREGION, G, Terms...>), dim3(g), dim3(G::NT), pipe_lds, stream, (T*)C, ga);
            return tc_check_launch("fused group kernel launch failed");
        }
    }
    if (pipe && full) hipLaunchKernelGGL((tc_group_pipe_kernel<NREGION, true, G, Terms...>), dim3((unsigned)grid), dim3(G::NT), pipe_lds, stream, (T*)C, ga);
    else if (pipe)    hipLaunchKernelGGL((tc_group_pipe_kernel<NREGION, false, G, Terms...>), dim3((unsigned)grid), dim3(G::NT), pipe_lds, stream, (T*)C, ga);
    else              hipLaunchKernelGGL((tc_group_kernel<G, Terms...>), dim3((unsigned)grid), dim3(G::NT), serial_lds, stream, (T*)C, ga);
    return tc_check_launch("fused group kernel launch failed");
}

// The reference's calling convention for a group: HOST pointers, result copied back.
template <class G, class... Terms>
int tc_group_run_host(const int* sizes, void* hC, const void* const* h_inputs)
{
    typedef typename G::T T;
    constexpr int N = (int)sizeof...(Terms);
    for (int i = 0; i < G::NIDX; i++)
        if (sizes[i] < 0) return tc_fail(TC_ERR_NEGATIVE_EXTENT, "negative extent");
    for (int i = 0; i < G::NIDX; i++)
        if (sizes[i] == 0) return TC_OK;
    if (!hC || !h_inputs) return tc_fail(TC_ERR_NULL_POINTER, "null tensor pointer");
    int64_t count[2 * N + 1];
    {
        int64_t nC = 1;
        for (int j = 0; j < G::CR; j++) nC *= sizes[G::c_id(j)];
        count[2 * N] = nC;
        int t = 0;
        auto sz = [&](auto term) {
            typedef decltype(term) Term;
            int64_t nx = 1, ny = 1;
            for (int j = 0; j < Term::XR; j++) nx *= sizes[Term::xo_id(j)];
            for (int j = 0; j < Term::YR; j++) ny *= sizes[Term::yo_id(j)];
            count[2 * t + (Term::X_IS_A ? 0 : 1)] = nx;
            count[2 * t + (Term::X_IS_A ? 1 : 0)] = ny;
            t++;
        };
        (sz(Terms()), ...);
    }
    void* dev[2 * N + 1];
    for (int i = 0; i <= 2 * N; i++) dev[i] = nullptr;
    int rc = TC_OK;
    for (int i = 0; i <= 2 * N && rc == TC_OK; i++) {
        const void* src = (i == 2 * N) ? hC : h_inputs[i];
        if (!src) { rc = tc_fail(TC_ERR_NULL_POINTER, "null tensor pointer"); break; }
        if (hipMalloc(&dev[i], count[i] * sizeof(T)) != hipSuccess) rc = tc_fail(TC_ERR_ALLOC, "device allocation failed");
        else if (hipMemcpy(dev[i], src, count[i] * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) rc = tc_fail(TC_ERR_ALLOC, "host to device copy failed");
    }
    if (rc == TC_OK) {
        rc = tc_group_run<G, Terms...>(sizes, dev[2 * N], (const void* const*)dev, nullptr, 0);
        if (rc == TC_OK && hipMemcpy(hC, dev[2 * N], count[2 * N] * sizeof(T), hipMemcpyDeviceToHost) != hipSuccess)
            rc = tc_fail(TC_ERR_LAUNCH, "kernel execution or device to host copy failed");
    }
    for (int i = 0; i <= 2 * N; i++) if (dev[i]) (void)hipFree(dev[i]);
    return rc;
}

}  // namespace cogent
