// Panel-resident streaming kernel: a second shape of the contraction kernel for outputs that are
// much larger than the inputs and have a short contracted range (a handful of K blocks).
//
// tc_mfma_kernel gives every output tile a workgroup of its own.  With few K blocks per tile that
// workgroup spends most of its life in latencies that nothing overlaps: the C tile read, the first
// slices, the write-back.  Here a workgroup is persistent over a RUN of output tiles that share
// their X-side tile:
//
//   * the panel of one side (its tile over the whole contracted range, NKB slices; the X panel below)
//     is loaded into LDS once per workgroup and stays;
//   * the Y slices of the tiles of the run pass through a two-stage LDS buffer as ONE stream, PD
//     slices requested ahead in registers, across tile boundaries: the first slices of the next tile
//     are in flight while the last K blocks of the current tile are contracted;
//   * the C tile of the NEXT output tile is read piece by piece (one MFMA tile per piece) during the
//     K blocks of the current one, into registers that the first K block has already consumed as the
//     matrix instruction's addend, so that a C read has a whole tile time to arrive and no load burst
//     stands in front of the slice loads in the in-order return path;
//   * the finished tile is stored while the next one is already being contracted.
//
// Either side can be the resident one (RES = 0: the X panel stays and the run walks Y tiles; RES = 1:
// the Y panel stays and the run walks X tiles): the side to keep is the one whose tile over the whole
// contracted range fits the LDS and is re-used by many tiles -- with a small matrix on one side that is
// the whole matrix.  Tiles padded to the MFMA granularity are allowed: the padding rows of the LDS
// buffers are cleared once and never written, the padding elements of the C tile are skipped.
//
// The K-block count NKB is a compile-time constant (the emitter takes it from the representative
// extents of the expression): every trip of a tile is a copy of its own, which is what lets the
// compiler count the loads in flight exactly.  The launcher uses this kernel only when the run-time
// extents give that K-block count and every tile is full; otherwise the call goes to tc_mfma_kernel.
#pragma once
#include "tc_kernel.hpp"

namespace cogent {

// Measurement builds only (never defined by the emitter or the build script): switches parts of the kernel off so
// that the cost of each can be read from the clock; the results are then wrong.
// bit 0: no C reads, bit 1: no C writes, bit 2: no loads of the streamed slices, bit 3: no matrix instructions
#ifndef TC_STREAM_ABLATE
#define TC_STREAM_ABLATE 0
#endif

struct TcStreamDims {
    unsigned nres;     // tiles of the whole output along the resident side
    unsigned nstr;     // ... along the streamed side
    unsigned run;      // consecutive streamed-side tiles handled by one workgroup
    unsigned nruns;    // workgroups per resident-side tile
};



// Position of a K block in the contracted range (first composite K index fastest) and the element
// offset of its slice inside an operand.  next() wraps from the last block to the first.
template <class Cfg, int SIDE>
struct KWalk {
    int c[Cfg::NK > 0 ? Cfg::NK : 1];
    __device__ __forceinline__ void reset()
    {
#pragma unroll
        for (int i = 0; i < Cfg::NK; i++) c[i] = 0;
    }
    __device__ __forceinline__ int64_t offset(const TcDims& d) const
    {
        int64_t o = 0;
#pragma unroll
        for (int i = 0; i < Cfg::NK; i++) o += (int64_t)(c[i] * Cfg::k_tile(i)) * Operand<Cfg, SIDE>::stride(d, Cfg::k_id(i));
        return o;
    }
    __device__ __forceinline__ void next(const TcDims& d)
    {
        bool carry = true;
#pragma unroll
        for (int i = 0; i < Cfg::NK; i++)
            if (carry) { c[i]++; carry = false; if (c[i] == d.nblk[Cfg::k_id(i)]) { c[i] = 0; carry = true; } }
    }
};

template <class Cfg, bool SWP>
__global__ __launch_bounds__(Cfg::NT, Cfg::SMW)
void tc_stream_kernel(typename Cfg::T* __restrict__ C, const typename Cfg::T* __restrict__ X,
                      const typename Cfg::T* __restrict__ Y, const TcDims d, const TcStreamDims s)
{
    typedef typename Cfg::T T;
    typedef Mfma<Cfg::MI> MM;
    typedef typename MM::Acc Acc;
    typedef Operand<Cfg, 0> OX;
    typedef Operand<Cfg, 1> OY;
    constexpr int RES = Cfg::SRES;                 // 0: X panel resident, 1: Y panel resident
    typedef Operand<Cfg, RES> OR;                  // the resident operand
    typedef Operand<Cfg, 1 - RES> OS;              // the streamed operand
    constexpr int MT = MM::MT, NREG = MM::NREG, KSTEP = MM::KSTEP;
    constexpr int TX = Cfg::TX, TY = Cfg::TY, NT = Cfg::NT;
    constexpr int NKB = Cfg::STREAM, PD = Cfg::SPD;
    static_assert(NKB >= 2 && PD >= 1 && PD <= NKB && NKB % PD == 0, "prefetch depth must divide the K-block count");
    constexpr bool PADDED = (Cfg::BKP != Cfg::BK) || (Cfg::BXP != Cfg::BX) || (Cfg::BYP != Cfg::BY);
    constexpr int VR = slice_vw<OR, true, true>(), VS = slice_vw<OS, true, true>();
    constexpr int SLOTS_R = slice_slots<Cfg, OR, VR>();
    constexpr int SLOTS_S = slice_slots<Cfg, OS, VS>();
    constexpr int LDS_R = lds_elems<OR, Cfg::BKP>();
    constexpr int LDS_S = lds_elems<OS, Cfg::BKP>();
    constexpr bool NEG_R = (RES == 1) && (Cfg::SIGN < 0);      // "-=" negates the Y operand while it is staged
    constexpr bool NEG_S = (RES == 0) && (Cfg::SIGN < 0);
    constexpr bool VEC4 = SWP;
    constexpr bool SOV = Cfg::SOV != 0;            // the panel's later slices are loaded behind the first tile
    constexpr bool NT_LD = (Cfg::NTC & 1) != 0, NT_ST = (Cfg::NTC & 2) != 0;
    typedef T T4 __attribute__((ext_vector_type(4)));

    T* const lds_r = (T*)tc_dynamic_lds;            // NKB slices of the resident tile
    T* const lds_s = lds_r + NKB * LDS_R;          // two stages of one slice of the streamed operand

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wx = wave % Cfg::WX;
    const int wy = wave / Cfg::WX;

    // ---- this workgroup's resident tile and its run of streamed-side tiles
    // Workgroups go to the 8 XCDs round-robin and every XCD has its own L2: give XCD x a contiguous
    // range of (resident tile, run) pairs, resident tiles fastest, so that neighbouring tiles are worked
    // on at the same time on one L2.
    unsigned vb;
    {
        const unsigned n = gridDim.x, xcd = blockIdx.x % 8u, idx = blockIdx.x / 8u;
        const unsigned q = n / 8u, r = n % 8u;
        vb = xcd * q + (xcd < r ? xcd : r) + idx;
    }
    const unsigned rt = vb % s.nres, rn = vb / s.nres;
    // The run of workgroup rn: ntiles streamed-side tiles, `step` apart.  Contiguous runs (SIL = 0): tiles rn * run,
    // rn * run + 1, ..  Interleaved runs (SIL = 1): tiles rn, rn + nruns, rn + 2 nruns, ..; at any moment the
    // workgroups are then on NEIGHBOURING tiles, so what is in flight chip-wide is one compact window of C moving
    // through the tensor instead of nruns windows scattered over it (a bare read-modify-write of the 72^4 fp64
    // output in these tiles: 4 % faster; the kernels with the X panel resident gain 2 to 6 %, the fp32 shapes with
    // the Y panel resident lose 5 %, hence an option).
    constexpr bool SIL = Cfg::SIL != 0;
    const unsigned step = SIL ? s.nruns : 1u;
    unsigned st = SIL ? rn : rn * s.run;
    const unsigned ntiles = SIL ? (s.nstr - rn + s.nruns - 1) / s.nruns : ((s.nstr - st) < s.run ? (s.nstr - st) : s.run);
    // origin of a tile along one side: offset inside C and inside that side's operand
    auto side_origin = [&](auto side_t, unsigned t, int64_t& oc, int64_t& oo) {
        constexpr int SIDE = decltype(side_t)::value;
        oc = 0; oo = 0;
#pragma unroll
        for (int i = 0; i < (SIDE == 0 ? Cfg::NX : Cfg::NY); i++) {
            const int id = SIDE == 0 ? Cfg::x_id(i) : Cfg::y_id(i);
            const int tile = SIDE == 0 ? Cfg::x_tile(i) : Cfg::y_tile(i);
            const unsigned nb = (unsigned)d.nblk[id];
            const int o = (int)(t % nb) * tile;
            t /= nb;
            oc += (int64_t)o * d.sC[id];
            oo += (int64_t)o * Operand<Cfg, SIDE>::stride(d, id);
        }
    };
    const std::integral_constant<int, RES> res_side;
    const std::integral_constant<int, 1 - RES> str_side;
    int64_t baseCr, baseR;
    side_origin(res_side, rt, baseCr, baseR);

    // ---- offsets of this lane's accumulator elements from a tile origin: the same for every tile
    int cx[TX][SWP ? NREG : 1];
    int cy[TY][SWP ? 1 : NREG];
    c_tile_offsets<Cfg, true, SWP, false>(lane, wx, wy, nullptr, d, cx, cy);
    // The sum of the two parts is formed at every use from an opaque copy: kept across the tile loop it
    // would cost one register per accumulator element on top of the two register tiles.
    auto c_off = [&](int ti, int tj, int r) -> unsigned {
        int part = cy[ti][SWP ? 0 : r];
        asm volatile("" : "+v"(part));
        return (unsigned)(cx[tj][SWP ? r : 0] + part) * (unsigned)sizeof(T);
    };
    // padded tiles: the accumulator elements that fall into the padding have no place in C
    auto c_ok = [&](int ti, int tj, int r) -> bool { return !PADDED || (cx[tj][SWP ? r : 0] >= 0 && cy[ti][SWP ? 0 : r] >= 0); };

    // CD: how many tiles ahead C is read.  cpre[t % CD] holds the C tile that tile t's first K block starts from;
    // once that block has taken it, the same registers receive the C tile of tile t + CD.  With CD = 2 a C read has
    // a whole tile time plus its own to arrive before anything waits for it.
    constexpr int CD = Cfg::SCD;
    static_assert(CD == 1 || CD == 2, "C is read one or two tiles ahead");
    Acc cpre_all[CD][TY][TX];
    Acc acc[TY][TX];
    auto c_read = [&](auto par_t, const T* base, int ti, int tj) {
        Acc (&cpre)[TY][TX] = cpre_all[decltype(par_t)::value];
        if (TC_STREAM_ABLATE & 1) {
#pragma unroll
            for (int r = 0; r < NREG; r++) cpre[ti][tj][r] = (T)0;
        } else if (VEC4) {
#pragma unroll
            for (int g = 0; g < NREG / 4; g++) {
                T4 v = {(T)0, (T)0, (T)0, (T)0};
                if (c_ok(ti, tj, 4 * g)) v = c_load<NT_LD>((const T4*)((const char*)base + c_off(ti, tj, 4 * g)));
#pragma unroll
                for (int e = 0; e < 4; e++) cpre[ti][tj][4 * g + e] = v[e];
            }
        } else {
#pragma unroll
            for (int r = 0; r < NREG; r++) {
                T v = (T)0;
                if (c_ok(ti, tj, r)) v = c_load<NT_LD>((const T*)((const char*)base + c_off(ti, tj, r)));
                cpre[ti][tj][r] = v;
            }
        }
    };
    auto c_write = [&](T* base, int ti, int tj) {
        if (TC_STREAM_ABLATE & 2) {
            // keep the accumulators alive without a store
#pragma unroll
            for (int r = 0; r < NREG; r++) asm volatile("" :: "v"(acc[ti][tj][r]));
        } else if (VEC4) {
#pragma unroll
            for (int g = 0; g < NREG / 4; g++) {
                T4 v;
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = acc[ti][tj][4 * g + e];
                if (c_ok(ti, tj, 4 * g)) c_store<NT_ST>(v, (T4*)((char*)base + c_off(ti, tj, 4 * g)));
            }
        } else {
#pragma unroll
            for (int r = 0; r < NREG; r++)
                if (c_ok(ti, tj, r)) c_store<NT_ST>(acc[ti][tj][r], (T*)((char*)base + c_off(ti, tj, r)));
        }
    };

    // ---- prologue: the resident panel, the first PD slices of the stream, the first C tile
    if (PADDED) {
        // the staging never writes the padding rows and columns of the LDS buffers: clear everything once
        for (int i = tid; i < NKB * LDS_R + 2 * LDS_S; i += NT) lds_r[i] = (T)0;
        __syncthreads();
    }
    int64_t oc, oo;
    side_origin(str_side, st, oc, oo);
    T* Cb = C + uniform64(baseCr + oc);
    T* C1 = Cb;                   // CD == 2: the tile after the current one
    if (CD == 2 && ntiles > 1) {
        int64_t oc1, oo1;
        side_origin(str_side, st + step, oc1, oo1);
        C1 = C + uniform64(baseCr + oc1);
    }
    const T* const Rsrc = (RES == 0 ? X : Y) + uniform64(baseR);
    const T* const Ssrc = (RES == 0 ? Y : X);
    const T* Sb = Ssrc + uniform64(oo);
    KWalk<Cfg, 1 - RES> ks;       // the K block of the next slice to request
    ks.reset();
    T rs[PD][SLOTS_S];
    auto s_load = [&](T (&reg)[SLOTS_S], const T* src) {
        if (TC_STREAM_ABLATE & 4) {
#pragma unroll
            for (int i = 0; i < SLOTS_S; i++) reg[i] = (T)(tid + i);
        } else {
            slice_load<Cfg, OS, true, true>(reg, src, d, nullptr, tid);
        }
    };
    {
        // The panel in groups of RG slices, all loads of a group in flight together (the accumulators
        // are not live yet, so the registers are there).  The requests for the first slices of the stream
        // and for the first C tile follow the last group's: loads return in order, and the panel and the
        // slices come from L2 while C comes from HBM.
        constexpr int RREG = SLOTS_R * (int)sizeof(T) / 4;
        // SOV: only the panel's FIRST slice is loaded here; slice j + 1 is requested during trip j of the first
        // tile, which needs no more than slice j of the panel.  The gather of a panel whose memory order does not
        // match the tile (16-byte pieces of distinct lines) is bound by the L2, not by HBM: behind the first tile's
        // C traffic it costs nothing, in front of it the whole chip waits.
        constexpr int NPRO = SOV ? 1 : NKB;
        constexpr int RG = (NPRO * RREG <= 96) ? NPRO : (96 / RREG < 1 ? 1 : 96 / RREG);
        constexpr int NG = (NPRO + RG - 1) / RG;
        KWalk<Cfg, RES> kr;
        kr.reset();
        static_for<NG>([&](auto gt) {
            constexpr int j0 = decltype(gt)::value * RG;
            constexpr int n = (NPRO - j0) < RG ? (NPRO - j0) : RG;
            T rr[n][SLOTS_R];
            static_for<n>([&](auto it) {
                slice_load<Cfg, OR, true, true>(rr[decltype(it)::value], Rsrc + uniform64(kr.offset(d)), d, nullptr, tid);
                kr.next(d);
            });
            if constexpr (decltype(gt)::value == NG - 1) {
                static_for<PD>([&](auto sg) {
                    s_load(rs[decltype(sg)::value], Sb + uniform64(ks.offset(d)));
                    ks.next(d);
                });
#pragma unroll
                for (int ti = 0; ti < TY; ti++)
#pragma unroll
                    for (int tj = 0; tj < TX; tj++) c_read(std::integral_constant<int, 0>(), Cb, ti, tj);
                if (CD == 2) {            // (a run of a single tile reads its own C a second time: no branch here)
#pragma unroll
                    for (int ti = 0; ti < TY; ti++)
#pragma unroll
                        for (int tj = 0; tj < TX; tj++) c_read(std::integral_constant<int, CD - 1>(), C1, ti, tj);
                }
            }
            static_for<n>([&](auto it) {
                slice_store<Cfg, OR, NEG_R, VR>(rr[decltype(it)::value], lds_r + (j0 + decltype(it)::value) * LDS_R, d, tid);
            });
        });
    }
    slice_store<Cfg, OS, NEG_S, VS>(rs[0], lds_s, d, tid);
    __syncthreads();
    int sbuf = 0;           // the LDS stage that holds the current tile's slice 0

    // ---- one output tile: NKB trips.  Slice j of the tile is in LDS stage (sbuf + j) % 2 when trip j
    // starts; register stage j % PD is free then and takes the request for slice j + PD of the stream.
    KWalk<Cfg, RES> kp;           // SOV: the panel slice to request next (slice 0 came with the prologue)
    kp.reset();
    kp.next(d);
    // PAR = t % CD; HAS_NEXT: tile t + 1 exists (its slices are requested here); HAS_FAR: tile t + CD exists (its C
    // is read here); FIRST: tile 0
    auto tile = [&](auto par_t, auto has_next_t, auto has_far_t, auto first_t) {
        constexpr bool HAS_NEXT = decltype(has_next_t)::value;
        constexpr bool HAS_FAR = decltype(has_far_t)::value;
        constexpr bool FIRST = SOV && decltype(first_t)::value;
        Acc (&cpre)[TY][TX] = cpre_all[decltype(par_t)::value];
        T* Cf = Cb;
        const T* Sn = Sb;
        if (HAS_NEXT) {
            side_origin(str_side, st + step, oc, oo);
            Sn = Ssrc + uniform64(oo);
            if (CD == 1) Cf = C + uniform64(baseCr + oc);
        }
        if (CD == 2 && HAS_FAR) {
            int64_t ocf, oof;
            side_origin(str_side, st + 2 * step, ocf, oof);
            Cf = C + uniform64(baseCr + ocf);
        }
        static_for<NKB>([&](auto jt) {
            constexpr int j = decltype(jt)::value;
            constexpr int S = j % PD;
            // first tile, SOV: the panel's slice j + 1, requested before anything else of this trip so that the
            // wait for it at the end of the trip (loads return in order) leaves the younger requests in flight
            constexpr bool PANEL = FIRST && (j + 1 < NKB);
            T rp[PANEL ? SLOTS_R : 1];
            if constexpr (PANEL) {
                slice_load<Cfg, OR, true, true>(rp, Rsrc + uniform64(kp.offset(d)), d, nullptr, tid);
                kp.next(d);
            }
            if constexpr (j + PD < NKB) {
                s_load(rs[S], Sb + uniform64(ks.offset(d)));
                ks.next(d);
            } else if constexpr (HAS_NEXT) {
                s_load(rs[S], Sn + uniform64(ks.offset(d)));
                ks.next(d);
            }
            // the C of tile t + CD, spread over trips 1 .. NKB-1: trip 0's first matrix step still reads these registers.
            // (Requesting it earlier -- from trip 0 on, or all of it right after that first step -- measured 3 to 10 %
            // slower on the 72^5 fp64 shape, all of it in the last trip 4 % slower.)
            if constexpr (HAS_FAR && j >= 1) {
                static_for<TY * TX>([&](auto ct) {
                    constexpr int c = decltype(ct)::value;
                    if constexpr (1 + (c * (NKB - 1)) / (TY * TX) == j) c_read(par_t, Cf, c / TX, c % TX);
                });
            }
            const T* lr = lds_r + j * LDS_R;
            const T* ls = lds_s + (NKB % 2 == 0 ? (j & 1) : (sbuf ^ (j & 1))) * LDS_S;
            const T* lx = RES == 0 ? lr : ls;
            const T* ly = RES == 0 ? ls : lr;
#pragma unroll
            for (int k4 = 0; k4 < Cfg::BKP / KSTEP; k4++) {
                const int kk = k4 * KSTEP + lane / MT;
                T a[TY], b[TX];
#pragma unroll
                for (int ti = 0; ti < TY; ti++) a[ti] = ly[lds_addr<OY>(kk, (wy * TY + ti) * MT + lane % MT)];
#pragma unroll
                for (int tj = 0; tj < TX; tj++) b[tj] = lx[lds_addr<OX>(kk, (wx * TX + tj) * MT + lane % MT)];
#pragma unroll
                for (int ti = 0; ti < TY; ti++)
#pragma unroll
                    for (int tj = 0; tj < TX; tj++) {
                        const Acc from = (j == 0 && k4 == 0) ? cpre[ti][tj] : acc[ti][tj];
                        if (TC_STREAM_ABLATE & 8) { asm volatile("" :: "v"(a[ti]), "v"(b[tj])); acc[ti][tj] = from; }
                        else acc[ti][tj] = SWP ? MM::mma(b[tj], a[ti], from) : MM::mma(a[ti], b[tj], from);
                    }
            }
            if constexpr (PANEL) slice_store<Cfg, OR, NEG_R, VR>(rp, lds_r + (j + 1) * LDS_R, d, tid);
            if constexpr (j + 1 < NKB || HAS_NEXT) {
                T* dst = lds_s + (NKB % 2 == 0 ? ((j + 1) & 1) : (sbuf ^ ((j + 1) & 1))) * LDS_S;
                slice_store<Cfg, OS, NEG_S, VS>(rs[(j + 1) % PD], dst, d, tid);
                __syncthreads();
            }
        });
#pragma unroll
        for (int ti = 0; ti < TY; ti++)
#pragma unroll
            for (int tj = 0; tj < TX; tj++) c_write(Cb, ti, tj);
        if (HAS_NEXT) {
            Cb = (CD == 1) ? Cf : C1;
            C1 = Cf;
            Sb = Sn; st += step;
            if (NKB % 2) sbuf ^= 1;
        }
    };

    // The first tile is a copy of its own so that the tiles inside the loop all start from the same
    // history of loads and stores in flight; the last tile requests nothing further.
    const std::integral_constant<int, 0> P0;
    const std::integral_constant<int, CD - 1> P1;       // parity 1 (CD == 1: the one register tile)
    const std::true_type yes;
    const std::false_type no;
    if (CD == 1) {
        if (ntiles > 1) {
            if (SOV) tile(P0, yes, yes, yes); else tile(P0, yes, yes, no);
            for (unsigned t = 2; t < ntiles; t++) tile(P0, yes, yes, no);
            tile(P0, no, no, no);
        } else {
            if (SOV) tile(P0, no, no, yes); else tile(P0, no, no, no);
        }
    } else {
        // tile 0, then pairs (odd, even) while at least four tiles remain, then the last one to three tiles
        unsigned left = ntiles;
        if (left >= 3)      { if (SOV) tile(P0, yes, yes, yes); else tile(P0, yes, yes, no); }
        else if (left == 2) { if (SOV) tile(P0, yes, no, yes); else tile(P0, yes, no, no); }
        else                { if (SOV) tile(P0, no, no, yes); else tile(P0, no, no, no); }
        left--;
        for (; left >= 4; left -= 2) { tile(P1, yes, yes, no); tile(P0, yes, yes, no); }
        if (left == 3)      { tile(P1, yes, yes, no); tile(P0, yes, no, no); tile(P1, no, no, no); }
        else if (left == 2) { tile(P1, yes, no, no); tile(P0, no, no, no); }
        else if (left == 1) { tile(P1, no, no, no); }
    }
}

}  // namespace cogent
