// Panel-resident streaming kernel: a second shape of the contraction kernel for outputs that are
// much larger than the inputs and have a short contracted range (a handful of K blocks).
//
// tc_mfma_kernel gives every output tile a workgroup of its own.  With few K blocks per tile that
// workgroup spends most of its life in latencies that nothing overlaps: the C tile read, the first
// slices, the write-back.  Here a workgroup is persistent over a RUN of output tiles that share
// their X-side tile:
//
//   * the X panel (the X tile over the whole contracted range, NKB slices) is loaded into LDS once
//     per workgroup and stays;
//   * the Y slices of the tiles of the run pass through a two-stage LDS buffer as ONE stream, PD
//     slices requested ahead in registers, across tile boundaries: the first slices of the next tile
//     are in flight while the last K blocks of the current tile are contracted;
//   * the C tile of the NEXT output tile is read piece by piece (one MFMA tile per piece) during the
//     K blocks of the current one, into registers that the first K block has already consumed as the
//     matrix instruction's addend, so that a C read has a whole tile time to arrive and no load burst
//     stands in front of the slice loads in the in-order return path;
//   * the finished tile is stored while the next one is already being contracted.
//
// The K-block count NKB is a compile-time constant (the emitter takes it from the representative
// extents of the expression): every trip of a tile is a copy of its own, which is what lets the
// compiler count the loads in flight exactly.  The launcher uses this kernel only when the run-time
// extents give that K-block count and every tile is full; otherwise the call goes to tc_mfma_kernel.
#pragma once
#include "tc_kernel.hpp"

namespace cogent {

struct TcStreamDims {
    unsigned nyt;      // Y-side tiles of the whole output
    unsigned run;      // consecutive Y-side tiles handled by one workgroup
    unsigned nruns;    // workgroups per X-side tile
};

extern __shared__ __attribute__((aligned(16))) unsigned char tc_stream_lds[];


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
    constexpr int MT = MM::MT, NREG = MM::NREG, KSTEP = MM::KSTEP;
    constexpr int TX = Cfg::TX, TY = Cfg::TY, NT = Cfg::NT;
    constexpr int NKB = Cfg::STREAM, PD = Cfg::SPD;
    static_assert(NKB >= 2 && PD >= 1 && PD <= NKB && NKB % PD == 0, "prefetch depth must divide the K-block count");
    static_assert(Cfg::BKP == Cfg::BK && Cfg::BXP == Cfg::BX && Cfg::BYP == Cfg::BY, "streaming kernel: unpadded tiles only");
    constexpr int SLOTS_X = (Cfg::BK * Cfg::BX + NT - 1) / NT;
    constexpr int SLOTS_Y = (Cfg::BK * Cfg::BY + NT - 1) / NT;
    constexpr int LDS_X = lds_elems<OX, Cfg::BKP>();
    constexpr int LDS_Y = lds_elems<OY, Cfg::BKP>();
    constexpr bool VEC4 = SWP;
    constexpr bool NT_LD = (Cfg::NTC & 1) != 0, NT_ST = (Cfg::NTC & 2) != 0;
    typedef T T4 __attribute__((ext_vector_type(4)));

    T* const lds_x = (T*)tc_stream_lds;            // NKB slices of the X tile
    T* const lds_y = lds_x + NKB * LDS_X;          // two stages of one Y slice

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wx = wave % Cfg::WX;
    const int wy = wave / Cfg::WX;

    // ---- this workgroup's X tile and its run of Y tiles
    // Workgroups go to the 8 XCDs round-robin and every XCD has its own L2: give XCD x a contiguous
    // range of (X tile, run) pairs, X tiles fastest, so that tiles that are neighbours along C's fastest
    // index -- and share the cache lines their rows end in -- are worked on at the same time on one L2.
    unsigned vb;
    {
        const unsigned n = gridDim.x, xcd = blockIdx.x % 8u, idx = blockIdx.x / 8u;
        const unsigned q = n / 8u, r = n % 8u;
        vb = xcd * q + (xcd < r ? xcd : r) + idx;
    }
    const unsigned xt = vb % d.nxt, rn = vb / d.nxt;
    unsigned yt = rn * s.run;
    const unsigned ntiles = (s.nyt - yt) < s.run ? (s.nyt - yt) : s.run;
    int64_t baseCx = 0, baseX = 0;
    {
        unsigned b = xt;
#pragma unroll
        for (int i = 0; i < Cfg::NX; i++) {
            const int id = Cfg::x_id(i);
            const unsigned nb = (unsigned)d.nblk[id];
            const int o = (int)(b % nb) * Cfg::x_tile(i);
            b /= nb;
            baseCx += (int64_t)o * d.sC[id];
            baseX += (int64_t)o * d.sX[id];
        }
    }
    auto y_origin = [&](unsigned t, int64_t& oc, int64_t& oy) {
        oc = 0; oy = 0;
#pragma unroll
        for (int i = 0; i < Cfg::NY; i++) {
            const int id = Cfg::y_id(i);
            const unsigned nb = (unsigned)d.nblk[id];
            const int o = (int)(t % nb) * Cfg::y_tile(i);
            t /= nb;
            oc += (int64_t)o * d.sC[id];
            oy += (int64_t)o * d.sY[id];
        }
    };

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

    Acc cpre[TY][TX];       // the C tile that the next first K block starts from
    Acc acc[TY][TX];
    auto c_read = [&](const T* base, int ti, int tj) {
        if (VEC4) {
#pragma unroll
            for (int g = 0; g < NREG / 4; g++) {
                const T4 v = c_load<NT_LD>((const T4*)((const char*)base + c_off(ti, tj, 4 * g)));
#pragma unroll
                for (int e = 0; e < 4; e++) cpre[ti][tj][4 * g + e] = v[e];
            }
        } else {
#pragma unroll
            for (int r = 0; r < NREG; r++) cpre[ti][tj][r] = c_load<NT_LD>((const T*)((const char*)base + c_off(ti, tj, r)));
        }
    };
    auto c_write = [&](T* base, int ti, int tj) {
        if (VEC4) {
#pragma unroll
            for (int g = 0; g < NREG / 4; g++) {
                T4 v;
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = acc[ti][tj][4 * g + e];
                c_store<NT_ST>(v, (T4*)((char*)base + c_off(ti, tj, 4 * g)));
            }
        } else {
#pragma unroll
            for (int r = 0; r < NREG; r++) c_store<NT_ST>(acc[ti][tj][r], (T*)((char*)base + c_off(ti, tj, r)));
        }
    };

    // ---- prologue: first C tile, the X panel, the first PD slices of the Y stream
    int64_t oc, oy;
    y_origin(yt, oc, oy);
    T* Cb = C + uniform64(baseCx + oc);
    const T* Yb = Y + uniform64(oy);
    const T* Xb = X + uniform64(baseX);
    KWalk<Cfg, 1> ky;       // the K block of the next slice to request
    ky.reset();
    T ry[PD][SLOTS_Y];
    {
        // The panel in groups of XG slices, all loads of a group in flight together (the accumulators
        // are not live yet, so the registers are there).  The requests for the first Y slices and for
        // the first C tile follow the last group's: loads return in order, and the panel and the slices
        // come from L2 while C comes from HBM.
        constexpr int XREG = SLOTS_X * (int)sizeof(T) / 4;
        constexpr int XG = (NKB * XREG <= 96) ? NKB : (96 / XREG < 1 ? 1 : 96 / XREG);
        constexpr int NG = (NKB + XG - 1) / XG;
        KWalk<Cfg, 0> kx;
        kx.reset();
        static_for<NG>([&](auto gt) {
            constexpr int j0 = decltype(gt)::value * XG;
            constexpr int n = (NKB - j0) < XG ? (NKB - j0) : XG;
            T rx[n][SLOTS_X];
            static_for<n>([&](auto it) {
                slice_load<Cfg, OX, true, true>(rx[decltype(it)::value], Xb + uniform64(kx.offset(d)), d, nullptr, tid);
                kx.next(d);
            });
            if constexpr (decltype(gt)::value == NG - 1) {
                static_for<PD>([&](auto st) {
                    slice_load<Cfg, OY, true, true>(ry[decltype(st)::value], Yb + uniform64(ky.offset(d)), d, nullptr, tid);
                    ky.next(d);
                });
#pragma unroll
                for (int ti = 0; ti < TY; ti++)
#pragma unroll
                    for (int tj = 0; tj < TX; tj++) c_read(Cb, ti, tj);
            }
            static_for<n>([&](auto it) {
                slice_store<Cfg, OX, false>(rx[decltype(it)::value], lds_x + (j0 + decltype(it)::value) * LDS_X, d, tid);
            });
        });
    }
    slice_store<Cfg, OY, (Cfg::SIGN < 0)>(ry[0], lds_y, d, tid);
    __syncthreads();
    int ybuf = 0;           // the LDS stage that holds the current tile's slice 0

    // ---- one output tile: NKB trips.  Slice j of the tile is in LDS stage (ybuf + j) % 2 when trip j
    // starts; register stage j % PD is free then and takes the request for slice j + PD of the stream.
    auto tile = [&](auto has_next_t) {
        constexpr bool HAS_NEXT = decltype(has_next_t)::value;
        T* Cn = Cb;
        const T* Yn = Yb;
        if (HAS_NEXT) {
            y_origin(yt + 1, oc, oy);
            Cn = C + uniform64(baseCx + oc);
            Yn = Y + uniform64(oy);
        }
        static_for<NKB>([&](auto jt) {
            constexpr int j = decltype(jt)::value;
            constexpr int S = j % PD;
            if constexpr (j + PD < NKB) {
                slice_load<Cfg, OY, true, true>(ry[S], Yb + uniform64(ky.offset(d)), d, nullptr, tid);
                ky.next(d);
            } else if constexpr (HAS_NEXT) {
                slice_load<Cfg, OY, true, true>(ry[S], Yn + uniform64(ky.offset(d)), d, nullptr, tid);
                ky.next(d);
            }
            // the next tile's C, spread over trips 1 .. NKB-1 (trip 0 still reads these registers)
            if constexpr (HAS_NEXT && j >= 1) {
                static_for<TY * TX>([&](auto ct) {
                    constexpr int c = decltype(ct)::value;
                    if constexpr (1 + (c * (NKB - 1)) / (TY * TX) == j) c_read(Cn, c / TX, c % TX);
                });
            }
            const T* lx = lds_x + j * LDS_X;
            const T* ly = lds_y + (NKB % 2 == 0 ? (j & 1) : (ybuf ^ (j & 1))) * LDS_Y;
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
                        acc[ti][tj] = SWP ? MM::mma(b[tj], a[ti], from) : MM::mma(a[ti], b[tj], from);
                    }
            }
            if constexpr (j + 1 < NKB || HAS_NEXT) {
                T* dst = lds_y + (NKB % 2 == 0 ? ((j + 1) & 1) : (ybuf ^ ((j + 1) & 1))) * LDS_Y;
                slice_store<Cfg, OY, (Cfg::SIGN < 0)>(ry[(j + 1) % PD], dst, d, tid);
                __syncthreads();
            }
        });
#pragma unroll
        for (int ti = 0; ti < TY; ti++)
#pragma unroll
            for (int tj = 0; tj < TX; tj++) c_write(Cb, ti, tj);
        if (HAS_NEXT) {
            Cb = Cn; Yb = Yn; yt++;
            if (NKB % 2) ybuf ^= 1;
        }
    };

    // The first tile is a copy of its own so that the tiles inside the loop all start from the same
    // history of loads and stores in flight; the last tile requests nothing further.
    if (ntiles > 1) {
        tile(std::true_type());
        for (unsigned t = 2; t < ntiles; t++) tile(std::true_type());
    }
    tile(std::false_type());
}

}  // namespace cogent
