// Host-side launch wrapper instantiated once per emitted expression.
//
// Takes the place of the host caller the reference generator writes out
// (`sd_t_d2_fusion`, cogent/src/codes/kernels/tc_interface.py:10-101: grid
// size, strides, the four-way full/partial kernel choice).  Differences, on
// purpose: the pointers are DEVICE pointers and nothing is allocated or copied
// here; every argument is validated and a status code is returned instead of
// running unchecked; C is read-modify-written.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <atomic>
#include "tc_kernel.hpp"
#include "tc_stream.hpp"

namespace cogent {

enum TcStatus {
    TC_OK = 0,
    TC_ERR_NULL_POINTER = 1,
    TC_ERR_NEGATIVE_EXTENT = 2,
    TC_ERR_TOO_LARGE = 3,      // a tensor has 2^31 or more elements, or the grid does not fit
    TC_ERR_LAUNCH = 4,         // the HIP runtime refused the launch
    TC_ERR_BAD_VARIANT = 5,
    TC_ERR_ALLOC = 6,          // host-pointer shim, or the stream-ordered buffer of a repacked input
};

inline char* tc_error_buffer() { static thread_local char buf[256] = ""; return buf; }
inline int tc_fail(int code, const char* msg)
{
    snprintf(tc_error_buffer(), 256, "%s", msg);
    return code;
}
// The runtime's "last error" is sticky per thread and may have been left by an unrelated earlier
// call (an event query that was not ready, for instance): clear it before a launch, read it after.
inline void tc_clear_hip_error() { (void)hipGetLastError(); }
inline int tc_check_launch(const char* what)
{
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return TC_OK;
    snprintf(tc_error_buffer(), 256, "%s: %s", what, hipGetErrorString(e));
    return TC_ERR_LAUNCH;
}

enum TcVariant { TC_VARIANT_AUTO = 0, TC_VARIANT_PLAIN = 1, TC_VARIANT_TILED = 2, TC_VARIANT_VALU = 3 };
// The VALU streaming kernel is never taken by TC_VARIANT_AUTO: measured at contracted extents 1, 2 and 3 (which do not
// fill the 4-deep step of the fp64 / fp32 matrix instructions) it is 45 to 85 % SLOWER than the tiled kernel with the
// slices zero-padded to one step (72^4 outer product 131 vs 77 us, 16^6 fp64 with 2 terms 70 vs 48 us, 16^6 fp32 with
// 3 terms 51 vs 28 us): its per-element gathers of the inputs cost more issue slots than a padded matrix step.

// Which kernel the last call of this thread launched (0: none yet, or the call returned before a launch).
enum TcKernelKind { TC_KERNEL_NONE = 0, TC_KERNEL_PLAIN = 1, TC_KERNEL_TILED = 2, TC_KERNEL_STREAM = 3, TC_KERNEL_VALU = 4 };
inline int& tc_last_kernel() { static thread_local int kind = TC_KERNEL_NONE; return kind; }

template <class Cfg, bool ONE_KB, bool SWP>
inline void tc_launch_full_partial(bool ext_full, bool int_full, dim3 g, dim3 b, hipStream_t stream,
                                   typename Cfg::T* c, const typename Cfg::T* x, const typename Cfg::T* y, const TcDims& d)
{
    constexpr size_t lds = tc_mfma_dynamic_lds<Cfg, ONE_KB>();
    if (lds > 0) {
        const void* fn = ext_full && int_full ? (const void*)&tc_mfma_kernel<Cfg, true, true, ONE_KB, SWP>
                       : ext_full             ? (const void*)&tc_mfma_kernel<Cfg, true, false, ONE_KB, SWP>
                       : int_full             ? (const void*)&tc_mfma_kernel<Cfg, false, true, ONE_KB, SWP>
                                              : (const void*)&tc_mfma_kernel<Cfg, false, false, ONE_KB, SWP>;
        // once per device and variant: raise the kernel's dynamic-LDS limit (not a stream operation).  Two host
        // threads may both find the flag clear and both set the same attribute; the flag itself is atomic.
        static std::atomic<bool> configured[64][4];
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return;                  // the launch check reports it
        std::atomic<bool>& done = configured[dev][(ext_full ? 2 : 0) + (int_full ? 1 : 0)];
        if (!done.load(std::memory_order_acquire)) {
            if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) return;
            done.store(true, std::memory_order_release);
        }
    }
    if (ext_full && int_full)   hipLaunchKernelGGL((tc_mfma_kernel<Cfg, true, true, ONE_KB, SWP>),   g, b, lds, stream, c, x, y, d);
    else if (ext_full)          hipLaunchKernelGGL((tc_mfma_kernel<Cfg, true, false, ONE_KB, SWP>),  g, b, lds, stream, c, x, y, d);
    else if (int_full)          hipLaunchKernelGGL((tc_mfma_kernel<Cfg, false, true, ONE_KB, SWP>),  g, b, lds, stream, c, x, y, d);
    else                        hipLaunchKernelGGL((tc_mfma_kernel<Cfg, false, false, ONE_KB, SWP>), g, b, lds, stream, c, x, y, d);
}

template <class Cfg>
inline void tc_launch_variant(bool one_kb, bool ext_full, bool int_full, bool swp, dim3 g, dim3 b, hipStream_t stream,
                              typename Cfg::T* c, const typename Cfg::T* x, const typename Cfg::T* y, const TcDims& d)
{
    if constexpr (Cfg::SWAP != 0) {
        if (swp) {
            if (one_kb) tc_launch_full_partial<Cfg, true, true>(ext_full, int_full, g, b, stream, c, x, y, d);
            else        tc_launch_full_partial<Cfg, false, true>(ext_full, int_full, g, b, stream, c, x, y, d);
            return;
        }
    }
    if (one_kb) tc_launch_full_partial<Cfg, true, false>(ext_full, int_full, g, b, stream, c, x, y, d);
    else        tc_launch_full_partial<Cfg, false, false>(ext_full, int_full, g, b, stream, c, x, y, d);
}

// The panel-resident streaming kernel, when the object carries one (Cfg::STREAM = its K-block count)
// and this call's extents are multiples of the tiles and give exactly that many K blocks.  Returns false
// when the call has to go to the per-tile kernel instead.  The grid is sized so that all workgroups are
// resident at once: every tile of the resident side gets as many runs of consecutive tiles of the other
// side as fill the CUs about once.
template <class Cfg>
inline bool tc_stream_launch(bool ext_div, bool int_div, int64_t nkb, bool swp, hipStream_t stream,
                             typename Cfg::T* c, const typename Cfg::T* x, const typename Cfg::T* y, const TcDims& d)
{
    if constexpr (Cfg::STREAM > 0) {
        typedef typename Cfg::T T;
        if (!ext_div || !int_div || nkb != Cfg::STREAM) return false;
        constexpr size_t lds_bytes = sizeof(T) * ((size_t)Cfg::STREAM * lds_elems<Operand<Cfg, Cfg::SRES>, Cfg::BKP>() +
                                                  2 * (size_t)lds_elems<Operand<Cfg, 1 - Cfg::SRES>, Cfg::BKP>());
        static_assert(lds_bytes <= 160 * 1024, "the resident panel does not fit the LDS");
        static_assert(Cfg::SK == 1, "the streaming kernel gives every output tile to one workgroup: no split K");
        // per device: its CU count, and the kernel's dynamic-LDS limit raised once (neither is a stream
        // operation, so a call that is being captured into a graph may do them)
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void)hipGetLastError(); return false; }
        static std::atomic<int> n_cu[64];
        static std::atomic<bool> configured[64][2];
        if (n_cu[dev].load(std::memory_order_acquire) == 0) {
            int v = 0;
            if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v < 1) {
                (void)hipGetLastError();
                return false;
            }
            n_cu[dev].store(v, std::memory_order_release);
        }
        if (!configured[dev][swp ? 1 : 0].load(std::memory_order_acquire)) {
            const void* fn = swp ? (const void*)&tc_stream_kernel<Cfg, Cfg::SWAP != 0> : (const void*)&tc_stream_kernel<Cfg, false>;
            if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess) {
                (void)hipGetLastError();
                return false;
            }
            configured[dev][swp ? 1 : 0].store(true, std::memory_order_release);
        }
        const int by_lds = (int)((160 * 1024) / lds_bytes), by_regs = (Cfg::SMW * 4 * 64) / Cfg::NT;
        const int64_t slots = (int64_t)n_cu[dev].load(std::memory_order_relaxed) * (by_lds < by_regs ? by_lds : (by_regs < 1 ? 1 : by_regs));
        TcStreamDims s;
        // tiles along the Y side from the tile counts themselves (d.nblocks may carry other grid factors)
        unsigned nyt = 1;
        for (int i = 0; i < Cfg::NY; i++) nyt *= (unsigned)d.nblk[Cfg::y_id(i)];
        s.nres = Cfg::SRES == 0 ? d.nxt : nyt;
        s.nstr = Cfg::SRES == 0 ? nyt : d.nxt;
        int64_t runs = slots / s.nres;                       // runs per resident tile: as many as keep the whole grid resident at once
        if (runs < 1) runs = 1;
        if (runs > s.nstr) runs = s.nstr;
        s.run = (unsigned)((s.nstr + runs - 1) / runs);
        s.nruns = (s.nstr + s.run - 1) / s.run;
        const dim3 g(s.nres * s.nruns), b(Cfg::NT);
        if (swp) hipLaunchKernelGGL((tc_stream_kernel<Cfg, Cfg::SWAP != 0>), g, b, lds_bytes, stream, c, x, y, d, s);
        else     hipLaunchKernelGGL((tc_stream_kernel<Cfg, false>), g, b, lds_bytes, stream, c, x, y, d, s);
        return true;
    } else {
        (void)ext_div; (void)int_div; (void)nkb; (void)swp; (void)stream; (void)c; (void)x; (void)y; (void)d;
        return false;
    }
}

// sizes[] holds one extent per index id: output indices in output order, then
// the contracted indices in sum() order -- the order of the entry point's
// `int size_*` parameters (cogent/src/codes/kernels/tc_interface.py:1459-1492).
//
// no_alloc: the call must not allocate.  A mapping with repacked inputs then puts the copies into the caller's
// workspace `ext_ws` of `ext_ws_bytes` bytes (the emitted object's static device array) instead of a
// stream-ordered allocation, and refuses inputs that do not fit it.
template <class Cfg>
int tc_run(const int* sizes, void* C, const void* A, const void* B, hipStream_t stream, int variant,
           void* ext_ws = nullptr, size_t ext_ws_bytes = 0, bool no_alloc = false)
{
    typedef typename Cfg::T T;
    tc_error_buffer()[0] = 0;
    tc_last_kernel() = TC_KERNEL_NONE;
    if (variant < 0 || variant > 3) return tc_fail(TC_ERR_BAD_VARIANT, "unknown kernel variant");
    for (int i = 0; i < Cfg::NIDX; i++)
        if (sizes[i] < 0) return tc_fail(TC_ERR_NEGATIVE_EXTENT, "negative extent");
    // empty output or empty sum: C is left as it is
    for (int i = 0; i < Cfg::NIDX; i++)
        if (sizes[i] == 0) return TC_OK;
    if (!C || !A || !B) return tc_fail(TC_ERR_NULL_POINTER, "null tensor pointer");

    // element strides: dense, first listed index fastest
    int64_t sC[TC_MAXI] = {0}, sA[TC_MAXI] = {0}, sB[TC_MAXI] = {0};
    int64_t nC = 1, nA = 1, nB = 1;
    for (int j = 0; j < Cfg::CR; j++) { sC[Cfg::c_id(j)] = nC; nC *= sizes[Cfg::c_id(j)]; }
    for (int j = 0; j < Cfg::AR; j++) { sA[Cfg::a_id(j)] = nA; nA *= sizes[Cfg::a_id(j)]; }
    for (int j = 0; j < Cfg::BR; j++) { sB[Cfg::b_id(j)] = nB; nB *= sizes[Cfg::b_id(j)]; }
    const int64_t lim = ((int64_t)1 << 31) - 1;
    if (nC > lim || nA > lim || nB > lim) return tc_fail(TC_ERR_TOO_LARGE, "a tensor has more than 2^31-1 elements");

    if (variant == TC_VARIANT_PLAIN) {
        TcPlainDims p;
        memset(&p, 0, sizeof(p));
        p.n_out = Cfg::CR;
        p.n_int = Cfg::NK;
        p.total = nC;
        p.ktotal = 1;
        p.sign = Cfg::SIGN;
        for (int j = 0; j < Cfg::CR; j++) {
            const int id = Cfg::c_id(j);
            p.ext_out[j] = sizes[id]; p.sA_out[j] = (int)sA[id]; p.sB_out[j] = (int)sB[id];
        }
        for (int j = 0; j < Cfg::NK; j++) {
            const int id = Cfg::sum_id(j);
            p.ext_k[j] = sizes[id]; p.sA_k[j] = (int)sA[id]; p.sB_k[j] = (int)sB[id];
            p.ktotal *= sizes[id];
        }
        const int64_t grid = (nC + 255) / 256;
        if (grid > lim) return tc_fail(TC_ERR_TOO_LARGE, "grid too large");
        tc_clear_hip_error();
        hipLaunchKernelGGL(tc_plain_kernel<T>, dim3((unsigned)grid), dim3(256), 0, stream,
                           (T*)C, (const T*)A, (const T*)B, p);
        tc_last_kernel() = TC_KERNEL_PLAIN;
        return tc_check_launch("plain kernel launch failed");
    }

    // Asked for: the VALU streaming kernel.  Blocks of 256 lanes walk C in memory order, 16 bytes per lane and 8 such
    // vectors in flight; a lane decodes the three fastest output indices itself.
    {
        int64_t kterms = 1;
        for (int j = 0; j < Cfg::NK; j++) kterms *= sizes[Cfg::sum_id(j)];
        if (variant == TC_VARIANT_VALU) {
            if (kterms > lim) return tc_fail(TC_ERR_TOO_LARGE, "contracted range too large");
            TcValuDims p;
            memset(&p, 0, sizeof(p));
            p.n_out = Cfg::CR; p.n_int = Cfg::NK; p.sign = Cfg::SIGN; p.ktotal = (int)kterms;
            int64_t plane = 1, nplanes = 1;
            for (int j = 0; j < Cfg::CR; j++) {
                const int id = Cfg::c_id(j);
                p.ext_out[j] = sizes[id]; p.sA_out[j] = (int)sA[id]; p.sB_out[j] = (int)sB[id];
                if (j < 3) plane *= sizes[id]; else nplanes *= sizes[id];
            }
            for (int j = 0; j < Cfg::NK; j++) {
                const int id = Cfg::sum_id(j);
                p.ext_k[j] = sizes[id]; p.sA_k[j] = (int)sA[id]; p.sB_k[j] = (int)sB[id];
            }
            constexpr int VFULL = 16 / (int)sizeof(T), U = 8;
            const bool vec = (sizes[Cfg::c_id(0)] % VFULL == 0) && (((uintptr_t)C & 15) == 0);
            const int64_t per_block = 256 * (int64_t)(vec ? VFULL : 1) * U;
            const int64_t chunks = (plane + per_block - 1) / per_block;
            if (chunks * nplanes > lim) return tc_fail(TC_ERR_TOO_LARGE, "grid too large");
            p.plane = (unsigned)plane; p.chunks = (unsigned)chunks; p.nplanes = (unsigned)nplanes;
            tc_clear_hip_error();
            const dim3 g((unsigned)(chunks * nplanes)), b(256);
            if (vec) hipLaunchKernelGGL((tc_valu_kernel<T, VFULL, U>), g, b, 0, stream, (T*)C, (const T*)A, (const T*)B, p);
            else     hipLaunchKernelGGL((tc_valu_kernel<T, 1, U>), g, b, 0, stream, (T*)C, (const T*)A, (const T*)B, p);
            tc_last_kernel() = TC_KERNEL_VALU;
            return tc_check_launch("VALU kernel launch failed");
        }
    }

    TcDims d;
    memset(&d, 0, sizeof(d));
    // strides of the two inputs as the kernel reads them: the tensors' own, or dense in tile order
    // for an input that is repacked below
    int64_t sX[TC_MAXI] = {0}, sY[TC_MAXI] = {0};
    { int64_t n = 1; for (int j = 0; j < Cfg::XR; j++) { sX[Cfg::xo_id(j)] = n; n *= sizes[Cfg::xo_id(j)]; } }
    { int64_t n = 1; for (int j = 0; j < Cfg::YR; j++) { sY[Cfg::yo_id(j)] = n; n *= sizes[Cfg::yo_id(j)]; } }
    for (int i = 0; i < Cfg::NIDX; i++) {
        d.ext[i] = sizes[i]; d.nblk[i] = 1;
        d.sC[i] = (int)sC[i]; d.sX[i] = (int)sX[i]; d.sY[i] = (int)sY[i];
    }
    bool ext_div = true, int_div = true;          // every extent a multiple of its tile
    int64_t grid = 1;
    for (int i = 0; i < Cfg::NX; i++) {
        const int id = Cfg::x_id(i), t = Cfg::x_tile(i);
        d.nblk[id] = (sizes[id] + t - 1) / t; grid *= d.nblk[id];
        if (sizes[id] % t) ext_div = false;
    }
    const int64_t nxt = grid;
    for (int i = 0; i < Cfg::NY; i++) {
        const int id = Cfg::y_id(i), t = Cfg::y_tile(i);
        d.nblk[id] = (sizes[id] + t - 1) / t; grid *= d.nblk[id];
        if (sizes[id] % t) ext_div = false;
    }
    int64_t nkb = 1;
    for (int i = 0; i < Cfg::NK; i++) {
        const int id = Cfg::k_id(i), t = Cfg::k_tile(i);
        d.nblk[id] = (sizes[id] + t - 1) / t; nkb *= d.nblk[id];
        if (sizes[id] % t) int_div = false;
    }
    // the unpredicated variants of the per-tile kernel also need tiles without MFMA padding
    const bool ext_full = ext_div && (Cfg::BX == Cfg::BXP) && (Cfg::BY == Cfg::BYP);
    const bool int_full = int_div && (Cfg::BK == Cfg::BKP);
    if (grid > lim || nkb > lim) return tc_fail(TC_ERR_TOO_LARGE, "grid too large");
    {
        // The kernels address the elements of a tile and of a slice by 32-bit BYTE offsets from a 64-bit origin:
        // the farthest element of a tile must lie within 4 GB of its first one.
        auto clip = [&](int id, int tile) { return (int64_t)((sizes[id] < tile ? sizes[id] : tile) - 1); };
        int64_t spanC = 0, spanX = 0, spanY = 0;
        for (int i = 0; i < Cfg::NX; i++) spanC += clip(Cfg::x_id(i), Cfg::x_tile(i)) * sC[Cfg::x_id(i)];
        for (int i = 0; i < Cfg::NY; i++) spanC += clip(Cfg::y_id(i), Cfg::y_tile(i)) * sC[Cfg::y_id(i)];
        for (int j = 0; j < Cfg::XR; j++) spanX += clip(Cfg::xo_id(j), Cfg::xo_tile(j)) * sX[Cfg::xo_id(j)];
        for (int j = 0; j < Cfg::YR; j++) spanY += clip(Cfg::yo_id(j), Cfg::yo_tile(j)) * sY[Cfg::yo_id(j)];
        const int64_t far = ((int64_t)1 << 32) / (int64_t)sizeof(T) - 4;       // a 16-byte access may start at the last element
        if (spanC >= far || spanX >= far || spanY >= far)
            return tc_fail(TC_ERR_TOO_LARGE, "a tile of this mapping spans 4 GB or more of a tensor (byte offsets inside a tile are 32-bit)");
    }
    d.nkb = (int)nkb;
    // split K only when there is a K loop to split; the single-K-block kernels ignore Cfg::SK
    const int sk = (nkb == 1) ? 1 : Cfg::SK;
    grid *= sk;
    if (grid > lim) return tc_fail(TC_ERR_TOO_LARGE, "grid too large");
    d.nblocks = (unsigned)grid;
    d.nxt = (unsigned)nxt;

    T* c = (T*)C;
    const T* x = (const T*)(Cfg::X_IS_A ? A : B);
    const T* y = (const T*)(Cfg::X_IS_A ? B : A);
    tc_clear_hip_error();

    // Repacked inputs: a copy in tile order (tiled externals, then K), made on the same stream in
    // memory that is allocated and freed in stream order, so calls on different streams do not share it.
    T* ws = nullptr;
    if (Cfg::RPX || Cfg::RPY) {
        const int64_t nx = Cfg::X_IS_A ? nA : nB, ny = Cfg::X_IS_A ? nB : nA;
        const int64_t off_y = Cfg::RPX ? ((nx + 31) / 32) * 32 : 0;              // keep the second copy 256-byte aligned
        const int64_t total = off_y + (Cfg::RPY ? ny : 0);
        if (no_alloc) {
            if (!ext_ws || (size_t)total * sizeof(T) > ext_ws_bytes) {
                snprintf(tc_error_buffer(), 256, "the repacked inputs need %lld bytes of scratch, the allocation-free entry point has %lld",
                         (long long)total * (long long)sizeof(T), (long long)ext_ws_bytes);
                return TC_ERR_TOO_LARGE;
            }
            ws = (T*)ext_ws;
        } else if (hipMallocAsync((void**)&ws, (size_t)total * sizeof(T), stream) != hipSuccess || !ws) {
            (void)hipGetLastError();
            return tc_fail(TC_ERR_ALLOC, "stream-ordered allocation of the repack buffer failed");
        }
        const int64_t* sXin = Cfg::X_IS_A ? sA : sB;
        const int64_t* sYin = Cfg::X_IS_A ? sB : sA;
        if (Cfg::RPX) {
            TcRepackDims r;
            memset(&r, 0, sizeof(r));
            r.n = Cfg::XR; r.total = nx;
            for (int j = 0; j < Cfg::XR; j++) { r.ext[j] = sizes[Cfg::xo_id(j)]; r.sin[j] = (int)sXin[Cfg::xo_id(j)]; }
            hipLaunchKernelGGL(tc_repack_kernel<T>, dim3((unsigned)((nx + 255) / 256)), dim3(256), 0, stream, x, ws, r);
            x = ws;
        }
        if (Cfg::RPY) {
            TcRepackDims r;
            memset(&r, 0, sizeof(r));
            r.n = Cfg::YR; r.total = ny;
            for (int j = 0; j < Cfg::YR; j++) { r.ext[j] = sizes[Cfg::yo_id(j)]; r.sin[j] = (int)sYin[Cfg::yo_id(j)]; }
            hipLaunchKernelGGL(tc_repack_kernel<T>, dim3((unsigned)((ny + 255) / 256)), dim3(256), 0, stream, y, ws + off_y, r);
            y = ws + off_y;
        }
        if (tc_check_launch("repack kernel launch failed") != TC_OK) { if (!no_alloc) (void)hipFreeAsync(ws, stream); return TC_ERR_LAUNCH; }
    }

    const dim3 g((unsigned)grid), b(Cfg::NT);
    // swapped MFMA roles with 128-bit C accesses: fp32 only, fastest extent a multiple of 4, C 16-byte aligned
    const bool swp = Cfg::SWAP && (sizes[Cfg::c_id(0)] % 4 == 0) && (((uintptr_t)C & 15) == 0);
    if (variant == TC_VARIANT_AUTO && tc_stream_launch<Cfg>(ext_div, int_div, nkb, swp, stream, c, x, y, d)) {
        tc_last_kernel() = TC_KERNEL_STREAM;
    } else {
        // (Cfg::OKP == 0: a single K block goes through the K-loop kernels, which run it as a loop of one trip, unless
        // every tile of the call is whole; only mappings without split K may say so)
        static_assert(Cfg::OKP != 0 || Cfg::SK == 1, "ok=0 needs a mapping without split K");
        const bool one_kb = nkb == 1 && ((int_full && ext_full) || Cfg::OKP != 0);
        tc_launch_variant<Cfg>(one_kb, ext_full, int_full, swp, g, b, stream, c, x, y, d);
        tc_last_kernel() = TC_KERNEL_TILED;
    }
    const int rc = tc_check_launch("tiled kernel launch failed");
    if (ws && !no_alloc && hipFreeAsync(ws, stream) != hipSuccess) { (void)hipGetLastError(); if (rc == TC_OK) return tc_fail(TC_ERR_ALLOC, "stream-ordered free of the repack buffer failed"); }
    return rc;
}

// The reference's calling convention: HOST pointers in, result copied back
// (cogent/src/codes/others/tc_pre_CUDA_Malloc.py:6-47 and
// cogent/src/codes/kernels/tc_interface.py:1368-1419).  Off the timed path.
template <class Cfg>
int tc_run_host(const int* sizes, void* hC, const void* hA, const void* hB)
{
    typedef typename Cfg::T T;
    for (int i = 0; i < Cfg::NIDX; i++)
        if (sizes[i] < 0) return tc_fail(TC_ERR_NEGATIVE_EXTENT, "negative extent");
    for (int i = 0; i < Cfg::NIDX; i++)
        if (sizes[i] == 0) return TC_OK;
    if (!hC || !hA || !hB) return tc_fail(TC_ERR_NULL_POINTER, "null tensor pointer");
    int64_t nC = 1, nA = 1, nB = 1;
    for (int j = 0; j < Cfg::CR; j++) nC *= sizes[Cfg::c_id(j)];
    for (int j = 0; j < Cfg::AR; j++) nA *= sizes[Cfg::a_id(j)];
    for (int j = 0; j < Cfg::BR; j++) nB *= sizes[Cfg::b_id(j)];
    T *dC = nullptr, *dA = nullptr, *dB = nullptr;
    int rc = TC_OK;
    if (hipMalloc(&dC, nC * sizeof(T)) != hipSuccess || hipMalloc(&dA, nA * sizeof(T)) != hipSuccess ||
        hipMalloc(&dB, nB * sizeof(T)) != hipSuccess) {
        rc = tc_fail(TC_ERR_ALLOC, "device allocation failed");
    } else if (hipMemcpy(dC, hC, nC * sizeof(T), hipMemcpyHostToDevice) != hipSuccess ||
               hipMemcpy(dA, hA, nA * sizeof(T), hipMemcpyHostToDevice) != hipSuccess ||
               hipMemcpy(dB, hB, nB * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) {
        rc = tc_fail(TC_ERR_ALLOC, "host to device copy failed");
    } else {
        rc = tc_run<Cfg>(sizes, dC, dA, dB, 0, TC_VARIANT_AUTO);
        if (rc == TC_OK && hipMemcpy(hC, dC, nC * sizeof(T), hipMemcpyDeviceToHost) != hipSuccess)
            rc = tc_fail(TC_ERR_LAUNCH, "kernel execution or device to host copy failed");
    }
    if (dC) (void)hipFree(dC);
    if (dA) (void)hipFree(dA);
    if (dB) (void)hipFree(dB);
    return rc;
}

}  // namespace cogent
