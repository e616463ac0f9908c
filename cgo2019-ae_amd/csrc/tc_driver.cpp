// Timing driver: the measuring half of the reference's bench scripts.
//
// The reference times one launch per benchmark with `nvprof --print-gpu-trace`
// and divides the printed operation count by the kernel's duration
// (cogent/bench_tccg.sh:85-93, cogent/data-tccg.py:26-49).  Here a loaded
// per-expression object is launched warm-up + N times on one stream with a HIP
// event between consecutive launches, so every launch gets its own duration;
// the output buffers are rotated so that a tensor smaller than the 256 MB
// Infinity Cache is not served from it on the next launch.  Device buffers are
// owned by the caller; nothing is allocated on the device here.
#include <hip/hip_runtime.h>
#include <dlfcn.h>
#include <stdio.h>
#include <string.h>
#include <vector>
#include <algorithm>

typedef int (*cogent_run_fn)(const int*, int, void*, const void*, const void*, void*, int);

static thread_local char g_err[256] = "";

extern "C" {

const char* cogent_driver_last_error(void) { return g_err; }

// Returns 0 on success.  ms_each (may be NULL) receives `iters` per-launch
// durations in milliseconds; stats[0..3] = mean, median, min, max of the launches bracketed one by one, stats[4] = mean of
// the same number of launches issued back to back between two events.
int cogent_driver_time(const char* so_path, const int* sizes, int n_sizes,
                       void* const* c_bufs, int n_c_bufs, const void* A, const void* B,
                       int warmup, int iters, int variant, float* ms_each, float* stats)
{
    g_err[0] = 0;
    if (!so_path || !sizes || !c_bufs || n_c_bufs < 1 || iters < 1 || warmup < 0) {
        snprintf(g_err, sizeof g_err, "bad argument");
        return 1;
    }
    void* h = dlopen(so_path, RTLD_NOW | RTLD_LOCAL);
    if (!h) { snprintf(g_err, sizeof g_err, "dlopen failed: %s", dlerror()); return 2; }
    cogent_run_fn run = (cogent_run_fn)dlsym(h, "cogent_run");
    if (!run) { snprintf(g_err, sizeof g_err, "cogent_run not exported by %s", so_path); dlclose(h); return 2; }

    hipStream_t stream = nullptr;   // default stream: where sd_t_d2_fusion_ launches too
    std::vector<hipEvent_t> ev(iters + 1);
    for (auto& e : ev) if (hipEventCreate(&e) != hipSuccess) { snprintf(g_err, sizeof g_err, "hipEventCreate failed"); return 3; }
    int rc = 0, it = 0;
    for (int i = 0; i < warmup && !rc; i++, it++) rc = run(sizes, n_sizes, c_bufs[it % n_c_bufs], A, B, stream, variant);
    if (!rc && hipStreamSynchronize(stream) != hipSuccess) rc = 4;
    if (!rc) (void)hipEventRecord(ev[0], stream);
    for (int i = 0; i < iters && !rc; i++, it++) {
        rc = run(sizes, n_sizes, c_bufs[it % n_c_bufs], A, B, stream, variant);
        (void)hipEventRecord(ev[i + 1], stream);
    }
    if (hipStreamSynchronize(stream) != hipSuccess && !rc) rc = 4;
    if (rc) {
        snprintf(g_err, sizeof g_err, "launch failed with status %d", rc);
    } else {
        std::vector<float> ms(iters);
        double sum = 0;
        for (int i = 0; i < iters; i++) { (void)hipEventElapsedTime(&ms[i], ev[i], ev[i + 1]); sum += ms[i]; if (ms_each) ms_each[i] = ms[i]; }
        std::sort(ms.begin(), ms.end());
        if (stats) { stats[0] = (float)(sum / iters); stats[1] = ms[iters / 2]; stats[2] = ms.front(); stats[3] = ms.back(); }
        // second pass: the same launches back to back between TWO events, no event between them (an event between two
        // launches costs 2-3 us of its own, a tenth of the shortest kernels here)
        (void)hipEventRecord(ev[0], stream);
        for (int i = 0; i < iters && !rc; i++, it++) rc = run(sizes, n_sizes, c_bufs[it % n_c_bufs], A, B, stream, variant);
        (void)hipEventRecord(ev[1], stream);
        if (hipStreamSynchronize(stream) != hipSuccess && !rc) rc = 4;
        float total = 0;
        (void)hipEventElapsedTime(&total, ev[0], ev[1]);
        if (stats) stats[4] = total / iters;
        if (rc) snprintf(g_err, sizeof g_err, "launch failed with status %d", rc);
    }
    for (auto& e : ev) (void)hipEventDestroy(e);
    dlclose(h);
    return rc;
}

// The same measurement for a fused-group object (cogent_run_group): inputs[] holds two pointers per term.
typedef int (*cogent_run_group_fn)(const int*, int, void*, const void* const*, int, const int*, void*);

int cogent_driver_time_group(const char* so_path, const int* sizes, int n_sizes,
                             void* const* c_bufs, int n_c_bufs, const void* const* inputs, int n_inputs,
                             int warmup, int iters, float* ms_each, float* stats)
{
    g_err[0] = 0;
    if (!so_path || !sizes || !c_bufs || !inputs || n_c_bufs < 1 || iters < 1 || warmup < 0) {
        snprintf(g_err, sizeof g_err, "bad argument");
        return 1;
    }
    void* h = dlopen(so_path, RTLD_NOW | RTLD_LOCAL);
    if (!h) { snprintf(g_err, sizeof g_err, "dlopen failed: %s", dlerror()); return 2; }
    cogent_run_group_fn run = (cogent_run_group_fn)dlsym(h, "cogent_run_group");
    if (!run) { snprintf(g_err, sizeof g_err, "cogent_run_group not exported by %s", so_path); dlclose(h); return 2; }
    hipStream_t stream = nullptr;
    std::vector<hipEvent_t> ev(iters + 1);
    for (auto& e : ev) if (hipEventCreate(&e) != hipSuccess) { snprintf(g_err, sizeof g_err, "hipEventCreate failed"); return 3; }
    int rc = 0, it = 0;
    for (int i = 0; i < warmup && !rc; i++, it++) rc = run(sizes, n_sizes, c_bufs[it % n_c_bufs], inputs, n_inputs, nullptr, stream);
    if (!rc && hipStreamSynchronize(stream) != hipSuccess) rc = 4;
    if (!rc) (void)hipEventRecord(ev[0], stream);
    for (int i = 0; i < iters && !rc; i++, it++) {
        rc = run(sizes, n_sizes, c_bufs[it % n_c_bufs], inputs, n_inputs, nullptr, stream);
        (void)hipEventRecord(ev[i + 1], stream);
    }
    if (hipStreamSynchronize(stream) != hipSuccess && !rc) rc = 4;
    if (rc) {
        snprintf(g_err, sizeof g_err, "launch failed with status %d", rc);
    } else {
        std::vector<float> ms(iters);
        double sum = 0;
        for (int i = 0; i < iters; i++) { (void)hipEventElapsedTime(&ms[i], ev[i], ev[i + 1]); sum += ms[i]; if (ms_each) ms_each[i] = ms[i]; }
        std::sort(ms.begin(), ms.end());
        if (stats) { stats[0] = (float)(sum / iters); stats[1] = ms[iters / 2]; stats[2] = ms.front(); stats[3] = ms.back(); }
        (void)hipEventRecord(ev[0], stream);
        for (int i = 0; i < iters && !rc; i++, it++) rc = run(sizes, n_sizes, c_bufs[it % n_c_bufs], inputs, n_inputs, nullptr, stream);
        (void)hipEventRecord(ev[1], stream);
        if (hipStreamSynchronize(stream) != hipSuccess && !rc) rc = 4;
        float total = 0;
        (void)hipEventElapsedTime(&total, ev[0], ev[1]);
        if (stats) stats[4] = total / iters;
        if (rc) snprintf(g_err, sizeof g_err, "launch failed with status %d", rc);
    }
    for (auto& e : ev) (void)hipEventDestroy(e);
    dlclose(h);
    return rc;
}

// Same measurement for a plain device-to-device copy of `bytes` bytes done by a
// grid-stride kernel: the yardstick the counter readings and the HBM fractions
// are scaled against.
__global__ void cogent_copy_kernel(const double2* __restrict__ s, double2* __restrict__ d, size_t n)
{
    size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) d[i] = s[i];
}

int cogent_driver_time_copy(const void* src, void* dst, long long bytes, int warmup, int iters, float* stats)
{
    if (!src || !dst || bytes < 16 || iters < 1) return 1;
    const size_t n = (size_t)bytes / 16;
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
    for (int i = 0; i < warmup; i++) hipLaunchKernelGGL(cogent_copy_kernel, dim3(65536), dim3(512), 0, 0, (const double2*)src, (double2*)dst, n);
    (void)hipEventRecord(e0, 0);
    for (int i = 0; i < iters; i++) hipLaunchKernelGGL(cogent_copy_kernel, dim3(65536), dim3(512), 0, 0, (const double2*)src, (double2*)dst, n);
    (void)hipEventRecord(e1, 0);
    if (hipEventSynchronize(e1) != hipSuccess) return 4;
    float ms = 0;
    (void)hipEventElapsedTime(&ms, e0, e1);
    if (stats) stats[0] = ms / iters;
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
    return 0;
}

}  // extern "C"

// ---------------------------------------------------------------------------------------------
// Read-modify-write yardsticks: what the memory system gives a kernel that does nothing but read a
// buffer, add one and write it back -- which is what a `+=` contraction does to its output.  The HBM
// fractions of the HBM-bound contractions are to be read against these, not only against the 8 TB/s
// of the data sheet.  Buffers are rotated by the caller (bufs[]) so that the Infinity Cache cannot
// serve a launch from the one before; the mean over `iters` back-to-back launches is returned.
//
// Flat form: blocks of 256 lanes, each lane `UNR` loads of 8 bytes in flight, then the stores, grid-stride.
template <int UNR, int NT>
__global__ __launch_bounds__(256) void cogent_rmw_flat_kernel(double* __restrict__ p, size_t n)
{
    size_t i = blockIdx.x * (size_t)256 * UNR + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256 * UNR;
    for (; i + (UNR - 1) * 256 < n; i += stride) {
        double v[UNR];
#pragma unroll
        for (int u = 0; u < UNR; u++) v[u] = (NT & 1) ? __builtin_nontemporal_load(&p[i + u * 256]) : p[i + u * 256];
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            if (NT & 2) __builtin_nontemporal_store(v[u] + 1.0, &p[i + u * 256]);
            else p[i + u * 256] = v[u] + 1.0;
        }
    }
}

// Tiled persistent form, the access pattern of the panel-resident streaming kernel on a 4-D fp64 output
// C[d,c,b,a] with all extents `e` (72 for BASELINE config 2): one workgroup of 12 wavefronts per CU walks a run
// of tiles (d: all, c: 2) x (b: 8, a: 8); a lane owns the 12 elements the MFMA accumulator layout gives it
// (16 lanes along d = one 128-byte line per row, 4 rows per instruction), reads the next tile before it
// writes the current one.  interleaved != 0: run r takes tiles r, r + nruns, ..; else a contiguous range.
struct CogentRmwTiles { int e, nres, nstr, run, nruns, nb_b, interleaved; };
__global__ __launch_bounds__(768) void cogent_rmw_tiles_kernel(double* __restrict__ C, CogentRmwTiles p)
{
    const unsigned n = gridDim.x, xcd = blockIdx.x % 8u, idx = blockIdx.x / 8u;
    const unsigned q = n / 8u, r = n % 8u;
    const unsigned vb = xcd * q + (xcd < r ? xcd : r) + idx;            // XCD-contiguous, as the contraction kernels
    const unsigned rt = vb % p.nres, rn = vb / p.nres;
    const unsigned step = p.interleaved ? p.nruns : 1u;
    const unsigned first = p.interleaved ? rn : rn * p.run;
    if (first >= (unsigned)p.nstr) return;
    const unsigned ntiles = p.interleaved ? (p.nstr - rn + p.nruns - 1) / p.nruns
                                          : ((p.nstr - first) < (unsigned)p.run ? (p.nstr - first) : p.run);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wx = wave % 3, wy = wave / 3;
    const long long sb = (long long)p.e * p.e, sa = sb * p.e;
    long long off[12];
#pragma unroll
    for (int tj = 0; tj < 3; tj++)
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            const int row = wy * 16 + 4 * rr + lane / 16;              // row = b + 8 a within the tile
            off[tj * 4 + rr] = (wx * 3 + tj) * 16 + lane % 16 + (row % 8) * sb + (row / 8) * sa;
        }
    auto base = [&](unsigned t) { return (long long)rt * 2 * p.e + (long long)(t % p.nb_b) * 8 * sb + (long long)(t / p.nb_b) * 8 * sa; };
    double v[2][12];
    long long b0 = base(first), b1 = 0;
#pragma unroll
    for (int k = 0; k < 12; k++) v[0][k] = __builtin_nontemporal_load(C + b0 + off[k]);
    for (unsigned i = 0; i < ntiles; i += 2) {
        if (i + 1 < ntiles) {
            b1 = base(first + (i + 1) * step);
#pragma unroll
            for (int k = 0; k < 12; k++) v[1][k] = __builtin_nontemporal_load(C + b1 + off[k]);
        }
#pragma unroll
        for (int k = 0; k < 12; k++) __builtin_nontemporal_store(v[0][k] + 1.0, C + b0 + off[k]);
        if (i + 1 < ntiles) {
            if (i + 2 < ntiles) {
                b0 = base(first + (i + 2) * step);
#pragma unroll
                for (int k = 0; k < 12; k++) v[0][k] = __builtin_nontemporal_load(C + b0 + off[k]);
            }
#pragma unroll
            for (int k = 0; k < 12; k++) __builtin_nontemporal_store(v[1][k] + 1.0, C + b1 + off[k]);
        }
    }
}

extern "C" {

// mode 0: flat, plain accesses; 1: flat, non-temporal loads and stores; 2: tiled persistent with contiguous runs
// (bytes must be 8 * 72^4, the output of config 2: the lane layout above is the one of its 144-wide tile);
// 3: the same with interleaved runs.  stats[0] = mean milliseconds per launch.
int cogent_driver_time_rmw(void* const* bufs, int n_bufs, long long bytes, int mode, int warmup, int iters, float* stats)
{
    if (!bufs || n_bufs < 1 || bytes < 4096 || iters < 1 || mode < 0 || mode > 3) return 1;
    const size_t n = (size_t)bytes / 8;
    CogentRmwTiles p = {0, 0, 0, 0, 0, 0, 0};
    unsigned grid = 8192;
    if (mode >= 2) {
        const int e = 72;
        if ((long long)e * e * e * e * 8 != bytes) return 1;
        int cus = 0, dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) return 3;
        p.e = e; p.nres = e / 2; p.nb_b = e / 8; p.nstr = (e / 8) * (e / 8);
        int runs = cus / p.nres; if (runs < 1) runs = 1; if (runs > p.nstr) runs = p.nstr;
        p.run = (p.nstr + runs - 1) / runs; p.nruns = (p.nstr + p.run - 1) / p.run; p.interleaved = mode == 3;
        grid = (unsigned)(p.nres * p.nruns);
    }
    auto launch = [&](int i) {
        double* b = (double*)bufs[i % n_bufs];
        if (mode == 0)      hipLaunchKernelGGL((cogent_rmw_flat_kernel<8, 0>), dim3(grid), dim3(256), 0, 0, b, n);
        else if (mode == 1) hipLaunchKernelGGL((cogent_rmw_flat_kernel<8, 3>), dim3(grid), dim3(256), 0, 0, b, n);
        else                hipLaunchKernelGGL(cogent_rmw_tiles_kernel, dim3(grid), dim3(768), 0, 0, b, p);
    };
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
    int it = 0;
    for (int i = 0; i < warmup; i++) launch(it++);
    (void)hipEventRecord(e0, 0);
    for (int i = 0; i < iters; i++) launch(it++);
    (void)hipEventRecord(e1, 0);
    if (hipEventSynchronize(e1) != hipSuccess) return 4;
    float ms = 0;
    (void)hipEventElapsedTime(&ms, e0, e1);
    if (stats) stats[0] = ms / iters;
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
    return hipGetLastError() == hipSuccess ? 0 : 4;
}

}  // extern "C"
