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
// durations in milliseconds; stats[0..3] = mean, median, min, max.
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
