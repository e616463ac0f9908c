// Emitted by cogent-mi355 for gfx950.  Do not edit: regenerate from the expression.
//   t3 [d,72,c,72,b,72,a,72] += sum(e,72) * t2 [b,e,a] * v2 [c,e,d];
//   element type double, mapping x=0:24,1:4;y=2:16,3:4;k=4:36;w=2x4;t=3x1;mi=0;lx=0;ly=0;rx=1
#include "tc_launch.hpp"

namespace {
struct Cfg {
    typedef double T;
    static constexpr int NIDX = 5, SIGN = 1;
    static constexpr bool X_IS_A = false;
    // tensors in memory order (index ids, fastest first)
    static constexpr int CR = 4, AR = 3, BR = 3;
    static constexpr __host__ __device__ int c_id(int i) { constexpr int v[4] = {0, 1, 2, 3}; return v[i]; }
    static constexpr __host__ __device__ int a_id(int i) { constexpr int v[3] = {2, 4, 3}; return v[i]; }
    static constexpr __host__ __device__ int b_id(int i) { constexpr int v[3] = {1, 4, 0}; return v[i]; }
    static constexpr __host__ __device__ int sum_id(int i) { constexpr int v[1] = {4}; return v[i]; }
    // composite tiles (fastest first): X side = externals of the input that holds C's fastest index
    static constexpr int NX = 2, NY = 2, NK = 1;
    static constexpr __host__ __device__ int x_id(int i) { constexpr int v[2] = {0, 1}; return v[i]; }
    static constexpr __host__ __device__ int x_tile(int i) { constexpr int v[2] = {24, 4}; return v[i]; }
    static constexpr __host__ __device__ int y_id(int i) { constexpr int v[2] = {2, 3}; return v[i]; }
    static constexpr __host__ __device__ int y_tile(int i) { constexpr int v[2] = {16, 4}; return v[i]; }
    static constexpr __host__ __device__ int k_id(int i) { constexpr int v[1] = {4}; return v[i]; }
    static constexpr __host__ __device__ int k_tile(int i) { constexpr int v[1] = {36}; return v[i]; }
    static constexpr int BX = 96, BY = 64, BK = 36;
    static constexpr int BXP = 96, BYP = 64, BKP = 36;
    // the X- and Y-side operands in the memory order the kernel reads: id, tile, contracted?, weight in the composite coordinate
    static constexpr int XR = 3;
    static constexpr __host__ __device__ int xo_id(int i) { constexpr int v[3] = {0, 1, 4}; return v[i]; }
    static constexpr __host__ __device__ int xo_tile(int i) { constexpr int v[3] = {24, 4, 36}; return v[i]; }
    static constexpr __host__ __device__ int xo_isk(int i) { constexpr int v[3] = {0, 0, 1}; return v[i]; }
    static constexpr __host__ __device__ int xo_mul(int i) { constexpr int v[3] = {1, 24, 1}; return v[i]; }
    static constexpr int YR = 3;
    static constexpr __host__ __device__ int yo_id(int i) { constexpr int v[3] = {2, 4, 3}; return v[i]; }
    static constexpr __host__ __device__ int yo_tile(int i) { constexpr int v[3] = {16, 36, 4}; return v[i]; }
    static constexpr __host__ __device__ int yo_isk(int i) { constexpr int v[3] = {0, 1, 0}; return v[i]; }
    static constexpr __host__ __device__ int yo_mul(int i) { constexpr int v[3] = {1, 1, 16}; return v[i]; }
    static constexpr int WX = 2, WY = 4, TX = 3, TY = 1, NT = 512;
    static constexpr int MI = 0, SK = 1, MINW = 1, LATEC = 0, NTC = 0, SWAP = 0, PD = 1, RPX = 1, RPY = 0;
    static constexpr int LAYX = 0, LDX = 112, LAYY = 0, LDY = 80;
};
}  // namespace

extern "C" {

// Public entry point, same name and argument order as the reference's generated interface;
// the three pointers are DEVICE pointers, the launch goes to the default stream and the call
// returns without synchronising.  Computes t3 += sum(t2 * v2).  Returns 0 on success.
int sd_t_d2_fusion_(int size_d, int size_c, int size_b, int size_a, int size_e, double* t3, double* t2, double* v2, int cond_kernel_1, int opt_register_transpose)
{
    (void)cond_kernel_1; (void)opt_register_transpose;
    const int sizes[5] = {size_d, size_c, size_b, size_a, size_e};
    return cogent::tc_run<Cfg>(sizes, t3, t2, v2, 0, cogent::TC_VARIANT_AUTO);
}

// Host-pointer form with the reference's behaviour: allocate, copy in (C included), run, copy C back, free.
int sd_t_d2_fusion_host_(int size_d, int size_c, int size_b, int size_a, int size_e, double* t3, double* t2, double* v2, int cond_kernel_1, int opt_register_transpose)
{
    (void)cond_kernel_1; (void)opt_register_transpose;
    const int sizes[5] = {size_d, size_c, size_b, size_a, size_e};
    return cogent::tc_run_host<Cfg>(sizes, t3, t2, v2);
}

// Array form for drivers that load several expressions: sizes[] in entry-point order.
int cogent_run(const int* sizes, int n_sizes, void* C, const void* A, const void* B, void* stream, int variant)
{
    if (!sizes || n_sizes != Cfg::NIDX) return cogent::tc_fail(cogent::TC_ERR_NULL_POINTER, "sizes[] must hold one extent per index");
    return cogent::tc_run<Cfg>(sizes, C, A, B, (hipStream_t)stream, variant);
}

int cogent_tc_x_run(const int* sizes, int n_sizes, void* C, const void* A, const void* B, void* stream, int variant)
{
    return cogent_run(sizes, n_sizes, C, A, B, stream, variant);
}

int cogent_num_indices(void) { return Cfg::NIDX; }
const char* cogent_last_error(void) { return cogent::tc_error_buffer(); }
const char* cogent_expression(void) { return "t3 [d,72,c,72,b,72,a,72] += sum(e,72) * t2 [b,e,a] * v2 [c,e,d];"; }
const char* cogent_info(void) { return "{\"dtype\": \"f64\", \"x_operand\": \"v2\", \"x\": [[\"d\", 24], [\"c\", 4]], \"y\": [[\"b\", 16], [\"a\", 4]], \"k\": [[\"e\", 36]], \"block_tile\": [96, 64, 36], \"padded\": [96, 64, 36], \"waves\": [2, 4], \"mfma_tiles_per_wave\": [3, 1], \"mfma\": \"v_mfma_f64_16x16x4_f64\", \"split_k\": 1, \"min_waves_per_simd\": 1, \"late_c\": 0, \"nontemporal_c\": 0, \"swapped_roles\": 0, \"prefetch_depth\": 1, \"repack\": [1, 0], \"threads\": 512, \"lds_layout\": [0, 0], \"lds_ld\": [112, 80], \"lds_bytes\": 55296, \"model\": {\"blocks\": 4860, \"k_steps\": 2, \"blocks_per_cu\": 2, \"t_hbm_us\": 96.775, \"t_l2_us\": 44.7898, \"t_mfma_us\": 76.8234, \"t_lds_us\": 23.9203, \"tail_eff\": 0.999178, \"cost_us\": 127.475}, \"spec\": \"x=0:24,1:4;y=2:16,3:4;k=4:36;w=2x4;t=3x1;mi=0;lx=0;ly=0;rx=1\"}"; }

}  // extern "C"
