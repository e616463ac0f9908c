// Emitted by cogent-mi355 for gfx950.  Do not edit: regenerate from the expression.
//   t3 [a,24,b,16,c,16,d,24,e,16,f,16] -= sum(g,24) * t2 [d,e,g,a] * v2 [g,f,b,c];
//   element type double, mapping x=0:24,3:6,4:1;y=1:16,2:2,5:1;k=6:24;w=3x2;t=3x1;mi=0;lx=0;ly=1
#include "tc_launch.hpp"

namespace {
struct Cfg {
    typedef double T;
    static constexpr int NIDX = 7, SIGN = -1;
    static constexpr bool X_IS_A = true;
    // tensors in memory order (index ids, fastest first)
    static constexpr int CR = 6, AR = 4, BR = 4;
    static constexpr __host__ __device__ int c_id(int i) { constexpr int v[6] = {0, 1, 2, 3, 4, 5}; return v[i]; }
    static constexpr __host__ __device__ int a_id(int i) { constexpr int v[4] = {3, 4, 6, 0}; return v[i]; }
    static constexpr __host__ __device__ int b_id(int i) { constexpr int v[4] = {6, 5, 1, 2}; return v[i]; }
    static constexpr __host__ __device__ int sum_id(int i) { constexpr int v[1] = {6}; return v[i]; }
    // composite tiles (fastest first): X side = externals of the input that holds C's fastest index
    static constexpr int NX = 3, NY = 3, NK = 1;
    static constexpr __host__ __device__ int x_id(int i) { constexpr int v[3] = {0, 3, 4}; return v[i]; }
    static constexpr __host__ __device__ int x_tile(int i) { constexpr int v[3] = {24, 6, 1}; return v[i]; }
    static constexpr __host__ __device__ int y_id(int i) { constexpr int v[3] = {1, 2, 5}; return v[i]; }
    static constexpr __host__ __device__ int y_tile(int i) { constexpr int v[3] = {16, 2, 1}; return v[i]; }
    static constexpr __host__ __device__ int k_id(int i) { constexpr int v[1] = {6}; return v[i]; }
    static constexpr __host__ __device__ int k_tile(int i) { constexpr int v[1] = {24}; return v[i]; }
    static constexpr __host__ __device__ int c_tile(int i) { constexpr int v[6] = {24, 16, 2, 6, 1, 1}; return v[i]; }
    static constexpr __host__ __device__ int cl_stride(int i) { constexpr int v[7] = {1, 24, 384, 768, 4608, 4608, 0}; return v[i]; }
    static constexpr int BX = 144, BY = 32, BK = 24;
    static constexpr int BXP = 144, BYP = 32, BKP = 24;
    // the X- and Y-side operands in the memory order the kernel reads: id, tile, contracted?, weight in the composite coordinate
    static constexpr int XR = 4;
    static constexpr __host__ __device__ int xo_id(int i) { constexpr int v[4] = {3, 4, 6, 0}; return v[i]; }
    static constexpr __host__ __device__ int xo_tile(int i) { constexpr int v[4] = {6, 1, 24, 24}; return v[i]; }
    static constexpr __host__ __device__ int xo_isk(int i) { constexpr int v[4] = {0, 0, 1, 0}; return v[i]; }
    static constexpr __host__ __device__ int xo_mul(int i) { constexpr int v[4] = {24, 144, 1, 1}; return v[i]; }
    static constexpr int YR = 4;
    static constexpr __host__ __device__ int yo_id(int i) { constexpr int v[4] = {6, 5, 1, 2}; return v[i]; }
    static constexpr __host__ __device__ int yo_tile(int i) { constexpr int v[4] = {24, 1, 16, 2}; return v[i]; }
    static constexpr __host__ __device__ int yo_isk(int i) { constexpr int v[4] = {1, 0, 0, 0}; return v[i]; }
    static constexpr __host__ __device__ int yo_mul(int i) { constexpr int v[4] = {1, 32, 1, 16}; return v[i]; }
    static constexpr int WX = 3, WY = 2, TX = 3, TY = 1, NT = 384;
    static constexpr int MI = 0, SK = 1, MINW = 1, LATEC = 0, NTC = 3, SWAP = 0, PD = 1, RPX = 0, RPY = 0, CLDS = 1;
    static constexpr int LAYX = 0, LDX = 144, LAYY = 1, LDY = 26;
};
}  // namespace

extern "C" {

// Public entry point, same name and argument order as the reference's generated interface;
// the three pointers are DEVICE pointers, the launch goes to the default stream and the call
// returns without synchronising.  Computes t3 -= sum(t2 * v2).  Returns 0 on success.
int sd_t_d2_fusion_(int size_a, int size_b, int size_c, int size_d, int size_e, int size_f, int size_g, double* t3, double* t2, double* v2, int cond_kernel_1, int opt_register_transpose)
{
    (void)cond_kernel_1; (void)opt_register_transpose;
    const int sizes[7] = {size_a, size_b, size_c, size_d, size_e, size_f, size_g};
    return cogent::tc_run<Cfg>(sizes, t3, t2, v2, 0, cogent::TC_VARIANT_AUTO);
}

// Host-pointer form with the reference's behaviour: allocate, copy in (C included), run, copy C back, free.
int sd_t_d2_fusion_host_(int size_a, int size_b, int size_c, int size_d, int size_e, int size_f, int size_g, double* t3, double* t2, double* v2, int cond_kernel_1, int opt_register_transpose)
{
    (void)cond_kernel_1; (void)opt_register_transpose;
    const int sizes[7] = {size_a, size_b, size_c, size_d, size_e, size_f, size_g};
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
const char* cogent_expression(void) { return "t3 [a,24,b,16,c,16,d,24,e,16,f,16] -= sum(g,24) * t2 [d,e,g,a] * v2 [g,f,b,c];"; }
const char* cogent_info(void) { return "{\"dtype\": \"f64\", \"x_operand\": \"t2\", \"x\": [[\"a\", 24], [\"d\", 6], [\"e\", 1]], \"y\": [[\"b\", 16], [\"c\", 2], [\"f\", 1]], \"k\": [[\"g\", 24]], \"block_tile\": [144, 32, 24], \"padded\": [144, 32, 24], \"waves\": [3, 2], \"mfma_tiles_per_wave\": [3, 1], \"mfma\": \"v_mfma_f64_16x16x4_f64\", \"split_k\": 1, \"min_waves_per_simd\": 1, \"late_c\": 0, \"nontemporal_c\": 3, \"swapped_roles\": 0, \"prefetch_depth\": 1, \"c_through_lds\": 1, \"repack\": [0, 0], \"threads\": 384, \"lds_layout\": [0, 1], \"lds_ld\": [144, 26], \"lds_bytes\": 34304, \"model\": {\"blocks\": 8192, \"k_steps\": 1, \"blocks_per_cu\": 3, \"t_hbm_us\": 118.792, \"t_l2_us\": 65.4311, \"t_mfma_us\": 49.3867, \"t_lds_us\": 11.2, \"tail_eff\": 1, \"cost_us\": 141.998}, \"spec\": \"x=0:24,3:6,4:1;y=1:16,2:2,5:1;k=6:24;w=3x2;t=3x1;mi=0;lx=0;ly=1\"}"; }

}  // extern "C"
