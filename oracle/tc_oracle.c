/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's host check.
 *
 * This file is the parity oracle for the contraction hot path.  It is linked
 * only by the tests, the smoke check and the CPU-baseline leg of the benchmark;
 * the product library never calls it.
 *
 * What it restates: the nested-loop contraction every reference driver carries
 * in post_Correctness():
 *   one contracted index   cogent/drivers/tccg/code_main_tccg_01.c:117-133
 *   two contracted indices cogent/drivers/tccg/code_main_tccg_20.c:118-141
 *   fp32 (float += float*float) cogent/drivers/tccg-float/code_main_tccg_43.c:137-154
 *   the "-=" operator      cogent/drivers/ccsd_t/code_main_sd2_1.c:562-575
 *
 * Conventions taken from those loops:
 *   - tensors are dense, column-major: the FIRST listed index is the fastest;
 *   - external indices are the outer loops, the first output index outermost;
 *   - contracted indices are the inner loops, in sum() order, first one outer;
 *   - every product is added straight into C[idx] in memory (C is NOT cleared
 *     here: the result is C_in +/- sum, in this exact summation order);
 *   - fp32 accumulates in float.
 * Build with -O3 -ffp-contract=off so that no multiply-add is fused and the
 * result equals the reference loop's bit for bit.
 *
 * Pinning: tests/test_oracle_pin.py compares every function here bit-exactly
 * with the reference's own compiled loops (oracle/_ref) for 3-D, 4-D, 2-D and
 * 6-D outputs with one and two contracted indices, fp64 and fp32, "+=" and
 * "-=", and with numpy einsum, closed forms and a brute-force Python loop.
 * The reference has no driver with three or more contracted indices or with
 * none; those two branches of the loop below are pinned by hand-written loop
 * nests with the same summation order (bit-exact), by numpy einsum, by the
 * two-index branch through a unit extent, and by the outer-product closed form.
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define TC_MAX_IDX 16

typedef struct {
    int n_all;                 /* number of distinct indices                       */
    int extent[TC_MAX_IDX];    /* extent per index id                              */
    int n_out;  int out_idx[TC_MAX_IDX];   /* output index ids, fastest first      */
    int n_int;  int int_idx[TC_MAX_IDX];   /* contracted index ids, sum() order    */
    int n_a;    int a_idx[TC_MAX_IDX];     /* first input's index ids              */
    int n_b;    int b_idx[TC_MAX_IDX];     /* second input's index ids             */
    int sign;                  /* +1 for "+=", -1 for "-="                         */
    /* optional sub-range of the LAST (slowest) output index: [lo, hi)            */
    int last_lo, last_hi;      /* hi <= 0 means the full extent                    */
} tc_desc;

static void strides_of(const tc_desc* d, int n, const int* idx, int64_t* stride_by_id)
{
    int64_t s = 1;
    for (int i = 0; i < TC_MAX_IDX; i++) stride_by_id[i] = 0;
    for (int i = 0; i < n; i++) { stride_by_id[idx[i]] = s; s *= d->extent[idx[i]]; }
}

int tc_oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

static int check(const tc_desc* d)
{
    if (!d || d->n_out < 1 || d->n_out > TC_MAX_IDX || d->n_int < 0 || d->n_all > TC_MAX_IDX) return -1;
    for (int i = 0; i < d->n_all; i++) if (d->extent[i] < 0) return -1;
    return 0;
}

#define DEFINE_ORACLE(NAME, T, ACC_T)                                                        \
int NAME(const tc_desc* d, T* C, const T* A, const T* B, int nthreads)                       \
{                                                                                            \
    if (check(d)) return -1;                                                                 \
    int64_t sC[TC_MAX_IDX], sA[TC_MAX_IDX], sB[TC_MAX_IDX];                                  \
    strides_of(d, d->n_out, d->out_idx, sC);                                                 \
    strides_of(d, d->n_a, d->a_idx, sA);                                                     \
    strides_of(d, d->n_b, d->b_idx, sB);                                                     \
    const int ne = d->n_out, nk = d->n_int;                                                  \
    int lo[TC_MAX_IDX], hi[TC_MAX_IDX];                                                      \
    for (int i = 0; i < ne; i++) { lo[i] = 0; hi[i] = d->extent[d->out_idx[i]]; }            \
    if (d->last_hi > 0) { lo[ne-1] = d->last_lo; hi[ne-1] = d->last_hi; }                    \
    for (int i = 0; i < ne; i++) if (hi[i] <= lo[i]) return 0;                               \
    for (int i = 0; i < nk; i++) if (d->extent[d->int_idx[i]] <= 0) return 0;                \
    int64_t kA[TC_MAX_IDX], kB[TC_MAX_IDX]; int kN[TC_MAX_IDX];                              \
    for (int i = 0; i < nk; i++) { kA[i] = sA[d->int_idx[i]]; kB[i] = sB[d->int_idx[i]];     \
                                   kN[i] = d->extent[d->int_idx[i]]; }                       \
    const T sgn = (T)(d->sign < 0 ? -1 : 1);                                                 \
    const int o0 = d->out_idx[0];                                                            \
    if (nthreads < 1) nthreads = 1;                                                          \
    /* the outermost loop (first output index) is the only parallel one, so each     */     \
    /* output element keeps its sequential summation order                            */     \
    _Pragma("omp parallel for schedule(static) num_threads(nthreads)")                       \
    for (int i0 = lo[0]; i0 < hi[0]; i0++) {                                                 \
        int e[TC_MAX_IDX];                                                                   \
        for (int i = 0; i < ne; i++) e[i] = lo[i];                                           \
        e[0] = i0;                                                                           \
        for (;;) {                                                                           \
            int64_t oc = 0, oa = 0, ob = 0;                                                  \
            for (int i = 0; i < ne; i++) { int id = d->out_idx[i];                           \
                oc += e[i] * sC[id]; oa += e[i] * sA[id]; ob += e[i] * sB[id]; }             \
            T* c = C + oc; const T* a = A + oa; const T* b = B + ob;                         \
            if (nk == 0) {                                                                   \
                *(volatile T*)c = (T)((ACC_T)*c + (ACC_T)(sgn * a[0]) * (ACC_T)b[0]);        \
            } else if (nk == 1) {                                                            \
                for (int k0 = 0; k0 < kN[0]; k0++) {                                         \
                    T p = a[k0 * kA[0]] * b[k0 * kB[0]];                                     \
                    if (d->sign < 0) *c -= p; else *c += p;                                  \
                }                                                                            \
            } else if (nk == 2) {                                                            \
                for (int k0 = 0; k0 < kN[0]; k0++)                                           \
                for (int k1 = 0; k1 < kN[1]; k1++) {                                         \
                    T p = a[k0 * kA[0] + k1 * kA[1]] * b[k0 * kB[0] + k1 * kB[1]];           \
                    if (d->sign < 0) *c -= p; else *c += p;                                  \
                }                                                                            \
            } else {                                                                         \
                int k[TC_MAX_IDX]; for (int i = 0; i < nk; i++) k[i] = 0;                    \
                for (;;) {                                                                   \
                    int64_t ka = 0, kb = 0;                                                  \
                    for (int i = 0; i < nk; i++) { ka += k[i] * kA[i]; kb += k[i] * kB[i]; } \
                    T p = a[ka] * b[kb];                                                     \
                    if (d->sign < 0) *c -= p; else *c += p;                                  \
                    int j = nk - 1;                                                          \
                    while (j >= 0 && ++k[j] == kN[j]) { k[j] = 0; j--; }                     \
                    if (j < 0) break;                                                        \
                }                                                                            \
            }                                                                                \
            /* advance the external odometer: LAST output index is the innermost loop */     \
            int j = ne - 1;                                                                  \
            while (j >= 1 && ++e[j] == hi[j]) { e[j] = lo[j]; j--; }                         \
            if (j < 1) break;                                                                \
        }                                                                                    \
    }                                                                                        \
    return 0;                                                                                \
}

/* fp64: double products added into double C (code_main_tccg_01.c:126-127)      */
DEFINE_ORACLE(tc_oracle_f64, double, double)
/* fp32: float products added into float C (tccg-float/code_main_tccg_43.c:148) */
DEFINE_ORACLE(tc_oracle_f32, float, float)

/*
 * Error-attribution variant, not a restatement of a reference loop: fp32
 * inputs, every product and the running sum kept in double, written to a
 * double output D = C_in +/- sum.  Pinned against numpy float64 einsum.
 */
int tc_oracle_f32_acc64(const tc_desc* d, double* D, const float* Cin, const float* A, const float* B, int nthreads)
{
    if (check(d)) return -1;
    int64_t sC[TC_MAX_IDX], sA[TC_MAX_IDX], sB[TC_MAX_IDX];
    strides_of(d, d->n_out, d->out_idx, sC);
    strides_of(d, d->n_a, d->a_idx, sA);
    strides_of(d, d->n_b, d->b_idx, sB);
    int64_t nC = 1;
    for (int i = 0; i < d->n_out; i++) nC *= d->extent[d->out_idx[i]];
    int64_t nK = 1;
    for (int i = 0; i < d->n_int; i++) nK *= d->extent[d->int_idx[i]];
    if (nthreads < 1) nthreads = 1;
    #pragma omp parallel for schedule(static) num_threads(nthreads)
    for (int64_t lin = 0; lin < nC; lin++) {
        int64_t r = lin, oa = 0, ob = 0;
        for (int i = 0; i < d->n_out; i++) {
            int id = d->out_idx[i]; int64_t e = r % d->extent[id]; r /= d->extent[id];
            oa += e * sA[id]; ob += e * sB[id];
        }
        double acc = (double)Cin[lin];
        for (int64_t kk = 0; kk < nK; kk++) {
            /* sum() order with the first contracted index outermost */
            int64_t q = kk, ka = 0, kb = 0;
            for (int i = d->n_int - 1; i >= 0; i--) {
                int id = d->int_idx[i]; int64_t k = q % d->extent[id]; q /= d->extent[id];
                ka += k * sA[id]; kb += k * sB[id];
            }
            double p = (double)A[oa + ka] * (double)B[ob + kb];
            if (d->sign < 0) acc -= p; else acc += p;
        }
        D[lin] = acc;
    }
    return 0;
}

/* wall-clock helper for the CPU-baseline leg */
double tc_oracle_now(void)
{
    struct timespec ts; clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}
