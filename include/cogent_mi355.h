/*
 * C ABI of the MI355X tensor-contraction engine.
 *
 * Two libraries export the symbols below.
 *
 * (1) libcogent_mi355.so -- host-only tools (no GPU needed): expression parser,
 *     gfx950 index-to-tile mapping pass, HIP source emitter, seeded input fill
 *     and work accounting.  They stand where the reference's Python generator
 *     stands: cogent/tc_code_generator.py:13-59 (five positional arguments),
 *     cogent/src/generators/tc_gen.py:48-99 (parse + mapping) and
 *     cogent/src/codes/tc_gen_code.py:22-447 (emission).
 *
 * (2) one shared object PER EXPRESSION, compiled from the emitted HIP source.
 *     It exports the reference's public entry point under the reference's name,
 *     `sd_t_d2_fusion_` (cogent/src/codes/kernels/tc_interface.py:1444-1516),
 *     whose parameter list depends on the expression and therefore cannot be
 *     declared once here; its shape is documented below together with the
 *     fixed-signature entry points every such object also exports.
 */
#ifndef COGENT_MI355_H
#define COGENT_MI355_H

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------
 * (1) host tools: libcogent_mi355.so
 * ---------------------------------------------------------------------- */

typedef struct cogent_plan cogent_plan;

/* Parse ONE expression in the reference grammar,
 *   `t3 [a,312,b,312,c,24] += sum(d,312) * t2 [b,d,a] * v2 [d,c];`
 * (column-major: the first listed index is the fastest; the numbers are the
 * representative sizes used for mapping only), and choose a gfx950 mapping.
 * `text` may hold '#' comment lines like the reference's .in files
 * (cogent/src/generators/tc_gen_etc.py:4-18) but exactly one expression.
 *   dtype        "DOUBLE" or "FLOAT"  (cogent/tc_code_generator.py:25)
 *   config_rank  -1: cheapest mapping by the model; k >= 0: the k-th cheapest
 *                (the reference's manual pick, cogent/src/generators/configurations.py:285-289)
 *   mapping_spec NULL, or an explicit mapping in the text form printed as "spec"
 *                by cogent_plan_json (overrides config_rank)
 * Returns 0 and a plan, or a non-zero code with cogent_host_last_error() set:
 *   1 parse error, 2 bad dtype, 3 no admissible mapping / bad spec, 4 more than one expression. */
int cogent_plan_create(const char* text, const char* dtype, int config_rank,
                       const char* mapping_spec, cogent_plan** out);
void cogent_plan_destroy(cogent_plan* plan);

/* JSON description: tensor names, index lists, operator, and the chosen mapping. */
const char* cogent_plan_json(const cogent_plan* plan);
/* JSON array with the k cheapest candidate mappings (for tuning sweeps). */
const char* cogent_plan_candidates_json(cogent_plan* plan, int k);
/* Number of `int size_*` arguments of the entry point: output indices in
 * output order, then summed indices in sum() order. */
int cogent_plan_num_indices(const cogent_plan* plan);
/* 2 * product of all extents (cogent/src/codes/kernels/tc_interface.py:289-305). */
long long cogent_plan_flops(const cogent_plan* plan, const int* sizes);
/* sizeof(T) * (|A| + |B| + 2 |C|): inputs read once, C read once and written once. */
long long cogent_plan_bytes(const cogent_plan* plan, const int* sizes);
/* Write the HIP translation unit for this plan (the counterpart of temp__NN.cu,
 * cogent/src/codes/tc_gen_code.py:27-30).  unique_name goes into the alias
 * `cogent_<unique_name>_run`.  Returns 0, or 5 when the file cannot be written. */
int cogent_plan_emit(const cogent_plan* plan, const char* unique_name, const char* out_path);
const char* cogent_host_last_error(void);

/* ---- fused groups ------------------------------------------------------------------------------
 * Entry points of an object emitted for a group of N expressions (kernels/tc_group.hpp), replacing the
 * reference's fused interface (cogent/src/codes/kernels/tc_interface.py:1444-1516 with N input pairs):
 *
 *   int sd_t_d2_fusion_(int size_<idx>..., T* out, T* a_1, T* b_1, ..., T* a_N, T* b_N,
 *                       int cond_kernel_1, ..., int cond_kernel_N, int opt_register_transpose);
 *   int sd_t_d2_fusion_host_(same parameters, HOST pointers);
 *   int cogent_run_group(const int* sizes, int n_sizes, void* C, const void* const* inputs, int n_inputs,
 *                        const int* enabled, void* stream);      inputs[] = a_1, b_1, a_2, ...; enabled may be NULL
 *   int cogent_num_terms(void);   plus cogent_num_indices / cogent_last_error / cogent_expression / cogent_info
 *
 * out <- out (+|-) sum a_1*b_1 (+|-) sum a_2*b_2 ...; a term whose cond_kernel flag is 0 is left out.
 * Same status codes as the single-expression entry points. */

/* Fused group: `text` holds two or more expressions with the same output tensor, output index list,
 * summed indices and sizes (the reference's outer group, cogent/src/algs/bases/tc_gen_inputs.py:113-123;
 * the CCSD(T) terms of cogent/drivers/ccsd_t/code_main_sd2_1.c:573-606).  Plans one tile of the output
 * for the whole group (tile_spec NULL/"" = search, or "ct=<tile>,..." one per output index, optionally followed by
 * ";kt=<K depth per block>;nw=<wavefronts per workgroup>;nr=<operand regions in LDS: 1, 2, or 0 for the kernel with one
 * pass per term>;ps=<1: persistent workgroups>") and, when
 * out_path is given, writes ONE translation unit whose kernel keeps the output tile on chip across the
 * terms.  Returns 0; 1 parse error; 2 data type; 3 no admissible tile / expressions do not form a group;
 * 5 file.  cogent_group_last_json() describes the plan of the last successful call. */
int cogent_group_emit(const char* text, const char* dtype, const char* tile_spec, const char* unique_name, const char* out_path);
const char* cogent_group_last_json(void);

/* Seeded inputs: element i = 2 * u_i - 1 with u_i in [0,1) taken from the top
 * bits of splitmix64(seed + (i + 1) * 0x9E3779B97F4A7C15), so the fill does not
 * depend on the tensor's shape.  (The reference fills with unseeded
 * rand()/RAND_MAX, cogent/drivers/tccg/code_main_tccg_01.c:95-103.) */
void cogent_fill_uniform_f64(double* dst, long long n, unsigned long long seed);
void cogent_fill_uniform_f32(float* dst, long long n, unsigned long long seed);

/* ------------------------------------------------------------------------
 * (2) per-expression shared objects
 * ----------------------------------------------------------------------
 *
 * int sd_t_d2_fusion_(int size_<i0>, ..., int size_<k0>, ...,
 *                     T* out, T* a, T* b,
 *                     int cond_kernel_1, int opt_register_transpose);
 *
 *   Replaces the generated `extern "C" void sd_t_d2_fusion_(...)` of
 *   cogent/src/codes/kernels/tc_interface.py:1444-1516, called by the drivers as
 *   `sd_t_d2_fusion_(size_a, ..., host_C, host_A, host_B, 1, -1)`
 *   (cogent/drivers/tccg/code_main_tccg_01.c:69).  Same name, same argument
 *   order, T = double or float by the generator flag; the last two ints are
 *   accepted and ignored.  Differences: out/a/b are DEVICE pointers; the kernel
 *   is enqueued on the default stream and the call does not synchronise; the
 *   result is out <- out +/- sum(a*b) (the reference kernel overwrites out);
 *   the return value is a status (0 = ok) that a caller declaring the function
 *   `void` may ignore.
 *
 * int sd_t_d2_fusion_host_(same parameters);
 *   Same computation on HOST pointers with the reference's allocate / copy in /
 *   run / copy back / free sequence (cogent/src/codes/kernels/tc_interface.py:10-101).
 */

/* Fixed-signature form of the same entry point.  sizes[] holds n_sizes extents
 * in entry-point order; stream is a hipStream_t (NULL = default stream);
 * variant 0 = the fastest kernel the object holds for these extents (the
 * panel-resident streaming kernel when it was emitted and the extents give full
 * tiles and its K-block count, otherwise the tiled MFMA kernel), 1 = plain
 * one-lane-per-element kernel whose summation order is the reference host
 * loop's, 2 = the tiled MFMA kernel with one workgroup per output tile, 3 = the
 * VALU streaming kernel (blocks walk C in memory order, every lane adds the terms of
 * its own elements in sum() order with separately rounded multiply and add: bit-exact
 * with the reference host loop; never taken by variant 0: even at contracted extents
 * below the 4-deep step of the matrix instructions the tiled kernel measured faster).
 * Status codes: 0 ok, 1 null pointer / bad sizes[], 2 negative extent,
 * 3 tensor or grid too large (2^31 elements, or a tile of the mapping spanning 4 GB or more
 * of a tensor), 4 launch failed, 5 bad variant. */
int cogent_run(const int* sizes, int n_sizes, void* C, const void* A, const void* B,
               void* stream, int variant);
/* cogent_run for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose host caller
 * allocates and frees on every call, cogent/src/codes/kernels/tc_interface.py:10-101).  Same arguments,
 * same kernels, same results as cogent_run; no hipMalloc, hipMallocAsync, hipFree or allocating library
 * routine is called on any path.  The one kernel path with a scratch buffer is a mapping that repacks its
 * inputs (rx=1 / ry=1): cogent_run takes the copies' memory from the stream-ordered allocator, this entry
 * point keeps them in a static device array of the object (16 MiB per GPU, held until the process ends)
 * and returns status 3 with a message naming both sizes when the repacked inputs need more.  Calls that
 * overlap on one GPU share that array and race: one call at a time per device.  The array's address is
 * looked up on the first call on each device, which therefore should not itself be captured.  An object
 * whose mapping needs no scratch memory exports the same symbol; there it is cogent_run. */
int cogent_run_noalloc(const int* sizes, int n_sizes, void* C, const void* A, const void* B,
                       void* stream, int variant);
int cogent_num_indices(void);
const char* cogent_last_error(void);   /* message of the last failing call on this thread */
int cogent_last_kernel(void);          /* kernel launched by this thread's last call: 0 none, 1 plain, 2 tiled (one
                                          workgroup per output tile), 3 panel-resident streaming kernel,
                                          4 VALU streaming kernel */
const char* cogent_expression(void);   /* the expression this object was emitted for      */
const char* cogent_info(void);         /* JSON: the mapping compiled into this object     */

#ifdef __cplusplus
}
#endif
#endif
