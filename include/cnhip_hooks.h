/* libcnhip: host-side test and tuning hooks.
 *
 * None of these has a counterpart in the reference and none belongs to the drop-in surface of cnhip.h:
 * they let the tests reach the library's host logic without a GPU (the work decomposition of a product,
 * the encoder's bucket table evaluated on the CPU exactly as a workgroup evaluates it) and let tests and
 * benchmarks pin a kernel choice that the library otherwise makes by itself.  The switches are process-wide
 * and not synchronised: set them while no call of the library is in flight.
 */
#ifndef CNHIP_HOOKS_H
#define CNHIP_HOOKS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The decomposition cn_gemm_f32 would choose for an M x N x K product on `num_cu` compute units with
 * `workspace_bytes` of partial-sum memory.  force_tile_n as in cn_host_force_gemm_tile_n.
 * out = { tiles_m, tiles_n, k_iters, splits, iters_per_split, units, tile_n, tile_m }. */
void cn_host_plan_gemm(int64_t M, int64_t N, int64_t K, int num_cu, size_t workspace_bytes, int force_tile_n,
                       int64_t out[8]);
/* The same for a product whose A is stored m by k (dot, dotT): where the 128 x 128 tile would need an even number of
 * sixteen and more K chunks, 64-row tiles with half as many take its place. */
void cn_host_plan_gemm_rows_along_k(int64_t M, int64_t N, int64_t K, int num_cu, size_t workspace_bytes,
                                    int force_tile_n, int64_t out[8]);

/* 0 = the planner chooses the tile; 128 / 256 = that width of the 128-row tile; 32 / 64 = the 32 x 128 /
 * 64 x 128 tile.  Any other value means 0. */
void cn_host_force_gemm_tile_n(int tile_n);

/* 0 = every output tile is written with 4-byte stores (the path that unaligned outputs take). */
void cn_host_gemm_wide_store(int enabled);

/* 0 = cn_gemm_f32_bias_maxout / cn_gemm_f32_expand_maxout_grad never take the kernel that applies them in the
 * product's own write-out (K not split, whole tiles): they then pass through the workspace, which the tests compare
 * against. */
/* 0 keeps the tiled kernel for every product on 8-bit weights; 1 (default) lets products of up to 1024 rows take the
 * kernel that decodes straight into registers. */
void cn_host_gemm_w8_rows(int enabled);
/* 0 keeps the tiled kernel (and its chunk sum) for every plain product; 1 (default) lets products too small to fill the
 * chip with tiles take the kernel that finishes them in one launch. */
void cn_host_gemm_small(int enabled);
void cn_host_gemm_epilogue_in_kernel(int enabled);
/* 0 starts a workgroup per tile for every product; 1 (default) lets an unsplit product of several rounds of
 * 128 x 256 tiles keep two workgroups per compute unit that walk the tiles.  Same bits. */
void cn_host_gemm_persistent(int enabled);
/* Which kernel the last product of this process took: 0 none yet, 1 the tiled kernel (a workgroup per tile and K chunk),
 * 2 the one-launch kernel for small products, 3 the kernel that decodes 8-bit weights into registers, 4 the tiled
 * kernel with persistent workgroups; *splits (if not NULL) receives its number of K chunks. */
int cn_host_last_gemm_kernel(int *splits);

/* Workgroups per compute unit for the codec and abs-max kernels; 0 = each kernel's own figure. */
void cn_host_codec_workgroups_per_cu(int per_cu);
/* Which encoder compression (all forms) takes: 0 = the library's choice by size, 1 = the literal procedure element by
 * element, 2 = the table on the quotient x / precision, 3 = the table built for the call's precision.  All give the
 * same bits; for tests of that equality and for measurements. */
void cn_host_codec_encoder(int which);
/* Over `patterns` consecutive fp32 bit patterns of x starting at `first_pattern`: how often the quotient that the
 * table encoder forms, (float)((double)x * (1.0 / (double)precision)), differs in its bits from x / precision on the
 * device (two NaNs and two results below the normal range count as equal).  Synchronises; -1 on a HIP error. */
long long cn_host_quotient_mismatches(float precision, uint32_t first_pattern, unsigned long long patterns);

/* Nonzero: the single-launch reductions (abs-max, max, sum) put a release fence at device scope between a
 * workgroup's partial result and its arrival count, the form the memory model prescribes, instead of ordering the
 * two by a data dependence; the last workgroup acquires either way.  Same results; for tests of that equality. */
void cn_host_reduction_fences(int enabled);

/* Synchronises the current device and returns how many of its ticket counters (the ones the streaming kernels draw
 * their tiles from) are not zero: 0 whenever no kernel is running; -1 if the device is not initialised. */
int cn_host_tile_counters_in_use(void);
/* The library's table of counter owners, on a fresh instance: slots_out[i] = the counter the i-th key (a stream handle) is
 * given when the keys ask in turn: the same key always the same slot, the first 32 distinct keys slots 0 .. 31, any later
 * key -1 (its kernels then take the form that does not draw).  Pure host logic. */
void cn_host_stream_slots(const uint64_t *keys, int n, int *slots_out);

/* cn_absmax_compress_8bit as one launch (abs-max, a wait across the resident grid, compression) instead of as two
 * kernels: 1 = wherever the single launch can run (aligned tensors below 2^26 elements), 0 = never, negative = the
 * library's own choice by size.  Same bits. */
void cn_host_absmax_compress_single_launch(int mode);

/* How often a workgroup of the single-launch cn_absmax_compress_8bit looks for the rest of the grid before it takes the maximum
 * by itself; negative = the library's figure.  0 lets the tests reach that path: every workgroup then gives up at once. */
void cn_host_absmax_compress_spin_limit(int spins);

/* 0 = sparse products never take the strip kernel (few long rows) / the kernel that keeps a strip of B in
 * LDS (maximum only); they then run on the general kernels, which the tests compare against. */
void cn_host_csr_strip_kernel(int enabled);
void cn_host_csr_lds_rows(int enabled);
/* 0 = the passes that turn a sparse product into codes and update the weights with them run every wavefront on
 * whole rows (product, codes, weights) instead of splitting a workgroup into wavefronts that produce codes and
 * wavefronts that stream the weights.  Same bits. */
void cn_host_csr_paired_rows(int enabled);
/* Workgroups per compute unit of the passes that turn a sparse product into codes (and updates); 0 = their own. */
void cn_host_csr_rows_workgroups_per_cu(int per_cu);
/* sums_device[0 .. n] = exclusive prefix sums of counts_device[0 .. n - 1] (n + 1 entries; in place allowed) as the CSR
 * builders form them, *total_host = the sum in 64 bits: exact whatever the entries add up to, and at least 2^31 - 1
 * whenever they add up to that or more (then the 32-bit prefix sums are not to be used).  Synchronises; returns a
 * cn_status. */
int cn_host_exclusive_scan(const int32_t *counts_device, int64_t n, int32_t *sums_device, int64_t *total_host);

/* The encoder's bucket table on the host.  cn_host_xlut_entries: number of 8-byte entries of a table;
 * cn_host_xlut_step_count: number of steps of the code function found at precision 1;
 * cn_host_xlut_build: fills entries[cn_host_xlut_entries()] and *first for `precision` the way a workgroup
 * does, returns 1 if the table must not be used for this precision (the encoder then runs the literal
 * procedure per element), else 0;
 * cn_host_xlut_encode_many: codes of x[0..n) as the device computes them, returns 1 if the table was used;
 * cn_host_encode_exact: the literal procedure (division and pivot search) for one value. */
int cn_host_xlut_entries(void);
int cn_host_xlut_step_count(void);
int cn_host_xlut_build(float precision, void *entries, uint32_t *first);
int cn_host_xlut_encode_many(float precision, const float *x, size_t n, uint8_t *codes);
int cn_host_encode_exact(float x, float precision);
/* The encoder on the quotient, evaluated on the CPU as a workgroup evaluates it: the table for precision 1 looked
 * up at (float)((double)x * (1.0 / (double)precision)).  Returns 1, or 0 if that table cannot be built. */
int cn_host_quotient_encode_many(float precision, const float *x, size_t n, uint8_t *codes);

#ifdef __cplusplus
}
#endif

#endif /* CNHIP_HOOKS_H */
