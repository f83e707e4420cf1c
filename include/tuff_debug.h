/* Knobs of the kernel libraries for measurements and tests.  None of them changes a result: each
 * chooses between ways of running a kernel that give the same bits (the tests force both ways and
 * compare), so production code has no reason to call them.
 *
 * They set process-wide variables of their library without a lock: call them from one thread,
 * while no other thread launches that library's kernels, and put the old value (which each
 * returns) back afterwards.
 */
#ifndef TUFF_DEBUG_H
#define TUFF_DEBUG_H

#ifdef __cplusplus
extern "C" {
#endif

/* ---- libtuff_attention_mfma.so: attention of single tokens, a workgroup a partition of 256 keys.
 * A negative argument only reads the value. */

/* Below how many workgroups a partition gets four waves (a unit of 64 keys each) instead of one. */
int tuff_attention_few_waves(int n);
/* From how many workgroups on the kv head changes fastest in the order of the workgroups. */
int tuff_attention_kv_fast_waves(int n);
/* From how many workgroups on keys of heads of up to 64 channels are read in whole lines through LDS. */
int tuff_attention_stage_k_waves(int n);
/* How many lanes fetch page numbers for partition `part` with pages of page_size positions: the pages
 * the partition touches.  Host arithmetic (the kernel's own function); -2 for nonsense. */
int tuff_attention_partition_pages(int part, int page_size);

/* ---- libtuff_gemm_bf16.so */

/* Products of at most 64 rows with a short K: from how many columns (min_n) up to how many (max_n) and
 * from how many rows on (min_m) they take blocks of 64 x 64 instead of slices of K.  An argument <= 0
 * leaves its value.  Returns min_n as it was. */
int tuff_gemm_bf16_wide64(int min_n, int max_n, int min_m);
/* Forces the block shape of products of more than 64 rows whose K is a multiple of 64
 * (0: 256 x 256, 1: 128 x 128 two a CU, 2: 128 x 128 one a CU, 3: 64 x 64, 4: 256 x 192; -1: by size). */
int tuff_gemm_bf16_force_tiled_shape(int shape);

#ifdef __cplusplus
}
#endif
#endif
