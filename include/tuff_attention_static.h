/* Attention over the paged bfloat16 cache without an allocation: entry points of
 * libtuff_attention_mfma.so for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).
 *
 * This entry point has no counterpart in the reference engine; it is tuff_attention_mfma with the
 * work space replaced by a static array of the library (16 MiB of device memory on every GPU the
 * library runs on, held until the process ends).
 *
 * All calls on one GPU share that GPU's array.  Calls that overlap on one GPU (two streams, two
 * threads) race; calls in one stream's order do not.  The array keeps the last call's contents and
 * nothing in it has to be cleared between calls.
 */
#ifndef TUFF_ATTENTION_STATIC_H
#define TUFF_ATTENTION_STATIC_H

#ifdef __cplusplus
extern "C" {
#endif

/* Return codes beyond those of tuff_attention_mfma (0 ok, -2 sizes refused, > 0 a HIP error). */
#define TUFF_STATIC_TOO_LARGE (-7)   /* the call needs more floats than the static array holds */
#define TUFF_STATIC_NO_DEVICE (-8)   /* no current device, or its number is beyond 63 */

/* Looks the array's address up on the current device.  Optional: the first attention call on a
 * device does it otherwise.  Allocates nothing. */
int tuff_attention_static_setup(void);

/* Floats a call with these sizes needs; *capacity (may be null) receives the array's size. */
long long tuff_attention_static_floats(int n_tokens, int H, int hd, int n_parts, long long *capacity);

/* Arguments as tuff_attention_mfma's, without ws_o and ws_ml.  stream is a hipStream_t.
 * q, out: bfloat16 [n_tokens, H * hd]; k_cache [pages, Hkv, page_size, hd], v_cache [pages, Hkv,
 * hd, page_size] bfloat16; block_table int32 [requests, max_blocks]; blk int32 [n_qblocks, 2] or
 * null; req_info int32 [requests, 4]; positions int32 [n_tokens]; n_parts >= ceil(longest
 * context / 256). */
int tuff_attention_mfma_static(const void *q, const void *k_cache, const void *v_cache, void *out,
                               const int *block_table, int max_blocks,
                               const int *blk, int n_qblocks, int nb, const int *req_info, const int *positions,
                               int n_tokens, int H, int Hkv, int hd, int page_size, int window, float scale,
                               int n_parts, void *stream);

#ifdef __cplusplus
}
#endif
#endif
