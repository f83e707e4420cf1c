/* tuff_amd.h -- the engine from plain C.
 *
 * Opaque handles, int return codes (0 = success, negative = failure; tuff_last_error() then
 * holds the message for the calling thread), no C++ in the interface: the manner of the
 * reference's include/lfm25_engine.h:100-145 (engine_init / free / set_sampler /
 * forward_token / forward_batch).  Where the reference has one sequence and a position
 * argument, this engine has requests, each with a cache of its own, and a step over a batch
 * of them; the scheduler calls take the place of the reference's loop in src/main.c:1743-1858.
 *
 * The library (libtuff_amd.so) carries the engine's host side as an embedded Python
 * interpreter; if the calling process already runs one (a Python program that loads this
 * library), that one is used.  All calls may come from any thread; they are serialised.
 *
 * Link: cc prog.c -Iinclude -L<dir of libtuff_amd.so> -ltuff_amd
 */
#ifndef TUFF_AMD_H
#define TUFF_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tuff_engine tuff_engine;

/* Sampling options with the reference's names and defaults (include/sampler.h:12-20). */
typedef struct tuff_sampling {
    float    temp;            /* <= 0: greedy */
    float    top_p;           /* 1: off */
    int32_t  top_k;           /* 0: off */
    float    min_p;           /* 0: off */
    float    repeat_penalty;  /* 1: off */
    int32_t  repeat_last_n;   /* 64 */
    uint64_t seed;            /* 0: from the clock */
    int32_t  max_new_tokens;  /* -n */
    int32_t  ignore_eos;      /* 0 / 1 */
} tuff_sampling;

/* One request's share of a step: its next tokens and the places among them whose logits are wanted. */
typedef struct tuff_step_entry {
    int64_t        request;
    const int32_t *tokens;
    int32_t        n_tokens;
    const int32_t *want;
    int32_t        n_want;
} tuff_step_entry;

/* What one scheduler step did for one request. */
typedef struct tuff_event {
    int64_t request;
    int32_t token;            /* the token drawn in this step, or -1 if the step only fed prompt tokens */
    int32_t finished;         /* 0: goes on; else one of TUFF_FINISH_* */
} tuff_event;

enum {
    TUFF_FINISH_STOP = 1,     /* end-of-sequence token */
    TUFF_FINISH_LENGTH = 2,   /* max_new_tokens reached */
    TUFF_FINISH_CONTEXT = 3,  /* context length reached */
    TUFF_FINISH_CAPACITY = 4, /* does not fit the cache even alone */
    TUFF_FINISH_ABORTED = 5,
    TUFF_FINISH_REJECTED = 6  /* prompt + max_new_tokens beyond the context length */
};

/* Message of the last failure in this thread ("" if none).  Valid until the thread's next call. */
const char *tuff_last_error(void);

/* Fills *s with the defaults. */
void tuff_sampling_default(tuff_sampling *s);

/* Writes a model folder (config.json, model.safetensors) with seeded random weights for the
 * configuration in the file config_json.  stored_dtype: "bfloat16" or "float32". */
int tuff_model_write_random(const char *config_json, uint64_t seed, const char *out_dir, const char *stored_dtype);

/* Loads the model of model_dir (config.json chooses the architecture) onto GPU 0.
 * dtype: "bfloat16" or "float32".  max_requests: requests live at a time.  ctx_size: longest
 * prompt + generation of one request (0: 4096, at most the model's limit).  The page pool holds
 * max_requests * ctx_size tokens. */
int  tuff_engine_open(tuff_engine **out, const char *model_dir, const char *dtype, int max_requests, int ctx_size);
void tuff_engine_close(tuff_engine *eng);

int tuff_engine_vocab_size(const tuff_engine *eng);
int tuff_engine_ctx_size(const tuff_engine *eng);
int tuff_engine_eos_token(const tuff_engine *eng);     /* -1 if the model names none */

/* The step function.  A request is begun, fed in steps, and ended; ending gives back its pages. */
int tuff_request_begin(tuff_engine *eng, int64_t request);
int tuff_request_end(tuff_engine *eng, int64_t request);
int tuff_request_length(const tuff_engine *eng, int64_t request);   /* tokens in its cache, or negative */

/* Runs the entries as one batch from the cache.  logits_out receives float32 [sum of n_want][vocab]
 * in the order of the entries and of want; rows_capacity is the room in rows.  If the pages run out
 * the call fails and every request is as it was before. */
int tuff_engine_step(tuff_engine *eng, const tuff_step_entry *entries, int n_entries,
                     float *logits_out, size_t rows_capacity);

/* The scheduler above it.  Requests are added at any time; every tuff_sched_step runs one step
 * (prompt portions under the token budget beside single decoded tokens), writes up to
 * events_capacity events and sets *n_events.  Returns the number of unfinished requests after the
 * step (0: nothing left), or negative.  Request numbers are the caller's; they are a namespace of
 * their own, apart from the numbers of tuff_request_begin. */
int tuff_request_add(tuff_engine *eng, int64_t request, const int32_t *prompt, int n_prompt, const tuff_sampling *s);
int tuff_request_abort(tuff_engine *eng, int64_t request);
int tuff_sched_step(tuff_engine *eng, tuff_event *events, int events_capacity, int *n_events);

/* One request from prompt to end: writes at most out_capacity tokens and sets *n_out. */
int tuff_generate(tuff_engine *eng, const int32_t *prompt, int n_prompt, const tuff_sampling *s,
                  int32_t *out, int out_capacity, int *n_out);

/* Ends the embedded interpreter if this library started it.  Optional; no call is valid afterwards. */
void tuff_shutdown(void);

#ifdef __cplusplus
}
#endif
#endif
