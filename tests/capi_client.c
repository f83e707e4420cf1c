/* A plain C program that drives the engine through include/tuff_amd.h; the tests compile it,
 * run it as a child process and compare what it prints and writes with the Python entry point
 * and the plain implementation.
 *
 *   capi_client write-random CONFIG.json SEED OUT_DIR DTYPE
 *   capi_client run MODEL_DIR DTYPE LOGITS_FILE N_NEW TOKEN,TOKEN,...
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "tuff_amd.h"

#define CHECK(call)                                                          \
    do {                                                                     \
        if ((call) < 0) {                                                    \
            fprintf(stderr, "FAILED %s: %s\n", #call, tuff_last_error());    \
            return 1;                                                        \
        }                                                                    \
    } while (0)

static int parse_tokens(const char *text, int32_t *out, int cap) {
    int n = 0;
    char *copy = strdup(text), *save = NULL;
    for (char *t = strtok_r(copy, ",", &save); t && n < cap; t = strtok_r(NULL, ",", &save)) out[n++] = atoi(t);
    free(copy);
    return n;
}

static void print_tokens(const char *label, const int32_t *t, int n) {
    printf("%s", label);
    for (int i = 0; i < n; ++i) printf(" %d", t[i]);
    printf("\n");
}

static int run(const char *model_dir, const char *dtype, const char *logits_file, int n_new, const char *tokens) {
    int32_t prompt[4096];
    int n = parse_tokens(tokens, prompt, 4096);
    if (n < 6) { fprintf(stderr, "give at least 6 tokens\n"); return 1; }

    tuff_engine *eng = NULL;
    CHECK(tuff_engine_open(&eng, model_dir, dtype, 4, 512));
    int vocab = tuff_engine_vocab_size(eng);
    printf("vocab %d ctx %d eos %d\n", vocab, tuff_engine_ctx_size(eng), tuff_engine_eos_token(eng));

    /* the step function: a portion, then a second request beside the rest, then single tokens */
    float *logits = malloc(sizeof(float) * (size_t)vocab * (size_t)(n + 2));
    size_t rows = 0;
    int head = n - 4;
    int32_t want_all[4096];
    for (int i = 0; i < n; ++i) want_all[i] = i;
    CHECK(tuff_request_begin(eng, 7));
    CHECK(tuff_request_begin(eng, 8));
    tuff_step_entry e[2];
    e[0] = (tuff_step_entry){7, prompt, head, want_all, head};
    CHECK(tuff_engine_step(eng, e, 1, logits + rows * vocab, (size_t)head));
    rows += (size_t)head;
    e[0] = (tuff_step_entry){8, prompt + 1, 5, NULL, 0};          /* another request, nothing wanted */
    e[1] = (tuff_step_entry){7, prompt + head, 2, want_all, 2};
    CHECK(tuff_engine_step(eng, e, 2, logits + rows * vocab, 2));
    rows += 2;
    for (int i = head + 2; i < n; ++i) {
        e[0] = (tuff_step_entry){7, prompt + i, 1, want_all, 1};
        CHECK(tuff_engine_step(eng, e, 1, logits + rows * vocab, 1));
        rows += 1;
    }
    printf("length %d %d\n", tuff_request_length(eng, 7), tuff_request_length(eng, 8));
    FILE *f = fopen(logits_file, "wb");
    if (!f || fwrite(logits, sizeof(float) * (size_t)vocab, rows, f) != rows) { perror(logits_file); return 1; }
    fclose(f);

    /* failures leave a message and the engine usable */
    e[0] = (tuff_step_entry){99, prompt, 2, NULL, 0};
    if (tuff_engine_step(eng, e, 1, NULL, 0) >= 0) { fprintf(stderr, "a step of an unknown request passed\n"); return 1; }
    printf("error-unknown: %s\n", tuff_last_error());
    e[0] = (tuff_step_entry){7, prompt, 1, want_all, 1};
    if (tuff_engine_step(eng, e, 1, logits, 0) >= 0) { fprintf(stderr, "a step without room for logits passed\n"); return 1; }
    printf("error-room: %s\n", tuff_last_error());
    printf("length-after-errors %d\n", tuff_request_length(eng, 7));
    CHECK(tuff_request_end(eng, 7));
    CHECK(tuff_request_end(eng, 8));

    /* one request from prompt to end */
    tuff_sampling s;
    tuff_sampling_default(&s);
    s.max_new_tokens = n_new;
    s.ignore_eos = 1;
    int32_t out[1024];
    int n_out = 0;
    CHECK(tuff_generate(eng, prompt, n, &s, out, 1024, &n_out));
    print_tokens("generate", out, n_out);

    /* the scheduler: three requests, the third added after two steps, one with temperature */
    int32_t got[3][1024];
    int n_got[3] = {0, 0, 0}, fin[3] = {0, 0, 0};
    CHECK(tuff_request_add(eng, 0, prompt, n, &s));
    tuff_sampling warm = s;
    warm.temp = 0.8f; warm.top_k = 20; warm.top_p = 0.9f; warm.seed = 11; warm.max_new_tokens = n_new + 3;
    CHECK(tuff_request_add(eng, 1, prompt + 2, n - 2, &warm));
    tuff_event ev[8];
    int n_ev = 0, left = 1, steps = 0;
    while (left > 0) {
        left = tuff_sched_step(eng, ev, 8, &n_ev);
        CHECK(left);
        for (int i = 0; i < n_ev; ++i) {
            int r = (int)ev[i].request;
            if (ev[i].token >= 0) got[r][n_got[r]++] = ev[i].token;
            if (ev[i].finished) fin[r] = ev[i].finished;
        }
        if (++steps == 2) {
            tuff_sampling shorter = s;
            shorter.max_new_tokens = 3;
            CHECK(tuff_request_add(eng, 2, prompt + 1, n - 1, &shorter));
            left = 1;
        }
    }
    for (int r = 0; r < 3; ++r) {
        char label[32];
        snprintf(label, sizeof label, "sched %d fin %d:", r, fin[r]);
        print_tokens(label, got[r], n_got[r]);
    }

    /* a request too long for the context is rejected, not run */
    tuff_sampling huge = s;
    huge.max_new_tokens = 100000;
    CHECK(tuff_request_add(eng, 5, prompt, n, &huge));
    left = tuff_sched_step(eng, ev, 8, &n_ev);
    CHECK(left);
    printf("rejected: left %d events %d request %d token %d finished %d\n", left, n_ev, (int)ev[0].request,
           ev[0].token, ev[0].finished);

    tuff_engine_close(eng);
    printf("closed\n");
    fflush(stdout);
    return 0;
}

int main(int argc, char **argv) {
    if (argc == 6 && strcmp(argv[1], "write-random") == 0) {
        if (tuff_model_write_random(argv[2], strtoull(argv[3], NULL, 10), argv[4], argv[5]) < 0) {
            fprintf(stderr, "FAILED: %s\n", tuff_last_error());
            return 1;
        }
        tuff_sampling s;
        tuff_sampling_default(&s);
        printf("defaults %g %g %d %g %g %d %llu %d %d\n", s.temp, s.top_p, s.top_k, s.min_p, s.repeat_penalty,
               s.repeat_last_n, (unsigned long long)s.seed, s.max_new_tokens, s.ignore_eos);
        tuff_shutdown();
        return 0;
    }
    if (argc == 7 && strcmp(argv[1], "run") == 0) return run(argv[2], argv[3], argv[4], atoi(argv[5]), argv[6]);
    fprintf(stderr, "usage: see the head of tests/capi_client.c\n");
    return 2;
}
