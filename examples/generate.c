/* Greedy generation from a C program through the engine's C boundary (tq_kv_amd/csrc/tq_engine.h),
 * in the manner of the reference's tq-kv/examples/test_ffi.c: make the handles, check every
 * status, free everything.
 *
 *   generate MODEL_DIR bfloat16|float32 MAX_NEW_TOKENS PROMPT [PROMPT ...]
 *
 * MODEL_DIR: a folder with config.json and *.safetensors (`tq random-weights` writes one).  A
 * prompt is token ids separated by commas.  The first prompt is also run through one step of the
 * step function by hand (the whole prompt, the logits of its last place copied to the host) and
 * the best token of those logits is printed, which is the first token generation gives for it.
 * Output, one line per request: "<index>: <token> <token> ...".
 *
 * Build (from the repository's root, after the libraries have been built):
 *   cc examples/generate.c -I tq_kv_amd/csrc -L tq_kv_amd/csrc -l:libtqengine_<hash>.so -Wl,-rpath,$PWD/tq_kv_amd/csrc -o generate
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "tq_engine.h"

static int fail(const char* what) {
    fprintf(stderr, "%s: %s\n", what, tqe_last_error());
    return 1;
}

static int parse_prompt(const char* text, int32_t* out, int cap) {
    int n = 0;
    const char* p = text;
    while (*p && n < cap) {
        char* end;
        long v = strtol(p, &end, 10);
        if (end == p) break;
        out[n++] = (int32_t)v;
        p = end;
        while (*p == ',' || *p == ' ') ++p;
    }
    return n;
}

int main(int argc, char** argv) {
    if (argc < 5) {
        fprintf(stderr, "usage: %s MODEL_DIR bfloat16|float32 MAX_NEW_TOKENS PROMPT [PROMPT ...]\n", argv[0]);
        return 2;
    }
    const int dtype = strcmp(argv[2], "float32") == 0 ? TQE_F32 : TQE_BF16;
    const int max_new = atoi(argv[3]);
    const int n_prompts = argc - 4;
    enum { CAP = 1 << 16 };
    int32_t* tokens = (int32_t*)malloc(sizeof(int32_t) * CAP);
    int32_t* lens = (int32_t*)malloc(sizeof(int32_t) * (size_t)n_prompts);
    int total = 0;
    for (int i = 0; i < n_prompts; ++i) {
        lens[i] = parse_prompt(argv[4 + i], tokens + total, CAP - total);
        total += lens[i];
    }

    tqe_model_t* model = tqe_model_load(argv[1], dtype, /* on_gpu */ 1, /* strict */ 1);
    if (!model) return fail("tqe_model_load");
    /* room for every request at once: prompt and new tokens, in whole pages */
    long long room = 0;
    for (int i = 0; i < n_prompts; ++i) room += (lens[i] + max_new + 2 * TQE_PAGE) / TQE_PAGE * TQE_PAGE;
    tqe_engine_t* engine = tqe_engine_new(model, room, /* max_slots */ 64, /* use_graphs */ 1);
    if (!engine) return fail("tqe_engine_new");

    /* one step by hand: the first prompt whole, the logits of its last place on the host */
    {
        const char* text = tqe_engine_describe(engine);
        if (!text) return fail("tqe_engine_describe");
        const char* at = strstr(text, "\"vocab_size\":");
        const long vocab = at ? strtol(at + 13, NULL, 10) : 0;
        if (vocab <= 0) { fprintf(stderr, "no vocabulary size in the engine's description\n"); return 1; }
        float* logits = (float*)malloc(sizeof(float) * (size_t)vocab);
        int32_t slot = -1;
        if (tqe_engine_open(engine, &slot, NULL) != TQE_OK) return fail("tqe_engine_open");
        const int32_t n_new = lens[0], want_count = 1, want_at = lens[0] - 1;
        if (tqe_step(engine, 1, &slot, &n_new, tokens, &want_count, &want_at, NULL, logits, /* on host */ 1, NULL, NULL) != TQE_OK)
            return fail("tqe_step");
        long best = 0;
        for (long v = 1; v < vocab; ++v)
            if (logits[v] > logits[best]) best = v;
        printf("step: %ld\n", best);
        if (tqe_engine_close(engine, slot) != TQE_OK) return fail("tqe_engine_close");
        free(logits);
    }

    tqe_generation_params_t params;
    tqe_generation_defaults(&params);
    params.max_tokens = max_new;
    params.temperature = 0.0f;          /* greedy */
    params.repeat_penalty = 1.0f;       /* off */
    int32_t* out = (int32_t*)calloc((size_t)n_prompts * (size_t)(max_new > 0 ? max_new : 1), sizeof(int32_t));
    int32_t* counts = (int32_t*)calloc((size_t)n_prompts, sizeof(int32_t));
    if (tqe_generate(engine, n_prompts, lens, tokens, &params, NULL, /* no stop tokens */ 0, /* max_batch */ 64, /* max_step_tokens */ 8192,
                     NULL, NULL, out, counts, NULL) != TQE_OK)
        return fail("tqe_generate");
    for (int i = 0; i < n_prompts; ++i) {
        printf("%d:", i);
        for (int k = 0; k < counts[i]; ++k) printf(" %d", out[(size_t)i * (size_t)max_new + k]);
        printf("\n");
    }

    /* a handle that is NULL is refused, not crashed on */
    if (tqe_engine_close(NULL, 0) == TQE_OK || tqe_step(NULL, 0, NULL, NULL, NULL, NULL, NULL, NULL, NULL, 0, NULL, NULL) == TQE_OK) {
        fprintf(stderr, "a NULL handle was accepted\n");
        return 1;
    }
    tqe_engine_free(engine);
    tqe_model_free(model);
    free(out); free(counts); free(tokens); free(lens);
    return 0;
}
