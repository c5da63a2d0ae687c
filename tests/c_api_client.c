/* A C program that serves requests through the engine's C ABI: usage
 *   c_api_client MODEL_DIR DTYPE MAX_TOKENS PROMPT [PROMPT ...]     (a prompt: comma-separated token ids)
 * prints, for every request in the order of the prompts, its new token ids on one line, then a
 * line "generated N". */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "tli_engine.h"

#define MAX_REQ 16

static int die(const char* what) {
    fprintf(stderr, "%s: %s\n", what, tli_engine_last_error());
    return 1;
}

int main(int argc, char** argv) {
    if (argc < 5 || argc - 4 > MAX_REQ) return 2;
    tli_engine_config config;
    tli_engine_default_config(&config);
    config.model_dir = argv[1];
    config.dtype = argv[2];
    config.max_model_len = 128;
    config.page_size = 8;
    config.num_kv_blocks = 48;
    config.max_num_seqs = 4;
    config.max_num_batched_tokens = 24;
    tli_engine* engine = NULL;
    if (tli_engine_create(&config, &engine)) return die("create");

    tli_sampling_params sampling;
    tli_engine_default_sampling(&sampling);
    sampling.max_tokens = atoi(argv[3]);
    sampling.ignore_eos = 1;
    uint64_t ids[MAX_REQ];
    int n_req = argc - 4;
    for (int r = 0; r < n_req; ++r) {
        int32_t prompt[512];
        int n = 0;
        char* copy = strdup(argv[4 + r]);
        for (char* tok = strtok(copy, ","); tok && n < 512; tok = strtok(NULL, ",")) prompt[n++] = atoi(tok);
        free(copy);
        if (tli_engine_add_request(engine, prompt, n, &sampling, &ids[r])) return die("add_request");
    }
    /* a request that cannot be served is refused with a message, and the engine goes on */
    int32_t bad[1] = {-5};
    if (tli_engine_add_request(engine, bad, 1, &sampling, NULL) == 0) return 3;
    fprintf(stderr, "refused as expected: %s\n", tli_engine_last_error());

    static int32_t out[MAX_REQ][256];
    int out_n[MAX_REQ] = {0};
    while (!tli_engine_is_finished(engine)) {
        int done = 0;
        if (tli_engine_step(engine, &done)) return die("step");
        for (int i = 0; i < done; ++i) {
            uint64_t id;
            const int32_t* tokens;
            int n;
            if (tli_engine_result(engine, i, &id, &tokens, &n)) return die("result");
            for (int r = 0; r < n_req; ++r)
                if (ids[r] == id) {
                    memcpy(out[r], tokens, (size_t)n * sizeof(int32_t));
                    out_n[r] = n;
                }
        }
    }
    for (int r = 0; r < n_req; ++r) {
        for (int i = 0; i < out_n[r]; ++i) printf(i ? " %d" : "%d", out[r][i]);
        printf("\n");
    }
    printf("generated %llu\n", (unsigned long long)tli_engine_total_generated_tokens(engine));
    tli_engine_destroy(engine);
    return 0;
}
