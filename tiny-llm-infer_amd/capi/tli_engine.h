/* The engine for C and C++ programs: requests of token ids in, tokens out.
 *
 * The surface is the reference's LLMEngine (engine/include/llm_engine.h:27-55: add_request
 * with token ids, step, is_finished, total_generated_tokens; generate is a loop over step)
 * as a C ABI.  Behind it is the engine of this package: the library starts a Python
 * interpreter in the calling process (or uses the one that is running) and drives
 * tiny_llm_infer_amd.engine.llm_engine.LLMEngine, whose device side is the HIP kernel
 * library.  Link with -ltli_engine; the package is found from the library's own place.
 *
 * Every function returns 0 on success; otherwise tli_engine_last_error() says why (for the
 * calling thread).  An engine is used from one thread at a time.
 */
#ifndef TLI_ENGINE_H_
#define TLI_ENGINE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tli_engine tli_engine;

typedef struct {
    const char* model_dir;            /* folder with config.json and model.safetensors, or NULL with config_json */
    const char* config_json;          /* a config.json for seeded random weights (model_dir NULL) */
    uint64_t weights_seed;            /* of the random weights */
    const char* dtype;                /* "bfloat16" or "float32" */
    int max_model_len;                /* most positions of a request */
    int page_size;                    /* tokens a cache page (16) */
    int num_kv_blocks;                /* cache pages; 0: from the memory left after the weights */
    int max_num_seqs;                 /* most requests in a step */
    int max_num_batched_tokens;       /* token budget of a step */
    float gpu_memory_utilization;     /* with num_kv_blocks 0 */
    int enable_prefix_caching;
} tli_engine_config;

typedef struct {
    int max_tokens;
    float temperature;                /* 0: greedy */
    float top_p;                      /* 1: off */
    int ignore_eos;
    uint64_t seed;                    /* 0: the request id */
} tli_sampling_params;

/* the defaults of the engine (bfloat16, 2048 positions, pages of 16, 16 requests, 256 tokens a step) */
void tli_engine_default_config(tli_engine_config* config);
void tli_engine_default_sampling(tli_sampling_params* sampling);

int tli_engine_create(const tli_engine_config* config, tli_engine** engine);
void tli_engine_destroy(tli_engine* engine);

int tli_engine_add_request(tli_engine* engine, const int32_t* prompt_tokens, int num_tokens,
                           const tli_sampling_params* sampling, uint64_t* request_id);

/* One step: schedule, run the batch, sample.  *num_finished requests ended in it; their results
 * stay readable with tli_engine_result until the next call of tli_engine_step. */
int tli_engine_step(tli_engine* engine, int* num_finished);
int tli_engine_result(tli_engine* engine, int index, uint64_t* request_id, const int32_t** token_ids,
                      int* num_tokens);

int tli_engine_is_finished(tli_engine* engine);                 /* 1: nothing waits or runs */
uint64_t tli_engine_total_generated_tokens(tli_engine* engine);

const char* tli_engine_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
