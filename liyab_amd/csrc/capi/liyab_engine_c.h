/* The engine as a C library: create an engine from a model folder, generate tokens, read the last
 * error. The names and meanings follow the reference's C ABI, through which all of its language
 * bindings go (include/liyab/liyab_c_api.h:128-146 parameters and statistics, :196 the token
 * callback, :223-252 liyab_engine_config_default / liyab_sampling_params_default /
 * liyab_engine_create / liyab_engine_destroy / liyab_engine_generate_tokens, liyab_last_error);
 * what concerns text (prompts as strings, tokenizing, chat templates) has no counterpart: this
 * engine takes and gives token ids.
 *
 * In this engine the loop that schedules, steps and samples is Python above native parts (the
 * HIP kernels, and the cache manager, scheduler and step metadata in C++). This library is the
 * way in for a C or C++ program: it starts a Python interpreter inside the process (or joins the
 * one that is running), imports `liyab_amd` from the tree this library was built in, and forwards
 * the calls. One engine may be driven by one thread at a time. */
#pragma once

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum liyab_status {
    LIYAB_OK = 0,
    LIYAB_INVALID_ARGUMENT = 1,
    LIYAB_INVALID_MODEL = 2,
    LIYAB_UNSUPPORTED = 3,
    LIYAB_OUT_OF_MEMORY = 4,   /* the page pool cannot hold the request */
    LIYAB_CONTEXT_FULL = 5,
    LIYAB_BUSY = 6,
    LIYAB_INTERNAL = 7,        /* the interpreter, the kernels, or anything unforeseen */
} liyab_status;

typedef struct liyab_engine liyab_engine;

typedef struct liyab_engine_config {
    const char* model_path;      /* folder with config.json and model.safetensors */
    const char* dtype;           /* "bfloat16" (default when NULL) or "float32": the precision of the whole path */
    int32_t context_length;      /* 0: the model's */
    int32_t page_size;           /* positions a cache page */
    int32_t num_pages;           /* 0: enough for every sequence at the full context */
    int32_t max_sequences;       /* requests that may run together */
    int32_t max_batched_tokens;  /* tokens a step may hold */
    int32_t prefill_chunk;       /* the longest portion of a prompt in one step */
    int32_t batch_invariant;     /* nonzero: bfloat16 replies that do not depend on the batch (slower) */
} liyab_engine_config;

typedef struct liyab_sampling_params {
    float temperature; /* <= 0: greedy */
    int32_t top_k;     /* <= 0: disabled */
    float top_p;       /* >= 1: disabled */
    uint64_t seed;     /* 0: random */
    int32_t max_tokens;
} liyab_sampling_params;

typedef struct liyab_generation_stats {
    int32_t prompt_tokens;
    int32_t generated_tokens;
    double prefill_ms;
    double ttft_ms;
    double decode_ms;
    double tokens_per_second;
    int64_t kv_cache_bytes;
    int32_t preemptions;
    int32_t cancelled;  /* the callback ended the generation */
} liyab_generation_stats;

/* Called with every generated token; returning 0 ends the generation (not an error). */
typedef int32_t (*liyab_token_callback)(int32_t token, void* user_data);

void liyab_engine_config_default(liyab_engine_config* config);
void liyab_sampling_params_default(liyab_sampling_params* params);  /* the reference's: 0.8, 40, 0.95, random, 256 */

/* Loads the model onto the GPU. *out_engine is set on success. */
liyab_status liyab_engine_create(const liyab_engine_config* config, liyab_engine** out_engine);
void liyab_engine_destroy(liyab_engine* engine);

/* Blocking generation from token ids. Up to `capacity` generated ids go to `out` (may be NULL with
 * capacity 0); *n_out (may be NULL) gets how many were generated; `callback` and `stats` may be NULL. */
liyab_status liyab_engine_generate_tokens(liyab_engine* engine, const int32_t* tokens, size_t n_tokens,
                                          const liyab_sampling_params* params, liyab_token_callback callback, void* user_data,
                                          int32_t* out, size_t capacity, size_t* n_out, liyab_generation_stats* stats);

/* The message of the calling thread's last failed call; valid until its next call. */
const char* liyab_engine_last_error(void);

#ifdef __cplusplus
}
#endif
