/* A C program that uses the engine through its C library and nothing else: creates an engine
 * from the folder in argv[1] (float32), generates argv[2] greedy tokens from the prompt ids that
 * follow, prints them on one line, then generates again with a callback that stops after three
 * tokens, and finally asks for a folder that does not exist. Used by tests/test_capi_gpu.py. */
#include <stdio.h>
#include <stdlib.h>

#include "liyab_engine_c.h"

static int32_t seen[64];
static int n_seen = 0;

static int32_t stop_after_three(int32_t token, void* user) {
    (void)user;
    seen[n_seen++] = token;
    return n_seen < 3;
}

int main(int argc, char** argv) {
    if (argc < 4) return 2;
    liyab_engine_config cfg;
    liyab_engine_config_default(&cfg);
    cfg.model_path = argv[1];
    cfg.dtype = "float32";
    cfg.max_sequences = 2;
    liyab_engine* engine = NULL;
    if (liyab_engine_create(&cfg, &engine) != LIYAB_OK) {
        fprintf(stderr, "create: %s\n", liyab_engine_last_error());
        return 1;
    }
    const int n_new = atoi(argv[2]);
    int32_t prompt[256];
    size_t n_prompt = 0;
    for (int i = 3; i < argc && n_prompt < 256; ++i) prompt[n_prompt++] = atoi(argv[i]);
    liyab_sampling_params sp;
    liyab_sampling_params_default(&sp);
    sp.temperature = 0.0f;
    sp.max_tokens = n_new;
    int32_t out[256];
    size_t n_out = 0;
    liyab_generation_stats stats;
    if (liyab_engine_generate_tokens(engine, prompt, n_prompt, &sp, NULL, NULL, out, 256, &n_out, &stats) != LIYAB_OK) {
        fprintf(stderr, "generate: %s\n", liyab_engine_last_error());
        return 1;
    }
    printf("tokens");
    for (size_t i = 0; i < n_out; ++i) printf(" %d", out[i]);
    printf("\nstats %d %d %d\n", stats.prompt_tokens, stats.generated_tokens, stats.cancelled);
    if (liyab_engine_generate_tokens(engine, prompt, n_prompt, &sp, stop_after_three, NULL, out, 256, &n_out, &stats) != LIYAB_OK) {
        fprintf(stderr, "generate with a callback: %s\n", liyab_engine_last_error());
        return 1;
    }
    printf("stopped %zu %d %d %d %d\n", n_out, stats.cancelled, seen[0], seen[1], seen[2]);
    prompt[0] = 1 << 30; /* no such token */
    liyab_status st = liyab_engine_generate_tokens(engine, prompt, n_prompt, &sp, NULL, NULL, out, 256, &n_out, NULL);
    printf("bad token: status %d: %s\n", (int)st, liyab_engine_last_error());
    liyab_engine_destroy(engine);
    cfg.model_path = "/no/such/folder";
    st = liyab_engine_create(&cfg, &engine);
    printf("bad folder: status %d: %s\n", (int)st, liyab_engine_last_error());
    return 0;
}
