/* A client of the C interface, in plain C: what a user of the reference's celeg_engine_* calls
 * (include/celeg/api.h:19-183) would write.
 *
 *   drive_engine describe MODEL_DIR
 *       without a GPU: version, option defaults, the folder's description, and the message a
 *       folder that is not there gives.
 *   drive_engine generate MODEL_DIR DTYPE MAX_NEW "1,2,3" "4,5" ...
 *       submits every prompt, steps until nothing is left, polls while it steps, cancels
 *       nothing; prints one line "tokens <request>: ..." per request, then "metrics {json}".
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "celeg_amd.h"

static int fail(const char* what) {
    fprintf(stderr, "%s: %s\n", what, celeg_last_error());
    return 1;
}

static int parse_tokens(const char* text, int32_t* out, int capacity) {
    int n = 0;
    const char* p = text;
    while (*p && n < capacity) {
        char* end;
        long v = strtol(p, &end, 10);
        if (end == p) break;
        out[n++] = (int32_t)v;
        p = (*end == ',') ? end + 1 : end;
    }
    return n;
}

static int describe(const char* dir) {
    celeg_engine_options eo;
    celeg_request_options ro;
    celeg_generation_options go;
    celeg_engine_options_init(&eo, sizeof eo);
    celeg_request_options_init(&ro, sizeof ro);
    celeg_generation_options_init(&go, sizeof go);
    printf("version %s\n", celeg_version());
    printf("capabilities %s\n", celeg_backend_capabilities());
    printf("forced_prefix_default %d %d\n", go.forced_prefix == NULL, go.n_forced_prefix);
    printf("engine_defaults %s %d %d %d %d %d\n", eo.dtype, eo.max_active_requests, eo.max_batched_tokens,
           eo.prefill_chunk_tokens, eo.page_tokens, eo.scheduler_policy);
    printf("request_defaults %d %d %d\n", ro.max_new_tokens, ro.n_eos_token_ids, ro.priority);
    printf("generation_defaults %.2f %d %.2f %.2f %llu\n", go.temperature, go.top_k, go.top_p, go.repetition_penalty,
           (unsigned long long)go.seed);
    const char* text = celeg_describe_folder(dir);
    if (!text) return fail("describe");
    printf("described %zu bytes\n", strlen(text));
    if (celeg_check_folder(dir) != CELEG_OK) return fail("check");
    printf("checked\n");
    if (celeg_describe_folder("/nonexistent/model") != NULL) return 1;
    printf("missing: %s\n", celeg_last_error());
    if (celeg_engine_create(dir, NULL, NULL) != CELEG_INVALID_ARGUMENT) return 1;
    printf("refused: %s\n", celeg_last_error());
    return 0;
}

static int generate(int argc, char** argv) {
    const char* dir = argv[2];
    celeg_engine_options eo;
    celeg_engine_options_init(&eo, sizeof eo);
    eo.dtype = argv[3];
    eo.max_active_requests = 2;          /* fewer than the prompts: some wait their turn */
    eo.max_batched_tokens = 32;
    eo.prefill_chunk_tokens = 8;
    eo.logical_kv_pages = 16;
    celeg_engine* engine = NULL;
    if (celeg_engine_create(dir, &eo, &engine) != CELEG_OK) return fail("create");

    const int n_requests = argc - 5;
    int64_t ids[16];
    int32_t generated[16][256];
    int counts[16] = {0};
    if (n_requests > 16) return 1;
    celeg_request_options ro;
    celeg_request_options_init(&ro, sizeof ro);
    ro.max_new_tokens = atoi(argv[4]);
    ro.n_eos_token_ids = 0;              /* no end token: every request runs to max_new_tokens */
    ro.generation.temperature = 0.0f;    /* greedy */
    ro.generation.repetition_penalty = 1.0f;
    for (int r = 0; r < n_requests; ++r) {
        int32_t prompt[512];
        const int n = parse_tokens(argv[5 + r], prompt, 512);
        if (celeg_engine_submit(engine, prompt, n, &ro, &ids[r]) != CELEG_OK) return fail("submit");
    }
    /* a request that cannot be: refused at the door, the engine goes on */
    int64_t bad;
    if (celeg_engine_submit(engine, NULL, 0, &ro, &bad) == CELEG_OK) return 1;

    int32_t has_work = 1;
    long steps = 0;
    while (has_work) {
        int32_t fed = 0;
        if (celeg_engine_step(engine, &fed) != CELEG_OK) return fail("step");
        ++steps;
        for (int r = 0; r < n_requests; ++r) {
            int32_t n = 0, status = 0;
            if (celeg_engine_poll(engine, ids[r], generated[r] + counts[r], 256 - counts[r], &n, &status) != CELEG_OK)
                return fail("poll");
            counts[r] += n;
            if (status == CELEG_REQUEST_FAILED) {
                fprintf(stderr, "request %lld failed: %s\n", (long long)ids[r], celeg_engine_request_error(engine, ids[r]));
                return 1;
            }
        }
        if (celeg_engine_has_work(engine, &has_work) != CELEG_OK) return fail("has_work");
        if (steps > 10000) return 1;
    }
    for (int r = 0; r < n_requests; ++r) {
        int32_t status = -1;
        if (celeg_engine_status(engine, ids[r], &status) != CELEG_OK || status != CELEG_REQUEST_FINISHED) return 1;
        printf("tokens %d:", r);
        for (int i = 0; i < counts[r]; ++i) printf(" %d", generated[r][i]);
        printf("\n");
    }
    int32_t status = 0;
    if (celeg_engine_status(engine, 123456, &status) != CELEG_NOT_FOUND) return 1;
    /* records go when they are released: a running request is refused, an ended one is unknown afterwards */
    int64_t late;
    int32_t one_token[1] = {1};
    if (celeg_engine_submit(engine, one_token, 1, &ro, &late) != CELEG_OK) return fail("submit");
    if (celeg_engine_release(engine, late) != CELEG_INVALID_ARGUMENT) return 1;
    if (celeg_engine_cancel(engine, late) != CELEG_OK || celeg_engine_run(engine) != CELEG_OK) return fail("cancel");
    if (celeg_engine_release(engine, late) != CELEG_OK) return fail("release");
    for (int r = 0; r < n_requests; ++r)
        if (celeg_engine_release(engine, ids[r]) != CELEG_OK) return fail("release");
    if (celeg_engine_status(engine, ids[0], &status) != CELEG_NOT_FOUND) return 1;
    if (celeg_engine_release(engine, ids[0]) != CELEG_NOT_FOUND) return 1;
    printf("metrics %s\n", celeg_engine_metrics(engine));
    celeg_engine_destroy(engine);
    return 0;
}

int main(int argc, char** argv) {
    if (argc >= 3 && strcmp(argv[1], "describe") == 0) return describe(argv[2]);
    if (argc >= 6 && strcmp(argv[1], "generate") == 0) return generate(argc, argv);
    fprintf(stderr, "usage: drive_engine describe DIR | generate DIR DTYPE MAX_NEW PROMPT...\n");
    return 2;
}
