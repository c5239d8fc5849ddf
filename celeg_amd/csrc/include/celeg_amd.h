/* celeg_amd: a single-GPU MI355X inference engine, C interface.
 *
 * Shaped after the reference's C API (include/celeg/api.h:19-183: opaque handles, option
 * structs that carry their own size and are filled by *_options_init, status codes,
 * engine create/submit/step/poll/status/cancel/destroy/last_error; defaults
 * src/api/options.cpp:7-101), plus the low-level step function that trace replay drives and
 * the hooks through which parts and architectures defined outside this library are registered.
 *
 * An engine or a model serves one thread at a time: calls on the same handle must not overlap
 * (different handles are independent; the registries are guarded).
 *
 * Every function that can fail returns a celeg_status; the message of the last failure on the
 * calling thread is celeg_last_error().  Functions that return text return a pointer that stays
 * valid until the calling thread's next call of a function of this library that returns text.
 */
#ifndef CELEG_AMD_H
#define CELEG_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct celeg_engine celeg_engine;   /* scheduler + sampler + step function */
typedef struct celeg_model celeg_model;     /* the step function alone: model, cache manager, runner */

typedef enum celeg_status {
    CELEG_OK = 0,
    CELEG_ERROR = 1,              /* a run-time failure; see celeg_last_error() */
    CELEG_INVALID_ARGUMENT = 2,
    CELEG_NOT_FOUND = 3           /* unknown request id */
} celeg_status;

typedef enum celeg_request_status {
    CELEG_REQUEST_QUEUED = 0,
    CELEG_REQUEST_PREFILL = 1,
    CELEG_REQUEST_DECODING = 2,
    CELEG_REQUEST_FINISHED = 3,
    CELEG_REQUEST_CANCELLED = 4,
    CELEG_REQUEST_FAILED = 5
} celeg_request_status;

enum { CELEG_POLICY_MAX_UTILIZATION = 0, CELEG_POLICY_GUARANTEED_NO_EVICT = 1 };
/* how bfloat16 steps of more than 64 rows multiply: the library's products, this library's tiled
 * products with norm, SwiGLU and residual sum folded in, or (the default) whichever was measured
 * faster at the model's width */
enum { CELEG_GEMM_LIBRARY = 0, CELEG_GEMM_TILES = 1, CELEG_GEMM_AUTO = 2 };

/* temperature 0.1, top_k 50, top_p 1, repetition_penalty 1.05, seed 1
 * (include/celeg/model/runtime_types.hpp:98-108); greedy when temperature <= 0 or top_k == 1 */
typedef struct celeg_generation_options {
    size_t struct_size;
    float temperature;
    int32_t top_k;
    float top_p;
    float repetition_penalty;
    uint64_t seed;
    /* tokens given out as the request's first generated tokens instead of sampled ones (they are
     * polled, counted and checked against the end tokens like sampled ones; the request's generator
     * is not advanced for them): ForcedTokenPrefix, include/celeg/model/runtime_types.hpp:93-104,
     * src/backend/cpu/sampler.cpp:31-34.  Copied at submission; null or 0: none. */
    const int32_t* forced_prefix;
    int32_t n_forced_prefix;
} celeg_generation_options;

/* max_active_requests 8, page_tokens 16, logical_kv_pages 0 (= enough for every request at the
 * full context), max-utilization policy as include/celeg/backend/cuda/concurrency.hpp:18-32;
 * max_batched_tokens 2048 and prefill_chunk_tokens 1024 (the reference's 512 / 256 leave an
 * MI355X idle); context 0 = the model's own maximum; dtype "bfloat16" or "float32" */
typedef struct celeg_engine_options {
    size_t struct_size;
    const char* dtype;
    int32_t device;
    int32_t max_active_requests;
    int32_t max_batched_tokens;
    int32_t prefill_chunk_tokens;
    int32_t page_tokens;
    int32_t logical_kv_pages;
    int32_t scheduler_policy;
    int32_t context;
    int32_t gemm_backend;
    int32_t use_graphs;          /* 1: decode steps are replayed from recorded HIP graphs */
    int32_t run_ahead;           /* 1: celeg_engine_run launches decode steps one ahead of their tokens */
    int32_t portion_granule;
    /* 0 (the default): tensors of the checkpoint that the model has no use for are named in a
     * warning on stderr and in celeg_model_describe ("unused_tensors"), as the reference binds by
     * name and leaves the rest alone; 1: they are an error */
    int32_t strict_weights;
} celeg_engine_options;

/* max_new_tokens 128, priority 0 (include/celeg/runtime/request_types.hpp:16-26);
 * n_eos_token_ids < 0: the model's own end tokens */
typedef struct celeg_request_options {
    size_t struct_size;
    int32_t max_new_tokens;
    const int32_t* eos_token_ids;
    int32_t n_eos_token_ids;
    int32_t priority;
    celeg_generation_options generation;
} celeg_request_options;

void celeg_generation_options_init(celeg_generation_options* options, size_t struct_size);
void celeg_engine_options_init(celeg_engine_options* options, size_t struct_size);
void celeg_request_options_init(celeg_request_options* options, size_t struct_size);

const char* celeg_last_error(void);
const char* celeg_version(void);
/* what this build can run and on what, in a sentence (the reference's celeg_backend_capabilities,
 * include/celeg/api.h:150, answers likewise for a backend's name; here there is one backend) */
const char* celeg_backend_capabilities(void);

/* ---- the engine ---- */
celeg_status celeg_engine_create(const char* model_dir, const celeg_engine_options* options, celeg_engine** out);
void celeg_engine_destroy(celeg_engine* engine);
celeg_status celeg_engine_submit(celeg_engine* engine, const int32_t* tokens, int32_t n_tokens,
                                 const celeg_request_options* options, int64_t* request_id);
/* one batch: admits, runs, samples, frees; tokens_fed may be null */
celeg_status celeg_engine_step(celeg_engine* engine, int32_t* tokens_fed);
/* steps until nothing is queued or active */
celeg_status celeg_engine_run(celeg_engine* engine);
/* at most `limit` steps (a step that was launched ahead is completed before the call returns) */
celeg_status celeg_engine_run_steps(celeg_engine* engine, int64_t limit, int64_t* steps);
celeg_status celeg_engine_has_work(celeg_engine* engine, int32_t* has_work);
/* drains up to `capacity` tokens generated since the last poll */
celeg_status celeg_engine_poll(celeg_engine* engine, int64_t request_id, int32_t* tokens, int32_t capacity,
                               int32_t* n_tokens, int32_t* status);
celeg_status celeg_engine_status(celeg_engine* engine, int64_t request_id, int32_t* status);
celeg_status celeg_engine_cancel(celeg_engine* engine, int64_t request_id);
/* forgets a request that has ended (its id is unknown afterwards); a request that is queued or running
 * is refused with CELEG_INVALID_ARGUMENT.  An engine keeps the record of every request until this call. */
celeg_status celeg_engine_release(celeg_engine* engine, int64_t request_id);
/* the message of a Failed request ("" otherwise) */
const char* celeg_engine_request_error(celeg_engine* engine, int64_t request_id);
const char* celeg_engine_last_error(celeg_engine* engine);
/* JSON: counters of the engine, the scheduler, the runner and the cache */
const char* celeg_engine_metrics(celeg_engine* engine);
/* JSON: prompt and generated tokens, time to first token, mean and longest time between tokens */
const char* celeg_engine_request_metrics(celeg_engine* engine, int64_t request_id);
/* the last step's logits, 32-bit [rows, vocab]; copies min(capacity, rows * vocab) floats */
celeg_status celeg_engine_last_logits(celeg_engine* engine, float* out, size_t capacity, int32_t* rows, int32_t* vocab);
/* the model underneath (owned by the engine) */
celeg_model* celeg_engine_model(celeg_engine* engine);

/* ---- the step function alone (what trace replay and tests drive) ---- */
celeg_status celeg_model_create(const char* model_dir, const celeg_engine_options* options, celeg_model** out);
void celeg_model_destroy(celeg_model* model);
/* JSON: {"config": typed configuration, "spec": model description, "cache_layout": .., "vocab_size", "max_context",
 *        "page_tokens", "max_requests", "graph_safe", "logit_width", "gemm_backend": "library" | "tiles" (what
 *        CELEG_GEMM_AUTO became)} */
const char* celeg_model_describe(celeg_model* model);
celeg_status celeg_model_open_slot(celeg_model* model, int32_t* slot);      /* -1: every slot is taken */
celeg_status celeg_model_close_slot(celeg_model* model, int32_t slot);
/* pages for positions [start, start + n): *ok 0 (and nothing taken) if the pool has too few */
celeg_status celeg_model_prepare(celeg_model* model, int32_t slot, int32_t start, int32_t n, int32_t* ok);
celeg_status celeg_model_check_cache(celeg_model* model);
/* JSON: {"free_slots", "free_pages": [..], "open_slots": [..], "pages_held": {slot: [[..]]}, "memory": ..} */
const char* celeg_model_cache_state(celeg_model* model);
/* One step.  Entry i: slot[i], start_pos[i], its n_tokens[i] tokens and n_want[i] wanted places, the
 * tokens and the places of all entries one after the other in `tokens` and `want`.  Writes the logits at
 * the wanted places, in the order of the entries and of their places, [sum n_want, logit width] 32-bit,
 * to `logits` (host memory of `capacity` floats; may be null if nothing is wanted). */
celeg_status celeg_model_step(celeg_model* model, int32_t n_entries, const int32_t* slot, const int32_t* start_pos,
                              const int32_t* n_tokens, const int32_t* tokens, const int32_t* n_want,
                              const int32_t* want, float* logits, size_t capacity);
/* ---- one request at a time on a model of its own (the reference's celeg_model_prefill / decode /
 * copy_logits / get_metrics, include/celeg/api.h:158-164, src/api/model.cpp:32-77): prefill starts a new
 * sequence with a prompt (what the model held of an earlier one is given back); decode chooses the next
 * token from the logits of the last step (by the generation options: celeg_generation_options_init's
 * defaults unless set), feeds it, and returns it; copy_logits gives the logits the next decode will
 * choose from.  Not for a model that belongs to an engine. ---- */
typedef struct celeg_metrics {
    size_t struct_size;
    double prefill_ms;          /* the last prefill */
    uint64_t prefill_tokens;
    double decode_ms;           /* all decode calls since that prefill */
    uint64_t decode_tokens;
} celeg_metrics;
/* the options of the sequences that later prefills start (null: the defaults) */
celeg_status celeg_model_set_generation(celeg_model* model, const celeg_generation_options* options);
celeg_status celeg_model_prefill(celeg_model* model, const int32_t* tokens, size_t count);
celeg_status celeg_model_decode(celeg_model* model, int32_t* token);
/* *required: the number of logits; CELEG_ERROR if output is null or capacity is smaller */
celeg_status celeg_model_copy_logits(celeg_model* model, float* output, size_t capacity, size_t* required);
celeg_status celeg_model_get_metrics(celeg_model* model, celeg_metrics* metrics);

/* knobs of the runner and the kernels' dispatch, by name (tests and tuning); JSON of the known names
 * and their values comes back from celeg_model_knobs */
celeg_status celeg_model_set_knob(celeg_model* model, const char* name, int32_t value);
const char* celeg_model_knobs(celeg_model* model);
/* Times of a step's phases (embedding, every layer's mixer and feed-forward, head), taken with events on
 * the stream: switched on here or by the environment variable CELEG_PROFILE_PHASES=1 at load time; steps
 * that are timed are not replayed from recorded graphs.  JSON {"steps", "tokens", "phases": {name:
 * {"ms", "calls"}}}, or "null" when nothing is timed.  With the environment variable set, a table is
 * also printed to stderr when the model goes.  CELEG_DUMP_HIDDEN=<folder> at load time writes the 32-bit
 * residual stream after every entry of the run order to <folder>/step<k>_layer<i>.f32 ([rows, width]). */
celeg_status celeg_model_time_phases(celeg_model* model, int32_t on);
const char* celeg_model_phase_times(celeg_model* model);
/* the raw HIP stream the model's work runs on */
void* celeg_model_stream(celeg_model* model);
/* waits for everything launched on that stream */
celeg_status celeg_model_synchronize(celeg_model* model);

/* ---- the kernels' dispatcher alone (tests of single kernels) ----
 * A dispatcher of its own (workspace, library plans, tables of cosines and sines): the same class the parts
 * of a model call, with its shape checks and its choice of kernel.  celeg_ops_call runs the method that `op`
 * names ("linear", "rmsnorm", "short_conv", "qk_norm_rope_store", "paged_attention", "fused_linear",
 * "tiled_linear", "sample", ...; "state" runs nothing) on `stream` (a hipStream_t) with the arguments in
 * args_json: tensors as {"data": address, "dtype": "float32" | "bfloat16" | "int32" | "uint8", "shape": [...],
 * "stride": [...]} (strides in elements), arrays of a step as addresses, a step and a cache view as objects of
 * addresses and counts, and optionally "knobs": {name: value} set before the call.  It returns JSON
 * ({"last_stat_blocks": n, ...}; "state" adds "paths", the launches counted by kernel family) that stays
 * valid until the next call on the same handle, or NULL with the reason in celeg_last_error(): a size that a
 * kernel does not take is refused here, before anything is launched. */
typedef struct celeg_ops celeg_ops;
celeg_status celeg_ops_create(celeg_ops** out);
void celeg_ops_destroy(celeg_ops* ops);
const char* celeg_ops_call(celeg_ops* ops, const char* op, const char* args_json, void* stream);

/* ---- plain C++ functions for what the kernels compute, on host memory (tests) ----
 * One beside each kernel (host/reference.cpp: loops in 32-bit floats over the same layouts of the cache pages
 * and the state slots): "embed", "rmsnorm", "linear", "swiglu", "short_conv", "qk_norm_rope", "kv_store",
 * "paged_attention", "sample".  args_json holds host addresses (as integers) and sizes under the functions'
 * parameter names.  Returns JSON ("sample": {"token": n}) or NULL with the reason in celeg_last_error().
 * Needs no GPU. */
const char* celeg_reference_call(const char* op, const char* args_json);

/* ---- without a GPU: what a folder holds ---- */
/* JSON {"config", "spec", "expected_tensors": [{"name", "shape", "kind", "init", "also"}]} of a model
 * folder (config.json, generation_config.json, and the checkpoint's tensor names for what they leave out) */
const char* celeg_describe_folder(const char* model_dir);
/* the same from a config.json text alone (shapes_json: {"name": [dims]} or null) */
const char* celeg_describe_config(const char* config_json, const char* shapes_json);
/* checks the folder's checkpoint against the model: CELEG_OK, or CELEG_ERROR with one message that lists
 * missing and unexpected tensors and wrong shapes.  A checkpoint that only holds tensors the model has no
 * use for passes (celeg_describe_folder names them under "unused_tensors") unless `strict`. */
celeg_status celeg_check_folder(const char* model_dir);
celeg_status celeg_check_folder_strict(const char* model_dir, int32_t strict);
const char* celeg_registered(const char* what);   /* "architectures", or a role of parts: JSON list of names */

/* ---- the host-side objects by themselves, without a GPU, by JSON calls (tests of the bookkeeping) ----
 * kinds: "pool", "cache", "scheduler", "batch"; see host/host_api.cpp for their arguments and methods.
 * celeg_host_new returns 0, celeg_host_call null, on failure (celeg_last_error() then starts with the
 * kind of error, e.g. "PageError: "). */
long long celeg_host_new(const char* kind, const char* args_json);
const char* celeg_host_call(long long handle, const char* method, const char* args_json);
void celeg_host_delete(long long handle);

/* ---- parts and architectures defined outside this library ---- */
typedef struct celeg_tensor_view {
    void* data;                 /* device memory */
    int32_t dtype;              /* 0 float32, 1 bfloat16, 2 int32, 3 uint8 */
    int32_t ndim;
    int64_t shape[4];
    int64_t stride[4];          /* in elements */
} celeg_tensor_view;

typedef struct celeg_step_view {
    int32_t n_tokens, n_seqs, n_logit_rows, decode_only, single_rows;
    /* device arrays (see the batch layout): */
    const int32_t *token_ids, *positions, *token_seq, *token_slot, *cu_seqlens, *seq_slot, *seq_start, *logit_rows;
    /* host copies for parts that plan on the host: */
    const int32_t *host_seq_slot, *host_seq_start, *host_cu_seqlens;
} celeg_step_view;

typedef struct celeg_cache_view {
    int32_t has_kv, writes_kv;
    void *k, *v;                /* K [n_pages, layers, kv_heads, page_tokens, head_dim], V [n_pages, layers, kv_heads, v_head_dim, page_tokens] */
    int32_t kv_dtype, layer, n_layers, page_tokens, kv_heads, head_dim, table_stride;
    const int32_t* table;       /* [slots + 1, table_stride] */
    int32_t n_states;
    const char* const* state_names;
    const celeg_tensor_view* states;    /* [slots + 1, shape...] each */
    int32_t v_head_dim, n_pages;        /* width of a value; pages of the pool, the spare one included */
} celeg_cache_view;

typedef struct celeg_forward_args {
    celeg_tensor_view x;        /* mixer, feed-forward: normalised rows; norm: the 32-bit stream; head: rows */
    celeg_tensor_view out;      /* where the result goes (allocated by the caller) */
    celeg_tensor_view delta;    /* norm: an addition to x to make first (data null: none) */
    const int32_t* rows;        /* norm: rows to read (null: all) */
    const int32_t* token_ids;   /* embedding */
    celeg_step_view step;
    celeg_cache_view cache;
    void* stream;
    int32_t dtype;              /* the run's activation dtype */
} celeg_forward_args;

/* A part as functions.  describe() returns JSON:
 *   {"weights": {role: {"shape": [..], "kind": "matrix"|"vector", "init": "normal"|"around_one"}},
 *    "kv_need": {"kv_heads", "head_dim", "window", "v_head_dim" (optional: values of another width)} or null, "states": [{"name", "shape", "dtype"}],
 *    "graph_safe": bool, "out_width": columns of what forward writes (mixer, ffn),
 *    "inv_freq": [..], "rotary_dim": n, "pairing": "halves"|"neighbours"  (position encodings: pair i of
 *    the first n values of a head, (i, i + n/2) or (2i, 2i + 1), turns by position * inv_freq[i])}
 * load() receives the tensors by role; forward() returns 0 or an error code. */
typedef struct celeg_part_functions {
    void* self;
    const char* (*describe)(void* self);
    int32_t (*load)(void* self, int32_t n, const char* const* roles, const celeg_tensor_view* tensors);
    int32_t (*forward)(void* self, const celeg_forward_args* args);
    void (*destroy)(void* self);
} celeg_part_functions;

/* builds a part from its spec ({"kind", "params", "tensors"} as JSON); returns 0 or an error code */
typedef int32_t (*celeg_part_factory)(const char* spec_json, void* user, celeg_part_functions* out);
/* role: "norm", "mixer", "ffn", "position", "embedding" or "head" */
celeg_status celeg_register_part(const char* role, const char* kind, celeg_part_factory factory, void* user);

/* turns config.json (and the checkpoint's tensor shapes, or "null") into JSON {"config": .., "spec": ..};
 * returns null on failure */
typedef const char* (*celeg_architecture_describe)(const char* config_json, const char* shapes_json, void* user);
celeg_status celeg_register_architecture(const char* name, celeg_architecture_describe describe, void* user);

#ifdef __cplusplus
}
#endif
#endif
