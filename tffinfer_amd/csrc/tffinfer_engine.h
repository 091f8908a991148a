// The engine for callers in C and C++: requests in, tokens (or logits) out.
//
// The reference exports its runtime class through a visibility macro (DEEP_TFF_API,
// include/ExportInc.h:6-16; class LLMInferRuntime, src/core/runtime/InferRuntime.h:32-45:
// load_model, init_runtime_context, encode, infer).  Here the same life cycle is cut into
// requests and steps, as a continuous-batching engine needs it, and exported as plain C.
//
// The engine behind these calls is the package's own (scheduler, step function, cache manager,
// kernels); its host side is Python, so the library (libtffinfer_engine.so) holds an interpreter:
// it starts one in a process that has none and uses the running one otherwise (a Python process
// that loads the library through ctypes).  Calls may come from any thread, one at a time per
// engine; the library takes the interpreter's lock around each.
//
// Every call that can fail returns NULL or a negative number and leaves a message for
// engine_last_error(), per thread.
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(TFF_ENGINE_BUILD)
#define TFF_ENGINE_API __attribute__((visibility("default")))
#else
#define TFF_ENGINE_API
#endif

typedef struct tff_engine tff_engine;

// A token that a step gave to a request.  token is -1 where the request ended without one
// (it was dropped because the cache cannot hold it even alone).
typedef struct {
    int64_t request_id;
    int32_t token;
    int32_t finished;      // 1: the request has ended with this event (length, stop token, abort, dropped)
} tff_step_event;

// One request's share of a raw step: its next tokens, and the places among them whose logits are asked for.
typedef struct {
    int64_t request_id;    // the caller's own numbering; apart from that of engine_add_request
    const int32_t* tokens;
    int32_t n_tokens;
    const int32_t* want;   // indices into tokens, may be empty
    int32_t n_want;
} tff_raw_entry;

// options_json: a JSON object with any of dtype ("bfloat16", "float32"), device, page_size,
// num_pages | kv_tokens | kv_bytes, max_num_seqs, max_num_batched_tokens, prefill_chunk,
// max_model_len, memory_fraction, use_graphs, run_ahead, warm_up, token_quantum; NULL or "" for the defaults.
// model_dir: a folder with config.json and model.safetensors; the model class is chosen by config.json.
TFF_ENGINE_API tff_engine* engine_create(const char* model_dir, const char* options_json);
// Seeded random weights for the configuration in config_json_file, no weight files.
TFF_ENGINE_API tff_engine* engine_create_random(const char* config_json_file, uint64_t seed, const char* options_json);
TFF_ENGINE_API void engine_destroy(tff_engine* e);
TFF_ENGINE_API int engine_vocab_size(tff_engine* e);

// params_json: max_new_tokens, eos_token_id, ignore_eos, sampling {type, temperature, top_k, top_p,
// min_p, repetition_penalty, seed}; NULL or "" for greedy and 64 tokens.  Returns the request's id.
TFF_ENGINE_API int64_t engine_add_request(tff_engine* e, const int32_t* token_ids, int32_t n, const char* params_json);
// Plans and runs one step (prompt portions beside decoded tokens, as the scheduler cuts them) and
// writes its events, at most capacity of them; returns their number.  Events that did not fit are
// returned by the next calls, before any new step runs.
TFF_ENGINE_API int engine_step(tff_engine* e, tff_step_event* events, int capacity);
TFF_ENGINE_API int engine_has_work(tff_engine* e);            // 1 while requests wait, run or have events left
TFF_ENGINE_API int engine_abort(tff_engine* e, int64_t request_id);   // 1 if the request was live

// One call of the step function with the entries as given: no scheduler, no sampling.  logits
// receives float32 [wanted, vocab] in the order of the entries and of want; capacity_floats is
// the room there.  Returns the number of rows written.  A request is opened by its first entry
// and holds its cache until engine_end_raw.
TFF_ENGINE_API int engine_step_raw(tff_engine* e, const tff_raw_entry* entries, int n_entries, float* logits,
                                   int64_t capacity_floats);
TFF_ENGINE_API int engine_end_raw(tff_engine* e, int64_t request_id);   // 1 if the request was open

// The message of the last call that failed on this thread ("" if none).
TFF_ENGINE_API const char* engine_last_error(void);

#ifdef __cplusplus
}
#endif
