/* C entry points of the engine: configuration, weights, models, the cache, the step function,
 * sampling and the generation loop.
 *
 * In the manner of the reference's C boundary (tq-kv/include/tq_kv.h:27-84,
 * tq-kv/src/ffi.rs:89-108): opaque handles that the library makes and frees, plain C
 * types, int32 status (0 ok, negative error), a message for the last error of the
 * calling thread.  No C++ exception crosses it.  Strings the library returns belong to it and
 * stay valid until the calling thread's next call into the library.
 *
 * The bookkeeping entry points (tqe_cache_*, tqe_plan_*, tqe_batch_*) touch no GPU and take host
 * pointers only.  The model and engine entry points say of each pointer where it lives; `stream`
 * is a hipStream_t (NULL: the default stream), and everything an engine does is ordered on the
 * stream it is called with: use one stream per engine at a time.
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TQE_PAGE 64             /* positions per cache page (the kernel library is asked for its own and must agree) */
#define TQE_KERNEL_ABI 13       /* the version of the kernel library's interface (tqk_abi_version) this engine is written against */
#define TQE_MAX_GROUPS 16       /* groups of cached runs a cache may have */

enum {
    TQE_OK = 0,
    TQE_ERR_ARGUMENT = -1,      /* null pointer, number out of range */
    TQE_ERR_FULL = -2,          /* no free slot, or not enough free pages: nothing was changed */
    TQE_ERR_STATE = -3,         /* a slot that is not held, something freed twice, a broken invariant */
    TQE_ERR_RANGE = -4,         /* a wanted place outside its sequence's tokens */
    TQE_ERR_STEP = -5,          /* a step the engine cannot run: see tqe_check_step */
    TQE_ERR_CONFIG = -6,        /* a config.json that cannot be used: missing key, wrong type, bad combination, unknown architecture */
    TQE_ERR_WEIGHTS = -7,       /* missing tensors, unexpected tensors, wrong shapes or kinds: the message lists all of them */
    TQE_ERR_WEIGHT_FILE = -8,   /* a folder or safetensors file that cannot be read */
    TQE_ERR_DEVICE = -9,        /* the GPU runtime or a library on it failed; no kernel library */
    TQE_ERR_KERNEL = -10,       /* a kernel entry point refused its arguments */
    TQE_ERR_GENERATION = -11,   /* requests the loop cannot serve: an empty prompt, more positions than the model has, more than the cache holds */
    TQE_ERR_PART = -12,         /* a part registered by the caller failed */
    TQE_NO_LIST = -100          /* tqe_cache_pages: the slot has no page list in the group (not an error) */
};

const char* tqe_last_error(void);
int tqe_last_status(void);      /* the status that went with it: what an entry point that returns NULL on failure would have returned */
/* JSON with the findings of the last TQE_ERR_WEIGHTS ({"missing": [...], "unexpected": [...], "wrong_shape": [[name, got, expected]...],
 * "wrong_kind": [...]}), or "" */
const char* tqe_last_error_detail(void);
/* a warning the last call left (tensors a folder holds that the model does not use, with strict off), or "" */
const char* tqe_last_warning(void);
int tqe_abi_version(void);
int tqe_page_size(void);        /* TQE_PAGE, as the library was built */

/* ---- the cache's bookkeeping ---------------------------------------------------------------- */
typedef struct tqe_cache tqe_cache_t;

/* max_slots sequences at most; group g has a pool of pages_per_group[g] pages and, if
 * window_per_group[g] > 0, gives a sequence's pages back once all their positions are further
 * back than the window of the next query.  Returns NULL on error. */
tqe_cache_t* tqe_cache_new(int max_slots, int n_groups, const int32_t* pages_per_group, const int32_t* window_per_group);
void tqe_cache_free(tqe_cache_t* cache);

/* A free slot with length 0 (TQE_ERR_FULL if there is none); everything a slot holds goes back. */
int tqe_cache_acquire(tqe_cache_t* cache, int32_t* slot_out);
int tqe_cache_release(tqe_cache_t* cache, int slot);
int tqe_cache_length(const tqe_cache_t* cache, int slot);
int tqe_cache_is_held(const tqe_cache_t* cache, int slot);
/* free and total slots (group -1) or pages of a group */
int tqe_cache_counts(const tqe_cache_t* cache, int group, int32_t* n_free, int32_t* n_total);

/* Room for n_new[i] more positions of slots[i] in every group, for all of them or
 * (TQE_ERR_FULL) for none.  Commit: the step has been launched, lengths grow, windows let go. */
int tqe_cache_reserve(tqe_cache_t* cache, int n, const int32_t* slots, const int32_t* n_new);
int tqe_cache_commit(tqe_cache_t* cache, int n, const int32_t* slots, const int32_t* n_new);
/* Gives a reservation back that was never committed: each slot keeps the pages its length needs. */
int tqe_cache_trim(tqe_cache_t* cache, int n, const int32_t* slots);

/* The pages of a slot in a group, -1 where given back: writes up to cap of them, returns how
 * many there are (TQE_NO_LIST if the slot never reserved anything in the group). */
int tqe_cache_pages(const tqe_cache_t* cache, int group, int slot, int32_t* out, int cap);

/* Nothing lost, held twice or freed twice: TQE_OK, or TQE_ERR_STATE with the finding. */
int tqe_cache_check(const tqe_cache_t* cache);

/* ---- the arrays of one step ----------------------------------------------------------------- */
/* What a step must satisfy before anything is reserved or launched (TQE_ERR_STEP with the
 * finding otherwise): at least one sequence, no slot twice, every sequence brings a token
 * (the reference's "Empty prompt", src/engine.rs:347-349), token ids inside the vocabulary,
 * and no sequence grows beyond max_positions.  tokens: all sequences' tokens one after the
 * other, or NULL where the host does not know them (they were chosen on the device). */
int tqe_check_step(const tqe_cache_t* cache, int n_seqs, const int32_t* slots, const int32_t* n_new,
                   const int32_t* tokens, int vocab_size, int max_positions);


/* Sequence i of the step lives in slots[i], held starts[i] positions before the step (NULL: what
 * the cache says) and brings n_new[i] tokens (tokens: all of them, sequence after sequence);
 * want_counts[i] of its places are wanted, want_idx lists them (indices among the sequence's
 * tokens, any order, repeats allowed).  Page table widths are rounded up to multiples of
 * width_step.
 *
 * out receives, each starting at a multiple of 4 values (offsets in meta):
 *   0 tokens  1 token's sequence  2 token's position  3 slot  4 start  5 count  6 first token of
 *   each sequence (n_seqs + 1)  7 wanted rows  8 the rows the last run computes (the wanted ones,
 *   each once, ascending; empty unless fewer than the step's tokens in a step that is not one
 *   token per sequence)  9 each wanted row's index among those  10, 11 their sequence and position
 *   12.. one page table [n_seqs][width] per group of the cache, -1 where there is no page
 * meta: TQE_META_* below, then 12 + TQE_MAX_GROUPS offsets, then TQE_MAX_GROUPS widths.
 * With out == NULL only meta is written (meta[TQE_META_TOTAL] values are needed). */
enum {
    TQE_META_TOTAL = 0, TQE_META_TOKENS, TQE_META_WANT, TQE_META_LAST, TQE_META_ALL_DECODE, TQE_META_PRUNE_LAST,
    TQE_META_MAX_NEW, TQE_META_MAX_END, TQE_META_GROUPS, TQE_META_OFFSETS = 12,
    TQE_META_SIZE = 12 + 12 + 2 * TQE_MAX_GROUPS
};
int tqe_plan_step(const tqe_cache_t* cache, int n_seqs, const int32_t* slots, const int32_t* starts, const int32_t* n_new,
                  const int32_t* tokens, const int32_t* want_counts, const int32_t* want_idx, int width_step,
                  int32_t* out, int out_cap, int32_t* meta);

/* ---- the generation loop's decisions -------------------------------------------------------
 * The loop computes nothing: it decides which requests run together, how their prompts are cut
 * into steps, and what becomes of every drawn token (the reference's loop for one request:
 * src/engine.rs:364-438). */

/* Cut the requests, in order, into batches that start together: at most max_batch requests each
 * and, where the cache holds pages (holds_pages), at most max_tokens positions, a request counted
 * as prompt + max_new - 1 positions rounded up to whole pages (its last token is never fed).
 * batch_of[i]: the number of request i's batch.  Returns the number of batches, or TQE_ERR_FULL
 * where one request alone needs more than max_tokens. */
int tqe_plan_batches(int n_requests, const int32_t* prompt_lens, int max_new, long long max_tokens, int max_batch,
                     int holds_pages, int32_t* batch_of);

/* Cut a batch's prompts into steps of at most max_step_tokens tokens: whole prompts together while
 * they fit, a longer one in pieces that come in order.  pieces: [capacity][4] = prompt, begin, end,
 * step.  Returns the number of pieces (none written beyond capacity: call again with as many). */
int tqe_prompt_steps(int n_prompts, const int32_t* lens, int max_step_tokens, int32_t* pieces, int capacity);

/* A batch's progress: how many tokens each of its requests has emitted and which have ended. */
typedef struct tqe_batch tqe_batch_t;
tqe_batch_t* tqe_batch_new(int n_requests, int max_new, const int32_t* stop_ids, int n_stop_ids);
void tqe_batch_free(tqe_batch_t* batch);
enum {
    TQE_TOKEN_FEED = 0,     /* emitted; the request goes on with it */
    TQE_TOKEN_LAST = 1,     /* emitted; the request has its max_new tokens and ends */
    TQE_TOKEN_STOP = 2,     /* a stop token, or nothing more was wanted: not emitted (src/engine.rs:381), the request ends */
    TQE_TOKEN_DROPPED = 3   /* the request had ended before (a step that ran ahead for nothing) */
};
/* What becomes of the token drawn for request `row`; counts it.  TQE_ERR_ARGUMENT for a bad row. */
int tqe_batch_accept(tqe_batch_t* batch, int row, int token);
/* Whether `row` will want another step after its next token unless that is a stop token. */
int tqe_batch_goes_on(const tqe_batch_t* batch, int row);
int tqe_batch_emitted(const tqe_batch_t* batch, int row);
int tqe_batch_ended(const tqe_batch_t* batch, int row);

/* ---- the library ------------------------------------------------------------------------------ */
/* dtype codes */
enum { TQE_F32 = 0, TQE_BF16 = 1, TQE_I32 = 2 };

/* The HIP kernels live in a shared library of their own (libtqkernels_*.so beside this one, or what
 * TQ_KERNEL_LIBRARY names); it is opened at first use.  tqe_set_kernel_library names it outright.
 * tqe_set_kernel_builder: a function of the caller's that is asked for the library's path when none is
 * found (the Python package compiles the kernels there); it returns null or "" if it cannot. */
int tqe_set_kernel_library(const char* path);
typedef const char* (*tqe_kernel_builder_t)(void);
void tqe_set_kernel_builder(tqe_kernel_builder_t builder);
const char* tqe_kernel_library(void);
/* Switches of the product and attention routines, for tests that compare one routine with another:
 * skinny, library, fused, prune_last, packed, mid, keep_rows, decode_mfma, prefill_mfma (all 1 to
 * start with).  tqe_policy_get: the value, or -1 for an unknown name. */
int tqe_policy_set(const char* name, int value);
int tqe_policy_get(const char* name);
/* Named ranges around the parts of a step (ROCTx), off to start with unless TQ_TRACE is set.
 * tqe_trace_enable returns 1 if ranges are on afterwards.  tqe_trace_sink: where ranges go instead
 * of ROCTx (both NULL: ROCTx again). */
int tqe_trace_enable(int on);
int tqe_trace_enabled(void);
void tqe_trace_sink(int (*push)(const char* name), int (*pop)(void));
void tqe_trace_push(const char* name);
void tqe_trace_pop(void);

/* ---- configuration (JSON in, JSON out) ---------------------------------------------------------- */
const char* tqe_known_architectures(void);                    /* ["Qwen2ForCausalLM", ...] */
const char* tqe_known_parts(const char* category);            /* kinds of a category: norm, position, mixer, feed_forward, block */
/* {"architecture": name, "config": {every key the architecture reads, defaults filled in}} of a config.json's text; NULL on error */
const char* tqe_config_parse(const char* config_json);
const char* tqe_config_spec(const char* config_json);         /* the model spec of a config.json's text */
const char* tqe_read_config(const char* model_dir);           /* the text of a folder's config.json, checked to be JSON */
/* [ids]: config.json's eos_token_id, generation_config.json's, and the ids of the reference's stop strings in tokenizer.json */
const char* tqe_stop_token_ids(const char* model_dir);

/* ---- tensors and parts that cross the boundary ----------------------------------------------- */
typedef struct tqe_tensor {
    void* data;                 /* NULL: no tensor (an optional argument that is absent) */
    int32_t dtype;              /* TQE_F32, TQE_BF16, TQE_I32 */
    int32_t ndim;
    int64_t shape[6];
    int64_t row_stride;         /* values from one row of the first dimension to the next; 0: the rows lie one after the other */
} tqe_tensor_t;

/* What a part registered by the caller sees of a step: the arrays of tqe_plan_step on the host and on
 * the device, the page tables, and the stream to work on. */
enum { TQE_STEP_ARRAYS = 12 };  /* tokens, tok_seq, tok_pos, seq_slot, seq_start, seq_new, cu, want_rows, last_rows, want_in_last, last_seq, last_pos */
typedef struct tqe_step_view {
    int32_t n_seqs, n_tokens, n_want, n_last, all_decode, prune_last, max_new, max_end, act_dtype, n_groups;
    const int32_t* host[TQE_STEP_ARRAYS];
    const int32_t* dev[TQE_STEP_ARRAYS];
    int32_t sizes[TQE_STEP_ARRAYS];
    const int32_t* table_host[TQE_MAX_GROUPS];
    const int32_t* table_dev[TQE_MAX_GROUPS];
    int32_t table_width[TQE_MAX_GROUPS];
    /* of the call at hand, for a mixer: which group's page table is its own, whether it writes its cache, whether only the
     * step's last_rows are asked for */
    int32_t entry_group, entry_writes, entry_window, last_rows_only;
    void* stream;
} tqe_step_view_t;

/* A kind of part made by the caller.  Every function returns 0 or a negative status, with the text of the failure from
 * last_error.  create returns a handle of the caller's for the new part.  describe returns JSON:
 *   {"tensors": {name: {"shape": [...], "init": "normal", "std": 0.02, "dtype": "float"}, ...},
 *    "cache_need": null | {"kind": "pages", "key_page": [...], "value_page": [...], "window": null | n} | {"kind": "state", "shape": [...], "dtype": "float32"},
 *    "graph_safe": false, "max_positions": n, "has_apply": false, "acts_on_stream": false, "trace_name": "part"}
 * load hands over the part's tensors (device memory that the engine keeps alive as long as the part lives).
 * call runs one method; its tensors, in order:
 *   norm          "forward": x, out         "add_norm": h, delta (may be absent), out        "gather_add_norm": h, delta (may be absent), rows, out
 *   position      "apply": q, k (changed in place; rows row_stride apart)                    "add_to_stream": h
 *   mixer         "forward": x, out, then the cache entry: keys, values (pages) or state
 *   feed_forward  "forward": x, out
 * Such parts run as they come, never inside a captured graph. */
typedef struct tqe_part_callbacks {
    int (*create)(void* user, const char* category, const char* kind, const char* params_json, int act_dtype, int on_gpu, void** instance);
    void (*destroy)(void* user, void* instance);
    const char* (*describe)(void* user, void* instance);
    int (*load)(void* user, void* instance, int n, const char* const* names, const tqe_tensor_t* tensors);
    int (*call)(void* user, void* instance, const char* method, const tqe_step_view_t* step, int n_args, const tqe_tensor_t* args);
    const char* (*last_error)(void* user);
} tqe_part_callbacks_t;
int tqe_register_part(const char* category, const char* kind, const tqe_part_callbacks_t* callbacks, void* user);
/* Another way to fill a random tensor than "normal", "one_plus_normal" and "zeros": fill writes the float32 values of the
 * tensor's elements begin .. begin + count - 1 (a function of seed, name and index alone). */
typedef int (*tqe_init_fill)(void* user, const char* tensor_name, const char* spec_json, uint64_t seed, int64_t begin, int64_t count, float* out);
int tqe_register_init(const char* kind, tqe_init_fill fill, void* user);

/* ---- models ------------------------------------------------------------------------------------ */
typedef struct tqe_model tqe_model_t;
/* on_gpu 0: host memory and no kernels (configuration, tensor lists and weights can be looked at; nothing runs) */
/* A model folder: config.json picks the architecture, *.safetensors hold the weights.  strict 0: tensors the model does not
 * use are a warning (tqe_last_warning), not an error. */
tqe_model_t* tqe_model_load(const char* model_dir, int dtype, int on_gpu, int strict);
/* Random weights made in memory from a config.json's text and a seed. */
tqe_model_t* tqe_model_random(const char* config_json, uint64_t seed, int dtype, int on_gpu);
/* A model without weights from a config.json's text, or from a model spec made by hand (JSON, as tqe_config_spec gives). */
tqe_model_t* tqe_model_new(const char* config_json, int dtype, int on_gpu);
tqe_model_t* tqe_model_from_spec(const char* spec_json, int dtype, int on_gpu);
/* Weights for such a model: every tensor of tqe_model_describe's "tensors" once (copied; data on the host, or on the device
 * with on_device), then tqe_model_finish, which checks names and shapes (one error that lists everything) and hands them
 * to the parts.  tqe_model_randomize: all of them from a seed instead. */
int tqe_model_set_tensor(tqe_model_t* model, const char* name, const tqe_tensor_t* tensor, int on_device, void* stream);
int tqe_model_finish(tqe_model_t* model, int strict, void* stream);
int tqe_model_randomize(tqe_model_t* model, uint64_t seed, void* stream);
/* Lets the matrix library try the kernels it proposes for every product of the model at `rows` rows (prompts: fewer rows than
 * the own kernels take never reach the library) and keep the fastest for later steps of that size; some milliseconds a shape. */
int tqe_model_tune_library(tqe_model_t* model, int rows, void* stream);
/* JSON: spec, config, dtype, graph_safe, loaded, stop_token_ids, needs (per run), cache_of, tensors (name -> spec) */
const char* tqe_model_describe(const tqe_model_t* model);
/* where a loaded tensor lives, by its name (tensors folded into others are gone: "layer prefix + qkv.weight",
 * "gate_up.weight", "*.packed" name what the parts made of them) */
int tqe_model_tensor(const tqe_model_t* model, const char* name, tqe_tensor_t* out);
int tqe_model_set_stop_tokens(tqe_model_t* model, int n, const int32_t* ids);
void tqe_model_free(tqe_model_t* model);
/* config.json and model.safetensors of a model with random weights (store_dtype TQE_BF16 or TQE_F32) */
int tqe_write_random_folder(const char* folder, const char* config_json, uint64_t seed, int store_dtype);
/* element values of the random stream of (seed, tensor name): count float32 values from `begin` */
int tqe_random_stream(uint64_t seed, const char* tensor_name, int64_t begin, int64_t count, float* out);
uint64_t tqe_tensor_key(uint64_t seed, const char* tensor_name);      /* the 64-bit key of that stream */
int tqe_random_stream_of_key(uint64_t key, int64_t begin, int64_t count, float* out);

/* ---- safetensors ---------------------------------------------------------------------------------- */
typedef struct tqe_folder tqe_folder_t;
tqe_folder_t* tqe_folder_open(const char* model_dir);
void tqe_folder_free(tqe_folder_t* folder);
const char* tqe_folder_describe(const tqe_folder_t* folder);   /* {name: {"dtype": "BF16", "shape": [...], "data": address, "bytes": n}} (memory-mapped, read-only) */
/* names, shapes and kinds of a folder against a list of wanted tensors ({name: tensor spec}) */
int tqe_check_weights(const tqe_folder_t* folder, const char* wanted_json, int strict);
/* writes tensors ({name: {"dtype": "F32", "shape": [...]}} in this order, data[i] the host bytes of the i-th) as one file */
int tqe_write_safetensors(const char* path, const char* tensors_json, const void* const* data, const char* metadata_json);

/* ---- single parts, a cache and a step of one's own (what the tests of single parts use) --------------- */
typedef struct tqe_part tqe_part_t;
typedef struct tqe_store tqe_store_t;
typedef struct tqe_stepctx tqe_stepctx_t;
tqe_part_t* tqe_part_new(const char* category, const char* spec_json, int act_dtype, int on_gpu);
void tqe_part_free(tqe_part_t* part);
const char* tqe_part_describe(const tqe_part_t* part);         /* as a caller's part describes itself */
int tqe_part_set_tensor(tqe_part_t* part, const char* name, const tqe_tensor_t* tensor, int on_device, void* stream);
int tqe_part_finish(tqe_part_t* part, void* stream);
int tqe_part_tensor(const tqe_part_t* part, const char* name, tqe_tensor_t* out);
/* methods and tensors as in tqe_part_callbacks.call; mixers take the cache entry of `run` of `store`; step may be NULL
 * for norms and feed-forwards */
int tqe_part_call(tqe_part_t* part, const char* method, tqe_stepctx_t* step, tqe_store_t* store, int run, int n_args,
                  const tqe_tensor_t* args, void* stream);
/* needs_json: [need per run], cache_of: per run -1 or the run whose cache it reads */
tqe_store_t* tqe_store_new(const char* needs_json, const int32_t* cache_of, int n_runs, long long max_tokens, int max_slots, int dtype, int on_gpu);
void tqe_store_free(tqe_store_t* store);
tqe_cache_t* tqe_store_cache(tqe_store_t* store);              /* its bookkeeping, for the tqe_cache_* calls */
const char* tqe_store_describe(const tqe_store_t* store);      /* groups: need, runs, pages, where keys, values and states live */
int tqe_store_acquire(tqe_store_t* store, int32_t* slot_out, void* stream);
/* the arrays of a step over a store's sequences (reserve first), uploaded */
tqe_stepctx_t* tqe_stepctx_new(tqe_store_t* store, int n_seqs, const int32_t* slots, const int32_t* n_new, const int32_t* tokens,
                               const int32_t* want_counts, const int32_t* want_idx, int act_dtype, void* stream);
void tqe_stepctx_free(tqe_stepctx_t* step);
int tqe_stepctx_view(tqe_stepctx_t* step, tqe_step_view_t* out);

/* ---- the engine ---------------------------------------------------------------------------------- */
typedef struct tqe_engine tqe_engine_t;
/* max_tokens: positions live sequences may hold together, each counted up to whole pages; max_slots: most live sequences.
 * The engine shares the model (which must outlive it). */
tqe_engine_t* tqe_engine_new(tqe_model_t* model, long long max_tokens, int max_slots, int use_graphs);
void tqe_engine_free(tqe_engine_t* engine);
int tqe_engine_open(tqe_engine_t* engine, int32_t* slot_out, void* stream);       /* a sequence starts: a slot with nothing in it */
int tqe_engine_close(tqe_engine_t* engine, int slot);                              /* it ends: slot and pages will be used again */
tqe_cache_t* tqe_engine_cache(tqe_engine_t* engine);
/* JSON: the cache's groups (as tqe_store_describe), holds_pages, max_slots, max_tokens, use_graphs, n_graphs, vocab_size, max_positions */
const char* tqe_engine_describe(const tqe_engine_t* engine);
/* One step: sequence i lives in slots[i] and brings n_new[i] tokens (tokens: all of them on the host, one sequence after the
 * other; or device_tokens: int32 [n_seqs] on the device for a step of one token each, tokens may then be NULL);
 * want_counts[i] of its places are wanted, want_idx lists them.  The float32 logits [wanted, vocab] are written to
 * logits_out: device memory, or host memory with logits_on_host (the call then waits for them).  logits_out NULL: they stay
 * in the engine's own memory until its next step; *logits_kept (if given) says where. */
int tqe_step(tqe_engine_t* engine, int n_seqs, const int32_t* slots, const int32_t* n_new, const int32_t* tokens,
             const int32_t* want_counts, const int32_t* want_idx, const int32_t* device_tokens,
             float* logits_out, int logits_on_host, const float** logits_kept, void* stream);

/* ---- sampling and the generation loop ------------------------------------------------------------------ */
/* names and defaults of the reference's GenerationParams (src/engine.rs:29-49) */
typedef struct tqe_generation_params {
    int32_t max_tokens;         /* 512 */
    float temperature;          /* 0.7; <= 0 is greedy */
    float top_p;                /* 0.9 */
    int32_t top_k;              /* 40; 0 switches it off */
    float repeat_penalty;       /* 1.1; 1.0 switches it off */
    uint64_t seed;              /* 0 */
} tqe_generation_params_t;
void tqe_generation_defaults(tqe_generation_params_t* params);
float tqe_draw_uniform(uint64_t seed, uint64_t request, uint64_t step);
typedef void (*tqe_on_tokens)(void* user, int n, const int32_t* requests, const int32_t* tokens);
/* Generates for n_prompts requests (prompt i: prompt_lens[i] tokens of `tokens`, one after the other) in batches that start
 * together.  stop_ids: stop tokens (n_stop_ids < 0: the model's own).  out_tokens: room for max_tokens ids per request,
 * request i's from out_tokens + i * max_tokens; out_counts[i] how many it emitted.  on_tokens (may be NULL): called after
 * every step with what it emitted.  max_batch: most requests that run together; max_step_tokens: most tokens one step runs. */
int tqe_generate(tqe_engine_t* engine, int n_prompts, const int32_t* prompt_lens, const int32_t* tokens,
                 const tqe_generation_params_t* params, const int32_t* stop_ids, int n_stop_ids, int max_batch, int max_step_tokens,
                 tqe_on_tokens on_tokens, void* user, int32_t* out_tokens, int32_t* out_counts, void* stream);
/* The same loop over an engine and a sampler of the caller's (stand-ins in tests): step gets the step's sequences (slot,
 * tokens, whether the last place is wanted), sample gives a token for each row of the last step's wanted places (rows: the
 * requests' indices in their batch; request_ids: their numbers in the whole run). */
typedef struct tqe_loop_callbacks {
    int (*open)(void* user, int32_t* slot_out);
    int (*close)(void* user, int slot);
    int (*step)(void* user, int n_seqs, const int32_t* slots, const int32_t* n_new, const int32_t* tokens, const int32_t* want_last);
    int (*new_batch)(void* user, int n_requests, const int32_t* request_ids);
    int (*sample)(void* user, int n_rows, const int32_t* rows, int32_t* tokens_out);
    const char* (*last_error)(void* user);
    long long max_tokens, max_positions;
    int32_t max_slots, holds_pages;
    /* optional, all three or none: a sampler that can start a draw without waiting for it and an engine that takes a
     * step's tokens from where the sampler left them.  draw: starts a draw from the last step's logits and names it;
     * step_ahead: a step of one token per sequence whose tokens are the draw's at `places`; read: the draw's tokens. */
    int (*draw)(void* user, int n_rows, const int32_t* rows, int32_t* draw_out);
    int (*step_ahead)(void* user, int n_seqs, const int32_t* slots, int draw, const int32_t* places);
    int (*read)(void* user, int draw, int n, int32_t* tokens_out);
} tqe_loop_callbacks_t;
int tqe_generate_with(const tqe_loop_callbacks_t* callbacks, void* user, int n_prompts, const int32_t* prompt_lens, const int32_t* tokens,
                      const tqe_generation_params_t* params, const int32_t* stop_ids, int n_stop_ids, int max_batch, int max_step_tokens,
                      tqe_on_tokens on_tokens, void* on_tokens_user, int32_t* out_tokens, int32_t* out_counts);
/* The device sampler alone: a batch's sampler, a draw from logits on the device (changed in place by the repeat penalty). */
typedef struct tqe_sampler tqe_sampler_t;
tqe_sampler_t* tqe_sampler_new(const tqe_generation_params_t* params, int n_requests, const int32_t* request_ids, int vocab, void* stream);
void tqe_sampler_free(tqe_sampler_t* sampler);
int tqe_sampler_sample(tqe_sampler_t* sampler, float* logits, int n_rows, const int32_t* rows, int32_t* tokens_out);

#ifdef __cplusplus
}
#endif
