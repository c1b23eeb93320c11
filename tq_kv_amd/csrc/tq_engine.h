/* C entry points of the engine's host side: slots, page lists and the arrays of a step.
 *
 * In the manner of the reference's C boundary (tq-kv/include/tq_kv.h:27-84,
 * tq-kv/src/ffi.rs:89-108): opaque handles that the library makes and frees, plain C
 * types, int32 status (0 ok, negative error), a message for the last error of the
 * calling thread.  Nothing here touches the GPU; all pointers are host pointers.
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TQE_PAGE 64             /* positions per cache page */
#define TQE_MAX_GROUPS 16       /* groups of cached runs a cache may have */

enum {
    TQE_OK = 0,
    TQE_ERR_ARGUMENT = -1,      /* null pointer, number out of range */
    TQE_ERR_FULL = -2,          /* no free slot, or not enough free pages: nothing was changed */
    TQE_ERR_STATE = -3,         /* a slot that is not held, something freed twice, a broken invariant */
    TQE_ERR_RANGE = -4,         /* a wanted place outside its sequence's tokens */
    TQE_ERR_STEP = -5,          /* a step the engine cannot run: see tqe_check_step */
    TQE_NO_LIST = -100          /* tqe_cache_pages: the slot has no page list in the group (not an error) */
};

const char* tqe_last_error(void);
int tqe_abi_version(void);

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

#ifdef __cplusplus
}
#endif
