/* An entry point of the gfx950 kernel library that allocates nothing.
 *
 * It has no counterpart in the reference.  It is for callers that cannot allocate device memory:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Plain C
 * types, int status (0 ok, -1 error, the message from tqk_last_error of csrc/tq_kernels.h).
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* tqk_argmax (csrc/tq_kernels.h) without a scratch buffer of the caller's.  The
 * chunks' results go to an array inside the library's image on the current GPU (128 KiB per GPU,
 * held until the process ends) in place of a caller's scratch; n_rows * ceil(vocab / 4096) must
 * not exceed tqk_argmax_static_max_pairs() (16384), more is refused with an error.  It calls no
 * hipMalloc, hipFree or allocating library routine.  Every call on a GPU shares that GPU's array:
 * calls that overlap in time on one GPU (different streams or threads) race; calls on one stream
 * are ordered.  The GPU whose stream is given must be the current one.  The array's address is
 * looked up at the first call on each GPU; tqk_argmax_static_prepare() does that lookup for the
 * current GPU ahead of time (call it before a graph capture that will hold tqk_argmax_static). */
int tqk_argmax_static_max_pairs(void);
int tqk_argmax_static_prepare(void);
int tqk_argmax_static(const float* logits, int n_rows, int vocab, int32_t* out, void* stream);

#ifdef __cplusplus
}
#endif
