// The entry points of the kernel library (csrc/tq_kernels.h) as the engine calls them: looked up
// by name at first use.  Launches raise with the library's message on failure; the queries
// (sizes of scratch memory, what a kernel takes) are plain host functions.
#pragma once
#include "core.h"

namespace tq {
namespace K {

#define TQ_KERNEL(name, ...) static Kernel<__VA_ARGS__> name("tqk_" #name)
#define TQ_QUERY(ret, name, ...) static KernelFn<ret(__VA_ARGS__)> name("tqk_" #name)
typedef const void* cptr;
typedef const int32_t* ci32;
typedef const float* cf32;

TQ_QUERY(int, abi_version);
TQ_QUERY(int, page_size);
TQ_QUERY(int, skinny_max_rows);
TQ_QUERY(int, mid_max_rows);
TQ_KERNEL(embed, cptr, int, ci32, int, int, int, float, float*, void*, cptr, float*, void*);
TQ_KERNEL(finish_logits, float*, int, int, cf32, float, float, void*);
TQ_KERNEL(random_normal, void*, int, long long, uint64_t, float, int, void*);
TQ_KERNEL(add_rmsnorm, float*, cptr, int, cptr, int, float, ci32, int, int, void*, int, void*);
TQ_KERNEL(add_rmsnorm_sums, float*, cf32, int, int, int, cptr, int, float, ci32, int, int, void*, int, void*);
TQ_QUERY(size_t, gemm_scratch_bytes, int, int, int, int, int, int, int);
TQ_KERNEL(gemm, cptr, int, cptr, int, cptr, int, void*, int, int, int, int, void*, void*);
TQ_KERNEL(fused_store, cptr, ci32, cf32, int, float, cptr, int, void*, int, int, int, int, void*);
TQ_KERNEL(fused_gated, cptr, cf32, int, float, cptr, int, void*, int, int, int, void*);
TQ_QUERY(int, fused_residual_parts, int, int);
TQ_KERNEL(fused_residual, cptr, cptr, int, float*, cptr, void*, float*, int, int, int, void*);
TQ_KERNEL(fused_qkv, cptr, cf32, int, float, cptr, int, cptr, cf32, cf32, int, ci32, ci32, int, void*, void*, int, void*, int, int, int, int,
          int, void*);
TQ_QUERY(int, mid_splits, int, int, int);
TQ_KERNEL(mid_store, cptr, cptr, void*, int, int, int, int, void*, int, void*);
TQ_KERNEL(mid_gated, cptr, cptr, void*, int, int, int, void*, void*);
TQ_KERNEL(rope_store, cptr, int, cptr, int, cf32, cf32, int, int, int, ci32, ci32, ci32, int, int, void*, void*, int, void*, int, int, int, int,
          int, void*);
TQ_QUERY(int, rope_store_takes_sums, int, int, int, int, int, int);
TQ_KERNEL(rope_store_sums, cf32, int, cptr, int, cf32, cf32, int, int, int, ci32, ci32, ci32, int, int, void*, void*, int, void*, int, int, int,
          int, int, void*);
TQ_QUERY(int, attention_max_head_dim);
TQ_KERNEL(attention, cptr, cptr, cptr, int, ci32, ci32, ci32, int, int, int, int, float, void*, int, int, int, int, void*);
TQ_QUERY(int, attention_decode_supported, int);
TQ_KERNEL(attention_decode, cptr, cptr, cptr, ci32, ci32, int, int, int, int, float, int, void*, void*, void*, int, int, int, void*);
TQ_QUERY(int, attention_prefill_supported, int);
TQ_QUERY(int, attention_prefill_tile, int, int, int, int);
TQ_KERNEL(attention_prefill, cptr, cptr, cptr, ci32, ci32, int, int, int, ci32, ci32, ci32, int, int, ci32, ci32, int, float, void*, int, int,
          int, int, void*);
TQ_KERNEL(swiglu, cptr, void*, int, int, int, void*);
TQ_QUERY(int, argmax_scratch_floats, int, int);
TQ_KERNEL(argmax, cf32, int, int, int32_t*, float*, void*);
TQ_KERNEL(repeat_penalty, float*, int, int, ci32, ci32, ci32, int, ci32, int, float, void*);
TQ_KERNEL(append_history, ci32, ci32, int32_t*, int32_t*, int, int32_t*, int, void*);
TQ_QUERY(size_t, sample_scratch_bytes, int, int, int, float);
TQ_KERNEL(sample, cf32, int, int, float, int, float, cf32, int32_t*, void*, void*);
// rows of any kind gathered by index; a bias added to every row; a weight into the few-row kernels' order
TQ_KERNEL(gather_rows, cptr, ci32, int, long long, void*, void*);
TQ_KERNEL(add_bias, void*, int, cptr, int, int, int, void*);
TQ_KERNEL(pack_weight, cptr, void*, int, int, int, void*);
TQ_KERNEL(unpack_weight, cptr, void*, int, int, int, void*);
TQ_KERNEL(convert, cptr, int, void*, int, long long, void*);

#undef TQ_KERNEL
#undef TQ_QUERY

}  // namespace K
}  // namespace tq
