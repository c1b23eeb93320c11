// y = x W^T (+ b): the one place that decides which matrix-product routine runs.
//
// The reference's linear layers are candle matmuls, i.e. library GEMMs
// (src/models/turbo_generic.rs:68-91).  Here:
//
//   float32 anywhere (the 32-bit path, or a weight stored in 32-bit)
//         -> the hand-written FMA kernel (no matrix cores, fixed summation order)
//   bfloat16, few rows (decoding, chosen logit rows; as many as the skinny kernel takes)
//         -> the hand-written weight-streaming MFMA kernel (alone here, with the neighbouring
//            norm, residual sum, gate or rotation folded in where parts ask).  It reads a second
//            copy of the weight, packed at loading time in the order its lanes take it.
//   bfloat16, more rows up to what the kernel for mid-sized steps takes, where the weight has a packed copy
//         -> the hand-written kernel that stages x in LDS and streams the packed weights
//   bfloat16, more rows (prompts, large decoding batches)
//         -> the library GEMM (hipBLASLt), float32 accumulation; float32 output where logits are wanted
#pragma once
#include "parts.h"
#include "step.h"

namespace tq {

// The bfloat16 routines can be switched off one by one (tests compare each with the plain
// kernel); nothing else reads these.  "packed": parts keep the second, packed copy of their
// weights for the few-row kernels (twice the weight memory, about an eighth less time per
// decoding step).  "keep_rows": off gives the rows up once a weight is packed (set it before
// loading): a product of more rows than the own kernels take then gets the rows back from the
// packed copy for its own length (or, with the library off, goes through the own kernels in pieces).
struct Policy {
    int skinny = 1, library = 1, fused = 1, prune_last = 1, packed = 1, mid = 1, keep_rows = 1;
    int decode_mfma = 1, prefill_mfma = 1;
};
Policy& policy();
int* policy_field(const std::string& name);        // nullptr for an unknown name

// A product's weight [n, k]: its rows as the checkpoint has them, its packed copy, or both.
struct Weight {
    OwnedPtr rows;           // null once given up
    OwnedPtr packed;         // null where the few-row kernels take the rows as they are
    int64_t n = 0, k = 0;
    int parts = 1;
    int dtype = BF16;
    bool defined() const { return n > 0; }
};
// Takes a loaded weight; makes its packed copy where the policy and the sizes allow; gives the
// rows up if the policy says so and nobody else needs them.
Weight make_weight(OwnedPtr rows, int parts, bool rows_needed, hipStream_t stream);

int skinny_max_rows();
int mid_max_rows();
// Whether the folded skinny kernels take a product of x_rows rows with this weight (adds: with
// the result added to the stream).
bool fusable(int64_t x_rows, const Weight& w, bool adds = false);
// Whether a product of x_rows rows goes through the kernel for mid-sized steps, which can leave its sums to the next norm.
bool leaves_sums(int64_t x_rows, const Weight& w);
// What kind of step this is for the parts' folding: small (norms and residual sums folded into
// the products), mid (sums over pieces of K left to the next kernel), or neither.
void classify_step(StepContext& c, int64_t hidden);

struct Product {
    Tensor t;
    PartialSums sums;
    bool is_sums = false;
};
// x [M, K] times weight^T -> [M, N] of out_dtype (into `out` if given, else workspace memory).
// leave_sums: the caller also takes the product unfinished where the kernel cuts K into pieces.
Product linear(StepContext& c, const Tensor& x, const Weight& w, const Tensor* bias, int out_dtype, bool leave_sums = false, Tensor* out = nullptr);
// silu(x Wg^T) * (x Wu^T) with Wg stacked on Wu: [M, K] x [2I, K] -> [M, I]
Tensor gated_silu_linear(StepContext& c, const Tensor& x, const Weight& w_gate_up);
// h += bfloat16(x weight^T), preparing stream.next_norm (small steps: in the product's epilogue;
// mid-sized ones: left pending for the next norm's kernel, as sums where that norm takes them)
void add_product(StepContext& c, Stream& stream, const Tensor& x, const Weight& w);

// the library product, bfloat16 in, bfloat16 or float32 out
void library_gemm(const Tensor& x, const Tensor& w_rows, Tensor& out, hipStream_t stream);
// Lets the library try the kernels it proposes for a product of m rows with a weight [n, k] and keeps the fastest for
// later calls of that shape (the first proposal is what an untried shape gets).  Takes some milliseconds per shape;
// it pays for prompts, whose products are the library's.  Returns the microseconds of the kept kernel.
double library_tune(int64_t m, int64_t n, int64_t k, int out_dtype, hipStream_t stream);
void library_release();

// thin typed wrappers over the kernel entry points that several files use
void k_add_rmsnorm(StepContext& c, float* h, const Pending& delta, const Tensor& weight, float eps, const int32_t* rows, int64_t n_rows,
                   int64_t src_rows, Tensor& out, bool write_back);
void k_gather_rows(StepContext& c, const Tensor& src, const int32_t* rows, int64_t n_rows, Tensor& out);

}  // namespace tq
