"""y = x W^T (+ b): the one place that decides which matrix-product routine runs.

The reference's linear layers are candle matmuls, i.e. library GEMMs
(src/models/turbo_generic.rs:68-91).  Here:

  float32 anywhere (the 32-bit path, or a weight stored in 32-bit)
        -> the hand-written FMA kernel (no matrix cores, fixed summation order)
  bfloat16, few rows (decoding, chosen logit rows)
        -> the hand-written weight-streaming MFMA kernel
  bfloat16, many rows (prompts)
        -> the library GEMM (hipBLASLt through torch.matmul), float32 accumulation
"""
import torch

from .. import kernels as K

# The bfloat16 routines can be switched off one by one (tests compare each with the
# plain kernel); nothing else reads these.
POLICY = {"skinny": True, "library": True, "skinny_max_rows": 64}


def linear(x, weight, bias=None, out_dtype=None):
    """x: [M,K]; weight: [N,K]; bias: [N] or None.  Returns [M,N] of out_dtype
    (default: x's dtype)."""
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise ValueError("linear: x has %d columns but the weight has %d" % (k, weight.shape[1]))
    out_dtype = out_dtype or x.dtype
    both_bf16 = x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
    if both_bf16 and bias is None:
        if POLICY["skinny"] and K.has_skinny() and k % 32 == 0 and m <= POLICY["skinny_max_rows"]:
            out = torch.empty((m, n), dtype=out_dtype, device=x.device)
            return K.skinny_bf16(x, weight, out)
        if POLICY["library"] and out_dtype == torch.bfloat16 and m > POLICY["skinny_max_rows"]:
            return torch.matmul(x, weight.t())
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    return K.gemm(x, weight, bias, out)
