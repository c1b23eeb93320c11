"""y = x W^T (+ b): the one place that decides which matrix-product routine runs.

The reference's linear layers are candle matmuls, i.e. library GEMMs
(src/models/turbo_generic.rs:68-91).  Here:

  float32 anywhere (the 32-bit path, or a weight stored in 32-bit)
        -> the hand-written FMA kernel (no matrix cores, fixed summation order)
  bfloat16, up to 16 rows (decoding, chosen logit rows)
        -> the hand-written weight-streaming MFMA kernel (kernels.fused_*: alone here, with
           the neighbouring norm, residual sum, gate or rotation folded in where parts ask).
           It reads a second copy of the weight, packed at loading time in the order its
           lanes take it (few_rows_form): a decoding step is bound by the weight bytes, and
           in that order they stream faster.
  bfloat16, 17 to 128 rows (decoding steps of larger batches) where the weight has a packed copy
        -> the hand-written kernel that stages x in LDS and streams the packed weights
           (kernels.mid_store, kernels.mid_gated)
  bfloat16, more rows (prompts, large decoding batches)
        -> the library GEMM (hipBLASLt through torch), float32 accumulation; float32
           output where logits are wanted
"""
import torch

from .. import kernels as K

# The bfloat16 routines can be switched off one by one (tests compare each with the
# plain kernel); nothing else reads these.
# Measured on MI355X at the Qwen2.5-7B sizes: up to 16 rows the skinny kernel is ahead of the
# library on every product; at 64 rows the library is ahead of it on every one, and the kernel
# for 17 to 128 rows ("mid") ahead of the library.
# "packed": parts keep the second, packed copy of their weights for the few-row kernels (twice
# the weight memory, about an eighth less time per decoding step).
# "keep_rows": False gives the rows up once a weight is packed (set it before loading): half the
# weight memory again; products of more than 128 rows (prompts) then go through the kernel for
# 17 to 128 rows in pieces, each of which streams the weight once, instead of the library.
POLICY = {"skinny": True, "library": True, "skinny_max_rows": 16, "fused": True, "prune_last": True, "packed": True,
          "mid": True, "keep_rows": True}


class Stream:
    """The residual stream of a step.  h: float32 [tokens, hidden].  pending: an update that
    has not been added to h yet (a tensor of the activation dtype, or a product's
    kernels.PartialSums for a norm that takes those), or None.

    In small decoding steps the kernels that add to h also prepare the next norm: xw is
    bfloat16(h * weight of norm `xw_for`) and ss the rows' sums of squares in n_ss pieces
    (valid only while nothing is pending).  next_norm is set by whoever runs a part, to the
    norm that will read the stream after that part."""

    def __init__(self, h, xw_buffer=None, ss_buffer=None):
        self.h, self.pending = h, None
        self.xw_buffer, self.ss_buffer = xw_buffer, ss_buffer
        self.xw_for, self.n_ss = None, 0
        self.next_norm = None

    def add_product(self, x, weight):
        """h += bfloat16(x weight^T), preparing next_norm.  weight: [N, K] or its few-row form.
        Up to 16 rows: in the product's epilogue.  17 to 128 rows (weight in its few-row form):
        the product, or where next_norm can add them up its sums over pieces of K, is left
        pending for the next norm's kernel."""
        if x.shape[0] > POLICY["skinny_max_rows"]:
            self.pending = K.mid_store(x, weight, finish=not getattr(self.next_norm, "takes_partial_sums", False))
            self.invalidate()
            return
        norm = self.next_norm if getattr(self.next_norm, "foldable", False) else None
        self.n_ss = K.fused_residual(x, weight, self.h, self.xw_buffer,
                                     norm.weight if norm is not None else None, self.ss_buffer)
        self.xw_for = norm
        self.pending = None

    def invalidate(self):
        self.xw_for = None


class LazyNorm:
    """An RMSNorm of the stream that has not been computed: xw is the stream times the norm's
    weight, norm = (sums of squares in pieces, number of pieces, eps); the product that takes
    it divides its result by the rows' rms."""

    def __init__(self, xw, ss, n_ss, eps):
        self.xw, self.norm = xw, (ss, n_ss, eps)


class PackedOnly:
    """Stands where a weight's rows were: its shape, dtype and device, no data.  The products
    take the packed copy (`few`) for any number of rows."""

    def __init__(self, weight):
        self.shape, self.dtype, self.device, self.is_cuda = tuple(weight.shape), weight.dtype, weight.device, weight.is_cuda

    def dim(self):
        return len(self.shape)


def rows_or_stand_in(weight, few, needed=False):
    """The weight itself, or (POLICY["keep_rows"] off, a packed copy there, and nobody else needing
    the rows) a PackedOnly in its place, so that the rows' memory is given back."""
    if POLICY["keep_rows"] or few is None or needed or not (POLICY["mid"] and POLICY["skinny"]):
        return weight
    return PackedOnly(weight)


def few_rows_form(weight, parts=1):
    """The copy of a weight [N, K] that the few-row kernels stream fastest (parts: stacked
    weights, as gate and up), or None where they take the weight as it is (float32, a K that
    is no multiple of 32, the policy switched off, not on the GPU)."""
    if not (POLICY["packed"] and POLICY["skinny"] and weight.dtype == torch.bfloat16 and weight.is_cuda
            and weight.dim() == 2 and weight.shape[1] % 32 == 0 and weight.shape[0] % parts == 0):
        return None
    return K.pack_weight(weight, parts)


def leaves_sums(x_rows, weight, few):
    """Whether a product of x_rows rows with this weight (few: its few-row form) goes through the
    kernel for 17 to 128 rows, which can leave its sums to the next norm (Stream.add_product)."""
    return (POLICY["mid"] and few is not None and weight.dtype == torch.bfloat16
            and POLICY["skinny_max_rows"] < x_rows <= K.MID_MAX_ROWS)


def fusable(x_rows, weight, adds=False):
    """Whether the folded skinny kernels take a product of x_rows rows with this weight
    (adds: with the result added to the stream)."""
    return (POLICY["fused"] and POLICY["skinny"] and x_rows <= 16 and weight.dtype == torch.bfloat16
            and weight.shape[1] % 32 == 0 and (not adds or weight.shape[0] % 4 == 0))


def tune_library(on=True, seconds=30):
    """Let the library try its kernels for each new product shape once and keep the fastest
    (PyTorch's TunableOp over hipBLASLt and rocBLAS).  The first call with a new shape then
    takes up to `seconds`; it pays for prompts, whose products are the library's."""
    import torch.cuda.tunable as tunable
    tunable.enable(bool(on))
    tunable.tuning_enable(bool(on))
    # what it finds is for this process: the file it may write when the process ends goes to the temp folder
    import os
    import tempfile
    tunable.set_filename(os.path.join(tempfile.gettempdir(), "tq_kv_amd_tunableop_%d.csv" % os.getpid()))
    if on:
        tunable.set_max_tuning_duration(int(seconds * 1000))
        tunable.record_untuned_enable(False)


def freeze_library_tuning():
    """Keep using what tuning has found so far, try nothing new."""
    import torch.cuda.tunable as tunable
    tunable.enable(True)
    tunable.tuning_enable(False)


def _skinny_ok(x, weight):
    return (POLICY["skinny"] and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
            and x.shape[1] % 32 == 0 and x.shape[0] <= POLICY["skinny_max_rows"])


def _mid_ok(x, weight, few):
    return x.dtype == torch.bfloat16 and leaves_sums(x.shape[0], weight, few)


def gated_silu_linear(x, weight_gate_up, few=None):
    """silu(x Wg^T) * (x Wu^T) with Wg stacked on Wu: [M, K] x [2I, K] -> [M, I].  For few
    rows of bfloat16 the gate and the up row of an output are computed by the same wave
    and never written; otherwise one product and the SwiGLU kernel.  few: the weight's
    few_rows_form (parts=2), if there is one."""
    m = x.shape[0]
    inter = weight_gate_up.shape[0] // 2
    act = torch.empty((m, inter), dtype=x.dtype, device=x.device)
    if _skinny_ok(x, weight_gate_up):
        return K.fused_gated(x, few or weight_gate_up, act)
    if _mid_ok(x, weight_gate_up, few):
        return K.mid_gated(x, few, act)
    if isinstance(weight_gate_up, PackedOnly):
        for piece, rows in _pieces(x, act):
            (K.fused_gated if piece.shape[0] <= POLICY["skinny_max_rows"] else K.mid_gated)(piece, few, rows)
        return act
    return K.swiglu(linear(x, weight_gate_up), act)


def _pieces(x, out):
    """x and out cut into pieces of as many rows as the kernel for 17 to 128 rows takes."""
    step = K.MID_MAX_ROWS
    return [(x[r:r + step], out[r:r + step]) for r in range(0, x.shape[0], step)]


def linear(x, weight, bias=None, out_dtype=None, few=None, leave_sums=False):
    """x: [M,K]; weight: [N,K]; bias: [N] or None.  Returns [M,N] of out_dtype
    (default: x's dtype).  few: the weight's few_rows_form, if there is one.  leave_sums: the
    caller also takes the product unfinished, as kernels.PartialSums (the kernel for 17 to 128
    rows gives those where it cuts K into pieces)."""
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise ValueError("linear: x has %d columns but the weight has %d" % (k, weight.shape[1]))
    out_dtype = out_dtype or x.dtype
    both_bf16 = x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
    if both_bf16 and bias is None:
        if _skinny_ok(x, weight):
            out = torch.empty((m, n), dtype=out_dtype, device=x.device)
            return K.fused_store(x, few or weight, out)
        if _mid_ok(x, weight, few):
            out = torch.empty((m, n), dtype=out_dtype, device=x.device)
            return K.mid_store(x, few, out, finish=not leave_sums)
        if isinstance(weight, PackedOnly):
            out = torch.empty((m, n), dtype=out_dtype, device=x.device)
            for piece, rows in _pieces(x, out):
                (K.fused_store if piece.shape[0] <= POLICY["skinny_max_rows"] else K.mid_store)(piece, few, rows)
            return out
        if POLICY["library"] and m > POLICY["skinny_max_rows"]:
            if out_dtype == torch.bfloat16:
                return torch.matmul(x, weight.t())
            if out_dtype == torch.float32:
                return torch.mm(x, weight.t(), out_dtype=torch.float32)
    if isinstance(weight, PackedOnly):
        raise RuntimeError("linear: this weight's rows were given up (POLICY['keep_rows']); only bfloat16 products without a bias take its packed copy")
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    return K.gemm(x, weight, bias, out)
