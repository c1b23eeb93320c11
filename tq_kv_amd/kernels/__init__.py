"""Python face of the gfx950 kernel library: one function per C entry point.

Every function checks device, dtype, contiguity and shapes on the host before the
kernel is launched, because a kernel that reads out of bounds can take the whole
GPU down.  There is no fallback: without the built library, or on tensors that
are not on the GPU, these functions raise.
"""
import ctypes

import torch

from ..csrc import build as _build

_LIB = None
KERNEL_ABI = 13         # tqk_abi_version of the kernel library these wrappers are written against

F32, BF16 = 0, 1
STYLE_NONE, STYLE_HALVES, STYLE_PAIRS = 0, 1, 2


from ..native import KernelError  # noqa: E402  (the same exception whichever face of the library raises it)


def library():
    """The loaded kernel library (built on first use if it is not there)."""
    global _LIB
    if _LIB is None:
        path = _build.ensure_built()
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError("cannot load the HIP kernel library %s: %s" % (path, e))
        lib.tqk_last_error.restype = ctypes.c_char_p
        lib.tqk_abi_version.restype = ctypes.c_int
        lib.tqk_sample_scratch_bytes.restype = ctypes.c_size_t
        lib.tqk_gemm_scratch_bytes.restype = ctypes.c_size_t
        from .. import native
        if int(lib.tqk_abi_version()) != KERNEL_ABI:
            raise KernelError("the kernel library %s has interface version %d, these wrappers are written against %d: build it from these sources"
                              % (path, lib.tqk_abi_version(), KERNEL_ABI))
        if int(lib.tqk_page_size()) != native.page_size():
            raise KernelError("the kernel library's cache pages hold %d positions, the engine library's %d: build both from the same sources"
                              % (lib.tqk_page_size(), native.page_size()))
        _LIB = lib
    return _LIB


def library_path():
    library()
    return _LIB._name


def _check(status, name):
    if status != 0:
        raise KernelError("%s: %s" % (name, library().tqk_last_error().decode("utf-8", "replace")))


def _code(dtype):
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError("unsupported dtype %s (float32 and bfloat16 only)" % dtype)


def _dev(t, name, dtype=None, shape=None):
    if not isinstance(t, torch.Tensor):
        raise KernelError("%s must be a tensor" % name)
    if t.device.type != "cuda":
        raise KernelError("%s is on %s: the kernels run on the GPU only" % (name, t.device))
    if not t.is_contiguous():
        raise KernelError("%s must be contiguous" % name)
    if dtype is not None and t.dtype != dtype:
        raise KernelError("%s must be %s, got %s" % (name, dtype, t.dtype))
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError("%s must have shape %s, got %s" % (name, tuple(shape), tuple(t.shape)))
    return ctypes.c_void_p(t.data_ptr())


def _opt(t, name, dtype=None, shape=None):
    return ctypes.c_void_p(0) if t is None else _dev(t, name, dtype, shape)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def embed(table, ids, out, copy=None, copy_weight=None, ss_out=None, scale=1.0):
    """out[t] = scale * float32(table[ids[t]]);  table [V,H], ids [T] int32, out [T,H] float32.
    copy (optional): the same as bfloat16 [T,H], times copy_weight [H] if given; ss_out
    (optional, float32, at least T values, T <= 16): sums of squares of the rows."""
    vocab, hidden = table.shape
    n = ids.shape[0]
    if ss_out is not None and ss_out.numel() < max(n, 1):
        raise KernelError("embed: ss_out holds %d values for %d tokens" % (ss_out.numel(), n))
    _check(library().tqk_embed(_dev(table, "table"), _code(table.dtype), _dev(ids, "ids", torch.int32, (n,)),
                               n, hidden, vocab, ctypes.c_float(scale), _dev(out, "out", torch.float32, (n, hidden)),
                               _opt(copy, "copy", torch.bfloat16, (n, hidden)),
                               _opt(copy_weight, "copy_weight", torch.bfloat16, (hidden,)),
                               _opt(ss_out, "ss_out", torch.float32), _stream()),
           "embed")
    return out


def random_normal(out, key, std, plus_one=False):
    """out (float32 or bfloat16, any shape) = std * z(key, i) (+ 1): the stream of
    weights.random_init for the 64-bit key, element i in the tensor's row-major order."""
    _check(library().tqk_random_normal(_dev(out, "out"), _code(out.dtype), ctypes.c_longlong(out.numel()),
                                       ctypes.c_uint64(int(key) & 0xFFFFFFFFFFFFFFFF), ctypes.c_float(std),
                                       1 if plus_one else 0, _stream()), "random_normal")
    return out


def probe_read(buf, repeats=5, shapes=((0, 256), (1024, 256), (2048, 64), (4096, 64), (4096, 256))):
    """GB/s of a plain streaming read of `buf` (a contiguous tensor of a multiple of 16 bytes): the best timed launch of
    `repeats` for each of a few grid shapes (blocks, threads per block; 0 blocks: two per compute unit), after one launch
    each that does not count.  How many waves stream at once moves the figure by a fifth, so the best shape is the probe."""
    n = buf.numel() * buf.element_size()
    sink = torch.zeros(1, dtype=torch.int32, device=buf.device)
    best = 0.0
    for blocks, threads in shapes:
        for i in range(repeats + 1):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            _check(library().tqk_probe_read(_dev(buf, "buf"), ctypes.c_longlong(n), int(blocks), int(threads), _dev(sink, "sink"), _stream()), "probe_read")
            b.record()
            b.synchronize()
            if i:
                best = max(best, n / (a.elapsed_time(b) * 1e-3) / 1e9)
    return best


def probe_mfma(turns=200000, repeats=3):
    """PFLOP/s of a loop of 32x32x16 bfloat16 matrix-core products on registers, all compute units busy."""
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    flops = ctypes.c_double(0.0)
    best = 0.0
    for i in range(repeats + 1):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        _check(library().tqk_probe_mfma(ctypes.c_longlong(turns if i else 1000), _dev(sink, "sink"), ctypes.byref(flops), _stream()), "probe_mfma")
        b.record()
        b.synchronize()
        if i:
            best = max(best, flops.value / (a.elapsed_time(b) * 1e-3) / 1e15)
    return best


def gather_rows(src, rows, out):
    """out[r] = src[rows[r]]: rows of any dtype and width gathered by int32 index (at most 65535 of them)."""
    n = rows.shape[0]
    row_bytes = src[0].numel() * src.element_size() if src.shape[0] else 0
    if out.shape[0] != n or out.dtype != src.dtype or tuple(out.shape[1:]) != tuple(src.shape[1:]):
        raise KernelError("gather_rows: out is %s of %s for %d rows of %s" % (tuple(out.shape), out.dtype, n, tuple(src.shape)))
    if n and (int(rows.min()) < 0 or int(rows.max()) >= src.shape[0]):
        raise KernelError("gather_rows: a row index outside the %d rows" % src.shape[0])
    _check(library().tqk_gather_rows(_dev(src, "src"), _dev(rows, "rows", torch.int32, (n,)), n, ctypes.c_longlong(row_bytes),
                                     _dev(out, "out"), _stream()), "gather_rows")
    return out


def add_bias(x, bias):
    """In place: x[r, :] += bias; x [rows, n], bias [n]; float32 or bfloat16 each."""
    rows, n = x.shape
    _check(library().tqk_add_bias(_dev(x, "x"), _code(x.dtype), _dev(bias, "bias", None, (n,)), _code(bias.dtype), rows, n, _stream()), "add_bias")
    return x


def convert(src, out):
    """out = src in out's dtype (float32 and bfloat16)."""
    if src.numel() != out.numel():
        raise KernelError("convert: %d values into %d" % (src.numel(), out.numel()))
    _check(library().tqk_convert(_dev(src, "src"), _code(src.dtype), _dev(out, "out"), _code(out.dtype), ctypes.c_longlong(src.numel()),
                                 _stream()), "convert")
    return out


def finish_logits(logits, bias=None, scale=1.0, cap=0.0):
    """In place: logits = (logits + bias) * scale, then cap * tanh(logits / cap) if cap > 0."""
    rows, vocab = logits.shape
    _check(library().tqk_finish_logits(_dev(logits, "logits", torch.float32), rows, vocab,
                                       _opt(bias, "bias", torch.float32, (vocab,)), ctypes.c_float(scale),
                                       ctypes.c_float(cap), _stream()), "finish_logits")
    return logits


def add_rmsnorm(h, delta, weight, eps, out, rows=None, write_back=False):
    """out = rmsnorm(h + delta) * weight; with write_back h becomes h + delta.

    h: [T,H] float32 or None.  delta: [T,H] of out's dtype, a product's PartialSums, or None.
    rows: int32 row indices (then out has one row per index) or None for all rows."""
    hidden = weight.shape[0]
    n_rows = out.shape[0]
    src_rows = (h if h is not None else delta).shape[0]
    if rows is None and src_rows != n_rows:
        raise KernelError("add_rmsnorm: %d input rows but %d output rows" % (src_rows, n_rows))
    if isinstance(delta, PartialSums):
        pieces = delta.sums.shape[0]
        if delta.dtype != out.dtype or tuple(delta.shape) != (src_rows, hidden):
            raise KernelError("add_rmsnorm: the update's sums are %s of %s, wanted %s of %s"
                              % (delta.shape, delta.dtype, (src_rows, hidden), out.dtype))
        _check(library().tqk_add_rmsnorm_sums(
            _opt(h, "h", torch.float32, (src_rows, hidden)), _dev(delta.sums, "sums", torch.float32), pieces, src_rows,
            _code(out.dtype), _dev(weight, "weight", None, (hidden,)), _code(weight.dtype), ctypes.c_float(eps),
            _opt(rows, "rows", torch.int32, (n_rows,)), n_rows, hidden, _dev(out, "out", None, (n_rows, hidden)),
            1 if write_back else 0, _stream()), "add_rmsnorm")
        return out
    _check(library().tqk_add_rmsnorm(
        _opt(h, "h", torch.float32, (src_rows, hidden)), _opt(delta, "delta", out.dtype, (src_rows, hidden)),
        _code(out.dtype), _dev(weight, "weight", None, (hidden,)), _code(weight.dtype), ctypes.c_float(eps),
        _opt(rows, "rows", torch.int32, (n_rows,)), n_rows, hidden, _dev(out, "out", None, (n_rows, hidden)),
        1 if write_back else 0, _stream()), "add_rmsnorm")
    return out


def gemm(x, w, bias, out):
    """out[M,N] = x[M,K] w[N,K]^T (+ bias[N]), float32 accumulation, any dtype mix."""
    m, k = x.shape
    n = w.shape[0]
    lib = library()
    bias_code = _code(bias.dtype) if bias is not None else 0
    need = int(lib.tqk_gemm_scratch_bytes(_code(x.dtype), _code(w.dtype), bias_code, _code(out.dtype), m, n, k))
    scratch = torch.empty((need,), dtype=torch.uint8, device=x.device) if need else None
    _check(lib.tqk_gemm(
        _dev(x, "x", None, (m, k)), _code(x.dtype), _dev(w, "w", None, (n, k)), _code(w.dtype),
        _opt(bias, "bias", None, (n,)), bias_code,
        _dev(out, "out", None, (m, n)), _code(out.dtype), m, n, k, _opt(scratch, "scratch"), _stream()), "gemm")
    return out


def rope_store(qkv, bias, cos, sin, rot_dim, style, tok_seq, tok_pos, page_table, keys, values, q_out,
               n_heads, n_kv_heads, head_dim, write_kv=True):
    """Bias, rotation of q and k, q to q_out, k and v into the cache pages
    (keys [pages, kv heads, 64, d], values [pages, kv heads, d, 64]).  qkv: [T, total], or where
    rope_store_takes_sums says so the product's PartialSums."""
    n = qkv.shape[0]
    total = (n_heads + 2 * n_kv_heads) * head_dim
    max_pos = 0
    if style != STYLE_NONE:
        max_pos = cos.shape[0]
        _dev(cos, "cos", torch.float32, (max_pos, rot_dim // 2))
        _dev(sin, "sin", torch.float32, (max_pos, rot_dim // 2))
    n_seqs, width, n_pages = 0, 0, 0
    if write_kv:
        n_seqs, width = page_table.shape
        n_pages = keys.shape[0]
        _dev(keys, "keys", qkv.dtype, (n_pages, n_kv_heads, 64, head_dim))
        _dev(values, "values", qkv.dtype, (n_pages, n_kv_heads, head_dim, 64))
    if isinstance(qkv, PartialSums):
        if tuple(qkv.shape) != (n, total) or qkv.dtype != torch.bfloat16:
            raise KernelError("rope_store: the product's sums are %s of %s, wanted %s of bfloat16" % (qkv.shape, qkv.dtype, (n, total)))
        _check(library().tqk_rope_store_sums(
            _dev(qkv.sums, "sums", torch.float32), qkv.sums.shape[0], _opt(bias, "bias", None, (total,)),
            _code(bias.dtype) if bias is not None else 0,
            _opt(cos if style != STYLE_NONE else None, "cos"), _opt(sin if style != STYLE_NONE else None, "sin"),
            rot_dim, style, max_pos, _opt(tok_seq, "tok_seq", torch.int32, (n,)), _dev(tok_pos, "tok_pos", torch.int32, (n,)),
            _opt(page_table if write_kv else None, "page_table", torch.int32), width, n_seqs,
            _opt(keys if write_kv else None, "keys"), _opt(values if write_kv else None, "values"), n_pages,
            _dev(q_out, "q_out", torch.bfloat16, (n, n_heads, head_dim)), n, n_heads, n_kv_heads, head_dim,
            1 if write_kv else 0, _stream()), "rope_store")
        return q_out
    _check(library().tqk_rope_store(
        _dev(qkv, "qkv", None, (n, total)), _code(qkv.dtype), _opt(bias, "bias", None, (total,)),
        _code(bias.dtype) if bias is not None else 0,
        _opt(cos if style != STYLE_NONE else None, "cos"), _opt(sin if style != STYLE_NONE else None, "sin"),
        rot_dim, style, max_pos, _opt(tok_seq, "tok_seq", torch.int32, (n,)), _dev(tok_pos, "tok_pos", torch.int32, (n,)),
        _opt(page_table if write_kv else None, "page_table", torch.int32), width, n_seqs,
        _opt(keys if write_kv else None, "keys"), _opt(values if write_kv else None, "values"), n_pages,
        _dev(q_out, "q_out", qkv.dtype, (n, n_heads, head_dim)), n, n_heads, n_kv_heads, head_dim,
        1 if write_kv else 0, _stream()), "rope_store")
    return q_out


def rope_store_takes_sums(act_dtype, bias, rot_dim, style, head_dim):
    """Whether rope_store takes a product's PartialSums in this case."""
    if act_dtype != torch.bfloat16:
        return False
    return bool(library().tqk_rope_store_takes_sums(BF16, 0 if bias is None else 1, _code(bias.dtype) if bias is not None else 0,
                                                    int(rot_dim), int(style), int(head_dim)))


def attention(q, keys, values, tok_seq, tok_pos, page_table, window, scale, out):
    """Generic softmax attention of q [T,heads,d] over the paged cache; out [T, heads*d]."""
    n, n_heads, head_dim = q.shape
    n_pages, n_kv_heads = keys.shape[0], keys.shape[1]
    n_seqs, width = page_table.shape
    _check(library().tqk_attention(
        _dev(q, "q"), _dev(keys, "keys", q.dtype, (n_pages, n_kv_heads, 64, head_dim)),
        _dev(values, "values", q.dtype, (n_pages, n_kv_heads, head_dim, 64)), _code(q.dtype),
        _dev(tok_seq, "tok_seq", torch.int32, (n,)), _dev(tok_pos, "tok_pos", torch.int32, (n,)),
        _dev(page_table, "page_table", torch.int32), width, n_seqs, n_pages, int(window or 0), ctypes.c_float(scale),
        _dev(out, "out", q.dtype, (n, n_heads * head_dim)), n, n_heads, n_kv_heads, head_dim, _stream()), "attention")
    return out


def swiglu(gate_up, out):
    """out[t,i] = silu(gate_up[t,i]) * gate_up[t,I+i]"""
    n, inter = out.shape
    _check(library().tqk_swiglu(_dev(gate_up, "gate_up", out.dtype, (n, 2 * inter)), _dev(out, "out"),
                                _code(out.dtype), n, inter, _stream()), "swiglu")
    return out


def argmax(logits, out):
    """out[r] = lowest index of the largest value of row r; logits [R,V] float32, out [R] int32."""
    rows, vocab = logits.shape
    scratch = torch.empty((library().tqk_argmax_scratch_floats(rows, vocab),), dtype=torch.float32, device=logits.device)
    _check(library().tqk_argmax(_dev(logits, "logits", torch.float32), rows, vocab,
                                _dev(out, "out", torch.int32, (rows,)), _dev(scratch, "scratch"), _stream()), "argmax")
    return out


def repeat_penalty(logits, row_req, hist, times, hist_len, penalty):
    """In place: for every token in the history of the row's request, once per occurrence,
    l > 0 ? l / penalty : l * penalty.  hist, times, hist_len: as append_history keeps them."""
    rows, vocab = logits.shape
    n_req, cap = hist.shape
    _check(library().tqk_repeat_penalty(
        _dev(logits, "logits", torch.float32), rows, vocab, _dev(row_req, "row_req", torch.int32, (rows,)),
        _dev(hist, "hist", torch.int32), _dev(times, "times", torch.int32, (n_req, cap)), cap,
        _dev(hist_len, "hist_len", torch.int32, (n_req,)), n_req, ctypes.c_float(penalty), _stream()), "repeat_penalty")
    return logits


def append_history(tokens, row_req, hist, times, hist_len):
    """tokens[r] joins the history of request row_req[r] (hist, times int32 [requests, cap], zeros
    and hist_len 0 at the start; different requests in one call)."""
    rows = tokens.shape[0]
    n_req, cap = hist.shape
    _check(library().tqk_append_history(
        _dev(tokens, "tokens", torch.int32, (rows,)), _dev(row_req, "row_req", torch.int32, (rows,)),
        _dev(hist, "hist", torch.int32), _dev(times, "times", torch.int32, (n_req, cap)), cap,
        _dev(hist_len, "hist_len", torch.int32, (n_req,)), rows, _stream()), "append_history")


def sample(logits, temperature, top_k, top_p, uniforms, out):
    """One draw per row of logits [R,V] float32 with the uniforms [R] float32; out [R] int32."""
    rows, vocab = logits.shape
    lib = library()
    need = int(lib.tqk_sample_scratch_bytes(rows, vocab, int(top_k), ctypes.c_float(top_p)))
    scratch = torch.empty((need,), dtype=torch.uint8, device=logits.device) if need else None
    _check(lib.tqk_sample(
        _dev(logits, "logits", torch.float32), rows, vocab, ctypes.c_float(temperature), int(top_k),
        ctypes.c_float(top_p), _dev(uniforms, "uniforms", torch.float32, (rows,)),
        _dev(out, "out", torch.int32, (rows,)), _opt(scratch, "scratch"), _stream()), "sample")
    return out


def attention_decode_supported(head_dim):
    return bool(library().tqk_attention_decode_supported(int(head_dim)))


def attention_decode(q, keys, values, tok_pos, page_table, window, scale, out, target_blocks=256, n_parts=None):
    """Attention of one new token per sequence (q [B, heads, d] bfloat16, row b belongs to
    sequence b at position tok_pos[b]) over the paged cache; out [B, heads*d].  n_parts: into how many partitions
    a sequence's pages are dealt (as many as the table is wide: a block of one wave per page)."""
    n, n_heads, head_dim = q.shape
    n_pages, n_kv_heads = keys.shape[0], keys.shape[1]
    n_seqs, width = page_table.shape
    if n_seqs != n:
        raise KernelError("attention_decode: %d query rows for %d sequences (one token each is required)" % (n, n_seqs))
    q_blocks = (n_heads // n_kv_heads + 15) // 16
    groups = max(1, n * n_kv_heads * q_blocks)
    # partitions take the live pages in turn, four waves each: no more than a quarter of the pages there can be
    if n_parts is None:
        n_parts = max(1, min((width + 3) // 4, target_blocks // groups))
    part_out = part_ml = None
    if n_parts > 1:
        part_out = torch.empty((n, n_heads, n_parts, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n, n_heads, n_parts, 2), dtype=torch.float32, device=q.device)
    _check(library().tqk_attention_decode(
        _dev(q, "q", torch.bfloat16), _dev(keys, "keys", torch.bfloat16, (n_pages, n_kv_heads, 64, head_dim)),
        _dev(values, "values", torch.bfloat16, (n_pages, n_kv_heads, head_dim, 64)),
        _dev(tok_pos, "tok_pos", torch.int32, (n,)), _dev(page_table, "page_table", torch.int32), width, n, n_pages,
        int(window or 0), ctypes.c_float(scale), n_parts, _opt(part_out, "part_out"), _opt(part_ml, "part_ml"),
        _dev(out, "out", torch.bfloat16, (n, n_heads * head_dim)), n_heads, n_kv_heads, head_dim, _stream()),
        "attention_decode")
    return out


def attention_prefill_supported(head_dim):
    return bool(library().tqk_attention_prefill_supported(int(head_dim)))


def attention_prefill_tile(n_tokens, n_heads, n_kv_heads, head_dim):
    """Queries per tile (16, 32, 64 or 128) that suit a step of n_tokens for these head counts."""
    return int(library().tqk_attention_prefill_tile(int(n_tokens), int(n_heads), int(n_kv_heads), int(head_dim)))


def attention_prefill(q, keys, values, tok_pos, page_table, tile_seq, tile_tok0, tile_count, seq_start, seq_new,
                      window, scale, out, tile_queries=64):
    """Causal attention of tiles of up to tile_queries (16, 32, 64 or 128) consecutive queries
    (q [T, heads, d] bfloat16) over the paged cache; out [T, heads*d].  tile_count must not
    exceed tile_queries (the caller built the tiles; the kernel covers no more)."""
    n, n_heads, head_dim = q.shape
    n_pages, n_kv_heads = keys.shape[0], keys.shape[1]
    n_seqs, width = page_table.shape
    n_tiles = tile_seq.shape[0]
    _check(library().tqk_attention_prefill(
        _dev(q, "q", torch.bfloat16), _dev(keys, "keys", torch.bfloat16, (n_pages, n_kv_heads, 64, head_dim)),
        _dev(values, "values", torch.bfloat16, (n_pages, n_kv_heads, head_dim, 64)),
        _dev(tok_pos, "tok_pos", torch.int32, (n,)), _dev(page_table, "page_table", torch.int32), width, n_seqs, n_pages,
        _dev(tile_seq, "tile_seq", torch.int32, (n_tiles,)), _dev(tile_tok0, "tile_tok0", torch.int32, (n_tiles,)),
        _dev(tile_count, "tile_count", torch.int32, (n_tiles,)), n_tiles, int(tile_queries),
        _dev(seq_start, "seq_start", torch.int32, (n_seqs,)), _dev(seq_new, "seq_new", torch.int32, (n_seqs,)),
        int(window or 0), ctypes.c_float(scale), _dev(out, "out", torch.bfloat16, (n, n_heads * head_dim)),
        n, n_heads, n_kv_heads, head_dim, _stream()), "attention_prefill")
    return out


# ---- skinny products with the neighbouring small operations folded in (decoding) ---------------
# A norm between two products is split over them: `fused_residual` (or `embed`) writes the
# stream times the next norm's weight and the rows' sums of squares in pieces; the consuming
# product gets both as `norm=(ss_parts, n_parts, eps)` and divides its result by the rows' rms.
def _norm_args(norm, m):
    if norm is None:
        return ctypes.c_void_p(0), 0, ctypes.c_float(0.0)
    ss_parts, n_parts, eps = norm
    if ss_parts.dtype != torch.float32 or ss_parts.numel() < 16 * n_parts or n_parts < 1:
        raise KernelError("sums of squares: %d float32 values for %d pieces of 16 rows" % (ss_parts.numel(), n_parts))
    return _dev(ss_parts, "ss_parts", torch.float32), int(n_parts), ctypes.c_float(eps)


class PackedWeight:
    """A bfloat16 weight [n, k] in the order the lanes of the few-row kernels take it:
    data [tiles, k/32, 64, 8], where tile t holds 16 rows, lane = 16 * ((k % 32) / 8) + row % 16.
    parts: the weight is that many stacked weights of n/parts rows (gate and up rows), each
    padded with zero rows to whole tiles."""

    dtype = torch.bfloat16

    def __init__(self, data, n, k, parts):
        self.data, self.shape, self.parts = data, (n, k), parts


def pack_weight(weight, parts=1):
    """The PackedWeight of a contiguous bfloat16 weight [n, k], k a multiple of 32 (runs
    wherever the weight lives; takes the weight's size in new memory)."""
    n, k = weight.shape
    if weight.dtype != torch.bfloat16 or k % 32 or n % parts:
        raise KernelError("pack_weight: needs bfloat16 [n, k] with k a multiple of 32 and n of %d parts, got %s %s"
                          % (parts, weight.dtype, tuple(weight.shape)))
    per = n // parts
    tiles = (per + 15) // 16
    if weight.is_cuda:
        data = torch.empty((parts * tiles, k // 32, 64, 8), dtype=torch.bfloat16, device=weight.device)
        _check(library().tqk_pack_weight(_dev(weight, "weight"), _dev(data, "data"), n, k, parts, _stream()), "pack_weight")
        return PackedWeight(data, n, k, parts)
    w = weight.reshape(parts, per, k)
    if per % 16:
        w = torch.cat([w, w.new_zeros((parts, tiles * 16 - per, k))], dim=1)
    # [part, tile, row, k step, k group, 8] -> [part, tile, k step, k group, row, 8]
    data = w.reshape(parts, tiles, 16, k // 32, 4, 8).permute(0, 1, 3, 4, 2, 5).contiguous()
    return PackedWeight(data.reshape(parts * tiles, k // 32, 64, 8), n, k, parts)


def unpack_weight(packed):
    """The rows [n, k] of a PackedWeight on the GPU (what pack_weight was given)."""
    n, k = packed.shape
    rows = torch.empty((n, k), dtype=torch.bfloat16, device=packed.data.device)
    _check(library().tqk_unpack_weight(_dev(packed.data, "data"), _dev(rows, "rows"), n, k, packed.parts, _stream()), "unpack_weight")
    return rows


def _weight(weight, name, n, k, parts=1):
    """Pointer and packed flag of a product's weight, row by row [n, k] or packed."""
    if isinstance(weight, PackedWeight):
        if tuple(weight.shape) != (n, k) or weight.parts != parts:
            raise KernelError("%s: the packed weight is %s in %d parts, wanted %s in %d"
                              % (name, tuple(weight.shape), weight.parts, (n, k), parts))
        return _dev(weight.data, name, torch.bfloat16), 1
    return _dev(weight, name, torch.bfloat16, (n, k)), 0


def fused_store(x, weight, out, norm=None, rows=None):
    """out[M,N] = x weight^T (divided by the rows' rms with `norm`); x bfloat16 [*, K]
    (rows: int32 indices of the M rows used).  Here and in the other fused_* products the
    weight is a tensor [N, K] or its PackedWeight."""
    m, n = out.shape
    k = weight.shape[1]
    if x.shape[1] != k or (rows is None and x.shape[0] != m) or x.shape[0] > 16:
        raise KernelError("fused_store: x is %s for %d rows of %d (at most 16 rows)" % (tuple(x.shape), m, k))
    ss, n_parts, eps = _norm_args(norm, m)
    w, packed = _weight(weight, "weight", n, k)
    _check(library().tqk_fused_store(
        _dev(x, "x", torch.bfloat16), _opt(rows, "rows", torch.int32, (m,)), ss, n_parts, eps,
        w, packed, _dev(out, "out"), _code(out.dtype), m, n, k, _stream()), "fused_store")
    return out


def fused_gated(x, weight_gate_up, out, norm=None):
    """out[M, I] = silu(gate) * up of x [gate; up]^T (normalised with `norm`)."""
    m, inter = out.shape
    k = weight_gate_up.shape[1]
    ss, n_parts, eps = _norm_args(norm, m)
    w, packed = _weight(weight_gate_up, "weight", 2 * inter, k, parts=2)
    _check(library().tqk_fused_gated(
        _dev(x, "x", torch.bfloat16, (m, k)), ss, n_parts, eps,
        w, packed, _dev(out, "out", torch.bfloat16), m, 2 * inter, k,
        _stream()), "fused_gated")
    return out


MID_MAX_ROWS = 128


class PartialSums:
    """A product [rows, n] that has not been added up: sums float32 [pieces, rows, n] over pieces
    of its K.  add_rmsnorm takes it as the update (adds the pieces in order, rounds to `dtype`
    as the finished product would be)."""

    def __init__(self, sums, dtype):
        self.sums, self.dtype = sums, dtype
        self.shape = tuple(sums.shape[1:])


def _mid_scratch(m, n, k, gated, device):
    splits = int(library().tqk_mid_splits(n, k, 1 if gated else 0))
    return torch.empty((splits, m, n), dtype=torch.float32, device=device) if splits > 1 else None


def mid_store(x, weight, out=None, finish=True):
    """out[M,N] = x weight^T for up to 128 rows of bfloat16; weight: a PackedWeight; out: bfloat16
    or float32, made here (bfloat16) if not given.  finish=False: where the kernel cuts K into
    pieces, their PartialSums (of out's dtype) are returned in place of out."""
    m, k = x.shape
    if not isinstance(weight, PackedWeight):
        raise KernelError("mid_store: the weight must be packed (pack_weight)")
    n = weight.shape[0]
    w, _ = _weight(weight, "weight", n, k)
    scratch = _mid_scratch(m, n, k, False, x.device)
    leave = not finish and scratch is not None
    dtype = out.dtype if out is not None else torch.bfloat16
    if out is None and not leave:
        out = torch.empty((m, n), dtype=dtype, device=x.device)
    _check(library().tqk_mid_store(_dev(x, "x", torch.bfloat16, (m, k)), w, _opt(None if leave else out, "out", None, (m, n)),
                                   _code(dtype), m, n, k, _opt(scratch, "scratch"), 0 if leave else 1, _stream()), "mid_store")
    return PartialSums(scratch, dtype) if leave else out


def mid_gated(x, weight_gate_up, out):
    """out[M, I] = silu(gate) * up of x [gate; up]^T for up to 128 rows; weight: a PackedWeight in 2 parts."""
    m, inter = out.shape
    k = x.shape[1]
    if not isinstance(weight_gate_up, PackedWeight):
        raise KernelError("mid_gated: the weight must be packed (pack_weight with parts=2)")
    w, _ = _weight(weight_gate_up, "weight", 2 * inter, k, parts=2)
    scratch = _mid_scratch(m, 2 * inter, k, True, x.device)
    _check(library().tqk_mid_gated(_dev(x, "x", torch.bfloat16, (m, k)), w, _dev(out, "out", torch.bfloat16), m, 2 * inter, k,
                                   _opt(scratch, "scratch"), _stream()), "mid_gated")
    return out


def fused_residual_parts(n, k):
    """In how many pieces fused_residual gives the sums of squares for a weight [n, k]
    (never more than ceil(n / 16))."""
    return int(library().tqk_fused_residual_parts(int(n), int(k)))


def fused_residual(x, weight, h, xw, next_norm_weight=None, ss_out=None):
    """h[M,N] += bfloat16(x weight^T) (float32 sum); xw = bfloat16(h * next_norm_weight) (or
    bfloat16(h)); ss_out (optional, float32 [fused_residual_parts(N, K), 16]): the rows' sums of
    squares in pieces.  Returns the number of pieces."""
    m, k = x.shape
    n = weight.shape[0]
    parts = fused_residual_parts(n, k)
    if ss_out is not None and ss_out.numel() < parts * 16:
        raise KernelError("fused_residual: ss_out holds %d values, %d pieces of 16 are written" % (ss_out.numel(), parts))
    w, packed = _weight(weight, "weight", n, k)
    _check(library().tqk_fused_residual(
        _dev(x, "x", torch.bfloat16), w, packed, _dev(h, "h", torch.float32, (m, n)),
        _opt(next_norm_weight, "next_norm_weight", torch.bfloat16, (n,)), _dev(xw, "xw", torch.bfloat16, (m, n)),
        _opt(ss_out, "ss_out", torch.float32), m, n, k, _stream()), "fused_residual")
    return parts


def fused_qkv(x, weight, bias, cos, sin, tok_pos, page_table, keys, values, q_out, n_heads, n_kv_heads, head_dim,
              norm=None):
    """q, k, v of a decoding step (row m is sequence m): product (normalised with `norm`),
    bias, rotation, q out, k and v into the cache pages."""
    m, k = x.shape
    total = (n_heads + 2 * n_kv_heads) * head_dim
    n_pages = keys.shape[0]
    width = page_table.shape[1]
    max_pos = cos.shape[0]
    ss, n_parts, eps = _norm_args(norm, m)
    w, packed = _weight(weight, "weight", total, k)
    _check(library().tqk_fused_qkv(
        _dev(x, "x", torch.bfloat16), ss, n_parts, eps,
        w, packed, _opt(bias, "bias", torch.bfloat16, (total,)),
        _dev(cos, "cos", torch.float32, (max_pos, head_dim // 2)), _dev(sin, "sin", torch.float32, (max_pos, head_dim // 2)), max_pos,
        _dev(tok_pos, "tok_pos", torch.int32, (m,)), _dev(page_table, "page_table", torch.int32, (m, width)), width,
        _dev(keys, "keys", torch.bfloat16, (n_pages, n_kv_heads, 64, head_dim)),
        _dev(values, "values", torch.bfloat16, (n_pages, n_kv_heads, head_dim, 64)), n_pages,
        _dev(q_out, "q_out", torch.bfloat16, (m, n_heads, head_dim)), m, n_heads, n_kv_heads, head_dim, k, _stream()),
        "fused_qkv")
    return q_out
