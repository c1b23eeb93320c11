"""Each kernel alone against a plain float32 torch expression of the same operation, at
sizes other than the tiny models': widths and vocabularies that are no power of two,
head sizes in steps of 16, odd numbers of heads and groups.  Inputs are made so that a
fault shows: one far key that dominates, keys just inside and just outside a window,
pages in scrambled order, NaN in everything that must not be read."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen2 as plain
from tq_kv_amd import kernels as K

pytestmark = pytest.mark.gpu
DEV = "cuda"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": dict(atol=1e-5, rtol=1e-5), "bfloat16": dict(atol=2e-2, rtol=2e-2)}


def rand(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def ints(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


def test_library_is_built_and_loaded():
    assert K.library().tqk_abi_version() == K.KERNEL_ABI == 13
    assert K.library_path().endswith(".so")
    with pytest.raises(K.KernelError, match="GPU only"):
        K.swiglu(torch.zeros(2, 4), torch.zeros(2, 2))
    with pytest.raises(K.KernelError, match="shape"):
        K.swiglu(torch.zeros(2, 5, device=DEV), torch.zeros(2, 2, device=DEV))


@pytest.mark.parametrize("shape,dtype", [((37, 70), torch.float32), ((5, 3, 16), torch.bfloat16), ((9, 7), torch.bfloat16), ((4, 33), torch.int32),
                                         ((300, 1), torch.int32), ((20, 4096), torch.float32)])
def test_gather_rows(shape, dtype):
    g = torch.Generator().manual_seed(1)
    src = (torch.randn(*shape, generator=g) * 100).to(dtype).to(DEV)
    idx = torch.randint(0, shape[0], (53,), generator=g).to(torch.int32).to(DEV)
    out = torch.full((53,) + tuple(shape[1:]), 7, dtype=dtype, device=DEV)
    assert torch.equal(K.gather_rows(src, idx, out), src[idx.long()])
    assert K.gather_rows(src, idx[:0], out[:0]).shape[0] == 0
    with pytest.raises(K.KernelError, match="outside"):
        K.gather_rows(src, ints([shape[0]]), out[:1])


@pytest.mark.parametrize("xd,bd", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.float32, torch.bfloat16),
                                   (torch.bfloat16, torch.float32)])
def test_add_bias_and_convert(xd, bd):
    x, b = rand(13, 77, seed=3, dtype=xd), rand(77, seed=4, dtype=bd)
    want = (x.float() + b.float()).to(xd)
    assert torch.equal(K.add_bias(x.clone(), b), want)
    out = torch.empty(13, 77, dtype=bd, device=DEV)
    assert torch.equal(K.convert(x, out), x.to(bd))


def test_pack_weight_on_the_gpu_equals_the_plain_reordering():
    for n, k, parts in ((40, 96, 1), (224, 96, 2), (3584, 512, 1), (19, 64, 1)):
        w = rand(n, k, seed=n, dtype=torch.bfloat16)
        got = K.pack_weight(w, parts)
        want = K.pack_weight(w.cpu(), parts)              # torch's reshape and permute on the host
        assert tuple(got.data.shape) == tuple(want.data.shape) and torch.equal(got.data.cpu(), want.data)


def test_unpack_weight_gives_the_rows_back():
    # parts whose rows are no multiple of 16 (the packed copy pads them), k of less and of more than a block's 512
    # columns and no multiple of them, and the width of a vocabulary
    for n, k, parts in ((40, 96, 1), (38, 96, 2), (224, 1056, 2), (3584, 512, 1), (19, 64, 1), (50000, 160, 1)):
        w = rand(n, k, seed=n + 1, dtype=torch.bfloat16)
        assert torch.equal(K.unpack_weight(K.pack_weight(w, parts)), w), (n, k, parts)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden", [70, 72, 3584, 9000])
def test_embed(dtype, hidden):
    table = rand(301, hidden, seed=1, dtype=DT[dtype])
    ids = ints([0, 300, 17, 17, 5])
    out = torch.full((5, hidden), float("nan"), device=DEV)
    K.embed(table, ids, out)
    assert torch.equal(out, table.float()[ids.long()])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden", [70, 72, 1000, 3584, 9000])
def test_add_rmsnorm(dtype, hidden):
    act = DT[dtype]
    h = rand(7, hidden, seed=2, scale=2.0)
    delta = rand(7, hidden, seed=3, dtype=act)
    w = (1 + rand(hidden, seed=4, scale=0.1)).to(act)
    eps = 3e-5
    want_h = h + delta.float()
    want = plain.rms_norm(want_h, w.float(), eps)
    h1 = h.clone()
    out = torch.empty(7, hidden, dtype=act, device=DEV)
    K.add_rmsnorm(h1, delta, w, eps, out, write_back=True)
    assert torch.equal(h1, want_h)
    torch.testing.assert_close(out.float(), want, **TOL[dtype])
    # without a delta h is only read; a float32 weight with bfloat16 activations is taken too
    h2 = h.clone()
    K.add_rmsnorm(h2, None, w.float(), eps, out)
    assert torch.equal(h2, h)
    torch.testing.assert_close(out.float(), plain.rms_norm(h, w.float(), eps), **TOL[dtype])
    # chosen rows only, h untouched
    rows = ints([6, 0, 3])
    out3 = torch.empty(3, hidden, dtype=act, device=DEV)
    K.add_rmsnorm(h2, delta, w, eps, out3, rows=rows)
    assert torch.equal(h2, h)
    torch.testing.assert_close(out3.float(), want[rows.long()], **TOL[dtype])
    # norm of an activation tensor alone
    K.add_rmsnorm(None, delta, w, eps, out)
    torch.testing.assert_close(out.float(), plain.rms_norm(delta.float(), w.float(), eps), **TOL[dtype])


@pytest.mark.parametrize("m,n,k", [(1, 7, 5), (3, 100, 33), (65, 129, 200), (130, 64, 48)])
@pytest.mark.parametrize("xd,wd,yd", [("float32", "float32", "float32"), ("bfloat16", "bfloat16", "bfloat16"),
                                      ("bfloat16", "bfloat16", "float32"), ("bfloat16", "float32", "bfloat16")])
def test_gemm_generic(m, n, k, xd, wd, yd):
    x, w, b = rand(m, k, seed=5, dtype=DT[xd]), rand(n, k, seed=6, dtype=DT[wd]), rand(n, seed=7, dtype=DT[wd])
    out = torch.empty(m, n, dtype=DT[yd], device=DEV)
    K.gemm(x, w, None, out)
    want = x.double() @ w.double().t()
    tol = dict(atol=1e-4, rtol=1e-5) if yd == "float32" else dict(atol=0.1, rtol=2e-2)
    torch.testing.assert_close(out.double(), want, **tol)
    K.gemm(x, w, b, out)
    torch.testing.assert_close(out.double(), want + b.double(), **tol)


@pytest.mark.parametrize("rows,n,k,bias", [(1, 130, 96, False), (3, 130, 2500, True), (16, 67, 1024, True),
                                           (7, 64, 3076, False), (5, 200, 1030, True), (2, 130, 97, True)])
def test_gemm_generic_rows_do_not_depend_on_the_batch(rows, n, k, bias):
    """Up to 16 float32 rows go through the kernel for few rows (k a multiple of 4), more through
    the tiled one: the same bits, over chunks and groups of k that are full or not."""
    x, w = rand(70, k, seed=8), rand(n, k, seed=9)
    b = rand(n, seed=10) if bias else None
    full = torch.empty(70, n, device=DEV)
    K.gemm(x, w, b, full)
    torch.testing.assert_close(full.double(), x.double() @ w.double().t() + (b.double() if bias else 0), atol=2e-4, rtol=1e-5)
    few = torch.full((rows, n), float("nan"), device=DEV)
    K.gemm(x[41:41 + rows].contiguous(), w, b, few)
    assert torch.equal(few, full[41:41 + rows])


def value_place(p):
    """Where position p of a page lies in a row of values: inside each 32 positions, the 4
    positions 4g..4g+3 of the first 16 are followed by 16+4g..16+4g+3 of the second 16."""
    return (p & 32) | (((p >> 2) & 3) << 3) | (((p >> 4) & 1) << 2) | (p & 3)


PLACES = [value_place(p) for p in range(64)]


def make_cache(n_pages, nkv, d, dtype):
    nan = float("nan")
    # keys [pages, kv heads, 64, d]; values are kept transposed inside a page
    return (torch.full((n_pages, nkv, 64, d), nan, dtype=dtype, device=DEV),
            torch.full((n_pages, nkv, d, 64), nan, dtype=dtype, device=DEV))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("style,rot", [("halves", 48), ("pairs", 48), ("halves", 32), ("none", 0)])
def test_rope_store(dtype, style, rot):
    act = DT[dtype]
    nh, nkv, d, n_pages = 5, 2, 48, 6
    # two sequences: 3 tokens at positions 62..64 (crossing a page), 2 tokens at 130, 131
    tok_seq, tok_pos = ints([0, 0, 0, 1, 1]), ints([62, 63, 64, 130, 131])
    table = ints([[4, 1, -1], [0, 5, 2]])
    qkv = rand(5, (nh + 2 * nkv) * d, seed=10, dtype=act)
    bias = rand((nh + 2 * nkv) * d, seed=11, dtype=act)
    keys, values = make_cache(n_pages, nkv, d, act)
    q = torch.empty(5, nh, d, dtype=act, device=DEV)
    if style == "none":
        cos = sin = None
        code = K.STYLE_NONE
    else:
        c, s = plain.rope_tables(rot, 777.0, 140)
        cos, sin = c.to(DEV), s.to(DEV)
        code = K.STYLE_HALVES if style == "halves" else K.STYLE_PAIRS
    K.rope_store(qkv, bias, cos, sin, rot, code, tok_seq, tok_pos, table, keys, values, q, nh, nkv, d)

    x = (qkv.float() + bias.float()).cpu()
    pos = tok_pos.cpu().long()

    def rotate(v):                       # v: [tokens, heads, d]
        if style == "none":
            return v
        c, s = plain.rope_tables(rot, 777.0, 140)
        c, s = c[pos][:, None, :], s[pos][:, None, :]
        r = v[..., :rot]
        if style == "halves":            # src/models/turbo_generic.rs:417-427
            x0, x1 = r[..., :rot // 2], r[..., rot // 2:]
            out = torch.cat([x0 * c - x1 * s, x0 * s + x1 * c], -1)
        else:                            # :430-443
            x0, x1 = r[..., 0::2], r[..., 1::2]
            out = torch.stack([x0 * c - x1 * s, x0 * s + x1 * c], -1).flatten(-2)
        return torch.cat([out, v[..., rot:]], -1)       # elements beyond rot_dim pass through (:752-761)
    want_q = rotate(x[:, :nh * d].reshape(5, nh, d))
    want_k = rotate(x[:, nh * d:(nh + nkv) * d].reshape(5, nkv, d))
    want_v = x[:, (nh + nkv) * d:].reshape(5, nkv, d)
    torch.testing.assert_close(q.float().cpu(), want_q, **TOL[dtype])
    written = torch.zeros(n_pages, 64, dtype=torch.bool)
    written_v = torch.zeros(n_pages, 64, dtype=torch.bool)
    for t in range(5):
        page = table.cpu()[tok_seq[t].item(), pos[t].item() // 64].item()
        slot = pos[t].item() % 64
        written[page, slot] = True
        written_v[page, value_place(slot)] = True
        torch.testing.assert_close(keys[page, :, slot].float().cpu(), want_k[t], **TOL[dtype])
        torch.testing.assert_close(values[page, :, :, value_place(slot)].float().cpu(), want_v[t], **TOL[dtype])
    # nothing else was touched
    assert torch.isnan(keys.float().cpu().transpose(1, 2)[~written]).all()
    assert torch.isnan(values.float().cpu().permute(0, 3, 1, 2)[~written_v]).all()
    # a run that reads another run's cache writes none
    keys2, values2 = make_cache(n_pages, nkv, d, act)
    K.rope_store(qkv, bias, cos, sin, rot, code, tok_seq, tok_pos, table, keys2, values2, q, nh, nkv, d, write_kv=False)
    assert torch.isnan(keys2.float()).all()
    torch.testing.assert_close(q.float().cpu(), want_q, **TOL[dtype])


@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("nh,nkv,d", [(28, 4, 128), (3, 1, 64), (7, 7, 8)])
def test_rope_store_vector_kernel_equals_the_general_one(nh, nkv, d, with_bias):
    # bfloat16, halves over the whole head: the kernel with 8-byte accesses.  A float32 bias of
    # the same values sends the same work through the general kernel.
    n_pages, n = 9, 6
    tok_seq, tok_pos = ints([0, 0, 1, 1, 1, 2]), ints([63, 64, 0, 1, 2, 399])
    table = ints([[3, 8, -1, -1, -1, -1, -1], [0, -1, -1, -1, -1, -1, -1], [4, 4, 4, 4, 4, 4, 7]])
    qkv = rand(n, (nh + 2 * nkv) * d, seed=12, dtype=torch.bfloat16)
    bias = rand((nh + 2 * nkv) * d, seed=13, dtype=torch.bfloat16) if with_bias else None
    c, s = plain.rope_tables(d, 1e4, 300)                # position 399 is beyond the table: not rotated
    cos, sin = c.to(DEV), s.to(DEV)
    results = []
    for general in (False, True):
        keys, values = make_cache(n_pages, nkv, d, torch.bfloat16)
        q = torch.empty(n, nh, d, dtype=torch.bfloat16, device=DEV)
        b = bias
        if general:
            b = bias.float() if with_bias else torch.zeros((nh + 2 * nkv) * d, device=DEV)
        K.rope_store(qkv, b, cos, sin, d, K.STYLE_HALVES, tok_seq, tok_pos, table, keys, values, q, nh, nkv, d)
        results.append((q, keys, values))
    for a, b in zip(*results):
        assert torch.equal(torch.isnan(a.float()), torch.isnan(b.float()))          # the same places written
        ok = ~torch.isnan(a.float())
        torch.testing.assert_close(a.float()[ok], b.float()[ok], atol=1e-2, rtol=1e-2)
        assert ok.any()


@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("nh,nkv,d", [(28, 4, 128), (3, 1, 64), (5, 5, 40)])
def test_rope_store_of_many_tokens_equals_the_general_kernel(nh, nkv, d, with_bias):
    # steps of 128 tokens and more store their values through a kernel of their own, whose lanes run
    # along the tokens: three sequences in a packed step (a prompt from 0, a piece that starts inside a
    # page, one token), scrambled pages; against the general kernel (reached with a float32 bias), and
    # with the product given as its sums over pieces of K
    starts, counts = [0, 37, 200], [150, 131, 1]
    tok_seq = ints([i for i, n in enumerate(counts) for _ in range(n)])
    tok_pos = ints([s + j for s, n in zip(starts, counts) for j in range(n)])
    n = sum(counts)
    n_pages = 12
    table = ints([[7, 2, 9, -1], [4, 11, 0, -1], [5, 8, 1, 3]])
    total = (nh + 2 * nkv) * d
    qkv = rand(n, total, seed=14, dtype=torch.bfloat16)
    bias = rand(total, seed=15, dtype=torch.bfloat16) if with_bias else None
    c, s_ = plain.rope_tables(d, 1e4, 300)
    cos, sin = c.to(DEV), s_.to(DEV)
    # the same product as sums of three pieces that add up to it exactly (a half and two quarters)
    sums = K.PartialSums(torch.stack([qkv.float() * 0.5, qkv.float() * 0.25, qkv.float() * 0.25]).contiguous(), torch.bfloat16)
    results = []
    for how in ("vector", "general", "sums"):
        keys, values = make_cache(n_pages, nkv, d, torch.bfloat16)
        q = torch.empty(n, nh, d, dtype=torch.bfloat16, device=DEV)
        b = bias
        if how == "general":
            b = bias.float() if with_bias else torch.zeros(total, device=DEV)
        K.rope_store(sums if how == "sums" else qkv, b, cos, sin, d, K.STYLE_HALVES, tok_seq, tok_pos, table, keys, values, q, nh, nkv, d)
        results.append((q, keys, values))
    for other in results[1:]:
        for a, b in zip(results[0], other):
            assert torch.equal(torch.isnan(a.float()), torch.isnan(b.float()))          # the same places written
            ok = ~torch.isnan(a.float())
            torch.testing.assert_close(a.float()[ok], b.float()[ok], atol=1e-2, rtol=1e-2)
            assert ok.any()
    # vector kernel and sums: the same numbers rounded the same way
    for a, b in zip(results[0], results[2]):
        assert torch.equal(torch.nan_to_num(a.float()), torch.nan_to_num(b.float()))
    # every value where the layout says: page of the position, kv head, element, place of the position
    v_want = (qkv.float() + (bias.float() if with_bias else 0)).to(torch.bfloat16).float()[:, (nh + nkv) * d:].reshape(n, nkv, d).cpu()
    got = results[0][2].float().cpu()
    for t in range(0, n, 7):
        page = table.cpu()[tok_seq[t].item(), tok_pos[t].item() // 64].item()
        assert torch.equal(got[page, :, :, value_place(tok_pos[t].item() % 64)], v_want[t]), t


def paged(k, v, page_ids, n_pages, dtype):
    """Lay k, v [nkv, S, d] out in pages given by page_ids; everything else is NaN."""
    nkv, s, d = k.shape
    keys, values = make_cache(n_pages, nkv, d, dtype)
    for i, p in enumerate(page_ids):
        n = min(64, s - 64 * i)
        if p >= 0 and n > 0:
            keys[p, :, :n] = k[:, 64 * i:64 * i + n].to(dtype)
            values[p][:, :, PLACES[:n]] = v[:, 64 * i:64 * i + n].transpose(1, 2).to(dtype).to(DEV)
    return keys, values


def attention_reference(q, k, v, pos, window, scale):
    """q [T, nh, d] at absolute positions pos over k, v [nkv, S, d]: plain softmax attention."""
    nh = q.shape[1]
    n_rep = nh // k.shape[0]
    kk, vv = plain.repeat_kv(k, n_rep), plain.repeat_kv(v, n_rep)
    att = torch.einsum("thd,hsd->hts", q, kk) * scale
    j = torch.arange(k.shape[1])[None, :]
    vis = j <= pos[:, None]
    if window:
        vis = vis & (j > pos[:, None] - window)
    att = torch.where(vis[None], att, torch.full_like(att, float("-inf")))
    return torch.einsum("hts,hsd->thd", plain.softmax_last(att), vv).reshape(q.shape[0], -1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,d", [(6, 2, 48), (5, 5, 16), (4, 1, 128), (3, 1, 80)])
@pytest.mark.parametrize("window", [0, 70])
def test_attention_generic(dtype, nh, nkv, d, window):
    act = DT[dtype]
    s = 300
    k, v = rand(nkv, s, d, seed=12).cpu(), rand(nkv, s, d, seed=13).cpu()
    # queries: a prompt chunk at positions 200..259 of sequence 0, and single tokens elsewhere
    pos = torch.tensor(list(range(200, 260)) + [0, 63, 64, 299])
    q = rand(len(pos), nh, d, seed=14).cpu()
    # make single keys stand out: for the query at 259 the far key 3, the key at the window's
    # edge (259-69 = 190) and the one just outside it (189)
    q[59] = 0.0
    q[59, :, 0] = 30.0
    k[:, :, 0] *= 0.01
    k[:, 3, 0], k[:, 190, 0], k[:, 189, 0] = 9.0, 8.0, 8.5
    k, v, q = k.to(act).float(), v.to(act).float(), q.to(act).float()
    page_ids = [7, 2, 9, 0, 5]
    keys, values = paged(k, v, page_ids, 11, act)
    table = ints([page_ids])
    tok_seq = torch.zeros(len(pos), dtype=torch.int32, device=DEV)
    out = torch.empty(len(pos), nh * d, dtype=act, device=DEV)
    scale = 1 / math.sqrt(d)
    K.attention(q.to(act).to(DEV), keys, values, tok_seq, pos.to(torch.int32).to(DEV), table, window, scale, out)
    want = attention_reference(q, k, v, pos, window, scale)
    torch.testing.assert_close(out.float().cpu(), want, **TOL[dtype])
    # the designed query really tells the cases apart
    other = attention_reference(q, k, v, pos, 0 if window else 70, scale)
    assert (other[59] - want[59]).abs().max() > 0.1


def test_attention_generic_two_sequences_share_nothing():
    nh, nkv, d = 4, 2, 32
    ka, va = rand(nkv, 100, d, seed=15).cpu(), rand(nkv, 100, d, seed=16).cpu()
    kb, vb = rand(nkv, 70, d, seed=17).cpu(), rand(nkv, 70, d, seed=18).cpu()
    keys, values = make_cache(6, nkv, d, torch.float32)
    for (k, v, ids) in ((ka, va, [4, 1]), (kb, vb, [0, 3])):
        kk, vv = paged(k, v, ids, 6, torch.float32)
        for p in ids:
            keys[p], values[p] = kk[p], vv[p]
    table = ints([[4, 1], [0, 3]])
    q = rand(3, nh, d, seed=19)
    out = torch.empty(3, nh * d, device=DEV)
    K.attention(q, keys, values, ints([0, 1, 1]), ints([99, 69, 5]), table, 0, 0.2, out)
    qa = q.cpu()
    want = torch.cat([attention_reference(qa[:1], ka, va, torch.tensor([99]), 0, 0.2),
                      attention_reference(qa[1:], kb, vb, torch.tensor([69, 5]), 0, 0.2)])
    torch.testing.assert_close(out.cpu(), want, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("inter", [250, 18944, 8])
def test_swiglu(dtype, inter):
    act = DT[dtype]
    gu = rand(9, 2 * inter, seed=20, scale=3.0, dtype=act)
    out = torch.empty(9, inter, dtype=act, device=DEV)
    K.swiglu(gu, out)
    want = F.silu(gu.float()[:, :inter]) * gu.float()[:, inter:]
    torch.testing.assert_close(out.float(), want, atol=TOL[dtype]["atol"], rtol=TOL[dtype]["rtol"] * 2)


def test_argmax_and_ties():
    logits = rand(6, 5003, seed=21)
    logits[1, 77] = logits[1, 4000] = 50.0          # a tie: the lower id wins
    logits[2, 5002] = 60.0                          # the last element
    logits[3] = -float("inf")
    logits[3, 9] = -1e30
    logits[4] = 1.0                                  # all equal
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    K.argmax(logits, out)
    want = [plain.greedy(r) for r in logits.cpu()]
    assert out.tolist() == want and want[1] == 77 and want[2] == 5002 and want[3] == 9 and want[4] == 0


def test_repeat_penalty():
    logits = rand(3, 1001, seed=22)
    base = logits.clone().cpu()
    histories = [[5, 9, 5, 1000, 5], [], [7, 7, 7, 7, 7, 7, 7, 7]]
    hist = torch.zeros(3, 8, dtype=torch.int32, device=DEV)
    times, hist_len = torch.zeros_like(hist), ints([0, 0, 0])
    for step in range(8):                            # the histories grow token by token, as in generation
        reqs = [r for r in range(3) if step < len(histories[r])]
        K.append_history(ints([histories[r][step] for r in reqs]), ints(reqs), hist, times, hist_len)
    assert hist_len.tolist() == [5, 0, 8] and hist[0, :5].tolist() == histories[0]
    assert times[0, :5].tolist() == [0, 1, 0, 1, 3] and times[2].tolist() == [0] * 7 + [8]
    K.repeat_penalty(logits, ints([0, 1, 2]), hist, times, hist_len, 1.3)
    for r in range(3):
        want = plain.apply_repeat_penalty(base[r], histories[r], 1.3)
        torch.testing.assert_close(logits[r].cpu(), want, atol=0, rtol=1e-6)
    # rows may point at any request
    logits2 = base.clone().to(DEV)
    K.repeat_penalty(logits2, ints([2, 2, 0]), hist, times, hist_len, 2.0)
    torch.testing.assert_close(logits2[1].cpu(), plain.apply_repeat_penalty(base[1], [7] * 8, 2.0), atol=0, rtol=1e-6)
    K.append_history(ints([11, 12, 13]), ints([0, 1, 2]), hist, times, hist_len)
    assert hist_len.tolist() == [6, 1, 8] and hist[0, 5].item() == 11 and hist[1, 0].item() == 12   # request 2 is full
    # a long history with many repeats: one pass each
    n = 3000
    long_hist = torch.randint(0, 50, (n,)).tolist()
    h2, t2, l2 = torch.zeros(1, n, dtype=torch.int32, device=DEV), torch.zeros(1, n, dtype=torch.int32, device=DEV), ints([0])
    for tok in long_hist:
        K.append_history(ints([tok]), ints([0]), h2, t2, l2)
    z = rand(1, 1001, seed=25)
    want = plain.apply_repeat_penalty(z[0].cpu(), long_hist, 1.01)
    K.repeat_penalty(z, ints([0]), h2, t2, l2, 1.01)
    torch.testing.assert_close(z[0].cpu(), want, atol=0, rtol=1e-5)


def draw(logits, temperature, top_k, top_p, us):
    rows = logits.repeat(len(us), 1).contiguous()
    out = torch.empty(len(us), dtype=torch.int32, device=DEV)
    K.sample(rows, temperature, top_k, top_p, torch.tensor(us, dtype=torch.float32, device=DEV), out)
    return out.tolist()


def test_sample_inverse_cdf_and_cuts():
    probs = torch.tensor([0.1, 0.4, 0.2, 0.3])
    logits = torch.log(probs)[None].to(DEV)
    us = [0.0, 0.09, 0.11, 0.49, 0.51, 0.69, 0.71, 0.999]
    assert draw(logits, 1.0, 0, 1.0, us) == [0, 0, 1, 1, 2, 2, 3, 3]
    # top-k 2 keeps ids 1 and 3 (0.4, 0.3): the cut between them is at 4/7
    assert draw(logits, 1.0, 2, 1.0, [0.0, 0.56, 0.58, 0.99]) == [1, 1, 3, 3]
    # top-p 0.69 keeps 0.4 + 0.3; 0.71 needs the 0.2 as well
    assert draw(logits, 1.0, 0, 0.69, [0.0, 0.56, 0.58, 0.99]) == [1, 1, 3, 3]
    assert draw(logits, 1.0, 0, 0.71, [0.0, 0.43, 0.46, 0.66, 0.68, 0.99]) == [1, 1, 2, 2, 3, 3]
    # top-k 3 then top-p 0.5 of the kept 0.9: 0.4 < 0.45 <= 0.7
    assert draw(logits, 1.0, 3, 0.5, [0.0, 0.56, 0.58, 0.99]) == [1, 1, 3, 3]
    # temperature: the weights become p^(1/T)
    w = probs ** 2
    cut = (w[0] / w.sum()).item()
    assert draw(logits, 0.5, 0, 1.0, [cut - 0.01, cut + 0.01]) == [0, 1]
    # equal logits: top-k keeps the lower ids
    flat = torch.zeros(1, 7, device=DEV)
    assert draw(flat, 1.0, 3, 1.0, [0.0, 0.32, 0.34, 0.65, 0.67, 0.99]) == [0, 0, 1, 1, 2, 2]


@pytest.mark.parametrize("vocab,top_k,top_p,temperature", [(5003, 0, 1.0, 0.8), (5003, 40, 0.9, 0.7), (1000, 0, 0.5, 1.3),
                                                           (151936, 40, 0.9, 0.7), (151936, 0, 0.95, 1.0), (300, 1000, 1.0, 1.0),
                                                           (151936, 256, 0.8, 1.0), (151936, 300, 0.8, 1.0), (20000, 200, 1.0, 1.2),
                                                           (4865, 1, 0.5, 1.0), (9000, 40, 0.3, 0.7)])
def test_sample_agrees_with_the_plain_rule(vocab, top_k, top_p, temperature):
    logits = rand(1, vocab, seed=23, scale=3.0)
    us = [0.001, 0.13, 0.37, 0.5, 0.77, 0.93, 0.9999]
    got = draw(logits, temperature, top_k, top_p, us)
    want = [plain.sample_token(logits[0].cpu(), [], temperature, top_k, top_p, 1.0, u) for u in us]
    assert got == want


def test_sample_top_k_over_chunks_of_the_row():
    # top-k first reduces every chunk of a few thousand logits to its own k best: equal logits all
    # over the row (the k lowest ids are kept), the best ones in far-apart chunks, NaN in between
    flat = torch.zeros(1, 12000, device=DEV)
    assert draw(flat, 1.0, 50, 1.0, [0.0, 0.011, 0.5, 0.985, 0.999]) == [0, 0, 25, 49, 49]
    z = rand(1, 30000, seed=24, scale=1.0)
    z[0, ::7] = float("nan")
    best = [29999, 5, 14001, 9000]
    for rank, i in enumerate(best):
        z[0, i] = 20.0 - rank
    # in order of id the weights are e^-1, e^-3, e^-2, e^0 of the total 1.5530: cuts at 0.2369, 0.2690, 0.3561
    assert draw(z, 1.0, 4, 1.0, [0.0, 0.23, 0.24, 0.265, 0.275, 0.35, 0.36, 0.999]) == [5, 5, 9000, 9000, 14001, 14001, 29999, 29999]
    assert draw(z, 1.0, 2, 1.0, [0.0, 0.26, 0.27, 0.99]) == [5, 5, 29999, 29999]       # e^-1 / (1 + e^-1) = 0.2689 first, by id
    assert draw(z, 1.0, 4, 0.7, [0.0, 0.26, 0.27, 0.99]) == [5, 5, 29999, 29999]       # from the largest down 0.6439 < 0.7 <= 0.8808: two kept
    assert draw(torch.full((1, 6000), float("nan"), device=DEV), 1.0, 10, 1.0, [0.5]) == [0]


@pytest.mark.parametrize("vocab", [151936, 5003])
def test_sample_top_p_alone_peaked_and_flat_rows_together(vocab):
    # without top-k a row is first tried on its few hundred best tokens; a flat row, whose top-p set
    # is larger than that, is left to the kernel that reads the whole row.  Both kinds in one call.
    rows = torch.stack([rand(vocab, seed=26, scale=9.0), rand(vocab, seed=27, scale=0.5),
                        torch.zeros(vocab, device=DEV), rand(vocab, seed=28, scale=4.0)])
    rows[3, 100:400] = 15.0                              # 300 equal best tokens: the cut falls among ties
    # (the plain rule sorts the row in Python: at the full vocabulary only a few draws)
    us = [0.003, 0.4, 0.77, 0.9999] if vocab < 10000 else [0.4]
    for top_p, temperature in ((0.9, 1.0), (0.5, 0.7), (0.999, 1.0)):
        out = torch.empty(4, dtype=torch.int32, device=DEV)
        for u in us:
            K.sample(rows.clone(), temperature, 0, top_p, torch.full((4,), u, device=DEV), out)
            want = [plain.sample_token(rows[r].cpu(), [], temperature, 0, top_p, 1.0, u) for r in range(4)]
            assert out.tolist() == want, (top_p, temperature, u)


def test_sample_frequencies_follow_the_softmax():
    logits = torch.tensor([[0.0, 1.0, -1.0, 2.0, 0.5]], device=DEV)
    n = 4000
    us = ((torch.arange(n) + 0.5) / n).tolist()
    got = torch.bincount(torch.tensor(draw(logits, 1.0, 0, 1.0, us)), minlength=5).float() / n
    torch.testing.assert_close(got, torch.softmax(logits[0].cpu(), 0), atol=1e-3, rtol=0)


FORMS = ["rows", "packed"]


def in_form(w, form, parts=1):
    """The weight as the checkpoint has it, or packed for the few-row kernels."""
    return K.pack_weight(w, parts) if form == "packed" else w


def test_packed_weight_layout():
    n, k = 40, 96                                   # 3 tiles, the last half empty
    w = rand(n, k, seed=29, dtype=torch.bfloat16)
    packed = K.pack_weight(w)
    assert tuple(packed.data.shape) == (3, 3, 64, 8) and packed.shape == (n, k) and packed.data.is_contiguous()
    for row, col in [(0, 0), (17, 40), (39, 95), (16, 31), (5, 64)]:
        lane = 16 * ((col % 32) // 8) + row % 16
        assert packed.data[row // 16, col // 32, lane, col % 8] == w[row, col]
    assert not packed.data[2, :, 8:16].any() and not packed.data[2, :, 24:32].any()       # rows 40..47 are zeros
    two = K.pack_weight(torch.cat([w, -w]), parts=2)                   # each part padded by itself
    assert tuple(two.data.shape) == (6, 3, 64, 8) and torch.equal(two.data[3:], -packed.data)
    with pytest.raises(K.KernelError, match="multiple of 32"):
        K.pack_weight(rand(16, 48, dtype=torch.bfloat16))
    with pytest.raises(K.KernelError, match="packed weight is"):
        K.fused_store(rand(2, k, dtype=torch.bfloat16), packed, torch.empty(2, n + 1, device=DEV))


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("m", [1, 3, 8, 16])
@pytest.mark.parametrize("n,k", [(100, 96), (3584, 3584), (1000, 18944), (4608, 1536), (48, 32), (65610, 64)])
def test_product_of_few_rows(m, n, k, form):
    x, w = rand(m, k, seed=30, dtype=torch.bfloat16), rand(n, k, seed=31, scale=0.05, dtype=torch.bfloat16)
    want = x.double() @ w.double().t()
    w = in_form(w, form)
    out = torch.full((m, n), float("nan"), device=DEV)
    K.fused_store(x, w, out)
    torch.testing.assert_close(out.double(), want, atol=2e-3, rtol=1e-3)
    out16 = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    K.fused_store(x, w, out16)
    assert torch.equal(out16, out.to(torch.bfloat16))
    # a row's result does not depend on the other rows: one order of summation whatever the batch
    if m > 1:
        one = torch.empty(1, n, device=DEV)
        K.fused_store(x[m - 1:].contiguous(), w, one)
        assert torch.equal(one[0], out[m - 1])


@pytest.mark.parametrize("m", [17, 32, 33, 64, 65, 100, 128])
@pytest.mark.parametrize("n,k", [(100, 96), (3584, 3584), (1000, 18944), (4608, 1536), (48, 32), (65610, 64), (152064, 128), (264, 1056)])
def test_product_of_17_to_128_rows(m, n, k):
    x, w = rand(m, k, seed=32, dtype=torch.bfloat16), rand(n, k, seed=33, scale=0.05, dtype=torch.bfloat16)
    want = x.double() @ w.double().t()
    packed = K.pack_weight(w)
    out = torch.full((m, n), float("nan"), device=DEV)
    K.mid_store(x, packed, out)
    torch.testing.assert_close(out.double(), want, atol=2e-3, rtol=1e-3)
    out16 = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    K.mid_store(x, packed, out16)
    assert torch.equal(out16, out.to(torch.bfloat16))
    # a row's result does not depend on the batch it is in: other rows, another number of rows
    few = torch.empty(20, n, device=DEV)
    K.mid_store(x[m - 20:].contiguous() if m >= 20 else torch.cat([x, x[:20 - m]]), packed, few)
    assert torch.equal(few[-1] if m >= 20 else few[m - 1], out[m - 1])
    with pytest.raises(K.KernelError, match="packed"):
        K.mid_store(x, w, out)


@pytest.mark.parametrize("m", [17, 40, 64, 65, 90, 128])
@pytest.mark.parametrize("inter,k", [(112, 64), (18944, 3584), (100, 96), (200, 1312), (18, 1312), (50, 2048), (7, 96)])
def test_gated_product_of_17_to_128_rows(m, inter, k):
    x = rand(m, k, seed=34, scale=1.5, dtype=torch.bfloat16)
    w = rand(2 * inter, k, seed=35, scale=0.4 / math.sqrt(k), dtype=torch.bfloat16)       # gate and up of size about 1
    out = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=DEV)
    K.mid_gated(x, K.pack_weight(w, parts=2), out)
    gu = (x.double() @ w.double().t()).float().to(torch.bfloat16).float()
    torch.testing.assert_close(out.float(), F.silu(gu[:, :inter]) * gu[:, inter:], atol=3e-2, rtol=3e-2)
    # the same as the product, rounded, through the gate kernel
    both = torch.empty(m, 2 * inter, dtype=torch.bfloat16, device=DEV)
    K.mid_store(x, K.pack_weight(w), both)
    act = torch.empty_like(out)
    K.swiglu(both, act)
    torch.testing.assert_close(out.float(), act.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("m,n,k", [(40, 96, 2048), (64, 3584, 3584), (17, 100, 1056), (33, 2050, 1024), (64, 3584, 18944), (128, 3584, 18944),
                                   (77, 100, 1056)])
def test_unfinished_sums_of_a_product_are_finished_by_the_next_norm(m, n, k):
    x, w = rand(m, k, seed=36, dtype=torch.bfloat16), rand(n, k, seed=37, scale=0.05, dtype=torch.bfloat16)
    packed = K.pack_weight(w)
    nw = (1 + rand(n, seed=38, scale=0.1)).to(torch.bfloat16)
    h = rand(m, n, seed=39, scale=2.0)
    done = K.mid_store(x, packed, torch.empty(m, n, dtype=torch.bfloat16, device=DEV))
    left = K.mid_store(x, packed, torch.empty(m, n, dtype=torch.bfloat16, device=DEV), finish=False)
    assert isinstance(left, K.PartialSums) and left.sums.shape[0] > 1 and left.shape == (m, n)     # these shapes are cut
    h1, h2 = h.clone(), h.clone()
    out1 = K.add_rmsnorm(h1, done, nw, 1e-6, torch.empty(m, n, dtype=torch.bfloat16, device=DEV), write_back=True)
    out2 = K.add_rmsnorm(h2, left, nw, 1e-6, torch.empty(m, n, dtype=torch.bfloat16, device=DEV), write_back=True)
    assert torch.equal(h1, h2)                       # the same sums, rounded the same way, added the same way
    torch.testing.assert_close(h1, h + done.float(), atol=0, rtol=0)
    # the norm's own sum of squares runs over more threads when it also adds up pieces: one bfloat16 step at most
    torch.testing.assert_close(out1.float(), out2.float(), atol=1e-3, rtol=2 ** -7)
    # some rows only, h left as it is; and without a stream
    rows = ints([m - 1, 0, 5])
    g1 = K.add_rmsnorm(h, done, nw, 1e-6, torch.empty(3, n, dtype=torch.bfloat16, device=DEV), rows=rows)
    g2 = K.add_rmsnorm(h, left, nw, 1e-6, torch.empty(3, n, dtype=torch.bfloat16, device=DEV), rows=rows)
    torch.testing.assert_close(g1.float(), g2.float(), atol=1e-3, rtol=2 ** -7)
    n1 = K.add_rmsnorm(None, done, nw, 1e-6, torch.empty(m, n, dtype=torch.bfloat16, device=DEV))
    n2 = K.add_rmsnorm(None, left, nw, 1e-6, torch.empty(m, n, dtype=torch.bfloat16, device=DEV))
    torch.testing.assert_close(n1.float(), n2.float(), atol=1e-3, rtol=2 ** -7)


@pytest.mark.parametrize("nh,nkv,d,k", [(28, 4, 128, 3584), (3, 1, 32, 2048), (6, 2, 64, 1056)])
def test_unfinished_sums_of_q_k_v_are_finished_by_the_rotation_kernel(nh, nkv, d, k):
    m, n_pages = 20, 24
    total = (nh + 2 * nkv) * d
    x = rand(m, k, seed=40, dtype=torch.bfloat16)
    packed = K.pack_weight(rand(total, k, seed=41, scale=1.0 / math.sqrt(k), dtype=torch.bfloat16))
    bias = rand(total, seed=42, scale=0.3, dtype=torch.bfloat16)
    c, s = plain.rope_tables(d, 1e4, 400)
    cos, sin = c.to(DEV), s.to(DEV)
    pos = ints([(37 * i) % 400 for i in range(m)])
    seq = ints(list(range(m)))
    table = ints([[(i + j) % n_pages for j in range(7)] for i in range(m)])
    assert K.rope_store_takes_sums(torch.bfloat16, bias, d, K.STYLE_HALVES, d)
    assert not K.rope_store_takes_sums(torch.bfloat16, bias, d // 2, K.STYLE_HALVES, d)
    done = K.mid_store(x, packed, torch.empty(m, total, dtype=torch.bfloat16, device=DEV))
    left = K.mid_store(x, packed, torch.empty(m, total, dtype=torch.bfloat16, device=DEV), finish=False)
    assert isinstance(left, K.PartialSums)
    res = []
    for qkv in (done, left):
        keys, values = make_cache(n_pages, nkv, d, torch.bfloat16)
        q = torch.empty(m, nh, d, dtype=torch.bfloat16, device=DEV)
        K.rope_store(qkv, bias, cos, sin, d, K.STYLE_HALVES, seq, pos, table, keys, values, q, nh, nkv, d)
        res.append((q, keys, values))
    for a, b in zip(res[0], res[1]):
        assert torch.equal(torch.isnan(a.float()), torch.isnan(b.float()))
        assert torch.equal(torch.nan_to_num(a.float()), torch.nan_to_num(b.float()))
    with pytest.raises(K.KernelError, match="only bfloat16"):
        K.rope_store(left, bias, cos[:, :d // 4].contiguous(), sin[:, :d // 4].contiguous(), d // 2, K.STYLE_HALVES, seq, pos, table,
                     keys, values, q, nh, nkv, d)


def test_products_of_17_to_128_rows_refuse_what_they_do_not_take():
    w = K.pack_weight(rand(16, 64, dtype=torch.bfloat16))
    with pytest.raises(K.KernelError, match="at most 128"):
        K.mid_store(rand(129, 64, dtype=torch.bfloat16), w, torch.empty(129, 16, device=DEV))
    with pytest.raises(K.KernelError, match="packed weight is"):
        K.mid_gated(rand(20, 64, dtype=torch.bfloat16), w, torch.empty(20, 8, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("nh,nkv,d", [(28, 4, 128), (6, 2, 64), (5, 5, 32), (3, 1, 96), (40, 2, 64), (4, 1, 256)])
@pytest.mark.parametrize("window", [0, 70])
@pytest.mark.parametrize("target_blocks", [1, 24, 100000, "a partition a page"])
def test_attention_decode(nh, nkv, d, window, target_blocks):
    # three sequences of lengths 300, 64 and 1, pages scrambled, everything unread is NaN
    lens = [300, 64, 1]
    n_pages = 12
    keys, values = make_cache(n_pages, nkv, d, torch.bfloat16)
    tables = [[7, 2, 9, 0, 5], [4, -1, -1, -1, -1], [11, -1, -1, -1, -1]]
    ks, vs = [], []
    for i, n in enumerate(lens):
        k, v = rand(nkv, n, d, seed=40 + i).cpu(), rand(nkv, n, d, seed=50 + i).cpu()
        if n == 300:
            k[:, :, 0] *= 0.01
            k[:, 3, 0], k[:, 230, 0], k[:, 229, 0] = 9.0, 8.0, 8.5     # far key, window edge (299-69), just outside
        k, v = k.to(torch.bfloat16).float(), v.to(torch.bfloat16).float()
        kk, vv = paged(k, v, tables[i], n_pages, torch.bfloat16)
        for p in tables[i]:
            if p >= 0:
                keys[p], values[p] = kk[p], vv[p]
        ks.append(k), vs.append(v)
    q = rand(3, nh, d, seed=60).cpu()
    q[0] = 0.0
    q[0, :, 0] = 30.0
    q = q.to(torch.bfloat16)
    pos = torch.tensor([n - 1 for n in lens])
    out = torch.empty(3, nh * d, dtype=torch.bfloat16, device=DEV)
    scale = 1 / math.sqrt(d)
    if isinstance(target_blocks, str):         # as many partitions as the table is wide: blocks of one wave, one page each
        K.attention_decode(q.to(DEV), keys, values, pos.to(torch.int32).to(DEV), ints(tables), window, scale, out, n_parts=len(tables[0]))
    else:
        K.attention_decode(q.to(DEV), keys, values, pos.to(torch.int32).to(DEV), ints(tables), window, scale, out,
                           target_blocks=target_blocks)
    for i in range(3):
        want = attention_reference(q[i:i + 1].float(), ks[i], vs[i], pos[i:i + 1], window, scale)
        torch.testing.assert_close(out[i:i + 1].float().cpu(), want, atol=2e-2, rtol=2e-2)
    other = attention_reference(q[:1].float(), ks[0], vs[0], pos[:1], 0 if window else 70, scale)
    assert (other - out[:1].float().cpu()).abs().max() > 0.1
    # the plain kernel agrees
    out2 = torch.empty_like(out)
    K.attention(q.to(DEV), keys, values, ints([0, 1, 2]), pos.to(torch.int32).to(DEV), ints(tables), window, scale, out2)
    torch.testing.assert_close(out.float(), out2.float(), atol=2e-2, rtol=2e-2)


def test_attention_decode_refuses_other_head_sizes():
    assert not K.attention_decode_supported(48) and K.attention_decode_supported(128)
    keys, values = make_cache(2, 1, 48, torch.bfloat16)
    with pytest.raises(K.KernelError, match="head_dim 48"):
        K.attention_decode(rand(1, 1, 48, dtype=torch.bfloat16), keys, values, ints([0]), ints([[0]]), 0, 1.0,
                           torch.empty(1, 48, dtype=torch.bfloat16, device=DEV))


# (short sequences: one set of waves a block; head size 32 in blocks of more than four waves with 10 heads on 2)
@pytest.mark.parametrize("nh,nkv,d", [(28, 4, 128), (6, 2, 64), (5, 5, 32), (10, 2, 32), (3, 1, 96), (40, 2, 64), (12, 2, 128)])
@pytest.mark.parametrize("window", [0, 70, 12])
@pytest.mark.parametrize("tile", [16, 32, 64, 128])
def test_attention_prefill(nh, nkv, d, window, tile):
    # sequence 0: 150 new queries at positions 150..299 behind 150 cached ones; sequence 1: a
    # whole prompt of 70; sequence 2: one token at position 0.  Pages scrambled, unread places NaN.
    spans = [(150, 300), (0, 70), (0, 1)]
    n_pages = 12
    keys, values = make_cache(n_pages, nkv, d, torch.bfloat16)
    tables = [[7, 2, 9, 0, 5], [4, 10, -1, -1, -1], [11, -1, -1, -1, -1]]
    ks, vs, qs = [], [], []
    for i, (a, b) in enumerate(spans):
        k, v = rand(nkv, b, d, seed=70 + i).cpu(), rand(nkv, b, d, seed=80 + i).cpu()
        qq = rand(b - a, nh, d, seed=90 + i).cpu()
        if i == 0:
            k[:, :, 0] *= 0.01
            k[:, 3, 0], k[:, 230, 0], k[:, 229, 0] = 9.0, 8.0, 8.5     # far key; edge of the window of 70 for 299; outside
            qq[-1] = 0.0
            qq[-1, :, 0] = 30.0
        k, v = k.to(torch.bfloat16).float(), v.to(torch.bfloat16).float()
        kk, vv = paged(k, v, tables[i], n_pages, torch.bfloat16)
        for p in tables[i]:
            if p >= 0:
                keys[p], values[p] = kk[p], vv[p]
        ks.append(k), vs.append(v), qs.append(qq.to(torch.bfloat16))
    q = torch.cat(qs).to(DEV)
    pos = torch.cat([torch.arange(a, b) for a, b in spans])
    tile_seq, tile_tok0, tile_count, off = [], [], [], 0
    for i, (a, b) in enumerate(spans):
        for s0 in range(0, b - a, tile):
            tile_seq.append(i), tile_tok0.append(off + s0), tile_count.append(min(tile, b - a - s0))
        off += b - a
    out = torch.empty(q.shape[0], nh * d, dtype=torch.bfloat16, device=DEV)
    scale = 1 / math.sqrt(d)
    K.attention_prefill(q, keys, values, pos.to(torch.int32).to(DEV), ints(tables), ints(tile_seq), ints(tile_tok0),
                        ints(tile_count), ints([a for a, _ in spans]), ints([b - a for a, b in spans]), window, scale, out,
                        tile_queries=tile)
    off = 0
    for i, (a, b) in enumerate(spans):
        want = attention_reference(qs[i].float(), ks[i], vs[i], torch.arange(a, b), window, scale)
        torch.testing.assert_close(out[off:off + b - a].float().cpu(), want, atol=2e-2, rtol=2e-2)
        off += b - a
    if window != 70:
        other = attention_reference(qs[0][-1:].float(), ks[0], vs[0], torch.tensor([299]), 70, scale)
        assert (other - out[149:150].float().cpu()).abs().max() > 0.1


# ---- skinny products with norm, residual sum, gate and rotation folded in ----------------------
def bf(x):
    return x.to(torch.bfloat16).float()


def prepared(h, nw):
    """What a kernel that adds to the stream leaves for the next norm: the stream times the
    norm's weight in bfloat16, and the rows' sums of squares in pieces of 16 columns."""
    m, k = h.shape
    xw = (h * nw.float()).to(torch.bfloat16)
    parts = (k + 15) // 16
    ss = torch.zeros(parts, 16, device=DEV)
    pad = torch.zeros(m, parts * 16, device=DEV)
    pad[:, :k] = h * h
    ss[:, :m] = pad.reshape(m, parts, 16).sum(-1).t()
    return xw, (ss, parts)


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("n,k", [(100, 96), (3584, 3584), (1000, 1536), (65610, 64)])       # the last: blocks of two tiles
def test_fused_store_with_and_without_norm(m, n, k, form):
    h = rand(16, k, seed=100, scale=2.0)
    w = rand(n, k, seed=101, scale=1.0 / math.sqrt(k), dtype=torch.bfloat16)
    w, w_rows = in_form(w, form), w
    nw = (1 + rand(k, seed=102, scale=0.1)).to(torch.bfloat16)
    rows = ints(list(range(15, 15 - m, -1)))                     # m rows of x, backwards
    out = torch.full((m, n), float("nan"), device=DEV)
    xb = h.to(torch.bfloat16)
    K.fused_store(xb, w, out, rows=rows)
    torch.testing.assert_close(out.double(), xb.double()[rows.long()] @ w_rows.double().t(), atol=2e-3, rtol=1e-3)
    eps = 1e-5
    xw, (ss, parts) = prepared(h, nw)
    K.fused_store(xw, w, out, (ss, parts, eps), rows=rows)
    want = plain.rms_norm(h[rows.long()], nw.float(), eps).double() @ w_rows.double().t()
    torch.testing.assert_close(out.double(), want, atol=2e-2, rtol=2e-2)
    if form == "packed":            # the same sums in the same order as from the rows
        same = torch.empty_like(out)
        K.fused_store(xw, w_rows, same, (ss, parts, eps), rows=rows)
        assert torch.equal(out, same)


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("m", [1, 8, 16])
@pytest.mark.parametrize("inter,k", [(112, 64), (18944, 3584), (100, 96)])
def test_fused_gated(m, inter, k, form):
    h = rand(m, k, seed=103, scale=1.5)
    w_rows = rand(2 * inter, k, seed=104, scale=0.4 / math.sqrt(k), dtype=torch.bfloat16)      # gate and up of size about 1
    w = in_form(w_rows, form, parts=2)
    nw = (1 + rand(k, seed=105, scale=0.1)).to(torch.bfloat16)
    out = torch.empty(m, inter, dtype=torch.bfloat16, device=DEV)
    xw, (ss, parts) = prepared(h, nw)
    K.fused_gated(xw, w, out, (ss, parts, 1e-6))
    gu = bf(plain.rms_norm(h, nw.float(), 1e-6).double() @ w_rows.double().t())
    torch.testing.assert_close(out.float(), F.silu(gu[:, :inter]) * gu[:, inter:], atol=3e-2, rtol=3e-2)
    xb = h.to(torch.bfloat16)
    K.fused_gated(xb, w, out)
    gu = bf(xb.double() @ w_rows.double().t())
    torch.testing.assert_close(out.float(), F.silu(gu[:, :inter]) * gu[:, inter:], atol=3e-2, rtol=3e-2)
    if form == "packed":
        same = torch.empty_like(out)
        K.fused_gated(xb, w_rows, same)
        assert torch.equal(out, same)


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("m", [1, 7, 16])
@pytest.mark.parametrize("n,k", [(96, 64), (3584, 18944), (100, 32)])
def test_fused_residual_prepares_the_next_norm(m, n, k, form):
    x = rand(m, k, seed=106, dtype=torch.bfloat16)
    w_rows = rand(n, k, seed=107, scale=0.02, dtype=torch.bfloat16)
    w = in_form(w_rows, form)
    nw = (1 + rand(n, seed=113, scale=0.1)).to(torch.bfloat16)
    h = rand(m, n, seed=108, scale=3.0)
    want = h + bf((x.double() @ w_rows.double().t()).float())
    xw = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ss = torch.full((K.fused_residual_parts(n, k), 16), float("nan"), device=DEV)
    parts = K.fused_residual(x, w, h, xw, nw, ss)
    torch.testing.assert_close(h, want, atol=4e-2, rtol=0)          # one bfloat16 step of the product at most
    assert torch.equal(xw, (h * nw.float()).to(torch.bfloat16))
    assert parts == K.fused_residual_parts(n, k) <= (n + 15) // 16
    torch.testing.assert_close(ss[:, :m].sum(0), (h * h).sum(-1), rtol=1e-5, atol=1e-5)
    # and what the next product makes of it is the norm of the new stream
    w2 = rand(48, n, seed=114, scale=1.0 / math.sqrt(n), dtype=torch.bfloat16)
    if n % 32 == 0:
        out = torch.empty(m, 48, device=DEV)
        K.fused_store(xw, w2, out, (ss, parts, 1e-6))
        torch.testing.assert_close(out.double(), plain.rms_norm(h, nw.float(), 1e-6).double() @ w2.double().t(), atol=2e-2, rtol=2e-2)
    # without a next norm: the plain copy, no sums
    h2 = h.clone()
    K.fused_residual(x, w, h2, xw)
    assert torch.equal(xw, h2.to(torch.bfloat16))


@pytest.mark.parametrize("hidden", [96, 100, 3584, 8200])
def test_embed_prepares_the_first_norm(hidden):
    table = rand(301, hidden, seed=115, dtype=torch.bfloat16)
    nw = (1 + rand(hidden, seed=116, scale=0.1)).to(torch.bfloat16)
    ids = ints([5, 300, 0])
    h, xw, ss = torch.empty(3, hidden, device=DEV), torch.empty(3, hidden, dtype=torch.bfloat16, device=DEV), torch.zeros(1, 16, device=DEV)
    K.embed(table, ids, h, copy=xw, copy_weight=nw, ss_out=ss)
    assert torch.equal(h, table.float()[ids.long()]) and torch.equal(xw, (h * nw.float()).to(torch.bfloat16))
    torch.testing.assert_close(ss[0, :3], (h * h).sum(-1), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("nh,nkv,d,k", [(28, 4, 128, 3584), (3, 1, 32, 96), (6, 2, 64, 160)])
def test_fused_qkv_equals_product_then_rotation_kernel(nh, nkv, d, k, form):
    m, n_pages = 5, 9
    total = (nh + 2 * nkv) * d
    h = rand(m, k, seed=109, scale=1.5)
    w = in_form(rand(total, k, seed=110, scale=1.0 / math.sqrt(k), dtype=torch.bfloat16), form)
    bias = rand(total, seed=111, scale=0.3, dtype=torch.bfloat16)
    nw = (1 + rand(k, seed=112, scale=0.1)).to(torch.bfloat16)
    c, s = plain.rope_tables(d, 1e4, 400)
    cos, sin = c.to(DEV), s.to(DEV)
    pos = ints([0, 63, 64, 200, 399])
    table = ints([[3, -1, -1, -1, -1, -1, -1], [8, -1, -1, -1, -1, -1, -1], [0, 5, -1, -1, -1, -1, -1],
                  [1, 1, 1, 2, -1, -1, -1], [4, 4, 4, 4, 4, 4, 7]])
    keys, values = make_cache(n_pages, nkv, d, torch.bfloat16)
    q = torch.empty(m, nh, d, dtype=torch.bfloat16, device=DEV)
    xw, (ss, parts) = prepared(h, nw)
    K.fused_qkv(xw, w, bias, cos, sin, pos, table, keys, values, q, nh, nkv, d, norm=(ss, parts, 1e-6))
    # the same with separate kernels: norm, product, rotation + cache write
    xn = torch.empty(m, k, dtype=torch.bfloat16, device=DEV)
    K.add_rmsnorm(h, None, nw, 1e-6, xn)
    qkv = torch.empty(m, total, dtype=torch.bfloat16, device=DEV)
    K.fused_store(xn, w, qkv)
    keys2, values2 = make_cache(n_pages, nkv, d, torch.bfloat16)
    q2 = torch.empty_like(q)
    K.rope_store(qkv, bias, cos, sin, d, K.STYLE_HALVES, ints([0, 1, 2, 3, 4]), pos, table, keys2, values2, q2, nh, nkv, d)
    torch.testing.assert_close(q.float(), q2.float(), atol=4e-2, rtol=3e-2)
    for a, b in ((keys, keys2), (values, values2)):
        assert torch.equal(torch.isnan(a.float()), torch.isnan(b.float()))          # the same places written
        ok = ~torch.isnan(a.float())
        torch.testing.assert_close(a.float()[ok], b.float()[ok], atol=4e-2, rtol=3e-2)
    # and without norm and bias
    K.fused_qkv(xn, w, None, cos, sin, pos, table, keys, values, q, nh, nkv, d)
    K.rope_store(qkv, None, cos, sin, d, K.STYLE_HALVES, ints([0, 1, 2, 3, 4]), pos, table, keys2, values2, q2, nh, nkv, d)
    torch.testing.assert_close(q.float(), q2.float(), atol=2e-2, rtol=2e-2)
    ok = ~torch.isnan(keys.float())
    torch.testing.assert_close(keys.float()[ok], keys2.float()[ok], atol=2e-2, rtol=2e-2)


def test_fused_kernels_refuse_what_they_do_not_take():
    w = rand(16, 64, dtype=torch.bfloat16)
    with pytest.raises(K.KernelError, match="at most 16"):
        K.fused_store(rand(17, 64, dtype=torch.bfloat16), w, torch.empty(17, 16, device=DEV))
    with pytest.raises(K.KernelError, match="multiple of 32"):
        K.fused_store(rand(2, 48, dtype=torch.bfloat16), rand(16, 48, dtype=torch.bfloat16), torch.empty(2, 16, device=DEV))


# ---- random weights: the same bits on the host and on the GPU ------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_random_normal_on_the_gpu_equals_the_hosts_bit_for_bit(dtype):
    import numpy as np
    from tq_kv_amd.weights import standard_normal_host, tensor_key
    key = tensor_key(11, "some.weight")
    n = 3_000_001
    for std, plus_one in ((0.02, False), (0.02, True), (1.0, False)):
        out = K.random_normal(torch.empty((n,), dtype=dtype, device="cuda"), key, std, plus_one)
        want = standard_normal_host(key, 0, n) * np.float32(std)
        if plus_one:
            want = np.float32(1.0) + want
        want = torch.from_numpy(want).to(dtype)
        got = out.cpu()
        view = torch.int32 if dtype == torch.float32 else torch.int16
        bad = (got.view(view) != want.view(view)).nonzero()
        assert bad.numel() == 0, "first difference at element %d: %r vs %r" % (bad[0], got[bad[0]], want[bad[0]])


def test_a_random_model_on_the_gpu_equals_the_folder_the_host_writes(tmp_path):
    """Model.random on the GPU and write_random_folder on the host: one seed, one model."""
    from safetensors.torch import load_file
    from tq_kv_amd import Model
    from tq_kv_amd.weights import random_tensors
    import helpers
    for name, (cfg, seed) in helpers.CONFIGS.items():
        for store in (torch.bfloat16, torch.float32):
            folder = Model.write_random_folder(str(tmp_path / ("%s_%s" % (name, store))), cfg, seed=seed, store_dtype=store)
            stored = load_file(folder + "/model.safetensors")
            specs = Model.from_config_dict(cfg, "float32", "cpu").tensor_specs()
            made = random_tensors(specs, seed, store, "cuda")
            assert set(made) == set(stored)
            for k in stored:
                assert torch.equal(made[k].cpu(), stored[k]), k


# ---- the attention kernels at the lengths that are benchmarked ------------------------------------
def scrambled_pages(n_pages_needed, n_pages, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randperm(n_pages, generator=g)[:n_pages_needed].tolist()


def long_sequence(nkv, n, d, seed, window, last):
    """Keys and values [nkv, n, d] (bfloat16 values, as float32) of a sequence whose first element
    is nearly silent, with loud keys planted where a mistake shows: in the first page, in the
    middle of the sequence, at the edge of the window of query `last` and just outside it."""
    k, v = rand(nkv, n, d, seed=seed).cpu(), rand(nkv, n, d, seed=seed + 1).cpu()
    k[:, :, 0] *= 0.01
    k[:, 3, 0], k[:, n // 2 + 5, 0] = 9.0, 8.8
    if window and last - window + 1 > 0:
        k[:, last - window + 1, 0], k[:, last - window, 0] = 8.0, 9.5       # the edge, and just outside
    return k.to(torch.bfloat16).float(), v.to(torch.bfloat16).float()


def padded_table(rows, multiple=8):
    width = (max(len(r) for r in rows) + multiple - 1) // multiple * multiple
    return [list(r) + [-1] * (width - len(r)) for r in rows]


@pytest.mark.parametrize("nh,nkv,d", [(28, 4, 128), (6, 2, 64)])
@pytest.mark.parametrize("n_keys", [2300, 8200])
@pytest.mark.parametrize("window", [0, 1000])
def test_attention_decode_over_thousands_of_keys(nh, nkv, d, n_keys, window):
    """One long sequence and one short one: dozens of pages scrambled over the pool, the table
    padded with -1 to a multiple of 8 pages as the graphed steps pad it, pages that have left the
    window given back (-1, their places NaN), eight and more partitions whose waves take several
    pages each."""
    lens = [n_keys, 70]
    n_pages = (n_keys + 63) // 64 + 40
    ids = scrambled_pages((n_keys + 63) // 64 + 2, n_pages, seed=n_keys)
    tables = [ids[:(n_keys + 63) // 64], ids[(n_keys + 63) // 64:]]
    keys, values = make_cache(n_pages, nkv, d, torch.bfloat16)
    ks, vs = [], []
    for i, n in enumerate(lens):
        k, v = long_sequence(nkv, n, d, 300 + 10 * i, window, n - 1)
        kk, vv = paged(k, v, tables[i], n_pages, torch.bfloat16)
        dead = (max(0, n - window) // 64) if window else 0              # pages wholly behind the window
        for j, p in enumerate(tables[i]):
            if j >= dead:
                keys[p], values[p] = kk[p], vv[p]
        tables[i] = [-1] * dead + tables[i][dead:]
        ks.append(k), vs.append(v)
    q = rand(2, nh, d, seed=61).cpu()
    q[0] = 0.0
    q[0, :, 0] = 30.0
    q = q.to(torch.bfloat16)
    pos = torch.tensor([n - 1 for n in lens])
    table = ints(padded_table(tables))
    assert table.shape[1] % 8 == 0 and table.shape[1] >= (n_keys + 63) // 64
    out = torch.empty(2, nh * d, dtype=torch.bfloat16, device=DEV)
    scale = 1 / math.sqrt(d)
    K.attention_decode(q.to(DEV), keys, values, pos.to(torch.int32).to(DEV), table, window, scale, out, target_blocks=256)
    for i in range(2):
        want = attention_reference(q[i:i + 1].float(), ks[i], vs[i], pos[i:i + 1], window, scale)
        torch.testing.assert_close(out[i:i + 1].float().cpu(), want, atol=2e-2, rtol=2e-2)
    # a partition per page of the table (most of them empty behind a window, or beyond the short sequence's end)
    thin = torch.full_like(out, float("nan"))
    K.attention_decode(q.to(DEV), keys, values, pos.to(torch.int32).to(DEV), table, window, scale, thin, n_parts=table.shape[1])
    torch.testing.assert_close(thin.float(), out.float(), atol=2e-2, rtol=2e-2)
    # the planted keys matter: without the window (or with it) the sharp query's answer is another
    other = attention_reference(q[:1].float(), ks[0], vs[0], pos[:1], 0 if window else 1000, scale)
    assert (other - out[:1].float().cpu()).abs().max() > 0.1
    out2 = torch.empty_like(out)
    K.attention(q.to(DEV), keys, values, ints([0, 1]), pos.to(torch.int32).to(DEV), table, window, scale, out2)
    torch.testing.assert_close(out.float(), out2.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("tile", [16, 64])
def test_attention_prefill_with_scores_far_below_zero(tile):
    # Every score of the first keys lies hundreds of powers of two below 0 (q = c, k = -c in every element), so the
    # running maximum starts far below the 0 it stands at before a column's first key, and later keys lie far above
    # (k = +c from position 100 on): what is summed up to then has to vanish without a trace, not turn into 0 * inf.
    nh, nkv, d, n = 4, 2, 128, 200
    c = 4.0
    q = torch.full((n, nh, d), c).to(torch.bfloat16)
    k = torch.full((nkv, n, d), -c)
    k[:, 100:] = c
    k[:, 150] = -c
    v = rand(nkv, n, d, seed=5).cpu().to(torch.bfloat16).float()
    table = [0, 1, 2, 3]
    kk, vv = paged(k, v, table, 4, torch.bfloat16)
    keys, values = kk.to(DEV), vv.to(DEV)
    pos = torch.arange(n)
    tile_tok0 = list(range(0, n, tile))
    out = torch.empty(n, nh * d, dtype=torch.bfloat16, device=DEV)
    scale = 1 / math.sqrt(d)
    K.attention_prefill(q.to(DEV), keys, values, pos.to(torch.int32).to(DEV), ints([table]), ints([0] * len(tile_tok0)), ints(tile_tok0),
                        ints([min(tile, n - t) for t in tile_tok0]), ints([0]), ints([n]), 0, scale, out, tile_queries=tile)
    want = attention_reference(q.float(), k, v, pos, 0, scale)
    assert torch.isfinite(out.float()).all()
    torch.testing.assert_close(out.float().cpu(), want, atol=2e-2, rtol=2e-2)
    # (before position 100 a query's output is the mean of the values it sees, afterwards that of the keys from 100 on)
    torch.testing.assert_close(want[50, :d], v[0, :51].mean(0), atol=1e-3, rtol=1e-3)


@pytest.mark.parametrize("nh,nkv,d,spans,tile", [
    (28, 4, 128, [(0, 2048)], 16),                    # the benchmarked prompt: two heads a wave, all blocks resident
    (28, 4, 128, [(0, 2048)], 64),
    (28, 4, 128, [(0, 4096)], 16),                    # more blocks than two a compute unit: one set of four waves a block
    (28, 4, 128, [(0, 3200)], 32),                    # a head a wave, blocks of seven waves shared out as they finish
    (28, 4, 128, [(0, 3200)], 128),
    (28, 4, 128, [(1100, 2100), (0, 70)], 32),        # a piece of a prompt behind 1100 cached positions
    (6, 2, 64, [(0, 2048), (500, 1300)], 128),
    (40, 2, 64, [(0, 1500), (300, 900)], 32),         # groups of 20 heads: three blocks a group
    (3, 1, 96, [(0, 2500)], 64),
    (5, 5, 32, [(0, 2100)], 128),
    (6, 2, 64, [(0, 1500)], 16),                      # few blocks of four waves of columns and long sequences: two sets of
    (3, 1, 96, [(0, 1200)], 32),                      # waves a block share each page's keys (as the first and the last line)
])
@pytest.mark.parametrize("window", [0, 1000, 20])        # 20: most queries see keys of one half of a page only (one set of waves sees none)
def test_attention_prefill_over_thousands_of_keys(nh, nkv, d, spans, tile, window):
    scale = 1 / math.sqrt(d)
    need = [(b + 63) // 64 for _, b in spans]
    n_pages = sum(need) + 30
    ids = scrambled_pages(sum(need), n_pages, seed=spans[0][1])
    tables, at = [], 0
    for n in need:
        tables.append(ids[at:at + n])
        at += n
    keys, values = make_cache(n_pages, nkv, d, torch.bfloat16)
    ks, vs, qs = [], [], []
    for i, (a, b) in enumerate(spans):
        k, v = long_sequence(nkv, b, d, 400 + 10 * i, window, b - 1)
        qq = rand(b - a, nh, d, seed=420 + i).cpu()
        for row in (b - a - 1, (b - a) // 2):               # sharp queries: the last one and one in the middle
            qq[row] = 0.0
            qq[row, :, 0] = 30.0
        kk, vv = paged(k, v, tables[i], n_pages, torch.bfloat16)
        for p in tables[i]:
            keys[p], values[p] = kk[p], vv[p]
        ks.append(k), vs.append(v), qs.append(qq.to(torch.bfloat16))
    q = torch.cat(qs).to(DEV)
    pos = torch.cat([torch.arange(a, b) for a, b in spans])
    tile_seq, tile_tok0, tile_count, off = [], [], [], 0
    for i, (a, b) in enumerate(spans):
        for s0 in range(0, b - a, tile):
            tile_seq.append(i), tile_tok0.append(off + s0), tile_count.append(min(tile, b - a - s0))
        off += b - a
    order = sorted(range(len(tile_seq)), key=lambda t: -(int(pos[tile_tok0[t]]) + tile_count[t]))      # as the engine orders them
    tile_seq, tile_tok0, tile_count = ([x[t] for t in order] for x in (tile_seq, tile_tok0, tile_count))
    out = torch.full((q.shape[0], nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    K.attention_prefill(q, keys, values, pos.to(torch.int32).to(DEV), ints(padded_table(tables)), ints(tile_seq), ints(tile_tok0),
                        ints(tile_count), ints([a for a, _ in spans]), ints([b - a for a, b in spans]), window, scale, out,
                        tile_queries=tile)
    assert not torch.isnan(out.float()).any()
    off = 0
    for i, (a, b) in enumerate(spans):
        n = b - a
        rows = sorted(set(list(range(0, n, 53)) + [r for r in (0, 1, 62, 63, 64, 65, 127, 128, 129, n // 2, n - 2, n - 1) if r < n]))
        want = attention_reference(qs[i][rows].float(), ks[i], vs[i], torch.tensor(rows) + a, window, scale)
        torch.testing.assert_close(out[off:off + n][rows].float().cpu(), want, atol=2e-2, rtol=2e-2,
                                   msg=lambda m: "sequence %d: %s" % (i, m))
        if i == 0:
            other = attention_reference(qs[0][-1:].float(), ks[0], vs[0], torch.tensor([b - 1]), 0 if window else 1000, scale)
            assert (other - out[off + n - 1:off + n].float().cpu()).abs().max() > 0.1
        off += n


def test_the_probes_read_and_multiply():
    """What the bench sets its figures against: a streaming read and a loop of matrix-core products.  Their figures are
    the GPU's; here only that they run, read every shape of grid they are asked for, and refuse what they cannot do."""
    buf = torch.ones(1 << 24, dtype=torch.float32, device=DEV)            # 64 MB
    assert K.probe_read(buf, repeats=2) > 200.0                              # GB/s: any GPU this runs on does that
    assert K.probe_read(buf[:4 * 1000 + 4], repeats=1, shapes=((3, 64), (7, 128))) > 0.0     # regions that do not divide evenly
    assert K.probe_mfma(turns=2000, repeats=1) > 0.01                       # PFLOP/s
    with pytest.raises(K.KernelError, match="blocks of 96 threads"):
        K.probe_read(buf, repeats=1, shapes=((8, 96),))
