// Softmax attention over the paged cache, one wave per (token, query head), float32
// arithmetic throughout.  It serves the float32 path for prompts and for decoding
// alike, and any head size; the bfloat16 path uses it where the MFMA kernels do
// not apply.
//
// Formulas: scores q.k / sqrt(d), mask, softmax (max-subtract, exp, normalise), p.v
// as src/models/turbo_generic.rs:1620-1631 and :56-62; query head h reads kv head
// h / (heads / kv_heads) (:195-204).  The reference's mask is only right for a
// prompt at position 0 (:1937-1956); here the query at absolute position i sees
// keys lo..i of its own sequence for any split into steps, lo being 0 or, with a
// window of W, max(0, i - W + 1).
//
// Work of one wave: keys are taken in blocks of 64 (one page); lane j computes the
// score of key j of the block, the softmax runs online over blocks, then lane c
// accumulates output element c (+64, +128, ...) over the block's keys.  The order of
// operations for a query depends only on its position, never on the batch.
// Cache pages: keys [kv head][position][head_dim], values [kv head][head_dim][place of
// the position] (value_place in common.h).
#include "common.h"
#include "tq_kernels.h"

#define ATT_WAVES 4
#define ATT_MAX_D 256

template <typename T>
__global__ __launch_bounds__(ATT_WAVES * TQK_WAVE)
void attention_generic_kernel(const T* __restrict__ q, const T* __restrict__ keys, const T* __restrict__ values,
                              const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                              const int32_t* __restrict__ page_table, int table_width, int window, float scale,
                              T* __restrict__ out, int n_tokens, int n_heads, int n_kv_heads, int head_dim) {
    __shared__ float q_lds[ATT_WAVES][ATT_MAX_D];
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int t = blockIdx.x * ATT_WAVES + wave;
    const int head = blockIdx.y;
    const bool live = t < n_tokens;
    if (live) {
        const T* qv = q + ((size_t)t * n_heads + head) * head_dim;
        for (int i = lane; i < head_dim; i += TQK_WAVE) q_lds[wave][i] = to_float(qv[i]);
    }
    __syncthreads();
    if (!live) return;

    const int pos = tok_pos[t];
    const int32_t* pages = page_table + (size_t)tok_seq[t] * table_width;
    const int kvh = head / (n_heads / n_kv_heads);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const size_t page_stride = (size_t)n_kv_heads * TQK_PAGE * head_dim;
    const float* qf = q_lds[wave];

    constexpr int NACC = ATT_MAX_D / TQK_WAVE;
    float acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.f;
    float m = -INFINITY, l = 0.f;

    for (int kb = (lo / TQK_PAGE) * TQK_PAGE; kb <= pos; kb += TQK_PAGE) {
        const int page = pages[kb / TQK_PAGE];
        const int j = kb + lane;
        const bool valid = j >= lo && j <= pos && page >= 0;
        const size_t base = (size_t)(page < 0 ? 0 : page) * page_stride + (size_t)kvh * TQK_PAGE * head_dim;
        float s = -INFINITY;
        if (valid) {
            const T* kr = keys + base + (size_t)lane * head_dim;
            float dot = 0.f;
            for (int i = 0; i < head_dim; ++i) dot = fmaf(qf[i], to_float(kr[i]), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));     // finite: the block holds at least key lo or kb
        const float p = valid ? expf(s - m_new) : 0.f;
        const float alpha = expf(m - m_new);            // exp(-inf) = 0 on the first block
        l = l * alpha + wave_sum(p);
        m = m_new;
        const int n_keys = min(TQK_PAGE, pos - kb + 1);
        const int first_key = max(0, lo - kb);           // keys before the window are never read
        const T* vb = values + base;
#pragma unroll
        for (int a = 0; a < NACC; ++a) {
            const int c = lane + a * TQK_WAVE;
            float sum = acc[a] * alpha;
            if (a * TQK_WAVE < head_dim) {
                for (int jj = first_key; jj < n_keys; ++jj) {
                    const float pj = __shfl(p, jj, TQK_WAVE);
                    if (c < head_dim) sum = fmaf(pj, to_float(vb[(size_t)c * TQK_PAGE + value_place(jj)]), sum);
                }
            }
            acc[a] = sum;
        }
    }
    T* o = out + ((size_t)t * n_heads + head) * head_dim;
#pragma unroll
    for (int a = 0; a < NACC; ++a) {
        const int c = lane + a * TQK_WAVE;
        if (c < head_dim) o[c] = from_float<T>(acc[a] / l);
    }
}

extern "C" int tqk_attention_max_head_dim(void) { return ATT_MAX_D; }

extern "C" int tqk_attention(const void* q, const void* keys, const void* values, int act_dtype,
                             const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* page_table,
                             int table_width, int n_seqs, int n_pages, int window, float scale, void* out,
                             int n_tokens, int n_heads, int n_kv_heads, int head_dim, void* stream) {
    TQK_REQUIRE(q && keys && values && tok_seq && tok_pos && page_table && out, "tqk_attention: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && head_dim > 0, "tqk_attention: bad sizes");
    TQK_REQUIRE(n_heads % n_kv_heads == 0, "tqk_attention: %d heads are not a multiple of %d kv heads", n_heads, n_kv_heads);
    TQK_REQUIRE(head_dim <= ATT_MAX_D, "tqk_attention: head_dim %d is more than %d", head_dim, ATT_MAX_D);
    TQK_REQUIRE(n_heads <= 65535, "tqk_attention: too many heads for the grid");
    TQK_REQUIRE(table_width > 0 && n_pages > 0 && n_seqs > 0, "tqk_attention: empty page table");
    TQK_REQUIRE(window >= 0, "tqk_attention: negative window");
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((n_tokens + ATT_WAVES - 1) / ATT_WAVES, n_heads);
    if (act_dtype == TQK_F32)
        attention_generic_kernel<float><<<grid, ATT_WAVES * TQK_WAVE, 0, s>>>(
            (const float*)q, (const float*)keys, (const float*)values, tok_seq, tok_pos, page_table, table_width,
            window, scale, (float*)out, n_tokens, n_heads, n_kv_heads, head_dim);
    else if (act_dtype == TQK_BF16)
        attention_generic_kernel<bf16_t><<<grid, ATT_WAVES * TQK_WAVE, 0, s>>>(
            (const bf16_t*)q, (const bf16_t*)keys, (const bf16_t*)values, tok_seq, tok_pos, page_table, table_width,
            window, scale, (bf16_t*)out, n_tokens, n_heads, n_kv_heads, head_dim);
    else
        return tqk_fail("tqk_attention: unknown dtype %d", act_dtype);
    return tqk_check_launch("tqk_attention");
}
