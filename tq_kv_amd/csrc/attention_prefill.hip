// Attention for prompts (and any step with many tokens per sequence): causal softmax
// attention of a tile of 64 consecutive queries of one sequence and one head over the
// sequence's pages of the cache, flash style: one pass over the keys, running maximum
// and sum, float32 softmax, bfloat16 MFMA products.  Formulas as
// src/models/turbo_generic.rs:1620-1631 and :56-62; the mask is right for queries that
// start at any position (the reference's is only for position 0, :1937-1956), with an
// optional window.
//
// A block of 4 waves owns the tile; wave w owns queries 16w..16w+15.  Tiles late in a
// sequence see more keys than early ones: the host lists the tiles longest first, and
// blocks are numbered heads-fastest, so that the blocks that share a compute unit have
// different lengths and the long ones start first.  The pages of keys
// (64 positions x head_dim) and of values (head_dim x 64 positions, stored transposed)
// are staged in LDS once per block and read by all four waves; the next page is on
// its way from global memory into registers while the current one is computed on.
//
// Matrix-core mapping as in the decoding kernel: scores^T = K Q^T puts a query in a
// lane's column and 4 keys of each group of 16 in its registers, which is exactly the
// operand layout that out^T = V^T P^T needs, so the probabilities never move.
// LDS rows are padded (keys by 8 elements, values by 8 places) so that the lanes of a
// read phase fall into different banks.
#include "common.h"
#include "tq_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

union pf_pack8 {
    bf16x8_t v;
    bf16x4_t h[2];
    __bf16 b[8];
    uint16_t u[8];
    uint4 q;
};

#define PF_TILE 64
#define PF_THREADS 256
#define PF_VPAD 8

template <int D>
__global__ __launch_bounds__(PF_THREADS)
void attention_prefill_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ keys,
                              const bf16_t* __restrict__ values, const int32_t* __restrict__ tok_pos,
                              const int32_t* __restrict__ page_table, int table_width,
                              const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_tok0,
                              const int32_t* __restrict__ tile_count, const int32_t* __restrict__ seq_start,
                              const int32_t* __restrict__ seq_new, int window, float scale,
                              bf16_t* __restrict__ out, int n_heads, int n_kv_heads) {
    constexpr int KB = D / 32, DB = D / 16;
    constexpr int KSTRIDE = D + 8;                   // elements per key row in LDS
    constexpr int VSTRIDE = TQK_PAGE + PF_VPAD;      // elements per value row in LDS
    constexpr int CHUNKS = D / 32;                   // 16-byte chunks per thread, per operand
    __shared__ __attribute__((aligned(16))) uint16_t k_lds[TQK_PAGE * KSTRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t v_lds[D * VSTRIDE];

    const int tid = threadIdx.x;
    const int wave = tid / TQK_WAVE, lane = tid % TQK_WAVE;
    const int col = lane % 16, g = lane / 16;
    const int tile = blockIdx.y, head = blockIdx.x;      // heads fastest: neighbouring blocks do equal work
    const int kvh = head / (n_heads / n_kv_heads);
    const int seq = tile_seq[tile], tok0 = tile_tok0[tile], count = tile_count[tile];
    const int pos0 = tok_pos[tok0];
    const int seq_end = seq_start[seq] + seq_new[seq];   // positions the cache holds after this step

    // this lane's query
    const int qi = wave * 16 + col;
    const bool q_live = qi < count;
    const int my_pos = q_live ? pos0 + qi : -1;
    const int my_lo = window > 0 ? max(0, my_pos - window + 1) : 0;
    // the wave's and the tile's ranges of positions
    const bool wave_live = wave * 16 < count;
    const int wave_last = min(pos0 + wave * 16 + 15, pos0 + count - 1);
    const int wave_first = pos0 + wave * 16;                  // the wave's first query: it sees the fewest late keys
    const int wave_lo = window > 0 ? max(0, wave_first - window + 1) : 0;
    const int wave_lo_last = window > 0 ? max(0, wave_last - window + 1) : 0;   // the wave's last query sees the fewest early keys
    const float c2 = scale * 1.44269504088896340736f;
    const int tile_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
    const int first_page = tile_lo / TQK_PAGE, last_page = (pos0 + count - 1) / TQK_PAGE;

    pf_pack8 zero;
    zero.q = make_uint4(0, 0, 0, 0);
    bf16x8_t bq[KB];
    {
        const bf16_t* qrow = q + ((size_t)(tok0 + (q_live ? qi : 0)) * n_heads + head) * D + g * 8;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
            bq[kb] = q_live ? *reinterpret_cast<const bf16x8_t*>(qrow + kb * 32) : zero.v;
    }

    float m = -INFINITY, l = 0.f;
    floatx4_t o[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i) o[i] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    const int32_t* pages = page_table + (size_t)seq * table_width;
    const size_t page_stride = (size_t)n_kv_heads * TQK_PAGE * D;
    uint4 kreg[CHUNKS], vreg[CHUNKS];

    auto fetch = [&](int pg) {
        const int page = pages[pg];
        const size_t base = (size_t)(page < 0 ? 0 : page) * page_stride + (size_t)kvh * TQK_PAGE * D;
        const uint4* kp = reinterpret_cast<const uint4*>(keys + base);
        const uint4* vp = reinterpret_cast<const uint4*>(values + base);
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            kreg[c] = kp[tid + c * PF_THREADS];
            vreg[c] = vp[tid + c * PF_THREADS];
        }
    };
    auto stage = [&](int pg) {
        const int key0 = pg * TQK_PAGE;
        const bool tail = key0 + TQK_PAGE > seq_end;       // the page holds places beyond the sequence
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int idx = tid + c * PF_THREADS;
            // keys: chunk idx is elements 8*(idx % (D/8)).. of key row idx / (D/8)
            const int krow = idx / (D / 8), kpart = idx % (D / 8);
            *reinterpret_cast<uint4*>(&k_lds[krow * KSTRIDE + kpart * 8]) = kreg[c];
            // values: chunk idx is positions 8*(idx % 8).. of element row idx / 8
            const int vrow = idx / 8, vpart = idx % 8;
            pf_pack8 v;
            v.q = vreg[c];
            if (tail) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (key0 + value_position(vpart * 8 + i) >= seq_end) v.u[i] = 0;   // nothing stored there may count
            }
            *reinterpret_cast<uint4*>(&v_lds[vrow * VSTRIDE + vpart * 8]) = v.q;
        }
    };

    fetch(first_page);
    for (int pg = first_page; pg <= last_page; ++pg) {
        __syncthreads();                       // everyone is done with the page in LDS
        stage(pg);
        __syncthreads();
        if (pg < last_page) fetch(pg + 1);
        const int key0 = pg * TQK_PAGE;
        if (!wave_live || key0 > wave_last || key0 + TQK_PAGE - 1 < wave_lo) continue;

        // four independent chains of products (one per group of 16 keys), interleaved
        floatx4_t s[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) s[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(&k_lds[(t * 16 + col) * KSTRIDE + kb * 32 + g * 8]);
                s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bq[kb], s[t], 0, 0, 0);
            }
        // Softmax in base 2: with c = scale * log2(e), p = 2^(s*c - m) where m is the running
        // maximum of s*c.  Only pages that cross a query's causal or window edge need the mask.
        const bool need_mask = key0 + TQK_PAGE - 1 > wave_first || key0 < wave_lo_last;
        float mx = -INFINITY;
        if (need_mask) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int j = key0 + t * 16 + g * 4 + r;
                    if (j < my_lo || j > my_pos) s[t][r] = -INFINITY;
                    mx = fmaxf(mx, s[t][r]);
                }
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[t][r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, TQK_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, TQK_WAVE));
        const float m_new = fmaxf(m, mx * c2);           // c2 > 0, so the maximum of s*c2 is c2 times the maximum of s
        // a query may have no key in this page yet (window, or a lane without a query)
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m - m_use);     // 2^(-inf) = 0 on a query's first keys
        m = m_new;
        float psum = 0.f;
        pf_pack8 pb[2];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float p = __builtin_amdgcn_exp2f(fmaf(s[t][r], c2, -m_use));
                // the probability enters the product as bfloat16; the sum uses the same rounded value
                const __bf16 pr16 = (__bf16)p;
                psum += (float)pr16;
                pb[t / 2].b[(t % 2) * 4 + r] = pr16;
            }
        l = l * alpha + psum;
        if (__any(alpha != 1.f)) {
#pragma unroll
            for (int db = 0; db < DB; ++db) { o[db][0] *= alpha; o[db][1] *= alpha; o[db][2] *= alpha; o[db][3] *= alpha; }
        }
        // the lane's 8 keys of each half page lie together (value_place); DB independent chains
#pragma unroll
        for (int pr = 0; pr < 2; ++pr)
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const bf16x8_t av = *reinterpret_cast<const bf16x8_t*>(&v_lds[(db * 16 + col) * VSTRIDE + g * 8 + pr * 32]);
                o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, pb[pr].v, o[db], 0, 0, 0);
            }
    }
    l += __shfl_xor(l, 16, TQK_WAVE);
    l += __shfl_xor(l, 32, TQK_WAVE);
    if (q_live) {
        // out^T[element db*16 + 4g + r][query col]
        bf16_t* orow = out + ((size_t)(tok0 + qi) * n_heads + head) * D;
        const float inv = 1.f / l;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) orow[db * 16 + g * 4 + r] = from_float<bf16_t>(o[db][r] * inv);
    }
}

extern "C" int tqk_attention_prefill_supported(int head_dim) {
    return head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128;
}

extern "C" int tqk_attention_prefill(const void* q, const void* keys, const void* values, const int32_t* tok_pos,
                                     const int32_t* page_table, int table_width, int n_seqs, int n_pages,
                                     const int32_t* tile_seq, const int32_t* tile_tok0, const int32_t* tile_count,
                                     int n_tiles, const int32_t* seq_start, const int32_t* seq_new, int window,
                                     float scale, void* out, int n_tokens, int n_heads, int n_kv_heads, int head_dim,
                                     void* stream) {
    TQK_REQUIRE(q && keys && values && tok_pos && page_table && tile_seq && tile_tok0 && tile_count && seq_start && seq_new && out,
                "tqk_attention_prefill: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_tiles >= 0 && n_heads > 0 && n_kv_heads > 0, "tqk_attention_prefill: bad sizes");
    TQK_REQUIRE(n_heads % n_kv_heads == 0, "tqk_attention_prefill: %d heads are not a multiple of %d kv heads", n_heads, n_kv_heads);
    TQK_REQUIRE(tqk_attention_prefill_supported(head_dim), "tqk_attention_prefill: head_dim %d is not one of 32, 64, 96, 128", head_dim);
    TQK_REQUIRE(table_width > 0 && n_pages > 0 && n_seqs > 0, "tqk_attention_prefill: empty page table");
    TQK_REQUIRE(window >= 0, "tqk_attention_prefill: negative window");
    TQK_REQUIRE(n_tiles <= 65535, "tqk_attention_prefill: %d tiles are more than the grid takes", n_tiles);
    if (n_tiles == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(n_heads, n_tiles);
#define LAUNCH(DD) attention_prefill_kernel<DD><<<grid, PF_THREADS, 0, s>>>( \
        (const bf16_t*)q, (const bf16_t*)keys, (const bf16_t*)values, tok_pos, page_table, table_width, tile_seq, tile_tok0, \
        tile_count, seq_start, seq_new, window, scale, (bf16_t*)out, n_heads, n_kv_heads)
    switch (head_dim) {
        case 32: LAUNCH(32); break;
        case 64: LAUNCH(64); break;
        case 96: LAUNCH(96); break;
        case 128: LAUNCH(128); break;
    }
#undef LAUNCH
    return tqk_check_launch("tqk_attention_prefill");
}
