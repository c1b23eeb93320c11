// Attention for prompts (and any step with many tokens per sequence): causal softmax
// attention of a tile of consecutive queries of one sequence and one head over the
// sequence's pages of the cache, flash style: one pass over the keys, running maximum
// and sum, float32 softmax, bfloat16 MFMA products.  Formulas as
// src/models/turbo_generic.rs:1620-1631 and :56-62; the mask is right for queries that
// start at any position (the reference's is only for position 0, :1937-1956), with an
// optional window.
//
// A block of 4 waves owns a tile of 64 or 128 queries; wave w owns 16 or 32 consecutive
// ones.  Tiles late in a sequence see more keys than early ones: the host lists the tiles
// longest first, and blocks are numbered heads-fastest, so that the blocks that share a
// compute unit have different lengths and the long ones start first.  The pages of keys
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
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));      // a native vector: copies of it stay in registers
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

#define PF_THREADS 256
#define PF_WAVES (PF_THREADS / TQK_WAVE)
#define PF_VPAD 8

// QB: blocks of 16 queries per wave.  A wave reads every key and value operand from LDS once
// and uses it for all its query blocks, so with QB = 2 (tiles of 128 queries) a query costs
// half the LDS reads and half the staging of QB = 1 (tiles of 64), and a wave has two
// independent chains of work; tiles of 64 leave fewer lanes idle on short prompts.
template <int D, int QB>
__global__ __launch_bounds__(PF_THREADS, 2)
void attention_prefill_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ keys,
                              const bf16_t* __restrict__ values, const int32_t* __restrict__ tok_pos,
                              const int32_t* __restrict__ page_table, int table_width,
                              const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_tok0,
                              const int32_t* __restrict__ tile_count, const int32_t* __restrict__ seq_start,
                              const int32_t* __restrict__ seq_new, int window, float scale,
                              bf16_t* __restrict__ out, int n_heads, int n_kv_heads, int n_tiles, int snake_width) {
    constexpr int KB = D / 32, DB = D / 16;
    constexpr int KSTRIDE = D + 8;                   // elements per key row in LDS
    constexpr int VSTRIDE = TQK_PAGE + PF_VPAD;      // elements per value row in LDS
    constexpr int CHUNKS = D / 32;                   // 16-byte chunks per thread, per operand
    constexpr int WQ = 16 * QB;                      // queries per wave
    __shared__ __attribute__((aligned(16))) uint16_t k_lds[TQK_PAGE * KSTRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t v_lds[D * VSTRIDE];

    const int tid = threadIdx.x;
    const int wave = tid / TQK_WAVE, lane = tid % TQK_WAVE;
    const int col = lane % 16, g = lane / 16;
    // Blocks in the order of their work, heads fastest (the host lists the tiles longest first).
    // With snake_width > 0 every other run of snake_width blocks is taken backwards: when all
    // blocks are resident at once, the compute units that got the longest get the shortest next.
    int order = blockIdx.x;
    if (snake_width > 0) {
        const int total = n_tiles * n_heads;
        const int round = order / snake_width, first = round * snake_width;
        const int size = min(snake_width, total - first);
        if (round & 1) order = first + size - 1 - (order - first);
    }
    const int tile = order / n_heads, head = order % n_heads;
    const int kvh = head / (n_heads / n_kv_heads);
    const int seq = tile_seq[tile], tok0 = tile_tok0[tile], count = tile_count[tile];
    const int pos0 = tok_pos[tok0];
    const int seq_end = seq_start[seq] + seq_new[seq];   // positions the cache holds after this step

    // this lane's queries, one per query block
    int qi[QB], my_pos[QB], my_lo[QB];
    bool q_live[QB];
#pragma unroll
    for (int b = 0; b < QB; ++b) {
        qi[b] = wave * WQ + b * 16 + col;
        q_live[b] = qi[b] < count;
        my_pos[b] = q_live[b] ? pos0 + qi[b] : -1;
        my_lo[b] = window > 0 ? max(0, my_pos[b] - window + 1) : 0;
    }
    // the wave's and the tile's ranges of positions
    const bool wave_live = wave * WQ < count;
    const int wave_last = min(pos0 + wave * WQ + WQ - 1, pos0 + count - 1);
    const int wave_first = pos0 + wave * WQ;                  // the wave's first query: it sees the fewest late keys
    const int wave_lo = window > 0 ? max(0, wave_first - window + 1) : 0;
    const int wave_lo_last = window > 0 ? max(0, wave_last - window + 1) : 0;   // the wave's last query sees the fewest early keys
    const float c2 = scale * 1.44269504088896340736f;
    const int tile_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
    const int first_page = tile_lo / TQK_PAGE, last_page = (pos0 + count - 1) / TQK_PAGE;

    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8_t bq[QB][KB];
#pragma unroll
    for (int b = 0; b < QB; ++b) {
        const bf16_t* qrow = q + ((size_t)(tok0 + (q_live[b] ? qi[b] : 0)) * n_heads + head) * D + g * 8;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
            bq[b][kb] = q_live[b] ? *reinterpret_cast<const bf16x8_t*>(qrow + kb * 32) : zero;
    }

    float m[QB], l[QB];
    floatx4_t o[QB][DB];
#pragma unroll
    for (int b = 0; b < QB; ++b) {
        m[b] = -INFINITY;
        l[b] = 0.f;
#pragma unroll
        for (int i = 0; i < DB; ++i) o[b][i] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    }

    const int32_t* pages = page_table + (size_t)seq * table_width;
    const size_t page_stride = (size_t)n_kv_heads * TQK_PAGE * D;
    u32x4_t kreg[CHUNKS], vreg[CHUNKS];

    // the next page's keys and values travel from global memory into registers while the
    // current page is computed on, and from there into LDS
    auto fetch = [&](int pg, u32x4_t (&kr)[CHUNKS], u32x4_t (&vr)[CHUNKS]) {
        const int page = pages[pg];
        const size_t base = (size_t)(page < 0 ? 0 : page) * page_stride + (size_t)kvh * TQK_PAGE * D;
        const u32x4_t* kp = reinterpret_cast<const u32x4_t*>(keys + base);
        const u32x4_t* vp = reinterpret_cast<const u32x4_t*>(values + base);
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            kr[c] = kp[tid + c * PF_THREADS];
            vr[c] = vp[tid + c * PF_THREADS];
        }
    };
    auto stage = [&](int pg, const u32x4_t (&kr)[CHUNKS], const u32x4_t (&vr)[CHUNKS]) {
        const int key0 = pg * TQK_PAGE;
        const bool tail = key0 + TQK_PAGE > seq_end;       // the page holds places beyond the sequence
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int idx = tid + c * PF_THREADS;
            // keys: chunk idx is elements 8*(idx % (D/8)).. of key row idx / (D/8)
            const int krow = idx / (D / 8), kpart = idx % (D / 8);
            *reinterpret_cast<u32x4_t*>(&k_lds[krow * KSTRIDE + kpart * 8]) = kr[c];
            // values: chunk idx is positions 8*(idx % 8).. of element row idx / 8
            const int vrow = idx / 8, vpart = idx % 8;
            uint32_t vw[4] = {vr[c].x, vr[c].y, vr[c].z, vr[c].w};
            if (tail) {
#pragma unroll
                for (int i = 0; i < 8; ++i)     // nothing stored beyond the sequence may count
                    if (key0 + value_position(vpart * 8 + i) >= seq_end) vw[i / 2] &= (i & 1) ? 0x0000ffffu : 0xffff0000u;
            }
            *reinterpret_cast<u32x4_t*>(&v_lds[vrow * VSTRIDE + vpart * 8]) = u32x4_t{vw[0], vw[1], vw[2], vw[3]};
        }
    };

    fetch(first_page, kreg, vreg);
    for (int pg = first_page; pg <= last_page; ++pg) {
        __syncthreads();                       // everyone is done with the page in LDS
        stage(pg, kreg, vreg);
        __syncthreads();
        fetch(min(pg + 1, last_page), kreg, vreg);           // (the last page again rather than a branch)
        const int key0 = pg * TQK_PAGE;
        if (!wave_live || key0 > wave_last || key0 + TQK_PAGE - 1 < wave_lo) continue;

        // independent chains of products (one per group of 16 keys and query block), interleaved
        floatx4_t s[QB][4];
#pragma unroll
        for (int b = 0; b < QB; ++b)
#pragma unroll
            for (int t = 0; t < 4; ++t) s[b][t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(&k_lds[(t * 16 + col) * KSTRIDE + kb * 32 + g * 8]);
#pragma unroll
                for (int b = 0; b < QB; ++b) s[b][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bq[b][kb], s[b][t], 0, 0, 0);
            }
        // Softmax in base 2: with c = scale * log2(e), p = 2^(s*c - m) where m is the running
        // maximum of s*c.  Only pages that cross a query's causal or window edge need the mask.
        const bool need_mask = key0 + TQK_PAGE - 1 > wave_first || key0 < wave_lo_last;
        bf16x8_t pb[QB][2];
#pragma unroll
        for (int b = 0; b < QB; ++b) {
            float mx = -INFINITY;
            if (need_mask) {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int j = key0 + t * 16 + g * 4 + r;
                        if (j < my_lo[b] || j > my_pos[b]) s[b][t][r] = -INFINITY;
                        mx = fmaxf(mx, s[b][t][r]);
                    }
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[b][t][r]);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, TQK_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, TQK_WAVE));
            const float m_new = fmaxf(m[b], mx * c2);        // c2 > 0, so the maximum of s*c2 is c2 times the maximum of s
            // a query may have no key in this page yet (window, or a lane without a query)
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m[b] - m_use);  // 2^(-inf) = 0 on a query's first keys
            m[b] = m_new;
            float psum = 0.f;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(s[b][t][r], c2, -m_use));
                    // the probability enters the product as bfloat16; the sum uses the same rounded value
                    const __bf16 pr16 = (__bf16)p;
                    psum += (float)pr16;
                    pb[b][t / 2][(t % 2) * 4 + r] = pr16;
                }
            l[b] = l[b] * alpha + psum;
            if (__any(alpha != 1.f)) {
#pragma unroll
                for (int db = 0; db < DB; ++db) { o[b][db][0] *= alpha; o[b][db][1] *= alpha; o[b][db][2] *= alpha; o[b][db][3] *= alpha; }
            }
        }
        // the lane's 8 keys of each half page lie together (value_place); independent chains
#pragma unroll
        for (int pr = 0; pr < 2; ++pr)
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const bf16x8_t av = *reinterpret_cast<const bf16x8_t*>(&v_lds[(db * 16 + col) * VSTRIDE + g * 8 + pr * 32]);
#pragma unroll
                for (int b = 0; b < QB; ++b) o[b][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, pb[b][pr], o[b][db], 0, 0, 0);
            }
    }
#pragma unroll
    for (int b = 0; b < QB; ++b) {
        float lb = l[b];
        lb += __shfl_xor(lb, 16, TQK_WAVE);
        lb += __shfl_xor(lb, 32, TQK_WAVE);
        if (q_live[b]) {
            // out^T[element db*16 + 4g + r][query col]
            bf16_t* orow = out + ((size_t)(tok0 + qi[b]) * n_heads + head) * D;
            const float inv = 1.f / lb;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) orow[db * 16 + g * 4 + r] = from_float<bf16_t>(o[b][db][r] * inv);
        }
    }
}

extern "C" int tqk_attention_prefill_supported(int head_dim) {
    return head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128;
}

extern "C" int tqk_attention_prefill(const void* q, const void* keys, const void* values, const int32_t* tok_pos,
                                     const int32_t* page_table, int table_width, int n_seqs, int n_pages,
                                     const int32_t* tile_seq, const int32_t* tile_tok0, const int32_t* tile_count,
                                     int n_tiles, int tile_queries, const int32_t* seq_start, const int32_t* seq_new,
                                     int window, float scale, void* out, int n_tokens, int n_heads, int n_kv_heads,
                                     int head_dim, void* stream) {
    TQK_REQUIRE(q && keys && values && tok_pos && page_table && tile_seq && tile_tok0 && tile_count && seq_start && seq_new && out,
                "tqk_attention_prefill: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_tiles >= 0 && n_heads > 0 && n_kv_heads > 0, "tqk_attention_prefill: bad sizes");
    TQK_REQUIRE(n_heads % n_kv_heads == 0, "tqk_attention_prefill: %d heads are not a multiple of %d kv heads", n_heads, n_kv_heads);
    TQK_REQUIRE(tqk_attention_prefill_supported(head_dim), "tqk_attention_prefill: head_dim %d is not one of 32, 64, 96, 128", head_dim);
    TQK_REQUIRE(table_width > 0 && n_pages > 0 && n_seqs > 0, "tqk_attention_prefill: empty page table");
    TQK_REQUIRE(window >= 0, "tqk_attention_prefill: negative window");
    TQK_REQUIRE(tile_queries == 64 || tile_queries == 128, "tqk_attention_prefill: tiles hold 64 or 128 queries, not %d", tile_queries);
    TQK_REQUIRE((long long)n_tiles * n_heads <= 0x7fffffffLL, "tqk_attention_prefill: %d tiles are more than the grid takes", n_tiles);
    if (n_tiles == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    // all blocks resident at once (two per compute unit): alternate the direction of the runs
    static int n_cus = 0;
    if (n_cus == 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
            return tqk_fail("tqk_attention_prefill: cannot read the number of compute units");
        n_cus = v;
    }
    const long long total = (long long)n_tiles * n_heads;
    const int snake = total <= 2LL * n_cus ? n_cus : 0;
    dim3 grid((unsigned)total);
#define LAUNCH(DD, QQ) attention_prefill_kernel<DD, QQ><<<grid, PF_THREADS, 0, s>>>( \
        (const bf16_t*)q, (const bf16_t*)keys, (const bf16_t*)values, tok_pos, page_table, table_width, tile_seq, tile_tok0, \
        tile_count, seq_start, seq_new, window, scale, (bf16_t*)out, n_heads, n_kv_heads, n_tiles, snake)
#define LAUNCH_D(DD) do { if (tile_queries == 128) LAUNCH(DD, 2); else LAUNCH(DD, 1); } while (0)
    switch (head_dim) {
        case 32: LAUNCH_D(32); break;
        case 64: LAUNCH_D(64); break;
        case 96: LAUNCH_D(96); break;
        case 128: LAUNCH_D(128); break;
    }
#undef LAUNCH_D
#undef LAUNCH
    return tqk_check_launch("tqk_attention_prefill");
}
