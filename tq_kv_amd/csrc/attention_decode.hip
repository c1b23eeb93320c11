// Attention for decoding: one new token per sequence attends over its sequence's pages
// of the cache.  bfloat16 in, MFMA, float32 softmax.  Bound by the bytes of keys and
// values, so the work is cut for memory: one wave per (sequence, kv head, partition of
// the positions); all query heads that share the kv head ride in the same wave, so the
// keys and values are read once for the whole group (the reference expands them per
// query head instead, src/models/turbo_generic.rs:195-204, 1620-1621).  A second kernel
// merges the partitions.  Formulas as src/models/turbo_generic.rs:1622-1631, :56-62.
//
// Matrix-core mapping (v_mfma_f32_16x16x32_bf16, D[16x16] += A[16x32] B[32x16]):
//   scores^T[key][head] = K[key][:] . Q^T[:][head]
//       A = 16 keys x 32 elements of head_dim: lane l reads 16 contiguous bytes of key row
//           l%16 straight from the page; B = the heads' query rows, read the same way.
//       The lane then holds, for head l%16, the keys 4*(l/16)+r (r=0..3) of the 16.
//   out^T[element][head] = V^T[element][key] . P^T[key][head]
//       B needs for head l%16 eight keys per lane: the lane already holds them, the four
//       of one group of 16 keys and the four of the next (slot j<4: key 4g+j, j>=4: key
//       16+4g+j-4), so P never leaves its registers.  A must pair the same keys with the
//       slots: values are stored transposed in a page ([head_dim][64 positions]), so the
//       four keys of a slot group are 8 contiguous bytes of an element's row.
// Keys outside [lo, pos] get probability exactly 0 and their values are replaced by 0
// before the product, so nothing stored at such places can reach the result.
#include "common.h"
#include "tq_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

union pack8 {
    bf16x8_t v;
    bf16x4_t h[2];
    uint16_t u[8];
};

template <int D>
__global__ __launch_bounds__(TQK_WAVE)
void attention_decode_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ keys,
                             const bf16_t* __restrict__ values, const int32_t* __restrict__ tok_pos,
                             const int32_t* __restrict__ page_table, int table_width, int window, float scale,
                             int pages_per_part, int n_parts, int n_heads, int n_kv_heads, int q_blocks,
                             float* __restrict__ part_out, float* __restrict__ part_ml) {
    constexpr int KB = D / 32;          // k-blocks of the score product
    constexpr int DB = D / 16;          // 16-element blocks of the output
    const int lane = threadIdx.x;
    const int col = lane % 16, g = lane / 16;
    const int part = blockIdx.x;
    const int kvh = blockIdx.y / q_blocks, qb = blockIdx.y % q_blocks;
    const int seq = blockIdx.z;
    const int n_rep = n_heads / n_kv_heads;
    const int pos = tok_pos[seq];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;

    // the query head of this lane's column
    const int rep = qb * 16 + col;
    const bool head_live = rep < n_rep;
    const int head = kvh * n_rep + (head_live ? rep : 0);

    const int first_page = part * pages_per_part;
    const int last_page = min(first_page + pages_per_part - 1, pos / TQK_PAGE);
    const int start_page = max(first_page, lo / TQK_PAGE);

    float m = -INFINITY, l = 0.f;
    floatx4_t o[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i) o[i] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    if (start_page <= last_page) {
        pack8 zero;
#pragma unroll
        for (int i = 0; i < 8; ++i) zero.u[i] = 0;
        // the heads' queries: B operand of the score product
        bf16x8_t bq[KB];
        const bf16_t* qrow = q + ((size_t)seq * n_heads + head) * D + g * 8;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
            bq[kb] = head_live ? *reinterpret_cast<const bf16x8_t*>(qrow + kb * 32) : zero.v;

        const int32_t* pages = page_table + (size_t)seq * table_width;
        const size_t page_stride = (size_t)n_kv_heads * TQK_PAGE * D;
        for (int pg = start_page; pg <= last_page; ++pg) {
            const int page = pages[pg];
            if (page < 0) continue;                     // the host never lets this happen
            const bf16_t* kp = keys + (size_t)page * page_stride + (size_t)kvh * TQK_PAGE * D;
            const bf16_t* vp = values + (size_t)page * page_stride + (size_t)kvh * TQK_PAGE * D;
            const int key0 = pg * TQK_PAGE;
            const bool edge = key0 < lo || key0 + TQK_PAGE - 1 > pos;

            // scores^T for the page's four groups of 16 keys
            floatx4_t s[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                s[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
                const bf16_t* krow = kp + (size_t)(t * 16 + col) * D + g * 8;
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) {
                    const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(krow + kb * 32);
                    s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bq[kb], s[t], 0, 0, 0);
                }
            }
            // mask, scale, running maximum (the lane's head is its column; its keys are
            // key0 + 16 t + 4 g + r)
            float mx = m;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int j = key0 + t * 16 + g * 4 + r;
                    const float v = (j >= lo && j <= pos) ? s[t][r] * scale : -INFINITY;
                    s[t][r] = v;
                    mx = fmaxf(mx, v);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, TQK_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, TQK_WAVE));
            // mx is finite: the page holds at least one key of [lo, pos]
            const float alpha = expf(m - mx);
            m = mx;
            float psum = 0.f;
            pack8 pb[2];
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = s[t][r] == -INFINITY ? 0.f : expf(s[t][r] - mx);
                    // the probability enters the product as bfloat16; the sum uses the same rounded value
                    const uint16_t pbits = float_to_bf16_bits(p);
                    psum += __uint_as_float(((uint32_t)pbits) << 16);
                    pb[t / 2].u[(t % 2) * 4 + r] = pbits;
                }
            l = l * alpha + psum;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                o[db][0] *= alpha; o[db][1] *= alpha; o[db][2] *= alpha; o[db][3] *= alpha;
                const bf16_t* vrow = vp + (size_t)(db * 16 + col) * TQK_PAGE + g * 4;
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    pack8 av;
                    av.h[0] = *reinterpret_cast<const bf16x4_t*>(vrow + (2 * pr) * 16);
                    av.h[1] = *reinterpret_cast<const bf16x4_t*>(vrow + (2 * pr + 1) * 16);
                    if (edge) {
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            const int j = key0 + (2 * pr + i / 4) * 16 + g * 4 + (i % 4);
                            if (j < lo || j > pos) av.u[i] = 0;
                        }
                    }
                    o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av.v, pb[pr].v, o[db], 0, 0, 0);
                }
            }
        }
        l += __shfl_xor(l, 16, TQK_WAVE);
        l += __shfl_xor(l, 32, TQK_WAVE);
    }

    // partial result of this partition: out^T[element db*16 + 4g + r][head col]
    if (head_live) {
        const size_t row = ((size_t)seq * n_heads + head) * n_parts + part;
        float* po = part_out + row * D;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) po[db * 16 + g * 4 + r] = o[db][r];
        if (g == 0) { part_ml[row * 2] = m; part_ml[row * 2 + 1] = l; }
    }
}

// out[seq, head, :] = sum_p exp(m_p - M) o_p / sum_p exp(m_p - M) l_p, partitions in order.
__global__ void attention_merge_kernel(const float* __restrict__ part_out, const float* __restrict__ part_ml,
                                       int n_parts, int head_dim, bf16_t* __restrict__ out) {
    const size_t row = blockIdx.x;                     // seq * n_heads + head
    const float* ml = part_ml + row * n_parts * 2;
    float M = -INFINITY;
    for (int p = 0; p < n_parts; ++p) M = fmaxf(M, ml[p * 2]);
    float denom = 0.f;
    for (int p = 0; p < n_parts; ++p) denom += ml[p * 2] == -INFINITY ? 0.f : expf(ml[p * 2] - M) * ml[p * 2 + 1];
    for (int c = threadIdx.x; c < head_dim; c += blockDim.x) {
        float acc = 0.f;
        for (int p = 0; p < n_parts; ++p) {
            if (ml[p * 2] == -INFINITY) continue;
            acc += expf(ml[p * 2] - M) * part_out[(row * n_parts + p) * head_dim + c];
        }
        out[row * head_dim + c] = from_float<bf16_t>(acc / denom);
    }
}

extern "C" int tqk_attention_decode_supported(int head_dim) {
    return head_dim == 64 || head_dim == 128 || head_dim == 256 || head_dim == 32 || head_dim == 96;
}

extern "C" int tqk_attention_decode(const void* q, const void* keys, const void* values, const int32_t* tok_pos,
                                    const int32_t* page_table, int table_width, int n_seqs, int n_pages, int window,
                                    float scale, int pages_per_part, int n_parts, void* part_out, void* part_ml,
                                    void* out, int n_heads, int n_kv_heads, int head_dim, void* stream) {
    TQK_REQUIRE(q && keys && values && tok_pos && page_table && part_out && part_ml && out, "tqk_attention_decode: null pointer");
    TQK_REQUIRE(n_seqs >= 0 && n_heads > 0 && n_kv_heads > 0, "tqk_attention_decode: bad sizes");
    TQK_REQUIRE(n_heads % n_kv_heads == 0, "tqk_attention_decode: %d heads are not a multiple of %d kv heads", n_heads, n_kv_heads);
    TQK_REQUIRE(tqk_attention_decode_supported(head_dim), "tqk_attention_decode: head_dim %d is not one of 32, 64, 96, 128, 256", head_dim);
    TQK_REQUIRE(table_width > 0 && n_pages > 0, "tqk_attention_decode: empty page table");
    TQK_REQUIRE(pages_per_part > 0 && n_parts > 0 && (long long)n_parts * pages_per_part >= table_width,
                "tqk_attention_decode: %d partitions of %d pages do not cover %d pages", n_parts, pages_per_part, table_width);
    TQK_REQUIRE(window >= 0, "tqk_attention_decode: negative window");
    TQK_REQUIRE(n_seqs <= 65535 && n_kv_heads * ((n_heads / n_kv_heads + 15) / 16) <= 65535, "tqk_attention_decode: grid too large");
    if (n_seqs == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int q_blocks = (n_heads / n_kv_heads + 15) / 16;
    dim3 grid(n_parts, n_kv_heads * q_blocks, n_seqs);
#define LAUNCH(DD) attention_decode_kernel<DD><<<grid, TQK_WAVE, 0, s>>>( \
        (const bf16_t*)q, (const bf16_t*)keys, (const bf16_t*)values, tok_pos, page_table, table_width, window, scale, \
        pages_per_part, n_parts, n_heads, n_kv_heads, q_blocks, (float*)part_out, (float*)part_ml)
    switch (head_dim) {
        case 32: LAUNCH(32); break;
        case 64: LAUNCH(64); break;
        case 96: LAUNCH(96); break;
        case 128: LAUNCH(128); break;
        case 256: LAUNCH(256); break;
    }
#undef LAUNCH
    if (tqk_check_launch("tqk_attention_decode")) return -1;
    attention_merge_kernel<<<n_seqs * n_heads, head_dim >= 128 ? 128 : 64, 0, s>>>(
        (const float*)part_out, (const float*)part_ml, n_parts, head_dim, (bf16_t*)out);
    return tqk_check_launch("tqk_attention_decode merge");
}
