// Attention for decoding: one new token per sequence attends over its sequence's pages
// of the cache.  bfloat16 in, MFMA, float32 softmax.  Bound by the bytes of keys and
// values, so the work is cut for memory: a block of 4 waves (2 in large grids, 1 where a block has one page) per (sequence, kv head,
// partition of the pages); the partitions take the live pages in turn (partition p the pages
// first + p, first + p + parts, ...: however long the sequence is, they get the same share)
// and so do the four waves inside a partition; all
// query heads that share the kv head ride in the same wave, so keys and values are
// read once for the whole group (the reference expands them per query head instead,
// src/models/turbo_generic.rs:195-204, 1620-1621).  The waves' results are merged
// through LDS; with one partition the block writes the result itself, with more a
// second kernel merges the partitions in their order.  (Merging in the last block to
// finish, behind a device-wide fence, was measured to cost more than the second launch.)
// Formulas as src/models/turbo_generic.rs:1622-1631, :56-62.
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
//       slots: the cache keeps values transposed and in exactly this order inside a page
//       (value_place in common.h), 16 contiguous bytes per lane.
// Keys outside [lo, pos] get probability exactly 0 and their values are replaced by 0
// before the product, so nothing stored at such places can reach the result.
#include "common.h"
#include "tq_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int wave_of_block() { return threadIdx.x / TQK_WAVE; }

union pack8 {
    bf16x8_t v;
    uint16_t u[8];
    uint4 q;
};

#define AD_WAVES 4            // the most; blocks of 2 where the grid alone is more than the memory can serve at once

template <int D, bool NT, int W>
__global__ __launch_bounds__(AD_WAVES * TQK_WAVE)
void attention_decode_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ keys,
                             const bf16_t* __restrict__ values, const int32_t* __restrict__ tok_pos,
                             const int32_t* __restrict__ page_table, int table_width, int window, float scale,
                             int n_parts, int n_heads, int n_kv_heads, int q_blocks,
                             float* __restrict__ part_out, float* __restrict__ part_ml,
                             bf16_t* __restrict__ out) {
    constexpr int KB = D / 32;          // k-blocks of the score product
    constexpr int DB = D / 16;          // 16-element blocks of the output
    constexpr int ROW = DB * 4 + 2;     // floats a lane hands over: its out^T values, m, l
    // Head size 128: a page comes in with loads of 1 KB of contiguous memory each and goes through LDS into the matrix
    // cores' order, a region of 16 KB per wave (see below); the waves' results change hands through the same memory.
    // (Worth it where the step reads so much that the memory's rate counts, which is where the loads are marked as
    // read-once, NT: 64 sequences of 2100 positions 56.2 -> 49.7 us, 128 sequences 106 -> 89 us; 8 sequences 13.2 -> 14.2.)
    constexpr bool VIA_LDS = D == 128 && NT;
    constexpr int XCH = (W > 1 ? W - 1 : 1) * TQK_WAVE * ROW;
    constexpr int TURN = VIA_LDS ? W * 4096 : 0;                 // floats: 1024 pieces of 16 bytes a wave
    __shared__ __attribute__((aligned(16))) float lds_all[XCH > TURN ? XCH : TURN];
    float* const xch = lds_all;
    u32x4_t* const turn = reinterpret_cast<u32x4_t*>(lds_all) + wave_of_block() * 1024;
    const int wave = threadIdx.x / TQK_WAVE, lane = threadIdx.x % TQK_WAVE;
    const int col = lane % 16, g = lane / 16;
    const int part = blockIdx.x;
    const int kvh = blockIdx.y / q_blocks, qb = blockIdx.y % q_blocks;
    const int seq = blockIdx.z;
    const int n_rep = n_heads / n_kv_heads;
    const int pos = __builtin_amdgcn_readfirstlane(tok_pos[seq]);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    // exponentials to base 2 (one instruction each): the scores carry log2(e), and so do the running
    // maxima m here, in part_ml and in the merge kernel
    const float scale2 = scale * 1.4426950408889634f;

    // the query head of this lane's column
    const int rep = qb * 16 + col;
    const bool head_live = rep < n_rep;
    const int head = kvh * n_rep + (head_live ? rep : 0);

    const int last_page = pos / TQK_PAGE;
    const int start_page = lo / TQK_PAGE + part + wave * n_parts;       // this wave's first page

    float m = -INFINITY, l = 0.f;
    floatx4_t o[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i) o[i] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    if (start_page <= last_page) {
        pack8 zero;
        zero.q = make_uint4(0, 0, 0, 0);
        // the heads' queries: B operand of the score product
        bf16x8_t bq[KB];
        const bf16_t* qrow = q + ((size_t)seq * n_heads + head) * D + g * 8;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
            bq[kb] = head_live ? *reinterpret_cast<const bf16x8_t*>(qrow + kb * 32) : zero.v;

        const int32_t* pages = page_table + (size_t)seq * table_width;
        const size_t page_stride = (size_t)n_kv_heads * TQK_PAGE * D;
        for (int pg = start_page; pg <= last_page; pg += W * n_parts) {
            const int page = __builtin_amdgcn_readfirstlane(pages[pg]);        // the same in all lanes: the page's address is then a scalar
            if (page < 0) continue;                     // the host never lets this happen
            const bf16_t* kp = keys + (size_t)page * page_stride + (size_t)kvh * TQK_PAGE * D;
            const bf16_t* vp = values + (size_t)page * page_stride + (size_t)kvh * TQK_PAGE * D;
            const int key0 = pg * TQK_PAGE;
            const bool edge = key0 < lo || key0 + TQK_PAGE - 1 > pos;

            // all of the page's loads first, so that they are in flight together
            bf16x8_t ka[4][KB], va[DB][2];
            u32x4_t vr[VIA_LDS ? 16 : 1];
            if constexpr (VIA_LDS) {
                // A load of a wave takes 1 KB of contiguous memory (four key rows, eight value rows): the memory serves
                // such loads at 6.9 TB/s and loads of 64 bytes out of each of 16 rows, which is what the matrix cores'
                // order asks of a page as it lies in the cache, at 5.9.  The pieces of 16 bytes then go through the wave's
                // region of LDS to the lanes that need them, XOR-swizzled so that neither the writes nor the reads meet
                // a bank twice: the keys first, and the values through the same region once the scores are done.
                const u32x4_t* kg = reinterpret_cast<const u32x4_t*>(kp) + lane;
                const u32x4_t* vg = reinterpret_cast<const u32x4_t*>(vp) + lane;
                u32x4_t kr[16];
#pragma unroll
                for (int j = 0; j < 16; ++j) kr[j] = NT ? __builtin_nontemporal_load(kg + j * 64) : kg[j * 64];
#pragma unroll
                for (int j = 0; j < 16; ++j) vr[j] = NT ? __builtin_nontemporal_load(vg + j * 64) : vg[j * 64];
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int key = 4 * j + lane / 16, oct = lane % 16;
                    turn[key * 16 + (oct ^ (key & 15))] = kr[j];
                }
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb) {
                        const int key = t * 16 + col, oct = kb * 4 + g;
                        const u32x4_t piece = turn[key * 16 + (oct ^ (key & 15))];
                        ka[t][kb] = __builtin_bit_cast(bf16x8_t, piece);
                    }
                __builtin_amdgcn_wave_barrier();
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb)
                        ka[t][kb] = NT ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(kp + (size_t)(t * 16 + col) * D + kb * 32 + g * 8)) : *reinterpret_cast<const bf16x8_t*>(kp + (size_t)(t * 16 + col) * D + kb * 32 + g * 8);
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int pr = 0; pr < 2; ++pr)
                        va[db][pr] = NT ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(vp + (size_t)(db * 16 + col) * TQK_PAGE + pr * 32 + g * 8)) : *reinterpret_cast<const bf16x8_t*>(vp + (size_t)(db * 16 + col) * TQK_PAGE + pr * 32 + g * 8);
            }

            // scores^T for the page's four groups of 16 keys
            floatx4_t s[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                s[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
                    s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[t][kb], bq[kb], s[t], 0, 0, 0);
            }
            // mask, scale, running maximum (the lane's head is its column; its keys are
            // key0 + 16 t + 4 g + r)
            float mx = m;
            if (edge) {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int j = key0 + t * 16 + g * 4 + r;
                        const float v = (j >= lo && j <= pos) ? s[t][r] * scale2 : -INFINITY;
                        s[t][r] = v;
                        mx = fmaxf(mx, v);
                    }
            } else {                                    // a page wholly inside [lo, pos]: nothing to mask
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        s[t][r] *= scale2;
                        mx = fmaxf(mx, s[t][r]);
                    }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, TQK_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, TQK_WAVE));
            // mx is finite: the page holds at least one key of [lo, pos]
            const float alpha = __builtin_amdgcn_exp2f(m - mx);     // 2^(-inf) = 0 on the wave's first page
            m = mx;
            float psum = 0.f;
            pack8 pb[2];
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = __builtin_amdgcn_exp2f(s[t][r] - mx);          // a masked key: 2^(-inf) = 0
                    // the probability enters the product as bfloat16; the sum uses the same rounded value
                    const uint16_t pbits = float_to_bf16_bits(p);
                    psum += __uint_as_float(((uint32_t)pbits) << 16);
                    pb[t / 2].u[(t % 2) * 4 + r] = pbits;
                }
            l = l * alpha + psum;
            if constexpr (VIA_LDS) {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int d = 8 * j + lane / 8, oct = lane % 8;
                    turn[d * 8 + (oct ^ ((d >> 1) & 7))] = vr[j];
                }
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int pr = 0; pr < 2; ++pr) {
                        const int d = db * 16 + col, oct = pr * 4 + g;
                        const u32x4_t piece = turn[d * 8 + (oct ^ ((d >> 1) & 7))];
                        va[db][pr] = __builtin_bit_cast(bf16x8_t, piece);
                    }
                __builtin_amdgcn_wave_barrier();
            }
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                o[db][0] *= alpha; o[db][1] *= alpha; o[db][2] *= alpha; o[db][3] *= alpha;
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    pack8 av;
                    av.v = va[db][pr];
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

    // the waves' results into wave 0, in wave order
    if (VIA_LDS && W > 1) __syncthreads();          // (the memory they change hands through is the regions of the pages)
    if (wave > 0) {
        float* mine = xch + ((size_t)(wave - 1) * TQK_WAVE + lane) * ROW;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) mine[db * 4 + r] = o[db][r];
        mine[DB * 4] = m;
        mine[DB * 4 + 1] = l;
    }
    __syncthreads();
    const size_t row = ((size_t)seq * n_heads + head) * n_parts + part;
    if (wave == 0) {
        for (int w = 1; w < W; ++w) {
            const float* theirs = xch + ((size_t)(w - 1) * TQK_WAVE + lane) * ROW;
            const float m2 = theirs[DB * 4], l2 = theirs[DB * 4 + 1];
            if (m2 == -INFINITY) continue;
            const float mn = fmaxf(m, m2);
            const float a1 = __builtin_amdgcn_exp2f(m - mn), a2 = __builtin_amdgcn_exp2f(m2 - mn);
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[db][r] = o[db][r] * a1 + theirs[db * 4 + r] * a2;
            l = l * a1 + l2 * a2;
            m = mn;
        }
        if (!head_live) return;
        if (n_parts == 1) {
            // the only partition: this is the result, out[head, element db*16 + 4g + r]
            bf16_t* po = out + ((size_t)seq * n_heads + head) * D;
            const float inv = 1.f / l;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) po[db * 16 + g * 4 + r] = from_float<bf16_t>(o[db][r] * inv);
        } else {
            float* po = part_out + row * D;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) po[db * 16 + g * 4 + r] = o[db][r];
            if (g == 0) { part_ml[row * 2] = m; part_ml[row * 2 + 1] = l; }
        }
    }
}

// out[seq, head, :] = sum_p exp(m_p - M) o_p / sum_p exp(m_p - M) l_p, partitions in order.
// No branch in the loops, so that the loads of several partitions are under way together; a
// partition without keys (m = -inf) has weight 0 and its (unwritten) output is not looked at.
__global__ void attention_merge_kernel(const float* __restrict__ part_out, const float* __restrict__ part_ml,
                                       int n_parts, int head_dim, bf16_t* __restrict__ out) {
    const size_t row = blockIdx.x;                     // seq * n_heads + head
    const float2* ml = reinterpret_cast<const float2*>(part_ml) + row * n_parts;
    float M = -INFINITY;
#pragma unroll 8
    for (int p = 0; p < n_parts; ++p) M = fmaxf(M, ml[p].x);
    for (int c = threadIdx.x; c < head_dim; c += blockDim.x) {
        float acc = 0.f, denom = 0.f;
        const float* po = part_out + row * n_parts * head_dim + c;
#pragma unroll 8
        for (int p = 0; p < n_parts; ++p) {
            const float2 s = ml[p];
            const float v = po[(size_t)p * head_dim];
            const bool live = s.x != -INFINITY;
            const float wgt = live ? __builtin_amdgcn_exp2f(s.x - M) : 0.f;
            denom += wgt * s.y;
            acc += live ? wgt * v : 0.f;
        }
        out[row * head_dim + c] = from_float<bf16_t>(acc / denom);
    }
}

extern "C" int tqk_attention_decode_supported(int head_dim) {
    return head_dim == 64 || head_dim == 128 || head_dim == 256 || head_dim == 32 || head_dim == 96;
}

extern "C" int tqk_attention_decode(const void* q, const void* keys, const void* values, const int32_t* tok_pos,
                                    const int32_t* page_table, int table_width, int n_seqs, int n_pages, int window,
                                    float scale, int n_parts, void* part_out, void* part_ml,
                                    void* out, int n_heads, int n_kv_heads, int head_dim, void* stream) {
    TQK_REQUIRE(q && keys && values && tok_pos && page_table && out, "tqk_attention_decode: null pointer");
    TQK_REQUIRE(n_parts == 1 || (part_out && part_ml), "tqk_attention_decode: more than one partition needs part_out and part_ml");
    TQK_REQUIRE(n_seqs >= 0 && n_heads > 0 && n_kv_heads > 0, "tqk_attention_decode: bad sizes");
    TQK_REQUIRE(n_heads % n_kv_heads == 0, "tqk_attention_decode: %d heads are not a multiple of %d kv heads", n_heads, n_kv_heads);
    TQK_REQUIRE(tqk_attention_decode_supported(head_dim), "tqk_attention_decode: head_dim %d is not one of 32, 64, 96, 128, 256", head_dim);
    TQK_REQUIRE(table_width > 0 && n_pages > 0, "tqk_attention_decode: empty page table");
    TQK_REQUIRE(n_parts > 0 && n_parts <= 65535, "tqk_attention_decode: %d partitions", n_parts);
    TQK_REQUIRE(window >= 0, "tqk_attention_decode: negative window");
    const int q_blocks = (n_heads / n_kv_heads + 15) / 16;
    TQK_REQUIRE(n_seqs <= 65535 && n_kv_heads * q_blocks <= 65535, "tqk_attention_decode: grid too large");
    if (n_seqs == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(n_parts, n_kv_heads * q_blocks, n_seqs);
    // Keys and values are read once per step.  Saying so in the loads pays where the step reads more of them than the
    // caches hold (64 sequences of 2100 positions at the 7B sizes: 56.2 against 57.5 us) and costs where it reads little
    // (8 sequences: 14.4 against 13.6 us), so it goes by the most that the step's tables can name.
    const bool nt = (double)n_seqs * table_width * n_kv_heads * TQK_PAGE * head_dim * 4.0 > 128e6;
    // Four waves a block; two where there are 512 blocks or more without partitions: then the memory has more
    // pages asked of it at once than it serves well (128 sequences x 4 kv heads of 2100 positions: 106 against 114 us).
    const bool two = n_parts == 1 && (long long)n_seqs * n_kv_heads * q_blocks >= 512;
#define LAUNCH_W(DD, NT, W) attention_decode_kernel<DD, NT, W><<<grid, W * TQK_WAVE, 0, s>>>( \
        (const bf16_t*)q, (const bf16_t*)keys, (const bf16_t*)values, tok_pos, page_table, table_width, window, scale, \
        n_parts, n_heads, n_kv_heads, q_blocks, (float*)part_out, (float*)part_ml, (bf16_t*)out)
    // A partition per page of the table: a block then has one page to read, and one wave does it (4 sequences of 2100
    // positions: 8.8 against 10.7 us with four waves on four pages each; one sequence 5.8 against 9.0).
    const bool one = n_parts > 1 && n_parts >= table_width;
#define LAUNCH(DD) { if (one) { if (nt) LAUNCH_W(DD, true, 1); else LAUNCH_W(DD, false, 1); } else if (two) { if (nt) LAUNCH_W(DD, true, 2); else LAUNCH_W(DD, false, 2); } else { if (nt) LAUNCH_W(DD, true, 4); else LAUNCH_W(DD, false, 4); } }
    switch (head_dim) {
        case 32: LAUNCH(32); break;
        case 64: LAUNCH(64); break;
        case 96: LAUNCH(96); break;
        case 128: LAUNCH(128); break;
        case 256: LAUNCH(256); break;
    }
#undef LAUNCH_W
#undef LAUNCH
    if (tqk_check_launch("tqk_attention_decode")) return -1;
    if (n_parts == 1) return 0;
    attention_merge_kernel<<<n_seqs * n_heads, head_dim >= 128 ? 128 : 64, 0, s>>>(
        (const float*)part_out, (const float*)part_ml, n_parts, head_dim, (bf16_t*)out);
    return tqk_check_launch("tqk_attention_decode merge");
}
