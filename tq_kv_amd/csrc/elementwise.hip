// Embedding gather, residual add + RMSNorm, bias + rotation + cache write, SwiGLU.
// Memory-bound kernels; all arithmetic in float32.
#include "common.h"
#include "tq_kernels.h"

// ---- embedding ------------------------------------------------------------------
// The reference looks rows up with candle's embedding op (src/models/turbo_generic.rs:1958).
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids,
                             int hidden, int vocab, float scale, float* __restrict__ out, bf16_t* __restrict__ copy,
                             const bf16_t* __restrict__ copy_weight, float* __restrict__ ss_out) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const int id = ids[t];
    float* o = out + (size_t)t * hidden;
    bf16_t* c = copy ? copy + (size_t)t * hidden : nullptr;
    const bool ok = id >= 0 && id < vocab;
    const T* row = table + (size_t)(ok ? id : 0) * hidden;
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float v = ok ? to_float(row[i]) * scale : 0.f;
        o[i] = v;
        ss = fmaf(v, v, ss);
        if (c) c[i] = from_float<bf16_t>(copy_weight ? v * to_float(copy_weight[i]) : v);
    }
    if (ss_out) {
        const float total = block_sum(ss, scratch);
        if (threadIdx.x == 0) ss_out[t] = total;
    }
}

// bfloat16 table, hidden a multiple of 8: 16 bytes per thread and load, one pass.
__global__ void embed_bf16x8_kernel(const bf16_t* __restrict__ table, const int32_t* __restrict__ ids,
                                    int hidden, int vocab, float scale, float* __restrict__ out, bf16_t* __restrict__ copy,
                                    const bf16_t* __restrict__ copy_weight, float* __restrict__ ss_out) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const int id = ids[t];
    const bool ok = id >= 0 && id < vocab;
    const uint4* row = reinterpret_cast<const uint4*>(table + (size_t)(ok ? id : 0) * hidden);
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden / 8; i += blockDim.x) {
        const uint4 raw = ok ? row[i] : make_uint4(0, 0, 0, 0);
        const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
        float v[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = __uint_as_float(words[j] << 16) * scale;
            v[2 * j + 1] = __uint_as_float(words[j] & 0xffff0000u) * scale;
        }
        float4* o = reinterpret_cast<float4*>(out + (size_t)t * hidden + (size_t)i * 8);
        o[0] = make_float4(v[0], v[1], v[2], v[3]);
        o[1] = make_float4(v[4], v[5], v[6], v[7]);
#pragma unroll
        for (int j = 0; j < 8; ++j) ss = fmaf(v[j], v[j], ss);
        if (copy) {
            uint4 packed = raw;
            if (copy_weight || scale != 1.0f) {
                const uint4 wraw = copy_weight ? reinterpret_cast<const uint4*>(copy_weight)[i]
                                               : make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);      // ones
                const uint32_t ww[4] = {wraw.x, wraw.y, wraw.z, wraw.w};
                uint32_t pw[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t lo = float_to_bf16_bits(v[2 * j] * __uint_as_float(ww[j] << 16));
                    const uint32_t hi = float_to_bf16_bits(v[2 * j + 1] * __uint_as_float(ww[j] & 0xffff0000u));
                    pw[j] = lo | (hi << 16);
                }
                packed = make_uint4(pw[0], pw[1], pw[2], pw[3]);
            }
            reinterpret_cast<uint4*>(copy + (size_t)t * hidden)[i] = packed;
        }
    }
    if (ss_out) {
        const float total = block_sum(ss, scratch);
        if (threadIdx.x == 0) ss_out[t] = total;
    }
}

extern "C" int tqk_embed(const void* table, int table_dtype, const int32_t* ids, int n_tokens,
                         int hidden, int vocab, float scale, float* out, void* copy_bf16, const void* copy_weight,
                         float* ss_out, void* stream) {
    TQK_REQUIRE(table && ids && out, "tqk_embed: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && hidden > 0 && vocab > 0, "tqk_embed: bad sizes tokens=%d hidden=%d vocab=%d", n_tokens, hidden, vocab);
    TQK_REQUIRE(!ss_out || n_tokens <= 16, "tqk_embed: sums of squares are kept for at most 16 tokens, got %d", n_tokens);
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (table_dtype == TQK_F32)
        embed_kernel<float><<<n_tokens, 256, 0, s>>>((const float*)table, ids, hidden, vocab, scale, out, (bf16_t*)copy_bf16,
                                                     (const bf16_t*)copy_weight, ss_out);
    else if (table_dtype == TQK_BF16 && hidden % 8 == 0 && (((uintptr_t)table | (uintptr_t)out | (uintptr_t)copy_bf16 | (uintptr_t)copy_weight) & 15) == 0) {
        const int threads = ((hidden / 8 + TQK_WAVE - 1) / TQK_WAVE) * TQK_WAVE;
        embed_bf16x8_kernel<<<n_tokens, threads > 1024 ? 1024 : threads, 0, s>>>((const bf16_t*)table, ids, hidden, vocab, scale, out, (bf16_t*)copy_bf16,
                                                                               (const bf16_t*)copy_weight, ss_out);
    } else if (table_dtype == TQK_BF16)
        embed_kernel<bf16_t><<<n_tokens, 256, 0, s>>>((const bf16_t*)table, ids, hidden, vocab, scale, out, (bf16_t*)copy_bf16,
                                                      (const bf16_t*)copy_weight, ss_out);
    else
        return tqk_fail("tqk_embed: unknown dtype %d", table_dtype);
    return tqk_check_launch("tqk_embed");
}

// ---- what an architecture may do to its logits after the head ------------------------------------
__global__ void finish_logits_kernel(float* __restrict__ logits, long long n, int vocab, const float* __restrict__ bias,
                                     float scale, float cap) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float l = logits[i];
        if (bias) l += bias[i % vocab];
        l *= scale;
        if (cap > 0.f) l = cap * tanhf(l / cap);
        logits[i] = l;
    }
}

extern "C" int tqk_finish_logits(float* logits, int n_rows, int vocab, const float* bias, float scale, float cap, void* stream) {
    TQK_REQUIRE(logits, "tqk_finish_logits: null pointer");
    TQK_REQUIRE(n_rows >= 0 && vocab > 0, "tqk_finish_logits: bad sizes rows=%d vocab=%d", n_rows, vocab);
    if (n_rows == 0) return 0;
    const long long n = (long long)n_rows * vocab;
    const long long want = (n + 255) / 256;
    finish_logits_kernel<<<(int)(want < 8192 ? want : 8192), 256, 0, (hipStream_t)stream>>>(logits, n, vocab, bias, scale, cap);
    return tqk_check_launch("tqk_finish_logits");
}

// ---- residual add + RMSNorm -----------------------------------------------------
// y = x / sqrt(mean(x^2) + eps) * w in float32, cast last, as
// src/models/turbo_generic.rs:41-51 does (division by the root, weight inside).
//
// The update can also come as a product's unfinished sums: float32 [n_sums][rows][hidden], the
// sums of the product over n_sums pieces of its K (mid_product.hip).  They are added up in their
// order and rounded to the activation type, as the finished product would have been, and then
// added as any other update: the product's own finishing pass and its round trip disappear.
struct PartSums { const float* sums; int n; size_t stride; };       // stride: rows * hidden

template <typename TA>
__device__ __forceinline__ float summed(const PartSums& ps, size_t at) {
    float a = 0.f;
    for (int s = 0; s < ps.n; ++s) a += ps.sums[(size_t)s * ps.stride + at];
    return to_float(from_float<TA>(a));
}

template <typename TA, typename TW>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const TA* __restrict__ delta, const PartSums ps,
                                   const TW* __restrict__ weight, float eps,
                                   const int32_t* __restrict__ rows, int hidden,
                                   TA* __restrict__ out, int write_back) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t row = rows ? (size_t)rows[r] : (size_t)r;
    float* hr = h ? h + row * hidden : nullptr;
    const TA* dr = delta ? delta + row * hidden : nullptr;
    TA* o = out + (size_t)r * hidden;
    float ss = 0.f;
    auto value = [&](int i) {
        float v = hr ? hr[i] : 0.f;
        if (dr) v += to_float(dr[i]);
        if (ps.sums) v += summed<TA>(ps, row * hidden + i);
        return v;
    };
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float v = value(i);
        if (write_back) hr[i] = v;
        ss += v * v;
    }
    const float total = block_sum(ss, scratch);
    const float rms = sqrtf(total / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        // the same thread wrote h[i] above, so with write_back the value is read back exactly
        const float v = write_back ? hr[i] : value(i);
        o[i] = from_float<TA>((v / rms) * to_float(weight[i]));
    }
}

// The same for rows of up to VPT * 4 * blockDim elements, a multiple of 4: every value is
// read once, in vectors of 4, and stays in registers between the two passes.
template <typename TA> struct Vec4;
template <> struct Vec4<float> { float4 v; __device__ float get(int i) const { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; } };
template <> struct Vec4<bf16_t> { uint2 v; __device__ float get(int i) const {
    const uint32_t word = i < 2 ? v.x : v.y;
    return __uint_as_float((i & 1) ? (word & 0xffff0000u) : (word << 16)); } };

template <typename T> __device__ __forceinline__ void store4(T* p, float a, float b, float c, float d);
template <> __device__ __forceinline__ void store4<float>(float* p, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, float a, float b, float c, float d) {
    uint2 o;
    o.x = (uint32_t)float_to_bf16_bits(a) | ((uint32_t)float_to_bf16_bits(b) << 16);
    o.y = (uint32_t)float_to_bf16_bits(c) | ((uint32_t)float_to_bf16_bits(d) << 16);
    *reinterpret_cast<uint2*>(p) = o;
}

template <typename TA, typename TW, int VPT>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ h, const TA* __restrict__ delta, const PartSums ps,
                                       const TW* __restrict__ weight, float eps,
                                       const int32_t* __restrict__ rows, int hidden,
                                       TA* __restrict__ out, int write_back) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t row = rows ? (size_t)rows[r] : (size_t)r;
    float* hr = h ? h + row * hidden : nullptr;
    const TA* dr = delta ? delta + row * hidden : nullptr;
    TA* o = out + (size_t)r * hidden;
    float v[VPT][4];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int i = (j * blockDim.x + threadIdx.x) * 4;
        if (i < hidden) {
            float4 hv = hr ? *reinterpret_cast<const float4*>(hr + i) : make_float4(0.f, 0.f, 0.f, 0.f);
            if (dr) {
                Vec4<TA> d;
                d.v = *reinterpret_cast<const decltype(d.v)*>(dr + i);
                hv.x += d.get(0); hv.y += d.get(1); hv.z += d.get(2); hv.w += d.get(3);
            }
            if (ps.sums) {
                float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
                const float* at = ps.sums + row * hidden + i;
                int s = 0;
                for (; s + 4 <= ps.n; s += 4) {             // four loads under way together, added in order
                    float4 part[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) part[u] = *reinterpret_cast<const float4*>(at + (size_t)(s + u) * ps.stride);
#pragma unroll
                    for (int u = 0; u < 4; ++u) { a.x += part[u].x; a.y += part[u].y; a.z += part[u].z; a.w += part[u].w; }
                }
                for (; s < ps.n; ++s) {
                    const float4 part = *reinterpret_cast<const float4*>(at + (size_t)s * ps.stride);
                    a.x += part.x; a.y += part.y; a.z += part.z; a.w += part.w;
                }
                hv.x += to_float(from_float<TA>(a.x)); hv.y += to_float(from_float<TA>(a.y));
                hv.z += to_float(from_float<TA>(a.z)); hv.w += to_float(from_float<TA>(a.w));
            }
            if (write_back) *reinterpret_cast<float4*>(hr + i) = hv;
            v[j][0] = hv.x; v[j][1] = hv.y; v[j][2] = hv.z; v[j][3] = hv.w;
            ss += hv.x * hv.x + hv.y * hv.y + hv.z * hv.z + hv.w * hv.w;
        }
    }
    const float total = block_sum(ss, scratch);
    const float rms = sqrtf(total / (float)hidden + eps);
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int i = (j * blockDim.x + threadIdx.x) * 4;
        if (i < hidden) {
            Vec4<TW> w;
            w.v = *reinterpret_cast<const decltype(w.v)*>(weight + i);
            store4<TA>(o + i, (v[j][0] / rms) * w.get(0), (v[j][1] / rms) * w.get(1),
                       (v[j][2] / rms) * w.get(2), (v[j][3] / rms) * w.get(3));
        }
    }
}

static int add_rmsnorm(float* h, const void* delta, const PartSums ps, int act_dtype, const void* weight,
                       int weight_dtype, float eps, const int32_t* rows, int n_rows,
                       int hidden, void* out, int write_back, void* stream) {
    TQK_REQUIRE(weight && out, "tqk_add_rmsnorm: null pointer");
    TQK_REQUIRE(h || delta || ps.sums, "tqk_add_rmsnorm: neither h nor an update given");
    TQK_REQUIRE(!write_back || (h && !rows), "tqk_add_rmsnorm: write_back needs h and no row list");
    TQK_REQUIRE(n_rows >= 0 && hidden > 0, "tqk_add_rmsnorm: bad sizes rows=%d hidden=%d", n_rows, hidden);
    TQK_REQUIRE(act_dtype == TQK_F32 || act_dtype == TQK_BF16, "tqk_add_rmsnorm: unknown activation dtype %d", act_dtype);
    TQK_REQUIRE(weight_dtype == TQK_F32 || weight_dtype == TQK_BF16, "tqk_add_rmsnorm: unknown weight dtype %d", weight_dtype);
    if (n_rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const bool aligned = ((((uintptr_t)h) | ((uintptr_t)delta) | ((uintptr_t)weight) | ((uintptr_t)out) | ((uintptr_t)ps.sums)) & 15) == 0;
    const int code = act_dtype * 2 + weight_dtype;
    if (hidden % 4 == 0 && hidden <= 8192 && aligned) {
        // sums of a product: several times the bytes per row, and few rows: more threads per row
        const int threads = ps.sums ? 1024 : 256;
#define LAUNCHV(TA, TW, VPT) add_rmsnorm_vec_kernel<TA, TW, VPT><<<n_rows, threads, 0, s>>>( \
        h, (const TA*)delta, ps, (const TW*)weight, eps, rows, hidden, (TA*)out, write_back)
#define PICK(TA, TW) do { const int per = (hidden + threads * 4 - 1) / (threads * 4); \
        if (per <= 1) LAUNCHV(TA, TW, 1); else if (per <= 2) LAUNCHV(TA, TW, 2); \
        else if (per <= 4) LAUNCHV(TA, TW, 4); else LAUNCHV(TA, TW, 8); } while (0)
        switch (code) {
            case 0: PICK(float, float); break;
            case 1: PICK(float, bf16_t); break;
            case 2: PICK(bf16_t, float); break;
            case 3: PICK(bf16_t, bf16_t); break;
        }
#undef PICK
#undef LAUNCHV
        return tqk_check_launch("tqk_add_rmsnorm");
    }
    const int threads = hidden >= 2048 ? 512 : 256;
#define LAUNCH(TA, TW) add_rmsnorm_kernel<TA, TW><<<n_rows, threads, 0, s>>>( \
        h, (const TA*)delta, ps, (const TW*)weight, eps, rows, hidden, (TA*)out, write_back)
    switch (code) {
        case 0: LAUNCH(float, float); break;
        case 1: LAUNCH(float, bf16_t); break;
        case 2: LAUNCH(bf16_t, float); break;
        case 3: LAUNCH(bf16_t, bf16_t); break;
    }
#undef LAUNCH
    return tqk_check_launch("tqk_add_rmsnorm");
}

extern "C" int tqk_add_rmsnorm(float* h, const void* delta, int act_dtype, const void* weight,
                               int weight_dtype, float eps, const int32_t* rows, int n_rows,
                               int hidden, void* out, int write_back, void* stream) {
    return add_rmsnorm(h, delta, PartSums{nullptr, 0, 0}, act_dtype, weight, weight_dtype, eps, rows, n_rows, hidden, out,
                       write_back, stream);
}

/* The same with the update given as a product's sums over n_sums pieces of its K, float32
 * [n_sums][sum_rows][hidden] (row r of the update is row rows[r], or r, of each piece). */
extern "C" int tqk_add_rmsnorm_sums(float* h, const float* sums, int n_sums, int sum_rows, int act_dtype, const void* weight,
                                    int weight_dtype, float eps, const int32_t* rows, int n_rows,
                                    int hidden, void* out, int write_back, void* stream) {
    TQK_REQUIRE(sums && n_sums > 0 && sum_rows > 0, "tqk_add_rmsnorm_sums: no sums given");
    return add_rmsnorm(h, nullptr, PartSums{sums, n_sums, (size_t)sum_rows * hidden}, act_dtype, weight, weight_dtype, eps,
                       rows, n_rows, hidden, out, write_back, stream);
}

// ---- bias + rotation + cache write ------------------------------------------------
// Rotation as src/models/turbo_generic.rs:417-427 (halves) and :430-443 (pairs), angle
// tables as :1654-1670, applied after the bias (:805-813, :832-833); the cache holds
// rotated keys.  A wave handles one head of one token; a thread computes one element
// and reads the partner it rotates with.
template <typename TA, typename TB>
__global__ void rope_store_kernel(const TA* __restrict__ qkv, const TB* __restrict__ bias,
                                  const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                                  int rot_dim, int style, int max_positions,
                                  const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                  const int32_t* __restrict__ page_table, int table_width,
                                  TA* __restrict__ keys, TA* __restrict__ values,
                                  TA* __restrict__ q_out, int n_heads, int n_kv_heads, int head_dim,
                                  int write_kv) {
    const int t = blockIdx.x;
    // a wave per head, four heads per block: 0..nh-1 q, then nkv k heads, then nkv v heads
    const int head = blockIdx.y * 4 + threadIdx.x / TQK_WAVE;
    const int lane = threadIdx.x % TQK_WAVE;
    if (head >= n_heads + 2 * n_kv_heads) return;
    const int total = (n_heads + 2 * n_kv_heads) * head_dim;
    const int pos = tok_pos[t];
    const int kind = head < n_heads ? 0 : (head < n_heads + n_kv_heads ? 1 : 2);
    if (kind != 0 && !write_kv) return;
    const TA* src = qkv + (size_t)t * total + (size_t)head * head_dim;
    const TB* b = bias ? bias + (size_t)head * head_dim : nullptr;

    // q rows and key rows are contiguous in head_dim; values are kept transposed inside a
    // page, [kv head][head_dim][place of the position], so that the matrix cores can read
    // the 8 positions a lane needs of one element as 16 contiguous bytes.
    TA* dst;
    size_t dst_stride = 1;
    if (kind == 0) {
        dst = q_out + ((size_t)t * n_heads + head) * head_dim;
    } else {
        const int kvh = kind == 1 ? head - n_heads : head - n_heads - n_kv_heads;
        const int page = page_table[(size_t)tok_seq[t] * table_width + pos / TQK_PAGE];
        if (page < 0) return;                          // the host never lets this happen
        const size_t base = ((size_t)page * n_kv_heads + kvh) * TQK_PAGE * head_dim;
        if (kind == 1) {
            dst = keys + base + (size_t)(pos % TQK_PAGE) * head_dim;
        } else {
            dst = values + base + value_place(pos % TQK_PAGE);
            dst_stride = TQK_PAGE;
        }
    }

    const int half_rot = rot_dim / 2;
    const bool rotate = style != 0 && kind != 2 && pos < max_positions;
    for (int i = lane; i < head_dim; i += TQK_WAVE) {
        float x = to_float(src[i]) + (b ? to_float(b[i]) : 0.f);
        if (rotate && i < rot_dim) {
            // `first`: this element is x0 of its pair, else x1; p is the pair's table column
            int p, partner; bool first;
            if (style == 1) { first = i < half_rot; p = first ? i : i - half_rot; partner = first ? i + half_rot : i - half_rot; }
            else { first = (i & 1) == 0; p = i >> 1; partner = i ^ 1; }
            const float y = to_float(src[partner]) + (b ? to_float(b[partner]) : 0.f);
            const float c = cos_table[(size_t)pos * half_rot + p];
            const float s = sin_table[(size_t)pos * half_rot + p];
            x = first ? x * c - y * s : y * s + x * c;
        }
        dst[(size_t)i * dst_stride] = from_float<TA>(x);
    }
}

// The values of a step of many tokens.  The cache keeps them transposed inside a page, so the kernel
// below, whose lanes run along head_dim, stores every element as 2 bytes into a row of its own:
// 8 of the 16 us it takes for 2048 tokens at the 7B sizes.  In these blocks the lanes run along the tokens (64
// per block, one kv head, the waves taking chunks of 8 elements in turn): where the tokens are
// neighbours in a sequence, as in a prompt, a wave's stores of one element fall into one 128-byte row.
// Every lane finds its own page and place, so nothing depends on the tokens being neighbours.
// job: (group of 64 tokens) * n_kv_heads + kv head.
__device__ __forceinline__ void store_values_bf16(int job, const bf16_t* __restrict__ qkv, const PartSums ps, const bf16_t* __restrict__ bias,
                                                  const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                                  const int32_t* __restrict__ page_table, int table_width, bf16_t* __restrict__ values,
                                                  int n_tokens, int n_heads, int n_kv_heads, int head_dim) {
    const int lane = threadIdx.x % TQK_WAVE, wave = threadIdx.x / TQK_WAVE, n_waves = blockDim.x / TQK_WAVE;
    const int t = (job / n_kv_heads) * TQK_WAVE + lane, kvh = job % n_kv_heads;
    if (t >= n_tokens) return;
    const int pos = tok_pos[t];
    const int page = page_table[(size_t)tok_seq[t] * table_width + pos / TQK_PAGE];
    if (page < 0) return;                              // the host never lets this happen
    bf16_t* dst = values + ((size_t)page * n_kv_heads + kvh) * TQK_PAGE * head_dim + value_place(pos % TQK_PAGE);
    const size_t total = (size_t)(n_heads + 2 * n_kv_heads) * head_dim;
    const size_t at = (size_t)t * total + (size_t)(n_heads + n_kv_heads + kvh) * head_dim;
    for (int c = wave * 8; c < head_dim; c += n_waves * 8) {
        float v[8];
        if (ps.sums) {
            float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
            for (int s = 0; s < ps.n; ++s) {
                const float4 pa = *reinterpret_cast<const float4*>(ps.sums + (size_t)s * ps.stride + at + c);
                const float4 pb = *reinterpret_cast<const float4*>(ps.sums + (size_t)s * ps.stride + at + c + 4);
                a.x += pa.x; a.y += pa.y; a.z += pa.z; a.w += pa.w;
                b.x += pb.x; b.y += pb.y; b.z += pb.z; b.w += pb.w;
            }
            const float sums[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = to_float(from_float<bf16_t>(sums[k]));
        } else {
            const uint4 raw = *reinterpret_cast<const uint4*>(qkv + at + c);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) { v[2 * k] = __uint_as_float(w[k] << 16); v[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u); }
        }
        if (bias) {
            const uint4 raw = *reinterpret_cast<const uint4*>(bias + (size_t)(n_heads + n_kv_heads + kvh) * head_dim + c);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) { v[2 * k] += __uint_as_float(w[k] << 16); v[2 * k + 1] += __uint_as_float(w[k] & 0xffff0000u); }
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) dst[(size_t)(c + k) * TQK_PAGE].bits = (uint16_t)float_to_bf16_bits(v[k]);
    }
}
// The common case in bfloat16 (halves layout over the whole head, head_dim a multiple of 8): a
// thread takes 4 neighbouring elements of the first half and the 4 they rotate with, 8 bytes
// per load and store; 16 heads of a token per block.  The q, k, v product may come unfinished, as
// its sums over pieces of K (see PartSums): they are added up and rounded here.
__global__ void rope_store_halves_bf16_kernel(const bf16_t* __restrict__ qkv, const PartSums ps, const bf16_t* __restrict__ bias,
                                              const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                                              int max_positions, const int32_t* __restrict__ tok_seq,
                                              const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ page_table,
                                              int table_width, bf16_t* __restrict__ keys, bf16_t* __restrict__ values,
                                              bf16_t* __restrict__ q_out, int n_heads, int n_kv_heads, int head_dim,
                                              int write_kv, int value_layer, int n_tokens) {
    // write_kv == 2: the values are stored by the blocks of the grid's last layer (blockIdx.y == value_layer)
    if (write_kv == 2 && (int)blockIdx.y == value_layer) {
        const int jobs = ((n_tokens + TQK_WAVE - 1) / TQK_WAVE) * n_kv_heads;
        for (int job = blockIdx.x; job < jobs; job += gridDim.x)
            store_values_bf16(job, qkv, ps, bias, tok_seq, tok_pos, page_table, table_width, values, n_tokens, n_heads, n_kv_heads, head_dim);
        return;
    }
    const int t = blockIdx.x;
    const int per_head = head_dim / 8;                  // threads per head
    const int slot = blockIdx.y * blockDim.x + threadIdx.x;
    const int head = slot / per_head, i = (slot % per_head) * 4, half = head_dim / 2;
    if (head >= n_heads + 2 * n_kv_heads) return;
    const int kind = head < n_heads ? 0 : (head < n_heads + n_kv_heads ? 1 : 2);
    if (kind != 0 && !write_kv) return;
    if (kind == 2 && write_kv == 2) return;            // the values are the last layer's
    const int pos = tok_pos[t];
    const size_t total = (size_t)(n_heads + 2 * n_kv_heads) * head_dim;
    float lo[4], hi[4];
    if (ps.sums) {
        const float* at = ps.sums + (size_t)t * total + (size_t)head * head_dim + i;
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
        for (int s = 0; s < ps.n; ++s) {
            const float4 pa = *reinterpret_cast<const float4*>(at + (size_t)s * ps.stride);
            const float4 pb = *reinterpret_cast<const float4*>(at + (size_t)s * ps.stride + half);
            a.x += pa.x; a.y += pa.y; a.z += pa.z; a.w += pa.w;
            b.x += pb.x; b.y += pb.y; b.z += pb.z; b.w += pb.w;
        }
        lo[0] = to_float(from_float<bf16_t>(a.x)); lo[1] = to_float(from_float<bf16_t>(a.y));
        lo[2] = to_float(from_float<bf16_t>(a.z)); lo[3] = to_float(from_float<bf16_t>(a.w));
        hi[0] = to_float(from_float<bf16_t>(b.x)); hi[1] = to_float(from_float<bf16_t>(b.y));
        hi[2] = to_float(from_float<bf16_t>(b.z)); hi[3] = to_float(from_float<bf16_t>(b.w));
    } else {
        const bf16_t* src = qkv + (size_t)t * total + (size_t)head * head_dim;
        const uint2 lo_raw = *reinterpret_cast<const uint2*>(src + i), hi_raw = *reinterpret_cast<const uint2*>(src + i + half);
        lo[0] = __uint_as_float(lo_raw.x << 16); lo[1] = __uint_as_float(lo_raw.x & 0xffff0000u);
        lo[2] = __uint_as_float(lo_raw.y << 16); lo[3] = __uint_as_float(lo_raw.y & 0xffff0000u);
        hi[0] = __uint_as_float(hi_raw.x << 16); hi[1] = __uint_as_float(hi_raw.x & 0xffff0000u);
        hi[2] = __uint_as_float(hi_raw.y << 16); hi[3] = __uint_as_float(hi_raw.y & 0xffff0000u);
    }
    if (bias) {
        const bf16_t* b = bias + (size_t)head * head_dim;
        const uint2 bl = *reinterpret_cast<const uint2*>(b + i), bh = *reinterpret_cast<const uint2*>(b + i + half);
        lo[0] += __uint_as_float(bl.x << 16); lo[1] += __uint_as_float(bl.x & 0xffff0000u);
        lo[2] += __uint_as_float(bl.y << 16); lo[3] += __uint_as_float(bl.y & 0xffff0000u);
        hi[0] += __uint_as_float(bh.x << 16); hi[1] += __uint_as_float(bh.x & 0xffff0000u);
        hi[2] += __uint_as_float(bh.y << 16); hi[3] += __uint_as_float(bh.y & 0xffff0000u);
    }
    if (kind != 2 && pos < max_positions) {
        const float4 c4 = *reinterpret_cast<const float4*>(cos_table + (size_t)pos * half + i);
        const float4 s4 = *reinterpret_cast<const float4*>(sin_table + (size_t)pos * half + i);
        const float c[4] = {c4.x, c4.y, c4.z, c4.w}, sn[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float x0 = lo[k], x1 = hi[k];
            lo[k] = x0 * c[k] - x1 * sn[k];
            hi[k] = x0 * sn[k] + x1 * c[k];
        }
    }
    uint32_t lo_bits[4], hi_bits[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) { lo_bits[k] = float_to_bf16_bits(lo[k]); hi_bits[k] = float_to_bf16_bits(hi[k]); }
    if (kind == 2) {
        // values are kept transposed inside a page: [kv head][head_dim][place of the position]
        const int kvh = head - n_heads - n_kv_heads;
        const int page = page_table[(size_t)tok_seq[t] * table_width + pos / TQK_PAGE];
        if (page < 0) return;                          // the host never lets this happen
        bf16_t* dst = values + ((size_t)page * n_kv_heads + kvh) * TQK_PAGE * head_dim + value_place(pos % TQK_PAGE);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            dst[(size_t)(i + k) * TQK_PAGE].bits = (uint16_t)lo_bits[k];
            dst[(size_t)(i + half + k) * TQK_PAGE].bits = (uint16_t)hi_bits[k];
        }
        return;
    }
    bf16_t* dst;
    if (kind == 0) {
        dst = q_out + ((size_t)t * n_heads + head) * head_dim;
    } else {
        const int page = page_table[(size_t)tok_seq[t] * table_width + pos / TQK_PAGE];
        if (page < 0) return;
        dst = keys + (((size_t)page * n_kv_heads + head - n_heads) * TQK_PAGE + pos % TQK_PAGE) * head_dim;
    }
    *reinterpret_cast<uint2*>(dst + i) = make_uint2(lo_bits[0] | (lo_bits[1] << 16), lo_bits[2] | (lo_bits[3] << 16));
    *reinterpret_cast<uint2*>(dst + i + half) = make_uint2(hi_bits[0] | (hi_bits[1] << 16), hi_bits[2] | (hi_bits[3] << 16));
}

#define STORE_VALUES_MIN_TOKENS 128        // fewer tokens: the plain way costs no more

// Whether the 8-byte kernel takes these (then the product may also come as its sums).
static bool rope_store_vector_case(int act_dtype, const void* bias, int bias_dtype, int rot_dim, int style, int head_dim) {
    return act_dtype == TQK_BF16 && (!bias || bias_dtype == TQK_BF16) && style == 1 && rot_dim == head_dim && head_dim % 8 == 0;
}

static int rope_store(const void* qkv, const PartSums ps, int act_dtype, const void* bias, int bias_dtype,
                      const float* cos_table, const float* sin_table, int rot_dim, int style,
                      int max_positions, const int32_t* tok_seq, const int32_t* tok_pos,
                      const int32_t* page_table, int table_width, int n_seqs, void* keys, void* values,
                      int n_pages, void* q_out, int n_tokens, int n_heads, int n_kv_heads,
                      int head_dim, int write_kv, void* stream) {
    TQK_REQUIRE((qkv || ps.sums) && tok_pos && q_out, "tqk_rope_store: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && head_dim > 0, "tqk_rope_store: bad sizes");
    TQK_REQUIRE(style >= 0 && style <= 2, "tqk_rope_store: unknown rotation style %d", style);
    if (style != 0) {
        TQK_REQUIRE(cos_table && sin_table, "tqk_rope_store: rotation without tables");
        TQK_REQUIRE(rot_dim > 0 && rot_dim % 2 == 0 && rot_dim <= head_dim, "tqk_rope_store: rot_dim %d must be even and <= head_dim %d", rot_dim, head_dim);
        TQK_REQUIRE(max_positions > 0, "tqk_rope_store: empty angle table");
    } else {
        rot_dim = 0;
    }
    if (write_kv) {
        TQK_REQUIRE(keys && values && tok_seq && page_table, "tqk_rope_store: cache write without cache pointers");
        TQK_REQUIRE(table_width > 0 && n_pages > 0 && n_seqs > 0, "tqk_rope_store: empty page table");
    }
    if (n_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (rope_store_vector_case(act_dtype, bias, bias_dtype, rot_dim, style, head_dim) &&
        ((((uintptr_t)qkv) | ((uintptr_t)ps.sums) | ((uintptr_t)bias) | ((uintptr_t)cos_table) | ((uintptr_t)sin_table) |
          ((uintptr_t)keys) | ((uintptr_t)q_out)) & 15) == 0) {
        const int slots = (n_heads + 2 * n_kv_heads) * (head_dim / 8);
        // (lanes along the tokens pay where neighbouring tokens share a page: prompts, not steps of one token per sequence,
        // where 128 sequences took 20 us that way and take 8 the plain way)
        const bool values_apart = write_kv && n_tokens >= STORE_VALUES_MIN_TOKENS && n_tokens >= 8 * n_seqs;
        const int layers = (slots + 255) / 256;
        dim3 vgrid(n_tokens, layers + (values_apart ? 1 : 0));
        rope_store_halves_bf16_kernel<<<vgrid, 256, 0, s>>>(
            (const bf16_t*)qkv, ps, (const bf16_t*)bias, cos_table, sin_table, max_positions, tok_seq, tok_pos, page_table,
            table_width, (bf16_t*)keys, (bf16_t*)values, (bf16_t*)q_out, n_heads, n_kv_heads, head_dim,
            values_apart ? 2 : (write_kv ? 1 : 0), layers, n_tokens);
        return tqk_check_launch("tqk_rope_store");
    }
    TQK_REQUIRE(!ps.sums, "tqk_rope_store_sums: only bfloat16, rotation in halves over the whole head, head_dim a multiple of 8, "
                          "16-byte aligned operands");
    dim3 grid(n_tokens, (n_heads + 2 * n_kv_heads + 3) / 4);
    const int threads = 4 * TQK_WAVE;
#define LAUNCH(TA, TB) rope_store_kernel<TA, TB><<<grid, threads, 0, s>>>( \
        (const TA*)qkv, (const TB*)bias, cos_table, sin_table, rot_dim, style, max_positions, tok_seq, tok_pos, \
        page_table, table_width, (TA*)keys, (TA*)values, (TA*)q_out, n_heads, n_kv_heads, head_dim, write_kv)
    if (act_dtype == TQK_F32 && bias_dtype == TQK_F32) LAUNCH(float, float);
    else if (act_dtype == TQK_F32 && bias_dtype == TQK_BF16) LAUNCH(float, bf16_t);
    else if (act_dtype == TQK_BF16 && bias_dtype == TQK_F32) LAUNCH(bf16_t, float);
    else if (act_dtype == TQK_BF16 && bias_dtype == TQK_BF16) LAUNCH(bf16_t, bf16_t);
    else return tqk_fail("tqk_rope_store: unknown dtypes act=%d bias=%d", act_dtype, bias_dtype);
#undef LAUNCH
    return tqk_check_launch("tqk_rope_store");
}

extern "C" int tqk_rope_store(const void* qkv, int act_dtype, const void* bias, int bias_dtype,
                              const float* cos_table, const float* sin_table, int rot_dim, int style,
                              int max_positions, const int32_t* tok_seq, const int32_t* tok_pos,
                              const int32_t* page_table, int table_width, int n_seqs, void* keys, void* values,
                              int n_pages, void* q_out, int n_tokens, int n_heads, int n_kv_heads,
                              int head_dim, int write_kv, void* stream) {
    return rope_store(qkv, PartSums{nullptr, 0, 0}, act_dtype, bias, bias_dtype, cos_table, sin_table, rot_dim, style, max_positions,
                      tok_seq, tok_pos, page_table, table_width, n_seqs, keys, values, n_pages, q_out, n_tokens, n_heads,
                      n_kv_heads, head_dim, write_kv, stream);
}

/* Whether tqk_rope_store_sums takes this case (bfloat16, bias none or bfloat16, halves over the whole head). */
extern "C" int tqk_rope_store_takes_sums(int act_dtype, int has_bias, int bias_dtype, int rot_dim, int style, int head_dim) {
    return rope_store_vector_case(act_dtype, has_bias ? (const void*)1 : nullptr, bias_dtype, rot_dim, style, head_dim) ? 1 : 0;
}

/* The same with the q, k, v product given as its sums over n_sums pieces of K, float32
 * [n_sums][n_tokens][(heads + 2 kv heads) * head_dim]; bfloat16 activations only. */
extern "C" int tqk_rope_store_sums(const float* sums, int n_sums, const void* bias, int bias_dtype,
                                   const float* cos_table, const float* sin_table, int rot_dim, int style,
                                   int max_positions, const int32_t* tok_seq, const int32_t* tok_pos,
                                   const int32_t* page_table, int table_width, int n_seqs, void* keys, void* values,
                                   int n_pages, void* q_out, int n_tokens, int n_heads, int n_kv_heads,
                                   int head_dim, int write_kv, void* stream) {
    TQK_REQUIRE(sums && n_sums > 0, "tqk_rope_store_sums: no sums given");
    const size_t stride = (size_t)n_tokens * (n_heads + 2 * n_kv_heads) * head_dim;
    return rope_store(nullptr, PartSums{sums, n_sums, stride}, TQK_BF16, bias, bias_dtype, cos_table, sin_table, rot_dim, style,
                      max_positions, tok_seq, tok_pos, page_table, table_width, n_seqs, keys, values, n_pages, q_out, n_tokens,
                      n_heads, n_kv_heads, head_dim, write_kv, stream);
}

// ---- SwiGLU ----------------------------------------------------------------------
// silu(gate) * up, src/models/turbo_generic.rs:105-111 and :64-66.
template <typename TA>
__global__ void swiglu_kernel(const TA* __restrict__ gate_up, TA* __restrict__ out, int inter, size_t total) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t t = i / inter, c = i % inter;
    const float g = to_float(gate_up[t * 2 * inter + c]);
    const float u = to_float(gate_up[t * 2 * inter + inter + c]);
    out[i] = from_float<TA>((g / (1.f + expf(-g))) * u);
}

// The same, 8 bfloat16 values (16 bytes) per thread; inter must be a multiple of 8.
__global__ void swiglu_bf16x8_kernel(const uint4* __restrict__ gate_up, uint4* __restrict__ out, int inter8, size_t total8) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total8) return;
    const size_t t = i / inter8, c = i % inter8;
    const uint4 g4 = gate_up[t * 2 * inter8 + c], u4 = gate_up[t * 2 * inter8 + inter8 + c];
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t ow[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
        const float r0 = (g0 / (1.f + expf(-g0))) * u0, r1 = (g1 / (1.f + expf(-g1))) * u1;
        ow[k] = (uint32_t)float_to_bf16_bits(r0) | ((uint32_t)float_to_bf16_bits(r1) << 16);
    }
    out[i] = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

extern "C" int tqk_swiglu(const void* gate_up, void* out, int act_dtype, int n_tokens, int inter, void* stream) {
    TQK_REQUIRE(gate_up && out, "tqk_swiglu: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && inter > 0, "tqk_swiglu: bad sizes");
    if (n_tokens == 0) return 0;
    const size_t total = (size_t)n_tokens * inter;
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == TQK_BF16 && inter % 8 == 0 && ((((uintptr_t)gate_up) | ((uintptr_t)out)) & 15) == 0) {
        const size_t total8 = total / 8;
        swiglu_bf16x8_kernel<<<(unsigned)((total8 + 255) / 256), 256, 0, s>>>((const uint4*)gate_up, (uint4*)out, inter / 8, total8);
        return tqk_check_launch("tqk_swiglu");
    }
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (act_dtype == TQK_F32) swiglu_kernel<float><<<blocks, 256, 0, s>>>((const float*)gate_up, (float*)out, inter, total);
    else if (act_dtype == TQK_BF16) swiglu_kernel<bf16_t><<<blocks, 256, 0, s>>>((const bf16_t*)gate_up, (bf16_t*)out, inter, total);
    else return tqk_fail("tqk_swiglu: unknown dtype %d", act_dtype);
    return tqk_check_launch("tqk_swiglu");
}
