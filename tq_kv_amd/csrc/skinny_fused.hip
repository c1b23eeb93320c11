// y[M,N] = x[M,K] w[N,K]^T for few rows M (up to 16: decoding steps, chosen logit rows): the
// weights are streamed from HBM exactly once and never staged; bfloat16 in, MFMA, float32
// accumulation.  The reference runs these products as candle matmuls
// (src/models/turbo_generic.rs:68-91); at these M they are bound by the weight bytes, so the
// kernel is laid out for memory, not for the matrix cores.
//
// v_mfma_f32_16x16x32_bf16 computes D[16x16] += A[16x32] B[32x16].  Here A is a tile of w (16
// output features x 32 k) and B a tile of x^T (32 k x 16 rows of x), so D[n][m] is a tile of
// y^T.  Lane l holds, of A, row l%16 and the 8 consecutive k starting at 8*(l/16): 16
// contiguous bytes of a weight row, loaded straight from global memory; of B the same 16
// bytes of x's row l%16; of D column m = l%16 and rows n = 4*(l/16) .. +3.
//
// The weights come as the checkpoint has them, [N, K] row by row, or packed in the order the
// lanes take them: [tile of 16 features][k step of 32][lane][8 values], so that one load
// instruction of a wave reads 1024 contiguous bytes and a tile's whole K is one contiguous
// run.  Rows beyond N in the last tile are zeros; a gated weight's gate rows and up rows are
// packed one after the other, each padded to whole tiles.  Measured at the Qwen2.5-7B sizes
// the packed order is worth 12 % of a decoding layer's time at 8 rows (the 64-byte pieces of
// 16 different rows that a load gathers otherwise keep a compute unit's memory path busier
// than the bytes warrant, and make the time depend on how evenly blocks fall on the units).
//
// A block owns one tile of 16 output features, or a pair of tiles that meet the same x (gate
// and up rows of one output; the two halves of a head that rotate with each other; two
// neighbouring tiles of a very wide product).  Its waves split K between them in chunks and
// add their partial tiles up through LDS in wave order, so the sum has a fixed order whatever
// the timing, and one that depends on the product's shape alone, not on M.
//
// The neighbouring small operations of a decoding step are folded into the kernel's two ends,
// so that a layer takes six kernel launches instead of nine: at these sizes a launch costs
// as much as the work of a norm or a rotation.
//
// The norm between two products is split over them.  RMSNorm is x / rms(x) * weight
// (src/models/turbo_generic.rs:41-51), and the division by the row's rms commutes with
// the product that follows.  So the kernel that adds to the residual stream h (back end
// "residual") also writes xw = bfloat16(h * weight of the next norm) and, per block, the
// sum of h^2 over its 16 columns; the product that consumes the norm (front end "norm")
// takes xw as it is, adds the blocks' sums up in their order, and divides its finished
// sums by sqrt(mean + eps).  The statistics are those of the float32 stream.
//
// Back ends:
//   store     y = result (bfloat16 or float32)
//   gated     rows n and n_out + n of w are gate and up: y = silu(gate) * up
//             (src/models/turbo_generic.rs:105-111)
//   residual  h += bfloat16(result) in float32: the residual sum of
//             src/models/turbo_generic.rs:1969, :1980; xw and the sums of squares as above
//   qkv       rows are q heads, k heads, v heads of head_dim each; bias, rotation in the
//             halves layout at the row's position (src/models/turbo_generic.rs:805-833,
//             :417-427), q to q_out, k and v into the row's cache page
//
// Rounding points are those of the separate kernels (products rounded to bfloat16
// before bias, rotation, gate or residual sum), so a decoded token and a prompt token
// go through the same roundings except for the place of the norm's division.
#include "common.h"
#include "tq_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

__device__ __forceinline__ bf16x8_t load8f(const bf16_t* p) {
    return *reinterpret_cast<const bf16x8_t*>(p);
}
// the weights: read once and never again, so the load says so (a plain streaming read of a gigabyte runs at
// 7.0 TB/s with this hint and at 6.2 without it on an MI355X)
__device__ __forceinline__ bf16x8_t load8w(const bf16_t* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(p));
}

enum { EPI_STORE = 0, EPI_GATED = 1, EPI_RESIDUAL = 2, EPI_QKV = 3 };

struct FusedArgs {
    const bf16_t* x;            // [rows of x, K]
    const int32_t* x_rows;      // row m of the product reads x row x_rows[m] (null: m)
    const float* ss_parts;      // [n_ss_parts, 16] sums of squares of x's rows, in pieces (front end "norm")
    int n_ss_parts;
    float eps;
    const bf16_t* w;            // [N, K], or packed (see below)
    int w_packed;
    int M, N, K;
    // store / gated
    void* y;
    // residual
    float* h;                   // [M, N]
    const bf16_t* next_norm_w;  // [N] weight of the norm that follows, or null
    bf16_t* xw_out;             // [M, N] bfloat16(h * next_norm_w), or bfloat16(h) without a weight
    float* ss_out;              // [blocks, 16] this block's sum of h^2 per row, or null
    // qkv
    const bf16_t* bias;         // [N] or null
    const float* cos_table;     // [max_positions, head_dim/2]
    const float* sin_table;
    const int32_t* tok_pos;     // [M]
    const int32_t* page_table;  // [M, table_width]: row m is sequence m
    int table_width, n_heads, n_kv_heads, head_dim, max_positions;
    bf16_t* q_out;              // [M, n_heads, head_dim]
    bf16_t* keys;               // [pages, kv heads, 64, head_dim]
    bf16_t* values;             // [pages, kv heads, head_dim, 64 places]
};


// RT: tiles of 16 output features next to each other per block, for the back ends "store" and
// "residual" (gated and qkv blocks always hold a pair of tiles).  All tiles of a block meet
// the same values of x, so x is read RT times less often.
template <bool NORM, int EPI, typename TY, bool GATHER, int RT>
__global__ __launch_bounds__(1024)
void skinny_fused_kernel(const FusedArgs p) {
    extern __shared__ float red[];                 // [waves][TILES * 4][64 lanes], then [waves][4 lanes] float4 of squares
    constexpr bool PAIR = EPI == EPI_GATED || EPI == EPI_QKV;
    static_assert(!PAIR || RT == 1, "gated and qkv blocks hold one pair of tiles");
    constexpr int TILES = PAIR ? 2 : RT;
    constexpr int SLOTS = TILES * 4;
    constexpr int SF_UNROLL = 4;                   // k steps of 32 whose loads are under way together
    const int lane = threadIdx.x % TQK_WAVE, wave = threadIdx.x / TQK_WAVE;
    const int n_waves = blockDim.x / TQK_WAVE;
    const int row = lane % 16, kgrp = lane / 16;
    const int K = p.K;

    // which rows of w: n_lo (and n_hi for the second tile)
    int n_lo0, n_hi0, n_out;
    int head = 0, j16 = 0;
    if (EPI == EPI_QKV) {
        const int tiles_per_head = p.head_dim / 32;             // pairs of tiles (lo half, hi half)
        head = blockIdx.x / tiles_per_head;
        j16 = (blockIdx.x % tiles_per_head) * 16;
        n_lo0 = head * p.head_dim + j16;
        n_hi0 = n_lo0 + p.head_dim / 2;
        n_out = p.N;
    } else if (EPI == EPI_GATED) {
        n_out = p.N / 2;
        n_lo0 = blockIdx.x * 16;
        n_hi0 = n_out + n_lo0;
    } else {
        n_out = p.N;
        n_lo0 = blockIdx.x * 16 * RT;
        n_hi0 = 0;
    }
    // The lane's 16 bytes of tile t at k step s lie at wrow[t] + 32 * s * kmul.
    const bf16_t* wrow[TILES];
    int kmul = 1;
    if (p.w_packed) {
        kmul = 16;
        const size_t tile_size = (size_t)(K / 32) * 512;
        if (PAIR) {
            wrow[0] = p.w + (size_t)(n_lo0 / 16) * tile_size + lane * 8;
            wrow[TILES - 1] = p.w + (size_t)(EPI == EPI_GATED ? (n_out + 15) / 16 + n_lo0 / 16 : n_hi0 / 16) * tile_size + lane * 8;
        } else {
#pragma unroll
            for (int t = 0; t < TILES; ++t) wrow[t] = p.w + (size_t)min(n_lo0 / 16 + t, (p.N + 15) / 16 - 1) * tile_size + lane * 8;
        }
    } else {
        const int n_clamp = (EPI == EPI_GATED) ? n_out - 1 : p.N - 1;
        if (PAIR) {
            wrow[0] = p.w + (size_t)min(n_lo0 + row, n_clamp) * K + kgrp * 8;
            wrow[TILES - 1] = p.w + (size_t)(EPI == EPI_GATED ? n_out + min(n_lo0 + row, n_clamp) : n_hi0 + row) * K + kgrp * 8;
        } else {
#pragma unroll
            for (int t = 0; t < TILES; ++t) wrow[t] = p.w + (size_t)min(n_lo0 + 16 * t + row, n_clamp) * K + kgrp * 8;
        }
    }

    // Column m of the result depends on row m of x alone, so the lanes of rows past M read
    // row 0 and their results are dropped.
    const int xr = row < p.M ? (GATHER ? p.x_rows[row] : row) : 0;
    const bf16_t* xrow = p.x + (size_t)xr * K + kgrp * 8;

    // The sums of squares [n_ss_parts, 16 rows] as float4s: thread t takes the float4s t, t + threads, ...,
    // which all hold rows 4*(t%4) .. +3.  The first is asked for here and used after the product.
    const int n_ss4 = NORM ? p.n_ss_parts * 4 : 0;
    const float4* ss4 = reinterpret_cast<const float4*>(p.ss_parts);
    float4 ssq = make_float4(0.f, 0.f, 0.f, 0.f);
    __builtin_amdgcn_sched_barrier(0);              // after the row's address is known: no wait covers this load
    if (NORM && (int)threadIdx.x < n_ss4) ssq = ss4[threadIdx.x];

    floatx4_t acc[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) acc[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    const int chunk = SF_UNROLL * 32;
    const int n_chunks = K / chunk;
    auto multiply_chunk = [&](const bf16x8_t (&a)[TILES][SF_UNROLL], const bf16x8_t (&bx)[SF_UNROLL]) {
#pragma unroll
        for (int u = 0; u < SF_UNROLL; ++u)
#pragma unroll
            for (int t = 0; t < TILES; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][u], bx[u], acc[t], 0, 0, 0);
    };

    // The first chunk stands apart: what the back end needs beside the product (the stream's
    // values and the next norm's weight; or the page, the angles and the bias at the row's
    // position) is asked for right behind its loads and looked at after the product, so it
    // arrives meanwhile.  Nothing here is under a condition, so that the waits can be counted:
    // lanes and blocks that need nothing load from a valid place and drop it.  With K below a
    // chunk (a wave then has no whole chunk) the first chunk's loads stay inside the row and
    // meet zeros.
    const int m = row, nb = 4 * kgrp;
    const int ml = m < p.M ? m : 0;
    float4 pre_f0[TILES], pre_f1 = make_float4(0.f, 0.f, 0.f, 0.f);
    uint2 pre_h0[TILES], pre_h1 = make_uint2(0, 0);
#pragma unroll
    for (int t = 0; t < TILES; ++t) { pre_f0[t] = pre_f1; pre_h0[t] = pre_h1; }
    int pos = 0, page = -1;
    if (EPI == EPI_QKV) pos = p.tok_pos[ml];
    {
        bf16x8_t a[TILES][SF_UNROLL], bx[SF_UNROLL];
        const bool whole = n_chunks > 0;            // then every wave has a first chunk: waves <= chunks
#pragma unroll
        for (int u = 0; u < SF_UNROLL; ++u) {
            const int k0 = min(wave * chunk + u * 32, K - 32);
#pragma unroll
            for (int t = 0; t < TILES; ++t) a[t][u] = load8w(wrow[t] + (size_t)k0 * kmul);
            bx[u] = load8f(xrow + k0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (EPI == EPI_RESIDUAL) {
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                const int n = min(n_lo0 + 16 * t + nb, p.N - 4);
                pre_f0[t] = *reinterpret_cast<const float4*>(p.h + (size_t)ml * p.N + n);
                pre_h0[t] = *reinterpret_cast<const uint2*>(p.next_norm_w ? p.next_norm_w + n : p.w);
            }
        }
        if (EPI == EPI_QKV) {
            const int half = p.head_dim / 2, i_lo = j16 + nb;
            page = p.page_table[(size_t)ml * p.table_width + pos / TQK_PAGE];
            const size_t angle = (size_t)min(pos, p.max_positions - 1) * half + i_lo;
            pre_f0[0] = *reinterpret_cast<const float4*>(p.cos_table + angle);
            pre_f1 = *reinterpret_cast<const float4*>(p.sin_table + angle);
            pre_h0[0] = *reinterpret_cast<const uint2*>(p.bias ? p.bias + head * p.head_dim + i_lo : p.w);
            pre_h1 = *reinterpret_cast<const uint2*>(p.bias ? p.bias + head * p.head_dim + i_lo + half : p.w);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (!whole) {
            const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int u = 0; u < SF_UNROLL; ++u) bx[u] = zero;
        }
        multiply_chunk(a, bx);
    }
    for (int c = wave + n_waves; c < n_chunks; c += n_waves) {
        bf16x8_t a[TILES][SF_UNROLL], bx[SF_UNROLL];
        const int k0 = c * chunk;
#pragma unroll
        for (int u = 0; u < SF_UNROLL; ++u) {
#pragma unroll
            for (int t = 0; t < TILES; ++t) a[t][u] = load8w(wrow[t] + (size_t)(k0 + u * 32) * kmul);
            bx[u] = load8f(xrow + k0 + u * 32);
        }
        __builtin_amdgcn_sched_barrier(0);          // every load of the chunk is on its way before the first product waits
        multiply_chunk(a, bx);
    }
    for (int s = n_chunks * SF_UNROLL + wave; s < K / 32; s += n_waves) {
        const int k0 = s * 32;
        const bf16x8_t bxs = load8f(xrow + k0);
#pragma unroll
        for (int t = 0; t < TILES; ++t)
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(load8w(wrow[t] + (size_t)k0 * kmul), bxs, acc[t], 0, 0, 0);
    }

    if (NORM) {
        for (int i = threadIdx.x + blockDim.x; i < n_ss4; i += blockDim.x) {
            const float4 v = ss4[i];
            ssq.x += v.x; ssq.y += v.y; ssq.z += v.z; ssq.w += v.w;
        }
        // lanes with equal lane%4 hold the same rows: add them up, fixed order
#pragma unroll
        for (int d = 4; d < TQK_WAVE; d *= 2) {
            ssq.x += __shfl_xor(ssq.x, d, TQK_WAVE);
            ssq.y += __shfl_xor(ssq.y, d, TQK_WAVE);
            ssq.z += __shfl_xor(ssq.z, d, TQK_WAVE);
            ssq.w += __shfl_xor(ssq.w, d, TQK_WAVE);
        }
    }

    // add the waves' partial tiles up in wave order
    if (n_waves > 1) {
        float* mine = red + (size_t)wave * SLOTS * TQK_WAVE;
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) mine[(t * 4 + r) * TQK_WAVE + lane] = acc[t][r];
        if (NORM && lane < 4) reinterpret_cast<float4*>(red + (size_t)n_waves * SLOTS * TQK_WAVE)[wave * 4 + lane] = ssq;
        __syncthreads();
        if (wave != 0) return;
        for (int ww = 1; ww < n_waves; ++ww) {
            const float* theirs = red + (size_t)ww * SLOTS * TQK_WAVE;
#pragma unroll
            for (int t = 0; t < TILES; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[t][r] += theirs[(t * 4 + r) * TQK_WAVE + lane];
            if (NORM) {
                const float4 v = reinterpret_cast<const float4*>(red + (size_t)n_waves * SLOTS * TQK_WAVE)[ww * 4 + lane % 4];
                ssq.x += v.x; ssq.y += v.y; ssq.z += v.z; ssq.w += v.w;
            }
        }
    }

    // the lane holds column m = row of the result, for features n0 + 4*kgrp + r
    float inv_rms = 1.f;
    if (NORM) {
        // the lanes l with l%4 == xr/4 hold row xr's sum of squares in component xr%4
        const float s0 = __shfl(ssq.x, xr / 4, TQK_WAVE), s1 = __shfl(ssq.y, xr / 4, TQK_WAVE);
        const float s2 = __shfl(ssq.z, xr / 4, TQK_WAVE), s3 = __shfl(ssq.w, xr / 4, TQK_WAVE);
        const float ss = (xr & 2) ? ((xr & 1) ? s3 : s2) : ((xr & 1) ? s1 : s0);
        inv_rms = 1.f / sqrtf(ss / (float)K + p.eps);
    }
    if (m >= p.M && EPI != EPI_RESIDUAL) return;

    if constexpr (EPI == EPI_STORE) {
        TY* y = (TY*)p.y;
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = n_lo0 + 16 * t + nb + r;
                if (n < p.N) y[(size_t)m * p.N + n] = from_float<TY>(acc[t][r] * inv_rms);
            }
    } else if constexpr (EPI == EPI_GATED) {
        bf16_t* y = (bf16_t*)p.y;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int n = n_lo0 + nb + r;
            if (n >= n_out) continue;
            const float g = to_float(from_float<bf16_t>(acc[0][r] * inv_rms));
            const float up = to_float(from_float<bf16_t>(acc[1][r] * inv_rms));
            y[(size_t)m * n_out + n] = from_float<bf16_t>((g / (1.f + expf(-g))) * up);
        }
    } else if constexpr (EPI == EPI_RESIDUAL) {
        float sq = 0.f;
        if (m < p.M) {
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                const float pre_h[4] = {pre_f0[t].x, pre_f0[t].y, pre_f0[t].z, pre_f0[t].w};
                const float pre_w[4] = {__uint_as_float(pre_h0[t].x << 16), __uint_as_float(pre_h0[t].x & 0xffff0000u),
                                        __uint_as_float(pre_h0[t].y << 16), __uint_as_float(pre_h0[t].y & 0xffff0000u)};
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int n = n_lo0 + 16 * t + nb + r;
                    if (n >= p.N) continue;
                    const size_t at = (size_t)m * p.N + n;
                    const float v = pre_h[r] + to_float(from_float<bf16_t>(acc[t][r]));
                    p.h[at] = v;
                    sq = fmaf(v, v, sq);
                    p.xw_out[at] = from_float<bf16_t>(p.next_norm_w ? v * pre_w[r] : v);
                }
            }
        }
        if (p.ss_out) {
            // this block's columns of row m: the four lanes of the row, in lane order
            const float s1 = __shfl_xor(sq, 16, TQK_WAVE);
            const float s2 = __shfl_xor(sq, 32, TQK_WAVE);
            const float s3 = __shfl_xor(s1, 32, TQK_WAVE);
            if (kgrp == 0 && m < p.M) p.ss_out[(size_t)blockIdx.x * 16 + m] = ((sq + s1) + s2) + s3;
        }
    } else {    // EPI_QKV
        const int d = p.head_dim, half = d / 2;
        const int kind = head < p.n_heads ? 0 : (head < p.n_heads + p.n_kv_heads ? 1 : 2);
        bf16_t* dst;
        size_t stride = 1;
        if (kind == 0) {
            dst = p.q_out + ((size_t)m * p.n_heads + head) * d;
        } else {
            const int kvh = kind == 1 ? head - p.n_heads : head - p.n_heads - p.n_kv_heads;
            if (page < 0) return;                   // the host never lets this happen
            const size_t base = ((size_t)page * p.n_kv_heads + kvh) * TQK_PAGE * d;
            if (kind == 1) dst = p.keys + base + (size_t)(pos % TQK_PAGE) * d;
            else { dst = p.values + base + value_place(pos % TQK_PAGE); stride = TQK_PAGE; }
        }
        const bool rotate = kind != 2 && pos < p.max_positions;
        const float pre_cos[4] = {pre_f0[0].x, pre_f0[0].y, pre_f0[0].z, pre_f0[0].w}, pre_sin[4] = {pre_f1.x, pre_f1.y, pre_f1.z, pre_f1.w};
        const float bias_lo[4] = {__uint_as_float(pre_h0[0].x << 16), __uint_as_float(pre_h0[0].x & 0xffff0000u),
                                  __uint_as_float(pre_h0[0].y << 16), __uint_as_float(pre_h0[0].y & 0xffff0000u)};
        const float bias_hi[4] = {__uint_as_float(pre_h1.x << 16), __uint_as_float(pre_h1.x & 0xffff0000u),
                                  __uint_as_float(pre_h1.y << 16), __uint_as_float(pre_h1.y & 0xffff0000u)};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int i_lo = j16 + nb + r, i_hi = i_lo + half;          // elements inside the head
            float lo = to_float(from_float<bf16_t>(acc[0][r] * inv_rms));
            float hi = to_float(from_float<bf16_t>(acc[1][r] * inv_rms));
            if (p.bias) {
                lo += bias_lo[r];
                hi += bias_hi[r];
            }
            if (rotate) {
                const float c = pre_cos[r], sn = pre_sin[r];
                const float r0 = lo * c - hi * sn, r1 = lo * sn + hi * c;
                lo = r0; hi = r1;
            }
            dst[(size_t)i_lo * stride] = from_float<bf16_t>(lo);
            dst[(size_t)i_hi * stride] = from_float<bf16_t>(hi);
        }
    }
}

// (17 to 32 rows through this kernel, two groups of 16 rows per wave against the same weights, were built and taken
// out again: every wave then reads twice as much of x beside its weights, and the products took 57.6 us (o + down),
// 56.5 us (gate + up) and 16.3 us (q/k/v) at the 7B sizes against 34.7, 48.7 and 12.0 with up to 16 rows; the kernels
// that stage x in LDS once per block, mid_product.hip, are the better way for those steps in spite of their eight
// launches a layer.)

// Tiles per block for the back ends "store" and "residual", from the product's shape alone
// (never from M: a row's sums then have one order in every batch).  Two tiles halve the
// reads of x, but also the number of blocks, and a block keeps one compute unit busy:
// measured, a pair pays only where there are thousands of blocks left (the vocabulary's product).
static int pick_tiles(int N, int K) {
    (void)K;
    return N / 32 >= 2048 ? 2 : 1;
}

// Waves per block, which split K between them: about a thousand waves on the chip keep HBM
// busy; no more than there are chunks of K to share out; a power of two.  (Two and four thousand
// waves, so that a wave has two rounds of loads instead of four, were measured no faster on the
// q/k/v and o products of the 7B sizes and slower on the down product.)
static int pick_waves(int blocks, int K, int tiles) {
    const int chunks = K / (4 * 32) > 0 ? K / (4 * 32) : 1;
    const int max_waves = tiles >= 2 ? 8 : 16;
    int waves = 1;
    while (waves < max_waves && blocks * waves < 1024 && waves * 2 <= chunks) waves *= 2;
    return waves;
}

template <bool NORM, int EPI, typename TY, bool GATHER = false, int RT = 1>
static int launch_fused(const FusedArgs& a, int blocks, hipStream_t s) {
    const int tiles = (EPI == EPI_GATED || EPI == EPI_QKV) ? 2 : RT;
    const int waves = pick_waves(blocks, a.K, tiles);
    const size_t lds = waves > 1 ? (size_t)waves * (tiles * 4) * TQK_WAVE * sizeof(float) + (NORM ? (size_t)waves * 16 * sizeof(float) : 0) : 0;
    skinny_fused_kernel<NORM, EPI, TY, GATHER, RT><<<blocks, waves * TQK_WAVE, lds, s>>>(a);
    return tqk_check_launch("tqk_skinny_fused");
}

// the same for 1 or 2 tiles per block
template <bool NORM, int EPI, typename TY, bool GATHER = false>
static int launch_tiled(const FusedArgs& a, hipStream_t s) {
    const int rt = pick_tiles(a.N, a.K);
    const int blocks = (a.N + 16 * rt - 1) / (16 * rt);
    if (rt == 2) return launch_fused<NORM, EPI, TY, GATHER, 2>(a, blocks, s);
    return launch_fused<NORM, EPI, TY, GATHER, 1>(a, blocks, s);
}

static int check_common(const FusedArgs& a, const char* what) {
    TQK_REQUIRE(a.x && a.w, "%s: null pointer", what);
    TQK_REQUIRE(a.M >= 0 && a.M <= 16, "%s: M=%d rows, this kernel takes at most 16", what, a.M);
    TQK_REQUIRE(a.N > 0 && a.K > 0 && a.K % 32 == 0, "%s: K=%d must be a positive multiple of 32 (N=%d)", what, a.K, a.N);
    TQK_REQUIRE((((uintptr_t)a.x) & 15) == 0 && (((uintptr_t)a.w) & 15) == 0, "%s: x and w must be 16-byte aligned", what);
    TQK_REQUIRE(!a.ss_parts || a.n_ss_parts > 0, "%s: sums of squares given in %d pieces", what, a.n_ss_parts);
    TQK_REQUIRE((((uintptr_t)a.ss_parts) & 15) == 0, "%s: the sums of squares must be 16-byte aligned", what);
    return 0;
}

/* y[M,N] = x w^T, or with ss_parts (the sums of squares of the stream's rows in n_ss_parts
 * pieces of 16 rows each; x is then the stream times the norm's weight) that divided by
 * sqrt(sum / K + eps).  x_rows (optional) picks the rows of x. */
extern "C" int tqk_skinny_max_rows(void) { return 16; }

extern "C" int tqk_fused_store(const void* x, const int32_t* x_rows, const float* ss_parts, int n_ss_parts, float eps,
                               const void* w, int w_packed, void* y, int y_dtype, int M, int N, int K, void* stream) {
    FusedArgs a = {};
    a.x = (const bf16_t*)x; a.x_rows = x_rows; a.ss_parts = ss_parts; a.n_ss_parts = n_ss_parts; a.eps = eps;
    a.w = (const bf16_t*)w; a.w_packed = w_packed; a.M = M; a.N = N; a.K = K; a.y = y;
    if (check_common(a, "tqk_fused_store")) return -1;
    TQK_REQUIRE(y, "tqk_fused_store: null output");
    TQK_REQUIRE(y_dtype == TQK_F32 || y_dtype == TQK_BF16, "tqk_fused_store: unknown output dtype %d", y_dtype);
    if (M == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (x_rows) {
        if (ss_parts) return y_dtype == TQK_F32 ? launch_tiled<true, EPI_STORE, float, true>(a, s) : launch_tiled<true, EPI_STORE, bf16_t, true>(a, s);
        return y_dtype == TQK_F32 ? launch_tiled<false, EPI_STORE, float, true>(a, s) : launch_tiled<false, EPI_STORE, bf16_t, true>(a, s);
    }
    if (ss_parts) return y_dtype == TQK_F32 ? launch_tiled<true, EPI_STORE, float>(a, s) : launch_tiled<true, EPI_STORE, bf16_t>(a, s);
    return y_dtype == TQK_F32 ? launch_tiled<false, EPI_STORE, float>(a, s) : launch_tiled<false, EPI_STORE, bf16_t>(a, s);
}

/* y[M, N/2] = silu(gate) * up of the (normalised) product, w = gate rows then up rows. */
extern "C" int tqk_fused_gated(const void* x, const float* ss_parts, int n_ss_parts, float eps, const void* w, int w_packed, void* y,
                               int M, int N, int K, void* stream) {
    FusedArgs a = {};
    a.x = (const bf16_t*)x; a.ss_parts = ss_parts; a.n_ss_parts = n_ss_parts; a.eps = eps; a.w = (const bf16_t*)w; a.w_packed = w_packed;
    a.M = M; a.N = N; a.K = K; a.y = y;
    if (check_common(a, "tqk_fused_gated")) return -1;
    TQK_REQUIRE(y && N % 2 == 0, "tqk_fused_gated: null output or odd N=%d", N);
    if (M == 0) return 0;
    const int blocks = (N / 2 + 15) / 16;
    hipStream_t s = (hipStream_t)stream;
    return ss_parts ? launch_fused<true, EPI_GATED, bf16_t>(a, blocks, s) : launch_fused<false, EPI_GATED, bf16_t>(a, blocks, s);
}

extern "C" int tqk_fused_residual_parts(int N, int K) {
    const int rt = pick_tiles(N, K);
    return (N + 16 * rt - 1) / (16 * rt);
}

/* h[M,N] += bfloat16(x w^T) in float32; xw_out = bfloat16(h * next_norm_w) (bfloat16(h)
 * without a weight); ss_out (optional) [tqk_fused_residual_parts(N, K), 16]: piece b, row m =
 * the sum of h[m, n]^2 over the columns n of block b. */
extern "C" int tqk_fused_residual(const void* x, const void* w, int w_packed, float* h, const void* next_norm_w, void* xw_out,
                                  float* ss_out, int M, int N, int K, void* stream) {
    FusedArgs a = {};
    a.x = (const bf16_t*)x; a.w = (const bf16_t*)w; a.w_packed = w_packed; a.M = M; a.N = N; a.K = K; a.h = h;
    a.next_norm_w = (const bf16_t*)next_norm_w; a.xw_out = (bf16_t*)xw_out; a.ss_out = ss_out;
    if (check_common(a, "tqk_fused_residual")) return -1;
    TQK_REQUIRE(h && xw_out, "tqk_fused_residual: null output");
    TQK_REQUIRE(N % 4 == 0, "tqk_fused_residual: N=%d must be a multiple of 4", N);
    TQK_REQUIRE(((((uintptr_t)h) | ((uintptr_t)next_norm_w)) & 15) == 0, "tqk_fused_residual: h and the norm's weight must be 16-byte aligned");
    if (M == 0) return 0;
    return launch_tiled<false, EPI_RESIDUAL, bf16_t>(a, (hipStream_t)stream);
}

/* The q, k, v product of a decoding step: the (normalised) product + bias, q and k rotated
 * (halves layout over the whole head) at tok_pos[m], q to q_out, k and v into the page of
 * row m's sequence (row m of page_table).  head_dim must be a multiple of 32. */
extern "C" int tqk_fused_qkv(const void* x, const float* ss_parts, int n_ss_parts, float eps, const void* w, int w_packed, const void* bias,
                             const float* cos_table, const float* sin_table, int max_positions,
                             const int32_t* tok_pos, const int32_t* page_table, int table_width,
                             void* keys, void* values, int n_pages, void* q_out,
                             int M, int n_heads, int n_kv_heads, int head_dim, int K, void* stream) {
    FusedArgs a = {};
    a.x = (const bf16_t*)x; a.ss_parts = ss_parts; a.n_ss_parts = n_ss_parts; a.eps = eps; a.w = (const bf16_t*)w; a.w_packed = w_packed;
    a.M = M; a.N = (n_heads + 2 * n_kv_heads) * head_dim; a.K = K;
    a.bias = (const bf16_t*)bias; a.cos_table = cos_table; a.sin_table = sin_table; a.max_positions = max_positions;
    a.tok_pos = tok_pos; a.page_table = page_table; a.table_width = table_width;
    a.n_heads = n_heads; a.n_kv_heads = n_kv_heads; a.head_dim = head_dim;
    a.q_out = (bf16_t*)q_out; a.keys = (bf16_t*)keys; a.values = (bf16_t*)values;
    TQK_REQUIRE(n_heads > 0 && n_kv_heads > 0 && head_dim > 0 && head_dim % 32 == 0,
                "tqk_fused_qkv: head_dim %d must be a positive multiple of 32", head_dim);
    if (check_common(a, "tqk_fused_qkv")) return -1;
    TQK_REQUIRE(cos_table && sin_table && max_positions > 0 && tok_pos && page_table && keys && values && q_out,
                "tqk_fused_qkv: null pointer");
    TQK_REQUIRE(table_width > 0 && n_pages > 0, "tqk_fused_qkv: empty page table");
    TQK_REQUIRE(((((uintptr_t)cos_table) | ((uintptr_t)sin_table) | ((uintptr_t)bias)) & 15) == 0,
                "tqk_fused_qkv: the angle tables and the bias must be 16-byte aligned");
    if (M == 0) return 0;
    const int blocks = (n_heads + 2 * n_kv_heads) * (head_dim / 32);
    hipStream_t s = (hipStream_t)stream;
    return ss_parts ? launch_fused<true, EPI_QKV, bf16_t>(a, blocks, s) : launch_fused<false, EPI_QKV, bf16_t>(a, blocks, s);
}
