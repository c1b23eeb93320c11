// y[M,N] = x[M,K] w[N,K]^T for few rows M (decoding, chosen logit rows): the weights
// are streamed from HBM exactly once and never staged; bfloat16 in, MFMA, float32
// accumulation.  The reference runs these products as candle matmuls
// (src/models/turbo_generic.rs:68-91); at M of 1 to 64 they are bound by the weight
// bytes, so the kernel is laid out for memory, not for the matrix cores.
//
// v_mfma_f32_16x16x32_bf16 computes D[16x16] += A[16x32] B[32x16].  Here A is a tile
// of w (16 output features x 32 k) and B a tile of x^T (32 k x 16 rows of x), so
// D[n][m] is a tile of y^T.  Lane l holds, of A, row l%16 and the 8 consecutive k
// starting at 8*(l/16): 16 contiguous bytes of a weight row, loaded straight from
// global memory; of B the same 16 bytes of x's row l%16; of D column m = l%16 and
// rows n = 4*(l/16) .. +3.
//
// A block owns one tile of 16 output features (for the gated epilogue: 16 gate rows
// and the 16 up rows that belong to them), or four neighbouring tiles when x has more
// than 16 rows.  Its waves split K between them in chunks and add their partial tiles
// up through LDS in wave order, so the sum has a fixed order whatever the timing.
// Rows of x beyond M are fed as zeros.
#include "common.h"
#include "tq_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

#define SK_UNROLL 4

__device__ __forceinline__ bf16x8_t load8(const bf16_t* p) {
    return *reinterpret_cast<const bf16x8_t*>(p);
}

template <int MB, int RT, bool GATED, typename TY>
__global__ __launch_bounds__(MB == 1 ? 1024 : 256)
void skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, TY* __restrict__ y,
                   int M, int N, int K, int n_out) {
    extern __shared__ float red[];                 // [waves][tiles][MB][64 lanes][4]
    // RT tiles of 16 output features per block, next to each other; gated: each with its up rows
    constexpr int TILES = RT * (GATED ? 2 : 1);
    constexpr int UNR = (MB == 1 && RT == 1) ? SK_UNROLL : SK_UNROLL / 2;
    const int lane = threadIdx.x % TQK_WAVE, wave = threadIdx.x / TQK_WAVE;
    const int n_waves = blockDim.x / TQK_WAVE;
    const int row = lane % 16, kgrp = lane / 16;
    const int n0 = blockIdx.x * 16 * RT;

    // weight rows of this lane (clamped: rows past the end are computed and not stored)
    const bf16_t* wrow[TILES];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        const int n = min(n0 + r * 16 + row, n_out - 1);
        wrow[r] = w + (size_t)n * K + kgrp * 8;
        if (GATED) wrow[RT + r] = w + (size_t)(n_out + n) * K + kgrp * 8;
    }
    // rows of x of this lane, one per block of 16
    const bf16_t* xrow[MB];
    bool xlive[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const int m = b * 16 + row;
        xlive[b] = m < M;
        xrow[b] = x + (size_t)(xlive[b] ? m : 0) * K + kgrp * 8;
    }

    floatx4_t acc[TILES][MB];
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int b = 0; b < MB; ++b) acc[t][b] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const int chunk = UNR * 32;
    const int n_chunks = K / chunk;
    for (int c = wave; c < n_chunks; c += n_waves) {
        const int k0 = c * chunk;
        bf16x8_t a[TILES][UNR], bx[MB][UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
#pragma unroll
            for (int t = 0; t < TILES; ++t) a[t][u] = load8(wrow[t] + k0 + u * 32);
#pragma unroll
            for (int b = 0; b < MB; ++b) bx[b][u] = xlive[b] ? load8(xrow[b] + k0 + u * 32) : zero;
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u)
#pragma unroll
            for (int t = 0; t < TILES; ++t)
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][u], bx[b][u], acc[t][b], 0, 0, 0);
    }
    // the steps of 32 that do not fill a chunk
    for (int s = n_chunks * UNR + wave; s < K / 32; s += n_waves) {
        const int k0 = s * 32;
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            const bf16x8_t at = load8(wrow[t] + k0);
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                const bf16x8_t bt = xlive[b] ? load8(xrow[b] + k0) : zero;
                acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(at, bt, acc[t][b], 0, 0, 0);
            }
        }
    }

    // add the waves' partial tiles up in wave order
    if (n_waves > 1) {
        float* mine = red + (size_t)wave * TILES * MB * TQK_WAVE * 4;
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int b = 0; b < MB; ++b)
#pragma unroll
                for (int r = 0; r < 4; ++r) mine[((t * MB + b) * 4 + r) * TQK_WAVE + lane] = acc[t][b][r];
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int b = 0; b < MB; ++b)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float s = acc[t][b][r];
                    for (int ww = 1; ww < n_waves; ++ww)
                        s += red[(size_t)ww * TILES * MB * TQK_WAVE * 4 + ((t * MB + b) * 4 + r) * TQK_WAVE + lane];
                    acc[t][b][r] = s;
                }
    }

    // store: lane holds y[m = b*16 + row][n0 + rt*16 + 4*kgrp + r]
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const int m = b * 16 + row;
        if (m >= M) continue;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = n0 + rt * 16 + 4 * kgrp + r;
                if (n >= n_out) continue;
                float v = acc[rt][b][r];
                if (GATED) {
                    // gate and up are rounded to bfloat16 first, as when they are stored and read back
                    const float g = to_float(from_float<bf16_t>(v));
                    const float up = to_float(from_float<bf16_t>(acc[RT + rt][b][r]));
                    v = (g / (1.f + expf(-g))) * up;
                }
                y[(size_t)m * n_out + n] = from_float<TY>(v);
            }
    }
}

template <int MB, int RT>
static int launch_mb(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, int epilogue,
                     int waves, hipStream_t s) {
    const int n_out = epilogue ? N / 2 : N;
    constexpr int RTG = RT > 1 ? RT / 2 : 1;       // gated blocks hold half as many tiles, each with its up rows
    const int tiles = epilogue ? 2 * RTG : RT;
    const unsigned blocks = (unsigned)((n_out + 16 * (epilogue ? RTG : RT) - 1) / (16 * (epilogue ? RTG : RT)));
    const size_t lds = waves > 1 ? (size_t)waves * tiles * MB * TQK_WAVE * 4 * sizeof(float) : 0;
    const bf16_t* xp = (const bf16_t*)x;
    const bf16_t* wp = (const bf16_t*)w;
    if (epilogue) {
        skinny_kernel<MB, RTG, true, bf16_t><<<blocks, waves * TQK_WAVE, lds, s>>>(xp, wp, (bf16_t*)y, M, N, K, n_out);
    } else if (y_dtype == TQK_F32) {
        skinny_kernel<MB, RT, false, float><<<blocks, waves * TQK_WAVE, lds, s>>>(xp, wp, (float*)y, M, N, K, n_out);
    } else {
        skinny_kernel<MB, RT, false, bf16_t><<<blocks, waves * TQK_WAVE, lds, s>>>(xp, wp, (bf16_t*)y, M, N, K, n_out);
    }
    return tqk_check_launch("tqk_skinny_bf16");
}

extern "C" int tqk_skinny_bf16(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K,
                               int epilogue, void* stream) {
    TQK_REQUIRE(x && w && y, "tqk_skinny_bf16: null pointer");
    TQK_REQUIRE(M >= 0 && M <= 64, "tqk_skinny_bf16: M=%d rows, this kernel takes at most 64", M);
    TQK_REQUIRE(N > 0 && K > 0 && K % 32 == 0, "tqk_skinny_bf16: K=%d must be a positive multiple of 32 (N=%d)", K, N);
    TQK_REQUIRE(epilogue == 0 || epilogue == 1, "tqk_skinny_bf16: unknown epilogue %d", epilogue);
    TQK_REQUIRE(!epilogue || N % 2 == 0, "tqk_skinny_bf16: gated epilogue needs an even N, got %d", N);
    TQK_REQUIRE(y_dtype == TQK_F32 || y_dtype == TQK_BF16, "tqk_skinny_bf16: unknown output dtype %d", y_dtype);
    TQK_REQUIRE(!epilogue || y_dtype == TQK_BF16, "tqk_skinny_bf16: the gated epilogue writes bfloat16");
    TQK_REQUIRE((((uintptr_t)x) & 15) == 0 && (((uintptr_t)w) & 15) == 0, "tqk_skinny_bf16: x and w must be 16-byte aligned");
    if (M == 0) return 0;
    // With more than 16 rows of x a wave takes four tiles of output features (two gate and up
    // pairs), so that it loads as many weight vectors as x vectors per step; with up to 16
    // rows one tile (pair).  Waves per block: about a thousand waves on the chip keep HBM busy
    // (measured: with more, each wave's share of K gets so short that start-up and the
    // reduction dominate), no more than there are chunks of K, a power of two, and such that
    // the LDS reduction fits.  Only "M > 16" plays a part, so within either kind a row's sum
    // has the same order in any batch.
    const int n_out = epilogue ? N / 2 : N;
    const int rt = M > 16 ? (epilogue ? 2 : 4) : 1;
    const int blocks = (n_out + 16 * rt - 1) / (16 * rt);
    const int chunks = K / ((rt > 1 ? SK_UNROLL / 2 : SK_UNROLL) * 32) > 0 ? K / ((rt > 1 ? SK_UNROLL / 2 : SK_UNROLL) * 32) : 1;
    const int max_waves = M > 16 ? 4 : (epilogue ? 8 : 16);      // 4 waves * 4 tiles * 4 blocks of x rows * 4 KB = 64 KB of LDS
    int waves = 1;
    while (waves < max_waves && blocks * waves < 1024 && waves * 2 <= chunks) waves *= 2;
    hipStream_t s = (hipStream_t)stream;
    const int mb = (M + 15) / 16;
    switch (mb) {
        case 1: return launch_mb<1, 1>(x, w, y, y_dtype, M, N, K, epilogue, waves, s);
        case 2: return launch_mb<2, 4>(x, w, y, y_dtype, M, N, K, epilogue, waves, s);
        case 3: return launch_mb<3, 4>(x, w, y, y_dtype, M, N, K, epilogue, waves, s);
        default: return launch_mb<4, 4>(x, w, y, y_dtype, M, N, K, epilogue, waves, s);
    }
}
