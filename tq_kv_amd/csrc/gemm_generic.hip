// y[M,N] = x[M,K] w[N,K]^T (+ bias): the plain product of the float32 path, and of
// any dtype mix the fast kernels do not take.  The reference's linear layers are
// candle matmuls (src/models/turbo_generic.rs:68-91, 779-781).
//
// LDS-tiled, 64x64 outputs per block, 4x4 per thread, float32 FMA only (no matrix
// cores, so no reduced-precision mode can slip in).
//
// The order of summation is fixed and the same for every kernel here, so that a result does
// not depend on M, on where a row stands in the batch, or on which kernel computed it: k is
// cut into chunks of 128 and groups of 8 chunks; a chunk is summed by fused multiply-adds in
// increasing k from zero, a group is the sum of its chunks in order, the result the sum of
// the groups in order (and then the bias).
//
// For up to 16 rows of x in float32 (decoding in the 32-bit path) the weights are the whole
// cost and the tiled kernel would use a sixty-fourth of its tile: there a wave takes 64
// output features (one per lane, x's values are the same for all lanes) and one group of k,
// writes the groups' sums, and a second kernel adds them up.
#include "common.h"
#include "tq_kernels.h"

#define GT 64      // tile edge
#define GK 16      // k per stage
#define G_CHUNK 128                 // k per chunk
#define G_GROUP (8 * G_CHUNK)       // k per group

template <typename TX, typename TW, typename TB, typename TY>
__global__ __launch_bounds__(256)
void gemm_generic_kernel(const TX* __restrict__ x, const TW* __restrict__ w, const TB* __restrict__ bias,
                         TY* __restrict__ y, int M, int N, int K) {
    __shared__ float xs[GK][GT + 4];
    __shared__ float ws[GK][GT + 4];
    const int tid = threadIdx.x;
    const int tm = tid / 16, tn = tid % 16;            // thread's 4x4 patch: rows tm*4.., cols tn*4..
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    float acc[4][4], group[4][4], total[4][4];      // the chunk, the group and the result so far
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = group[i][j] = total[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GK) {
        // 64 rows x 16 k = 1024 elements per operand, 4 per thread
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int idx = tid + e * 256;
            const int r = idx / GK, kk = idx % GK;
            const int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
            xs[kk][r] = (gm < M && gk < K) ? to_float(x[(size_t)gm * K + gk]) : 0.f;
            ws[kk][r] = (gn < N && gk < K) ? to_float(w[(size_t)gn * K + gk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][tm * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tn * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
        const int k_done = k0 + GK;
        if (k_done % G_CHUNK == 0 || k_done >= K) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) { group[i][j] += acc[i][j]; acc[i][j] = 0.f; }
        }
        if (k_done % G_GROUP == 0 || k_done >= K) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) { total[i][j] += group[i][j]; group[i][j] = 0.f; }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = m0 + tm * 4 + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tn * 4 + j;
            if (gn >= N) continue;
            float v = total[i][j];
            if (bias) v += to_float(bias[gn]);
            y[(size_t)gm * N + gn] = from_float<TY>(v);
        }
    }
}

// Up to MR rows of x (float32): a wave per (64 output features, one group of k); lane = feature.
template <int MR>
__global__ __launch_bounds__(TQK_WAVE)
void gemm_few_rows_kernel(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ group_sums,
                          int M, int N, int K) {
    const int n = blockIdx.x * TQK_WAVE + threadIdx.x;
    const float* wrow = w + (size_t)min(n, N - 1) * K;
    const int k_begin = blockIdx.y * G_GROUP, k_end = min(K, k_begin + G_GROUP);
    const float* xrow[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) xrow[m] = x + (size_t)min(m, M - 1) * K;     // rows past M repeat the last and are dropped
    float group[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) group[m] = 0.f;
    for (int c0 = k_begin; c0 < k_end; c0 += G_CHUNK) {
        float acc[MR];
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[m] = 0.f;
        const int c_end = min(c0 + G_CHUNK, k_end);
#pragma unroll 4
        for (int k = c0; k < c_end; k += 4) {           // K is a multiple of 4
            const float4 w4 = *reinterpret_cast<const float4*>(wrow + k);
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                const float4 x4 = *reinterpret_cast<const float4*>(xrow[m] + k);     // the same for all lanes
                acc[m] = fmaf(x4.x, w4.x, acc[m]);
                acc[m] = fmaf(x4.y, w4.y, acc[m]);
                acc[m] = fmaf(x4.z, w4.z, acc[m]);
                acc[m] = fmaf(x4.w, w4.w, acc[m]);
            }
        }
#pragma unroll
        for (int m = 0; m < MR; ++m) group[m] += acc[m];
    }
    if (n < N) {
#pragma unroll
        for (int m = 0; m < MR; ++m)
            if (m < M) group_sums[((size_t)blockIdx.y * M + m) * N + n] = group[m];
    }
}

__global__ void gemm_few_rows_sum_kernel(const float* __restrict__ group_sums, const float* __restrict__ bias,
                                         float* __restrict__ y, int n_groups, int M, int N) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)M * N) return;
    float total = 0.f;
    for (int g = 0; g < n_groups; ++g) total += group_sums[(size_t)g * M * N + i];
    if (bias) total += bias[i % N];
    y[i] = total;
}

static bool few_rows_case(int x_dtype, int w_dtype, const void* bias, int bias_dtype, int y_dtype, int M, int K,
                          const void* x, const void* w) {
    return M <= 16 && K % 4 == 0 && x_dtype == TQK_F32 && w_dtype == TQK_F32 && y_dtype == TQK_F32 &&
           (!bias || bias_dtype == TQK_F32) && ((((uintptr_t)x) | ((uintptr_t)w)) & 15) == 0;
}

/* Bytes of device scratch tqk_gemm wants for these sizes and dtypes (0: none). */
extern "C" size_t tqk_gemm_scratch_bytes(int x_dtype, int w_dtype, int bias_dtype, int y_dtype, int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0 || !few_rows_case(x_dtype, w_dtype, nullptr, bias_dtype, y_dtype, M, K, nullptr, nullptr)) return 0;
    return (size_t)((K + G_GROUP - 1) / G_GROUP) * M * N * sizeof(float);
}

template <typename TX, typename TW, typename TB>
static int launch_y(const void* x, const void* w, const void* bias, void* y, int y_dtype,
                    int M, int N, int K, hipStream_t s) {
    dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT);
    if (y_dtype == TQK_F32)
        gemm_generic_kernel<TX, TW, TB, float><<<grid, 256, 0, s>>>((const TX*)x, (const TW*)w, (const TB*)bias, (float*)y, M, N, K);
    else if (y_dtype == TQK_BF16)
        gemm_generic_kernel<TX, TW, TB, bf16_t><<<grid, 256, 0, s>>>((const TX*)x, (const TW*)w, (const TB*)bias, (bf16_t*)y, M, N, K);
    else
        return tqk_fail("tqk_gemm: unknown output dtype %d", y_dtype);
    return tqk_check_launch("tqk_gemm");
}

extern "C" int tqk_gemm(const void* x, int x_dtype, const void* w, int w_dtype, const void* bias,
                        int bias_dtype, void* y, int y_dtype, int M, int N, int K, void* scratch, void* stream) {
    TQK_REQUIRE(x && w && y, "tqk_gemm: null pointer");
    TQK_REQUIRE(M >= 0 && N > 0 && K > 0, "tqk_gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    TQK_REQUIRE((M + GT - 1) / GT <= 65535, "tqk_gemm: M=%d is more than the grid takes", M);
    if (M == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (scratch && few_rows_case(x_dtype, w_dtype, bias, bias_dtype, y_dtype, M, K, x, w)) {
        const int n_groups = (K + G_GROUP - 1) / G_GROUP;
        TQK_REQUIRE(n_groups <= 65535, "tqk_gemm: K=%d is more than the grid takes", K);
        dim3 grid((N + TQK_WAVE - 1) / TQK_WAVE, n_groups);
        const float* xf = (const float*)x;
        const float* wf = (const float*)w;
        float* sums = (float*)scratch;
        if (M == 1) gemm_few_rows_kernel<1><<<grid, TQK_WAVE, 0, s>>>(xf, wf, sums, M, N, K);
        else if (M == 2) gemm_few_rows_kernel<2><<<grid, TQK_WAVE, 0, s>>>(xf, wf, sums, M, N, K);
        else if (M <= 4) gemm_few_rows_kernel<4><<<grid, TQK_WAVE, 0, s>>>(xf, wf, sums, M, N, K);
        else if (M <= 8) gemm_few_rows_kernel<8><<<grid, TQK_WAVE, 0, s>>>(xf, wf, sums, M, N, K);
        else gemm_few_rows_kernel<16><<<grid, TQK_WAVE, 0, s>>>(xf, wf, sums, M, N, K);
        if (tqk_check_launch("tqk_gemm few rows")) return -1;
        const size_t total = (size_t)M * N;
        gemm_few_rows_sum_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(sums, (const float*)bias, (float*)y, n_groups, M, N);
        return tqk_check_launch("tqk_gemm few rows sum");
    }
    if (!bias) bias_dtype = w_dtype;
    const int code = x_dtype * 4 + w_dtype * 2 + bias_dtype;
    switch (code) {
        case 0: return launch_y<float, float, float>(x, w, bias, y, y_dtype, M, N, K, s);
        case 1: return launch_y<float, float, bf16_t>(x, w, bias, y, y_dtype, M, N, K, s);
        case 2: return launch_y<float, bf16_t, float>(x, w, bias, y, y_dtype, M, N, K, s);
        case 3: return launch_y<float, bf16_t, bf16_t>(x, w, bias, y, y_dtype, M, N, K, s);
        case 4: return launch_y<bf16_t, float, float>(x, w, bias, y, y_dtype, M, N, K, s);
        case 5: return launch_y<bf16_t, float, bf16_t>(x, w, bias, y, y_dtype, M, N, K, s);
        case 6: return launch_y<bf16_t, bf16_t, float>(x, w, bias, y, y_dtype, M, N, K, s);
        case 7: return launch_y<bf16_t, bf16_t, bf16_t>(x, w, bias, y, y_dtype, M, N, K, s);
    }
    return tqk_fail("tqk_gemm: unknown dtypes x=%d w=%d bias=%d", x_dtype, w_dtype, bias_dtype);
}
