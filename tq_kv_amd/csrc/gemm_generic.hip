// y[M,N] = x[M,K] w[N,K]^T (+ bias): the plain product of the float32 path, and of
// any dtype mix the fast kernels do not take.  The reference's linear layers are
// candle matmuls (src/models/turbo_generic.rs:68-91, 779-781).
//
// LDS-tiled, 64x64 outputs per block, 4x4 per thread, float32 FMA only (no matrix
// cores, so no reduced-precision mode can slip in).  Each output is summed over k in
// increasing order by one thread: the result does not depend on M or on where a
// row stands in the batch.
#include "common.h"
#include "tq_kernels.h"

#define GT 64      // tile edge
#define GK 16      // k per stage

template <typename TX, typename TW, typename TB, typename TY>
__global__ __launch_bounds__(256)
void gemm_generic_kernel(const TX* __restrict__ x, const TW* __restrict__ w, const TB* __restrict__ bias,
                         TY* __restrict__ y, int M, int N, int K) {
    __shared__ float xs[GK][GT + 4];
    __shared__ float ws[GK][GT + 4];
    const int tid = threadIdx.x;
    const int tm = tid / 16, tn = tid % 16;            // thread's 4x4 patch: rows tm*4.., cols tn*4..
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

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
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = m0 + tm * 4 + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tn * 4 + j;
            if (gn >= N) continue;
            float v = acc[i][j];
            if (bias) v += to_float(bias[gn]);
            y[(size_t)gm * N + gn] = from_float<TY>(v);
        }
    }
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
                        int bias_dtype, void* y, int y_dtype, int M, int N, int K, void* stream) {
    TQK_REQUIRE(x && w && y, "tqk_gemm: null pointer");
    TQK_REQUIRE(M >= 0 && N > 0 && K > 0, "tqk_gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    TQK_REQUIRE((M + GT - 1) / GT <= 65535, "tqk_gemm: M=%d is more than the grid takes", M);
    if (M == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
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
