// Random weights on the GPU with the same bits as the host makes them
// (tq_kv_amd/weights/random_init.py holds the recipe and the host's version of it).
//
// Element i of a stream is a function of (key, i): a 64-bit hash, then Box and Muller's
// transform built from integer operations and from float32 multiplications and additions
// that are each rounded on their own.  The compiler must not fuse a multiplication with
// the addition after it, or the bits would differ from the host's: contraction is
// switched off for this file's arithmetic.
#include "common.h"
#include "tq_kernels.h"

#pragma clang fp contract(off)

namespace {

__device__ __forceinline__ float horner(const float* coef, int n, float x) {
#pragma clang fp contract(off)
    float acc = coef[n - 1];
    for (int k = n - 2; k >= 0; --k) {
        acc = acc * x;
        acc = acc + coef[k];
    }
    return acc;
}

__device__ __forceinline__ float standard_normal(uint64_t key, uint64_t index) {
#pragma clang fp contract(off)
    const float LOG_Q[11] = {1.0f, -0.5f, 0.33333301544189453f, -0.2500002384185791f, 0.2000257670879364f,
                             -0.16668042540550232f, 0.14212606847286224f, -0.1239922046661377f, 0.11923925578594208f,
                             -0.11727229505777359f, 0.06740232557058334f};
    const float COS_C[7] = {1.0f, -0.5f, 0.0416666679084301f, -0.0013888884568586946f, 2.4801040126476437e-05f,
                            -2.752467764821631e-07f, 1.990758891068367e-09f};
    uint64_t x = key + (index + 1ull) * 0x9E3779B97F4A7C15ull;
    x ^= x >> 30; x *= 0xBF58476D1CE4E5B9ull;
    x ^= x >> 27; x *= 0x94D049BB133111EBull;
    x ^= x >> 31;
    const uint32_t hi = (uint32_t)(x >> 32), lo = (uint32_t)x;
    // ln u1, u1 = ((hi >> 8) + 1) / 2^24 = m * 2^e
    const int n = (int)(hi >> 8) + 1;
    const int bits = __float_as_int((float)n);
    int e = (bits >> 23) - 151;
    float m = __int_as_float((bits & 0x7FFFFF) | 0x3F800000);
    if (m > 1.4142135f) { m = m * 0.5f; e += 1; }
    const float t = m - 1.0f;
    const float q = horner(LOG_Q, 11, t);
    const float a1 = (float)e * 0.6931471805599453f;
    const float a2 = t * q;
    const float ln_u = a1 + a2;
    // r = sqrt(v), v = -2 ln u1: three Newton steps for 1/sqrt(v)
    const float v = ln_u * -2.0f;
    float y = __int_as_float(0x5F3759DF - (__float_as_int(v) >> 1));
    const float hv = v * 0.5f;
    for (int k = 0; k < 3; ++k) {
        const float yy = y * y;
        const float p = hv * yy;
        const float s = 1.5f - p;
        y = y * s;
    }
    const float r = v * y;
    // cosine: quadrant and 23 bits of angle inside it, odd quadrants mirrored
    const uint32_t quadrant = lo >> 30;
    int f = (int)((lo >> 7) & 0x7FFFFFu);
    if (quadrant & 1u) f = 0x7FFFFF - f;
    const float frac = (float)(2 * f + 1) * 5.9604644775390625e-08f;          // 2^-24, exact
    const float a = frac * 1.5707963267948966f;
    const float aa = a * a;
    const float c = horner(COS_C, 7, aa);
    const float z = r * c;
    return (quadrant == 1u || quadrant == 2u) ? -z : z;
}

template <typename T>
__global__ __launch_bounds__(256)
void random_normal_kernel(T* __restrict__ out, long long n, uint64_t key, float std_dev, int plus_one) {
#pragma clang fp contract(off)
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float v = standard_normal(key, (uint64_t)i) * std_dev;
        if (plus_one) v = 1.0f + v;
        out[i] = from_float<T>(v);
    }
}

}  // namespace

extern "C" int tqk_random_normal(void* out, int dtype, long long n, uint64_t key, float std_dev, int plus_one, void* stream) {
    TQK_REQUIRE(out || n == 0, "tqk_random_normal: null pointer");
    TQK_REQUIRE(n >= 0, "tqk_random_normal: bad size %lld", n);
    TQK_REQUIRE(dtype == TQK_F32 || dtype == TQK_BF16, "tqk_random_normal: unknown dtype code %d", dtype);
    if (n == 0) return 0;
    const long long want = (n + 255) / 256;
    const int blocks = (int)(want < 16384 ? want : 16384);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TQK_F32)
        random_normal_kernel<float><<<blocks, 256, 0, s>>>((float*)out, n, key, std_dev, plus_one);
    else
        random_normal_kernel<bf16_t><<<blocks, 256, 0, s>>>((bf16_t*)out, n, key, std_dev, plus_one);
    return tqk_check_launch("tqk_random_normal");
}
