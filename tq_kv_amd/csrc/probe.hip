// Two probes of what the GPU at hand can do, for the bench to set its figures against: a plain
// streaming read by all compute units, and a loop of matrix-core instructions on registers.
// Neither is part of the model; both are measured by the caller (events around the launch).
#include "common.h"
#include "tq_kernels.h"

namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// every block reads a region of its own front to back, four pieces of 16 bytes per thread under way; the loads say
// that nothing is read twice; the sum keeps them alive
__global__ __launch_bounds__(256)
void probe_read_kernel(const u32x4_t* __restrict__ src, long long n16, uint32_t* __restrict__ sink) {
    const long long per = (n16 + gridDim.x - 1) / gridDim.x;
    const long long begin = per * blockIdx.x, end = begin + per < n16 ? begin + per : n16;
    u32x4_t acc = {0u, 0u, 0u, 0u};
    const long long step = blockDim.x;
    long long i = begin + threadIdx.x;
    for (; i + 3 * step < end; i += 4 * step) {
        const u32x4_t a = __builtin_nontemporal_load(src + i), b = __builtin_nontemporal_load(src + i + step);
        const u32x4_t c = __builtin_nontemporal_load(src + i + 2 * step), d = __builtin_nontemporal_load(src + i + 3 * step);
        acc ^= a ^ b ^ c ^ d;
    }
    for (; i < end; i += step) acc ^= __builtin_nontemporal_load(src + i);
    const uint32_t v = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (v == 0x9E3779B9u) sink[0] = v;              // (never, in practice: the store is only there so that the loads are)
}

// four independent 32x32x16 products per wave and turn, operands that never leave the registers
__global__ __launch_bounds__(256)
void probe_mfma_kernel(long long turns, float* __restrict__ sink) {
    bf16x8_t a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(0.001f * (float)(threadIdx.x % 7 + i)); b[i] = (__bf16)(0.002f * (float)(threadIdx.x % 5 + i)); }
    f32x16_t c0 = {}, c1 = {}, c2 = {}, c3 = {};
    for (long long t = 0; t < turns; ++t) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
    }
    float s = 0.f;
    for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
    if (s == 12345.678f) sink[0] = s;
}

}  // namespace

/* Reads `bytes` bytes (a multiple of 16, 16-byte aligned) once, by `blocks` blocks of `threads` threads (64, 128 or 256; blocks 0:
 * two blocks of 256 per compute unit), each block a region of its own.  sink: 4 bytes of device memory (nothing meaningful is
 * written).  The caller times the launch and tries several shapes: bytes / time of the best is what a kernel that only reads reaches. */
extern "C" int tqk_probe_read(const void* src, long long bytes, int blocks, int threads, void* sink, void* stream) {
    TQK_REQUIRE(src && sink && bytes > 0 && bytes % 16 == 0 && (((uintptr_t)src) & 15) == 0, "tqk_probe_read: needs a 16-byte aligned buffer of a multiple of 16 bytes");
    TQK_REQUIRE(blocks >= 0 && blocks <= (1 << 20) && (threads == 64 || threads == 128 || threads == 256), "tqk_probe_read: %d blocks of %d threads", blocks, threads);
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    probe_read_kernel<<<blocks ? blocks : cus * 2, threads, 0, (hipStream_t)stream>>>((const u32x4_t*)src, bytes / 16, (uint32_t*)sink);
    return tqk_check_launch("tqk_probe_read");
}

/* `turns` times four 32x32x16 bfloat16 matrix-core products per wave, 8 blocks of 4 waves per compute unit.  *flops_out (host): the
 * floating-point operations of the launch.  The caller times it: flops / time is what the matrix cores give when nothing else is in the way. */
extern "C" int tqk_probe_mfma(long long turns, void* sink, double* flops_out, void* stream) {
    TQK_REQUIRE(sink && turns > 0, "tqk_probe_mfma: bad arguments");
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    const int blocks = cus * 8;
    probe_mfma_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>(turns, (float*)sink);
    if (flops_out) *flops_out = (double)blocks * 4.0 * (double)turns * 4.0 * 2.0 * 32.0 * 32.0 * 16.0;
    return tqk_check_launch("tqk_probe_mfma");
}
