// Shared device helpers for the gfx950 kernels: bfloat16 storage, wave and block
// reductions with a fixed order, error reporting of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TQK_WAVE 64
#define TQK_PAGE 64

// ---- storage types ----------------------------------------------------------
// bfloat16 is kept as its 16 bits; every computation is in float.
struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

// Round to nearest even, NaN stays NaN: gfx950 has an instruction for it (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
    return __builtin_bit_cast(uint16_t, (__bf16)f);
}

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { bf16_t r; r.bits = float_to_bf16_bits(v); return r; }

// ---- places of values inside a page ---------------------------------------------
// A page of values is [kv head][head_dim][64 places]: an element's values of the page's
// 64 positions lie together, but not in order of position.  Position p (0..63) lies at
// place value_place(p): inside each group of 32 positions, the 4 positions 4g..4g+3 of
// the first 16 are followed by the 4 positions 16+4g..16+4g+3 of the second 16.  These
// are the 8 keys one lane feeds to the matrix cores in the product P.V (see
// attention_decode.hip), so a lane reads its 8 values as 16 contiguous bytes.
__device__ __host__ __forceinline__ int value_place(int p) {
    return (p & 32) | (((p >> 2) & 3) << 3) | (((p >> 4) & 1) << 2) | (p & 3);
}
__device__ __host__ __forceinline__ int value_position(int place) {
    return (place & 32) | (((place >> 2) & 1) << 4) | (((place >> 3) & 3) << 2) | (place & 3);
}

// ---- reductions ---------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, TQK_WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, TQK_WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `scratch`
// holds one float per wave.  The order of additions is fixed by the block shape.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (TQK_WAVE - 1), wave = threadIdx.x / TQK_WAVE;
    const int n_waves = (blockDim.x + TQK_WAVE - 1) / TQK_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < n_waves; ++w) total += scratch[w];
    return total;
}

// ---- host side ------------------------------------------------------------------
enum { TQK_F32 = 0, TQK_BF16 = 1 };

int tqk_fail(const char* fmt, ...);           // records the message, returns -1
int tqk_check_launch(const char* what);       // 0, or -1 with the HIP error recorded

#define TQK_REQUIRE(cond, ...) do { if (!(cond)) return tqk_fail(__VA_ARGS__); } while (0)
