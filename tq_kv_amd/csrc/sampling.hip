// Choosing the next token on the device: argmax, and temperature / top-k / top-p /
// repeat-penalty sampling by inverse CDF.  One block per row of logits.
//
// The reference samples on the host from a copy of the logits
// (src/engine.rs:353-373, 403-423): argmax if temperature <= 0, else top-k then
// top-p at a temperature, after a repeat penalty over the generated tokens.  What
// "top-k then top-p" keeps at ties, and how the draw is made, is defined here:
//
//   z_i   = logit_i, then for every generated token (once per occurrence)
//           z > 0 ? z / penalty : z * penalty, then z / temperature
//   p_i   = softmax(z)_i
//   top-k : the k tokens with the largest z; among equal z the lower ids first
//   top-p : of those, every token with p_i >= p_c, where c is the token at which the
//           cumulative kept probability, taken from the largest down, first reaches
//           top_p times the kept total
//   draw  : with one uniform u in [0,1), the first kept token, in order of id, whose
//           cumulative kept probability exceeds u times the kept total
//
// Every sum is taken in a fixed order (per-thread contiguous segments in order of id,
// then a fixed scan over threads), so a row's result depends on nothing but the row,
// the history and u.
#include "common.h"
#include "tq_kernels.h"

#define SAMP_THREADS 1024

// ---- argmax ----------------------------------------------------------------------
// Two stages, so that a handful of rows still spread over the chip: blocks of 256 threads
// each find the best of a chunk of a row, then one block per row finds the best chunk.
// "Best" is the largest value, the lowest index among equals; NaN never wins.
#define AM_CHUNK 4096
#define AM_THREADS 256

__device__ __forceinline__ void better(float& bv, int& bi, float ov, int oi) {
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
}

__device__ __forceinline__ void block_best(float& bv, int& bi, float* sv, int* si) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) better(bv, bi, __shfl_xor(bv, o, TQK_WAVE), __shfl_xor(bi, o, TQK_WAVE));
    const int lane = threadIdx.x % TQK_WAVE, wave = threadIdx.x / TQK_WAVE;
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0)
        for (int w = 1; w < (int)(blockDim.x / TQK_WAVE); ++w) better(bv, bi, sv[w], si[w]);
}

__global__ __launch_bounds__(AM_THREADS)
void argmax_chunk_kernel(const float* __restrict__ logits, int vocab, int n_chunks,
                         float* __restrict__ best_v, int32_t* __restrict__ best_i) {
    __shared__ float sv[AM_THREADS / TQK_WAVE];
    __shared__ int si[AM_THREADS / TQK_WAVE];
    const float* row = logits + (size_t)blockIdx.y * vocab;
    const int begin = blockIdx.x * AM_CHUNK, end = min(vocab, begin + AM_CHUNK);
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = begin + threadIdx.x; i < end; i += AM_THREADS) better(bv, bi, row[i], i);
    block_best(bv, bi, sv, si);
    if (threadIdx.x == 0) { best_v[(size_t)blockIdx.y * n_chunks + blockIdx.x] = bv; best_i[(size_t)blockIdx.y * n_chunks + blockIdx.x] = bi; }
}

__global__ __launch_bounds__(AM_THREADS)
void argmax_final_kernel(const float* __restrict__ best_v, const int32_t* __restrict__ best_i, int n_chunks,
                         int32_t* __restrict__ out) {
    __shared__ float sv[AM_THREADS / TQK_WAVE];
    __shared__ int si[AM_THREADS / TQK_WAVE];
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int c = threadIdx.x; c < n_chunks; c += AM_THREADS)
        better(bv, bi, best_v[(size_t)blockIdx.x * n_chunks + c], best_i[(size_t)blockIdx.x * n_chunks + c]);
    block_best(bv, bi, sv, si);
    if (threadIdx.x == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

extern "C" int tqk_argmax_scratch_floats(int n_rows, int vocab) {
    return 2 * n_rows * ((vocab + AM_CHUNK - 1) / AM_CHUNK);
}

extern "C" int tqk_argmax(const float* logits, int n_rows, int vocab, int32_t* out, float* scratch, void* stream) {
    TQK_REQUIRE(logits && out && scratch, "tqk_argmax: null pointer");
    TQK_REQUIRE(n_rows >= 0 && vocab > 0, "tqk_argmax: bad sizes rows=%d vocab=%d", n_rows, vocab);
    TQK_REQUIRE(n_rows <= 65535, "tqk_argmax: too many rows for the grid");
    if (n_rows == 0) return 0;
    const int n_chunks = (vocab + AM_CHUNK - 1) / AM_CHUNK;
    float* best_v = scratch;
    int32_t* best_i = reinterpret_cast<int32_t*>(scratch + (size_t)n_rows * n_chunks);
    hipStream_t s = (hipStream_t)stream;
    argmax_chunk_kernel<<<dim3(n_chunks, n_rows), AM_THREADS, 0, s>>>(logits, vocab, n_chunks, best_v, best_i);
    if (tqk_check_launch("tqk_argmax")) return -1;
    argmax_final_kernel<<<n_rows, AM_THREADS, 0, s>>>(best_v, best_i, n_chunks, out);
    return tqk_check_launch("tqk_argmax final");
}

// ---- helpers for one-block-per-row passes ---------------------------------------
// Order-preserving map from float to unsigned: a < b  <=>  key(a) < key(b).
__device__ __forceinline__ uint32_t float_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Exclusive scan of one value per thread over the block, in thread order; `total`
// receives the sum of all.  scratch: one slot per wave.
template <typename V>
__device__ __forceinline__ V block_exclusive_scan(V v, V* scratch, V* total) {
    const int lane = threadIdx.x % TQK_WAVE, wave = threadIdx.x / TQK_WAVE;
    const int n_waves = blockDim.x / TQK_WAVE;
    V incl = v;
#pragma unroll
    for (int o = 1; o < TQK_WAVE; o <<= 1) {
        const V up = __shfl_up(incl, o, TQK_WAVE);
        if (lane >= o) incl += up;
    }
    __syncthreads();
    if (lane == TQK_WAVE - 1) scratch[wave] = incl;
    __syncthreads();
    V before = 0, all = 0;
    for (int w = 0; w < n_waves; ++w) {
        const V s = scratch[w];
        if (w < wave) before += s;
        all += s;
    }
    *total = all;
    return before + incl - v;
}

template <typename V>
__device__ __forceinline__ V block_sum_any(V v, V* scratch) {
    V total;
    block_exclusive_scan<V>(v, scratch, &total);
    return total;
}

__device__ __forceinline__ float block_max_f(float v, float* scratch) {
    const int lane = threadIdx.x % TQK_WAVE, wave = threadIdx.x / TQK_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float m = scratch[0];
    for (int w = 1; w < (int)(blockDim.x / TQK_WAVE); ++w) m = fmaxf(m, scratch[w]);
    return m;
}

// ---- repeat penalty ----------------------------------------------------------------
// src/engine.rs:403-419: for every generated token, once per occurrence,
// l > 0 ? l / penalty : l * penalty.  The thread that holds a token's first occurrence
// applies the penalty as often as the token occurs.
__global__ void repeat_penalty_kernel(float* __restrict__ logits, int vocab, const int32_t* __restrict__ row_req,
                                      const int32_t* __restrict__ hist, int hist_cap,
                                      const int32_t* __restrict__ hist_len, float penalty) {
    float* row = logits + (size_t)blockIdx.x * vocab;
    const int req = row_req[blockIdx.x];
    const int32_t* h = hist + (size_t)req * hist_cap;
    const int n = min(hist_len[req], hist_cap);
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int tok = h[i];
        if (tok < 0 || tok >= vocab) continue;
        bool first = true;
        for (int j = 0; j < i; ++j) if (h[j] == tok) { first = false; break; }
        if (!first) continue;
        int count = 1;
        for (int j = i + 1; j < n; ++j) count += (h[j] == tok);
        float z = row[tok];
        for (int c = 0; c < count; ++c) z = z > 0.f ? z / penalty : z * penalty;
        row[tok] = z;
    }
}

extern "C" int tqk_repeat_penalty(float* logits, int n_rows, int vocab, const int32_t* row_req,
                                  const int32_t* hist, int hist_cap, const int32_t* hist_len, int n_req,
                                  float penalty, void* stream) {
    TQK_REQUIRE(logits && row_req && hist && hist_len, "tqk_repeat_penalty: null pointer");
    TQK_REQUIRE(n_rows >= 0 && vocab > 0 && hist_cap > 0 && n_req > 0, "tqk_repeat_penalty: bad sizes");
    TQK_REQUIRE(penalty > 0.f, "tqk_repeat_penalty: penalty must be positive, got %g", (double)penalty);
    if (n_rows == 0) return 0;
    repeat_penalty_kernel<<<n_rows, 256, 0, (hipStream_t)stream>>>(logits, vocab, row_req, hist, hist_cap, hist_len, penalty);
    return tqk_check_launch("tqk_repeat_penalty");
}

__global__ void append_history_kernel(const int32_t* __restrict__ tokens, const int32_t* __restrict__ row_req,
                                      int32_t* __restrict__ hist, int hist_cap, int32_t* __restrict__ hist_len, int n_rows) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= n_rows) return;
    const int req = row_req[r];
    const int n = hist_len[req];
    if (n < hist_cap) { hist[(size_t)req * hist_cap + n] = tokens[r]; hist_len[req] = n + 1; }
}

extern "C" int tqk_append_history(const int32_t* tokens, const int32_t* row_req, int32_t* hist, int hist_cap,
                                  int32_t* hist_len, int n_rows, void* stream) {
    TQK_REQUIRE(tokens && row_req && hist && hist_len, "tqk_append_history: null pointer");
    TQK_REQUIRE(n_rows >= 0 && hist_cap > 0, "tqk_append_history: bad sizes");
    if (n_rows == 0) return 0;
    append_history_kernel<<<(n_rows + 255) / 256, 256, 0, (hipStream_t)stream>>>(tokens, row_req, hist, hist_cap, hist_len, n_rows);
    return tqk_check_launch("tqk_append_history");
}

// ---- temperature / top-k / top-p draw ------------------------------------------------
__global__ __launch_bounds__(SAMP_THREADS)
void sample_kernel(const float* __restrict__ logits, int vocab, float temperature, int top_k, float top_p,
                   const float* __restrict__ uniforms, int32_t* __restrict__ out) {
    __shared__ float fscratch[SAMP_THREADS / TQK_WAVE];
    __shared__ int iscratch[SAMP_THREADS / TQK_WAVE];
    __shared__ int hist[256];
    __shared__ uint32_t sh_prefix;
    __shared__ int sh_remaining;
    __shared__ int sh_pick;

    const float* row = logits + (size_t)blockIdx.x * vocab;
    const int tid = threadIdx.x;
    const float inv_t = 1.f / temperature;

    // largest logit (NaN never wins a comparison)
    float zmax = -INFINITY;
    for (int i = tid; i < vocab; i += SAMP_THREADS) zmax = fmaxf(zmax, row[i]);
    zmax = block_max_f(zmax, fscratch);
    // weight of a token: e_i = exp((z_i - zmax) / T); probabilities are e_i / sum
#define WEIGHT(z) expf(((z) - zmax) * inv_t)

    // top-k: key of the k-th largest logit by radix select over the keys' bytes
    const bool use_k = top_k > 0 && top_k < vocab;
    uint32_t tkey = 0;          // kept_k: key > tkey, or key == tkey for the `ties` lowest ids
    int ties = 0x7fffffff;
    if (use_k) {
        if (tid == 0) { sh_prefix = 0; sh_remaining = top_k; }
        for (int shift = 24; shift >= 0; shift -= 8) {
            for (int b = tid; b < 256; b += SAMP_THREADS) hist[b] = 0;
            __syncthreads();
            const uint32_t prefix = sh_prefix;
            const uint32_t mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
            for (int i = tid; i < vocab; i += SAMP_THREADS) {
                const float z = row[i];
                const uint32_t key = float_key(z);
                if (z == z && (key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 0xff], 1);
            }
            __syncthreads();
            if (tid == 0) {
                int remaining = sh_remaining, b = 255;
                for (; b > 0; --b) { if (hist[b] >= remaining) break; remaining -= hist[b]; }
                sh_prefix = prefix | ((uint32_t)b << shift);
                sh_remaining = remaining;
            }
            __syncthreads();
        }
        tkey = sh_prefix;
        ties = sh_remaining;     // how many tokens with key == tkey are kept (at least 1)
    }

    // top-p: the largest key tp >= tkey such that the kept_k tokens with key >= tp hold at
    // least top_p of kept_k's weight
    uint32_t tp = tkey;
    if (top_p < 1.f) {
        float mass = 0.f, tie_w = 0.f;
        uint32_t kmax = 0;
        for (int i = tid; i < vocab; i += SAMP_THREADS) {
            const float z = row[i];
            const uint32_t key = float_key(z);
            if (z == z) kmax = max(kmax, key);
            if (use_k ? key > tkey : z == z) mass += WEIGHT(z);
        }
        mass = block_sum_any<float>(mass, fscratch);
        if (use_k) {
            // all ties have the same logit, hence the same weight
            const uint32_t u = (tkey & 0x80000000u) ? (tkey & 0x7fffffffu) : ~tkey;
            tie_w = WEIGHT(__uint_as_float(u));
            mass += (float)ties * tie_w;
        }
        // exact max of kmax over the block
        {
            uint32_t m = kmax;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, o, TQK_WAVE));
            __syncthreads();
            if (tid % TQK_WAVE == 0) iscratch[tid / TQK_WAVE] = (int)m;
            __syncthreads();
            m = 0;
            for (int w = 0; w < SAMP_THREADS / TQK_WAVE; ++w) m = max(m, (uint32_t)iscratch[w]);
            kmax = m;
        }
        const float target = top_p * mass;
        uint32_t lo = tkey, hi = kmax;
        while (lo < hi) {
            const uint32_t mid = lo + (hi - lo + 1) / 2;      // mid > lo >= tkey
            float g = 0.f;
            for (int i = tid; i < vocab; i += SAMP_THREADS) {
                const float z = row[i];
                if (z == z && float_key(z) >= mid) g += WEIGHT(z);
            }
            g = block_sum_any<float>(g, fscratch);
            if (g >= target) lo = mid; else hi = mid - 1;
        }
        tp = lo;
    }

    // draw: walk the kept tokens in order of id
    const bool keep_ties = tp == tkey;
    const int seg = (vocab + SAMP_THREADS - 1) / SAMP_THREADS;
    const int begin = min(vocab, tid * seg), end = min(vocab, begin + seg);
    int my_ties = 0;
    if (use_k && keep_ties)
        for (int i = begin; i < end; ++i) my_ties += (float_key(row[i]) == tkey);
    int all_ties;
    const int ties_before = block_exclusive_scan<int>(my_ties, iscratch, &all_ties);
    float my_mass = 0.f;
    {
        int rank = ties_before;
        for (int i = begin; i < end; ++i) {
            const float z = row[i];
            if (!(z == z)) continue;
            const uint32_t key = float_key(z);
            bool kept;
            if (!use_k) kept = key >= tp;
            else if (key > tkey) kept = key >= tp;
            else if (key == tkey) { kept = keep_ties && rank < ties; ++rank; }
            else kept = false;
            if (kept) my_mass += WEIGHT(z);
        }
    }
    float total;
    const float before = block_exclusive_scan<float>(my_mass, fscratch, &total);
    const float target = uniforms[blockIdx.x] * total;
    // the owner: the last thread with kept weight whose segment starts at or below the target
    int cand = (my_mass > 0.f && before <= target) ? tid : -1;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cand = max(cand, __shfl_xor(cand, o, TQK_WAVE));
    __syncthreads();
    if (tid % TQK_WAVE == 0) iscratch[tid / TQK_WAVE] = cand;
    if (tid == 0) sh_pick = -1;
    __syncthreads();
    int owner = -1;
    for (int w = 0; w < SAMP_THREADS / TQK_WAVE; ++w) owner = max(owner, iscratch[w]);
    if (tid == owner) {
        float cum = before;
        int rank = ties_before, pick = -1, last = -1;
        for (int i = begin; i < end && pick < 0; ++i) {
            const float z = row[i];
            if (!(z == z)) continue;
            const uint32_t key = float_key(z);
            bool kept;
            if (!use_k) kept = key >= tp;
            else if (key > tkey) kept = key >= tp;
            else if (key == tkey) { kept = keep_ties && rank < ties; ++rank; }
            else kept = false;
            if (!kept) continue;
            last = i;
            cum += WEIGHT(z);
            if (cum > target) pick = i;
        }
        sh_pick = pick >= 0 ? pick : last;
    }
    __syncthreads();
    if (tid == 0) out[blockIdx.x] = sh_pick >= 0 ? sh_pick : 0;
#undef WEIGHT
}

extern "C" int tqk_sample(const float* logits, int n_rows, int vocab, float temperature, int top_k, float top_p,
                          const float* uniforms, int32_t* out, void* stream) {
    TQK_REQUIRE(logits && uniforms && out, "tqk_sample: null pointer");
    TQK_REQUIRE(n_rows >= 0 && vocab > 0, "tqk_sample: bad sizes rows=%d vocab=%d", n_rows, vocab);
    TQK_REQUIRE(temperature > 0.f, "tqk_sample: temperature must be positive (use argmax for greedy), got %g", (double)temperature);
    TQK_REQUIRE(top_k >= 0, "tqk_sample: top_k must not be negative");
    TQK_REQUIRE(top_p > 0.f, "tqk_sample: top_p must be positive, got %g", (double)top_p);
    if (n_rows == 0) return 0;
    sample_kernel<<<n_rows, SAMP_THREADS, 0, (hipStream_t)stream>>>(logits, vocab, temperature, top_k, top_p, uniforms, out);
    return tqk_check_launch("tqk_sample");
}
