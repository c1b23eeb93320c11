// Choosing the next token on the device: argmax, and temperature / top-k / top-p /
// repeat-penalty sampling by inverse CDF.  The rows of logits are read by many blocks each
// (argmax; top-k up to 256: the chunks' best first, then one block per row on those few);
// other settings of top-k take one block per row.
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
#include "tq_no_alloc.h"

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

// ---- argmax without a caller's scratch -------------------------------------------------------
// The same two kernels with the chunks' best values and indices in an array that is part of
// the library's image on every GPU it runs on (the process holds it until it ends), so the
// call needs no device memory beyond its input and output.  Host code reaches the array only
// through the address that hipGetSymbolAddress gives on the GPU that is current; every GPU
// has its own copy at its own address.
#define AM_STATIC_MAX_PAIRS 16384        // rows * chunks of a call, at most (128 KiB)
#define AM_STATIC_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[AM_STATIC_MAX_PAIRS * 8];

#include <mutex>
static std::mutex g_static_mutex;
static void* g_static_ptr[AM_STATIC_MAX_DEVICES];        // per GPU: where its copy of the array lies

// The current GPU's address of the array, or null with the error recorded.
static void* static_scratch_of_current_device(const char* who) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { tqk_fail("%s: hipGetDevice: %s", who, hipGetErrorString(e)); return nullptr; }
    if (dev < 0 || dev >= AM_STATIC_MAX_DEVICES) { tqk_fail("%s: GPU %d is beyond the %d this library keeps scratch for", who, dev, AM_STATIC_MAX_DEVICES); return nullptr; }
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) { tqk_fail("%s: hipGetSymbolAddress on GPU %d: %s", who, dev, hipGetErrorString(e)); return nullptr; }
        g_static_ptr[dev] = ptr;
    }
    return g_static_ptr[dev];
}

extern "C" int tqk_argmax_static_max_pairs(void) { return AM_STATIC_MAX_PAIRS; }

extern "C" int tqk_argmax_static_prepare(void) {
    return static_scratch_of_current_device("tqk_argmax_static_prepare") ? 0 : -1;
}

extern "C" int tqk_argmax_static(const float* logits, int n_rows, int vocab, int32_t* out, void* stream) {
    TQK_REQUIRE(logits && out, "tqk_argmax_static: null pointer");
    TQK_REQUIRE(n_rows >= 0 && vocab > 0, "tqk_argmax_static: bad sizes rows=%d vocab=%d", n_rows, vocab);
    if (n_rows == 0) return 0;
    const int n_chunks = (vocab + AM_CHUNK - 1) / AM_CHUNK;
    TQK_REQUIRE((long long)n_rows * n_chunks <= AM_STATIC_MAX_PAIRS,
                "tqk_argmax_static: %d rows of %d chunks of %d need %lld scratch entries, the library holds %d (use tqk_argmax with a scratch buffer of your own)",
                n_rows, n_chunks, AM_CHUNK, (long long)n_rows * n_chunks, AM_STATIC_MAX_PAIRS);
    void* ptr = static_scratch_of_current_device("tqk_argmax_static");
    if (!ptr) return -1;
    // every entry the second kernel reads is written by the first: nothing has to start at zero
    float* best_v = reinterpret_cast<float*>(ptr);
    int32_t* best_i = reinterpret_cast<int32_t*>(best_v + (size_t)n_rows * n_chunks);
    hipStream_t s = (hipStream_t)stream;
    argmax_chunk_kernel<<<dim3(n_chunks, n_rows), AM_THREADS, 0, s>>>(logits, vocab, n_chunks, best_v, best_i);
    if (tqk_check_launch("tqk_argmax_static")) return -1;
    argmax_final_kernel<<<n_rows, AM_THREADS, 0, s>>>(best_v, best_i, n_chunks, out);
    return tqk_check_launch("tqk_argmax_static final");
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

// The radix-select step over a histogram of 256 bins in LDS, by the block's first wave: the
// highest bin b such that the bins above it hold fewer than `remaining` entries and with it
// at least that many; `remaining` is lowered by what the bins above hold.  Lane 0 gets the result.
__device__ __forceinline__ void pick_bin(const int* hist, int remaining, int* bin, int* left) {
    const int lane = threadIdx.x;                      // 0..63: bins 255-4*lane down to 252-4*lane
    int h[4], sum = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) { h[i] = hist[255 - (4 * lane + i)]; sum += h[i]; }
    int incl = sum;
#pragma unroll
    for (int o = 1; o < TQK_WAVE; o <<= 1) {
        const int up = __shfl_up(incl, o, TQK_WAVE);
        if (lane >= o) incl += up;
    }
    int before = incl - sum, found = -1, found_before = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (found < 0 && before + h[i] >= remaining) { found = 255 - (4 * lane + i); found_before = before; }
        before += h[i];
    }
    // the first lane that found one
    const unsigned long long who = __ballot(found >= 0);
    const int first = who ? __ffsll((long long)who) - 1 : TQK_WAVE - 1;
    const int b = __shfl(found, first, TQK_WAVE), fb = __shfl(found_before, first, TQK_WAVE);
    *bin = who ? b : 0;
    *left = who ? remaining - fb : remaining - (__shfl(incl, TQK_WAVE - 1, TQK_WAVE) - hist[0]);
}

// ---- repeat penalty ----------------------------------------------------------------
// src/engine.rs:403-419: for every generated token, once per occurrence,
// l > 0 ? l / penalty : l * penalty.  The history of a request is kept as its tokens and, for
// each entry, how often the penalty is to be applied on its behalf: for the last occurrence
// of a token the number of its occurrences, for the earlier ones 0.  Appending a token keeps
// that up (one pass over the request's history), so applying the penalty is one pass too.
__global__ void repeat_penalty_kernel(float* __restrict__ logits, int vocab, const int32_t* __restrict__ row_req,
                                      const int32_t* __restrict__ hist, const int32_t* __restrict__ times, int hist_cap,
                                      const int32_t* __restrict__ hist_len, float penalty) {
    float* row = logits + (size_t)blockIdx.x * vocab;
    const int req = row_req[blockIdx.x];
    const int32_t* h = hist + (size_t)req * hist_cap;
    const int32_t* tm = times + (size_t)req * hist_cap;
    const int n = min(hist_len[req], hist_cap);
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int count = tm[i], tok = h[i];
        if (count <= 0 || tok < 0 || tok >= vocab) continue;
        float z = row[tok];
        for (int c = 0; c < count; ++c) z = z > 0.f ? z / penalty : z * penalty;
        row[tok] = z;
    }
}

extern "C" int tqk_repeat_penalty(float* logits, int n_rows, int vocab, const int32_t* row_req,
                                  const int32_t* hist, const int32_t* times, int hist_cap, const int32_t* hist_len,
                                  int n_req, float penalty, void* stream) {
    TQK_REQUIRE(logits && row_req && hist && times && hist_len, "tqk_repeat_penalty: null pointer");
    TQK_REQUIRE(n_rows >= 0 && vocab > 0 && hist_cap > 0 && n_req > 0, "tqk_repeat_penalty: bad sizes");
    TQK_REQUIRE(penalty > 0.f, "tqk_repeat_penalty: penalty must be positive, got %g", (double)penalty);
    if (n_rows == 0) return 0;
    repeat_penalty_kernel<<<n_rows, 256, 0, (hipStream_t)stream>>>(logits, vocab, row_req, hist, times, hist_cap, hist_len, penalty);
    return tqk_check_launch("tqk_repeat_penalty");
}

// One block per row: the row's token goes to the end of its request's history; the earlier
// occurrences of the token hand their count over to it.  Rows of one call name different requests.
__global__ void append_history_kernel(const int32_t* __restrict__ tokens, const int32_t* __restrict__ row_req,
                                      int32_t* __restrict__ hist, int32_t* __restrict__ times, int hist_cap,
                                      int32_t* __restrict__ hist_len) {
    __shared__ int scratch[256 / TQK_WAVE];
    const int r = blockIdx.x;
    const int req = row_req[r], tok = tokens[r];
    int32_t* h = hist + (size_t)req * hist_cap;
    int32_t* tm = times + (size_t)req * hist_cap;
    const int n = hist_len[req];
    if (n >= hist_cap) return;                         // full: the token is dropped
    int seen = 0;
    for (int i = threadIdx.x; i < n; i += blockDim.x)
        if (h[i] == tok) { ++seen; tm[i] = 0; }
    const int total = block_sum_any<int>(seen, scratch);
    if (threadIdx.x == 0) { h[n] = tok; tm[n] = total + 1; hist_len[req] = n + 1; }
}

extern "C" int tqk_append_history(const int32_t* tokens, const int32_t* row_req, int32_t* hist, int32_t* times,
                                  int hist_cap, int32_t* hist_len, int n_rows, void* stream) {
    TQK_REQUIRE(tokens && row_req && hist && times && hist_len, "tqk_append_history: null pointer");
    TQK_REQUIRE(n_rows >= 0 && hist_cap > 0, "tqk_append_history: bad sizes");
    if (n_rows == 0) return 0;
    append_history_kernel<<<n_rows, 256, 0, (hipStream_t)stream>>>(tokens, row_req, hist, times, hist_cap, hist_len);
    return tqk_check_launch("tqk_append_history");
}

// ---- temperature / top-k / top-p draw ------------------------------------------------
__global__ __launch_bounds__(SAMP_THREADS)
void sample_kernel(const float* __restrict__ logits, int vocab, float temperature, int top_k, float top_p,
                   const float* __restrict__ uniforms, int32_t* __restrict__ out, const int32_t* __restrict__ done) {
    if (done && done[blockIdx.x]) return;              // the row has been drawn from its candidates
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
            if (tid < TQK_WAVE) {
                int b, left;
                pick_bin(hist, sh_remaining, &b, &left);
                if (tid == 0) { sh_prefix = prefix | ((uint32_t)b << shift); sh_remaining = left; }
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

// ---- the usual case, 0 < top_k <= 256: candidates first ---------------------------------
// Only the top_k largest logits of a row can be drawn, so the row is read once, by many
// blocks: each block takes a chunk of the row into LDS and finds the chunk's top_k there
// (the row's top_k are among the chunks' top_k); then one block per row picks the top_k of
// the candidates and does top-p and the draw on those few, with the rules stated above.
#define CAND_THREADS 256
#define CAND_CHUNK 4864            // most logits per chunk (19 per thread; keys in LDS)
#define CAND_MAX_K 256
#define CAND_MAX_CHUNKS 64
#define CAND_MAX_TOTAL 6144        // most candidates per row in the second kernel's LDS (48 KB)

// key of a logit for selection: 0 for NaN (never taken), else float_key > 0
__device__ __forceinline__ uint32_t select_key(float z) { return z == z ? float_key(z) : 0u; }
__device__ __forceinline__ float key_value(uint32_t key) {
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

// Among keys[0..n) in LDS (n > want > 0): the key of the want-th largest, and how many of the
// entries with exactly that key belong to the want largest (lower indices first).  hist: 256
// ints in LDS; box: 2 uint32 in LDS.  Every thread of the block calls it.
__device__ void radix_select_lds(const uint32_t* keys, int n, int want, int* hist, uint32_t* box,
                                 uint32_t* tkey, int* ties) {
    if (threadIdx.x == 0) { box[0] = 0; box[1] = (uint32_t)want; }
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int b = threadIdx.x; b < 256; b += blockDim.x) hist[b] = 0;
        __syncthreads();
        const uint32_t prefix = box[0];
        const uint32_t mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const uint32_t key = keys[i];
            if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 0xff], 1);
        }
        __syncthreads();
        if (threadIdx.x < TQK_WAVE) {
            int b, left;
            pick_bin(hist, (int)box[1], &b, &left);
            if (threadIdx.x == 0) { box[0] = prefix | ((uint32_t)b << shift); box[1] = (uint32_t)left; }
        }
        __syncthreads();
    }
    *tkey = box[0];
    *ties = (int)box[1];
}

// The entries of keys[0..n) that belong to the `want` largest (all of them if n <= want; key 0
// never), copied in order of index to out_key / out_id (ids: first_id + index, or ids[index]).
// Returns how many.  scan: one int per wave in LDS.
__device__ int take_largest(const uint32_t* keys, const int32_t* ids, int first_id, int n, int want,
                            int* hist, uint32_t* box, int* scan, uint32_t* out_key, int32_t* out_id) {
    uint32_t tkey = 0;
    int ties = 0x7fffffff;
    if (n > want) radix_select_lds(keys, n, want, hist, box, &tkey, &ties);
    const int seg = (n + blockDim.x - 1) / blockDim.x;
    const int begin = min(n, (int)threadIdx.x * seg), end = min(n, begin + seg);
    int my_ties = 0, my_above = 0;
    for (int i = begin; i < end; ++i) {
        const uint32_t key = keys[i];
        my_ties += (key == tkey && key != 0);
        my_above += (key > tkey);
    }
    int all_ties, all_above;
    const int ties_before = block_exclusive_scan<int>(my_ties, scan, &all_ties);
    // of this thread's ties, those with rank below `ties` are taken
    const int my_taken_ties = max(0, min(my_ties, ties - ties_before));
    int total;
    int at = block_exclusive_scan<int>(my_above + my_taken_ties, scan, &total);
    (void)all_above;
    int rank = ties_before;
    for (int i = begin; i < end; ++i) {
        const uint32_t key = keys[i];
        bool take = key > tkey;
        if (key == tkey && key != 0) { take = rank < ties; ++rank; }
        if (take) { out_key[at] = key; out_id[at] = ids ? ids[i] : first_id + i; ++at; }
    }
    return total;
}

// largest of one unsigned value per thread; scratch: two words in LDS
__device__ __forceinline__ uint32_t block_max_u(uint32_t v, uint32_t* scratch) {
    __syncthreads();
    if (threadIdx.x == 0) scratch[0] = 0;
    __syncthreads();
    atomicMax(&scratch[0], v);
    __syncthreads();
    const uint32_t m = scratch[0];
    __syncthreads();
    return m;
}

__global__ __launch_bounds__(CAND_THREADS)
void sample_candidates_kernel(const float* __restrict__ logits, int vocab, int chunk, int n_chunks, int top_k,
                              uint32_t* __restrict__ cand_key, int32_t* __restrict__ cand_id, int32_t* __restrict__ cand_n,
                              float inv_t, float2* __restrict__ chunk_mass) {
    __shared__ uint32_t keys[CAND_CHUNK];
    __shared__ int hist[256];
    __shared__ uint32_t box[2];
    __shared__ int scan[CAND_THREADS / TQK_WAVE];
    __shared__ float fscan[CAND_THREADS / TQK_WAVE];
    const int row = blockIdx.y, blk = blockIdx.x;
    const int first = blk * chunk, n = max(0, min(vocab - first, chunk));
    const float* src = logits + (size_t)row * vocab + first;
    uint32_t kmax = 0;
    for (int i = threadIdx.x; i < n; i += CAND_THREADS) { const uint32_t key = select_key(src[i]); keys[i] = key; kmax = max(kmax, key); }
    __syncthreads();
    const size_t slot = (size_t)row * n_chunks + blk;
    if (chunk_mass) {
        // the chunk's largest logit and the weight of all its tokens relative to it
        // (the order of float_key is that of the values, so the largest key is the largest logit)
        const float cmax = key_value(block_max_u(kmax, box));
        float w = 0.f;
        for (int i = threadIdx.x; i < n; i += CAND_THREADS) { const uint32_t key = keys[i]; if (key) w += expf((key_value(key) - cmax) * inv_t); }
        w = block_sum_any<float>(w, fscan);
        if (threadIdx.x == 0) chunk_mass[slot] = make_float2(cmax, w);
    }
    const int taken = take_largest(keys, nullptr, first, n, top_k, hist, box, scan,
                                   cand_key + slot * top_k, cand_id + slot * top_k);
    if (threadIdx.x == 0) cand_n[slot] = taken;
}

__global__ __launch_bounds__(CAND_THREADS)
void sample_draw_kernel(const uint32_t* __restrict__ cand_key, const int32_t* __restrict__ cand_id,
                        const int32_t* __restrict__ cand_n, int n_chunks, int top_k, float temperature, float top_p,
                        const float* __restrict__ uniforms, int32_t* __restrict__ out,
                        const float2* __restrict__ chunk_mass, int32_t* __restrict__ done) {
    // With chunk_mass (no top-k asked for: top_k is only the number of candidates) top-p is cut
    // against the weight of the whole row; the row is drawn here if the cut lies inside the
    // candidates for certain, else it is left (done[row] = 0) to the kernel that reads the whole row.
    extern __shared__ uint32_t pool[];                 // keys [n_chunks * top_k], then ids
    __shared__ int hist[256];
    __shared__ uint32_t box[2];
    __shared__ int scan[CAND_THREADS / TQK_WAVE];
    __shared__ float fscan[CAND_THREADS / TQK_WAVE];
    __shared__ uint32_t fkey[CAND_MAX_K];              // the top_k, in order of id
    __shared__ int32_t fid[CAND_MAX_K];
    __shared__ float sorted_w[CAND_MAX_K];             // weights from the largest down
    __shared__ uint32_t sorted_key[CAND_MAX_K];
    __shared__ int sh_first;
    const int row = blockIdx.x, tid = threadIdx.x;
    uint32_t* keys = pool;
    int32_t* ids = reinterpret_cast<int32_t*>(pool + (size_t)n_chunks * top_k);

    // the chunks' candidates, chunk after chunk: in order of id
    int n = 0;
    for (int c = 0; c < n_chunks; ++c) {
        const size_t slot = (size_t)row * n_chunks + c;
        const int cn = cand_n[slot];
        for (int i = tid; i < cn; i += CAND_THREADS) { keys[n + i] = cand_key[slot * top_k + i]; ids[n + i] = cand_id[slot * top_k + i]; }
        n += cn;
    }
    __syncthreads();
    const int m = take_largest(keys, ids, 0, n, top_k, hist, box, scan, fkey, fid);
    __syncthreads();
    if (m == 0) {                                      // a row of NaN
        if (tid == 0) { out[row] = 0; if (done) done[row] = 1; }
        return;
    }
    // rank from the largest down, lower ids first among equals (the list is in order of id)
    const uint32_t my_key = tid < m ? fkey[tid] : 0u;
    int rank = 0;
    uint32_t kmax = 0;
    for (int j = 0; j < m; ++j) {
        const uint32_t kj = fkey[j];
        kmax = max(kmax, kj);
        rank += (kj > my_key) || (kj == my_key && j < tid);
    }
    const float inv_t = 1.f / temperature;
    const float zmax = key_value(kmax);
    const float my_w = tid < m ? expf((key_value(my_key) - zmax) * inv_t) : 0.f;
    if (tid < m) { sorted_w[rank] = my_w; sorted_key[rank] = my_key; }
    __syncthreads();
    // top-p: the place, from the largest down, where the cumulative weight first reaches top_p of the total
    uint32_t cut_key = 0;                              // keep keys >= cut_key
    if (top_p < 1.f) {
        const float w = tid < m ? sorted_w[tid] : 0.f;
        float total;
        const float before = block_exclusive_scan<float>(w, fscan, &total);
        if (chunk_mass) {
            // the whole row's weight: the chunks' weights, each moved to the row's largest logit, in order
            float cw = 0.f;
            if (tid < n_chunks) { const float2 cm = chunk_mass[(size_t)row * n_chunks + tid]; cw = cm.y > 0.f ? cm.y * expf((cm.x - zmax) * inv_t) : 0.f; }
            total = block_sum_any<float>(cw, fscan);
        }
        __syncthreads();
        if (tid == 0) sh_first = chunk_mass ? 0x7fffffff : m - 1;
        __syncthreads();
        if (tid < m && before + w >= top_p * total) atomicMin(&sh_first, tid);
        __syncthreads();
        const int first = sh_first;
        // for certain inside: reached at all, and above the smallest candidate unless these are all tokens
        if (chunk_mass && (first == 0x7fffffff || (n >= top_k && !(sorted_key[first] > sorted_key[m - 1])))) {
            if (tid == 0) done[row] = 0;
            return;
        }
        cut_key = sorted_key[first];
    }
    // the draw, in order of id
    const bool kept = tid < m && my_key >= cut_key;
    const float kw = kept ? my_w : 0.f;
    float total_kept;
    const float before = block_exclusive_scan<float>(kw, fscan, &total_kept);
    const float target = uniforms[row] * total_kept;
    __syncthreads();
    if (tid == 0) { box[0] = 0x7fffffffu; box[1] = 0; }
    __syncthreads();
    if (kept) {
        if (before + kw > target) atomicMin(&box[0], (uint32_t)tid);
        atomicMax(&box[1], (uint32_t)tid);
    }
    __syncthreads();
    if (tid == 0) { out[row] = fid[box[0] != 0x7fffffffu ? box[0] : box[1]]; if (done) done[row] = 1; }
}

static int sample_chunks(int vocab) { return (vocab + CAND_CHUNK - 1) / CAND_CHUNK; }

// top_k asked for and small: its candidates decide the row
static bool sample_by_candidates(int vocab, int top_k) {
    const int chunks = sample_chunks(vocab);
    return top_k > 0 && top_k <= CAND_MAX_K && top_k < vocab && chunks <= CAND_MAX_CHUNKS &&
           (long long)chunks * top_k <= CAND_MAX_TOTAL;
}

// no top-k but top-p: how many candidates a chunk gives for a try (0: no try)
static int sample_open_candidates(int vocab, int top_k, float top_p) {
    const int chunks = sample_chunks(vocab);
    if ((top_k > 0 && top_k < vocab) || !(top_p < 1.f) || chunks > CAND_MAX_CHUNKS || chunks > CAND_THREADS) return 0;
    const int k = CAND_MAX_TOTAL / chunks < CAND_MAX_K ? CAND_MAX_TOTAL / chunks : CAND_MAX_K;
    return k >= 16 ? k : 0;
}

/* Bytes of device scratch that tqk_sample wants for these sizes (0: none). */
extern "C" size_t tqk_sample_scratch_bytes(int n_rows, int vocab, int top_k, float top_p) {
    if (n_rows <= 0 || vocab <= 0) return 0;
    const int k = sample_by_candidates(vocab, top_k) ? top_k : sample_open_candidates(vocab, top_k, top_p);
    if (k == 0) return 0;
    const size_t slots = (size_t)n_rows * sample_chunks(vocab);
    return slots * k * 8 + slots * 4 + slots * 8 + (size_t)n_rows * 4;
}

extern "C" int tqk_sample(const float* logits, int n_rows, int vocab, float temperature, int top_k, float top_p,
                          const float* uniforms, int32_t* out, void* scratch, void* stream) {
    TQK_REQUIRE(logits && uniforms && out, "tqk_sample: null pointer");
    TQK_REQUIRE(n_rows >= 0 && vocab > 0, "tqk_sample: bad sizes rows=%d vocab=%d", n_rows, vocab);
    TQK_REQUIRE(temperature > 0.f, "tqk_sample: temperature must be positive (use argmax for greedy), got %g", (double)temperature);
    TQK_REQUIRE(top_k >= 0, "tqk_sample: top_k must not be negative");
    TQK_REQUIRE(top_p > 0.f, "tqk_sample: top_p must be positive, got %g", (double)top_p);
    TQK_REQUIRE(n_rows <= 65535, "tqk_sample: too many rows for the grid");
    if (n_rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const bool closed = sample_by_candidates(vocab, top_k);
    const int k = closed ? top_k : sample_open_candidates(vocab, top_k, top_p);
    int32_t* done = nullptr;
    if (k > 0) {
        TQK_REQUIRE(scratch, "tqk_sample: these sizes need scratch memory (tqk_sample_scratch_bytes)");
        const int chunks = sample_chunks(vocab), chunk = (vocab + chunks - 1) / chunks;
        const size_t slots = (size_t)n_rows * chunks;
        float2* chunk_mass = (float2*)scratch;                        // 8-byte values first
        uint32_t* cand_key = (uint32_t*)(chunk_mass + slots);
        int32_t* cand_id = (int32_t*)(cand_key + slots * k);
        int32_t* cand_n = cand_id + slots * k;
        done = cand_n + slots;
        sample_candidates_kernel<<<dim3(chunks, n_rows), CAND_THREADS, 0, s>>>(logits, vocab, chunk, chunks, k, cand_key, cand_id, cand_n,
                                                                             1.f / temperature, closed ? nullptr : chunk_mass);
        if (tqk_check_launch("tqk_sample candidates")) return -1;
        const size_t lds = (size_t)chunks * k * 8;
        sample_draw_kernel<<<n_rows, CAND_THREADS, lds, s>>>(cand_key, cand_id, cand_n, chunks, k, temperature, top_p, uniforms, out,
                                                             closed ? nullptr : chunk_mass, closed ? nullptr : done);
        if (tqk_check_launch("tqk_sample draw")) return -1;
        if (closed) return 0;
    }
    // the whole row by one block: every setting; after a try with candidates only the rows that the try left
    sample_kernel<<<n_rows, SAMP_THREADS, 0, s>>>(logits, vocab, temperature, top_k, top_p, uniforms, out, done);
    return tqk_check_launch("tqk_sample");
}
