// y[M,N] = x[M,K] w[N,K]^T for 17 to 128 rows (decoding steps of larger batches, the wanted rows
// of many prompts): bfloat16 in, MFMA, float32 accumulation.  The reference runs these products
// as candle matmuls (src/models/turbo_generic.rs:68-91).  At these M the product is still bound
// by the weight bytes, which are streamed from HBM once, straight into registers, from the copy
// packed in the lanes' order ([tile of 16 rows][K/32][lane][8 values], see skinny_fused.hip).
//
// With this many rows x is no longer small beside a tile of weights: every wave needs all of it.
// So a block is 4 to 8 waves that walk K together in chunks of 128; each chunk of x is staged once
// per block in LDS, in the order the lanes read it ([16 rows][k step][lane] x 16 bytes, so both
// the block's write and the waves' reads are linear), double buffered with one barrier per
// chunk, while each wave multiplies its own tiles of 16 output features with it.  The loads of
// the next two chunks are under way while the current one is multiplied.
//
// v_mfma_f32_16x16x32_bf16: A = a tile of w (16 features x 32 k), B = 32 k x 16 rows of x, so
// D[n][m] is a tile of y^T: lane l holds row m = l%16 of its 16-row group and the four features
// 4*(l/16) .. +3, which it stores as one 8- or 16-byte piece.
//
// Where N alone gives too few blocks for the chip, K is split over blockIdx.y: each split writes
// its sums to scratch [split][M][N] and a second kernel adds them in split order and finishes
// (store, or the gate: silu(gate) * up of src/models/turbo_generic.rs:105-111).  The number of
// splits depends on the product's shape alone, never on M, so a row's result does not depend on
// the batch it is in.
//
// Beyond 64 rows (8 row groups) every compute unit pulls all of x through its first-level cache
// beside its own share of the weights (0.9 MB beside 1.15 MB at 128 rows of the 7B gate+up
// product), and that path, not HBM, sets the time: 4.1 TB/s of weights at 128 rows against 4.9 at
// 64.  Measured there and left: reads of x two steps ahead, one or two extra waves that only bring
// x in, a deeper ring of LDS operands (the waves wait for x behind the weights in the same
// queue, whoever asks for it).
#include "common.h"
#include "tq_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

enum { MID_STORE = 0, MID_GATED = 1 };
#define MID_CHUNK 128           // k per stage
#define MID_MIN_WAVES 4          // waves per block: from the product's shape (mid_plan)
#define MID_MAX_WAVES 8
#define MID_MAX_ROWS 128

struct MidArgs {
    const bf16_t* x;            // [M, K]
    const bf16_t* w;            // packed [tiles][K/32][64][8]
    void* y;                    // store: [M, N]; gated: [M, N/2] bfloat16
    float* partial;             // [splits][M][N] when the grid has splits
    int M, N, K, k_per_split;   // k_per_split: a multiple of MID_CHUNK
};

__device__ __forceinline__ uint2 pack4_bf16(float a, float b, float c, float d) {
    return make_uint2((uint32_t)float_to_bf16_bits(a) | ((uint32_t)float_to_bf16_bits(b) << 16),
                      (uint32_t)float_to_bf16_bits(c) | ((uint32_t)float_to_bf16_bits(d) << 16));
}

__device__ __forceinline__ float gate_times_up(float gate_sum, float up_sum) {
    const float g = to_float(from_float<bf16_t>(gate_sum)), up = to_float(from_float<bf16_t>(up_sum));
    return (g / (1.f + expf(-g))) * up;
}

// MT: groups of 16 rows of x (2: up to 32 rows, 4: up to 64, 8: up to 128).  TN: tiles of 16
// features per wave (gated: the gate tile and its up tile).
// PAR: 256-thread groups of the block that bring x in (2 in a block of 8 waves, else 1).
template <int MT, int TN, int EPI, typename TY, int PAR>
__global__ __launch_bounds__(MID_MAX_WAVES * TQK_WAVE)
void mid_product_kernel(const MidArgs p) {
    constexpr int SLOTS = MT * 256;                 // 16-byte pieces of a chunk of x: [row group][k step][lane]
    constexpr bool WIDE = MT > 4;                   // 8 row groups: registers are short, see below
    constexpr int XS = WIDE ? MT / PAR : SLOTS / (MID_MIN_WAVES * TQK_WAVE);       // pieces of x per thread at most
    static_assert(EPI != MID_GATED || TN == 2, "a gated block holds pairs of tiles");
    extern __shared__ u32x4_t xs[];                 // [2][SLOTS]
    const int lane = threadIdx.x % TQK_WAVE, wave = threadIdx.x / TQK_WAVE;
    const int n_waves = blockDim.x / TQK_WAVE;
    const int row = lane % 16, kgrp = lane / 16;
    const int K = p.K;
    const int k_begin = blockIdx.y * p.k_per_split, k_end = min(K, k_begin + p.k_per_split);

    const int n_out = EPI == MID_GATED ? p.N / 2 : p.N;             // features one part of the weight has
    const int part_tiles = (n_out + 15) / 16;
    const int tile0 = (blockIdx.x * n_waves + wave) * (EPI == MID_GATED ? 1 : TN);
    const int n_lo0 = tile0 * 16;
    const size_t tile_size = (size_t)(K / 32) * 512;
    const bf16_t* wtile[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        // tiles past the end repeat the last one; their results are dropped
        const int tile = EPI == MID_GATED ? t * part_tiles + min(tile0, part_tiles - 1) : min(tile0 + t, part_tiles - 1);
        wtile[t] = p.w + (size_t)tile * tile_size + lane * 8;
    }
    // Up to 4 row groups: a thread's pieces of a chunk of x are those at its number plus multiples of
    // the block's size; rows past M repeat the last row.  Pieces past the chunk's end (whole waves
    // of them, with more than 4 waves) are loaded again and not stored.
    const bf16_t* xsrc[WIDE ? 1 : XS];
    int xk[WIDE ? 1 : XS];
    if constexpr (!WIDE) {
#pragma unroll
        for (int i = 0; i < XS; ++i) {
            const int s = min((int)threadIdx.x + i * (int)blockDim.x, SLOTS - 1);
            const int mt = s / 256, ks = (s / 64) % 4, ln = s % 64;
            xk[i] = ks * 32 + (ln / 16) * 8;
            xsrc[i] = p.x + (size_t)min(mt * 16 + ln % 16, p.M - 1) * K;
        }
    }
    // 8 row groups: the block's first 256 threads bring x in, thread t piece t ([k step][lane]) of
    // every row group, so that its pieces lie 16 rows apart and need one address; in a block of 8
    // waves the second 256 threads take every other row group (PAR = 2).
    const int st_half = threadIdx.x / 256;
    const bool stages = st_half < PAR;
    const int st_row = threadIdx.x % 16, st_k = ((threadIdx.x / 64) % 4) * 32 + ((threadIdx.x % 64) / 16) * 8;
    floatx4_t acc[TN][MT];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // Loads past the end of K stay inside the row (and are valid memory); x is zeroed there as it
    // goes into LDS, so they add nothing.  Nothing is under a condition: the waits can be counted.
    // (Measured: with the loads of a wave whose pieces all lie past the chunk left out under a
    // condition, the compiler waits for all loads at every use, and a step of 64 rows at the 7B
    // sizes takes 16.6 ms instead of 4.1.)
    auto load_x = [&](int c, u32x4_t (&xr)[XS]) {
        if constexpr (WIDE) {
            if (!stages) return;
            const uint32_t kk = (uint32_t)min(c + st_k, K - 8);
#pragma unroll
            for (int i = 0; i < XS; ++i) {
                const uint32_t r = (uint32_t)min((i * PAR + st_half) * 16 + st_row, p.M - 1);
                xr[i] = *reinterpret_cast<const u32x4_t*>(p.x + (r * (uint32_t)K + kk));
            }
        } else {
#pragma unroll
            for (int i = 0; i < XS; ++i) xr[i] = *reinterpret_cast<const u32x4_t*>(xsrc[i] + min(c + xk[i], K - 8));
        }
    };
    auto store_x = [&](int c, int buf, const u32x4_t (&xr)[XS]) {
        if constexpr (WIDE) {
            if (!stages) return;
            const bool past = c + st_k >= k_end;
#pragma unroll
            for (int i = 0; i < XS; ++i) xs[buf * SLOTS + (i * PAR + st_half) * 256 + threadIdx.x % 256] = past ? u32x4_t{0, 0, 0, 0} : xr[i];
        } else {
#pragma unroll
            for (int i = 0; i < XS; ++i) {
                u32x4_t v = xr[i];
                if (c + xk[i] >= k_end) v = u32x4_t{0, 0, 0, 0};
                const int s = threadIdx.x + i * blockDim.x;
                if (s < SLOTS) xs[buf * SLOTS + s] = v;
            }
        }
    };
    auto load_w = [&](int c, bf16x8_t (&a)[TN][4]) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t at = (size_t)min(c / 32 + u, K / 32 - 1) * 512;
#pragma unroll
            for (int t = 0; t < TN; ++t) a[t][u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wtile[t] + at));      // read once
        }
    };
    // x comes from LDS four row groups at a time (two where registers are short), the next ones on
    // their way while these are multiplied.
    // RING (8 row groups, where registers are short): a k step's weight registers are asked for
    // again, for the chunk after those under way, as soon as its products are issued, so that two
    // register sets keep nearly two chunks on their way.
    constexpr bool RING = WIDE;
    auto multiply = [&](int buf, bf16x8_t (&a)[TN][4], int refill_c) {
        constexpr int G = RING && TN > 1 ? 2 : (MT < 4 ? MT : 4), NG = MT / G, STEPS = 4 * NG;
        u32x4_t bx[2][G];
#pragma unroll
        for (int g = 0; g < G; ++g) bx[0][g] = xs[buf * SLOTS + (g * 4) * 64 + lane];
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
            const int u = st / NG, grp = st % NG;
            if (st + 1 < STEPS) {
                const int u1 = (st + 1) / NG, grp1 = (st + 1) % NG;
#pragma unroll
                for (int g = 0; g < G; ++g) bx[(st + 1) & 1][g] = xs[buf * SLOTS + ((grp1 * G + g) * 4 + u1) * 64 + lane];
            }
#pragma unroll
            for (int g = 0; g < G; ++g)
#pragma unroll
                for (int t = 0; t < TN; ++t)
                    acc[t][grp * G + g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][u], __builtin_bit_cast(bf16x8_t, bx[st & 1][g]),
                                                                                  acc[t][grp * G + g], 0, 0, 0);
            if constexpr (RING) {
                if (grp == NG - 1) {
                    const size_t at = (size_t)min(refill_c / 32 + u, K / 32 - 1) * 512;
#pragma unroll
                    for (int t = 0; t < TN; ++t) a[t][u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wtile[t] + at));      // read once
                }
                __builtin_amdgcn_sched_barrier(0);       // or the reads of many steps are issued at once and held
            }
        }
    };

    // Chunk j is multiplied while the weights of chunks j+1 and j+2 and x of chunk j+2 are on their
    // way: what a step waits for was asked for two steps (weights) or one step (x, which comes
    // from the cache) earlier.  Three register sets of weights, two of x and two LDS buffers take
    // turns, so six steps are written out for the names to come round.
    // With 8 row groups the registers hold one set of x only: the next chunk's x is asked for at the
    // start of a step and stored at its end (XA = 1), and the weights go round as said above, in
    // two sets with two tiles per wave, in three with one.
    constexpr int XA = RING ? 1 : 2;
    constexpr int WA = RING && TN > 1 ? 2 : 3;
    bf16x8_t a[WA][TN][4];
    u32x4_t xr[XA][XS];
    load_w(k_begin, a[0]);
    load_w(k_begin + MID_CHUNK, a[1]);
    if constexpr (RING && WA == 3) load_w(k_begin + 2 * MID_CHUNK, a[WA - 1]);
    load_x(k_begin, xr[0]);
    if constexpr (XA == 2) load_x(k_begin + MID_CHUNK, xr[XA - 1]);
    store_x(k_begin, 0, xr[0]);
    __syncthreads();
#define MID_STEP(J) { \
        const int c = base + (J) * MID_CHUNK; \
        load_x(c + XA * MID_CHUNK, xr[XA == 2 ? (J) % 2 : 0]); \
        if constexpr (!RING) load_w(c + 2 * MID_CHUNK, a[((J) + 2) % WA]); \
        __builtin_amdgcn_sched_barrier(0); \
        multiply((J) % 2, a[(J) % WA], c + WA * MID_CHUNK); \
        store_x(c + MID_CHUNK, ((J) + 1) % 2, xr[XA == 2 ? ((J) + 1) % 2 : 0]); \
        __syncthreads(); }
    int base = k_begin, left = (k_end - k_begin + MID_CHUNK - 1) / MID_CHUNK;
    for (; left >= 6; left -= 6, base += 6 * MID_CHUNK) {
        MID_STEP(0) MID_STEP(1) MID_STEP(2) MID_STEP(3) MID_STEP(4) MID_STEP(5)
    }
    if (left > 0) {
        MID_STEP(0)
        if (left > 1) {
            MID_STEP(1)
            if (left > 2) {
                MID_STEP(2)
                if (left > 3) {
                    MID_STEP(3)
                    if (left > 4) MID_STEP(4)
                }
            }
        }
    }
#undef MID_STEP

    const int nb = 4 * kgrp;
    if (gridDim.y > 1) {
        const bool vec = p.N % 4 == 0 && n_out % 4 == 0;           // the up rows' sums start at n_out
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int m = mt * 16 + row;
                const int n = EPI == MID_GATED ? t * n_out + n_lo0 + nb : n_lo0 + 16 * t + nb;
                const int n_lim = EPI == MID_GATED ? t * n_out + n_out : p.N;
                if (m >= p.M) continue;
                float* dst = p.partial + ((size_t)blockIdx.y * p.M + m) * p.N + n;
                if (vec && n + 3 < n_lim) { *reinterpret_cast<floatx4_t*>(dst) = acc[t][mt]; continue; }
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < n_lim) dst[r] = acc[t][mt][r];
            }
        return;
    }
    if constexpr (EPI == MID_STORE) {
        TY* y = (TY*)p.y;
        const bool vec = p.N % 4 == 0;
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int m = mt * 16 + row;
                const int n = n_lo0 + 16 * t + nb;
                if (m >= p.M) continue;
                TY* dst = y + (size_t)m * p.N + n;
                if (vec && n + 3 < p.N) {
                    if constexpr (sizeof(TY) == 4) *reinterpret_cast<floatx4_t*>(dst) = acc[t][mt];
                    else *reinterpret_cast<uint2*>(dst) = pack4_bf16(acc[t][mt][0], acc[t][mt][1], acc[t][mt][2], acc[t][mt][3]);
                    continue;
                }
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < p.N) dst[r] = from_float<TY>(acc[t][mt][r]);
            }
    } else {
        bf16_t* y = (bf16_t*)p.y;
        const bool vec = n_out % 4 == 0;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + row;
            const int n = n_lo0 + nb;
            if (m >= p.M) continue;
            float o[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) o[r] = gate_times_up(acc[0][mt][r], acc[TN - 1][mt][r]);
            bf16_t* dst = y + (size_t)m * n_out + n;
            if (vec && n + 3 < n_out) { *reinterpret_cast<uint2*>(dst) = pack4_bf16(o[0], o[1], o[2], o[3]); continue; }
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < n_out) dst[r] = from_float<bf16_t>(o[r]);
        }
    }
}

// Adds the splits' sums in split order and finishes as the product kernel does without splits.
template <int EPI, typename TY>
__global__ void mid_finish_kernel(const float* __restrict__ partial, void* __restrict__ yv, int splits, int M, int N) {
    const int n_out = EPI == MID_GATED ? N / 2 : N;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)M * n_out) return;
    const int m = (int)(i / n_out), n = (int)(i % n_out);
    float a = 0.f, b = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float* src = partial + ((size_t)s * M + m) * N;
        a += src[n];
        if (EPI == MID_GATED) b += src[n_out + n];
    }
    if (EPI == MID_GATED) ((bf16_t*)yv)[i] = from_float<bf16_t>(gate_times_up(a, b));
    else ((TY*)yv)[i] = from_float<TY>(a);
}

// How a product of this shape is cut: tiles per wave, waves per block, splits of K.  From N and K
// alone.  Measured: the time is that of the compute unit with the most blocks, so the blocks
// should fall evenly on the 256 units, and about one block per unit streams fastest.
struct MidPlan { int tn, waves, blocks, splits, k_per_split; };
#define MID_UNITS 256

static MidPlan mid_plan(int N, int K, bool gated) {
    MidPlan plan;
    const int n_out = gated ? N / 2 : N;
    const int tiles = (n_out + 15) / 16;
    // two tiles per wave halve the reads of x from LDS, but also the waves: only where many are left
    plan.tn = gated ? 2 : (tiles >= 8192 ? 2 : 1);
    const int items = gated ? tiles : (tiles + plan.tn - 1) / plan.tn;        // what a wave takes
    const int chunks = (K + MID_CHUNK - 1) / MID_CHUNK;
    plan.waves = MID_MAX_WAVES;
    plan.splits = 1;
    if (items >= MID_UNITS * MID_MIN_WAVES) {
        // enough for every unit: the waves per block and rounds of blocks that leave the fewest idle
        double best = 0.0;
        for (int rounds = 1; rounds <= 8; ++rounds) {
            int waves = (items + MID_UNITS * rounds - 1) / (MID_UNITS * rounds);
            if (waves > MID_MAX_WAVES) continue;
            if (waves < MID_MIN_WAVES) waves = MID_MIN_WAVES;
            const double used = (double)items / ((double)MID_UNITS * rounds * waves);
            if (used > best + 0.02) { best = used; plan.waves = waves; }
        }
        plan.blocks = (items + plan.waves - 1) / plan.waves;
    } else {
        // Few features: K cut so that there is about a block per unit, no piece shorter than 4 chunks; and as many
        // waves per block (8 down to 4) as leave the fewest units without a block.  A unit alone pulls a 256th of what
        // the memory gives, so a product that covers a fifth of the units runs at a fifth of the rate whatever its
        // waves do (a width of 1536 and K of 1536: 36 blocks of 8 waves, 72 of 4).
        double best = 0.0;
        for (int waves = MID_MAX_WAVES; waves >= MID_MIN_WAVES; --waves) {
            const int blocks = (items + waves - 1) / waves;
            int splits = MID_UNITS / blocks;
            if (splits > chunks / 4) splits = chunks / 4;
            if (splits < 1) splits = 1;
            const int total = blocks * splits, rounds = (total + MID_UNITS - 1) / MID_UNITS;
            const double covered = (double)total / ((double)rounds * MID_UNITS);
            if (waves == MID_MAX_WAVES || covered > best + 0.02) { best = covered; plan.waves = waves; plan.blocks = blocks; plan.splits = splits; }
        }
    }
    if (gated && plan.splits > 1) {
        // A gated product in pieces needs a kernel of its own to add them up and apply the gate (4 to 5 us); where the
        // blocks of the whole K already cover half the units, that costs more than the pieces gain.  Estimated with a
        // unit pulling 34 GB/s and the memory giving 6.5 TB/s (a width of 1536 and 8960 gate rows, 55 MB: 15.4 us whole
        // against 13.9 + 4.6 in three pieces).
        const double bytes = 2.0 * (double)N * (double)K;
        auto time_us = [&](int blocks) { return 4.0 + bytes / (1e6 * (blocks * 0.034 < 6.5 ? blocks * 0.034 : 6.5)); };
        double best_whole = 1e30;
        int whole_waves = 0;
        for (int waves = MID_MAX_WAVES; waves >= MID_MIN_WAVES; --waves) {
            const int blocks = (items + waves - 1) / waves;
            if (blocks > MID_UNITS) continue;
            const double t = time_us(blocks);
            if (t < best_whole - 0.1) { best_whole = t; whole_waves = waves; }
        }
        if (whole_waves && best_whole < time_us(plan.blocks * plan.splits) + 4.6) {
            plan.waves = whole_waves;
            plan.blocks = (items + whole_waves - 1) / whole_waves;
            plan.splits = 1;
        }
    }
    const int per = (chunks + plan.splits - 1) / plan.splits;
    plan.splits = (chunks + per - 1) / per;             // no empty piece
    plan.k_per_split = per * MID_CHUNK;
    return plan;
}

/* Into how many pieces the product's K is cut (1: none, no scratch is needed). */
extern "C" int tqk_mid_max_rows(void) { return MID_MAX_ROWS; }

extern "C" int tqk_mid_splits(int N, int K, int gated) {
    if (N <= 0 || K <= 0) return 1;
    return mid_plan(N, K, gated != 0).splits;
}

static size_t mid_scratch_bytes(int M, int N, int K, bool gated) {
    const int splits = tqk_mid_splits(N, K, gated);
    return splits > 1 && M > 0 ? (size_t)splits * M * N * sizeof(float) : 0;
}

template <int MT, int TN, int EPI, typename TY>
static int launch_mid(const MidArgs& a, const MidPlan& plan, bool finish, hipStream_t s) {
    dim3 grid(plan.blocks, plan.splits);
    constexpr int PAR8 = (MT > 4) ? 2 : 1;
    if (PAR8 == 2 && plan.waves == MID_MAX_WAVES) mid_product_kernel<MT, TN, EPI, TY, PAR8><<<grid, plan.waves * TQK_WAVE, 2 * MT * 256 * 16, s>>>(a);
    else mid_product_kernel<MT, TN, EPI, TY, 1><<<grid, plan.waves * TQK_WAVE, 2 * MT * 256 * 16, s>>>(a);
    if (tqk_check_launch("tqk_mid product")) return -1;
    if (plan.splits > 1 && finish) {
        const size_t total = (size_t)a.M * (EPI == MID_GATED ? a.N / 2 : a.N);
        mid_finish_kernel<EPI, TY><<<(unsigned)((total + 255) / 256), 256, 0, s>>>(a.partial, a.y, plan.splits, a.M, a.N);
        return tqk_check_launch("tqk_mid finish");
    }
    return 0;
}

template <int EPI, typename TY>
static int launch_rows(const MidArgs& a, const MidPlan& plan, bool finish, hipStream_t s) {
    if constexpr (EPI == MID_GATED) {
        if (a.M > 64) return launch_mid<8, 2, EPI, TY>(a, plan, finish, s);
        return a.M > 32 ? launch_mid<4, 2, EPI, TY>(a, plan, finish, s) : launch_mid<2, 2, EPI, TY>(a, plan, finish, s);
    } else {
        if (a.M > 64) return plan.tn == 2 ? launch_mid<8, 2, EPI, TY>(a, plan, finish, s) : launch_mid<8, 1, EPI, TY>(a, plan, finish, s);
        if (a.M > 32) return plan.tn == 2 ? launch_mid<4, 2, EPI, TY>(a, plan, finish, s) : launch_mid<4, 1, EPI, TY>(a, plan, finish, s);
        return plan.tn == 2 ? launch_mid<2, 2, EPI, TY>(a, plan, finish, s) : launch_mid<2, 1, EPI, TY>(a, plan, finish, s);
    }
}

static int check_mid(const MidArgs& a, const void* scratch, bool gated, bool finish, const char* what) {
    TQK_REQUIRE(a.x && a.w, "%s: null pointer", what);
    TQK_REQUIRE(a.y || (!finish && tqk_mid_splits(a.N, a.K, gated) > 1), "%s: null output", what);
    TQK_REQUIRE(a.M >= 0 && a.M <= MID_MAX_ROWS, "%s: M=%d rows, this kernel takes at most %d", what, a.M, MID_MAX_ROWS);
    TQK_REQUIRE(a.N > 0 && a.K > 0 && a.K % 32 == 0, "%s: K=%d must be a positive multiple of 32 (N=%d)", what, a.K, a.N);
    TQK_REQUIRE(!gated || a.N % 2 == 0, "%s: odd N=%d", what, a.N);
    TQK_REQUIRE(((((uintptr_t)a.x) | ((uintptr_t)a.w) | ((uintptr_t)a.y) | ((uintptr_t)scratch)) & 15) == 0,
                "%s: x, w, y and scratch must be 16-byte aligned", what);
    TQK_REQUIRE(scratch || mid_scratch_bytes(a.M, a.N, a.K, gated) == 0, "%s: no scratch given", what);
    return 0;
}

/* y[M,N] = x w^T, M <= 128, w packed; scratch: float32 [tqk_mid_splits(N, K, 0)][M][N] where that
 * is more than 1.  finish == 0: with more than one piece the pieces' sums are left in scratch
 * (for tqk_add_rmsnorm_sums) and y is not written. */
extern "C" int tqk_mid_store(const void* x, const void* w_packed, void* y, int y_dtype, int M, int N, int K,
                             void* scratch, int finish, void* stream) {
    MidArgs a = {(const bf16_t*)x, (const bf16_t*)w_packed, y, (float*)scratch, M, N, K, 0};
    if (check_mid(a, scratch, false, finish != 0, "tqk_mid_store")) return -1;
    TQK_REQUIRE(y_dtype == TQK_F32 || y_dtype == TQK_BF16, "tqk_mid_store: unknown output dtype %d", y_dtype);
    if (M == 0) return 0;
    const MidPlan plan = mid_plan(N, K, false);
    a.k_per_split = plan.k_per_split;
    hipStream_t s = (hipStream_t)stream;
    return y_dtype == TQK_F32 ? launch_rows<MID_STORE, float>(a, plan, finish != 0, s)
                              : launch_rows<MID_STORE, bf16_t>(a, plan, finish != 0, s);
}

/* y[M, N/2] = silu(gate) * up, w = gate rows then up rows, packed in two parts. */
extern "C" int tqk_mid_gated(const void* x, const void* w_packed, void* y, int M, int N, int K, void* scratch, void* stream) {
    MidArgs a = {(const bf16_t*)x, (const bf16_t*)w_packed, y, (float*)scratch, M, N, K, 0};
    if (check_mid(a, scratch, true, true, "tqk_mid_gated")) return -1;
    if (M == 0) return 0;
    const MidPlan plan = mid_plan(N, K, true);
    a.k_per_split = plan.k_per_split;
    return launch_rows<MID_GATED, bf16_t>(a, plan, true, (hipStream_t)stream);
}
