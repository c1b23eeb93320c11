// Attention for prompts (and any step with many tokens per sequence): causal softmax
// attention of a tile of consecutive queries of one sequence over the sequence's pages of
// the cache, flash style: one pass over the keys, running maximum and sum, float32 softmax,
// bfloat16 MFMA products.  Formulas as src/models/turbo_generic.rs:1620-1631 and :56-62; the
// mask is right for queries that start at any position (the reference's is only for
// position 0, :1937-1956), with an optional window.
//
// Work of a block: one tile of queries, one kv head, and the query heads that share it (up
// to 256 / tile of them; more are split over blocks): a page of keys and values is staged
// in LDS once and serves all those heads, where the reference expands keys and values per
// query head (src/models/turbo_generic.rs:195-204).  The columns (head, query) of the block
// are dealt out 32 to a wave.  LDS holds two pages: the next page travels from global
// memory into registers while this one is computed on and is written to the other buffer
// afterwards, so a page costs one barrier.
//
// A prompt of a thousand or two tokens gives a block or two per compute unit, the last tile's block
// walks the most pages, and once the short blocks are gone its waves are alone on their SIMDs, where
// a page takes a wave nearly as long as it takes each of two waves that share a SIMD.  Such steps run
// with two sets of waves per block (SPLIT = 2): both sets hold the same columns, the first set takes
// the first 32 keys of every page and the second set the other 32, and the sets' running maxima, sums
// and outputs are put together through LDS at the end.  A page then costs a wave one tile instead of
// two (1024 tokens: 30.8 -> 28.5 us, 2048 tokens: 61.9 -> 60.9 with 7 heads a group of size 128);
// with more blocks than two per unit the later meeting of eight waves at the barrier costs more than
// that gains, and the step runs with one set.
//
// Matrix-core mapping, v_mfma_f32_32x32x16_bf16 (D[32x32] += A[32x16] B[16x32]; a lane
// holds of A row l%32 and the 8 k starting at 8*(l/32), of B the same k of column l%32, of
// D column l%32 and the rows 8*(i/4) + 4*(l/32) + i%4, i = 0..15):
//   scores^T[key][column] = K[key][:] . Q^T[:][column]   A = keys from LDS, B = the queries, kept in registers
//   out^T[element][column] = V^T[element][key] . P^T[key][column]
// The probabilities never move: the lane's registers 8s..8s+7 of a score tile are the B
// operand of step s of the second product, if the keys are dealt to the rows of the first
// product so that those registers hold the 8 keys whose values lie together in the cache
// (the cache keeps values transposed with the positions of a page in the order
// value_place of common.h): row r = 8a + 4h + j of a tile of 32 keys is key
// 4*(2*(a/2) + h) + 16*(a%2) + j.
//
// In LDS a row of keys takes 64, 128 or 256 bytes (head sizes 32, 64, 96 and 128; 96 is
// padded), a row of values 128; the 16-byte pieces of a row are XOR-swizzled so that the lanes
// of a read phase meet different banks.
//
// Softmax in base 2 (c = scale * log2 e): p = 2^(s*c - m).  The running maximum m is
// raised only when a score exceeds it by more than 2^8 (then out and sum are rescaled);
// until then p may be up to 2^8, which float32 sums and bfloat16 products carry as well.
#include "common.h"
#include "tq_kernels.h"
#include <type_traits>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
// pointers into LDS, typed as such: the compiler then tells the page being read from the page
// under way (restrict) and does not make the reads wait for the loads
typedef __attribute__((address_space(3))) unsigned char lds_byte;
typedef __attribute__((address_space(3))) bf16x8_t lds_bf16x8;
typedef __attribute__((address_space(3))) uint16_t lds_u16;
typedef __attribute__((address_space(3))) u32x4_t lds_u32x4;

#define PF_MAX_WAVES 8
#define PF_LAZY 8.0f            // how far (in powers of two) a score may exceed the running maximum before it is raised

namespace {

// the key (0..31) that row r of a score tile holds
__device__ __forceinline__ int tile_key(int r) {
    const int a = r >> 3, h = (r >> 2) & 1, j = r & 3;
    return 4 * (2 * (a >> 1) + h) + 16 * (a & 1) + j;
}

template <int D>
struct Layout {
    static constexpr int KROW = D <= 32 ? 64 : (D <= 64 ? 128 : 256);    // bytes of a key row in LDS
    static constexpr int K_BYTES = 64 * KROW;
    static constexpr int V_BYTES = D * 128;
    // Where piece c of key row `key` lies, and where the 8 places pc*8.. of value row d (byte offsets
    // inside a buffer).  Rows lie one after the other; the pieces of a row are XOR-swizzled with
    // bits of the row's number, chosen so that the lanes that read together (8 or 16 lanes with
    // consecutive rows of one tile of 32, see tile_key) meet different banks, whether a read phase
    // covers 128 or 256 bytes of banks.
    __device__ static __forceinline__ int k_at(int key, int c) {
        const int f = KROW == 256 ? ((key & 7) | (((key >> 4) & 1) << 3))
                    : KROW == 128 ? ((key & 7) ^ ((key >> 4) & 1))
                                  : (((key >> 1) & 3) ^ ((key >> 4) & 1));
        return key * KROW + ((c ^ f) << 4);
    }
    __device__ static __forceinline__ int v_at(int d, int pc) {
        return d * 128 + ((pc ^ ((d & 7) ^ ((d >> 3) & 1))) << 4);
    }
};

struct PrefillArgs {
    const bf16_t* q;
    const bf16_t* keys;
    const bf16_t* values;
    const int32_t* tok_pos;
    const int32_t* page_table;
    int table_width;
    const int32_t* tile_seq;
    const int32_t* tile_tok0;
    const int32_t* tile_count;
    const int32_t* seq_start;
    const int32_t* seq_new;
    int window;
    float scale;
    bf16_t* out;
    int n_heads, n_kv_heads, n_tiles;
    int tq_shift;            // log2 of the queries per tile
    int heads_per_block, head_chunks;
    int col_waves;           // waves that hold the block's columns; with SPLIT = 2 the block has twice as many
    int snake_width;
};

// What a wave knows about its place in the block's tile, and what it carries from page to page.
template <int D>
struct Wave {
    static constexpr int KS = D / 16;           // k steps of the score product
    static constexpr int DT = D / 32;           // tiles of 32 elements of the output
    int tid, n_threads, wave, n_waves, lane, c32, h;
    int set;                                     // SPLIT = 2: which 32 keys of every page this wave takes
    int kvh;
    int my_pos, my_lo;                           // this lane's query and the first key it sees
    bool wave_live;
    int wave_first, wave_last, wave_lo, wave_lo_last;
    int seq_end, last_page;
    float c2;
    const bf16_t* keys;
    const bf16_t* values;
    size_t page_stride;
    // Where this lane's operands lie in a page's buffer (byte offsets): the keys' pieces of step ks of a tile's first
    // row, and the values' pieces of step st of tile t, of the first 32 elements.  Worked out once and held as they
    // are: a read's address is then one of these registers plus a constant that is part of the instruction.
    int k_off[KS], v_off[2][2];
    bf16x8_t bq[KS];                             // the queries: B operand of the score product
    // The running maximum m that the exponents are set against (0 while the column has no key yet), the running sum l,
    // and how far a score must pass m to raise it: PF_LAZY, and -inf while there is no key yet (any score then does).
    float m, l, pass;
    floatx16_t o[DT];
};

// A page travels in two legs: from global memory into registers (fetch_page: 16 bytes a lane and
// load, asked for before the work on the page before it and waited for after), and from there into
// LDS (stage_page), each piece to its swizzled place.  Piece i of the keys is piece i % (D/8) of
// key row i / (D/8); piece i of the values holds places 8 (i % 8) .. of element row i / 8.
template <int D>
__device__ __forceinline__ void fetch_page(const Wave<D>& w, int page, u32x4_t (&kr)[D / 32], u32x4_t (&vr)[D / 32]) {
    const size_t base = (size_t)(page < 0 ? 0 : page) * w.page_stride + (size_t)w.kvh * TQK_PAGE * D;
    const u32x4_t* kg = reinterpret_cast<const u32x4_t*>(w.keys + base);
    const u32x4_t* vg = reinterpret_cast<const u32x4_t*>(w.values + base);
    const int wave_first = __builtin_amdgcn_readfirstlane(w.tid);
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
        // a wave whose pieces all lie beyond the page asks for nothing: a load of nothing takes the wave's turn at the
        // compute unit's memory port as long as a load of a kilobyte (a block of eight waves: every other load)
        if (wave_first + c * w.n_threads >= 8 * D) continue;
        const int i = min(w.tid + c * w.n_threads, 8 * D - 1);      // (lanes beyond the page: its last piece again, not stored)
        kr[c] = kg[i];
        vr[c] = vg[i];
    }
}

template <int D>
__device__ __forceinline__ void stage_page(const Wave<D>& w, const u32x4_t (&kr)[D / 32], const u32x4_t (&vr)[D / 32],
                                           lds_byte* __restrict__ kd, lds_byte* __restrict__ vd) {
    using L = Layout<D>;
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
        const int i = w.tid + c * w.n_threads;
        if (i < 8 * D) {
            *(lds_u32x4*)(kd + L::k_at(i / (D / 8), i % (D / 8))) = kr[c];
            *(lds_u32x4*)(vd + L::v_at(i >> 3, i & 7)) = vr[c];
        }
    }
}

// The work on one page, held in kc, vc.
template <int D, int SPLIT>
__device__ __forceinline__ void page_step(Wave<D>& w, int pg, int page_now, lds_byte* __restrict__ kc, lds_byte* __restrict__ vc) {
    using L = Layout<D>;
    constexpr int KS = Wave<D>::KS, DT = Wave<D>::DT;
    const int key0 = pg * TQK_PAGE;
    const int c32 = w.c32, h = w.h;
    if (key0 + TQK_PAGE > w.seq_end) {
        // the page holds places beyond the sequence: whatever is stored there must not count,
        // not even with probability 0 (0 * NaN); their values become zeros
        const int valid = w.seq_end - key0;
        for (int e = w.tid; e < D * 8; e += w.n_threads) {
            const int d = e >> 3, pc = e & 7;
            lds_u16* at = (lds_u16*)(vc + L::v_at(d, pc));
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (value_position(pc * 8 + i) >= valid) at[i] = 0;
        }
        __syncthreads();
    }
    if (!w.wave_live || page_now < 0) return;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        // a tile of 32 keys at a time
        const int k0 = key0 + 32 * t;
        if (SPLIT == 2 && t != w.set) continue;
        if (k0 > w.wave_last || k0 + 31 < w.wave_lo) continue;
        // all operands of the tile's score product first, so that their reads are under way together
        bf16x8_t ka[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) ka[ks] = *(lds_bf16x8*)(kc + 32 * t * L::KROW + w.k_off[ks]);
        __builtin_amdgcn_sched_barrier(0);
        floatx16_t s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[ks], w.bq[ks], s, 0, 0, 0);
        // and the values of the second product, which arrive during the softmax
        bf16x8_t va[2][DT];
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) va[st][dt] = *(lds_bf16x8*)(vc + 32 * dt * 128 + w.v_off[t][st]);
        __builtin_amdgcn_sched_barrier(0);
        // the mask is needed only on tiles that cross a query's causal or window edge
        const bool need_mask = k0 + 31 > w.wave_first || k0 < w.wave_lo_last;
        if (need_mask) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int a = i >> 2;
                const int j = k0 + 4 * (2 * (a >> 1) + h) + 16 * (a & 1) + (i & 3);
                if (j < w.my_lo || j > w.my_pos) s[i] = -INFINITY;
            }
        }
        // The scores against the running maximum as it stands, in powers of two: t = s c - m.  Nearly always they are
        // the exponents already; the largest of them says whether the maximum has to be raised first.  (The maximum
        // is taken of these, not of the raw scores: a product of the matrix cores would have to be made canonical
        // value by value before a maximum may look at it.)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = fmaf(s[i], w.c2, -w.m);
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i += 2) mx = fmaxf(mx, fmaxf(s[i], s[i + 1]));
        {
            // the column's other 16 keys, held by the lane 32 further on: the two halves of the wave change places in
            // the registers themselves (v_permlane32_swap), no trip through LDS
            const auto both = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
            mx = fmaxf(__uint_as_float(both[0]), __uint_as_float(both[1]));
        }
        const bool raise = mx > w.pass;
        if (__any(raise)) {
            const float up = raise ? mx : 0.f;                 // by how much
            // (a column's first key may lie below 0, the maximum's stand-in until then: out and l are 0 there, and alpha
            // must only stay finite)
            const float alpha = __builtin_amdgcn_exp2f(-fmaxf(up, 0.f));
            w.m += up;
            if (raise) w.pass = PF_LAZY;
            w.l *= alpha;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) w.o[dt][i] *= alpha;
#pragma unroll
            for (int i = 0; i < 16; ++i) s[i] -= up;
        }
        // (a column without a key so far: every t is -inf and every p is 2^(-inf) = 0)
        bf16x8_t pb[2];
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float pr = __builtin_amdgcn_exp2f(s[i]);
            psum += pr;
            pb[i >> 3][i & 7] = (__bf16)pr;
        }
        w.l += psum;
        // out^T += V^T P^T: step st takes the lane's registers 8 st .. 8 st + 7 and the 16 bytes of
        // values that hold the same keys
        // (at a higher priority than the vector work of the SIMD's other wave: its operands are all there, and the
        // sooner the chain is under way the sooner the matrix cores work beside that wave's softmax; 8192 tokens in
        // tiles of 64: 528 -> 514 us)
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) w.o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[st][dt], pb[st], w.o[dt], 0, 0, 0);
        __builtin_amdgcn_s_setprio(0);
    }
}

// What the second set of waves hands to the first at the end, a tile of 32 output elements at a time: 16 values a
// lane, and with the first tile the running maximum and sum.  [value][column wave][lane]: the lanes' words lie side by side.
#define PF_SPLIT_COL_WAVES 4
#define PF_HANDOVER_BYTES (18 * PF_SPLIT_COL_WAVES * TQK_WAVE * 4)

template <int D, int SPLIT>
__global__ __launch_bounds__(PF_MAX_WAVES * TQK_WAVE)
void attention_prefill_kernel(const PrefillArgs p) {
    using L = Layout<D>;
    constexpr int KS = Wave<D>::KS, DT = Wave<D>::DT;
    constexpr int PAGES_BYTES = 2 * L::K_BYTES + 2 * L::V_BYTES;
    constexpr int LDS_BYTES = SPLIT == 2 && PAGES_BYTES < PF_HANDOVER_BYTES ? PF_HANDOVER_BYTES : PAGES_BYTES;
    __shared__ __attribute__((aligned(1024))) unsigned char lds[LDS_BYTES];
    lds_byte* const kb = (lds_byte*)lds;
    lds_byte* const vb = kb + 2 * L::K_BYTES;

    Wave<D> w;
    w.tid = threadIdx.x;
    w.n_threads = blockDim.x;
    w.wave = w.tid / TQK_WAVE;
    w.lane = w.tid % TQK_WAVE;
    w.n_waves = blockDim.x / TQK_WAVE;
    w.c32 = w.lane & 31;
    w.h = w.lane >> 5;
    // the wave's place among those that hold columns
    const int cw = SPLIT == 2 ? w.wave % p.col_waves : w.wave;
    w.set = SPLIT == 2 ? __builtin_amdgcn_readfirstlane(w.wave / p.col_waves) : 0;

    // Blocks in the order of their work (the host lists the tiles longest first), kv heads and
    // head chunks fastest.  With snake_width > 0 every other run of snake_width blocks is taken
    // backwards: when all blocks are resident at once, the compute units that got the longest
    // get the shortest next.
    const int per_tile = p.n_kv_heads * p.head_chunks;
    int order = blockIdx.x;
    if (p.snake_width > 0) {
        const int total = p.n_tiles * per_tile;
        const int round = order / p.snake_width, first = round * p.snake_width;
        const int size = min(p.snake_width, total - first);
        if (round & 1) order = first + size - 1 - (order - first);
    }
    const int tile = order / per_tile, chunk = order % p.head_chunks;
    w.kvh = (order % per_tile) / p.head_chunks;
    const int n_rep = p.n_heads / p.n_kv_heads;
    const int head0 = w.kvh * n_rep + chunk * p.heads_per_block;
    const int heads_here = min(p.heads_per_block, n_rep - chunk * p.heads_per_block);
    const int seq = p.tile_seq[tile], tok0 = p.tile_tok0[tile], count = p.tile_count[tile];
    const int pos0 = p.tok_pos[tok0];
    w.seq_end = p.seq_start[seq] + p.seq_new[seq];       // positions the cache holds after this step
    const int tq = 1 << p.tq_shift;

    // this lane's column: a query of a head
    const int col = cw * 32 + w.c32;
    const int head_local = col >> p.tq_shift, qi = col & (tq - 1);
    const bool live = head_local < heads_here && qi < count;
    const int head = head0 + (live ? head_local : 0);
    w.my_pos = live ? pos0 + qi : -1;
    w.my_lo = p.window > 0 ? max(0, w.my_pos - p.window + 1) : 0;
    // the wave's range of queries (the same for all its heads)
    const int wq_first = (cw * 32) & (tq - 1);
    const int wq_last = min(tq >= 32 ? wq_first + 31 : tq - 1, count - 1);
    // (the same in all lanes of the wave, and said so: what is decided from them is then decided once per wave, by
    // scalar compares and branches)
    w.wave_live = __builtin_amdgcn_readfirstlane((cw * 32 >> p.tq_shift) < heads_here && wq_first < count);
    w.wave_first = __builtin_amdgcn_readfirstlane(pos0 + wq_first);
    w.wave_last = __builtin_amdgcn_readfirstlane(pos0 + wq_last);
    w.wave_lo = p.window > 0 ? max(0, w.wave_first - p.window + 1) : 0;            // first key any of its queries sees
    w.wave_lo_last = p.window > 0 ? max(0, w.wave_last - p.window + 1) : 0;        // first key all of them see
    w.c2 = p.scale * 1.44269504088896340736f;
    const int tile_lo = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
    const int first_page = tile_lo / TQK_PAGE;
    w.last_page = (pos0 + count - 1) / TQK_PAGE;
    w.keys = p.keys;
    w.values = p.values;
    w.page_stride = (size_t)p.n_kv_heads * TQK_PAGE * D;

    const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    {
        const bf16_t* qrow = p.q + ((size_t)(tok0 + (live ? qi : 0)) * p.n_heads + head) * D + w.h * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) w.bq[ks] = live ? *reinterpret_cast<const bf16x8_t*>(qrow + ks * 16) : zero8;
    }
    {
        // (the swizzles of k_at and v_at look only at bits of the row's number that the tile's and the element tile's
        // first rows, multiples of 32, leave alone)
        const int krow = tile_key(w.c32);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            w.k_off[ks] = L::k_at(krow, 2 * ks + w.h);
            asm volatile("" : "+v"(w.k_off[ks]));
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                w.v_off[t][st] = L::v_at(w.c32, 4 * t + 2 * st + w.h);
                asm volatile("" : "+v"(w.v_off[t][st]));
            }
    }
    w.m = 0.f;
    w.pass = -INFINITY;
    w.l = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) w.o[dt][i] = 0.f;

    // Two buffers: while a page is worked on, the next one is on its way into registers, and goes
    // into the other buffer afterwards; one barrier per page.
    // The numbers of the pages are read 64 at a time, a lane each, and handed round inside the wave: a
    // page's loads then do not wait for the load of its number, which would cost a trip to memory per page.
    const int32_t* pages = p.page_table + (size_t)seq * p.table_width;
    int my_pages = pages[min(first_page + w.lane, w.last_page)];
    u32x4_t kr[D / 32], vr[D / 32];
    int page_now = __builtin_amdgcn_readfirstlane(__shfl(my_pages, 0, TQK_WAVE));
    fetch_page<D>(w, page_now, kr, vr);
    stage_page<D>(w, kr, vr, kb, vb);
    // The loop is written out for its two buffers (the first page lies in the first one): which buffer a
    // read or write goes to is then part of the instruction, not an addition in front of each of them.
    int pg = first_page;
    auto one_page = [&](auto which) {
        constexpr int cur = decltype(which)::value;
        __syncthreads();                      // the page is whole; all are done with the other buffer
        int page_next = -1;
        if (pg < w.last_page) {
            const int ahead = (pg + 1 - first_page) & (TQK_WAVE - 1);
            if (ahead == 0) my_pages = pages[min(pg + 1 + w.lane, w.last_page)];
            page_next = __builtin_amdgcn_readfirstlane(__shfl(my_pages, ahead, TQK_WAVE));
            fetch_page<D>(w, page_next, kr, vr);
        }
        page_step<D, SPLIT>(w, pg, page_now, kb + cur * L::K_BYTES, vb + cur * L::V_BYTES);
        if (pg < w.last_page) stage_page<D>(w, kr, vr, kb + (cur ^ 1) * L::K_BYTES, vb + (cur ^ 1) * L::V_BYTES);
        page_now = page_next;
        ++pg;
    };
    while (pg <= w.last_page) {
        one_page(std::integral_constant<int, 0>());
        if (pg > w.last_page) break;
        one_page(std::integral_constant<int, 1>());
    }
    if constexpr (SPLIT == 2) {
        // The second set's columns saw the other keys: out = (o0 2^(m0 - m) + o1 2^(m1 - m)) / (l0 2^(m0 - m) + l1 2^(m1 - m)),
        // m the larger of the two maxima (a set that saw no key has m = -inf and counts for nothing).
        __attribute__((address_space(3))) float* hand = (__attribute__((address_space(3))) float*)lds + cw * TQK_WAVE + w.lane;
        constexpr int STEP = PF_SPLIT_COL_WAVES * TQK_WAVE;
        float mine = 1.f, theirs = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            __syncthreads();                  // all are done with the pages (or with the tile handed over before)
            if (w.set == 1) {
#pragma unroll
                for (int i = 0; i < 16; ++i) hand[i * STEP] = w.o[dt][i];
                if (dt == 0) {
                    hand[16 * STEP] = w.pass == -INFINITY ? -INFINITY : w.m;
                    hand[17 * STEP] = w.l;
                }
            }
            __syncthreads();
            if (w.set == 0) {
                if (dt == 0) {
                    const float m1 = hand[16 * STEP], l1 = hand[17 * STEP];
                    const float m0 = w.pass == -INFINITY ? -INFINITY : w.m;
                    const float m = fmaxf(m0, m1);
                    mine = m0 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m0 - m);
                    theirs = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m1 - m);
                    w.l = w.l * mine + l1 * theirs;
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) w.o[dt][i] = w.o[dt][i] * mine + hand[i * STEP] * theirs;
            }
        }
    }
    float l = w.l;
    l += __shfl_xor(l, 32, TQK_WAVE);
    if (live && w.set == 0) {
        // out^T[element 32 dt + 8 (i/4) + 4 h + i%4][this column]
        bf16_t* orow = p.out + ((size_t)(tok0 + qi) * p.n_heads + head) * D;
        const float inv = 1.f / l;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                uint16_t w4[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) w4[j] = float_to_bf16_bits(w.o[dt][4 * a + j] * inv);
                *reinterpret_cast<uint2*>(orow + 32 * dt + 8 * a + 4 * w.h) =
                    make_uint2((uint32_t)w4[0] | ((uint32_t)w4[1] << 16), (uint32_t)w4[2] | ((uint32_t)w4[3] << 16));
            }
    }
}

}  // namespace

// Up to this many blocks per compute unit a step runs with two sets of waves per block.  Measured with 7 heads a
// group and head size 128, causal prompts alone, one set against two: 1024 tokens (one block a unit) 29.7 -> 27.0 us,
// 1536 tokens 43.4 -> 37.3, 2048 tokens (two blocks a unit) 56.4 -> 54.6, 4096 tokens (four) 178 -> 191.
#define PF_SPLIT_BLOCKS_PER_CU 2
#define PF_SPLIT_MIN_TOKENS 512         // new tokens a sequence, on average
extern "C" int tqk_attention_prefill_supported(int head_dim) {
    return head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128;
}

// Heads of a group that one block takes for tiles of tile_queries, and in how many chunks the
// group is then cut: as many heads as 8 waves of 32 columns hold, dealt out evenly.
static void prefill_heads(int n_rep, int tile_queries, int* heads_per_block, int* chunks) {
    const int most = 32 * PF_MAX_WAVES / tile_queries;
    *chunks = (n_rep + most - 1) / most;
    *heads_per_block = (n_rep + *chunks - 1) / *chunks;
}

static int prefill_compute_units(void) {
    static int n_cus = 0;
    if (n_cus == 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
            return 0;
        n_cus = v;
    }
    return n_cus;
}

/* Queries per tile that suit a step of n_tokens: tiles of 64 (a wave holds 32 queries of one
 * head, a block four heads) where that gives several blocks per compute unit to share out,
 * tiles of 16 (two heads a wave) for shorter steps; groups of few heads take longer tiles, so
 * that a block has at least four waves. */
extern "C" int tqk_attention_prefill_tile(int n_tokens, int n_heads, int n_kv_heads, int head_dim) {
    (void)head_dim;
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads) return 64;
    const int n_rep = n_heads / n_kv_heads;
    if (n_rep == 1) return 128;
    if (n_rep <= 3) return 64;
    int n_cus = prefill_compute_units();
    if (n_cus <= 0) n_cus = 256;
    int hb, chunks;
    prefill_heads(n_rep, 32, &hb, &chunks);
    const long long blocks32 = (long long)((n_tokens + 31) / 32) * n_kv_heads * chunks;
    // measured with groups of 7 heads of 128: 2048 tokens run fastest in tiles of 16 (512 blocks of
    // four waves), 8192 and more in tiles of 64 (blocks of 8 and 6 waves)
    if (blocks32 >= 2LL * n_cus) return 64;
    return n_rep == 4 ? 32 : 16;
}

extern "C" int tqk_attention_prefill(const void* q, const void* keys, const void* values, const int32_t* tok_pos,
                                     const int32_t* page_table, int table_width, int n_seqs, int n_pages,
                                     const int32_t* tile_seq, const int32_t* tile_tok0, const int32_t* tile_count,
                                     int n_tiles, int tile_queries, const int32_t* seq_start, const int32_t* seq_new,
                                     int window, float scale, void* out, int n_tokens, int n_heads, int n_kv_heads,
                                     int head_dim, void* stream) {
    TQK_REQUIRE(q && keys && values && tok_pos && page_table && tile_seq && tile_tok0 && tile_count && seq_start && seq_new && out,
                "tqk_attention_prefill: null pointer");
    TQK_REQUIRE(n_tokens >= 0 && n_tiles >= 0 && n_heads > 0 && n_kv_heads > 0, "tqk_attention_prefill: bad sizes");
    TQK_REQUIRE(n_heads % n_kv_heads == 0, "tqk_attention_prefill: %d heads are not a multiple of %d kv heads", n_heads, n_kv_heads);
    TQK_REQUIRE(tqk_attention_prefill_supported(head_dim), "tqk_attention_prefill: head_dim %d is not one of 32, 64, 96, 128", head_dim);
    TQK_REQUIRE(table_width > 0 && n_pages > 0 && n_seqs > 0, "tqk_attention_prefill: empty page table");
    TQK_REQUIRE(window >= 0, "tqk_attention_prefill: negative window");
    TQK_REQUIRE(tile_queries == 16 || tile_queries == 32 || tile_queries == 64 || tile_queries == 128,
                "tqk_attention_prefill: tiles hold 16, 32, 64 or 128 queries, not %d", tile_queries);
    TQK_REQUIRE((((uintptr_t)q | (uintptr_t)keys | (uintptr_t)values | (uintptr_t)out) & 15) == 0,
                "tqk_attention_prefill: q, keys, values and out must be 16-byte aligned");
    if (n_tiles == 0) return 0;
    PrefillArgs a;
    a.q = (const bf16_t*)q; a.keys = (const bf16_t*)keys; a.values = (const bf16_t*)values;
    a.tok_pos = tok_pos; a.page_table = page_table; a.table_width = table_width;
    a.tile_seq = tile_seq; a.tile_tok0 = tile_tok0; a.tile_count = tile_count;
    a.seq_start = seq_start; a.seq_new = seq_new; a.window = window; a.scale = scale;
    a.out = (bf16_t*)out; a.n_heads = n_heads; a.n_kv_heads = n_kv_heads; a.n_tiles = n_tiles;
    a.tq_shift = tile_queries == 16 ? 4 : (tile_queries == 32 ? 5 : (tile_queries == 64 ? 6 : 7));
    prefill_heads(n_heads / n_kv_heads, tile_queries, &a.heads_per_block, &a.head_chunks);
    // at least four waves: the page's journey through registers is dealt out to 256 threads or more
    a.col_waves = max(4, (a.heads_per_block * tile_queries + 31) / 32);
    const long long total = (long long)n_tiles * n_kv_heads * a.head_chunks;
    TQK_REQUIRE(total <= 0x7fffffffLL, "tqk_attention_prefill: %d tiles are more than the grid takes", n_tiles);
    const int n_cus = prefill_compute_units();
    TQK_REQUIRE(n_cus > 0, "tqk_attention_prefill: cannot read the number of compute units");
    // two sets of waves per block where the columns leave room for them and the blocks are few (see the top)
    // (and the sequences are long enough for the walk to outweigh the handing over at the end: 256 tokens 11.7 -> 12.8 us
    // with two sets, 512 tokens 17.7 -> 17.4, 1536 tokens 43.4 -> 37.3)
    const bool split = a.col_waves == PF_SPLIT_COL_WAVES && total <= (long long)PF_SPLIT_BLOCKS_PER_CU * n_cus &&
                       n_tokens >= PF_SPLIT_MIN_TOKENS * n_seqs;
    const int waves = split ? 2 * a.col_waves : a.col_waves;
    // Blocks that are all resident at once (a compute unit holds 8 such waves) are not shared out
    // as they finish: then the runs of one block per compute unit alternate their direction.
    const int per_cu = waves <= 4 ? 2 : 1;
    a.snake_width = (total > n_cus && total <= (long long)per_cu * n_cus) ? n_cus : 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)total);
#define LAUNCH(DD) do { if (split) attention_prefill_kernel<DD, 2><<<grid, waves * TQK_WAVE, 0, s>>>(a); \
                        else attention_prefill_kernel<DD, 1><<<grid, waves * TQK_WAVE, 0, s>>>(a); } while (0)
    switch (head_dim) {
        case 32: LAUNCH(32); break;
        case 64: LAUNCH(64); break;
        case 96: LAUNCH(96); break;
        case 128: LAUNCH(128); break;
    }
#undef LAUNCH
    return tqk_check_launch("tqk_attention_prefill");
}
