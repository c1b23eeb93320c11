// Small kernels the engine needs around the model's own: rows gathered by index, a bias added
// to every row, a weight copied into the few-row kernels' order, a change of dtype; and what
// the library says about itself (page size, how many rows its product kernels take).
#include "common.h"
#include "tq_kernels.h"

namespace {

// dst row r = src row rows[r]; a row is row_bytes bytes, moved in pieces of `unit` bytes
template <typename U>
__global__ __launch_bounds__(256)
void gather_rows_kernel(const U* __restrict__ src, const int32_t* __restrict__ rows, long long units_per_row, U* __restrict__ dst) {
    const long long r = blockIdx.y;
    const long long from = (long long)rows[r] * units_per_row, to = r * units_per_row;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < units_per_row; i += (long long)gridDim.x * blockDim.x)
        dst[to + i] = src[from + i];
}

template <typename T, typename B>
__global__ __launch_bounds__(256)
void add_bias_kernel(T* __restrict__ x, const B* __restrict__ bias, long long total, int n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x)
        x[i] = from_float<T>(to_float(x[i]) + to_float(bias[i % n]));
}

template <typename A, typename B>
__global__ __launch_bounds__(256)
void convert_kernel(const A* __restrict__ src, B* __restrict__ dst, long long n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
        dst[i] = from_float<B>(to_float(src[i]));
}

// out [parts * tiles][k / 32][64 lanes][8]: tile t of a part holds its rows 16 t .. 16 t + 15, lane =
// 16 * ((k % 32) / 8) + row % 16; rows beyond a part's last are zeros
__global__ __launch_bounds__(256)
void pack_weight_kernel(const uint16_t* __restrict__ w, uint16_t* __restrict__ out, int per, int k, int tiles, long long total) {
    const int ksteps = k / 32;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int j = (int)(i & 7);
        const int lane = (int)((i >> 3) & 63);
        const long long rest = i >> 9;
        const int kstep = (int)(rest % ksteps);
        const long long pt = rest / ksteps;             // part * tiles + tile
        const int tile = (int)(pt % tiles), part = (int)(pt / tiles);
        const int row = tile * 16 + (lane & 15);
        const int col = kstep * 32 + (lane >> 4) * 8 + j;
        out[i] = row < per ? w[((long long)part * per + row) * k + col] : (uint16_t)0;
    }
}

// The other way round, for products of many rows that go to the library: 16 rows x 512 columns a block (16 k steps
// of a tile: 16 KB that lie together in the packed copy), turned through LDS so that both the reads and the writes
// are runs of a kilobyte.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
#define UNPACK_KSTEPS 16
__global__ __launch_bounds__(256)
void unpack_weight_kernel(const u32x4_t* __restrict__ packed, u32x4_t* __restrict__ rows, int per, int k, int tiles) {
    __shared__ u32x4_t turn[16][UNPACK_KSTEPS * 4 + 1];           // [row][piece of 8 columns]; the odd pitch keeps the rows' banks apart
    const int ksteps = k / 32, ks0 = blockIdx.x * UNPACK_KSTEPS, n_ks = min(UNPACK_KSTEPS, ksteps - ks0);
    const long long pt = blockIdx.y;                               // part * tiles + tile
    for (int i = threadIdx.x; i < n_ks * 64; i += blockDim.x) {
        const int lane = i % 64;
        turn[lane % 16][(i / 64) * 4 + lane / 16] = packed[(pt * ksteps + ks0) * 64 + i];
    }
    __syncthreads();
    const int tile = (int)(pt % tiles), part = (int)(pt / tiles), pieces = n_ks * 4;
    for (int i = threadIdx.x; i < 16 * pieces; i += blockDim.x) {
        const int r = i / pieces, c = i % pieces, row = tile * 16 + r;
        if (row < per) rows[(((long long)part * per + row) * k + ks0 * 32) / 8 + c] = turn[r][c];
    }
}

int blocks_for(long long n) {
    const long long want = (n + 255) / 256;
    return (int)(want < 1 ? 1 : want > 65535 ? 65535 : want);
}

}  // namespace

extern "C" int tqk_page_size(void) { return TQK_PAGE; }

extern "C" int tqk_gather_rows(const void* src, const int32_t* rows, int n_rows, long long row_bytes, void* dst, void* stream) {
    TQK_REQUIRE(n_rows >= 0 && row_bytes >= 0, "tqk_gather_rows: bad sizes");
    if (n_rows == 0 || row_bytes == 0) return 0;
    TQK_REQUIRE(src && rows && dst, "tqk_gather_rows: null pointer");
    TQK_REQUIRE(n_rows <= 65535, "tqk_gather_rows: %d rows are more than the grid takes", n_rows);
    hipStream_t s = (hipStream_t)stream;
    const uintptr_t both = (uintptr_t)src | (uintptr_t)dst | (uintptr_t)row_bytes;
    if ((both & 15) == 0) {
        const long long units = row_bytes / 16;
        gather_rows_kernel<uint4><<<dim3(blocks_for(units) > 64 ? 64 : blocks_for(units), n_rows), 256, 0, s>>>((const uint4*)src, rows, units, (uint4*)dst);
    } else if ((both & 3) == 0) {
        const long long units = row_bytes / 4;
        gather_rows_kernel<uint32_t><<<dim3(blocks_for(units) > 64 ? 64 : blocks_for(units), n_rows), 256, 0, s>>>((const uint32_t*)src, rows, units, (uint32_t*)dst);
    } else {
        gather_rows_kernel<uint8_t><<<dim3(blocks_for(row_bytes) > 64 ? 64 : blocks_for(row_bytes), n_rows), 256, 0, s>>>((const uint8_t*)src, rows, row_bytes, (uint8_t*)dst);
    }
    return tqk_check_launch("tqk_gather_rows");
}

extern "C" int tqk_add_bias(void* x, int x_dtype, const void* bias, int bias_dtype, int n_rows, int n, void* stream) {
    TQK_REQUIRE(n_rows >= 0 && n > 0, "tqk_add_bias: bad sizes");
    if (n_rows == 0) return 0;
    TQK_REQUIRE(x && bias, "tqk_add_bias: null pointer");
    const long long total = (long long)n_rows * n;
    hipStream_t s = (hipStream_t)stream;
    const int b = blocks_for(total);
    if (x_dtype == TQK_F32 && bias_dtype == TQK_F32) add_bias_kernel<float, float><<<b, 256, 0, s>>>((float*)x, (const float*)bias, total, n);
    else if (x_dtype == TQK_F32 && bias_dtype == TQK_BF16) add_bias_kernel<float, bf16_t><<<b, 256, 0, s>>>((float*)x, (const bf16_t*)bias, total, n);
    else if (x_dtype == TQK_BF16 && bias_dtype == TQK_F32) add_bias_kernel<bf16_t, float><<<b, 256, 0, s>>>((bf16_t*)x, (const float*)bias, total, n);
    else if (x_dtype == TQK_BF16 && bias_dtype == TQK_BF16) add_bias_kernel<bf16_t, bf16_t><<<b, 256, 0, s>>>((bf16_t*)x, (const bf16_t*)bias, total, n);
    else return tqk_fail("tqk_add_bias: unknown dtype codes %d, %d", x_dtype, bias_dtype);
    return tqk_check_launch("tqk_add_bias");
}

extern "C" int tqk_convert(const void* src, int src_dtype, void* dst, int dst_dtype, long long n, void* stream) {
    TQK_REQUIRE(n >= 0, "tqk_convert: bad size");
    if (n == 0) return 0;
    TQK_REQUIRE(src && dst, "tqk_convert: null pointer");
    hipStream_t s = (hipStream_t)stream;
    const int b = blocks_for(n);
    if (src_dtype == TQK_F32 && dst_dtype == TQK_BF16) convert_kernel<float, bf16_t><<<b, 256, 0, s>>>((const float*)src, (bf16_t*)dst, n);
    else if (src_dtype == TQK_BF16 && dst_dtype == TQK_F32) convert_kernel<bf16_t, float><<<b, 256, 0, s>>>((const bf16_t*)src, (float*)dst, n);
    else if (src_dtype == TQK_F32 && dst_dtype == TQK_F32) convert_kernel<float, float><<<b, 256, 0, s>>>((const float*)src, (float*)dst, n);
    else if (src_dtype == TQK_BF16 && dst_dtype == TQK_BF16) convert_kernel<bf16_t, bf16_t><<<b, 256, 0, s>>>((const bf16_t*)src, (bf16_t*)dst, n);
    else return tqk_fail("tqk_convert: unknown dtype codes %d, %d", src_dtype, dst_dtype);
    return tqk_check_launch("tqk_convert");
}

extern "C" int tqk_unpack_weight(const void* packed, void* rows, int n, int k, int parts, void* stream) {
    TQK_REQUIRE(packed && rows, "tqk_unpack_weight: null pointer");
    TQK_REQUIRE(n > 0 && k > 0 && parts > 0 && k % 32 == 0 && n % parts == 0,
                "tqk_unpack_weight: needs bfloat16 [n, k] with k a multiple of 32 and n of %d parts, got [%d, %d]", parts, n, k);
    TQK_REQUIRE((((uintptr_t)packed | (uintptr_t)rows) & 15) == 0, "tqk_unpack_weight: both copies must be 16-byte aligned");
    const int per = n / parts, tiles = (per + 15) / 16;
    TQK_REQUIRE((long long)parts * tiles <= 65535, "tqk_unpack_weight: %d rows are more than the grid takes", n);
    dim3 grid((k / 32 + UNPACK_KSTEPS - 1) / UNPACK_KSTEPS, parts * tiles);
    unpack_weight_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const u32x4_t*)packed, (u32x4_t*)rows, per, k, tiles);
    return tqk_check_launch("tqk_unpack_weight");
}

extern "C" int tqk_pack_weight(const void* w, void* out, int n, int k, int parts, void* stream) {
    TQK_REQUIRE(w && out, "tqk_pack_weight: null pointer");
    TQK_REQUIRE(n > 0 && k > 0 && parts > 0 && k % 32 == 0 && n % parts == 0,
                "tqk_pack_weight: needs bfloat16 [n, k] with k a multiple of 32 and n of %d parts, got [%d, %d]", parts, n, k);
    const int per = n / parts, tiles = (per + 15) / 16;
    const long long total = (long long)parts * tiles * (k / 32) * 512;
    pack_weight_kernel<<<blocks_for(total), 256, 0, (hipStream_t)stream>>>((const uint16_t*)w, (uint16_t*)out, per, k, tiles, total);
    return tqk_check_launch("tqk_pack_weight");
}
