// Weight gradient of a Linear layer for gfx950:  dW[n][k] = sum_r dy[r][n] * x[r][k]
// with bf16 operands, fp32 accumulation on the matrix cores and an fp32 result.
//
// In the PPO update (reference: train/rl/ppo.py:1417-1425 back-propagating through the trunk's
// nn.Linear layers, models/yemong/attention.py:60-74 and griffin.py:238-247) the contraction runs
// over the rows, several hundred thousand of them, while N and K are 128..512.  The library
// GEMM picks a tiling for large M x N and runs these at 6-20x the time the operands need to
// cross HBM once (393,216 rows, 128 x 128: 815 us against a 40 us floor).  Here the rows are
// split into slices, one work-group per (128 x 128 output tile, slice), so the chip is filled
// by the long dimension (the tiles of one slice placed on one XCD, so the operand rows they share
// cross HBM once):
//   * a work-group walks its slice in chunks of 64 rows.  A thread fetches an 8 x 8 block of one
//     operand (eight coalesced 16-byte loads, the next chunk prefetched into registers),
//     transposes it in registers (32 byte-permutes) and stores it column-major in LDS, because
//     the matrix cores want the contraction index (the row) along each lane's 8 operand values;
//   * the 16-byte position of a column's row block is XOR-ed with the column index, so both the
//     transposed stores and the operand loads (one ds_read_b128 per MFMA operand) spread over
//     all banks;
//   * wave w owns a 64 x 64 quarter of the tile (2 x 2 accumulator tiles: two A and two B
//     operands feed four MFMAs), every slice writes its partial tile, and a second small kernel
//     adds the slices in a fixed order (deterministic, unlike atomics) into dW, optionally on top
//     of what is there.
// Bound: HBM (each operand element read once per output tile column/row it meets).

#include "common.h"

namespace bnb {

constexpr int kWgTile = 128;   // output tile edge
constexpr int kWgRows = 64;    // rows per chunk
constexpr int kWgThreads = 256;

// halfs offset of (column c, row block rb of 8 rows) in a column-major staged tile of 128 columns x 64 rows
__device__ __forceinline__ int wg_slot(int c, int rb) { return c * kWgRows + 8 * ((rb ^ c ^ (c >> 3)) & 7); }

__global__ __launch_bounds__(kWgThreads) void linear_wgrad_kernel(
    const uint16_t *__restrict__ dy, int64_t dy_stride, const uint16_t *__restrict__ x, int64_t x_stride,
    float *__restrict__ partials, int64_t R, int N, int K, int64_t rows_per_slice, int slices, int64_t dy_tile_stride,
    int64_t x_tile_stride)
{
    __shared__ __align__(16) uint16_t s_t[2][kWgTile * kWgRows];  // [operand: dy, x][column][row], swizzled

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31;
    const int half = lane >> 5;
    // work-group -> (output tile, slice): the tiles of one slice share the second operand's rows, so they
    // are given ids that differ by multiples of 8 and close together: work-groups are dealt to the 8 XCDs in
    // turn, which puts them on one XCD (one L2) at about the same time
    const int tiles_n = N / kWgTile, tiles = tiles_n * (K / kWgTile);
    const int full = slices / 8 * 8 * tiles;
    int tile, slice_i;
    if ((int)blockIdx.x < full) {
        const int group = blockIdx.x / (8 * tiles), within = blockIdx.x - group * 8 * tiles;
        tile = within >> 3;
        slice_i = group * 8 + (within & 7);
    } else {
        const int r = blockIdx.x - full;
        tile = r % tiles;
        slice_i = slices / 8 * 8 + r / tiles;
    }
    const int n0 = (tile % tiles_n) * kWgTile, k0 = (tile / tiles_n) * kWgTile;
    const int64_t slice = slice_i;
    const int64_t r_begin = slice * rows_per_slice;
    const int64_t r_end = r_begin + rows_per_slice < R ? r_begin + rows_per_slice : R;

    // this thread's 8 x 8 block: operand tid/128, rows 8*rg .. +7 of the chunk, columns 8*cb .. +7
    const int operand = tid >> 7;  // uniform per wave
    const int rg = (tid & 127) >> 4;
    const int cb = tid & 15;
    // the 128 columns of a tile start `tile stride` elements after those of the tile before (128 for plain row-major
    // operands; R * 128 for operands stored tile by tile)
    const uint16_t *src = operand ? x + (k0 / kWgTile) * x_tile_stride + 8 * cb : dy + (n0 / kWgTile) * dy_tile_stride + 8 * cb;
    const int64_t src_stride = operand ? x_stride : dy_stride;
    uint16_t *dst = s_t[operand];

    u32x4 stage_a[8];  // the next chunk's operand rows, in flight while this one is multiplied
    auto fetch = [&](u32x4(&stage)[8], int64_t row0) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int64_t r = row0 + 8 * rg + j;
            const u32x4 v = *reinterpret_cast<const u32x4 *>(src + (r < r_end ? r : r_begin) * src_stride);
            stage[j] = r < r_end ? v : u32x4{0u, 0u, 0u, 0u};  // rows past the slice add nothing
        }
    };
    auto stash = [&](const u32x4(&stage)[8]) {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            // column c of the block: rows 0..7 as four words of two halfs
            const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = __builtin_amdgcn_perm(stage[2 * j + 1][c >> 1], stage[2 * j][c >> 1], sel);
            *reinterpret_cast<u32x4 *>(dst + wg_slot(8 * cb + c, rg)) = u32x4{w[0], w[1], w[2], w[3]};
        }
    };
    auto operand8 = [&](const uint16_t *tile, int c, int rb) -> bf16x8 {
        return __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(tile + wg_slot(c, rb)));
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][t][v] = 0.0f;

    const int nw = 64 * (wave >> 1), kw = 64 * (wave & 1);  // this wave's quarter of the tile
    auto chunk = [&](u32x4(&stage)[8], int64_t row0) {
        __syncthreads();  // everyone is done reading the previous chunk
        stash(stage);
        if (row0 + kWgRows < r_end) fetch(stage, row0 + kWgRows);
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < kWgRows / 16; ++ks) {
            const int rb = 2 * ks + half;
            const bf16x8 a0 = operand8(s_t[0], nw + m, rb), a1 = operand8(s_t[0], nw + 32 + m, rb);
            const bf16x8 b0 = operand8(s_t[1], kw + m, rb), b1 = operand8(s_t[1], kw + 32 + m, rb);
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, acc[1][1], 0, 0, 0);
        }
    };
    if (r_begin < r_end) fetch(stage_a, r_begin);
    for (int64_t row0 = r_begin; row0 < r_end; row0 += kWgRows) chunk(stage_a, row0);
    // partial tile of this slice: lane holds column k = kw + 32t + m, rows n = nw + 32i + 8(v/4) + 4*half + v%4
    float *pt = partials + (slice * N + n0 + nw + 4 * half) * K + k0 + kw + m;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) pt[(int64_t)(32 * i + 8 * (v >> 2) + (v & 3)) * K + 32 * t] = acc[i][t][v];
}

// dW (+)= sum over the slices in a fixed order: a work-group owns 64 consecutive elements (16 lanes x 4 floats);
// its 16 lane groups each add every 16th slice, then group 0 adds the 16 sums in group order.
__global__ __launch_bounds__(256) void sum_slices_kernel(const float *__restrict__ partials, float *__restrict__ dw,
                                                         int64_t elems, int slices, int accumulate)
{
    __shared__ f32x4 s_sum[16][16];
    const int q = threadIdx.x & 15, g = threadIdx.x >> 4;
    const int64_t i = ((int64_t)blockIdx.x * 16 + q) * 4;  // elems is a multiple of 64
    f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
    int k = g;
    for (; k + 48 < slices; k += 64) {
        f32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const f32x4 *>(partials + (int64_t)(k + 16 * u) * elems + i);
#pragma unroll
        for (int u = 0; u < 4; ++u) s.x += v[u].x, s.y += v[u].y, s.z += v[u].z, s.w += v[u].w;
    }
    for (; k < slices; k += 16) {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(partials + (int64_t)k * elems + i);
        s.x += v.x, s.y += v.y, s.z += v.z, s.w += v.w;
    }
    s_sum[g][q] = s;
    __syncthreads();
    if (g == 0) {
        f32x4 t = accumulate ? *reinterpret_cast<const f32x4 *>(dw + i) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const f32x4 v = s_sum[u][q];
            t.x += v.x, t.y += v.y, t.z += v.z, t.w += v.w;
        }
        *reinterpret_cast<f32x4 *>(dw + i) = t;
    }
}

int launch_sum_slices(const float *partials, float *out, int64_t elems, int slices, int accumulate, hipStream_t stream)
{
    if (elems <= 0 || elems % 64 != 0 || slices < 0) return BNB_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(sum_slices_kernel, dim3((unsigned)(elems / 64)), dim3(256), 0, stream, partials, out, elems, slices,
                       accumulate);
    return (int)hipGetLastError();
}

}  // namespace bnb

extern "C" int bnb_linear_wgrad_slices(int64_t R, int N, int K)
{
    // slices such that tiles x slices is about three work-groups per CU (all resident at once: 148 registers, 32 KB of LDS each), every slice at least 256 rows
    if (R <= 0 || N <= 0 || K <= 0) return 1;
    const int64_t tiles = (int64_t)(N / bnb::kWgTile) * (K / bnb::kWgTile);
    int64_t s = 768 / (tiles > 0 ? tiles : 1);
    const int64_t by_rows = (R + 255) / 256;
    if (s > by_rows) s = by_rows;
    if (s < 1) s = 1;
    if (s > 1024) s = 1024;
    return (int)s;
}

extern "C" int bnb_linear_wgrad_tiled_fwd(const void *dy, int64_t dy_row_stride, int64_t dy_tile_stride, const void *x,
                                          int64_t x_row_stride, int64_t x_tile_stride, float *partials, int slices, float *dw,
                                          int accumulate, int64_t R, int N, int K, void *stream)
{
    using namespace bnb;
    if (R < 0 || N < 1 || K < 1 || slices < 1) return BNB_ERR_BAD_SHAPE;
    if (N % kWgTile != 0 || K % kWgTile != 0 || slices > 65535) return BNB_ERR_UNSUPPORTED;
    if (!dw || !partials || (R > 0 && (!dy || !x))) return BNB_ERR_NULL_POINTER;
    // row-major operands hold all their columns in a row; tile-by-tile ones 128 per row
    if (dy_row_stride < (dy_tile_stride == kWgTile ? N : kWgTile) || x_row_stride < (x_tile_stride == kWgTile ? K : kWgTile) ||
        dy_tile_stride < kWgTile || x_tile_stride < kWgTile)
        return BNB_ERR_BAD_SHAPE;
    if ((R > 0 && (!aligned16(dy) || !aligned16(x))) || !aligned16(partials) || !aligned16(dw) || dy_row_stride % 8 != 0 ||
        x_row_stride % 8 != 0 || dy_tile_stride % 8 != 0 || x_tile_stride % 8 != 0)
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    const int64_t rows_per_slice = ((R + slices - 1) / slices + kWgRows - 1) / kWgRows * kWgRows;
    const int64_t groups = (int64_t)(N / kWgTile) * (K / kWgTile) * slices;
    if (groups > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(linear_wgrad_kernel, dim3((unsigned)groups), dim3(kWgThreads), 0, s, (const uint16_t *)dy, dy_row_stride,
                       (const uint16_t *)x, x_row_stride, partials, R, N, K, rows_per_slice > 0 ? rows_per_slice : kWgRows, slices,
                       dy_tile_stride, x_tile_stride);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return launch_sum_slices(partials, dw, (int64_t)N * K, slices, accumulate, s);
}

extern "C" int bnb_linear_wgrad_fwd(const void *dy, int64_t dy_row_stride, const void *x, int64_t x_row_stride,
                                    float *partials, int slices, float *dw, int accumulate, int64_t R, int N, int K,
                                    void *stream)
{
    return bnb_linear_wgrad_tiled_fwd(dy, dy_row_stride, bnb::kWgTile, x, x_row_stride, bnb::kWgTile, partials, slices, dw,
                                      accumulate, R, N, K, stream);
}
