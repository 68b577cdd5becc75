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

// ------------------------------------------------------------------------------------------------
// The same product with the operand rows travelling global -> LDS directly and transposed on the way
// out of LDS by the hardware (gfx950: global_load_lds_dwordx4, ds_read_b64_tr_b16):
//   * a chunk is 32 rows of both 128-column operand tiles (16 KB), kept ROW-major in LDS; a wave moves
//     four whole 256-byte rows per instruction (lane l fills bytes 16 l .. 16 l + 15 of the wave's KB),
//     no lane spends registers or instructions on staging, and four chunk buffers let three chunks be
//     in flight while one is multiplied (the register-staged form above has one);
//   * the matrix cores want the contraction index (the row) along a lane's eight operand values:
//     ds_read_b64_tr_b16 delivers, inside a group of 16 lanes, element i%4 of the 8-byte pieces that
//     lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12 point at, so with source lane r pointing at row r/4 and
//     the 4-column block r%4, lane i receives column i of four rows: two such reads are one operand;
//   * a lane may fetch ANY 16-byte piece of its row into its fixed LDS slot, so piece c of row r is kept
//     in slot c ^ 2(r%4): the four rows a 16-lane group reads then sit on different banks although the
//     row pitch is 256 bytes.
// Rows past the end of a slice are zeroed in LDS by the lanes that fetched them (last chunk only).

constexpr int kWdRows = 32;                         // rows per chunk
constexpr int kWdStages = 4;
constexpr int kWdStageBytes = 2 * kWdRows * 256;    // both operands: 16 KB

__device__ __forceinline__ void wd_dma16(const void *sbase, uint32_t voff, uint32_t lds_base)
{
    // 16 bytes per lane from sbase + voff to LDS byte address lds_base + 16 * lane (no immediate offset: the
    // instruction would add it to the LDS address as well as to the global one)
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0" : : "s"(sbase), "v"(voff), "s"(lds_base) : "memory", "m0");
}

__device__ __forceinline__ bf16x8 wd_operand(const unsigned char *p)
{
    typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
    typedef bf16x4_t __attribute__((address_space(3))) * lds_ptr;
    const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_ptr)p);
    const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_ptr)(p + 4 * 256));  // four rows further on
    return bf16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

__global__ __launch_bounds__(kWgThreads) void linear_wgrad_dma_kernel(
    const uint16_t *__restrict__ dy, int64_t dy_stride, const uint16_t *__restrict__ x, int64_t x_stride,
    float *__restrict__ partials, int64_t R, int N, int K, int64_t rows_per_slice, int slices, int64_t dy_tile_stride,
    int64_t x_tile_stride)
{
    __shared__ __align__(1024) unsigned char s_st[kWdStages][kWdStageBytes];  // [stage][operand][row][16 slots of 16 B]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31;
    const int half = lane >> 5;
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
    const int n_chunks = r_begin < r_end ? (int)((r_end - r_begin + kWdRows - 1) / kWdRows) : 0;

    // DMA role: wave w moves rows 8w .. 8w+7 of both operands of a chunk, four instructions of four rows;
    // lane l of an instruction: row l/16 of its four, LDS slot l%16, global piece (l%16) ^ 2(row%4).
    // The instruction takes a wave-uniform base and a 32-bit byte offset per lane: the base is the first row of
    // the four (clamped to the last row of the matrix), the offset the lane's row within them and its piece.
    const int d_row = lane >> 4;                       // 0..3, also row % 4 (instruction rows start at multiples of 4)
    const int d_piece = (lane & 15) ^ (2 * d_row);
    const uint16_t *dy_tile = dy + (n0 / kWgTile) * dy_tile_stride;
    const uint16_t *x_tile = x + (k0 / kWgTile) * x_tile_stride;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)&s_st[0][0];
    auto issue = [&](int chunk, int stage) {
        const int64_t row0 = r_begin + (int64_t)chunk * kWdRows + 8 * wave;  // wave-uniform
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int64_t first = row0 + 4 * q;
            const int64_t base_row = first < R ? first : R - 1;              // uniform, in bounds
            const int64_t r = first + d_row;
            const uint32_t extra = (uint32_t)((r < R ? r : R - 1) - base_row);  // 0..3 rows below the base
            const uint32_t lds = lds0 + (uint32_t)(stage * kWdStageBytes + (8 * wave + 4 * q) * 256);
            wd_dma16(dy_tile + base_row * dy_stride, (extra * (uint32_t)dy_stride + 8u * (uint32_t)d_piece) * 2u, lds);
            wd_dma16(x_tile + base_row * x_stride, (extra * (uint32_t)x_stride + 8u * (uint32_t)d_piece) * 2u, lds + kWdRows * 256);
        }
    };
    // rows of the last chunk that lie past the slice: the lanes that fetched them overwrite them with zeros
    auto zero_tail = [&](int chunk, int stage) {
        const int64_t row0 = r_begin + (int64_t)chunk * kWdRows + 8 * wave;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int64_t r = row0 + 4 * q + d_row;
            if (r >= r_end) {
                unsigned char *p = &s_st[stage][0] + (8 * wave + 4 * q) * 256 + lane * 16;
                *reinterpret_cast<u32x4 *>(p) = u32x4{0u, 0u, 0u, 0u};
                *reinterpret_cast<u32x4 *>(p + kWdRows * 256) = u32x4{0u, 0u, 0u, 0u};
            }
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][t][v] = 0.0f;

    // operand read role: 16-lane group g = lane/16: columns 16 (g%2) + (lane%16) of a 32-column block, k-slots
    // = rows 8 (g/2) + 0..7 of a 16-row step.  As a SOURCE lane j = lane%16 of its group it points at row
    // 8 (g/2) + j/4 (+4 for the second read) and the 4-column block j%4 of the group's 16 columns.
    const int nw = 64 * (wave >> 1), kw = 64 * (wave & 1);  // this wave's quarter of the tile
    const int j = lane & 15, g = lane >> 4;
    const int src_row = 8 * (g >> 1) + (j >> 2);                 // row within a 16-row step; row % 4 == j / 4
    auto src_off = [&](int col0) {                               // byte offset inside an operand tile, step 0
        const int col = col0 + 16 * (g & 1) + 4 * (j & 3);       // first of the 4 columns this lane points at
        const int piece = col >> 3;
        return src_row * 256 + ((piece ^ (2 * (j >> 2))) * 16) + (col & 4) * 2;
    };
    const int a_off[2] = {src_off(nw), src_off(nw + 32)};
    const int b_off[2] = {kWdRows * 256 + src_off(kw), kWdRows * 256 + src_off(kw + 32)};

    // prologue: up to three chunks in flight
#pragma unroll
    for (int c = 0; c < kWdStages - 1; ++c)
        if (c < n_chunks) issue(c, c);
    for (int c = 0; c < n_chunks; ++c) {
        const int stage = c & (kWdStages - 1);
        // chunk c has landed when at most the younger chunks' instructions of this wave are outstanding (4 per chunk)
        const int younger = n_chunks - 1 - c < kWdStages - 2 ? n_chunks - 1 - c : kWdStages - 2;
        if (younger >= 2) __builtin_amdgcn_s_waitcnt(0x0f78);       // vmcnt(8)
        else if (younger == 1) __builtin_amdgcn_s_waitcnt(0x0f74);  // vmcnt(4)
        else __builtin_amdgcn_s_waitcnt(0x0f70);                    // vmcnt(0)
        if (c == n_chunks - 1) zero_tail(c, stage);
        __syncthreads();  // every wave's rows of chunk c are in; everyone is done reading chunk c - 1
        if (c + kWdStages - 1 < n_chunks) issue(c + kWdStages - 1, (c + kWdStages - 1) & (kWdStages - 1));
        const unsigned char *st = &s_st[stage][0];
#pragma unroll
        for (int ks = 0; ks < kWdRows / 16; ++ks) {
            const bf16x8 a0 = wd_operand(st + a_off[0] + ks * 16 * 256), a1 = wd_operand(st + a_off[1] + ks * 16 * 256);
            const bf16x8 b0 = wd_operand(st + b_off[0] + ks * 16 * 256), b1 = wd_operand(st + b_off[1] + ks * 16 * 256);
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, acc[1][1], 0, 0, 0);
        }
    }
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

// Column sums of a (R, N) matrix (a bias gradient): a work-group owns a run of consecutive rows, a lane eight
// consecutive columns of every (256 / (N / 8))-th row of the run; the lanes of a column group are added in lane order
// through LDS into one partial row per work-group, the partial rows by sum_slices.
constexpr int kColSumMaxSlices = 1024;

template <typename T>
__global__ __launch_bounds__(256) void column_sums_kernel(const T *__restrict__ x, int64_t row_stride, float *__restrict__ partials,
                                                          int64_t R, int N, int64_t rows_per_slice)
{
    __shared__ float s_part[256 * 8];
    const int groups = N >> 3;                    // lanes per row
    const int lanes_rows = 256 / groups;          // rows in flight per pass
    const int local_row = threadIdx.x / groups, c0 = (threadIdx.x - local_row * groups) << 3;
    const int64_t first = (int64_t)blockIdx.x * rows_per_slice;
    const int64_t last = first + rows_per_slice < R ? first + rows_per_slice : R;
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (local_row < lanes_rows) {
        int64_t r = first + local_row;
        for (; r + 3 * lanes_rows < last; r += 4 * lanes_rows) {
            Row8 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = load8_stream(x + (r + (int64_t)u * lanes_rows) * row_stride + c0);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] += v[u].v[e];
        }
        for (; r < last; r += lanes_rows) {
            const Row8 v = load8_stream(x + r * row_stride + c0);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] += v.v[e];
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) s_part[threadIdx.x * 8 + e] = acc[e];
    __syncthreads();
    for (int c = threadIdx.x; c < N; c += 256) {
        const int g = c >> 3, e = c & 7;
        float t = 0.0f;
        for (int j = 0; j < lanes_rows; ++j) t += s_part[(j * groups + g) * 8 + e];
        partials[(int64_t)blockIdx.x * N + c] = t;
    }
}

}  // namespace bnb

extern "C" int bnb_column_sums_slices(int64_t R, int N)
{
    if (R <= 0 || N < 8) return 1;
    const int64_t lanes_rows = 256 / (N / 8) > 0 ? 256 / (N / 8) : 1;
    int64_t s = (R + 16 * lanes_rows - 1) / (16 * lanes_rows);  // at least sixteen passes per work-group
    if (s > bnb::kColSumMaxSlices) s = bnb::kColSumMaxSlices;
    return (int)(s < 1 ? 1 : s);
}

extern "C" int bnb_column_sums(const void *x, int x_dtype, int64_t x_row_stride, float *partials, int slices, float *out,
                               int accumulate, int64_t R, int N, void *stream)
{
    using namespace bnb;
    if (R < 0 || N < 1 || slices < 1 || slices > kColSumMaxSlices || x_row_stride < N) return BNB_ERR_BAD_SHAPE;
    if (N % 64 != 0 || N > 2048) return BNB_ERR_UNSUPPORTED;
    if (x_dtype != BNB_F32 && x_dtype != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (!out || !partials || (R > 0 && !x)) return BNB_ERR_NULL_POINTER;
    if ((R > 0 && !aligned16(x)) || !aligned16(partials) || !aligned16(out) || x_row_stride % 8 != 0) return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    if (R == 0) return launch_sum_slices(partials, out, N, 0, accumulate, s);
    const int64_t rows_per_slice = (R + slices - 1) / slices;
    const int used = (int)((R + rows_per_slice - 1) / rows_per_slice);  // trailing work-groups without rows are not launched
    if (x_dtype == BNB_BF16)
        hipLaunchKernelGGL((column_sums_kernel<uint16_t>), dim3((unsigned)used), dim3(256), 0, s, (const uint16_t *)x, x_row_stride,
                           partials, R, N, rows_per_slice);
    else
        hipLaunchKernelGGL((column_sums_kernel<float>), dim3((unsigned)used), dim3(256), 0, s, (const float *)x, x_row_stride, partials,
                           R, N, rows_per_slice);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return launch_sum_slices(partials, out, N, used, accumulate, s);
}

namespace bnb {
// BNB_WGRAD_PATH_AUTO picks the direct-to-LDS kernel; the register-staged one stays selectable for comparisons
static int g_wgrad_path = BNB_WGRAD_PATH_AUTO;
static bool wgrad_dma() { return g_wgrad_path != BNB_WGRAD_PATH_STAGED; }
}  // namespace bnb

extern "C" int bnb_linear_wgrad_path(int path)
{
    if (path != BNB_WGRAD_PATH_AUTO && path != BNB_WGRAD_PATH_STAGED && path != BNB_WGRAD_PATH_DMA) return BNB_ERR_BAD_SHAPE;
    bnb::g_wgrad_path = path;
    return 0;
}

extern "C" int bnb_linear_wgrad_slices(int64_t R, int N, int K)
{
    // slices such that tiles x slices fills the chip once (all work-groups resident), every slice at least 256 rows
    if (R <= 0 || N <= 0 || K <= 0) return 1;
    const int64_t tiles = (int64_t)(N / bnb::kWgTile) * (K / bnb::kWgTile);
    // work-groups resident at once: three per CU for the register-staged kernel (32 KB of LDS), two for the
    // direct-to-LDS one (64 KB)
    int64_t s = (bnb::wgrad_dma() ? 512 : 768) / (tiles > 0 ? tiles : 1);
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
    if (wgrad_dma())
        hipLaunchKernelGGL(linear_wgrad_dma_kernel, dim3((unsigned)groups), dim3(kWgThreads), 0, s, (const uint16_t *)dy,
                           dy_row_stride, (const uint16_t *)x, x_row_stride, partials, R, N, K,
                           rows_per_slice > 0 ? rows_per_slice : kWgRows, slices, dy_tile_stride, x_tile_stride);
    else
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
