// RMSNorm + Linear as ONE kernel on the matrix cores (gfx950), optionally over gathered rows.
//
//   n   = x[row] * rsqrt(mean(x[row]^2) + eps) * w_norm               x fp32, 128 channels
//   out = bf16(n W^T + bias)                                          W (N, 128) bf16, N % 64 == 0
// Reference: `self.kv_bullet(self.norm_bullet(bullets))` (models/yemong/attention.py:150-151),
// `self.qkv(self.norm1(x))` (:94-96,132) and the temporal block's `linear1(norm1(x))`
// (models/yemong/griffin.py:269-272) as they run under bf16 autocast: nn.RMSNorm, autocast's
// cast, nn.Linear.
//
// With `row_index` the kernel reads row row_index[r] of x for output row r, and with `n_rows`
// (a device-side count) it stops after that many rows: the projection then runs over the
// bullets in flight only (a compact list built on the device), never over the empty slots,
// without the host ever learning how many there are.
//
// A wave owns 32 rows.  Rows come in as whole 256-byte runs through LDS (two passes of 64
// channels), each lane ends up with its row's channels in the k-slot order
//   ch(ks, h, e) = 16ks + 8(e/4) + 4h + e%4      (lane = 32h + m, k-slot e of step ks)
// which is the B operand of out^T = W n^T on v_mfma_f32_32x32x16_bf16.  The packed weights
// list output features so that a lane's 16 results per 32-feature block are two runs of 8
// consecutive features (16-byte stores, the two lanes of a row side by side):
//   [fb][ks][l][e] = W[32fb + 16((r/8)/2) + 8((r/4)%2) + 4((r/8)%2) + r%4][ch(ks, l/32, e)],  r = l%32
// Weights stream through LDS in chunks of 64 features (16 KB), double-buffered.

#include "common.h"

namespace bnb {

constexpr int kNlD = 128;
constexpr int kNlWaves = 4;
constexpr int kNlThreads = kNlWaves * kWave;
constexpr int kNlChunkFeatures = 64;
constexpr int kNlChunkHalfs = kNlChunkFeatures * kNlD;                 // 8192 bf16 = 16 KB
constexpr int kNlPrefetch = kNlChunkHalfs / 8 / kNlThreads;           // 16-byte pieces per thread per chunk
constexpr int kNlHalfPitch = 64 + 4;                                   // floats per staged half row (bank spread)

__global__ __launch_bounds__(kNlThreads) void norm_linear_kernel(
    const float *__restrict__ x, int64_t x_stride, const int32_t *__restrict__ row_index,
    const int32_t *__restrict__ n_rows, const float *__restrict__ norm_w, float eps,
    const uint16_t *__restrict__ wpack, const float *__restrict__ bias, uint16_t *__restrict__ out, int64_t R, int N,
    uint16_t *__restrict__ n_out = nullptr)
{
    // staging area for the rows (prologue) and the two weight buffers (loop) share this space
    constexpr int kStageFloats = kNlWaves * 32 * kNlHalfPitch;                       // 8704 floats = 34 KB
    constexpr int kLdsBytes = kStageFloats * 4 > 2 * kNlChunkHalfs * 2 ? kStageFloats * 4 : 2 * kNlChunkHalfs * 2;
    __shared__ __align__(16) unsigned char s_raw[kLdsBytes];
    float *s_stage = reinterpret_cast<float *>(s_raw);
    uint16_t *s_w = reinterpret_cast<uint16_t *>(s_raw);

    const int64_t rows = n_rows != nullptr ? (int64_t)*n_rows : R;
    const int64_t block_row0 = (int64_t)blockIdx.x * (kNlWaves * 32);
    if (block_row0 >= rows) return;  // whole work-group past the end of the (device-side) row count

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31;
    const int half = lane >> 5;

    u32x4 pre[kNlPrefetch];
    auto fetch = [&](int c) {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(wpack + (int64_t)c * kNlChunkHalfs);
#pragma unroll
        for (int q = 0; q < kNlPrefetch; ++q) pre[q] = src[tid + q * kNlThreads];
    };
    auto stash = [&](int buf) {
        u32x4 *dst = reinterpret_cast<u32x4 *>(s_w + buf * kNlChunkHalfs);
#pragma unroll
        for (int q = 0; q < kNlPrefetch; ++q) dst[tid + q * kNlThreads] = pre[q];
    };
    fetch(0);

    // ---- rows in: a quarter-wave per 256-byte half row, two passes over the channels ----
    const int64_t row0 = block_row0 + wave * 32;
    float *stage = s_stage + wave * (32 * kNlHalfPitch);
    const int io_row = lane >> 4;        // 4 rows per instruction
    const int io_col = (lane & 15) * 4;  // this lane's four channels within the half row
    int64_t src_row[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        int64_t r = row0 + 4 * j + io_row;
        r = r < rows ? r : rows - 1;
        src_row[j] = row_index != nullptr ? (int64_t)row_index[r] : r;
    }
    // The per-row factor rsqrt(mean(x^2) + eps) is a scalar of the output row, so it is applied
    // to the products instead of the operand: the operand is bf16(x * w_norm), formed as the
    // channels arrive (the row never sits in registers as fp32), same relative rounding.
    bf16x8 nb[8];
    float ss = 0.0f;
    // both passes' rows are requested before the first one is staged: one round trip to memory instead of two
    f32x4 xv[2][8];
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            xv[pass][j] = __builtin_nontemporal_load(
                reinterpret_cast<const f32x4 *>(x + src_row[j] * x_stride + 64 * pass + io_col));
    }
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            *reinterpret_cast<f32x4 *>(stage + (4 * j + io_row) * kNlHalfPitch + io_col) = xv[pass][j];
        __syncthreads();
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4) {  // contraction step ks = 4 pass + k4: channels 16 ks + ...
            const int ks = 4 * pass + k4;
            const float *sp = stage + m * kNlHalfPitch + 16 * k4 + 4 * half;
            const f32x4 lo = *reinterpret_cast<const f32x4 *>(sp);
            const f32x4 hi = *reinterpret_cast<const f32x4 *>(sp + 8);
            const f32x4 wl = *reinterpret_cast<const f32x4 *>(norm_w + 16 * ks + 4 * half);
            const f32x4 wh = *reinterpret_cast<const f32x4 *>(norm_w + 16 * ks + 8 + 4 * half);
            const float t[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            const float wv[8] = {wl.x, wl.y, wl.z, wl.w, wh.x, wh.y, wh.z, wh.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                nb[ks][e] = (__bf16)(t[e] * wv[e]);
                ss = fmaf(t[e], t[e], ss);
            }
        }
        __syncthreads();
    }
    ss += __shfl_xor(ss, 32);
    const float rstd = rsqrtf(ss * (1.0f / kNlD) + eps);

    if (n_out != nullptr) {
        // The update keeps the normalised rows for the weight gradient: the operand this kernel multiplies is
        // rstd * bf16(x * w_norm); its bfloat16 rounding leaves as whole 256-byte rows through this wave's slice
        // of the staging area (32 rows x 136 halfs fit in the 32 x 68 floats of the slice).
        constexpr int kNPitch = kNlD + 8;
        static_assert(kNPitch * 2 <= kNlHalfPitch * 4, "a staged bf16 row fits the slice's row pitch");
        uint16_t *stage_n = reinterpret_cast<uint16_t *>(stage);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            float t[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] = (float)nb[ks][e] * rstd;
            uint16_t *sp = stage_n + m * kNPitch + 16 * ks + 4 * half;
            *reinterpret_cast<u32x2 *>(sp) = u32x2{pack_bf16x2(t[0], t[1]), pack_bf16x2(t[2], t[3])};
            *reinterpret_cast<u32x2 *>(sp + 8) = u32x2{pack_bf16x2(t[4], t[5]), pack_bf16x2(t[6], t[7])};
        }
        wave_lds_handover();
        const int a_row = lane >> 4, a_col = (lane & 15) * 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int64_t r = row0 + 4 * j + a_row;
            const u32x4 v = *reinterpret_cast<const u32x4 *>(stage_n + (4 * j + a_row) * kNPitch + a_col);
            if (r < rows) __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(n_out + r * kNlD + a_col));
        }
        __syncthreads();  // the slices are read out before the weights move in
    }

    stash(0);
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();

    const int64_t row = row0 + m;
    const int chunks = N / kNlChunkFeatures;
    for (int c = 0; c < chunks; ++c) {
        const int buf = c & 1;
        if (c + 1 < chunks) fetch(c + 1);
        const uint16_t *wb = s_w + buf * kNlChunkHalfs + lane * 8;
        f32x16 z0 = {0.0f}, z1 = {0.0f};
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const bf16x8 a0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wb + ks * 512));
            const bf16x8 a1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wb + 4096 + ks * 512));
            z0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, nb[ks], z0, 0, 0, 0);
            z1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, nb[ks], z1, 0, 0, 0);
        }
        if (row < rows) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const f32x16 &z = b ? z1 : z0;
                const int f0 = c * kNlChunkFeatures + 32 * b + 8 * half;  // first feature of this lane's first run
#pragma unroll
                for (int run = 0; run < 2; ++run) {
                    float r[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) r[e] = z[8 * run + e] * rstd;
                    if (bias != nullptr) {
                        const f32x4 bl = *reinterpret_cast<const f32x4 *>(bias + f0 + 16 * run);
                        const f32x4 bh = *reinterpret_cast<const f32x4 *>(bias + f0 + 16 * run + 4);
                        r[0] += bl.x; r[1] += bl.y; r[2] += bl.z; r[3] += bl.w;
                        r[4] += bh.x; r[5] += bh.y; r[6] += bh.z; r[7] += bh.w;
                    }
                    const u32x4 w = {pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3]), pack_bf16x2(r[4], r[5]),
                                     pack_bf16x2(r[6], r[7])};
                    *reinterpret_cast<u32x4 *>(out + row * N + f0 + 16 * run) = w;
                }
            }
        }
        if (c + 1 < chunks) stash(buf ^ 1);
        __syncthreads();
    }
}

// ------------------------------------------------------------------------------------
// compact list of the rows whose mask byte is set (the bullets in flight)
// ------------------------------------------------------------------------------------

// counts[b] = number of set bytes in mask row b (one work-group per row).
__global__ __launch_bounds__(256) void mask_count_kernel(const uint8_t *__restrict__ mask, int32_t *__restrict__ counts,
                                                         int n)
{
    __shared__ int s_part[4];
    const uint8_t *row = mask + (int64_t)blockIdx.x * n;
    int c = 0;
    for (int j = threadIdx.x; j < n; j += 256) c += row[j] != 0 ? 1 : 0;
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off);
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) counts[blockIdx.x] = s_part[0] + s_part[1] + s_part[2] + s_part[3];
}

// index[offsets[b] + k] = b*n + j for the k-th set byte j of mask row b, ascending (one
// work-group of one wave per row keeps the order without any cross-wave bookkeeping).
__global__ __launch_bounds__(64) void mask_fill_kernel(const uint8_t *__restrict__ mask,
                                                       const int32_t *__restrict__ offsets,
                                                       int32_t *__restrict__ index, int n)
{
    const uint8_t *row = mask + (int64_t)blockIdx.x * n;
    int base = offsets[blockIdx.x];
    const int lane = threadIdx.x;
    for (int j0 = 0; j0 < n; j0 += 64) {
        const int j = j0 + lane;
        const bool on = j < n && row[j] != 0;
        const uint64_t ballot = __ballot(on);
        if (on) index[base + (int)__popcll(ballot & ((1ull << lane) - 1ull))] = blockIdx.x * n + j;
        base += (int)__popcll(ballot);
    }
}

}  // namespace bnb

extern "C" int bnb_norm_linear_fwd(const float *x, int64_t x_row_stride, const int32_t *row_index,
                                   const int32_t *n_rows, const float *norm_weight, float eps,
                                   const void *weight_packed, const float *bias, void *out, int64_t R, int D, int N,
                                   void *stream)
{
    using namespace bnb;
    if (R < 0 || x_row_stride < D || N < 1) return BNB_ERR_BAD_SHAPE;
    if (D != kNlD || N % kNlChunkFeatures != 0) return BNB_ERR_UNSUPPORTED;
    if (R == 0) return 0;
    if (!x || !norm_weight || !weight_packed || !out) return BNB_ERR_NULL_POINTER;
    if (!aligned16(x) || !aligned16(out) || !aligned16(norm_weight) || !aligned16(weight_packed) ||
        (bias && !aligned16(bias)) || (x_row_stride % 4) != 0)
        return BNB_ERR_MISALIGNED;
    if ((reinterpret_cast<uintptr_t>(row_index) | reinterpret_cast<uintptr_t>(n_rows)) & 3u) return BNB_ERR_MISALIGNED;
    const int64_t blocks = (R + kNlWaves * 32 - 1) / (kNlWaves * 32);
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(norm_linear_kernel, dim3((unsigned)blocks), dim3(kNlThreads), 0, (hipStream_t)stream, x,
                       x_row_stride, row_index, n_rows, norm_weight, eps, (const uint16_t *)weight_packed, bias,
                       (uint16_t *)out, R, N);
    return (int)hipGetLastError();
}

extern "C" int bnb_norm_linear_train_fwd(const float *x, int64_t x_row_stride, const float *norm_weight, float eps,
                                         const void *weight_packed, void *out, void *n_out, int64_t R, int D, int N,
                                         void *stream)
{
    using namespace bnb;
    if (R < 0 || x_row_stride < D || N < 1) return BNB_ERR_BAD_SHAPE;
    if (D != kNlD || N % kNlChunkFeatures != 0) return BNB_ERR_UNSUPPORTED;
    if (R == 0) return 0;
    if (!x || !norm_weight || !weight_packed || !out || !n_out) return BNB_ERR_NULL_POINTER;
    if (!aligned16(x) || !aligned16(out) || !aligned16(n_out) || !aligned16(norm_weight) || !aligned16(weight_packed) ||
        (x_row_stride % 4) != 0)
        return BNB_ERR_MISALIGNED;
    const int64_t blocks = (R + kNlWaves * 32 - 1) / (kNlWaves * 32);
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(norm_linear_kernel, dim3((unsigned)blocks), dim3(kNlThreads), 0, (hipStream_t)stream, x,
                       x_row_stride, (const int32_t *)nullptr, (const int32_t *)nullptr, norm_weight, eps,
                       (const uint16_t *)weight_packed, (const float *)nullptr, (uint16_t *)out, R, N, (uint16_t *)n_out);
    return (int)hipGetLastError();
}

extern "C" int bnb_mask_count(const uint8_t *mask, int32_t *counts, int B, int n, void *stream)
{
    using namespace bnb;
    if (B < 0 || n < 1) return BNB_ERR_BAD_SHAPE;
    if (B == 0) return 0;
    if (!mask || !counts) return BNB_ERR_NULL_POINTER;
    hipLaunchKernelGGL(mask_count_kernel, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, mask, counts, n);
    return (int)hipGetLastError();
}

extern "C" int bnb_mask_fill(const uint8_t *mask, const int32_t *offsets, int32_t *index, int B, int n, void *stream)
{
    using namespace bnb;
    if (B < 0 || n < 1 || (int64_t)B * n > 0x7fffffffLL) return BNB_ERR_BAD_SHAPE;
    if (B == 0) return 0;
    if (!mask || !offsets || !index) return BNB_ERR_NULL_POINTER;
    hipLaunchKernelGGL(mask_fill_kernel, dim3((unsigned)B), dim3(64), 0, (hipStream_t)stream, mask, offsets, index, n);
    return (int)hipGetLastError();
}
