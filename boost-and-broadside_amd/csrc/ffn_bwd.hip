// Backward of the gated MLP on the matrix cores (gfx950), with the 1024-wide gate/up activations
// recomputed on chip instead of saved by the forward:
//
//   given  n  (R, 128) bf16   the normalised rows the forward projected
//          dy (R, 128)        gradient of y = h Wd^T                 (fp32 or bf16; used as bf16)
//   g, u = n Wg^T, n Wu^T                     (recomputed, fp32 accumulators)
//   dh   = dy Wd                              (R, 512)
//   h    = bf16(gelu(g) * u)                  -> written for the weight gradient dWd = dy^T h
//   dg   = bf16(dh * u * gelu'(g)), du = bf16(dh * gelu(g))   -> written for dWg = dg^T n, dWu = du^T n
//   dn   = bf16(dg Wg + du Wu)                -> the gradient that goes back into the norm
//
// Reference: the backward of `down_proj(F.gelu(gate_proj(x)) * up_proj(x))`, models/yemong/attention.py:21-37
// (GatedMLP), as autograd runs it under bf16 autocast in train/rl/ppo.py:1417-1425.  As library GEMMs
// and element-wise kernels this chain reads and writes the 512/1024-wide tensors five times (and the
// forward has to save g, u and h); here a wave owns 32 rows and the wide tensors exist only in
// registers, apart from the three bf16 operands of the weight-gradient kernel that leave once.
//
// Everything is computed transposed, as in the forward tail kernel: G^T (hidden x rows) =
// Wg (A) n^T (B), dH^T = Wd^T (A) dy^T (B), dN^T (channels x rows) += Wg^T (A) dG^T (B) + Wu^T (A) dU^T (B);
// a lane holds one row's column of every result, so dG^T and dU^T go from the accumulators straight
// into the B operands of the last product.  The weights (640 KB bf16 in this arrangement) stream
// through LDS in 16 chunks of 32 hidden units (40 KB) with two buffers; the next chunk travels
// from L2 straight into LDS while the current one is used; one barrier per chunk.  One work-group of
// eight waves per CU (80 KB of LDS, 256 registers per lane).
//
// Which hidden unit an MFMA row stands for is free, and chosen so that stores are dense without a
// trip through LDS: MFMA row 8i + 4b + j (i = 0..3, b = 0..1, j = 0..3) is hidden unit (or, in the last
// product, channel)  pi = 16 (i / 2) + 8 b + 4 (i % 2) + j  of its block of 32.  A lane (row m, half b)
// then owns two runs of eight consecutive units, 8b.. and 16 + 8b..; lanes m and m + 16 trade runs
// (v_permlane16_swap) and one store instruction writes the whole 64-byte piece of 16 rows.
//
// Layouts of the three weight-gradient operands (chosen for 128-byte lines per row and chunk, read by
// the weight-gradient kernel through its tile stride; Rp = R rounded up to the 256 rows of a work-group):
//   dgu [8][Rp][128]: pair p = chunk / 2, columns 64 (chunk % 2) + {dg: 0..31, du: 32..63}
//   h   [4][Rp][128]: quad q = chunk / 4, columns 32 (chunk % 4) + 0..31   (hidden order 128 q + column)
//
// Pack layout (bf16, built on the host side), chunk c, lane l = 32 b + m, e = 0..7, pi(m) as above:
//   [c][0][ks][l][e] = Wg[32c + pi(m)][16ks + 8b + e]          ks = 0..7   (gate)
//   [c][1][ks][l][e] = Wu[32c + pi(m)][16ks + 8b + e]                      (up)
//   [c][2][ks][l][e] = Wd[16ks + 8b + e][32c + pi(m)]                      (dh)
//   [c][3][cb][t][l][e] = Wg[32c + 16t + 8b + e][32cb + pi(m)]  cb = 0..3, t = 0..1   (dn through g)
//   [c][4][cb][t][l][e] = Wu[32c + 16t + 8b + e][32cb + pi(m)]                        (dn through u)
// Every MFMA A operand is one contiguous 1 KB run read with a single ds_read_b128.

#include <type_traits>

#include "common.h"
#include "ffn_math.h"

namespace bnb {

constexpr int kFbSection = 8 * 64 * 8;             // halfs per section: 4096 (8 KB)
constexpr int kFbChunkHalfs = 5 * kFbSection;      // 40 KB
constexpr int kFbWaves = 8;
constexpr int kFbThreads = kFbWaves * kWave;
constexpr int kFbPrefetch = kFbChunkHalfs / 8 / kFbThreads;  // 16-byte pieces per thread per chunk: 5
constexpr int kFbPitch = kFfnD + 8;                // halfs per staged operand row

template <typename DYT>
__global__ __launch_bounds__(kFbThreads) void ffn_bwd_kernel(
    const uint16_t *__restrict__ n, const DYT *__restrict__ dy, int64_t dy_stride, const uint16_t *__restrict__ wpack,
    uint16_t *__restrict__ dn, uint16_t *__restrict__ dgu, uint16_t *__restrict__ h, uint16_t *__restrict__ dy_lp, int64_t R,
    int64_t out_rows)
{
    __shared__ __align__(16) uint16_t s_w[2][kFbChunkHalfs];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31;
    const int half = lane >> 5;

    u32x4 pre[kFbPrefetch];
    auto fetch = [&](int c) {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(wpack + (int64_t)c * kFbChunkHalfs);
#pragma unroll
        for (int q = 0; q < kFbPrefetch; ++q) pre[q] = src[tid + q * kFbThreads];
    };
    auto stash = [&](int buf) {
        u32x4 *dst = reinterpret_cast<u32x4 *>(s_w[buf]);
#pragma unroll
        for (int q = 0; q < kFbPrefetch; ++q) dst[tid + q * kFbThreads] = pre[q];
    };
    fetch(0);

    const int64_t row0 = ((int64_t)blockIdx.x * kFbWaves + wave) * 32;

    // ---- n and dy as B operands: whole rows in, this lane's row out (k-slot e of step ks = channel 16ks + 8half + e) ----
    // through this wave's slice of the weight buffers, which the chunk loop does not need yet
    uint16_t *stage = &s_w[0][0] + wave * (32 * kFbPitch);
    const int a_row = lane >> 4;        // four bf16 rows per instruction
    const int a_col = (lane & 15) * 8;  // this lane's eight channels
    bf16x8 nb[8], db[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int64_t r = row0 + 4 * j + a_row;
        const int64_t rs = r < R ? r : R - 1;
        const u32x4 av = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(n + rs * kFfnD + a_col));
        *reinterpret_cast<u32x4 *>(stage + (4 * j + a_row) * kFbPitch + a_col) = av;
    }
    wave_lds_handover();
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
        nb[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(stage + m * kFbPitch + 16 * ks + 8 * half));
    wave_lds_handover();
    if constexpr (std::is_same<DYT, float>::value) {
        const int io_row = lane >> 5;        // two fp32 rows per instruction
        const int io_col = (lane & 31) * 4;  // this lane's four channels
        // all sixteen loads in flight before the first is used (a branch between them would serialise the round trips)
        f32x4 v[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int64_t r = row0 + 2 * j + io_row;
            const int64_t rs = r < R ? r : R - 1;
            v[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(dy + rs * dy_stride + io_col));
        }
        u32x2 pk[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            pk[j] = u32x2{pack_bf16x2(v[j].x, v[j].y), pack_bf16x2(v[j].z, v[j].w)};
            *reinterpret_cast<u32x2 *>(stage + (2 * j + io_row) * kFbPitch + io_col) = pk[j];
        }
        if (dy_lp != nullptr) {
#pragma unroll
            for (int j = 0; j < 16; ++j)
                __builtin_nontemporal_store(pk[j], reinterpret_cast<u32x2 *>(dy_lp + (row0 + 2 * j + io_row) * kFfnD + io_col));
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int64_t r = row0 + 4 * j + a_row;
            const int64_t rs = r < R ? r : R - 1;
            const u32x4 av = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(dy + rs * dy_stride + a_col));
            *reinterpret_cast<u32x4 *>(stage + (4 * j + a_row) * kFbPitch + a_col) = av;
        }
    }
    wave_lds_handover();
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
        db[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(stage + m * kFbPitch + 16 * ks + 8 * half));

    __syncthreads();  // every wave has its rows out of the staging area
    stash(0);
    __syncthreads();

    // from here on a chunk travels global -> LDS directly (global_load_lds_dwordx4: a wave moves 1 KB per
    // instruction, lane l filling bytes 16 l .. 16 l + 15 of its kilobyte): no registers, no LDS store instructions
    const uint32_t lds_w = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)&s_w[0][0];
    constexpr int kDmaPerWave = kFbChunkHalfs / 512 / kFbWaves;  // 1 KB pieces per wave and chunk: 5
    auto dma_chunk = [&](int c, int buf) {
        const uint16_t *src = wpack + (int64_t)c * kFbChunkHalfs + wave * (kDmaPerWave * 512);  // wave-uniform
        const uint32_t dst = lds_w + (uint32_t)(buf * kFbChunkHalfs * 2 + wave * (kDmaPerWave * 1024));
#pragma unroll
        for (int q = 0; q < kDmaPerWave; ++q)
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0"
                         :
                         : "s"(src + q * 512), "v"((uint32_t)(lane * 16)), "s"(dst + (uint32_t)(q * 1024))
                         : "memory", "m0");
    };

    f32x16 acc[4];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[cb][v] = 0.0f;

    // where this lane's pieces of a chunk's results go: rows m % 16 and 16 + m % 16 of the wave's 32,
    // eight units starting at 16 (m / 16) + 8 half of the chunk's 32
    // Every store is unconditional: the results have room for all rows of the launch's work-groups (out_rows, a
    // multiple of the 256 rows of a work-group; rows past R hold copies of row R - 1's results).  A store under a
    // branch would make the wait for the weight prefetch below also wait for the stores issued after it.
    const int64_t out_row = row0 + (m & 15);
    const int out_col = 16 * (m >> 4) + 8 * half;
    // lanes m and m + 16 trade runs: w[0] becomes the piece of row m % 16, w[1] that of row 16 + m % 16
    auto trade = [&](u32x4 (&w)[2]) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const u32x2 t = __builtin_amdgcn_permlane16_swap(w[0][q], w[1][q], false, false);
            w[0][q] = t.x, w[1][q] = t.y;
        }
    };

#pragma unroll 1
    for (int c = 0; c < kFfnChunks; ++c) {
        // chunk c + 1 into the buffer that chunk c - 1 was read from (everyone is past the barrier that ended it)
        if (c + 1 < kFfnChunks) dma_chunk(c + 1, (c + 1) & 1);
        const uint16_t *wb = s_w[c & 1] + lane * 8;
        f32x16 g, u, dh;
#pragma unroll
        for (int v = 0; v < 16; ++v) g[v] = u[v] = dh[v] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const bf16x8 ag = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wb + ks * 512));
            const bf16x8 au = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wb + kFbSection + ks * 512));
            const bf16x8 ad = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wb + 2 * kFbSection + ks * 512));
            g = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ag, nb[ks], g, 0, 0, 0);
            u = __builtin_amdgcn_mfma_f32_32x32x16_bf16(au, nb[ks], u, 0, 0, 0);
            dh = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ad, db[ks], dh, 0, 0, 0);
        }
        // accumulator register v = 4i + j of half b is MFMA row 8i + 4b + j, i.e. unit 16(i/2) + 8b + 4(i%2) + j:
        // registers 0..7 are units 8b..8b+7, registers 8..15 units 16 + 8b..; k-slot e of step t of the last
        // product is register 8t + e, unit 16t + 8b + e
        u32x4 hw[2], gw[2], uw[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            float hv[8], gv[8], uv[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float gg = g[8 * t + e], uu = u[8 * t + e], dd = dh[8 * t + e];
                const float cdf = normal_cdf_fit(gg);
                const float gl = gg * cdf;
                hv[e] = gl * uu;
                uv[e] = dd * gl;
                gv[e] = (dd * uu) * fmaf(gg, normal_pdf(gg), cdf);
            }
            hw[t] = u32x4{pack_bf16x2(hv[0], hv[1]), pack_bf16x2(hv[2], hv[3]), pack_bf16x2(hv[4], hv[5]), pack_bf16x2(hv[6], hv[7])};
            gw[t] = u32x4{pack_bf16x2(gv[0], gv[1]), pack_bf16x2(gv[2], gv[3]), pack_bf16x2(gv[4], gv[5]), pack_bf16x2(gv[6], gv[7])};
            uw[t] = u32x4{pack_bf16x2(uv[0], uv[1]), pack_bf16x2(uv[2], uv[3]), pack_bf16x2(uv[4], uv[5]), pack_bf16x2(uv[6], uv[7])};
        }
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const bf16x8 a3 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wb + 3 * kFbSection + (cb * 2 + t) * 512));
                const bf16x8 a4 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wb + 4 * kFbSection + (cb * 2 + t) * 512));
                acc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3, __builtin_bit_cast(bf16x8, gw[t]), acc[cb], 0, 0, 0);
                acc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a4, __builtin_bit_cast(bf16x8, uw[t]), acc[cb], 0, 0, 0);
            }
        }
        // the three weight-gradient operands of this chunk leave as 64-byte pieces of 16 rows per instruction
        trade(hw);
        trade(gw);
        trade(uw);
        {
            uint16_t *hp = h + ((int64_t)(c >> 2) * out_rows + out_row) * 128 + 32 * (c & 3) + out_col;
            uint16_t *gp = dgu + ((int64_t)(c >> 1) * out_rows + out_row) * 128 + 64 * (c & 1) + out_col;
            __builtin_nontemporal_store(hw[0], reinterpret_cast<u32x4 *>(hp));
            __builtin_nontemporal_store(gw[0], reinterpret_cast<u32x4 *>(gp));
            __builtin_nontemporal_store(uw[0], reinterpret_cast<u32x4 *>(gp + 32));
            __builtin_nontemporal_store(hw[1], reinterpret_cast<u32x4 *>(hp + 16 * 128));
            __builtin_nontemporal_store(gw[1], reinterpret_cast<u32x4 *>(gp + 16 * 128));
            __builtin_nontemporal_store(uw[1], reinterpret_cast<u32x4 *>(gp + 16 * 128 + 32));
        }
        // this wave's part of chunk c + 1 has landed when at most the six stores above (issued after it) are
        // outstanding: vmcnt counts loads and stores in issue order
        __builtin_amdgcn_s_waitcnt(0x0f76);  // vmcnt(6)
        __syncthreads();
    }

    // ---- dn: register v = 4i + j of block cb is channel 32cb + 16(i/2) + 8half + 4(i%2) + j, the same two runs ----
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) {
        u32x4 w[2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
            w[t] = u32x4{pack_bf16x2(acc[cb][8 * t], acc[cb][8 * t + 1]), pack_bf16x2(acc[cb][8 * t + 2], acc[cb][8 * t + 3]),
                         pack_bf16x2(acc[cb][8 * t + 4], acc[cb][8 * t + 5]), pack_bf16x2(acc[cb][8 * t + 6], acc[cb][8 * t + 7])};
        trade(w);
        uint16_t *p = dn + out_row * kFfnD + 32 * cb + out_col;
        __builtin_nontemporal_store(w[0], reinterpret_cast<u32x4 *>(p));
        __builtin_nontemporal_store(w[1], reinterpret_cast<u32x4 *>(p + 16 * kFfnD));
    }
}

}  // namespace bnb

extern "C" int bnb_ffn_bwd(const void *n, const void *dy, int dy_dtype, int64_t dy_row_stride, const void *weights_packed,
                           void *dn, void *dgu, void *h, void *dy_bf16, int64_t R, int64_t out_rows, int D, int hidden,
                           void *stream)
{
    using namespace bnb;
    if (R < 0 || dy_row_stride < D || out_rows < R || out_rows % (kFbWaves * 32) != 0) return BNB_ERR_BAD_SHAPE;
    if (D != kFfnD || hidden != kFfnHidden) return BNB_ERR_UNSUPPORTED;
    if (dy_dtype != BNB_F32 && dy_dtype != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (R == 0) return 0;
    if (!n || !dy || !weights_packed || !dn || !dgu || !h) return BNB_ERR_NULL_POINTER;
    if (!aligned16(n) || !aligned16(dy) || !aligned16(weights_packed) || !aligned16(dn) || !aligned16(dgu) || !aligned16(h) ||
        (dy_bf16 && !aligned16(dy_bf16)) || dy_row_stride % (dy_dtype == BNB_F32 ? 4 : 8) != 0)
        return BNB_ERR_MISALIGNED;
    const int64_t blocks = (R + kFbWaves * 32 - 1) / (kFbWaves * 32);
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    if (dy_dtype == BNB_F32)
        hipLaunchKernelGGL((ffn_bwd_kernel<float>), dim3((unsigned)blocks), dim3(kFbThreads), 0, s, (const uint16_t *)n,
                           (const float *)dy, dy_row_stride, (const uint16_t *)weights_packed, (uint16_t *)dn, (uint16_t *)dgu,
                           (uint16_t *)h, (uint16_t *)dy_bf16, R, out_rows);
    else
        hipLaunchKernelGGL((ffn_bwd_kernel<uint16_t>), dim3((unsigned)blocks), dim3(kFbThreads), 0, s, (const uint16_t *)n,
                           (const uint16_t *)dy, dy_row_stride, (const uint16_t *)weights_packed, (uint16_t *)dn,
                           (uint16_t *)dgu, (uint16_t *)h, nullptr, R, out_rows);
    return (int)hipGetLastError();
}
