// Residual add + RMSNorm + gated MLP + residual add as ONE kernel on the matrix cores (gfx950).
//
//   s   = x + delta                                   (fp32 residual stream, delta bf16)
//   n   = bf16(s * rsqrt(mean(s^2) + eps) * w_norm)
//   g,u = n Wg^T, n Wu^T                              (D = 128 -> hidden = 512, fp32 accumulators)
//   h   = bf16(gelu(g) * u)
//   out = s + h Wd^T                                  (fp32)
// Reference: `x = x + attn(...)`, `x + self.ffn(self.norm2(x))` of models/yemong/attention.py:97-99
// with GatedMLP :21-37, and the same tail of the temporal block, models/yemong/griffin.py:284-286,
// as they run under bf16 autocast.
//
// As separate library GEMMs this sublayer moves the 1024-wide gate/up activations through
// memory three times; here a wave owns 32 tokens and nothing but x, delta and out touches
// HBM.  Everything is computed transposed so that results feed the next MFMA from registers:
//   G^T (hidden x tokens) = Wg (A) * n^T (B),  out^T (channels x tokens) += Wd (A) * h^T (B).
// v_mfma_f32_32x32x16_bf16 leaves a lane with one token column of G^T (16 hidden units), and
// those 16 values are exactly the B operand the lane must supply for out^T when the A operand
// (Wd) lists the hidden units in the same order; the weights are stored pre-arranged for that
// (pack layout below).  The lane also owns its token's s values in the accumulator layout of
// out^T, so `s` is simply the initial accumulator, and with the channel order chosen in the
// pack the same registers are the B operand of the first GEMM after normalisation.
// The weights (384 KB bf16) stream through LDS in 16 chunks of 32 hidden units (24 KB) with
// three buffers: chunk c+2 travels from L2 straight into LDS (global_load_lds_dwordx4, no registers and
// no LDS store instructions) while the down projection of chunk c and the gate/up products of chunk c+1
// are formed; one barrier per chunk.
//
// Channel order: k-slot e of contraction step ks in a lane of half h stands for channel
//   ch(ks, h, e) = 16ks + 8(e/4) + 4h + e%4
// (the two lanes holding one token then own interleaved runs of four channels: 16-byte LDS
// accesses on both sides of the staging area).  x, delta and out move between HBM and the
// token-owning lanes through LDS, so that global accesses are whole rows: per-token 16-byte
// pieces 512 bytes apart ran the same traffic at less than half the bandwidth.
//
// Pack layout (bf16, built once on the host side), chunk c = hidden units 32c..32c+31,
// lane l = 32*h + m, e = 0..7:
//   [c][0][ks][l][e] = Wg[32c + m][ch(ks, h, e)]                              ks = 0..7
//   [c][1][ks][l][e] = Wu[32c + m][ch(ks, h, e)]
//   [c][2][cb][t][l][e] = Wd[32cb + m][32c + 16t + 8(e/4) + 4h + e%4]         cb = 0..3, t = 0..1
// i.e. every MFMA A operand is one contiguous 1 KB run read with a single ds_read_b128.

#include <type_traits>

#include "common.h"
#include "ffn_math.h"

namespace bnb {

constexpr int kFfnChunkHalfs = 3 * 32 * kFfnD;  // 12288 bf16 = 24 KB
constexpr int kFfnWaves = 4;
constexpr int kFfnThreads = kFfnWaves * kWave;
constexpr int kFfnPrefetch = kFfnChunkHalfs / 8 / kFfnThreads;  // 16-byte pieces per thread per chunk

// What is added to x before the norm (the output of the sublayer the tail belongs to):
//   kDeltaNone  nothing;  kDeltaRows  the bf16 rows `delta`;
//   kDeltaProj  rows_a Wp^T  (the block's output projection: attention.py:168-169 `out_proj`)
//   kDeltaGate  (bf16(gelu(rows_a)) * rows_b) Wp^T  (griffin.py:281-283: `b1_out * gelu(linear2(..))`
//               through `linear_out`), with the roundings torch's bf16 gelu and product have.
// The projection is a 128 x 128 matrix product on the same MFMA layouts: its operand rows come
// in through the staging area like x, the 32 KB of Wp sit in the weight buffers before the
// chunk loop needs them, and the products accumulate straight onto x in the accumulators.
enum { kDeltaNone = 0, kDeltaRows = 1, kDeltaProj = 2, kDeltaGate = 3 };
constexpr int kProjPitch = kFfnD + 8;  // halfs per staged operand row (bank spread, 16-byte aligned)

// TRAIN: the update path's forward.  It also writes what the backward needs and nothing else saves: the
// residual sum `s` (when there is a delta; otherwise s is x) and the normalised rows `n` in bf16.
// HEAD: the kernel goes on to the head of the NEXT sublayer, which is a norm and a projection of the rows it has
// just produced (`qkv(norm1(x))` of models/yemong/attention.py:94-96,132, `[linear1 | linear2](norm1(x))` of
// griffin.py:269-283): head = bf16(rmsnorm(out) * next_norm_w) Wh^T, N_h features (a multiple of 64), written
// as bf16 rows.  The rows never come back from memory for it, and one launch with its own row I/O disappears.
// Wh streams through the same three weight buffers as chunks 16, 17, ... of the pipeline, 64 features (16 KB) at
// a time: [c][b][ks][l][e] = Wh[64c + 32b + pi(l%32)][16ks + 8(e/4) + 4(l/32) + e%4] with
// pi(m) = 16(m/16) + 8((m/4)%2) + 4((m/8)%2) + m%4, the row order that leaves a lane with two runs of eight
// consecutive features, which lanes m and m + 16 trade (v_permlane16_swap) so that a store instruction writes whole
// 64-byte pieces of 16 rows.  The stores are unconditional: next_out has room for whole work-groups of 128 rows.
template <int MODE, bool TRAIN = false, bool HEAD = false>
__global__ __launch_bounds__(kFfnThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void ffn_fused_kernel(
    const float *__restrict__ x, int64_t x_stride, const uint16_t *__restrict__ delta,
    const uint16_t *__restrict__ rows_b, const uint16_t *__restrict__ wproj, const float *__restrict__ norm_w,
    float eps, const uint16_t *__restrict__ wpack, float *__restrict__ out, int64_t R, int64_t rows_a_stride, int64_t rows_b_stride, unsigned first_round,
    float *__restrict__ s_out = nullptr, uint16_t *__restrict__ n_out = nullptr, const float *__restrict__ next_norm_w = nullptr,
    float next_eps = 0.0f, const uint16_t *__restrict__ next_wpack = nullptr, uint16_t *__restrict__ next_out = nullptr,
    int next_features = 0)
{
    constexpr bool HAS_DELTA = MODE == kDeltaRows;
    // three weight buffers: chunk c is used while chunk c+1 is already complete (its operands
    // are read one chunk ahead) and chunk c+2 is on its way in
    __shared__ __align__(16) uint16_t s_w[3][kFfnChunkHalfs];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31;
    const int half = lane >> 5;

    u32x4 pre[kFfnPrefetch], pre1[kFfnPrefetch];
    auto fetch = [&](int c, u32x4 (&dst)[kFfnPrefetch]) {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(wpack + (int64_t)c * kFfnChunkHalfs);
#pragma unroll
        for (int q = 0; q < kFfnPrefetch; ++q) dst[q] = src[tid + q * kFfnThreads];
    };
    auto stash = [&](int buf, const u32x4 (&src)[kFfnPrefetch]) {
        u32x4 *dst = reinterpret_cast<u32x4 *>(s_w[buf]);
#pragma unroll
        for (int q = 0; q < kFfnPrefetch; ++q) dst[tid + q * kFfnThreads] = src[q];
    };
    // inside the loop a chunk travels global -> LDS directly (global_load_lds_dwordx4: a wave moves 1 KB per
    // instruction, lane l filling bytes 16 l .. 16 l + 15 of its kilobyte): no registers, no LDS store instructions
    const uint32_t lds_w = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)&s_w[0][0];
    constexpr int kDmaPerWave = kFfnChunkHalfs / 512 / kFfnWaves;  // 1 KB pieces per wave and chunk: 6
    auto dma_chunk = [&](int c, int buf) {
        const uint16_t *src = wpack + (int64_t)c * kFfnChunkHalfs + wave * (kDmaPerWave * 512);  // wave-uniform
        const uint32_t dst = lds_w + (uint32_t)(buf * kFfnChunkHalfs * 2 + wave * (kDmaPerWave * 1024));
#pragma unroll
        for (int q = 0; q < kDmaPerWave; ++q)
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0"
                         :
                         : "s"(src + q * 512), "v"((uint32_t)(lane * 16)), "s"(dst + (uint32_t)(q * 1024))
                         : "memory", "m0");
    };
    // a chunk of the next sublayer's head: 64 features = 16 KB, four 1 KB pieces per wave, into the front of a buffer
    constexpr int kHeadChunkHalfs = 64 * kFfnD;
    auto dma_head = [&](int hc, int buf) {
        const uint16_t *src = next_wpack + (int64_t)hc * kHeadChunkHalfs + wave * (4 * 512);  // wave-uniform
        const uint32_t dst = lds_w + (uint32_t)(buf * kFfnChunkHalfs * 2 + wave * (4 * 1024));
#pragma unroll
        for (int q = 0; q < 4; ++q)
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0"
                         :
                         : "s"(src + q * 512), "v"((uint32_t)(lane * 16)), "s"(dst + (uint32_t)(q * 1024))
                         : "memory", "m0");
    };
    // Every work-group takes the same time, so the two that share a CU would move in lockstep for
    // the whole launch: both reading rows, then both on the matrix cores, then both writing,
    // and neither HBM nor the CU is busy all the time.  A short head start for every other
    // work-group of the first round (the later ones inherit it: a slot frees when its
    // predecessor ends) lets one work-group's row I/O run under the other's arithmetic.
    // Measured at 655,360 rows: 460 -> 388 us when the same launch repeats back to back (the
    // length of the pause hardly matters, 2..12 us); behind other kernels, whose ragged ends
    // already stagger the first round, the effect is within noise.
    if (blockIdx.x < first_round && (blockIdx.x & 1)) __builtin_amdgcn_s_sleep(64);
    fetch(0, pre);
    fetch(1, pre1);

    const int64_t row0 = ((int64_t)blockIdx.x * kFfnWaves + wave) * 32;
    // ---- operand rows of the projection (modes Proj / Gate): whole 256-byte rows in, k-slot order out ----
    bf16x8 mb[8];
    if (MODE == kDeltaProj || MODE == kDeltaGate) {
        uint16_t *stage_a = &s_w[0][0] + wave * (32 * kProjPitch);
        const int a_row = lane >> 4;        // four rows per instruction
        const int a_col = (lane & 15) * 8;  // this lane's eight channels
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int64_t r = row0 + 4 * j + a_row;
            const int64_t rs = r < R ? r : R - 1;
            u32x4 av = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(delta + rs * rows_a_stride + a_col));
            if (MODE == kDeltaGate) {
                const Row8 g = load8(reinterpret_cast<const uint16_t *>(&av));
                const Row8 y = load8_stream(rows_b + rs * rows_b_stride + a_col);
                float p[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) p[e] = round_to_bf16(gelu_phi(g.v[e])) * y.v[e];  // 2.6e-5 from erf-GELU, far below the bf16 rounding that follows
                av = u32x4{pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]),
                           pack_bf16x2(p[6], p[7])};
            }
            *reinterpret_cast<u32x4 *>(stage_a + (4 * j + a_row) * kProjPitch + a_col) = av;
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const uint16_t *sp = stage_a + m * kProjPitch + 16 * ks + 4 * half;
            const u32x2 lo = *reinterpret_cast<const u32x2 *>(sp);
            const u32x2 hi = *reinterpret_cast<const u32x2 *>(sp + 8);
            mb[ks] = __builtin_bit_cast(bf16x8, u32x4{lo.x, lo.y, hi.x, hi.y});
        }
        __syncthreads();
    }

    // ---- s = x + delta for this wave's 32 tokens ----
    // Read as whole rows (a half-wave per 512-byte row, 16 bytes per lane) and handed to the
    // lanes that own the tokens through this wave's slice of the still unused weight buffers:
    // row r at r * kRowPitch floats, the pitch keeping the 32 row starts on different banks.
    constexpr int kRowPitch = kFfnD + 4;
    float *stage = reinterpret_cast<float *>(&s_w[0][0]) + wave * (32 * kRowPitch);
    const int io_row = lane >> 5;        // which of the two rows of one instruction
    const int io_col = (lane & 31) * 4;  // first of this lane's four channels
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int64_t r = row0 + 2 * j + io_row;
        const int64_t rs = r < R ? r : R - 1;
        f32x4 sv = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(x + rs * x_stride + io_col));
        if (HAS_DELTA) {
            const u32x2 dv = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(delta + rs * kFfnD + io_col));
            sv.x += __uint_as_float(dv.x << 16);
            sv.y += __uint_as_float(dv.x & 0xffff0000u);
            sv.z += __uint_as_float(dv.y << 16);
            sv.w += __uint_as_float(dv.y & 0xffff0000u);
            if (TRAIN && r < R) __builtin_nontemporal_store(sv, reinterpret_cast<f32x4 *>(s_out + r * kFfnD + io_col));
        }
        *reinterpret_cast<f32x4 *>(stage + (2 * j + io_row) * kRowPitch + io_col) = sv;
    }
    __syncthreads();

    // the lane's own token in the accumulator layout, and its sum of squares
    f32x16 acc[4];
    float ss = 0.0f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
        // k-slots 0..3 / 4..7 of step ks: channels 16ks + 4half + 0..3 and 16ks + 8 + 4half + 0..3;
        // they are accumulator registers 8(ks%2) + 0..7 of channel block ks/2
        const float *sp = stage + m * kRowPitch + 16 * ks + 4 * half;
        const f32x4 lo = *reinterpret_cast<const f32x4 *>(sp);
        const f32x4 hi = *reinterpret_cast<const f32x4 *>(sp + 8);
        const float sv[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[ks >> 1][8 * (ks & 1) + e] = sv[e];
    }
    if (MODE == kDeltaProj || MODE == kDeltaGate) {
        // Wp (128 x 128 bf16, packed [cb][ks][lane][8] = Wp[32cb + lane%32][ch(ks, lane/32, .)]) into the
        // weight buffers once everyone is done with the staging area, then 32 MFMAs onto x
        __syncthreads();
        {
            const u32x4 *src = reinterpret_cast<const u32x4 *>(wproj);
            u32x4 *dst = reinterpret_cast<u32x4 *>(&s_w[0][0]);
            u32x4 t[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) t[q] = src[tid + q * kFfnThreads];
#pragma unroll
            for (int q = 0; q < 8; ++q) dst[tid + q * kFfnThreads] = t[q];
        }
        __syncthreads();
        const uint16_t *wp = &s_w[0][0] + lane * 8;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
#pragma unroll
            for (int cb = 0; cb < 4; ++cb) {
                const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wp + (cb * 8 + ks) * 512));
                acc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, mb[ks], acc[cb], 0, 0, 0);
            }
        }
    }
    if (TRAIN && (MODE == kDeltaProj || MODE == kDeltaGate)) {
        // s exists only in the accumulators here: out through the staging area as whole rows, like `out` at the end
        __syncthreads();  // every wave is done reading Wp out of the weight buffers
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const f32x16 &a = acc[ks >> 1];
            const int v0 = 8 * (ks & 1);
            float *sp = stage + m * kRowPitch + 16 * ks + 4 * half;
            *reinterpret_cast<f32x4 *>(sp) = f32x4{a[v0], a[v0 + 1], a[v0 + 2], a[v0 + 3]};
            *reinterpret_cast<f32x4 *>(sp + 8) = f32x4{a[v0 + 4], a[v0 + 5], a[v0 + 6], a[v0 + 7]};
        }
        wave_lds_handover();
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int64_t r = row0 + 2 * j + io_row;
            const f32x4 sv = *reinterpret_cast<const f32x4 *>(stage + (2 * j + io_row) * kRowPitch + io_col);
            if (r < R) __builtin_nontemporal_store(sv, reinterpret_cast<f32x4 *>(s_out + r * kFfnD + io_col));
        }
    }
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) ss = fmaf(acc[cb][v], acc[cb][v], ss);
    }
    ss += __shfl_xor(ss, 32);
    const float rstd = rsqrtf(ss * (1.0f / kFfnD) + eps);

    // ---- n = rmsnorm(s) as the B operand of the first GEMM (k-slot e of step ks = channel ch(ks, half, e)) ----
    bf16x8 nb[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
        const f32x4 wl = *reinterpret_cast<const f32x4 *>(norm_w + 16 * ks + 4 * half);
        const f32x4 wh = *reinterpret_cast<const f32x4 *>(norm_w + 16 * ks + 8 + 4 * half);
        const float wv[8] = {wl.x, wl.y, wl.z, wl.w, wh.x, wh.y, wh.z, wh.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) nb[ks][e] = (__bf16)((acc[ks >> 1][8 * (ks & 1) + e] * rstd) * wv[e]);
    }

    if (TRAIN) {
        // n leaves as whole 256-byte rows through this wave's slice of the staging area
        uint16_t *stage_n = reinterpret_cast<uint16_t *>(stage);
        wave_lds_handover();
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const u32x4 v = __builtin_bit_cast(u32x4, nb[ks]);
            uint16_t *sp = stage_n + m * kProjPitch + 16 * ks + 4 * half;
            *reinterpret_cast<u32x2 *>(sp) = u32x2{v.x, v.y};
            *reinterpret_cast<u32x2 *>(sp + 8) = u32x2{v.z, v.w};
        }
        wave_lds_handover();
        const int a_row = lane >> 4, a_col = (lane & 15) * 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int64_t r = row0 + 4 * j + a_row;
            const u32x4 v = *reinterpret_cast<const u32x4 *>(stage_n + (4 * j + a_row) * kProjPitch + a_col);
            if (r < R) __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(n_out + r * kFfnD + a_col));
        }
    }
    __syncthreads();  // every wave has its tokens out of the staging area
    stash(0, pre);
    stash(1, pre1);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // every load so far is back: no wait on them inside the loop
    __syncthreads();

    // ---- the chunk loop, software-pipelined inside the wave ----
    // Step c issues the gate/up MFMAs of chunk c+1 between the GELU arithmetic of chunk c
    // (two elements per pair of MFMAs: about eight vector-ALU operations per MFMA, the ratio
    // at which neither pipe waits for the other), then the down-projection MFMAs of chunk c.
    // The LDS latency of the operand reads hides behind the same arithmetic.
    auto gate_up_pair = [&](const uint16_t *wgu, int ks, f32x16 &gn, f32x16 &un) {
        const bf16x8 a0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wgu + ks * 512));
        const bf16x8 a1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wgu + 4096 + ks * 512));
        gn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, nb[ks], gn, 0, 0, 0);
        un = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, nb[ks], un, 0, 0, 0);
    };
    f32x16 gA = {0.0f}, uA = {0.0f}, gB = {0.0f}, uB = {0.0f};
    {
        const uint16_t *wgu = s_w[0] + lane * 8;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) gate_up_pair(wgu, ks, gA, uA);
    }

    // FETCH: chunk c+2 exists and is brought in; NEXT: chunk c+1 exists and its gate/up products are formed
    auto step = [&](auto fetch_tag, auto next_tag, int c, int buf, const f32x16 &g, const f32x16 &u, f32x16 &gn,
                    f32x16 &un) {
        constexpr bool FETCH = decltype(fetch_tag)::value, NEXT = decltype(next_tag)::value;
        const int buf1 = buf == 2 ? 0 : buf + 1;
        const int buf2 = buf1 == 2 ? 0 : buf1 + 1;
        if (FETCH) {  // into the buffer chunk c - 1 was read from: everyone is past the barrier that ended it
            if (!HEAD || c + 2 < kFfnChunks) dma_chunk(c + 2, buf2);
            else dma_head(c + 2 - kFfnChunks, buf2);  // the pipeline goes on with the head's weights
        }
        const uint16_t *wgu = s_w[buf1] + lane * 8;
        const uint16_t *wd = s_w[buf] + lane * 8 + 8192;
        bf16x8 hb[2];
        if (NEXT) {
#pragma unroll
            for (int v = 0; v < 16; ++v) gn[v] = un[v] = 0.0f;
        }
        // operands are read one MFMA pair ahead of their use, the first down-projection operands
        // during the last of the GELU arithmetic (into registers g and u give up)
        u32x4 a0 = {0u, 0u, 0u, 0u}, a1 = a0, ad[8];
        if (NEXT) {
            a0 = *reinterpret_cast<const u32x4 *>(wgu);
            a1 = *reinterpret_cast<const u32x4 *>(wgu + 4096);
        }
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            u32x4 n0 = a0, n1 = a1;
            if (NEXT && ks < 7) {
                n0 = *reinterpret_cast<const u32x4 *>(wgu + (ks + 1) * 512);
                n1 = *reinterpret_cast<const u32x4 *>(wgu + 4096 + (ks + 1) * 512);
            }
            if (NEXT) {
                gn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a0), nb[ks], gn, 0, 0, 0);
                un = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a1), nb[ks], un, 0, 0, 0);
            }
            // h = bf16(gelu(g) * u): one rounding where the library composition has four
#pragma unroll
            for (int v = 2 * ks; v < 2 * ks + 2; ++v) hb[v >> 3][v & 7] = (__bf16)(gelu_phi(g[v]) * u[v]);
            if (ks >= 6) {
                ad[2 * (ks - 6)] = *reinterpret_cast<const u32x4 *>(wd + (2 * (ks - 6)) * 512);
                ad[2 * (ks - 6) + 1] = *reinterpret_cast<const u32x4 *>(wd + (2 * (ks - 6) + 1) * 512);
            }
            a0 = n0;
            a1 = n1;
        }
        // operand (cb, t) sits at index 2cb + t; blocks 0 and 1 are in, 2 and 3 follow while those MFMAs run
#pragma unroll
        for (int q = 0; q < 4; ++q) ad[4 + q] = *reinterpret_cast<const u32x4 *>(wd + (4 + q) * 512);
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
                acc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ad[cb * 2 + t]), hb[t],
                                                                  acc[cb], 0, 0, 0);
        }
        if (FETCH) __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of chunk c + 2 is in LDS
        __syncthreads();
    };
    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;
    int buf = 0;  // chunk % 3
    for (int c = 0; c < kFfnChunks - 2; c += 2) {
        step(yes{}, yes{}, c, buf, gA, uA, gB, uB);
        buf = buf == 2 ? 0 : buf + 1;
        step(yes{}, yes{}, c + 1, buf, gB, uB, gA, uA);
        buf = buf == 2 ? 0 : buf + 1;
    }
    using more = std::integral_constant<bool, HEAD>;
    step(more{}, yes{}, kFfnChunks - 2, buf, gA, uA, gB, uB);
    buf = buf == 2 ? 0 : buf + 1;
    step(more{}, no{}, kFfnChunks - 1, buf, gB, uB, gA, uA);

    if constexpr (HEAD) {
        // ---- head of the next sublayer: n2 = rmsnorm(out) as B operand, as n was formed from s above ----
        float ss2 = 0.0f;
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) {
#pragma unroll
            for (int v = 0; v < 16; ++v) ss2 = fmaf(acc[cb][v], acc[cb][v], ss2);
        }
        ss2 += __shfl_xor(ss2, 32);
        const float rstd2 = rsqrtf(ss2 * (1.0f / kFfnD) + next_eps);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const f32x4 wl = *reinterpret_cast<const f32x4 *>(next_norm_w + 16 * ks + 4 * half);
            const f32x4 wh = *reinterpret_cast<const f32x4 *>(next_norm_w + 16 * ks + 8 + 4 * half);
            const float wv[8] = {wl.x, wl.y, wl.z, wl.w, wh.x, wh.y, wh.z, wh.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) nb[ks][e] = (__bf16)((acc[ks >> 1][8 * (ks & 1) + e] * rstd2) * wv[e]);
        }
        const int nhc = next_features >> 6;
        const int64_t out_row = row0 + (m & 15);
        for (int hc = 0; hc < nhc; ++hc) {
            buf = buf == 2 ? 0 : buf + 1;  // buffer of pipeline chunk 16 + hc
            const int buf1 = buf == 2 ? 0 : buf + 1;
            const int buf2 = buf1 == 2 ? 0 : buf1 + 1;
            if (hc + 2 < nhc) dma_head(hc + 2, buf2);
            const uint16_t *wb = s_w[buf] + lane * 8;
            f32x16 z0 = {0.0f}, z1 = {0.0f};
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                const bf16x8 a0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wb + ks * 512));
                const bf16x8 a1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(wb + 4096 + ks * 512));
                z0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, nb[ks], z0, 0, 0, 0);
                z1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, nb[ks], z1, 0, 0, 0);
            }
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const f32x16 &z = b ? z1 : z0;
                // registers 0..7: features 8 half .. + 7 of the block, registers 8..15: 16 + 8 half ..
                u32x4 w[2];
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    w[t] = u32x4{pack_bf16x2(z[8 * t], z[8 * t + 1]), pack_bf16x2(z[8 * t + 2], z[8 * t + 3]),
                                 pack_bf16x2(z[8 * t + 4], z[8 * t + 5]), pack_bf16x2(z[8 * t + 6], z[8 * t + 7])};
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const u32x2 t = __builtin_amdgcn_permlane16_swap(w[0][q], w[1][q], false, false);
                    w[0][q] = t.x, w[1][q] = t.y;
                }
                // w[0]: row m % 16, w[1]: row 16 + m % 16; features 16 (m / 16) + 8 half .. + 7 of the block
                uint16_t *p = next_out + out_row * next_features + hc * 64 + 32 * b + 16 * (m >> 4) + 8 * half;
                *reinterpret_cast<u32x4 *>(p) = w[0];
                *reinterpret_cast<u32x4 *>(p + 16 * (int64_t)next_features) = w[1];
            }
            // this wave's part of head chunk hc + 2 has landed when at most the four stores above (issued after
            // it) are outstanding: vmcnt counts loads and stores in issue order
            __builtin_amdgcn_s_waitcnt(0x0f74);  // vmcnt(4)
            __syncthreads();
        }
    }

    // ---- out: back through the staging area (the loop's last barrier has freed the weight
    //      buffers) so that rows leave as whole 512-byte runs ----
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
        const f32x16 &a = acc[ks >> 1];
        const int v0 = 8 * (ks & 1);
        float *sp = stage + m * kRowPitch + 16 * ks + 4 * half;
        *reinterpret_cast<f32x4 *>(sp) = f32x4{a[v0], a[v0 + 1], a[v0 + 2], a[v0 + 3]};
        *reinterpret_cast<f32x4 *>(sp + 8) = f32x4{a[v0 + 4], a[v0 + 5], a[v0 + 6], a[v0 + 7]};
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int64_t r = row0 + 2 * j + io_row;
        const f32x4 ov = *reinterpret_cast<const f32x4 *>(stage + (2 * j + io_row) * kRowPitch + io_col);
        if (r < R) __builtin_nontemporal_store(ov, reinterpret_cast<f32x4 *>(out + r * kFfnD + io_col));
    }
}

}  // namespace bnb

namespace bnb {

struct NextHead {
    const float *norm_weight = nullptr;
    float eps = 0.0f;
    const void *packed = nullptr;
    void *out = nullptr;
    int features = 0;
};

template <int MODE, bool TRAIN = false, bool HEAD = false>
static int launch_ffn(const float *x, int64_t x_stride, const void *rows_a, const void *rows_b, const void *wproj,
                      const float *norm_weight, float eps, const void *weights_packed, float *out, int64_t R,
                      int64_t rows_a_stride, int64_t rows_b_stride, hipStream_t s, float *s_out = nullptr,
                      uint16_t *n_out = nullptr, NextHead next = NextHead())
{
    const int64_t blocks = (R + kFfnWaves * 32 - 1) / (kFfnWaves * 32);
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    // work-groups resident at once: two per CU (registers and LDS)
    static unsigned first_round = 0;
    if (first_round == 0) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        first_round = 2u * (unsigned)cus;
    }
    hipLaunchKernelGGL((ffn_fused_kernel<MODE, TRAIN, HEAD>), dim3((unsigned)blocks), dim3(kFfnThreads), 0, s, x, x_stride,
                       (const uint16_t *)rows_a, (const uint16_t *)rows_b, (const uint16_t *)wproj, norm_weight, eps,
                       (const uint16_t *)weights_packed, out, R, rows_a_stride, rows_b_stride, first_round, s_out, n_out,
                       next.norm_weight, next.eps, (const uint16_t *)next.packed, (uint16_t *)next.out, next.features);
    return (int)hipGetLastError();
}

static int ffn_common_checks(const float *x, int64_t x_row_stride, const float *norm_weight,
                             const void *weights_packed, const float *out, int64_t R, int D, int hidden)
{
    if (R < 0 || x_row_stride < D) return BNB_ERR_BAD_SHAPE;
    if (D != kFfnD || hidden != kFfnHidden) return BNB_ERR_UNSUPPORTED;
    if (R == 0) return 0;
    if (!x || !norm_weight || !weights_packed || !out) return BNB_ERR_NULL_POINTER;
    if (!aligned16(x) || !aligned16(out) || !aligned16(norm_weight) || !aligned16(weights_packed) ||
        (x_row_stride % 4) != 0)
        return BNB_ERR_MISALIGNED;
    return 0;
}

}  // namespace bnb

extern "C" int bnb_ffn_fused_fwd(const float *x, int64_t x_row_stride, const void *delta, int delta_dtype,
                                 const float *norm_weight, float eps, const void *weights_packed, float *out,
                                 int64_t R, int D, int hidden, void *stream)
{
    using namespace bnb;
    const int rc = ffn_common_checks(x, x_row_stride, norm_weight, weights_packed, out, R, D, hidden);
    if (rc != 0 || R == 0) return rc;
    if (delta && delta_dtype != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (delta && !aligned16(delta)) return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    if (delta)
        return launch_ffn<kDeltaRows>(x, x_row_stride, delta, nullptr, nullptr, norm_weight, eps, weights_packed, out,
                                      R, kFfnD, kFfnD, s);
    return launch_ffn<kDeltaNone>(x, x_row_stride, nullptr, nullptr, nullptr, norm_weight, eps, weights_packed, out, R,
                                  kFfnD, kFfnD, s);
}

extern "C" int bnb_ffn_fused_train_fwd(const float *x, int64_t x_row_stride, const void *delta, int delta_dtype,
                                       const float *norm_weight, float eps, const void *weights_packed, float *out,
                                       float *s_out, void *n_out, int64_t R, int D, int hidden, void *stream)
{
    using namespace bnb;
    const int rc = ffn_common_checks(x, x_row_stride, norm_weight, weights_packed, out, R, D, hidden);
    if (rc != 0 || R == 0) return rc;
    if (delta && delta_dtype != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (!n_out || (delta && !s_out)) return BNB_ERR_NULL_POINTER;
    if ((delta && !aligned16(delta)) || !aligned16(n_out) || (s_out && !aligned16(s_out))) return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    if (delta)
        return launch_ffn<kDeltaRows, true>(x, x_row_stride, delta, nullptr, nullptr, norm_weight, eps, weights_packed,
                                            out, R, kFfnD, kFfnD, s, s_out, (uint16_t *)n_out);
    return launch_ffn<kDeltaNone, true>(x, x_row_stride, nullptr, nullptr, nullptr, norm_weight, eps, weights_packed,
                                        out, R, kFfnD, kFfnD, s, nullptr, (uint16_t *)n_out);
}

extern "C" int bnb_ffn_fused_proj_next_fwd(const float *x, int64_t x_row_stride, const void *rows_a, int64_t rows_a_stride,
                                           const void *rows_b, int64_t rows_b_stride, const void *proj_packed,
                                           const float *norm_weight, float eps, const void *weights_packed, float *out,
                                           const float *next_norm_weight, float next_eps, const void *next_packed,
                                           void *next_out, int next_features, int64_t next_out_rows, int64_t R, int D,
                                           int hidden, void *stream)
{
    using namespace bnb;
    const int rc = ffn_common_checks(x, x_row_stride, norm_weight, weights_packed, out, R, D, hidden);
    if (rc != 0 || R == 0) return rc;
    if (!rows_a || !proj_packed || !next_norm_weight || !next_packed || !next_out) return BNB_ERR_NULL_POINTER;
    if (rows_a_stride == 0) rows_a_stride = kFfnD;
    if (rows_b_stride == 0) rows_b_stride = kFfnD;
    if (rows_a_stride < kFfnD || rows_b_stride < kFfnD) return BNB_ERR_BAD_SHAPE;
    // the head's stores are unconditional: room for every row of every work-group
    if (next_features < 128 || next_features % 64 != 0 || next_out_rows < (R + kFfnWaves * 32 - 1) / (kFfnWaves * 32) * (kFfnWaves * 32))
        return BNB_ERR_BAD_SHAPE;
    if (!aligned16(rows_a) || rows_a_stride % 8 != 0 || !aligned16(proj_packed) ||
        (rows_b && (!aligned16(rows_b) || rows_b_stride % 8 != 0)) || !aligned16(next_norm_weight) || !aligned16(next_packed) ||
        !aligned16(next_out))
        return BNB_ERR_MISALIGNED;
    NextHead next;
    next.norm_weight = next_norm_weight, next.eps = next_eps, next.packed = next_packed, next.out = next_out, next.features = next_features;
    hipStream_t s = (hipStream_t)stream;
    if (rows_b)
        return launch_ffn<kDeltaGate, false, true>(x, x_row_stride, rows_a, rows_b, proj_packed, norm_weight, eps, weights_packed,
                                                   out, R, rows_a_stride, rows_b_stride, s, nullptr, nullptr, next);
    return launch_ffn<kDeltaProj, false, true>(x, x_row_stride, rows_a, nullptr, proj_packed, norm_weight, eps, weights_packed, out,
                                               R, rows_a_stride, kFfnD, s, nullptr, nullptr, next);
}

extern "C" int bnb_ffn_fused_proj_train_fwd(const float *x, int64_t x_row_stride, const void *rows_a, int64_t rows_a_stride,
                                            const void *proj_packed, const float *norm_weight, float eps,
                                            const void *weights_packed, float *out, float *s_out, void *n_out, int64_t R,
                                            int D, int hidden, void *stream)
{
    using namespace bnb;
    const int rc = ffn_common_checks(x, x_row_stride, norm_weight, weights_packed, out, R, D, hidden);
    if (rc != 0 || R == 0) return rc;
    if (!rows_a || !proj_packed || !s_out || !n_out) return BNB_ERR_NULL_POINTER;
    if (rows_a_stride == 0) rows_a_stride = kFfnD;
    if (rows_a_stride < kFfnD) return BNB_ERR_BAD_SHAPE;
    if (!aligned16(rows_a) || rows_a_stride % 8 != 0 || !aligned16(proj_packed) || !aligned16(s_out) || !aligned16(n_out))
        return BNB_ERR_MISALIGNED;
    return launch_ffn<kDeltaProj, true>(x, x_row_stride, rows_a, nullptr, proj_packed, norm_weight, eps, weights_packed, out,
                                        R, rows_a_stride, kFfnD, (hipStream_t)stream, s_out, (uint16_t *)n_out);
}

extern "C" int bnb_ffn_fused_proj_fwd(const float *x, int64_t x_row_stride, const void *rows_a, int64_t rows_a_stride,
                                      const void *rows_b, int64_t rows_b_stride,
                                      const void *proj_packed, const float *norm_weight, float eps,
                                      const void *weights_packed, float *out, int64_t R, int D, int hidden,
                                      void *stream)
{
    using namespace bnb;
    const int rc = ffn_common_checks(x, x_row_stride, norm_weight, weights_packed, out, R, D, hidden);
    if (rc != 0 || R == 0) return rc;
    if (!rows_a || !proj_packed) return BNB_ERR_NULL_POINTER;
    if (rows_a_stride == 0) rows_a_stride = kFfnD;
    if (rows_b_stride == 0) rows_b_stride = kFfnD;
    if (rows_a_stride < kFfnD || rows_b_stride < kFfnD) return BNB_ERR_BAD_SHAPE;
    if (!aligned16(rows_a) || rows_a_stride % 8 != 0 || !aligned16(proj_packed) ||
        (rows_b && (!aligned16(rows_b) || rows_b_stride % 8 != 0)))
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    if (rows_b)
        return launch_ffn<kDeltaGate>(x, x_row_stride, rows_a, rows_b, proj_packed, norm_weight, eps, weights_packed,
                                      out, R, rows_a_stride, rows_b_stride, s);
    return launch_ffn<kDeltaProj>(x, x_row_stride, rows_a, nullptr, proj_packed, norm_weight, eps, weights_packed, out,
                                  R, rows_a_stride, kFfnD, s);
}
