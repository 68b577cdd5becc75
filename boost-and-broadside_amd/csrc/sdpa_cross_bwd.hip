// Backward of the bullet read over long key axes, for gfx950: bf16, head size 32, up to 160 queries
// per environment and ANY number of live keys (the bullet axis has 10 slots per ship: 1520 at 64v88).
//
// Reference: what autograd computes through models/yemong/attention.py:149-166 (the entity queries'
// cross-attention to the bullets in flight, additive finfo.min/2 bias on the others, an environment
// without a bullet gated off) during train/rl/ppo.py:1417-1425.  With S = Q K^T / sqrt(dh),
// P = softmax over the live keys, O = P V:
//   dV = P^T dO,  dP = dO V^T,  dS = P * (dP - rowsum(dO * O)),  dQ = dS K / sqrt(dh),  dK = dS^T Q / sqrt(dh).
//
// The live keys of environment b are named by `ranges` (b's keys are entries ranges[b] .. ranges[b+1]-1
// of one list for all environments) and, optionally, `row_index` (entry e is row row_index[e] of the
// key/value buffer; without it entry e IS row e: the rows were compacted beforehand).  Dead slots are
// never touched, so cost follows the bullets in flight.
//
// Two kernels, one work-group per (environment, head), one wave per block of 32 queries:
//   * cross_bwd_dq_kernel: the key axis streams through LDS in tiles of 32 * waves keys (the next tile
//     is on its way in registers while the current one is multiplied).  Pass A forms S^T = K Q^T per
//     key block (rows = keys, lane = query) only for the running maximum and sum, which gives
//     L = log2-sum-exp per query; pass B forms it again with P^T = exp2(S^T c - L), dP^T = V dO^T,
//     dS^T = P^T (dP^T - delta) / sqrt(dh) and dQ^T += K^T dS^T, dS^T going from the accumulator
//     registers straight into the B operand (K^T comes from a transposed copy of the tile).  L and
//     delta = rowsum(dO * O) are written to `stats` for the second kernel.
//   * cross_bwd_dkv_kernel: Q, dO and their transposed copies sit in LDS for the life of the work-group;
//     wave w walks key blocks w, w + waves, ... on its own (no barrier in the loop): its 32 keys' K
//     and V rows are B operands straight from global memory, S = Q K^T and dP = dO V^T per query block
//     (rows = queries, lane = key), P and dS from the per-query L and delta, dK^T += Q^T dS,
//     dV^T += dO^T P.
// P and dS are rounded to bf16 for the second product of each pair, as in the forward kernel.  Every sum
// runs in a fixed order.

#include "common.h"

#include <math.h>

namespace bnb {

constexpr int kCbDh = 32;
constexpr int kCbPitch = kCbDh + 8;  // halfs per token row in LDS (80 bytes: 16-byte aligned, bank-spread)

struct CbStaged {
    u32x4 a[2], b[2];
};

// An operand of the first product of a pair: row tok, channels 8*half.. and 16 + 8*half..
__device__ __forceinline__ void cb_row_operand(const uint16_t *rows, int tok, int half, bf16x8 &lo, bf16x8 &hi)
{
    const uint16_t *p = rows + tok * kCbPitch + half * 8;
    lo = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(p));
    hi = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(p + 16));
}

// The A operand of the second product: channel m, tokens in the order the accumulator rows 8t.. hold them.
template <int TP>
__device__ __forceinline__ bf16x8 cb_tr_operand(const uint16_t *tr, int m, int half, int blk, int t)
{
    const uint16_t *p = tr + m * TP + blk * 32 + 16 * t + 4 * half;
    const u32x2 lo = *reinterpret_cast<const u32x2 *>(p);
    const u32x2 hi = *reinterpret_cast<const u32x2 *>(p + 8);
    return __builtin_bit_cast(bf16x8, u32x4{lo.x, lo.y, hi.x, hi.y});
}

__device__ __forceinline__ bf16x8 cb_pack8(const float (&x)[16], int t)
{
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (__bf16)x[8 * t + e];
    return r;
}

// A (32 channels x 32 tokens) accumulator to one row of a gradient tensor: lane = token, registers = channels 8i + 4*half + j.
__device__ __forceinline__ void cb_store_row(const f32x16 &acc, uint16_t *dst)
{
#pragma unroll
    for (int i = 0; i < 4; ++i)
        *reinterpret_cast<u32x2 *>(dst + 8 * i) = u32x2{pack_bf16x2(acc[4 * i], acc[4 * i + 1]), pack_bf16x2(acc[4 * i + 2], acc[4 * i + 3])};
}

// HAVE_LSE: the forward pass handed over the log2-sum-exp of every query (`lse_in`, (B, H, NQ) floats); pass A,
// which otherwise recomputes it from the keys (all the scores twice), is skipped.
// Registers: five waves per work-group only come three to a CU at 96 registers or fewer (a CU wants room for two more
// waves on every SIMD before it takes such a work-group); the handful of values that spills at that bound costs less
// than the third work-group brings (kernel trace at 4096 environments x 160 queries x 380 keys: 701 -> 637..658 us).
template <int NB, bool HAVE_LSE>
__global__ __launch_bounds__(kWave *NB, NB == 5 ? 5 : 3) void cross_bwd_dq_kernel(
    const uint16_t *__restrict__ q, int64_t q_row_stride, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,
    int64_t kv_row_stride, const int32_t *__restrict__ ranges, const int32_t *__restrict__ row_index, int64_t capacity,
    const uint16_t *__restrict__ out, const uint16_t *__restrict__ dout, uint16_t *__restrict__ dq_out, float *__restrict__ stats,
    const float *__restrict__ lse_in, int B, int NQ, int H, float scale)
{
    constexpr int CAP = NB * 32;  // keys per tile
    constexpr int TP = CAP + 4;   // halfs per row of the transposed copy
    constexpr int NT = kWave * NB;
    __shared__ __align__(16) uint16_t s_rows[2][CAP * kCbPitch];  // K and V of the tile, token-major
    __shared__ __align__(16) uint16_t s_kt[kCbDh * TP];           // K^T of the tile

    const int chunk = gridDim.x >> 3;
    const int logical = (blockIdx.x & 7) * chunk + (blockIdx.x >> 3);  // the heads of an environment on one XCD
    if (logical >= B * H) return;
    const int env = logical / H, head = logical - env * H;
    const int D = H * kCbDh;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31, half = lane >> 5;
    const float c = scale * 1.4426950408889634f;
    const u32x4 zero4 = {0u, 0u, 0u, 0u};

    const int64_t first = ranges[env];
    int64_t cnt64 = (int64_t)ranges[env + 1] - first;
    if (cnt64 > capacity - first) cnt64 = capacity - first;
    const int cnt = cnt64 < 0 ? 0 : (int)cnt64;
    const int nqb = (NQ + 31) >> 5;  // <= NB
    const int own = wave * 32 + m;   // this lane's query
    const int64_t q_base = (int64_t)env * NQ;
    uint16_t *dq_row = dq_out + (q_base + own) * D + head * kCbDh + 4 * half;
    float *stat_row = stats + (((int64_t)env * H + head) * NQ + own) * 2;
    if (cnt == 0) {
        // the forward gated this environment off: nothing depends on its queries
        if (own < NQ) {
            const f32x16 z16 = {0.0f};
            cb_store_row(z16, dq_row);
            if (half == 0) stat_row[0] = 0.0f, stat_row[1] = 0.0f;
        }
        return;
    }
    const int ntiles = (cnt + CAP - 1) / CAP;

    // ---- this lane's query row, its output and output gradient ----
    const int64_t q_row = q_base + (own < NQ ? own : NQ - 1);
    const int64_t own_q = q_row * q_row_stride + head * kCbDh + half * 8, own_o = q_row * D + head * kCbDh + half * 8;
    u32x4 w0 = *reinterpret_cast<const u32x4 *>(q + own_q), w1 = *reinterpret_cast<const u32x4 *>(q + own_q + 16);
    u32x4 g0 = *reinterpret_cast<const u32x4 *>(dout + own_o), g1 = *reinterpret_cast<const u32x4 *>(dout + own_o + 16);
    const Row8 o0 = load8(out + own_o), o1 = load8(out + own_o + 16);

    // ---- key tiles: global -> registers -> LDS ----
    auto stage_load = [&](int t, bool need_v) -> CbStaged {
        CbStaged r;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int item = tid + it * NT;
            const int tok = item >> 2, c8 = (item & 3) * 8 + head * kCbDh;
            const int pos = t * CAP + tok;
            const bool valid = pos < cnt;
            const int64_t entry = first + (valid ? pos : cnt - 1);  // a padding position reads the last key and discards it
            const int64_t row = row_index != nullptr ? (int64_t)row_index[entry] : entry;
            const u32x4 aw = *reinterpret_cast<const u32x4 *>(k + row * kv_row_stride + c8);
            r.a[it] = valid ? aw : zero4;
            r.b[it] = zero4;
            if (need_v) {
                const u32x4 bw = *reinterpret_cast<const u32x4 *>(v + row * kv_row_stride + c8);
                r.b[it] = valid ? bw : zero4;
            }
        }
        return r;
    };
    auto stage_store = [&](const CbStaged &r, bool all) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int item = tid + it * NT;
            const int tok = item >> 2, c8 = (item & 3) * 8;
            *reinterpret_cast<u32x4 *>(s_rows[0] + tok * kCbPitch + c8) = r.a[it];
            if (all) {
                *reinterpret_cast<u32x4 *>(s_rows[1] + tok * kCbPitch + c8) = r.b[it];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const uint32_t wa = r.a[it][e >> 1];
                    s_kt[(c8 + e) * TP + tok] = (uint16_t)((e & 1) ? wa >> 16 : wa & 0xffffu);
                }
            }
        }
    };

    float delta;
    {
        float d = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t p0 = g0[e >> 1], p1 = g1[e >> 1];
            const float a0 = __uint_as_float((e & 1) ? p0 & 0xffff0000u : p0 << 16), a1 = __uint_as_float((e & 1) ? p1 & 0xffff0000u : p1 << 16);
            d = fmaf(a0, o0.v[e], fmaf(a1, o1.v[e], d));
        }
        delta = d + __shfl_xor(d, 32);
    }
    if (own >= NQ) w0 = w1 = g0 = g1 = zero4, delta = 0.0f;  // padding queries: nothing flows through them
    const bf16x8 qs0 = __builtin_bit_cast(bf16x8, w0), qs1 = __builtin_bit_cast(bf16x8, w1);
    const bf16x8 gb0 = __builtin_bit_cast(bf16x8, g0), gb1 = __builtin_bit_cast(bf16x8, g1);

    // S^T of key block kb of tile t; positions past the last key start at -inf (P = 0 exactly)
    auto scores_t = [&](int t, int kb) -> f32x16 {
        f32x16 z = {0.0f};
        const int block_first = t * CAP + kb * 32;
        if (block_first + 32 > cnt) {
#pragma unroll
            for (int vv = 0; vv < 16; ++vv)
                if (block_first + 8 * (vv >> 2) + 4 * half + (vv & 3) >= cnt) z[vv] = -INFINITY;
        }
        bf16x8 k0, k1;
        cb_row_operand(s_rows[0], kb * 32 + m, half, k0, k1);
        z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k0, qs0, z, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(k1, qs1, z, 0, 0, 0);
    };
    auto blocks_of = [&](int t) {
        const int left = cnt - t * CAP;
        return left >= CAP ? NB : (left + 31) >> 5;
    };

    // ---- pass A: log2-sum-exp of every query over all keys ----
    const bool single = !HAVE_LSE && ntiles == 1;  // one tile: staged once, with V and K^T, for both passes
    float mx = -INFINITY, sum = 0.0f;
    CbStaged cur;
    if (!HAVE_LSE) cur = stage_load(0, single);
    for (int t = 0; !HAVE_LSE && t < ntiles; ++t) {
        __syncthreads();  // the previous tile has been read by every wave
        stage_store(cur, single);
        __syncthreads();
        if (t + 1 < ntiles) cur = stage_load(t + 1, false);
        if (wave < nqb) {
            const int nb = blocks_of(t);
            float tmx = -INFINITY;
            for (int kb = 0; kb < nb; ++kb) {
                const f32x16 z = scores_t(t, kb);
#pragma unroll
                for (int vv = 0; vv < 16; ++vv) tmx = fmaxf(tmx, z[vv]);
            }
            tmx = fmaxf(tmx, __shfl_xor(tmx, 32));
            const float mnew = fmaxf(mx, tmx);  // finite: every tile holds at least one key
            sum *= __builtin_amdgcn_exp2f((mx - mnew) * c);
            mx = mnew;
            const float mc = mx * c;
            for (int kb = 0; kb < nb; ++kb) {
                const f32x16 z = scores_t(t, kb);
#pragma unroll
                for (int vv = 0; vv < 16; ++vv) sum += __builtin_amdgcn_exp2f(fmaf(z[vv], c, -mc));
            }
        }
    }
    sum += __shfl_xor(sum, 32);
    // log2 of the sum of exp2(z c)
    const float lse = HAVE_LSE ? lse_in[((int64_t)env * H + head) * NQ + (own < NQ ? own : NQ - 1)] : mx * c + __builtin_amdgcn_logf(sum);
    if (own < NQ && half == 0) stat_row[0] = lse, stat_row[1] = delta;

    // ---- pass B: dQ ----
    f32x16 dq = {0.0f};
    if (!single) cur = stage_load(0, true);
    for (int t = 0; t < ntiles; ++t) {
        if (!single) {
            __syncthreads();
            stage_store(cur, true);
            __syncthreads();
            if (t + 1 < ntiles) cur = stage_load(t + 1, true);
        }
        if (wave < nqb) {
            const int nb = blocks_of(t);
            for (int kb = 0; kb < nb; ++kb) {
                const f32x16 z = scores_t(t, kb);
                bf16x8 v0, v1;
                cb_row_operand(s_rows[1], kb * 32 + m, half, v0, v1);
                f32x16 dp = {0.0f};
                dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v0, gb0, dp, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v1, gb1, dp, 0, 0, 0);
                float ds[16];
#pragma unroll
                for (int vv = 0; vv < 16; ++vv) ds[vv] = __builtin_amdgcn_exp2f(fmaf(z[vv], c, -lse)) * (dp[vv] - delta);  // * scale: once, on dq
#pragma unroll
                for (int t2 = 0; t2 < 2; ++t2)
                    dq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cb_tr_operand<TP>(s_kt, m, half, kb, t2), cb_pack8(ds, t2), dq, 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int vv = 0; vv < 16; ++vv) dq[vv] *= scale;
    if (own < NQ) cb_store_row(dq, dq_row);
}

// Waves: the key blocks are dealt to the waves in turn, so their number is free; never more than four.  A CU places
// a work-group only while each of its four SIMDs has room for ceil(waves / 4) more waves: at this kernel's
// register count a work-group of five waves came out as the only one on its CU, four-wave ones are three.
template <int NB>
__global__ __launch_bounds__(kWave *(NB < 4 ? NB : 4), 3) void cross_bwd_dkv_kernel(
    const uint16_t *__restrict__ q, int64_t q_row_stride, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,
    int64_t kv_row_stride, const int32_t *__restrict__ ranges, const int32_t *__restrict__ row_index, int64_t capacity,
    const uint16_t *__restrict__ dout, const float *__restrict__ stats, uint16_t *__restrict__ dk_out, uint16_t *__restrict__ dv_out,
    int64_t dkv_row_stride, int B, int NQ, int H, float scale)
{
    constexpr int CAP = NB * 32;  // queries staged
    constexpr int TP = CAP + 4;
    constexpr int NW = NB < 4 ? NB : 4;
    constexpr int NT = kWave * NW;
    __shared__ __align__(16) uint16_t s_rows[2][CAP * kCbPitch];  // Q and dO, token-major
    __shared__ __align__(16) uint16_t s_tr[2][kCbDh * TP];        // Q^T and dO^T
    __shared__ __align__(16) float s_lse[CAP], s_delta[CAP];

    const int chunk = gridDim.x >> 3;
    const int logical = (blockIdx.x & 7) * chunk + (blockIdx.x >> 3);
    if (logical >= B * H) return;
    const int env = logical / H, head = logical - env * H;
    const int D = H * kCbDh;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31, half = lane >> 5;
    const float c = scale * 1.4426950408889634f;
    const u32x4 zero4 = {0u, 0u, 0u, 0u};

    const int64_t first = ranges[env];
    int64_t cnt64 = (int64_t)ranges[env + 1] - first;
    if (cnt64 > capacity - first) cnt64 = capacity - first;
    const int cnt = cnt64 < 0 ? 0 : (int)cnt64;
    if (cnt == 0) return;
    const int nqb = (NQ + 31) >> 5, nkb = (cnt + 31) >> 5;
    const int64_t q_base = (int64_t)env * NQ;

    // this wave's first key block, requested before the queries are staged
    struct KeyRows {
        u32x4 k0, k1, v0, v1;
        int64_t row;
        bool valid;
    };
    auto load_keys = [&](int kb) -> KeyRows {
        KeyRows r;
        const int pos = kb * 32 + m;
        r.valid = pos < cnt;
        const int64_t entry = first + (r.valid ? pos : cnt - 1);
        r.row = row_index != nullptr ? (int64_t)row_index[entry] : entry;
        const int64_t off = r.row * kv_row_stride + head * kCbDh + half * 8;
        r.k0 = *reinterpret_cast<const u32x4 *>(k + off), r.k1 = *reinterpret_cast<const u32x4 *>(k + off + 16);
        r.v0 = *reinterpret_cast<const u32x4 *>(v + off), r.v1 = *reinterpret_cast<const u32x4 *>(v + off + 16);
        return r;
    };
    KeyRows nxt;
    nxt.k0 = nxt.k1 = nxt.v0 = nxt.v1 = zero4, nxt.row = 0, nxt.valid = false;
    if (wave < nkb) nxt = load_keys(wave);

    // ---- Q, dO of the environment: token-major and channel-major copies; rows past NQ are zero ----
#pragma unroll
    for (int it = 0; it < (4 * CAP + NT - 1) / NT; ++it) {
        const int item = tid + it * NT;
        if (item >= 4 * CAP) break;
        const int tok = item >> 2, c8 = (item & 3) * 8;
        const bool valid = tok < NQ;
        const int64_t row = q_base + (valid ? tok : NQ - 1);
        u32x4 a = *reinterpret_cast<const u32x4 *>(q + row * q_row_stride + head * kCbDh + c8);
        u32x4 b = *reinterpret_cast<const u32x4 *>(dout + row * D + head * kCbDh + c8);
        if (!valid) a = b = zero4;
        *reinterpret_cast<u32x4 *>(s_rows[0] + tok * kCbPitch + c8) = a;
        *reinterpret_cast<u32x4 *>(s_rows[1] + tok * kCbPitch + c8) = b;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t wa = a[e >> 1], wb = b[e >> 1];
            s_tr[0][(c8 + e) * TP + tok] = (uint16_t)((e & 1) ? wa >> 16 : wa & 0xffffu);
            s_tr[1][(c8 + e) * TP + tok] = (uint16_t)((e & 1) ? wb >> 16 : wb & 0xffffu);
        }
    }
    if (tid < CAP) {  // CAP <= NT
        const float *st = stats + (((int64_t)env * H + head) * NQ + (tid < NQ ? tid : 0)) * 2;
        s_lse[tid] = tid < NQ ? st[0] : 0.0f;
        s_delta[tid] = tid < NQ ? st[1] : 0.0f;
    }
    __syncthreads();

    // ---- this wave's key blocks ----
    for (int kb = wave; kb < nkb; kb += NW) {
        const KeyRows cur = nxt;
        if (kb + NW < nkb) nxt = load_keys(kb + NW);
        const bf16x8 ks0 = __builtin_bit_cast(bf16x8, cur.valid ? cur.k0 : zero4), ks1 = __builtin_bit_cast(bf16x8, cur.valid ? cur.k1 : zero4);
        const bf16x8 vb0 = __builtin_bit_cast(bf16x8, cur.valid ? cur.v0 : zero4), vb1 = __builtin_bit_cast(bf16x8, cur.valid ? cur.v1 : zero4);
        const float col_bias = cur.valid ? 0.0f : -INFINITY;
        f32x16 dk = {0.0f}, dv = {0.0f};
        for (int qb = 0; qb < nqb; ++qb) {
            f32x16 z;
#pragma unroll
            for (int vv = 0; vv < 16; ++vv) z[vv] = col_bias;
            bf16x8 a0, a1;
            cb_row_operand(s_rows[0], qb * 32 + m, half, a0, a1);
            z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, ks0, z, 0, 0, 0);
            z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, ks1, z, 0, 0, 0);
            cb_row_operand(s_rows[1], qb * 32 + m, half, a0, a1);
            f32x16 dp = {0.0f};
            dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, vb0, dp, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, vb1, dp, 0, 0, 0);
            float p[16], ds[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f32x4 l4 = *reinterpret_cast<const f32x4 *>(s_lse + qb * 32 + 8 * i + 4 * half);
                const f32x4 d4 = *reinterpret_cast<const f32x4 *>(s_delta + qb * 32 + 8 * i + 4 * half);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int vv = 4 * i + j;
                    p[vv] = __builtin_amdgcn_exp2f(fmaf(z[vv], c, -l4[j]));
                    ds[vv] = p[vv] * (dp[vv] - d4[j]);  // * scale: once per key block, on dk
                }
            }
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                dk = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cb_tr_operand<TP>(s_tr[0], m, half, qb, t), cb_pack8(ds, t), dk, 0, 0, 0);
                dv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cb_tr_operand<TP>(s_tr[1], m, half, qb, t), cb_pack8(p, t), dv, 0, 0, 0);
            }
        }
        if (cur.valid) {
            const int64_t off = cur.row * dkv_row_stride + head * kCbDh + 4 * half;
#pragma unroll
            for (int vv = 0; vv < 16; ++vv) dk[vv] *= scale;
            cb_store_row(dk, dk_out + off);
            cb_store_row(dv, dv_out + off);
        }
    }
}

template <int NB>
static int launch_cross_stream_bwd(const void *q, int64_t q_row_stride, const void *kv, int64_t kv_row_stride, const int32_t *ranges,
                                   const int32_t *row_index, int64_t capacity, const void *out, const void *dout, void *dq, void *dkv,
                                   float *stats, const float *lse, int64_t B, int NQ, int H, hipStream_t stream)
{
    const int64_t groups = (B * H + 7) / 8 * 8;  // a multiple of 8: the XCD mapping deals whole rounds
    if (groups > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    const int D = H * kCbDh;
    const uint16_t *kp = (const uint16_t *)kv;
    uint16_t *g = (uint16_t *)dkv;
    const float scale = 1.0f / sqrtf((float)kCbDh);
    if (lse != nullptr)
        hipLaunchKernelGGL((cross_bwd_dq_kernel<NB, true>), dim3((unsigned)groups), dim3(kWave * NB), 0, stream, (const uint16_t *)q,
                           q_row_stride, kp, kp + D, kv_row_stride, ranges, row_index, capacity, (const uint16_t *)out,
                           (const uint16_t *)dout, (uint16_t *)dq, stats, lse, (int)B, NQ, H, scale);
    else
        hipLaunchKernelGGL((cross_bwd_dq_kernel<NB, false>), dim3((unsigned)groups), dim3(kWave * NB), 0, stream, (const uint16_t *)q,
                           q_row_stride, kp, kp + D, kv_row_stride, ranges, row_index, capacity, (const uint16_t *)out,
                           (const uint16_t *)dout, (uint16_t *)dq, stats, lse, (int)B, NQ, H, scale);
    int rc = (int)hipGetLastError();
    if (rc != 0) return rc;
    hipLaunchKernelGGL((cross_bwd_dkv_kernel<NB>), dim3((unsigned)groups), dim3(kWave * (NB < 4 ? NB : 4)), 0, stream, (const uint16_t *)q, q_row_stride, kp,
                       kp + D, kv_row_stride, ranges, row_index, capacity, (const uint16_t *)dout, (const float *)stats, g, g + D,
                       2 * (int64_t)D, (int)B, NQ, H, scale);
    return (int)hipGetLastError();
}

}  // namespace bnb

namespace bnb {
static int cross_stream_bwd(const void *q, int64_t q_row_stride, int NQ, const void *kv, int64_t kv_row_stride,
                            const int32_t *ranges, const int32_t *row_index, int64_t capacity, const void *out, const void *dout,
                            void *dq, void *dkv, float *stats, const float *lse, int64_t B, int H, int dh, int dtype, void *stream)
{
    if (B < 0 || NQ < 1 || H < 1 || dh < 1 || capacity < 1) return BNB_ERR_BAD_SHAPE;
    if (dtype != BNB_BF16 || dh != kCbDh || NQ > 160) return BNB_ERR_UNSUPPORTED;
    const int D = H * dh;
    if (q_row_stride < D || kv_row_stride < 2 * (int64_t)D) return BNB_ERR_BAD_SHAPE;
    if (B == 0) return 0;
    if (!q || !kv || !ranges || !out || !dout || !dq || !dkv || !stats) return BNB_ERR_NULL_POINTER;
    if (!aligned16(q) || !aligned16(kv) || !aligned16(out) || !aligned16(dout) || !aligned16(dq) || !aligned16(dkv) ||
        (q_row_stride % 8) != 0 || (kv_row_stride % 8) != 0)
        return BNB_ERR_MISALIGNED;
    if (B > 0x7fffffffLL / H) return BNB_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
#define BNB_CSB(NBV) return launch_cross_stream_bwd<NBV>(q, q_row_stride, kv, kv_row_stride, ranges, row_index, capacity, out, dout, dq, dkv, stats, lse, B, NQ, H, s)
    switch ((NQ + 31) / 32) {
        case 1: BNB_CSB(1);
        case 2: BNB_CSB(2);
        case 3: BNB_CSB(3);
        case 4: BNB_CSB(4);
        case 5: BNB_CSB(5);
        default: return BNB_ERR_UNSUPPORTED;
    }
#undef BNB_CSB
}
}  // namespace bnb

extern "C" int bnb_sdpa_cross_stream_bwd(const void *q, int64_t q_row_stride, int NQ, const void *kv, int64_t kv_row_stride,
                                         const int32_t *ranges, const int32_t *row_index, int64_t capacity, const void *out,
                                         const void *dout, void *dq, void *dkv, float *stats, int64_t B, int H, int dh, int dtype,
                                         void *stream)
{
    return bnb::cross_stream_bwd(q, q_row_stride, NQ, kv, kv_row_stride, ranges, row_index, capacity, out, dout, dq, dkv, stats,
                                 nullptr, B, H, dh, dtype, stream);
}

extern "C" int bnb_sdpa_cross_stream_bwd_lse(const void *q, int64_t q_row_stride, int NQ, const void *kv, int64_t kv_row_stride,
                                             const int32_t *ranges, const int32_t *row_index, int64_t capacity, const void *out,
                                             const void *dout, const float *lse, void *dq, void *dkv, float *stats, int64_t B,
                                             int H, int dh, int dtype, void *stream)
{
    if (lse == nullptr && B > 0) return BNB_ERR_NULL_POINTER;
    if (reinterpret_cast<uintptr_t>(lse) & 3u) return BNB_ERR_MISALIGNED;
    return bnb::cross_stream_bwd(q, q_row_stride, NQ, kv, kv_row_stride, ranges, row_index, capacity, out, dout, dq, dkv, stats,
                                 lse, B, H, dh, dtype, stream);
}
