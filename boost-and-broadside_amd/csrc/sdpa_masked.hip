// Masked multi-head attention over each environment's entity tokens, for gfx950.
//
// out[b,i,h,:] = sum_j softmax_j(q[b,i,h].k[b,j,h] / sqrt(dh) + bias[b,j]) v[b,j,h,:]
// (reference: models/yemong/attention.py:101-112,136-147,168).  The additive bias of the
// reference (0 for a live key, finfo.min/2 for a dead one) has two exact consequences that
// the kernels implement directly instead of adding a huge constant:
//   * an environment with at least one live key gives every dead key weight exactly 0, so
//     dead keys are dropped from the key list before any arithmetic (their K/V rows are
//     never even read);
//   * an environment with no live key has every score rounded to the same constant, i.e.
//     an exactly uniform softmax over ALL keys: the output is the mean of V.
// Queries are never masked.
//
// Two kernels:
//   sdpa_valu_kernel   any dtype, dh in {8,16,32,64}, any NM that fits LDS; one lane per
//                      (environment, head, query) row, K/V of a group of environments
//                      staged in LDS as fp32, chunked online softmax.  This is the fp32 path
//                      and the path for head sizes other than 32.
//   sdpa_mfma_kernel   bf16, dh = 32, NM <= 160; one work-group per (environment,
//                      head), one wavefront per 32 queries; S^T = K Q^T and O^T = V^T P^T on
//                      v_mfma_f32_32x32x16_bf16 so that the softmax reductions over keys
//                      stay inside a lane.

#include <type_traits>

#include "common.h"

namespace bnb {

constexpr float kLog2eA = 1.4426950408889634f;
constexpr int kValuThreads = 256;
constexpr int kValuEnvPad = 16;   // floats between environments in LDS (bank spreading)
constexpr int kValuHeadPad = 4;   // floats after every head row in LDS (bank spreading)

// ------------------------------------------------------------------------------------
// VALU kernel
// ------------------------------------------------------------------------------------

// LDS: K then V, each [G][NM][nh][DH + pad] fp32 (+ env pad), then alive bytes [G][NM],
// then one "has a live key" flag per environment.
template <typename T, int DH>
__global__ __launch_bounds__(kValuThreads) void sdpa_valu_kernel(
    const T *__restrict__ qkv, int64_t row_stride, const uint8_t *__restrict__ alive, T *__restrict__ out,
    int B, int NM, int H, int G, int nh, float scale_log2e)
{
    extern __shared__ __align__(16) unsigned char s_raw[];
    constexpr int HP = DH + kValuHeadPad;
    const int D = H * DH;
    const int env_pitch = NM * nh * HP + kValuEnvPad;  // floats
    float *s_k = reinterpret_cast<float *>(s_raw);
    float *s_v = s_k + (size_t)G * env_pitch;
    uint8_t *s_alive = reinterpret_cast<uint8_t *>(s_v + (size_t)G * env_pitch);
    int *s_any = reinterpret_cast<int *>(s_alive + (((size_t)G * NM + 15) & ~(size_t)15));

    const int env0 = blockIdx.x * G;
    const int h0 = blockIdx.y * nh;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;  // a multiple of 64, at most kValuThreads

    if (tid < G) s_any[tid] = (alive == nullptr) ? 1 : 0;
    __syncthreads();

    // alive bytes (benign race on s_any: every writer stores 1)
    for (int idx = tid; idx < G * NM; idx += nthreads) {
        const int g = idx / NM;
        const int env = env0 + g;
        uint8_t a = 1;
        if (alive != nullptr) a = (env < B) ? alive[(int64_t)env * NM + (idx - g * NM)] : 1;
        s_alive[idx] = a;
        if (a) s_any[g] = 1;
    }

    // K and V tiles, 8 elements per lane per trip
    constexpr int V8 = DH / 8;
    const int per_mat = G * NM * nh * V8;
    for (int idx = tid; idx < 2 * per_mat; idx += nthreads) {
        const int mat = idx / per_mat;
        int rem = idx - mat * per_mat;
        const int c8 = rem % V8;
        rem /= V8;
        const int hh = rem % nh;
        rem /= nh;
        const int j = rem % NM;
        const int g = rem / NM;
        const int env = env0 + g;
        Row8 r;
        if (env < B) {
            r = load8(qkv + ((int64_t)env * NM + j) * row_stride + (1 + mat) * D + (h0 + hh) * DH + c8 * 8);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) r.v[e] = 0.0f;
        }
        float *dst = (mat ? s_v : s_k) + (size_t)g * env_pitch + (j * nh + hh) * HP + c8 * 8;
        *reinterpret_cast<f32x4 *>(dst) = f32x4{r.v[0], r.v[1], r.v[2], r.v[3]};
        *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{r.v[4], r.v[5], r.v[6], r.v[7]};
    }
    __syncthreads();

    const int rows = G * nh * NM;
    for (int row = tid; row < rows; row += nthreads) {
        const int g = row / (nh * NM);
        const int rem = row - g * (nh * NM);
        const int hh = rem / NM;
        const int i = rem - hh * NM;
        const int env = env0 + g;
        if (env >= B) continue;

        float q[DH];
        const T *qp = qkv + ((int64_t)env * NM + i) * row_stride + (h0 + hh) * DH;
#pragma unroll
        for (int c8 = 0; c8 < V8; ++c8) {
            const Row8 r = load8(qp + c8 * 8);
#pragma unroll
            for (int e = 0; e < 8; ++e) q[c8 * 8 + e] = r.v[e] * scale_log2e;
        }

        const bool any = s_any[g] != 0;
        const uint8_t *al = s_alive + g * NM;
        const float *kbase = s_k + (size_t)g * env_pitch + hh * HP;
        const float *vbase = s_v + (size_t)g * env_pitch + hh * HP;

        float m = -INFINITY, l = 0.0f;
        float o[DH];
#pragma unroll
        for (int d = 0; d < DH; ++d) o[d] = 0.0f;

        for (int j0 = 0; j0 < NM; j0 += 4) {
            float s[4];
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const int j = j0 + jj;
                s[jj] = -INFINITY;
                if (j < NM) {
                    const float *kr = kbase + (size_t)j * nh * HP;
                    float dot = 0.0f;
#pragma unroll
                    for (int d4 = 0; d4 < DH / 4; ++d4) {
                        const f32x4 kv = *reinterpret_cast<const f32x4 *>(kr + d4 * 4);
                        dot = fmaf(q[d4 * 4 + 0], kv.x, dot);
                        dot = fmaf(q[d4 * 4 + 1], kv.y, dot);
                        dot = fmaf(q[d4 * 4 + 2], kv.z, dot);
                        dot = fmaf(q[d4 * 4 + 3], kv.w, dot);
                    }
                    s[jj] = any ? (al[j] ? dot : -INFINITY) : 0.0f;
                }
            }
            const float m_new = fmaxf(fmaxf(m, fmaxf(s[0], s[1])), fmaxf(s[2], s[3]));
            if (m_new == -INFINITY) continue;  // nothing live seen yet
            const float alpha = __builtin_amdgcn_exp2f(m - m_new);  // 0 when m = -inf
            l *= alpha;
#pragma unroll
            for (int d = 0; d < DH; ++d) o[d] *= alpha;
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const int j = j0 + jj;
                if (j < NM) {
                    const float p = __builtin_amdgcn_exp2f(s[jj] - m_new);
                    l += p;
                    const float *vr = vbase + (size_t)j * nh * HP;
#pragma unroll
                    for (int d4 = 0; d4 < DH / 4; ++d4) {
                        const f32x4 vv = *reinterpret_cast<const f32x4 *>(vr + d4 * 4);
                        o[d4 * 4 + 0] = fmaf(p, vv.x, o[d4 * 4 + 0]);
                        o[d4 * 4 + 1] = fmaf(p, vv.y, o[d4 * 4 + 1]);
                        o[d4 * 4 + 2] = fmaf(p, vv.z, o[d4 * 4 + 2]);
                        o[d4 * 4 + 3] = fmaf(p, vv.w, o[d4 * 4 + 3]);
                    }
                }
            }
            m = m_new;
        }

        const float inv_l = 1.0f / l;
        T *op = out + ((int64_t)env * NM + i) * D + (h0 + hh) * DH;
#pragma unroll
        for (int c8 = 0; c8 < V8; ++c8) {
            Row8 r;
#pragma unroll
            for (int e = 0; e < 8; ++e) r.v[e] = o[c8 * 8 + e] * inv_l;
            store8(op + c8 * 8, r);
        }
    }
}

// ------------------------------------------------------------------------------------
// MFMA kernel (bf16, dh = 32)
// ------------------------------------------------------------------------------------
//
// v_mfma_f32_32x32x16_bf16, wave64: lane = 32*half + m.
//   A (32 x 16): lane supplies row m,    contraction slots 8*half .. 8*half+7
//   B (16 x 32): lane supplies column m, contraction slots 8*half .. 8*half+7
//   D (32 x 32): lane holds column m, rows 8*(v/4) + 4*half + (v%4) for v = 0..15
// S^T block (keys x queries) = K_blk (A) * Q_blk^T (B): a lane ends up with 16 scores of
// ONE query per key block, so max and sum over keys are in-lane plus one exchange between
// the two halves.  O^T (dh x queries) = V^T (A) * P^T (B): the probabilities a lane holds
// are exactly the B operand it must supply, provided the A operand (V^T from LDS) lists the
// keys in the same order: slot e of MFMA (kb,t) is key 32*kb + 16*t + 8*(e/4) + 4*half + e%4.

constexpr int kDh = 32;
constexpr int kKeyPitch = kDh + 8;  // halfs per K row in LDS: 80 bytes, 16-byte aligned, bank-spread

// The A operand of O^T = V^T P^T (per lane eight keys of ONE channel) out of ROW-MAJOR V rows in LDS (32 channels = 64
// bytes per key, keys dense): ds_read_b64_tr_b16 hands lane i of a group of 16 lanes element i%4 of the 8-byte pieces
// that lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12 of the group address.  As SOURCE lane r = lane%16 of group g = lane/16 a
// lane therefore points at key 4 (g/2) + r/4 of the 16 keys of one product and at the four channels of output-row
// block rb = 4 (g%2) + r%4; MFMA row 8i + 4 half + j is channel 16 (i/2) + 8 half + 4 (i%2) + j (the output stage's
// order), i.e. row block rb is channel block 4 (rb/4) + 2 (rb%2) + (rb/2)%2.  No transposed copy of V is written.
__device__ __forceinline__ int v_tr_offset(int lane)
{
    const int grp = lane >> 4, r = lane & 15;
    const int rb = 4 * (grp & 1) + (r & 3);
    const int cb = 4 * (rb >> 2) + 2 * (rb & 1) + ((rb >> 1) & 1);
    return (4 * (grp >> 1) + (r >> 2)) * kDh + cb * 4;  // halfs; + 16 t + 32 kb keys, + 8 keys for the operand's second half
}

__device__ __forceinline__ bf16x8 v_tr_operand(const uint16_t *p)
{
    typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
    typedef bf16x4_t __attribute__((address_space(3))) * lds_ptr;
    const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_ptr)p);
    const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_ptr)(p + 8 * kDh));
    return bf16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

// One work-group per (environment, head); wave w owns queries 32w .. 32w+31 and all waves
// share the K rows and the transposed V rows of the live keys in LDS.
//
// The same kernel serves self-attention over the entity tokens (q, k, v are the three thirds
// of one packed buffer, NQ == NK) and, with CROSS, the read of bullet key/values by the entity
// queries (models/yemong/attention.py:149-166): keys and values come from a second buffer,
// an environment without any live key contributes nothing (the reference gates it off
// instead of letting the uniform average through), and the result is added to `accum`.
// NKB = key blocks and waves of the work-group: max(ceil(NK/32), ceil(NQ/32)).
template <int NKB, bool CROSS>
__global__ __launch_bounds__(kWave * NKB) __attribute__((amdgpu_waves_per_eu(8, 8))) void sdpa_mfma_kernel(
    const uint16_t *__restrict__ q, int64_t q_stride, const uint16_t *__restrict__ k,
    const uint16_t *__restrict__ v, int64_t kv_stride, const uint8_t *__restrict__ alive,
    const uint16_t *accum, uint16_t *out, int B, int NQ, int NK, int H, float scale_log2e)
{
    constexpr int KCAP = NKB * 32;
    constexpr int NT = kWave * NKB;
    __shared__ __align__(16) uint16_t s_k[KCAP * kKeyPitch];
    __shared__ __align__(16) uint16_t s_v[KCAP * kDh];  // V rows as they come, 64 bytes per key (see v_tr_offset)
    __shared__ uint16_t s_cnt[2 * NKB];  // live keys per 16-key slice, in key order

    // Work-groups are dealt round-robin to the 8 XCDs; hand each XCD a contiguous run of
    // (environment, head) pairs so the 4 heads of an environment share one L2.
    const int chunk = gridDim.x >> 3;
    const int logical = (blockIdx.x & 7) * chunk + (blockIdx.x >> 3);
    if (logical >= B * H) return;
    const int env = logical / H;
    const int head = logical - env * H;
    const int D = H * kDh;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keep it scalar
    const int m = lane & 31;
    const int half = lane >> 5;

    const uint16_t *q_base = q + (int64_t)env * NQ * q_stride;

    // ---- this wave's queries (loaded together with the K/V rows, after the alive bytes: the
    //      alive row is tiny and usually an L2 hit, and nothing else can start before it) ----
    const int qrow = wave * 32 + m;
    const int qsafe = qrow < NQ ? qrow : NQ - 1;
    const uint16_t *qp = q_base + (uint32_t)qsafe * (uint32_t)q_stride + (uint32_t)(head * kDh + half * 8);
    u32x4 qw0 = {0u, 0u, 0u, 0u}, qw1 = {0u, 0u, 0u, 0u};

    // ---- K rows and V^T of the live keys into LDS, compacted ----
    // Thread -> (key, 8 channels), two items per thread.  A thread reads its key's alive
    // byte, starts its K/V loads at once if the key is live, and only then works out the
    // key's position among the live keys (ballot inside the wave, per-wave counts through
    // LDS), so the position arithmetic overlaps the loads.
    const uint8_t *alive_env = alive == nullptr ? nullptr : alive + (int64_t)env * NK;
    int cnt = 0;
    bool uniform = false;
    for (int pass = 0; pass < 2; ++pass) {
        // Branch-free on purpose: every lane issues its alive-byte loads back to back, then
        // its K/V loads back to back; a lane whose key is dead or out of range reads key
        // row 0 instead (one cached row) and discards it.
        bool live[2];
        u32x4 kw[2], vw[2];
        uint32_t ab[2] = {1u, 1u};
        if (alive_env != nullptr && !uniform) {
#pragma unroll
            for (int it = 0; it < 2; ++it) {
                const int key = (tid + it * NT) >> 2;
                ab[it] = alive_env[key < NK ? key : NK - 1];
            }
        }
        const uint32_t stride32 = (uint32_t)kv_stride;
        const int64_t kv_env = (int64_t)env * NK * kv_stride + head * kDh + (tid & 3) * 8;
        const uint16_t *k_base = k + kv_env;
        const uint16_t *v_base = v + kv_env;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int key = (tid + it * NT) >> 2;
            live[it] = key < NK && ab[it] != 0;
            const uint32_t off = (live[it] ? (uint32_t)key : 0u) * stride32;
            kw[it] = *reinterpret_cast<const u32x4 *>(k_base + off);
            vw[it] = *reinterpret_cast<const u32x4 *>(v_base + off);
        }
        if (pass == 0) {
            qw0 = *reinterpret_cast<const u32x4 *>(qp);
            qw1 = *reinterpret_cast<const u32x4 *>(qp + 16);
        }
        int before[2];
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const uint64_t mask = __ballot(live[it] && (lane & 3) == 0);  // one bit per live key
            before[it] = __popcll(mask & ((1ull << (lane & ~3)) - 1ull));
            if (lane == 0) s_cnt[it * NKB + wave] = (uint16_t)__popcll(mask);
        }
        __syncthreads();
        int base0 = 0, base1 = 0;
        cnt = 0;
#pragma unroll
        for (int ch = 0; ch < 2 * NKB; ++ch) {
            const int c = s_cnt[ch];
            if (ch < wave) base0 += c;
            if (ch < NKB + wave) base1 += c;
            cnt += c;
        }
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            if (live[it]) {
                // live keys fill the END of the nkb*32 positions; the padding sits in front
                const int pos = (((cnt + 31) & ~31) - cnt) + (it ? base1 : base0) + before[it];
                const int c8 = (tid & 3) * 8;
                *reinterpret_cast<u32x4 *>(s_k + pos * kKeyPitch + c8) = kw[it];
                *reinterpret_cast<u32x4 *>(s_v + pos * kDh + c8) = vw[it];
            }
        }
        if (cnt != 0 || CROSS) break;
        // no live key at all: every key takes part with the same weight; stage them all
        uniform = true;
        __syncthreads();  // s_cnt is rewritten by the second pass
    }
    const int nkb = (cnt + 31) >> 5;
    const int pad = nkb * 32 - cnt;  // positions [0, pad) of key block 0 hold no key
    for (int idx = tid; idx < pad * 4; idx += NT) {
        const int pos = idx >> 2;
        const int c8 = (idx & 3) * 8;
        *reinterpret_cast<u32x4 *>(s_k + pos * kKeyPitch + c8) = u32x4{0u, 0u, 0u, 0u};
        *reinterpret_cast<u32x4 *>(s_v + pos * kDh + c8) = u32x4{0u, 0u, 0u, 0u};
    }
    __syncthreads();
    if (wave * 32 >= NQ) return;  // waves that only helped staging (more key blocks than query blocks)

    // ---- S^T = K Q^T for this wave's 32 queries ----
    // With no live key every score is the same constant: zero queries give exactly that.
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    const bf16x8 qb0 = __builtin_bit_cast(bf16x8, uniform ? zero4 : qw0);
    const bf16x8 qb1 = __builtin_bit_cast(bf16x8, uniform ? zero4 : qw1);
    // Padding is confined to key block 0, where it enters as the initial accumulator (made where it is used: sixteen
    // registers that would otherwise stay occupied from here to the rarely taken second try).
    auto pad_bias = [&](int pad_rows) -> f32x16 {
        f32x16 b;
#pragma unroll
        for (int v = 0; v < 16; ++v) b[v] = (8 * (v >> 2) + 4 * half + (v & 3) < pad_rows) ? -INFINITY : 0.0f;
        return b;
    };

    auto scores = [&](int kb, int pad_rows) -> f32x16 {
        const uint16_t *kp = s_k + (kb * 32 + m) * kKeyPitch + half * 8;
        const bf16x8 ka0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(kp));
        const bf16x8 ka1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(kp + 16));
        f32x16 z = {0.0f};
        if (kb == 0) z = pad_bias(pad_rows);
        z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka0, qb0, z, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka1, qb1, z, 0, 0, 0);
    };

    // ---- P = exp2(scale S - shift), O^T = V^T P^T ----
    // Softmax does not depend on the shift, only the exponent range does.  First try: no shift at all, one sweep
    // (no K Q^T just to find the maximum).  That is exact to rounding whenever the sum of a query's weights stays
    // well inside the float32 range; a wave with a query whose sum does not (scores beyond +-60 in log2 units, or not
    // finite) throws the try away and takes the two sweeps with the true maximum as shift.
    float sum = 0.0f;
    f32x16 o = {0.0f};
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    const int v_off = v_tr_offset(lane);
    auto sweep = [&](auto shifted, float mc, int pad_rows) {
        sum = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; ++v) o[v] = 0.0f;
        for (int kb = 0; kb < nkb; ++kb) {
            const f32x16 z = scores(kb, pad_rows);
            float p[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                if constexpr (decltype(shifted)::value) p[v] = __builtin_amdgcn_exp2f(fmaf(z[v], scale_log2e, -mc));
                else p[v] = __builtin_amdgcn_exp2f(z[v] * scale_log2e);
            }
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                bf16x8 pb;
#pragma unroll
                for (int e = 0; e < 8; ++e) pb[e] = (__bf16)p[8 * t + e];
                // the normaliser adds the weights as the matrix product sees them (rounded to bfloat16), a pair per
                // instruction: a query with one live key then gets that key's value row back exactly
#pragma unroll
                for (int e = 0; e < 8; e += 2) sum = __builtin_amdgcn_fdot2_f32_bf16(bf16x2{pb[e], pb[e + 1]}, ones, sum, false);
                const bf16x8 va = v_tr_operand(s_v + (kb * 32 + 16 * t) * kDh + v_off);
                o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb, o, 0, 0, 0);
            }
        }
        sum += __shfl_xor(sum, 32);
    };
    sweep(std::false_type{}, 0.0f, pad);
    const bool in_range = (sum >= 0x1p-60f && sum <= 0x1p60f) || (CROSS && cnt == 0);  // false for NaN
    if (!__all(in_range)) {
        int pad_again = pad;
        asm volatile("" : "+v"(pad_again));  // a value of its own: nothing of the first try is kept for this one
        float mx = -INFINITY;
        for (int kb = 0; kb < nkb; ++kb) {
            const f32x16 z = scores(kb, pad_again);
#pragma unroll
            for (int v = 0; v < 16; ++v) mx = fmaxf(mx, z[v]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        sweep(std::true_type{}, mx * scale_log2e, pad_again);
    }
    // CROSS with no live key: nkb == 0, o == 0 and the contribution is exactly zero
    const float inv = (CROSS && cnt == 0) ? 0.0f : __builtin_amdgcn_rcpf(sum);

    // The MFMA leaves a lane with rows 8i + 4*half + j (i, j = 0..3) of O^T.  V^T was stored
    // with its rows permuted so that MFMA row 8i + 4*half + j is channel
    // 16*(i/2) + 8*half + 4*(i%2) + j: the lane then owns two runs of 8 consecutive channels,
    // 16 bytes each.  Stored as they are, one instruction would write 32 bytes of each of 32 rows.
    // Lanes m and m + 16 first trade runs (v_permlane16_swap: the second run of query m goes to the
    // lane of query m + 16, whose first run comes back), so that one store instruction writes the
    // whole 64-byte head row of 16 queries and the other the rows of the other 16.
    {
        u32x4 w[2];
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            float r[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) r[e] = o[8 * g + e] * inv;
            if (CROSS && accum != nullptr) {
                // bf16 + bf16 as torch adds them: the read result is rounded first, then the sum
                const int qs = qrow < NQ ? qrow : NQ - 1;
                const Row8 a = load8(accum + ((int64_t)env * NQ + qs) * D + head * kDh + 8 * half + 16 * g);
#pragma unroll
                for (int e = 0; e < 8; ++e) r[e] = a.v[e] + round_to_bf16(r[e]);
            }
            w[g] = u32x4{pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3]), pack_bf16x2(r[4], r[5]), pack_bf16x2(r[6], r[7])};
        }
#pragma unroll
        for (int cdw = 0; cdw < 4; ++cdw) {
            const u32x2 t = __builtin_amdgcn_permlane16_swap(w[0][cdw], w[1][cdw], false, false);
            w[0][cdw] = t.x, w[1][cdw] = t.y;
        }
        // lane (m, half) now holds, of query 32 wave + m%16: channels 16 (m/16) + 8 half .. +7 in w[0];
        // of query 32 wave + 16 + m%16: the same channels in w[1]
        const int row_a = wave * 32 + (m & 15);
        const int ch = head * kDh + 16 * (m >> 4) + 8 * half;
        if (row_a < NQ) *reinterpret_cast<u32x4 *>(out + ((int64_t)env * NQ + row_a) * D + ch) = w[0];
        if (row_a + 16 < NQ) *reinterpret_cast<u32x4 *>(out + ((int64_t)env * NQ + row_a + 16) * D + ch) = w[1];
    }
}

// ------------------------------------------------------------------------------------
// Two heads per wavefront for NM <= 16 (bf16, dh = 32): the 4v4 rollout shape
// ------------------------------------------------------------------------------------
//
// With 12 tokens a 32x32 MFMA tile is mostly padding and the kernel is bound by the vector
// instructions a wave issues, not by the matrix cores or HBM; those instructions cost the
// same whether 12 or 32 columns of the tile carry data.  Here one wave works on two heads of
// one environment at once: head s (0/1) owns key positions and query columns 16s .. 16s+15 of
// the tile, the products between the two halves are switched off by the same -inf
// accumulator that hides dead keys, and since P is zero there the single O^T = V^T P^T
// product returns each head's output in its own columns (V^T holds head 0's values at key
// positions 0..15 and head 1's at 16..31).  Keys are not compacted (nothing to save inside
// one tile).  Same all-dead rule, same layouts and output stage as sdpa_mfma_kernel.
__global__ __launch_bounds__(kWave) void sdpa_mfma_pair_kernel(
    const uint16_t *__restrict__ qkv, int64_t stride, const uint8_t *__restrict__ alive, uint16_t *__restrict__ out,
    int B, int NM, int H, float scale_log2e)
{
    constexpr int VP = 32 + 4;
    __shared__ __align__(16) uint16_t s_k[32 * kKeyPitch];
    __shared__ __align__(16) uint16_t s_vt[kDh * VP];

    const int pairs_per_env = H >> 1;
    const int chunk = gridDim.x >> 3;
    const int logical = (blockIdx.x & 7) * chunk + (blockIdx.x >> 3);
    if (logical >= B * pairs_per_env) return;
    const int env = logical / pairs_per_env;
    const int head0 = 2 * (logical - env * pairs_per_env);
    const int D = H * kDh;

    const int lane = threadIdx.x;
    const int m = lane & 31;
    const int half = lane >> 5;
    const uint16_t *base = qkv + (int64_t)env * NM * stride;

    // item it of this thread: head head0 + it, key lane/4, channels 8*(lane%4) .. +7
    const int key = lane >> 2;
    const int c8 = (lane & 3) * 8;
    uint32_t ab = 1u;
    if (alive != nullptr) ab = alive[(int64_t)env * NM + (key < NM ? key : NM - 1)];
    const bool present = key < NM;
    const uint32_t row_off = (uint32_t)(present ? key : 0) * (uint32_t)stride;
    u32x4 kw[2], vw[2];
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const uint16_t *p = base + row_off + (head0 + it) * kDh + c8;
        kw[it] = *reinterpret_cast<const u32x4 *>(p + D);
        vw[it] = *reinterpret_cast<const u32x4 *>(p + 2 * D);
    }
    // this lane's query: column m of the tile = head m/16, token m%16
    const int qi = m & 15;
    const int qhead = head0 + (m >> 4);
    const uint16_t *qp = base + (uint32_t)(qi < NM ? qi : NM - 1) * (uint32_t)stride + qhead * kDh + half * 8;
    u32x4 qw0 = *reinterpret_cast<const u32x4 *>(qp);
    u32x4 qw1 = *reinterpret_cast<const u32x4 *>(qp + 16);

    // live keys of the environment (both heads share the mask), one bit per key at bit 4*key;
    // none alive: every key takes part with the same weight
    uint64_t live_mask = __ballot(present && ab != 0 && (lane & 3) == 0);
    const bool uniform = live_mask == 0;
    if (uniform) live_mask = __ballot(present && (lane & 3) == 0);
    const bool live = (live_mask >> (lane & ~3)) & 1ull;
    // Keys stay at their own position 16*head + key; a dead or absent key is stored as zeros
    // (its weight is exactly 0 and 0 * finite keeps the product clean whatever memory holds).
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int pos = 16 * it + key;
        const u32x4 z4 = {0u, 0u, 0u, 0u};
        const u32x4 kk = live ? kw[it] : z4;
        const u32x4 vv = live ? vw[it] : z4;
        *reinterpret_cast<u32x4 *>(s_k + pos * kKeyPitch + c8) = kk;
        // channel d = c8 + e goes to V^T row vt_row(d) (see the output stage of sdpa_mfma_kernel)
        uint16_t *dst = s_vt + (16 * (c8 >> 4) + 4 * ((c8 >> 3) & 1)) * VP + pos;
        dst[0 * VP] = (uint16_t)(vv.x & 0xffffu);
        dst[1 * VP] = (uint16_t)(vv.x >> 16);
        dst[2 * VP] = (uint16_t)(vv.y & 0xffffu);
        dst[3 * VP] = (uint16_t)(vv.y >> 16);
        dst[8 * VP] = (uint16_t)(vv.z & 0xffffu);
        dst[9 * VP] = (uint16_t)(vv.z >> 16);
        dst[10 * VP] = (uint16_t)(vv.w & 0xffffu);
        dst[11 * VP] = (uint16_t)(vv.w >> 16);
    }
    __syncthreads();

    // Row r of the score tile (key position r) counts for this lane's query iff it belongs to
    // the same head and its key is live; everything else enters as -inf through the initial
    // accumulator.  A lane holds rows 8i + 4*half + j: key (8i + 4*half + j) % 16 of head i/2,
    // whose live bit sits at 32*(i%2) + 16*half + 4*j.  With no live key every score is the
    // same constant: zero queries give exactly that.
    if (uniform) qw0 = qw1 = u32x4{0u, 0u, 0u, 0u};
    const uint64_t mine = live_mask >> (16 * half);
    const int qsub = m >> 4;
    f32x16 z;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const bool on = (v >> 3) == qsub && ((mine >> (32 * ((v >> 2) & 1) + 4 * (v & 3))) & 1ull);
        z[v] = on ? 0.0f : -INFINITY;
    }
    {
        const uint16_t *kp = s_k + m * kKeyPitch + half * 8;
        const bf16x8 ka0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(kp));
        const bf16x8 ka1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(kp + 16));
        z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka0, __builtin_bit_cast(bf16x8, qw0), z, 0, 0, 0);
        z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka1, __builtin_bit_cast(bf16x8, qw1), z, 0, 0, 0);
    }
    // weights without a shift first, with the maximum as shift when a query's sum leaves the safe exponent range
    // (see sdpa_mfma_kernel); the scores stay in registers here, so the second try costs no matrix product
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    float sum;
    bf16x8 pb[2];
    auto weights = [&](auto shifted, float mc) {
        sum = 0.0f;
        float p[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            if constexpr (decltype(shifted)::value) p[v] = __builtin_amdgcn_exp2f(fmaf(z[v], scale_log2e, -mc));
            else p[v] = __builtin_amdgcn_exp2f(z[v] * scale_log2e);
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int e = 0; e < 8; ++e) pb[t][e] = (__bf16)p[8 * t + e];
#pragma unroll
            for (int e = 0; e < 8; e += 2) sum = __builtin_amdgcn_fdot2_f32_bf16(bf16x2{pb[t][e], pb[t][e + 1]}, ones, sum, false);
        }
        sum += __shfl_xor(sum, 32);
    };
    weights(std::false_type{}, 0.0f);
    if (!__all(sum >= 0x1p-60f && sum <= 0x1p60f)) {
        float mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; ++v) mx = fmaxf(mx, z[v]);
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        weights(std::true_type{}, mx * scale_log2e);
    }
    f32x16 o = {0.0f};
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const uint16_t *vp = s_vt + m * VP + 16 * t + 4 * half;
        const u32x2 lo = *reinterpret_cast<const u32x2 *>(vp);
        const u32x2 hi = *reinterpret_cast<const u32x2 *>(vp + 8);
        const u32x4 vq = {lo.x, lo.y, hi.x, hi.y};
        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vq), pb[t], o, 0, 0, 0);
    }
    const float inv = __builtin_amdgcn_rcpf(sum);
    // Lanes m and m + 16 hold the same token of the pair's two heads.  They trade runs as in
    // sdpa_mfma_kernel, so that one store instruction writes the whole 64-byte row of the first
    // head for every token and the other the row of the second head (instead of 32 bytes of each).
    u32x4 w[2];
#pragma unroll
    for (int g = 0; g < 2; ++g)
        w[g] = u32x4{pack_bf16x2(o[8 * g + 0] * inv, o[8 * g + 1] * inv), pack_bf16x2(o[8 * g + 2] * inv, o[8 * g + 3] * inv),
                     pack_bf16x2(o[8 * g + 4] * inv, o[8 * g + 5] * inv), pack_bf16x2(o[8 * g + 6] * inv, o[8 * g + 7] * inv)};
#pragma unroll
    for (int cdw = 0; cdw < 4; ++cdw) {
        const u32x2 t = __builtin_amdgcn_permlane16_swap(w[0][cdw], w[1][cdw], false, false);
        w[0][cdw] = t.x, w[1][cdw] = t.y;
    }
    if (qi < NM) {
        // w[0]: head head0, w[1]: head head0 + 1; channels 16 (m/16) + 8 half .. +7 of each
        const int64_t o_off = ((int64_t)env * NM + qi) * D + head0 * kDh + 16 * (m >> 4) + 8 * half;
        *reinterpret_cast<u32x4 *>(out + o_off) = w[0];
        *reinterpret_cast<u32x4 *>(out + o_off + kDh) = w[1];
    }
}

// ------------------------------------------------------------------------------------
// fp32 on the matrix cores (dh = 32, up to 512 tokens): evaluation without autocast
// ------------------------------------------------------------------------------------
//
// v_mfma_f32_32x32x2_f32 takes one fp32 per lane for A and for B (row / column l%32, k = l/32)
// and accumulates in fp32, so the result meets the fp32 bar while the products leave the
// vector ALUs (which the fp32 vector kernel saturates from ~64 tokens on).  Same formulation
// as sdpa_mfma_kernel: one work-group per (environment, head), wave w owns queries 32w..32w+31,
// live keys compacted to the end of the staged positions, S^T = K Q^T with keys on the M axis.
// Differences that the operand shape allows:
//   * the k index of a product may run in any order as long as A and B agree, so K Q^T walks
//     channel 16*half + s at step s (a lane's 16 query values are one contiguous 64-byte load,
//     K rows sit in LDS at an odd pitch) and V^T P^T walks key 8(s/4) + 4*half + s%4 -- exactly
//     the key whose score the lane holds in accumulator register s, so P never moves and V is
//     read from LDS as stored (32 consecutive channels per key: no transposed copy);
//   * one sweep with a running maximum (the matrix cores are the bound here, 32 MFMAs of 64
//     cycles per key block, and rescaling 16 accumulators per block is free next to that).
constexpr int kF32KeyPitch = kDh + 1;  // floats per K row in LDS: odd, so 32 rows hit 32 banks

__global__ __launch_bounds__(1024) void sdpa_mfma_f32_kernel(
    const float *__restrict__ qkv, int64_t stride, const uint8_t *__restrict__ alive, float *__restrict__ out, int B,
    int NM, int H, float scale_log2e)
{
    extern __shared__ __align__(16) float s_f32[];
    const int nwaves = blockDim.x >> 6;
    const int kcap = nwaves * 32;
    float *s_k = s_f32;                         // [kcap][33]
    float *s_v = s_k + kcap * kF32KeyPitch;     // [kcap][32]
    int *s_cnt = reinterpret_cast<int *>(s_v + kcap * kDh);  // [2 * nwaves]

    const int chunk = gridDim.x >> 3;
    const int logical = (blockIdx.x & 7) * chunk + (blockIdx.x >> 3);
    if (logical >= B * H) return;
    const int env = logical / H;
    const int head = logical - env * H;
    const int D = H * kDh;
    const int tid = threadIdx.x;
    const int NT = blockDim.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31;
    const int half = lane >> 5;
    const float *base = qkv + (int64_t)env * NM * stride;

    // this lane's query values: channels 16*half .. +15 of query 32*wave + m
    const int qrow = wave * 32 + m;
    const float *qp = base + (int64_t)(qrow < NM ? qrow : NM - 1) * stride + head * kDh + 16 * half;
    f32x4 qv[4];

    // ---- K and V rows of the live keys into LDS, compacted (thread = key, 8 channels; two items) ----
    const uint8_t *alive_env = alive == nullptr ? nullptr : alive + (int64_t)env * NM;
    int cnt = 0;
    bool uniform = false;
    for (int pass = 0; pass < 2; ++pass) {
        bool live[2];
        f32x4 kw[2][2], vw[2][2];
        uint32_t ab[2] = {1u, 1u};
        if (alive_env != nullptr && !uniform) {
#pragma unroll
            for (int it = 0; it < 2; ++it) {
                const int key = (tid + it * NT) >> 2;
                ab[it] = alive_env[key < NM ? key : NM - 1];
            }
        }
        const float *k_base = base + D + head * kDh + (tid & 3) * 8;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int key = (tid + it * NT) >> 2;
            live[it] = key < NM && ab[it] != 0;
            const float *kp = k_base + (int64_t)(live[it] ? key : 0) * stride;
            kw[it][0] = *reinterpret_cast<const f32x4 *>(kp);
            kw[it][1] = *reinterpret_cast<const f32x4 *>(kp + 4);
            vw[it][0] = *reinterpret_cast<const f32x4 *>(kp + D);
            vw[it][1] = *reinterpret_cast<const f32x4 *>(kp + D + 4);
        }
        if (pass == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) qv[i] = *reinterpret_cast<const f32x4 *>(qp + 4 * i);
        }
        int before[2];
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const uint64_t mask = __ballot(live[it] && (lane & 3) == 0);  // one bit per live key
            before[it] = __popcll(mask & ((1ull << (lane & ~3)) - 1ull));
            if (lane == 0) s_cnt[it * nwaves + wave] = (int)__popcll(mask);
        }
        __syncthreads();
        int base0 = 0, base1 = 0;
        cnt = 0;
        for (int ch = 0; ch < 2 * nwaves; ++ch) {
            const int c = s_cnt[ch];
            if (ch < wave) base0 += c;
            if (ch < nwaves + wave) base1 += c;
            cnt += c;
        }
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            if (live[it]) {
                // live keys fill the END of the nkb*32 positions; the padding sits in front
                const int pos = (((cnt + 31) & ~31) - cnt) + (it ? base1 : base0) + before[it];
                const int c8 = (tid & 3) * 8;
                float *kd = s_k + pos * kF32KeyPitch + c8;
                kd[0] = kw[it][0].x, kd[1] = kw[it][0].y, kd[2] = kw[it][0].z, kd[3] = kw[it][0].w;
                kd[4] = kw[it][1].x, kd[5] = kw[it][1].y, kd[6] = kw[it][1].z, kd[7] = kw[it][1].w;
                *reinterpret_cast<f32x4 *>(s_v + pos * kDh + c8) = vw[it][0];
                *reinterpret_cast<f32x4 *>(s_v + pos * kDh + c8 + 4) = vw[it][1];
            }
        }
        if (cnt != 0) break;
        // no live key at all: every key takes part with the same weight; stage them all
        uniform = true;
        __syncthreads();  // s_cnt is rewritten by the second pass
    }
    const int nkb = (cnt + 31) >> 5;
    const int pad = nkb * 32 - cnt;  // positions [0, pad) of key block 0 hold no key
    for (int idx = tid; idx < pad * kDh; idx += NT) {
        const int pos = idx >> 5, c = idx & 31;
        s_k[pos * kF32KeyPitch + c] = 0.0f;
        s_v[pos * kDh + c] = 0.0f;
    }
    __syncthreads();
    if (wave * 32 >= NM) return;  // waves that only helped staging

    // with no live key every score is the same constant: zero queries give exactly that
    float q[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        q[4 * i + 0] = uniform ? 0.0f : qv[i].x, q[4 * i + 1] = uniform ? 0.0f : qv[i].y;
        q[4 * i + 2] = uniform ? 0.0f : qv[i].z, q[4 * i + 3] = uniform ? 0.0f : qv[i].w;
    }

    float run_max = -INFINITY, sum = 0.0f;
    f32x16 o = {0.0f};
    for (int kb = 0; kb < nkb; ++kb) {
        f32x16 z = {0.0f};
        if (kb == 0) {
#pragma unroll
            for (int v = 0; v < 16; ++v) z[v] = (8 * (v >> 2) + 4 * half + (v & 3) < pad) ? -INFINITY : 0.0f;
        }
        const float *kp = s_k + (kb * 32 + m) * kF32KeyPitch + 16 * half;
#pragma unroll
        for (int st = 0; st < 16; ++st) z = __builtin_amdgcn_mfma_f32_32x32x2f32(kp[st], q[st], z, 0, 0, 0);
        float bmax = z[0];
#pragma unroll
        for (int v = 1; v < 16; ++v) bmax = fmaxf(bmax, z[v]);
        bmax = fmaxf(bmax, __shfl_xor(bmax, 32));
        const float new_max = fmaxf(run_max, bmax);  // finite: every key block holds at least one live key
        const float alpha = __builtin_amdgcn_exp2f((run_max - new_max) * scale_log2e);
        run_max = new_max;
        const float mc = new_max * scale_log2e;
        sum *= alpha;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            o[v] *= alpha;
            z[v] = __builtin_amdgcn_exp2f(fmaf(z[v], scale_log2e, -mc));
            sum += z[v];
        }
        // V^T P^T: step st pairs accumulator register st (key 8(st/4) + 4*half + st%4) with that key's V row
        const float *vp = s_v + (kb * 32 + 4 * half) * kDh + m;
#pragma unroll
        for (int st = 0; st < 16; ++st)
            o = __builtin_amdgcn_mfma_f32_32x32x2f32(vp[(8 * (st >> 2) + (st & 3)) * kDh], z[st], o, 0, 0, 0);
    }
    sum += __shfl_xor(sum, 32);
    const float inv = 1.0f / sum;
    if (qrow < NM) {
        // the lane holds channels 8a + 4*half + b (a, b = 0..3) of its query: four 16-byte pieces
        float *op = out + ((int64_t)env * NM + qrow) * D + head * kDh + 4 * half;
#pragma unroll
        for (int a = 0; a < 4; ++a)
            *reinterpret_cast<f32x4 *>(op + 8 * a) =
                f32x4{o[4 * a + 0] * inv, o[4 * a + 1] * inv, o[4 * a + 2] * inv, o[4 * a + 3] * inv};
    }
}

// ------------------------------------------------------------------------------------
// Streaming MFMA kernel for the bullet read with many keys (bf16, dh = 32)
// ------------------------------------------------------------------------------------
//
// The bullet axis is N*K slots long (80 .. 1520 in the shipped scenarios) and mostly
// empty: only bullets in flight are keys.  One work-group per (environment, head), one
// wave per 32 queries (up to four waves, see below).  The work-group first compacts the indices
// of the live bullets into LDS, then walks them in tiles of 32 keys per wave: the K rows and
// transposed V rows of the next tile are gathered from global memory into registers while the
// matrix cores work on the current tile out of LDS (two LDS buffers, one barrier per tile), with
// the running maximum / sum / output of an online softmax carried across tiles.  Key
// positions, operand layouts and the output stage are those of sdpa_mfma_kernel.
//
// Waves per work-group: a CU places a work-group only while every one of its four SIMDs has room for
// ceil(waves / 4) more waves, and the waves of a work-group move in step (one barrier per tile), so a
// work-group of five waves runs at the pace of the SIMD that holds two of them.  Hence never more than
// four waves: with five blocks of queries (129 .. 160 queries) waves 0..3 own blocks 0..3, and the fifth
// block is shared - in every tile of 128 keys wave w takes its key block w for those 32 queries, with its
// own running maximum, sum and output, and the four partial results are merged through LDS at the end.

constexpr int kStreamMaxKeys = 2048;

template <int NQB, bool LSE>
__global__ __launch_bounds__(kWave *(NQB < 4 ? NQB : 4), 3) void sdpa_cross_stream_kernel(
    const uint16_t *__restrict__ q, int64_t q_stride, const uint16_t *__restrict__ k,
    const uint16_t *__restrict__ v, int64_t kv_stride, const uint8_t *__restrict__ alive,
    const int32_t *__restrict__ ranges, const uint16_t *accum, uint16_t *out, float *__restrict__ lse_out, int B, int NQ,
    int NK, int H, float scale_log2e)
{
    constexpr int NW = NQB < 4 ? NQB : 4;  // waves, and key blocks per tile
    constexpr bool SPLIT = NQB > NW;       // a fifth block of queries, shared by the four waves
    static_assert(NQB <= 5, "at most one shared block of queries");
    constexpr int TK = 32 * NW;   // keys per tile
    constexpr int NT = kWave * NW;
    __shared__ __align__(16) uint16_t s_k[2][TK * kKeyPitch];
    __shared__ __align__(16) uint16_t s_v[2][TK * kDh];  // V rows as they come, 64 bytes per key
    __shared__ uint16_t s_idx[kStreamMaxKeys];  // indices of the live keys, ascending
    __shared__ int s_wcnt[NW];
    static_assert(!SPLIT || sizeof(s_k) >= (size_t)NW * (16 * kWave + 3 * 32) * sizeof(float),
                  "the partial results of the shared block are merged through the K buffers");

    const int chunk = gridDim.x >> 3;
    const int logical = (blockIdx.x & 7) * chunk + (blockIdx.x >> 3);
    if (logical >= B * H) return;
    const int env = logical / H;
    const int head = logical - env * H;
    const int D = H * kDh;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31;
    const int half = lane >> 5;

    // this wave's queries, in flight while the key list is set up
    const int qrow = wave * 32 + m;
    const int qsafe = qrow < NQ ? qrow : NQ - 1;
    const uint16_t *qp = q + (int64_t)env * NQ * q_stride + (uint32_t)qsafe * (uint32_t)q_stride +
                         (uint32_t)(head * kDh + half * 8);
    const u32x4 qw0 = *reinterpret_cast<const u32x4 *>(qp);
    const u32x4 qw1 = *reinterpret_cast<const u32x4 *>(qp + 16);
    // the shared block of queries (rows 32 NW ..)
    const int srow = NW * 32 + m;
    const int ssafe = srow < NQ ? srow : NQ - 1;
    u32x4 sw0 = {0u, 0u, 0u, 0u}, sw1 = {0u, 0u, 0u, 0u};
    if (SPLIT) {
        const uint16_t *sp = q + (int64_t)env * NQ * q_stride + (uint32_t)ssafe * (uint32_t)q_stride +
                             (uint32_t)(head * kDh + half * 8);
        sw0 = *reinterpret_cast<const u32x4 *>(sp);
        sw1 = *reinterpret_cast<const u32x4 *>(sp + 16);
    }

    // Two ways to name the live keys of the environment: `ranges` (the K/V rows were already
    // compacted: rows ranges[env] .. ranges[env+1]-1 of one list for all environments), or a
    // mask over NK slots per environment, compacted here into an index list in LDS.
    int cnt;
    uint32_t first_row = 0;
    if (ranges != nullptr) {
        first_row = (uint32_t)ranges[env];
        cnt = ranges[env + 1] - (int)first_row;
        if (cnt == 0 && accum == out) return;
    } else {
        // wave w scans keys [w*J*64, (w+1)*J*64), 64 per ballot
        const uint8_t *alive_env = alive == nullptr ? nullptr : alive + (int64_t)env * NK;
        const int J = (NK + NT - 1) / NT;  // <= 32 because NK <= kStreamMaxKeys
        const int key0 = wave * J * 64 + lane;
        uint32_t bits = 0;
        int mine = 0;
        // without a mask every slot is a key: the scan reads a byte that is never zero (a branch on the pointer
        // between the loads would make the compiler wait for each load inside its own branch, one round trip per byte)
        static __device__ const uint8_t kAllAlive[1] = {1};
        const uint8_t *alive_src = alive_env != nullptr ? alive_env : kAllAlive;
        const int alive_last = alive_env != nullptr ? NK - 1 : 0;
        for (int j0 = 0; j0 < J; j0 += 8) {
            // eight independent byte loads in flight, then their ballots
            uint32_t a[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int key = key0 + (j0 + u) * 64;
                const bool in = j0 + u < J && key < NK;
                a[u] = alive_src[key < alive_last ? key : alive_last];
                a[u] = in ? a[u] : 0u;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const bool on = a[u] != 0;
                bits |= (on ? 1u : 0u) << ((j0 + u) & 31);
                mine += (int)__popcll(__ballot(on));
            }
        }
        if (lane == 0) s_wcnt[wave] = mine;
        __syncthreads();
        int base = 0;
        cnt = 0;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const int c = s_wcnt[w];
            if (w < wave) base += c;
            cnt += c;
        }
        // nothing in flight in this environment: the read contributes exactly zero
        if (cnt == 0 && accum == out) return;
        for (int j = 0; j < J; ++j) {
            const bool a = (bits >> j) & 1u;
            const uint64_t mask = __ballot(a);
            if (a) s_idx[base + (int)__popcll(mask & ((1ull << lane) - 1ull))] = (uint16_t)(key0 + j * 64);
            base += (int)__popcll(mask);
        }
        __syncthreads();
    }

    const int nkb = (cnt + 31) >> 5;
    const int pad = nkb * 32 - cnt;  // positions [0, pad) of the first key block hold no key
    const int ntiles = (nkb + NW - 1) / NW;

    // thread -> (position in tile, 8 channels), two items per thread
    const uint32_t stride32 = (uint32_t)kv_stride;
    const int64_t kv_env = (ranges != nullptr ? 0 : (int64_t)env * NK * kv_stride) + head * kDh + (tid & 3) * 8;
    const uint16_t *k_base = k + kv_env;
    const uint16_t *v_base = v + kv_env;
    u32x4 kw[2], vw[2];
    auto gather = [&](int t) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int li = t * TK + ((tid + it * NT) >> 2) - pad;  // index among the live keys
            const int lc = (li >= 0 && li < cnt) ? li : 0;
            const uint32_t key = ranges != nullptr ? first_row + (uint32_t)lc : (uint32_t)s_idx[lc];
            kw[it] = *reinterpret_cast<const u32x4 *>(k_base + key * stride32);
            vw[it] = *reinterpret_cast<const u32x4 *>(v_base + key * stride32);
        }
    };
    auto stash = [&](int t, int buf) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int lp = (tid + it * NT) >> 2;
            const int li = t * TK + lp - pad;
            if (li < cnt) {
                const u32x4 zero4 = {0u, 0u, 0u, 0u};
                const u32x4 kk = li >= 0 ? kw[it] : zero4;  // padding: zero K and V rows
                const u32x4 vv = li >= 0 ? vw[it] : zero4;
                const int c8 = (tid & 3) * 8;
                *reinterpret_cast<u32x4 *>(&s_k[buf][lp * kKeyPitch + c8]) = kk;
                *reinterpret_cast<u32x4 *>(&s_v[buf][lp * kDh + c8]) = vv;
            }
        }
    };

    const bf16x8 qb0 = __builtin_bit_cast(bf16x8, qw0);
    const bf16x8 qb1 = __builtin_bit_cast(bf16x8, qw1);
    const bf16x8 sb0 = __builtin_bit_cast(bf16x8, sw0);
    const bf16x8 sb1 = __builtin_bit_cast(bf16x8, sw1);
    float mx = -INFINITY, sum = 0.0f;
    f32x16 o = {0.0f};
    // this wave's part of the shared block: its own maximum, sum and output over the key blocks it takes
    float smx = -INFINITY, ssum = 0.0f;
    f32x16 so = {0.0f};

    // the rows this lane will add its result to, fetched while the first tile is gathered
    const int64_t o_off = ((int64_t)env * NQ + qsafe) * D + head * kDh + 8 * half;
    u32x4 acc0 = {0u, 0u, 0u, 0u}, acc1 = {0u, 0u, 0u, 0u};
    if (accum != nullptr) {
        acc0 = *reinterpret_cast<const u32x4 *>(accum + o_off);
        acc1 = *reinterpret_cast<const u32x4 *>(accum + o_off + 16);
    }
    // The walk over the tiles, in two forms.  First try (`shifted` false): weights exp2(scale S) without any shift - no
    // sweep for the maximum, no rescaling between tiles, one K Q^T per key block.  Softmax does not depend on the
    // shift, only the exponent range does: when a query's sum of weights leaves the safe float32 range (scores beyond
    // +-60 in log2 units, or not finite), the whole work-group throws the try away and walks the tiles again in the
    // second form, an online softmax with the running maximum as shift (two sweeps per tile).
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    const int v_off = v_tr_offset(lane);
    float esum = 0.0f, sesum = 0.0f;  // the weights before rounding, for the log-sum-exp a backward pass asks for (LSE)
    auto walk = [&](auto shifted) {
        constexpr bool SHIFT = decltype(shifted)::value;
        if (ntiles > 0) {
            gather(0);
            stash(0, 0);
        }
        // Every load issued so far has to be back before the loop: otherwise the compiler guards
        // the first use of the query registers inside the loop with a wait for ALL outstanding
        // loads, and that wait would also stall every iteration on the next tile's gather.
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0), expcnt/lgkmcnt untouched
        __syncthreads();
        for (int t = 0; t < ntiles; ++t) {
            const int buf = t & 1;
            if (t + 1 < ntiles) gather(t + 1);
            int nb = nkb - t * NW;
            nb = nb < NW ? nb : NW;
            // K Q^T of key block kb.  Only the very first key block can hold padding positions; they
            // get -inf there.  The empty asm keeps that rare fix-up a real branch: folded into
            // selects it would cost 16 extra instructions in every key block.
            auto scores_of = [&](int kb, const bf16x8 &q0, const bf16x8 &q1) -> f32x16 {
                const uint16_t *kp = &s_k[buf][(kb * 32 + m) * kKeyPitch + half * 8];
                const bf16x8 ka0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(kp));
                const bf16x8 ka1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(kp + 16));
                f32x16 z = {0.0f};
                z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka0, q0, z, 0, 0, 0);
                return __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka1, q1, z, 0, 0, 0);
            };
            auto scores = [&](int kb) -> f32x16 { return scores_of(kb, qb0, qb1); };
            auto mask_padding = [&](f32x16 &z) {
                asm volatile("" ::: "memory");
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    if (8 * (e >> 2) + 4 * half + (e & 3) < pad) z[e] = -INFINITY;
            };
            // the normaliser adds the weights as the matrix product sees them (rounded to bfloat16, a pair per
            // instruction): a query with one live key gets that key's value row back exactly
            auto weigh_into = [&](int kb, const f32x16 &z, float mc, float &total, float &exact, f32x16 &acc) {
                float p[16];
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    if constexpr (SHIFT) p[e] = __builtin_amdgcn_exp2f(fmaf(z[e], scale_log2e, -mc));
                    else p[e] = __builtin_amdgcn_exp2f(z[e] * scale_log2e);
                    if (LSE) exact += p[e];
                }
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2) {
                    bf16x8 pb;
#pragma unroll
                    for (int e = 0; e < 8; ++e) pb[e] = (__bf16)p[8 * h2 + e];
#pragma unroll
                    for (int e = 0; e < 8; e += 2) total = __builtin_amdgcn_fdot2_f32_bf16(bf16x2{pb[e], pb[e + 1]}, ones, total, false);
                    const bf16x8 va = v_tr_operand(&s_v[buf][(kb * 32 + 16 * h2) * kDh + v_off]);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb, acc, 0, 0, 0);
                }
            };
            auto weigh = [&](int kb, const f32x16 &z, float mc) { weigh_into(kb, z, mc, sum, esum, o); };
            if (wave * 32 < NQ) {
                float mc = 0.0f;
                int kb = 0;
                if constexpr (SHIFT) {
                    // two key blocks per iteration: two independent MFMA chains in flight
                    float tmx = -INFINITY;
                    for (; kb + 1 < nb; kb += 2) {
                        f32x16 z0 = scores(kb);
                        const f32x16 z1 = scores(kb + 1);
                        if (t == 0 && kb == 0 && pad != 0) mask_padding(z0);
#pragma unroll
                        for (int e = 0; e < 16; ++e) tmx = fmaxf(tmx, z0[e]);  // one chain: max(z0[e], z1[e]) first would have both
#pragma unroll
                        for (int e = 0; e < 16; ++e) tmx = fmaxf(tmx, z1[e]);  // operands quieted by a v_max x, x each (56 ops, not 16)
                    }
                    if (kb < nb) {
                        f32x16 z0 = scores(kb);
                        if (t == 0 && kb == 0 && pad != 0) mask_padding(z0);
#pragma unroll
                        for (int e = 0; e < 16; ++e) tmx = fmaxf(tmx, z0[e]);
                    }
                    tmx = fmaxf(tmx, __shfl_xor(tmx, 32));
                    const float mnew = fmaxf(mx, tmx);  // finite: every key block holds at least one live key
                    const float alpha = __builtin_amdgcn_exp2f((mx - mnew) * scale_log2e);
                    mx = mnew;
                    sum *= alpha;
                    if (LSE) esum *= alpha;
#pragma unroll
                    for (int e = 0; e < 16; ++e) o[e] *= alpha;
                    mc = mx * scale_log2e;
                    kb = 0;
                }
                for (; kb + 1 < nb; kb += 2) {
                    f32x16 z0 = scores(kb);
                    const f32x16 z1 = scores(kb + 1);
                    if (t == 0 && kb == 0 && pad != 0) mask_padding(z0);
                    weigh(kb, z0, mc);
                    weigh(kb + 1, z1, mc);
                }
                if (kb < nb) {
                    f32x16 z0 = scores(kb);
                    if (t == 0 && kb == 0 && pad != 0) mask_padding(z0);
                    weigh(kb, z0, mc);
                }
            }
            if (SPLIT && wave < nb) {
                // the shared block of queries against key block `wave` of the tile
                f32x16 z = scores_of(wave, sb0, sb1);
                if (t == 0 && wave == 0 && pad != 0) mask_padding(z);
                if constexpr (SHIFT) {
                    // one online-softmax step
                    float tmx = z[0];
#pragma unroll
                    for (int e = 1; e < 16; ++e) tmx = fmaxf(tmx, z[e]);
                    tmx = fmaxf(tmx, __shfl_xor(tmx, 32));
                    const float mnew = fmaxf(smx, tmx);  // finite: the key block holds at least one live key
                    const float alpha = __builtin_amdgcn_exp2f((smx - mnew) * scale_log2e);  // 0 the first time
                    smx = mnew;
                    ssum *= alpha;
                    if (LSE) sesum *= alpha;
#pragma unroll
                    for (int e = 0; e < 16; ++e) so[e] *= alpha;
                } else {
                    smx = 0.0f;  // this wave met a key block: its part counts, with shift zero
                }
                weigh_into(wave, z, smx * scale_log2e, ssum, sesum, so);
            }
            if (t + 1 < ntiles) stash(t + 1, buf ^ 1);
            __syncthreads();
        }
    };
    walk(std::false_type{});
    {
        // one vote of the work-group: the second walk shares tiles and barriers, so all waves take it or none does
        const float whole = sum + __shfl_xor(sum, 32);
        bool fine = (whole >= 0x1p-60f && whole <= 0x1p60f) || cnt == 0 || wave * 32 >= NQ;  // false for NaN
        if (SPLIT) {
            const float part = ssum + __shfl_xor(ssum, 32);
            // a part may be empty (no key block met); one that is merely tiny next to the others also sends the
            // work-group to the second walk, which is always right
            fine = fine && ((part >= 0x1p-60f && part <= 0x1p60f) || smx == -INFINITY);
        }
        if (lane == 0) s_wcnt[wave] = __all(fine) ? 1 : 0;
        __syncthreads();
        bool redo = false;
#pragma unroll
        for (int w = 0; w < NW; ++w) redo = redo || s_wcnt[w] == 0;
        if (redo) {
            mx = -INFINITY, sum = 0.0f, esum = 0.0f, smx = -INFINITY, ssum = 0.0f, sesum = 0.0f;
#pragma unroll
            for (int e = 0; e < 16; ++e) o[e] = 0.0f, so[e] = 0.0f;
            walk(std::true_type{});
        } else {
            mx = 0.0f;
        }
    }
    sum += __shfl_xor(sum, 32);
    const float inv = cnt == 0 ? 0.0f : __builtin_amdgcn_rcpf(sum);
    // log2 of the sum over the keys of exp2(score * scale_log2e), for a backward pass that would otherwise recompute it
    // (meaningless for an environment without keys, which that pass does not read)
    float *lse_env = lse_out == nullptr ? nullptr : lse_out + ((int64_t)env * H + head) * NQ;
    if (LSE) {
        esum += __shfl_xor(esum, 32);
        if (lse_env != nullptr && qrow < NQ && half == 0) lse_env[qrow] = fmaf(mx, scale_log2e, __builtin_amdgcn_logf(esum));
    }

    if (SPLIT) {
        // Merge the four partial results of the shared block.  Every wave has passed the barrier of the last tile,
        // so the K buffers are free: o as [wave][e][lane], then maximum and sum as [wave][query].
        float *part = reinterpret_cast<float *>(&s_k[0][0]);
        float *stat = part + NW * 16 * kWave;
        ssum += __shfl_xor(ssum, 32);
        if (LSE) sesum += __shfl_xor(sesum, 32);
#pragma unroll
        for (int e = 0; e < 16; ++e) part[(wave * 16 + e) * kWave + lane] = so[e];
        if (half == 0) {
            stat[(wave * 3 + 0) * 32 + m] = smx;
            stat[(wave * 3 + 1) * 32 + m] = ssum;
            if (LSE) stat[(wave * 3 + 2) * 32 + m] = sesum;
        }
        __syncthreads();
        // wave w finishes accumulator registers 4w .. 4w+3 of the 32 queries: rows 8w + 4*half + 0..3 of V^T as it
        // lies in LDS, which the stash fills so that they are channels 16 (w / 2) + 8*half + 4 (w % 2) + 0..3
        float mall = -INFINITY;
#pragma unroll
        for (int j = 0; j < NW; ++j) mall = fmaxf(mall, stat[(j * 3 + 0) * 32 + m]);
        float total = 0.0f, etotal = 0.0f;
        float r[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < NW; ++j) {
            const float mj = stat[(j * 3 + 0) * 32 + m];
            // a wave that met no key block holds (-inf, 0, 0); with no key at all every part is like that
            const float f = mj == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f((mj - mall) * scale_log2e);
            total = fmaf(f, stat[(j * 3 + 1) * 32 + m], total);
            if (LSE) etotal = fmaf(f, stat[(j * 3 + 2) * 32 + m], etotal);
#pragma unroll
            for (int i = 0; i < 4; ++i) r[i] = fmaf(f, part[(j * 16 + wave * 4 + i) * kWave + lane], r[i]);
        }
        const float sinv = cnt == 0 ? 0.0f : __builtin_amdgcn_rcpf(total);
        if (LSE && lse_env != nullptr && wave == 0 && srow < NQ && half == 0)
            lse_env[srow] = fmaf(mall, scale_log2e, __builtin_amdgcn_logf(etotal));
        if (srow < NQ) {
            const int64_t at = ((int64_t)env * NQ + srow) * D + head * kDh + 16 * (wave >> 1) + 8 * half + 4 * (wave & 1);
#pragma unroll
            for (int i = 0; i < 4; ++i) r[i] *= sinv;
            if (accum != nullptr) {
                // bf16 + bf16 as torch adds them: the read result is rounded first, then the sum
                const u32x2 aw = *reinterpret_cast<const u32x2 *>(accum + at);
                r[0] = __uint_as_float(aw.x << 16) + round_to_bf16(r[0]);
                r[1] = __uint_as_float(aw.x & 0xffff0000u) + round_to_bf16(r[1]);
                r[2] = __uint_as_float(aw.y << 16) + round_to_bf16(r[2]);
                r[3] = __uint_as_float(aw.y & 0xffff0000u) + round_to_bf16(r[3]);
            }
            *reinterpret_cast<u32x2 *>(out + at) = u32x2{pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3])};
        }
    }

    {
        u32x4 w[2];
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            float r[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) r[e] = o[8 * g + e] * inv;
            if (accum != nullptr) {
                // bf16 + bf16 as torch adds them: the read result is rounded first, then the sum
                const u32x4 aw = g ? acc1 : acc0;
                const uint32_t a2[4] = {aw.x, aw.y, aw.z, aw.w};
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float a = __uint_as_float((e & 1) ? (a2[e >> 1] & 0xffff0000u) : (a2[e >> 1] << 16));
                    r[e] = a + round_to_bf16(r[e]);
                }
            }
            w[g] = u32x4{pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3]), pack_bf16x2(r[4], r[5]), pack_bf16x2(r[6], r[7])};
        }
        // whole 64-byte head rows per store instruction (lanes m and m + 16 trade runs, see sdpa_mfma_kernel)
#pragma unroll
        for (int cdw = 0; cdw < 4; ++cdw) {
            const u32x2 t = __builtin_amdgcn_permlane16_swap(w[0][cdw], w[1][cdw], false, false);
            w[0][cdw] = t.x, w[1][cdw] = t.y;
        }
        const int row_a = wave * 32 + (m & 15);
        const int ch = head * kDh + 16 * (m >> 4) + 8 * half;
        if (row_a < NQ) *reinterpret_cast<u32x4 *>(out + ((int64_t)env * NQ + row_a) * D + ch) = w[0];
        if (row_a + 16 < NQ) *reinterpret_cast<u32x4 *>(out + ((int64_t)env * NQ + row_a + 16) * D + ch) = w[1];
    }
}

// ------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------

constexpr size_t kLdsDefault = 64 * 1024;
constexpr size_t kLdsMax = 160 * 1024;

static size_t valu_lds_bytes(int G, int NM, int nh, int DH)
{
    const size_t env_pitch = (size_t)NM * nh * (DH + kValuHeadPad) + kValuEnvPad;
    return 2 * (size_t)G * env_pitch * sizeof(float) + (((size_t)G * NM + 15) & ~(size_t)15) + (size_t)G * sizeof(int);
}

template <typename T, int DH>
static int launch_valu(const void *qkv, int64_t row_stride, const uint8_t *alive, void *out, int B, int NM,
                       int H, hipStream_t stream)
{
    // all heads of an environment in one block when they fit, else one head per block
    int nh = H;
    if (valu_lds_bytes(1, NM, H, DH) > kLdsDefault) nh = 1;
    int G = kValuThreads / (nh * NM);
    if (G < 1) G = 1;
    if (G > 8) G = 8;
    while (G > 1 && valu_lds_bytes(G, NM, nh, DH) > kLdsDefault) --G;
    if (G > B) G = B;
    // small batches: fewer environments per block so that every CU still gets several blocks
    while (G > 1 && (int64_t)((B + G - 1) / G) * (H / nh) < 1024) --G;
    int threads = (G * nh * NM + kWave - 1) / kWave * kWave;
    if (threads > kValuThreads) threads = kValuThreads;
    const size_t lds = valu_lds_bytes(G, NM, nh, DH);
    if (lds > kLdsMax) return BNB_ERR_UNSUPPORTED;
    auto kernel = sdpa_valu_kernel<T, DH>;
    if (lds > kLdsDefault) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsMax);
        if (e != hipSuccess) return (int)e;
    }
    const dim3 grid((unsigned)((B + G - 1) / G), (unsigned)(H / nh));
    const float scale_log2e = kLog2eA / sqrtf((float)DH);
    hipLaunchKernelGGL(kernel, grid, dim3(threads), lds, stream, (const T *)qkv, row_stride, alive,
                       (T *)out, B, NM, H, G, nh, scale_log2e);
    return (int)hipGetLastError();
}

template <typename T>
static int dispatch_valu(const void *qkv, int64_t row_stride, const uint8_t *alive, void *out, int B, int NM,
                         int H, int dh, hipStream_t stream)
{
    switch (dh) {
        case 8: return launch_valu<T, 8>(qkv, row_stride, alive, out, B, NM, H, stream);
        case 16: return launch_valu<T, 16>(qkv, row_stride, alive, out, B, NM, H, stream);
        case 32: return launch_valu<T, 32>(qkv, row_stride, alive, out, B, NM, H, stream);
        case 64: return launch_valu<T, 64>(qkv, row_stride, alive, out, B, NM, H, stream);
        default: return BNB_ERR_UNSUPPORTED;
    }
}

template <int NKB, bool CROSS>
static int launch_mfma(const void *q, int64_t q_stride, const void *k, const void *v, int64_t kv_stride,
                       const uint8_t *alive, const void *accum, void *out, int B, int NQ, int NK, int H,
                       hipStream_t stream)
{
    const int64_t pairs = (int64_t)B * H;
    const int64_t blocks = (pairs + 7) / 8 * 8;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    const float scale_log2e = kLog2eA / sqrtf((float)kDh);
    hipLaunchKernelGGL((sdpa_mfma_kernel<NKB, CROSS>), dim3((unsigned)blocks), dim3(kWave * NKB), 0, stream,
                       (const uint16_t *)q, q_stride, (const uint16_t *)k, (const uint16_t *)v, kv_stride, alive,
                       (const uint16_t *)accum, (uint16_t *)out, B, NQ, NK, H, scale_log2e);
    return (int)hipGetLastError();
}

template <bool CROSS>
static int dispatch_mfma(const void *q, int64_t q_stride, const void *k, const void *v, int64_t kv_stride,
                         const uint8_t *alive, const void *accum, void *out, int B, int NQ, int NK, int H,
                         hipStream_t stream)
{
    const int blocks = ((NQ > NK ? NQ : NK) + 31) / 32;
    switch (blocks) {
        case 1: return launch_mfma<1, CROSS>(q, q_stride, k, v, kv_stride, alive, accum, out, B, NQ, NK, H, stream);
        case 2: return launch_mfma<2, CROSS>(q, q_stride, k, v, kv_stride, alive, accum, out, B, NQ, NK, H, stream);
        case 3: return launch_mfma<3, CROSS>(q, q_stride, k, v, kv_stride, alive, accum, out, B, NQ, NK, H, stream);
        case 4: return launch_mfma<4, CROSS>(q, q_stride, k, v, kv_stride, alive, accum, out, B, NQ, NK, H, stream);
        case 5: return launch_mfma<5, CROSS>(q, q_stride, k, v, kv_stride, alive, accum, out, B, NQ, NK, H, stream);
        default: return BNB_ERR_UNSUPPORTED;
    }
}

template <int NQB>
static int launch_cross_stream(const void *q, int64_t q_stride, const void *k, const void *v, int64_t kv_stride,
                               const uint8_t *alive, const int32_t *ranges, const void *accum, void *out, float *lse, int B,
                               int NQ, int NK, int H, hipStream_t stream)
{
    const int64_t pairs = (int64_t)B * H;
    const int64_t blocks = (pairs + 7) / 8 * 8;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    const float scale_log2e = kLog2eA / sqrtf((float)kDh);
    // the log-sum-exp (asked for by the update's forward) costs sixteen additions per key block: a form of its own
    if (lse != nullptr)
        hipLaunchKernelGGL((sdpa_cross_stream_kernel<NQB, true>), dim3((unsigned)blocks), dim3(kWave * (NQB < 4 ? NQB : 4)), 0,
                           stream, (const uint16_t *)q, q_stride, (const uint16_t *)k, (const uint16_t *)v, kv_stride, alive,
                           ranges, (const uint16_t *)accum, (uint16_t *)out, lse, B, NQ, NK, H, scale_log2e);
    else
        hipLaunchKernelGGL((sdpa_cross_stream_kernel<NQB, false>), dim3((unsigned)blocks), dim3(kWave * (NQB < 4 ? NQB : 4)), 0,
                           stream, (const uint16_t *)q, q_stride, (const uint16_t *)k, (const uint16_t *)v, kv_stride, alive,
                           ranges, (const uint16_t *)accum, (uint16_t *)out, lse, B, NQ, NK, H, scale_log2e);
    return (int)hipGetLastError();
}

static int dispatch_cross_stream(const void *q, int64_t q_stride, const void *k, const void *v, int64_t kv_stride,
                                 const uint8_t *alive, const int32_t *ranges, const void *accum, void *out, float *lse,
                                 int B, int NQ, int NK, int H, hipStream_t stream)
{
    switch ((NQ + 31) / 32) {
        case 1: return launch_cross_stream<1>(q, q_stride, k, v, kv_stride, alive, ranges, accum, out, lse, B, NQ, NK, H, stream);
        case 2: return launch_cross_stream<2>(q, q_stride, k, v, kv_stride, alive, ranges, accum, out, lse, B, NQ, NK, H, stream);
        case 3: return launch_cross_stream<3>(q, q_stride, k, v, kv_stride, alive, ranges, accum, out, lse, B, NQ, NK, H, stream);
        case 4: return launch_cross_stream<4>(q, q_stride, k, v, kv_stride, alive, ranges, accum, out, lse, B, NQ, NK, H, stream);
        case 5: return launch_cross_stream<5>(q, q_stride, k, v, kv_stride, alive, ranges, accum, out, lse, B, NQ, NK, H, stream);
        default: return BNB_ERR_UNSUPPORTED;
    }
}

// defined in sdpa_env.hip: bf16, 4 heads of 32 channels, NM <= 160, one work-group per environment
int dispatch_env(const void *qkv, int64_t stride, const uint8_t *alive, void *out, int B, int NM, hipStream_t stream);

// defined in sdpa_env.hip: bf16, heads of 32 channels, NM <= 160, one work-group per (environment, head), rows straight into LDS
int dispatch_head(const void *qkv, int64_t stride, const uint8_t *alive, void *out, int B, int NM, int H, hipStream_t stream);

// defined in sdpa_cross_f32.hip
int launch_cross_f32(const void *q, int64_t q_stride, const void *k, const void *v, int64_t kv_stride, const uint8_t *key_mask,
                     const void *accum, void *out, int B, int NQ, int NK, int H, hipStream_t stream);

}  // namespace bnb

extern "C" int bnb_sdpa_masked_fwd_path(const void *qkv, int64_t qkv_row_stride, const uint8_t *alive,
                                        void *out, int B, int NM, int H, int dh, int dtype, int path,
                                        void *stream)
{
    using namespace bnb;
    if (B < 0 || NM < 0 || H < 1 || dh < 1) return BNB_ERR_BAD_SHAPE;
    if (dtype != BNB_F32 && dtype != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (path < BNB_SDPA_PATH_AUTO || path > BNB_SDPA_PATH_HEAD) return BNB_ERR_UNSUPPORTED;
    if (B == 0 || NM == 0) return 0;
    if (!qkv || !out) return BNB_ERR_NULL_POINTER;
    if (qkv_row_stride < (int64_t)3 * H * dh) return BNB_ERR_BAD_SHAPE;
    if (NM > 512) return BNB_ERR_UNSUPPORTED;
    const size_t esize = dtype == BNB_BF16 ? 2 : 4;
    if (!aligned16(qkv) || !aligned16(out) || (qkv_row_stride * esize) % 16 != 0) return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;

    // the matrix-core kernel addresses rows inside one environment with 32-bit offsets
    const bool mfma_ok = dtype == BNB_BF16 && dh == kDh && NM <= 160 && (int64_t)NM * qkv_row_stride < (1LL << 30);
    if (path == BNB_SDPA_PATH_MFMA && !mfma_ok) return BNB_ERR_UNSUPPORTED;
    // one work-group per environment, rows straight into LDS: four heads only, byte offsets inside an environment in 32 bits
    const bool env_ok = mfma_ok && H == 4 && (int64_t)NM * qkv_row_stride < (1LL << 30);
    if (path == BNB_SDPA_PATH_ENV && !env_ok) return BNB_ERR_UNSUPPORTED;
    if (path == BNB_SDPA_PATH_ENV)
        return dispatch_env(qkv, qkv_row_stride, alive, out, B, NM, s);
    if (path == BNB_SDPA_PATH_HEAD && !mfma_ok) return BNB_ERR_UNSUPPORTED;
    if (path == BNB_SDPA_PATH_HEAD) return dispatch_head(qkv, qkv_row_stride, alive, out, B, NM, H, s);
    // measured on MI355X the matrix-core kernel wins at every token count it covers, 4v4 included
    // (12 tokens: 24.7 us vs 45.5 us for 8192 environments), so AUTO takes it whenever it applies
    const bool use_mfma = path == BNB_SDPA_PATH_MFMA || (path == BNB_SDPA_PATH_AUTO && mfma_ok);
    if (use_mfma && NM <= 16 && (H & 1) == 0) {
        // two heads per wave: 23.4 us vs 28.5 us for the one-head form at 12 tokens x 8192 environments
        const int64_t pairs = (int64_t)B * (H / 2);
        const int64_t blocks = (pairs + 7) / 8 * 8;
        if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
        hipLaunchKernelGGL(sdpa_mfma_pair_kernel, dim3((unsigned)blocks), dim3(kWave), 0, s, (const uint16_t *)qkv,
                           qkv_row_stride, alive, (uint16_t *)out, B, NM, H, kLog2eA / sqrtf((float)kDh));
        return (int)hipGetLastError();
    }
    if (use_mfma) {
        const uint16_t *base = (const uint16_t *)qkv;
        const int D = H * dh;
        return dispatch_mfma<false>(base, qkv_row_stride, base + D, base + 2 * D, qkv_row_stride, alive, nullptr, out,
                                    B, NM, NM, H, s);
    }
    if (dtype == BNB_BF16) return dispatch_valu<uint16_t>(qkv, qkv_row_stride, alive, out, B, NM, H, dh, s);
    // fp32, head size 32: the fp32 matrix-core kernel (no slower at 12 tokens, and measured against the
    // vector kernel at 1024 environments: 84 tokens 129 -> 51 us, 160 tokens 404 -> 139 us, 320 tokens x 256
    // environments 855 -> 132 us); taken by AUTO, the VALU path stays the vector kernel
    if (dh == kDh && NM > 0 && path != BNB_SDPA_PATH_VALU && (int64_t)NM * qkv_row_stride < (1LL << 31)) {
        const int nwaves = (NM + 31) / 32;
        const size_t lds = (size_t)nwaves * 32 * (kF32KeyPitch + kDh) * sizeof(float) + (size_t)2 * nwaves * sizeof(int);
        if (lds <= kLdsMax) {
            const int64_t pairs = (int64_t)B * H;
            const int64_t blocks = (pairs + 7) / 8 * 8;
            if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
            if (lds > kLdsDefault) {
                const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(sdpa_mfma_f32_kernel),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsMax);
                if (e != hipSuccess) return (int)e;
            }
            hipLaunchKernelGGL(sdpa_mfma_f32_kernel, dim3((unsigned)blocks), dim3(nwaves * kWave), lds, s,
                               (const float *)qkv, qkv_row_stride, alive, (float *)out, B, NM, H,
                               kLog2eA / sqrtf((float)kDh));
            return (int)hipGetLastError();
        }
    }
    return dispatch_valu<float>(qkv, qkv_row_stride, alive, out, B, NM, H, dh, s);
}

extern "C" int bnb_sdpa_masked_fwd(const void *qkv, int64_t qkv_row_stride, const uint8_t *alive, void *out,
                                   int B, int NM, int H, int dh, int dtype, void *stream)
{
    return bnb_sdpa_masked_fwd_path(qkv, qkv_row_stride, alive, out, B, NM, H, dh, dtype, BNB_SDPA_PATH_AUTO,
                                    stream);
}

extern "C" int bnb_sdpa_cross_fwd(const void *q, int64_t q_row_stride, int NQ, const void *k, const void *v,
                                  int64_t kv_row_stride, int NK, const uint8_t *key_mask, const void *accum,
                                  void *out, int B, int H, int dh, int dtype, void *stream)
{
    using namespace bnb;
    if (B < 0 || NQ < 0 || NK < 0 || H < 1 || dh < 1) return BNB_ERR_BAD_SHAPE;
    if (dtype != BNB_BF16 && dtype != BNB_F32) return BNB_ERR_BAD_DTYPE;
    if (dh != kDh || NK == 0) return BNB_ERR_UNSUPPORTED;  // NK == 0: nothing to read, the caller keeps `accum` as it is
    if (dtype == BNB_F32) {
        if (NQ > 512 || NK > 4096) return BNB_ERR_UNSUPPORTED;
        if (B == 0 || NQ == 0) return 0;
        if (!q || !out || !k || !v) return BNB_ERR_NULL_POINTER;
        if (q_row_stride < (int64_t)H * dh || kv_row_stride < (int64_t)H * dh) return BNB_ERR_BAD_SHAPE;
        if (!aligned16(q) || !aligned16(out) || (accum && !aligned16(accum)) || (q_row_stride * 4) % 16 != 0 || !aligned16(k) ||
            !aligned16(v) || (kv_row_stride * 4) % 16 != 0)
            return BNB_ERR_MISALIGNED;
        return launch_cross_f32(q, q_row_stride, k, v, kv_row_stride, key_mask, accum, out, B, NQ, NK, H, (hipStream_t)stream);
    }
    if (NQ > 160 || NK > kStreamMaxKeys) return BNB_ERR_UNSUPPORTED;
    if (B == 0 || NQ == 0) return 0;
    if (!q || !out || !k || !v) return BNB_ERR_NULL_POINTER;
    if (q_row_stride < (int64_t)H * dh || kv_row_stride < (int64_t)H * dh) return BNB_ERR_BAD_SHAPE;
    if ((int64_t)NQ * q_row_stride >= (1LL << 30) || (int64_t)NK * kv_row_stride >= (1LL << 30))
        return BNB_ERR_UNSUPPORTED;
    if (!aligned16(q) || !aligned16(out) || (accum && !aligned16(accum)) || (q_row_stride * 2) % 16 != 0 ||
        !aligned16(k) || !aligned16(v) || (kv_row_stride * 2) % 16 != 0)
        return BNB_ERR_MISALIGNED;
    if (NK > 160)
        return dispatch_cross_stream(q, q_row_stride, k, v, kv_row_stride, key_mask, nullptr, accum, out, nullptr, B, NQ, NK,
                                     H, (hipStream_t)stream);
    return dispatch_mfma<true>(q, q_row_stride, k, v, kv_row_stride, key_mask, accum, out, B, NQ, NK, H,
                               (hipStream_t)stream);
}

namespace bnb {
static int cross_ranges_fwd(const void *q, int64_t q_row_stride, int NQ, const void *kv_rows, int64_t kv_row_stride,
                            const int32_t *ranges, int64_t kv_capacity, const void *accum, void *out, float *lse, int B, int H,
                            int dh, int dtype, void *stream)
{
    if (B < 0 || NQ < 0 || H < 1 || dh < 1 || kv_capacity < 0) return BNB_ERR_BAD_SHAPE;
    if (dtype != BNB_BF16 || dh != kDh || NQ > 160) return BNB_ERR_UNSUPPORTED;
    if (B == 0 || NQ == 0) return 0;
    if (!q || !out || !kv_rows || !ranges) return BNB_ERR_NULL_POINTER;
    if (q_row_stride < (int64_t)H * dh || kv_row_stride < (int64_t)2 * H * dh) return BNB_ERR_BAD_SHAPE;
    // rows inside an environment (q) and inside the whole list (kv) are addressed with 32-bit offsets
    if ((int64_t)NQ * q_row_stride >= (1LL << 30) || kv_capacity * kv_row_stride >= (1LL << 32))
        return BNB_ERR_UNSUPPORTED;
    if (!aligned16(q) || !aligned16(out) || (accum && !aligned16(accum)) || (q_row_stride * 2) % 16 != 0 ||
        !aligned16(kv_rows) || (kv_row_stride * 2) % 16 != 0 || (reinterpret_cast<uintptr_t>(ranges) & 3u))
        return BNB_ERR_MISALIGNED;
    const uint16_t *kp = (const uint16_t *)kv_rows;
    return dispatch_cross_stream(q, q_row_stride, kp, kp + (int64_t)H * dh, kv_row_stride, nullptr, ranges, accum, out, lse,
                                 B, NQ, 0, H, (hipStream_t)stream);
}
}  // namespace bnb

extern "C" int bnb_sdpa_cross_ranges_fwd(const void *q, int64_t q_row_stride, int NQ, const void *kv_rows,
                                         int64_t kv_row_stride, const int32_t *ranges, int64_t kv_capacity,
                                         const void *accum, void *out, int B, int H, int dh, int dtype,
                                         void *stream)
{
    return bnb::cross_ranges_fwd(q, q_row_stride, NQ, kv_rows, kv_row_stride, ranges, kv_capacity, accum, out, nullptr, B, H, dh,
                                 dtype, stream);
}

extern "C" int bnb_sdpa_cross_ranges_fwd_lse(const void *q, int64_t q_row_stride, int NQ, const void *kv_rows,
                                             int64_t kv_row_stride, const int32_t *ranges, int64_t kv_capacity,
                                             const void *accum, void *out, float *lse, int B, int H, int dh, int dtype,
                                             void *stream)
{
    if (lse == nullptr && B > 0 && NQ > 0) return BNB_ERR_NULL_POINTER;
    if (reinterpret_cast<uintptr_t>(lse) & 3u) return BNB_ERR_MISALIGNED;
    return bnb::cross_ranges_fwd(q, q_row_stride, NQ, kv_rows, kv_row_stride, ranges, kv_capacity, accum, out, lse, B, H, dh,
                                 dtype, stream);
}
