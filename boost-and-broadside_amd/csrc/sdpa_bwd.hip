// Backward of the masked multi-head attention over each environment's tokens, for gfx950, for the
// small token counts the PPO update runs at (4v4: 12 tokens, 8v11: 27 tokens) with head size 32.
//
// Reference: what autograd computes through models/yemong/attention.py:136-147 (head split, additive
// key bias finfo.min/2 on dead keys, scaled_dot_product_attention, head merge) during
// train/rl/ppo.py:1417-1425.  With S = Q K^T / sqrt(dh) + bias, P = softmax(S), O = P V:
//   dV = P^T dO,  dP = dO V^T,  dS = P * (dP - rowsum(dO * O)),  dQ = dS K / sqrt(dh),  dK = dS^T Q / sqrt(dh).
// The library runs this as head-split copies, a bias tensor and a generic fused kernel sized for
// long sequences (629 us for 32,768 environments of 12 tokens, against ~90 us for the tensors to
// cross HBM once).  Here the problem is so small per environment that plain vector FMAs are enough:
//   * a work-group holds a few environments, one thread per (token, head);
//   * phase 1, thread = (query i, head): K and V of the environment sit in LDS (fp32, heads 36 floats
//     apart so the four heads of a wave hit different banks), Q_i, dO_i in registers; scores, the
//     softmax, dP and dS for all keys, dQ_i accumulated in registers; P and dS/sqrt(dh) are left in LDS;
//   * phase 2, thread = (key j, head): Q and dO of the environment take K and V's place in LDS;
//     dK_j and dV_j are sums over the queries of P, dS (LDS) times Q_i, dO_i (LDS).
// Every sum runs in a fixed order.  Dead keys have P = 0 exactly, so they receive zero dK and dV; an
// environment without a live key has P = 1/NM for all keys, as the bias makes it in the reference.
// Bound: vector ALU (160 * NM FMAs per thread); HBM traffic is qkv, O, dO in and dqkv out, once.

#include "common.h"

namespace bnb {

constexpr int kSbDh = 32;          // head size
constexpr int kSbHeadPitch = 36;   // floats between heads of one LDS row
constexpr int kSbMaxTokens = 32;
constexpr int kSbMfmaFrom = 11;  // AUTO: the matrix-core kernel above this many tokens (bf16); below, the vector kernel is as fast
constexpr int kSbLdsBudget = 78 * 1024;  // two work-groups per CU

struct SbShape {
    int threads_per_env, envs_per_block, threads, row_pitch, env_floats;
    size_t lds_bytes;
};

static SbShape sb_shape(int NM, int H)
{
    SbShape s;
    s.threads_per_env = NM * H;
    s.row_pitch = 2 * H * kSbHeadPitch;
    s.env_floats = (NM * s.row_pitch + 2 * H * NM * NM + 3) / 4 * 4;
    int e = 256 / s.threads_per_env;
    const int by_lds = kSbLdsBudget / (int)(s.env_floats * sizeof(float));
    if (e > by_lds) e = by_lds;
    if (e < 1) e = 1;
    s.envs_per_block = e;
    s.threads = (e * s.threads_per_env + 63) / 64 * 64;
    s.lds_bytes = (size_t)e * s.env_floats * sizeof(float);
    return s;
}

template <typename T>
__device__ __forceinline__ void load_head(const T *p, float (&dst)[kSbDh])
{
#pragma unroll
    for (int c = 0; c < kSbDh / 8; ++c) {
        const Row8 r = load8(p + 8 * c);
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[8 * c + e] = r.v[e];
    }
}

template <typename T>
__device__ __forceinline__ void store_head(T *p, const float (&src)[kSbDh])
{
#pragma unroll
    for (int c = 0; c < kSbDh / 8; ++c) {
        Row8 r;
#pragma unroll
        for (int e = 0; e < 8; ++e) r.v[e] = src[8 * c + e];
        store8(p + 8 * c, r);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void sdpa_bwd_small_kernel(
    const T *__restrict__ qkv, int64_t qkv_row_stride, const uint8_t *__restrict__ alive, const T *__restrict__ out,
    const T *__restrict__ dout, T *__restrict__ dqkv, int64_t B, int NM, int H, int envs_per_block, int row_pitch,
    int env_floats, float scale)
{
    extern __shared__ __align__(16) float sb_lds[];
    const int D = H * kSbDh;
    const int threads_per_env = NM * H;
    const int e = threadIdx.x / threads_per_env;
    const int local = threadIdx.x - e * threads_per_env;
    const int64_t env = (int64_t)blockIdx.x * envs_per_block + e;
    const bool active = e < envs_per_block && env < B;
    const int i = local / H, h = local - i * H;  // token, head

    float *rows = sb_lds + (active ? e : 0) * env_floats;  // [NM][K: H x 36 | V: H x 36], later [Q | dO]
    float *pbuf = rows + NM * row_pitch;                    // [H][NM][NM]: scores, then P
    float *dsbuf = pbuf + H * NM * NM;                      // [H][NM][NM]: dS / sqrt(dh)
    const float scale_log2e = scale * 1.4426950408889634f;

    float q[kSbDh], go[kSbDh];
    float delta = 0.0f;
    uint32_t live = 0;
    if (active) {
        const int64_t tok = env * NM + i;
        load_head(qkv + tok * qkv_row_stride + h * kSbDh, q);
        load_head(dout + tok * D + h * kSbDh, go);
        float o[kSbDh];
        load_head(out + tok * D + h * kSbDh, o);
#pragma unroll
        for (int d = 0; d < kSbDh; ++d) delta = fmaf(go[d], o[d], delta);
        if (alive != nullptr) {
            for (int j = 0; j < NM; ++j) live |= (alive[env * NM + j] != 0 ? 1u : 0u) << j;
        } else {
            live = 0xffffffffu;
        }
        // K and V of the environment into LDS: piece c of a row = 8 channels of [K | V]
        const int pieces_per_row = 2 * D / 8;
        for (int p = local; p < NM * pieces_per_row; p += threads_per_env) {
            const int row = p / pieces_per_row, c = p - row * pieces_per_row;
            const int ch = 8 * c;  // channel within [K | V]
            const int operand = ch / D, within = ch - operand * D;
            const Row8 r = load8(qkv + (env * NM + row) * qkv_row_stride + D + ch);
            float *dst = rows + row * row_pitch + operand * H * kSbHeadPitch + (within / kSbDh) * kSbHeadPitch + (within % kSbDh);
            *reinterpret_cast<f32x4 *>(dst) = f32x4{r.v[0], r.v[1], r.v[2], r.v[3]};
            *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{r.v[4], r.v[5], r.v[6], r.v[7]};
        }
    }
    __syncthreads();

    const bool none_live = live == 0 || (NM < 32 && (live & ((1u << NM) - 1u)) == 0);
    if (active) {
        if (none_live) live = 0xffffffffu;  // equal biases on every key: the plain softmax over all keys
        float *srow = pbuf + (h * NM + i) * NM;
        float *dsrow = dsbuf + (h * NM + i) * NM;
        // scores (log2 domain) and their maximum over the live keys
        float m = -INFINITY;
        for (int j = 0; j < NM; ++j) {
            const float *kj = rows + j * row_pitch + h * kSbHeadPitch;
            float s = 0.0f;
#pragma unroll
            for (int d = 0; d < kSbDh; d += 4) {
                const f32x4 k4 = *reinterpret_cast<const f32x4 *>(kj + d);
                s = fmaf(q[d], k4.x, s), s = fmaf(q[d + 1], k4.y, s), s = fmaf(q[d + 2], k4.z, s), s = fmaf(q[d + 3], k4.w, s);
            }
            s = none_live ? 0.0f : s * scale_log2e;
            srow[j] = s;
            if ((live >> j) & 1u) m = fmaxf(m, s);
        }
        float l = 0.0f;
        for (int j = 0; j < NM; ++j) {
            const float pe = ((live >> j) & 1u) ? __builtin_amdgcn_exp2f(srow[j] - m) : 0.0f;
            srow[j] = pe;
            l += pe;
        }
        const float inv_l = 1.0f / l;
        float dq[kSbDh];
#pragma unroll
        for (int d = 0; d < kSbDh; ++d) dq[d] = 0.0f;
        for (int j = 0; j < NM; ++j) {
            const float *kj = rows + j * row_pitch + h * kSbHeadPitch;
            const float *vj = kj + H * kSbHeadPitch;
            const float p = srow[j] * inv_l;
            float dp = 0.0f;
#pragma unroll
            for (int d = 0; d < kSbDh; d += 4) {
                const f32x4 v4 = *reinterpret_cast<const f32x4 *>(vj + d);
                dp = fmaf(go[d], v4.x, dp), dp = fmaf(go[d + 1], v4.y, dp), dp = fmaf(go[d + 2], v4.z, dp), dp = fmaf(go[d + 3], v4.w, dp);
            }
            const float ds = p * (dp - delta) * scale;
#pragma unroll
            for (int d = 0; d < kSbDh; d += 4) {
                const f32x4 k4 = *reinterpret_cast<const f32x4 *>(kj + d);
                dq[d] = fmaf(ds, k4.x, dq[d]), dq[d + 1] = fmaf(ds, k4.y, dq[d + 1]);
                dq[d + 2] = fmaf(ds, k4.z, dq[d + 2]), dq[d + 3] = fmaf(ds, k4.w, dq[d + 3]);
            }
            srow[j] = p;
            dsrow[j] = ds;
        }
        store_head(dqkv + (env * NM + i) * 3 * (int64_t)D + h * kSbDh, dq);
    }
    __syncthreads();  // everyone is done with K and V

    if (active) {
        float *mine = rows + i * row_pitch + h * kSbHeadPitch;
#pragma unroll
        for (int d = 0; d < kSbDh; d += 4) {
            *reinterpret_cast<f32x4 *>(mine + d) = f32x4{q[d], q[d + 1], q[d + 2], q[d + 3]};
            *reinterpret_cast<f32x4 *>(mine + H * kSbHeadPitch + d) = f32x4{go[d], go[d + 1], go[d + 2], go[d + 3]};
        }
    }
    __syncthreads();

    if (active) {
        // this thread is now (key j = i, head h)
        float dk[kSbDh], dvv[kSbDh];
#pragma unroll
        for (int d = 0; d < kSbDh; ++d) dk[d] = dvv[d] = 0.0f;
        for (int qi = 0; qi < NM; ++qi) {
            const float p = pbuf[(h * NM + qi) * NM + i];
            const float ds = dsbuf[(h * NM + qi) * NM + i];
            const float *qr = rows + qi * row_pitch + h * kSbHeadPitch;
            const float *gr = qr + H * kSbHeadPitch;
#pragma unroll
            for (int d = 0; d < kSbDh; d += 4) {
                const f32x4 q4 = *reinterpret_cast<const f32x4 *>(qr + d);
                const f32x4 g4 = *reinterpret_cast<const f32x4 *>(gr + d);
                dk[d] = fmaf(ds, q4.x, dk[d]), dk[d + 1] = fmaf(ds, q4.y, dk[d + 1]);
                dk[d + 2] = fmaf(ds, q4.z, dk[d + 2]), dk[d + 3] = fmaf(ds, q4.w, dk[d + 3]);
                dvv[d] = fmaf(p, g4.x, dvv[d]), dvv[d + 1] = fmaf(p, g4.y, dvv[d + 1]);
                dvv[d + 2] = fmaf(p, g4.z, dvv[d + 2]), dvv[d + 3] = fmaf(p, g4.w, dvv[d + 3]);
            }
        }
        T *dst = dqkv + (env * NM + i) * 3 * (int64_t)D + h * kSbDh;
        store_head(dst + D, dk);
        store_head(dst + 2 * D, dvv);
    }
}

template <typename T>
static int launch_sdpa_bwd(const void *qkv, int64_t qkv_row_stride, const uint8_t *alive, const void *out, const void *dout,
                           void *dqkv, int64_t B, int NM, int H, hipStream_t stream)
{
    const SbShape s = sb_shape(NM, H);
    const int64_t blocks = (B + s.envs_per_block - 1) / s.envs_per_block;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    if (s.lds_bytes > 64 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_bwd_small_kernel<T>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)s.lds_bytes);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL((sdpa_bwd_small_kernel<T>), dim3((unsigned)blocks), dim3(s.threads), s.lds_bytes, stream, (const T *)qkv,
                       qkv_row_stride, alive, (const T *)out, (const T *)dout, (T *)dqkv, B, NM, H, s.envs_per_block, s.row_pitch,
                       s.env_floats, 1.0f / sqrtf((float)kSbDh));
    return (int)hipGetLastError();
}

// ------------------------------------------------------------------------------------
// bf16 on the matrix cores, up to 160 tokens
// ------------------------------------------------------------------------------------
//
// One work-group per (environment, head), one wave per block of 32 tokens.  Nothing is reduced
// across waves: the products are formed twice, once per orientation.
//   pass 0/1, wave = query block: S^T = K Q^T per key block (rows = keys, lane = query), row
//     maximum and sum as in the forward kernel, L = log2-sum-exp and delta = rowsum(dO * O) per
//     query (kept in LDS for pass 2); then P^T = exp2(S^T c - L), dP^T = V dO^T,
//     dS^T = P^T (dP^T - delta) / sqrt(dh), and dQ^T += K^T dS^T with dS^T going from the
//     accumulator registers straight into the B operand (the key order of the A operand, read
//     from a transposed copy of K in LDS, follows the accumulator's row order);
//   pass 2, wave = key block: S = Q K^T per query block (rows = queries, lane = key), P and dS from
//     the per-query L and delta, dK^T += Q^T dS and dV^T += dO^T P the same way (transposed
//     copies of Q and dO in LDS).
// K, V (pass 1) and Q, dO (pass 2) share the same LDS.  Dead and padding keys enter as -inf in the
// accumulator (P = 0 exactly); an environment without a live key uses zero scores over all its keys.
// P and dS are rounded to bf16 for the second product of each pair, as the operands of the forward
// kernel's second product are.

constexpr int kMbPitch = kSbDh + 8;  // halfs per token row in LDS (80 bytes: 16-byte aligned, bank-spread)

// NB = blocks of 32 tokens on the longer of the two axes (waves of the work-group).  CROSS: the keys and
// values come from a second buffer kv (B, NK, 2*H*32) with its own mask (the bullet read,
// models/yemong/attention.py:149-166): an environment without a live key contributed exactly nothing
// in the forward (the reference gates it off), so all its gradients are zero; `out` is that read's own
// result, before it was added to anything.
// PAIR (NB = 1, up to 16 tokens, an even number of heads): two heads of one environment share the tile, as
// in the forward kernel for small fleets.  Row r of every staged operand is token r % 16 of head
// 2 * pair + r / 16, and the score blocks between the two heads start at -inf like a dead key, so P and
// dS are exactly zero there and every second product returns each head's gradient in its own columns.
template <int NB, bool CROSS, bool PAIR>
__global__ __launch_bounds__(kWave * NB) __attribute__((amdgpu_waves_per_eu(NB == 1 && !PAIR ? 3 : 4))) void sdpa_bwd_mfma_kernel(
    const uint16_t *__restrict__ q, int64_t q_row_stride, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,
    int64_t kv_row_stride, const uint8_t *__restrict__ alive, const int32_t *__restrict__ ranges, int64_t kv_capacity,
    const uint16_t *__restrict__ out, const uint16_t *__restrict__ dout, uint16_t *__restrict__ dq_out, int64_t dq_row_stride,
    uint16_t *__restrict__ dk_out, uint16_t *__restrict__ dv_out, int64_t dkv_row_stride, int B, int NQ, int NK_all, int H,
    float scale)
{
    constexpr int CAP = NB * 32;
    constexpr int TP = CAP + 4;  // halfs per row of a transposed copy
    constexpr int NT = kWave * NB;
    // with one block of 32 tokens a lane's own rows (loaded below for the other orientation) are the
    // token-major operands too, so no token-major copy is staged
    constexpr bool OWN_ROWS = NB == 1;
    __shared__ __align__(16) uint16_t s_rows[2][OWN_ROWS ? 8 : CAP * kMbPitch];  // [K | V], later [Q | dO]: token-major
    __shared__ __align__(16) uint16_t s_tr[2][kSbDh * TP];        // K^T, later [Q^T | dO^T]: channel-major
    __shared__ __align__(16) float s_lse[CAP], s_delta[CAP];
    __shared__ __align__(16) float s_bias[CAP];  // 0 for a key that takes part, -inf for a dead or padding key

    const int chunk = gridDim.x >> 3;
    const int logical = (blockIdx.x & 7) * chunk + (blockIdx.x >> 3);  // the heads of an environment on one XCD
    const int per_env = PAIR ? H >> 1 : H;  // work-groups per environment
    if (logical >= B * per_env) return;
    const int env = logical / per_env, head = (logical - env * per_env) * (PAIR ? 2 : 1);  // PAIR: the first head of the pair
    const int D = H * kSbDh;
    static_assert(!PAIR || (NB == 1 && !CROSS), "two heads share one 32 x 32 tile of self-attention");
    // tile row -> (token, first channel of its head)
    auto tok_of = [&](int r) { return PAIR ? r & 15 : r; };
    auto ch_of = [&](int r) { return (head + (PAIR ? r >> 4 : 0)) * kSbDh; };
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31, half = lane >> 5;
    const float c = scale * 1.4426950408889634f;
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    // keys of this environment: rows env*NK_all .. of the key/value buffer, or with `ranges` (a list of the
    // live rows only, CROSS) rows ranges[env] .. ranges[env+1]-1, all of them live
    int64_t k_base = (int64_t)env * NK_all;
    int NK = NK_all;
    if (ranges != nullptr) {
        k_base = ranges[env];
        int64_t cnt = (int64_t)ranges[env + 1] - k_base;
        if (cnt > kv_capacity - k_base) cnt = kv_capacity - k_base;
        NK = cnt < 0 ? 0 : (cnt > CAP ? CAP : (int)cnt);
    }
    const int nqb = (NQ + 31) >> 5, nkb = (NK + 31) >> 5;  // <= NB

    // token-major and channel-major copies of two (n, 32) operands; rows past n are zero.  The loads of
    // both phases are issued at the start of the kernel, so their latency is paid once.
    struct Staged {
        u32x4 a[2], b[2];
    };
    auto stage_load = [&](const uint16_t *a, int64_t a_stride, const uint16_t *b, int64_t b_stride, int64_t base, int n,
                          bool need_b) -> Staged {
        Staged r;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int item = tid + it * NT;
            const int tile_row = item >> 2, tok = tok_of(tile_row), c8 = (item & 3) * 8 + ch_of(tile_row);
            const int safe = tok < n ? tok : (n > 0 ? n - 1 : 0);
            const int64_t row = n > 0 ? base + safe : 0;  // an empty range reads row 0 of the buffer and discards it
            const u32x4 aw = *reinterpret_cast<const u32x4 *>(a + row * a_stride + c8);
            r.a[it] = tok < n ? aw : zero4;
            r.b[it] = zero4;
            if (need_b) {
                const u32x4 bw = *reinterpret_cast<const u32x4 *>(b + row * b_stride + c8);
                r.b[it] = tok < n ? bw : zero4;
            }
        }
        return r;
    };
    auto stage_store = [&](const Staged &r, bool transpose_a, bool transpose_b) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int item = tid + it * NT;
            const int tok = item >> 2, c8 = (item & 3) * 8;
            if (!OWN_ROWS) {
                *reinterpret_cast<u32x4 *>(s_rows[0] + tok * kMbPitch + c8) = r.a[it];
                *reinterpret_cast<u32x4 *>(s_rows[1] + tok * kMbPitch + c8) = r.b[it];
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t wa = r.a[it][e >> 1], wb = r.b[it][e >> 1];
                if (transpose_a) s_tr[0][(c8 + e) * TP + tok] = (uint16_t)((e & 1) ? wa >> 16 : wa & 0xffffu);
                if (transpose_b) s_tr[1][(c8 + e) * TP + tok] = (uint16_t)((e & 1) ? wb >> 16 : wb & 0xffffu);
            }
        }
    };
    // an operand of the first product of a pair: row (or column) tok, channels 8*half.. and 16 + 8*half..
    auto row_operand = [&](const uint16_t *rows, int tok, bf16x8 &lo, bf16x8 &hi) {
        const uint16_t *p = rows + tok * kMbPitch + half * 8;
        lo = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(p));
        hi = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(p + 16));
    };
    // the A operand of the second product: channel m, tokens in the order the accumulator rows 8t.. hold them
    auto tr_operand = [&](const uint16_t *tr, int blk, int t) -> bf16x8 {
        const uint16_t *p = tr + m * TP + blk * 32 + 16 * t + 4 * half;
        const u32x2 lo = *reinterpret_cast<const u32x2 *>(p);
        const u32x2 hi = *reinterpret_cast<const u32x2 *>(p + 8);
        return __builtin_bit_cast(bf16x8, u32x4{lo.x, lo.y, hi.x, hi.y});
    };
    auto pack8 = [&](const float (&x)[16], int t) -> bf16x8 {
        bf16x8 r;
#pragma unroll
        for (int e = 0; e < 8; ++e) r[e] = (__bf16)x[8 * t + e];
        return r;
    };
    // a (32 channels x 32 tokens) accumulator to rows of a gradient tensor: lane = token, rows = channels 8i + 4*half + j
    auto store_grad = [&](const f32x16 &acc, uint16_t *base, int64_t row_stride, int64_t first_row, int tile_row, int n) {
        const int tok = tok_of(tile_row);
        if (tok >= n) return;
        uint16_t *dst = base + (first_row + tok) * row_stride + ch_of(tile_row) + 4 * half;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            *reinterpret_cast<u32x2 *>(dst + 8 * i) = u32x2{pack_bf16x2(acc[4 * i], acc[4 * i + 1]), pack_bf16x2(acc[4 * i + 2], acc[4 * i + 3])};
    };

    // ---- every global load of the kernel ----
    const int own = wave * 32 + m;  // this lane's query in pass 1, its key in pass 2 (a tile row)
    const int own_tok = tok_of(own), own_ch = ch_of(own);
    const int64_t q_base = (int64_t)env * NQ;
    const int64_t q_row = q_base + (own_tok < NQ ? own_tok : NQ - 1);
    const int64_t k_row = NK > 0 ? k_base + (own_tok < NK ? own_tok : NK - 1) : 0;
    const int64_t own_q = q_row * q_row_stride + own_ch + half * 8, own_o = q_row * D + own_ch + half * 8;
    const int64_t own_k = k_row * kv_row_stride + own_ch + half * 8;
    bool any_live = false, my_live = false;
    if (tid < CAP) {  // CAP <= NT
        const int t = tok_of(tid);
        my_live = t < NK && (alive == nullptr || ranges != nullptr || alive[k_base + t] != 0);
        any_live = my_live;
    }
    // PAIR: accumulator rows 0..15 (v < 8) belong to the first head, 16..31 to the second; a lane's column to head m / 16
    auto other_head = [&](int vv) { return PAIR && ((vv >> 3) != (m >> 4)); };
    const Staged kv_in = stage_load(k, kv_row_stride, v, kv_row_stride, k_base, NK, !OWN_ROWS);
    u32x4 w0 = *reinterpret_cast<const u32x4 *>(q + own_q), w1 = *reinterpret_cast<const u32x4 *>(q + own_q + 16);
    u32x4 g0 = *reinterpret_cast<const u32x4 *>(dout + own_o), g1 = *reinterpret_cast<const u32x4 *>(dout + own_o + 16);
    const Row8 o0 = load8(out + own_o), o1 = load8(out + own_o + 16);
    u32x4 kw0 = *reinterpret_cast<const u32x4 *>(k + own_k), kw1 = *reinterpret_cast<const u32x4 *>(k + own_k + 16);
    u32x4 vw0 = *reinterpret_cast<const u32x4 *>(v + own_k), vw1 = *reinterpret_cast<const u32x4 *>(v + own_k + 16);
    const Staged qd_in = stage_load(q, q_row_stride, dout, D, q_base, NQ, true);

    // ---- live keys ----
    const bool none_live = __syncthreads_or(any_live ? 1 : 0) == 0;
    if (CROSS && none_live) {
        // the forward gated this environment off: nothing depends on its inputs
        const f32x16 z16 = {0.0f};
        if (wave < nqb) store_grad(z16, dq_out, dq_row_stride, q_base, own, NQ);
        if (wave < nkb) {
            store_grad(z16, dk_out, dkv_row_stride, k_base, own, NK);
            store_grad(z16, dv_out, dkv_row_stride, k_base, own, NK);
        }
        return;
    }
    const bool uniform = none_live;  // self-attention without a live key: equal weights over all keys
    if (tid < CAP) s_bias[tid] = (uniform ? tok_of(tid) < NK : my_live) ? 0.0f : -INFINITY;
    stage_store(kv_in, true, false);
    __syncthreads();

    // ---- pass 0 and 1: this wave's queries ----
    float delta;
    {
        const Row8 a0 = Row8{{__uint_as_float(g0.x << 16), __uint_as_float(g0.x & 0xffff0000u), __uint_as_float(g0.y << 16),
                              __uint_as_float(g0.y & 0xffff0000u), __uint_as_float(g0.z << 16), __uint_as_float(g0.z & 0xffff0000u),
                              __uint_as_float(g0.w << 16), __uint_as_float(g0.w & 0xffff0000u)}};
        const Row8 a1 = Row8{{__uint_as_float(g1.x << 16), __uint_as_float(g1.x & 0xffff0000u), __uint_as_float(g1.y << 16),
                              __uint_as_float(g1.y & 0xffff0000u), __uint_as_float(g1.z << 16), __uint_as_float(g1.z & 0xffff0000u),
                              __uint_as_float(g1.w << 16), __uint_as_float(g1.w & 0xffff0000u)}};
        float d = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) d = fmaf(a0.v[e], o0.v[e], fmaf(a1.v[e], o1.v[e], d));
        delta = d + __shfl_xor(d, 32);
    }
    if (own_tok >= NQ) w0 = w1 = g0 = g1 = zero4, delta = 0.0f;  // padding queries: nothing flows through them
    if (own_tok >= NK) kw0 = kw1 = vw0 = vw1 = zero4;
    const bf16x8 qs0 = __builtin_bit_cast(bf16x8, uniform ? zero4 : w0), qs1 = __builtin_bit_cast(bf16x8, uniform ? zero4 : w1);
    const bf16x8 gb0 = __builtin_bit_cast(bf16x8, g0), gb1 = __builtin_bit_cast(bf16x8, g1);

    if (wave < nqb) {
        auto scores_t = [&](int kb) -> f32x16 {
            f32x16 z;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f32x4 b4 = *reinterpret_cast<const f32x4 *>(s_bias + kb * 32 + 8 * i + 4 * half);
                z[4 * i] = b4.x, z[4 * i + 1] = b4.y, z[4 * i + 2] = b4.z, z[4 * i + 3] = b4.w;
            }
            if (PAIR) {
#pragma unroll
                for (int vv = 0; vv < 16; ++vv) z[vv] = other_head(vv) ? -INFINITY : z[vv];
            }
            bf16x8 k0, k1;
            if (OWN_ROWS)
                k0 = __builtin_bit_cast(bf16x8, kw0), k1 = __builtin_bit_cast(bf16x8, kw1);
            else
                row_operand(s_rows[0], kb * 32 + m, k0, k1);
            z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k0, qs0, z, 0, 0, 0);
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(k1, qs1, z, 0, 0, 0);
        };
        float mx = -INFINITY;
        for (int kb = 0; kb < nkb; ++kb) {
            const f32x16 z = scores_t(kb);
#pragma unroll
            for (int vv = 0; vv < 16; ++vv) mx = fmaxf(mx, z[vv]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float mc = mx * c;
        float sum = 0.0f;
        for (int kb = 0; kb < nkb; ++kb) {
            const f32x16 z = scores_t(kb);
#pragma unroll
            for (int vv = 0; vv < 16; ++vv) sum += __builtin_amdgcn_exp2f(fmaf(z[vv], c, -mc));
        }
        sum += __shfl_xor(sum, 32);
        const float lse = mc + __builtin_amdgcn_logf(sum);  // log2 of the sum of exp2(z c)
        if (half == 0) s_lse[own] = lse, s_delta[own] = delta;

        f32x16 dq = {0.0f};
        for (int kb = 0; kb < nkb; ++kb) {
            const f32x16 z = scores_t(kb);
            bf16x8 v0, v1;
            if (OWN_ROWS)
                v0 = __builtin_bit_cast(bf16x8, vw0), v1 = __builtin_bit_cast(bf16x8, vw1);
            else
                row_operand(s_rows[1], kb * 32 + m, v0, v1);
            f32x16 dp = {0.0f};
            dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v0, gb0, dp, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v1, gb1, dp, 0, 0, 0);
            float ds[16];
#pragma unroll
            for (int vv = 0; vv < 16; ++vv) ds[vv] = __builtin_amdgcn_exp2f(fmaf(z[vv], c, -lse)) * (dp[vv] - delta) * scale;
#pragma unroll
            for (int t = 0; t < 2; ++t) dq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_operand(s_tr[0], kb, t), pack8(ds, t), dq, 0, 0, 0);
        }
        store_grad(dq, dq_out, dq_row_stride, q_base, own, NQ);
    }
    __syncthreads();  // K, V and K^T are no longer needed; L and delta of every query are in LDS

    // ---- pass 2: this wave's keys ----
    stage_store(qd_in, true, true);
    const float col_bias = s_bias[own];
    const bf16x8 ks0 = __builtin_bit_cast(bf16x8, uniform ? zero4 : kw0), ks1 = __builtin_bit_cast(bf16x8, uniform ? zero4 : kw1);
    const bf16x8 vb0 = __builtin_bit_cast(bf16x8, vw0), vb1 = __builtin_bit_cast(bf16x8, vw1);
    __syncthreads();
    if (wave >= nkb) return;

    f32x16 dk = {0.0f}, dv = {0.0f};
    for (int qb = 0; qb < nqb; ++qb) {
        f32x16 z;
#pragma unroll
        for (int vv = 0; vv < 16; ++vv) z[vv] = other_head(vv) ? -INFINITY : col_bias;
        bf16x8 a0, a1;
        if (OWN_ROWS)
            a0 = __builtin_bit_cast(bf16x8, w0), a1 = __builtin_bit_cast(bf16x8, w1);
        else
            row_operand(s_rows[0], qb * 32 + m, a0, a1);
        z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, ks0, z, 0, 0, 0);
        z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, ks1, z, 0, 0, 0);
        if (OWN_ROWS)
            a0 = gb0, a1 = gb1;
        else
            row_operand(s_rows[1], qb * 32 + m, a0, a1);
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
                ds[vv] = p[vv] * (dp[vv] - d4[j]) * scale;
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            dk = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_operand(s_tr[0], qb, t), pack8(ds, t), dk, 0, 0, 0);
            dv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_operand(s_tr[1], qb, t), pack8(p, t), dv, 0, 0, 0);
        }
    }
    store_grad(dk, dk_out, dkv_row_stride, k_base, own, NK);
    store_grad(dv, dv_out, dkv_row_stride, k_base, own, NK);
}

template <int NB, bool CROSS, bool PAIR = false>
static int launch_sdpa_bwd_mfma(const void *q, int64_t q_row_stride, const void *k, const void *v, int64_t kv_row_stride,
                                const uint8_t *alive, const int32_t *ranges, int64_t kv_capacity, const void *out, const void *dout,
                                void *dq, int64_t dq_row_stride, void *dk, void *dv, int64_t dkv_row_stride, int64_t B, int NQ,
                                int NK, int H, hipStream_t stream)
{
    const int64_t groups = (B * (PAIR ? H / 2 : H) + 7) / 8 * 8;  // a multiple of 8: the XCD mapping deals whole rounds
    if (groups > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((sdpa_bwd_mfma_kernel<NB, CROSS, PAIR>), dim3((unsigned)groups), dim3(kWave * NB), 0, stream, (const uint16_t *)q,
                       q_row_stride, (const uint16_t *)k, (const uint16_t *)v, kv_row_stride, alive, ranges, kv_capacity,
                       (const uint16_t *)out, (const uint16_t *)dout, (uint16_t *)dq, dq_row_stride, (uint16_t *)dk, (uint16_t *)dv, dkv_row_stride, (int)B,
                       NQ, NK, H, 1.0f / sqrtf((float)kSbDh));
    return (int)hipGetLastError();
}

template <bool CROSS>
static int dispatch_sdpa_bwd_mfma(const void *q, int64_t q_row_stride, const void *k, const void *v, int64_t kv_row_stride,
                                  const uint8_t *alive, const int32_t *ranges, int64_t kv_capacity, const void *out, const void *dout,
                                  void *dq, int64_t dq_row_stride, void *dk, void *dv, int64_t dkv_row_stride, int64_t B, int NQ,
                                  int NK, int H, hipStream_t s)
{
    const int nb = ((NQ > NK ? NQ : NK) + 31) / 32;
    if (!CROSS && NQ <= 16 && H % 2 == 0)
        return launch_sdpa_bwd_mfma<1, false, true>(q, q_row_stride, k, v, kv_row_stride, alive, ranges, kv_capacity, out, dout, dq,
                                                    dq_row_stride, dk, dv, dkv_row_stride, B, NQ, NK, H, s);
#define BNB_SBM(NBV) \
    return launch_sdpa_bwd_mfma<NBV, CROSS>(q, q_row_stride, k, v, kv_row_stride, alive, ranges, kv_capacity, out, dout, dq, \
                                            dq_row_stride, dk, dv, dkv_row_stride, B, NQ, NK, H, s)
    switch (nb) {
        case 1: BNB_SBM(1);
        case 2: BNB_SBM(2);
        case 3: BNB_SBM(3);
        case 4: BNB_SBM(4);
        case 5: BNB_SBM(5);
        default: return BNB_ERR_UNSUPPORTED;
    }
#undef BNB_SBM
}

}  // namespace bnb

extern "C" int bnb_sdpa_masked_bwd_path(const void *qkv, int64_t qkv_row_stride, const uint8_t *alive, const void *out,
                                        const void *dout, void *dqkv, int64_t B, int NM, int H, int dh, int dtype, int path,
                                        void *stream)
{
    using namespace bnb;
    if (B < 0 || NM < 1 || H < 1 || dh < 1) return BNB_ERR_BAD_SHAPE;
    const bool small = NM <= kSbMaxTokens && H <= 8 && NM * H <= 256;
    const bool mfma = dtype == BNB_BF16 && NM <= 160 && B <= 0x7fffffffLL / (H > 0 ? H : 1);
    if (dh != kSbDh || (!small && !mfma)) return BNB_ERR_UNSUPPORTED;
    if (dtype != BNB_F32 && dtype != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (qkv_row_stride < 3 * (int64_t)H * dh) return BNB_ERR_BAD_SHAPE;
    if (B == 0) return 0;
    if (!qkv || !out || !dout || !dqkv) return BNB_ERR_NULL_POINTER;
    const int64_t esz = dtype == BNB_BF16 ? 2 : 4;
    if (!aligned16(qkv) || !aligned16(out) || !aligned16(dout) || !aligned16(dqkv) || (qkv_row_stride * esz) % 16 != 0)
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    if (path != BNB_SDPA_PATH_AUTO && path != BNB_SDPA_PATH_VALU && path != BNB_SDPA_PATH_MFMA) return BNB_ERR_BAD_SHAPE;
    if (path == BNB_SDPA_PATH_MFMA && !mfma) return BNB_ERR_UNSUPPORTED;
    if (mfma && (path == BNB_SDPA_PATH_MFMA || (path == BNB_SDPA_PATH_AUTO && NM > kSbMfmaFrom))) {
        const uint16_t *p = (const uint16_t *)qkv;
        const int D = H * dh;
        uint16_t *g = (uint16_t *)dqkv;
        return dispatch_sdpa_bwd_mfma<false>(p, qkv_row_stride, p + D, p + 2 * D, qkv_row_stride, alive, nullptr, 0, out, dout, g,
                                             3 * (int64_t)D, g + D, g + 2 * D, 3 * (int64_t)D, B, NM, NM, H, s);
    }
    if (!small) return BNB_ERR_UNSUPPORTED;
    if (dtype == BNB_BF16) return launch_sdpa_bwd<uint16_t>(qkv, qkv_row_stride, alive, out, dout, dqkv, B, NM, H, s);
    return launch_sdpa_bwd<float>(qkv, qkv_row_stride, alive, out, dout, dqkv, B, NM, H, s);
}

extern "C" int bnb_sdpa_masked_bwd(const void *qkv, int64_t qkv_row_stride, const uint8_t *alive, const void *out,
                                   const void *dout, void *dqkv, int64_t B, int NM, int H, int dh, int dtype, void *stream)
{
    return bnb_sdpa_masked_bwd_path(qkv, qkv_row_stride, alive, out, dout, dqkv, B, NM, H, dh, dtype, BNB_SDPA_PATH_AUTO, stream);
}

extern "C" int bnb_sdpa_cross_bwd(const void *q, int64_t q_row_stride, int NQ, const void *kv, int64_t kv_row_stride, int NK,
                                  const uint8_t *key_mask, const void *out, const void *dout, void *dq, void *dkv, int64_t B,
                                  int H, int dh, int dtype, void *stream)
{
    using namespace bnb;
    if (B < 0 || NQ < 1 || NK < 1 || H < 1 || dh < 1) return BNB_ERR_BAD_SHAPE;
    if (dtype != BNB_BF16 || dh != kSbDh || NQ > 160 || NK > 160) return BNB_ERR_UNSUPPORTED;
    const int D = H * dh;
    if (q_row_stride < D || kv_row_stride < 2 * (int64_t)D) return BNB_ERR_BAD_SHAPE;
    if (B == 0) return 0;
    if (!q || !kv || !out || !dout || !dq || !dkv) return BNB_ERR_NULL_POINTER;
    if (!aligned16(q) || !aligned16(kv) || !aligned16(out) || !aligned16(dout) || !aligned16(dq) || !aligned16(dkv) ||
        (q_row_stride % 8) != 0 || (kv_row_stride % 8) != 0)
        return BNB_ERR_MISALIGNED;
    if (B > 0x7fffffffLL / H) return BNB_ERR_UNSUPPORTED;
    const uint16_t *kp = (const uint16_t *)kv;
    uint16_t *g = (uint16_t *)dkv;
    return dispatch_sdpa_bwd_mfma<true>(q, q_row_stride, kp, kp + D, kv_row_stride, key_mask, nullptr, 0, out, dout, dq, D, g, g + D,
                                        2 * (int64_t)D, B, NQ, NK, H, (hipStream_t)stream);
}

extern "C" int bnb_sdpa_cross_ranges_bwd(const void *q, int64_t q_row_stride, int NQ, const void *kv_rows, int64_t kv_row_stride,
                                         const int32_t *ranges, int64_t capacity, int max_keys, const void *out, const void *dout,
                                         void *dq, void *dkv_rows, int64_t B, int H, int dh, int dtype, void *stream)
{
    using namespace bnb;
    if (B < 0 || NQ < 1 || H < 1 || dh < 1 || capacity < 1 || max_keys < 1) return BNB_ERR_BAD_SHAPE;  // an empty list: nothing to call
    if (dtype != BNB_BF16 || dh != kSbDh || NQ > 160 || max_keys > 160) return BNB_ERR_UNSUPPORTED;
    const int D = H * dh;
    if (q_row_stride < D || kv_row_stride < 2 * (int64_t)D) return BNB_ERR_BAD_SHAPE;
    if (B == 0) return 0;
    if (!q || !ranges || !out || !dout || !dq || !kv_rows || !dkv_rows) return BNB_ERR_NULL_POINTER;
    if (!aligned16(q) || !aligned16(kv_rows) || !aligned16(out) || !aligned16(dout) || !aligned16(dq) || !aligned16(dkv_rows) ||
        (q_row_stride % 8) != 0 || (kv_row_stride % 8) != 0)
        return BNB_ERR_MISALIGNED;
    if (B > 0x7fffffffLL / H) return BNB_ERR_UNSUPPORTED;
    const uint16_t *kp = (const uint16_t *)kv_rows;
    uint16_t *g = (uint16_t *)dkv_rows;
    return dispatch_sdpa_bwd_mfma<true>(q, q_row_stride, kp, kp + D, kv_row_stride, nullptr, ranges, capacity, out, dout, dq, D, g,
                                        g + D, 2 * (int64_t)D, B, NQ, max_keys, H, (hipStream_t)stream);
}
