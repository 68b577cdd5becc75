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

}  // namespace bnb

extern "C" int bnb_sdpa_masked_bwd(const void *qkv, int64_t qkv_row_stride, const uint8_t *alive, const void *out,
                                   const void *dout, void *dqkv, int64_t B, int NM, int H, int dh, int dtype, void *stream)
{
    using namespace bnb;
    if (B < 0 || NM < 1 || H < 1 || dh < 1) return BNB_ERR_BAD_SHAPE;
    if (dh != kSbDh || NM > kSbMaxTokens || H > 8 || NM * H > 256) return BNB_ERR_UNSUPPORTED;
    if (dtype != BNB_F32 && dtype != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (qkv_row_stride < 3 * (int64_t)H * dh) return BNB_ERR_BAD_SHAPE;
    if (B == 0) return 0;
    if (!qkv || !out || !dout || !dqkv) return BNB_ERR_NULL_POINTER;
    const int64_t esz = dtype == BNB_BF16 ? 2 : 4;
    if (!aligned16(qkv) || !aligned16(out) || !aligned16(dout) || !aligned16(dqkv) || (qkv_row_stride * esz) % 16 != 0)
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == BNB_BF16) return launch_sdpa_bwd<uint16_t>(qkv, qkv_row_stride, alive, out, dout, dqkv, B, NM, H, s);
    return launch_sdpa_bwd<float>(qkv, qkv_row_stride, alive, out, dout, dqkv, B, NM, H, s);
}
