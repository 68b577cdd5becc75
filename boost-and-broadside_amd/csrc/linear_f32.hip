// Float32 Linear layers of the trunk with their neighbours folded in, on the fp32 matrix cores (gfx950).
//
// Evaluation runs the policy without autocast (evaluation/agents.py:214-219), so every Linear of the
// trunk (models/yemong/attention.py:21-37,60-74; models/yemong/griffin.py:165-167,238-247) is a
// float32 GEMM with a 128- or 512-wide contraction, and between them sit RMSNorm, residual adds and
// the gelu gates as separate element-wise passes.  One kernel covers all of them:
//
//     out[r, :] = ( A[r, :] W^T + bias ) (+ resid[r, :])        A = x                     plain
//                                                                  | rmsnorm(x) * norm_w     NORM
//                                                                  | gelu(x) * x2            MULGELU
//     GATE: W = [gate rows ; up rows] interleaved by blocks of 32, out[r, u] = gelu(g[r, u]) * up[r, u]
//
// True fp32 products and accumulation (v_mfma_f32_32x32x2_f32), so the 1e-5 bar holds.
//
// A wave owns 32 rows and a run of 32-feature blocks: out (rows x features) = A (rows x K) W^T, rows on
// the M axis, so a lane ends up with ONE feature of 16 rows and a store instruction writes 128
// contiguous bytes of two rows.  The contraction index of a product may run in any order as long as
// both operands agree: step s pairs channel s (lanes 0..31) with channel K/2 + s (lanes 32..63), so a
// lane's A values are one contiguous half row, loaded once per 128-channel slab and kept in
// registers (norm and gate are applied there), and W arrives pre-packed so that a lane's four next
// steps are one 16-byte load of a 1 KB contiguous wave read, straight from L2, a few loads ahead.

#include "common.h"

namespace bnb {

constexpr int kLfSlab = 64;  // steps per slab: 128 channels (64 per half wave)

// erf-GELU without branches: erf from the five-term Abramowitz-Stegun form 7.1.26 (|error| <= 1.5e-7,
// |error of gelu| <= 5e-7 over |v| <= 12, far inside the float32 bar), 14 vector instructions against
// about 30 for the library's erff.  gelu(v) = v/2 + |v|/2 * erf(|v| / sqrt 2).
__device__ __forceinline__ float gelu_erf_lf(float v)
{
    const float x = fabsf(v) * 0.70710678118654752f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, x, 1.0f));
    float poly = fmaf(1.061405429f, t, -1.453152027f);
    poly = fmaf(poly, t, 1.421413741f);
    poly = fmaf(poly, t, -0.284496736f);
    poly = fmaf(poly, t, 0.254829592f);
    const float e = __builtin_amdgcn_exp2f((x * x) * -1.4426950408889634f);
    const float erf_abs = fmaf(-(poly * t), e, 1.0f);
    const float hv = 0.5f * v;
    return fmaf(fabsf(hv), erf_abs, hv);
}

template <bool NORM, bool MULGELU, bool GATE>
__global__ __launch_bounds__(64, 2) void linear_f32_kernel(
    const float *__restrict__ x, int64_t x_stride, const float *__restrict__ x2, int64_t x2_stride,
    const float *__restrict__ norm_w, float eps, const float *__restrict__ w_packed, const float *__restrict__ bias,
    const float *resid, int64_t resid_stride, float *out, int64_t out_stride, int64_t R, int K, int n_blocks,
    int blocks_per_wave)
{
    // one wave per work-group: the waves that share a row tile (consecutive work-groups, each a run of feature blocks) are
    // independent, so a finished wave's slot is refilled at once
    const int lane = threadIdx.x;
    const int m = lane & 31, half = lane >> 5;
    const int unit = GATE ? 2 : 1;  // weight blocks per output block
    const int n_out_all = n_blocks / unit;
    const int waves_per_tile = (n_out_all + blocks_per_wave - 1) / blocks_per_wave;
    const int64_t row0 = (int64_t)(blockIdx.x / waves_per_tile) * 32;
    const int first = (blockIdx.x % waves_per_tile) * blocks_per_wave;  // first OUTPUT block of this wave
    const int n_out_blocks = n_blocks / unit;
    if (first >= n_out_blocks) return;
    const int last = first + blocks_per_wave < n_out_blocks ? first + blocks_per_wave : n_out_blocks;

    const int64_t row = row0 + m < R ? row0 + m : R - 1;  // rows past the end repeat the last one and are not stored
    const int slabs = K / (2 * kLfSlab);
    const int half_k = K >> 1;
    const int s4_per_block = K >> 3;  // 16-byte loads per lane and weight block

    // this lane's A values of one slab: channels half*K/2 + 64 t + (0..63) of its row, norm / gate applied
    float a[kLfSlab];
    auto load_slab = [&](int t) {
        const float *xp = x + row * x_stride + half * half_k + t * kLfSlab;
#pragma unroll
        for (int i = 0; i < kLfSlab / 4; ++i) {
            const f32x4 v = *reinterpret_cast<const f32x4 *>(xp + 4 * i);
            a[4 * i] = v.x, a[4 * i + 1] = v.y, a[4 * i + 2] = v.z, a[4 * i + 3] = v.w;
        }
        if (NORM) {
            // K == 128: one slab holds the whole row
            float ss = 0.0f;
#pragma unroll
            for (int i = 0; i < kLfSlab; ++i) ss = fmaf(a[i], a[i], ss);
            ss += __shfl_xor(ss, 32);
            const float rstd = rsqrtf(ss * (1.0f / (2 * kLfSlab)) + eps);
            const float *nw = norm_w + half * half_k;
#pragma unroll
            for (int i = 0; i < kLfSlab / 4; ++i) {
                const f32x4 w4 = *reinterpret_cast<const f32x4 *>(nw + 4 * i);
                a[4 * i] = a[4 * i] * rstd * w4.x, a[4 * i + 1] = a[4 * i + 1] * rstd * w4.y;
                a[4 * i + 2] = a[4 * i + 2] * rstd * w4.z, a[4 * i + 3] = a[4 * i + 3] * rstd * w4.w;
            }
        }
        if (MULGELU) {
            const float *yp = x2 + row * x2_stride + half * half_k + t * kLfSlab;
#pragma unroll
            for (int i = 0; i < kLfSlab / 4; ++i) {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(yp + 4 * i);
                a[4 * i] = gelu_erf_lf(a[4 * i]) * v.x, a[4 * i + 1] = gelu_erf_lf(a[4 * i + 1]) * v.y;
                a[4 * i + 2] = gelu_erf_lf(a[4 * i + 2]) * v.z, a[4 * i + 3] = gelu_erf_lf(a[4 * i + 3]) * v.w;
            }
        }
    };
    if (slabs == 1) load_slab(0);  // a 128-wide contraction keeps its operand across all feature blocks

    // Weight groups (one 16-byte load per lane = four contraction steps) are requested AHEAD groups before
    // they are used, across slab and block boundaries, so that the matrix cores never wait for L2 at
    // the start of a block: the ring wq/wq2 is carried through all loops.
    constexpr int GROUPS = kLfSlab / 4;  // 16 groups per slab
    constexpr int AHEAD = GATE ? 4 : 8;  // divides GROUPS, so a group's ring slot is the same in every slab
    static_assert(GROUPS % AHEAD == 0, "the ring slot of a group must not depend on the slab");
    f32x4 wq[AHEAD], wq2[AHEAD];
    const int64_t block_floats = (int64_t)s4_per_block * 256;  // one packed 32-feature block
    const float *w_lane = w_packed + lane * 4;
    {
        const float *ws = w_lane + (int64_t)first * unit * block_floats;
#pragma unroll
        for (int i = 0; i < AHEAD; ++i) {
            wq[i] = *reinterpret_cast<const f32x4 *>(ws + (int64_t)i * 256);
            if (GATE) wq2[i] = *reinterpret_cast<const f32x4 *>(ws + block_floats + (int64_t)i * 256);
        }
    }

    for (int ob = first; ob < last; ++ob) {
        f32x16 acc = {0.0f}, acc2 = {0.0f};
        for (int t = 0; t < slabs; ++t) {
            if (slabs > 1) load_slab(t);
            // this slab's groups, and where the groups after it live (the next slab of this block, else the
            // first slab of the next block; after the very last one the loads repeat this slab and are dropped)
            const float *ws = w_lane + (int64_t)ob * unit * block_floats + (int64_t)t * GROUPS * 256;
            const float *wn = ws;
            if (t + 1 < slabs) wn = ws + (int64_t)GROUPS * 256;
            else if (ob + 1 < last) wn = w_lane + (int64_t)(ob + 1) * unit * block_floats;
#pragma unroll
            for (int s4 = 0; s4 < GROUPS; ++s4) {
                const int slot = s4 % AHEAD;
                const f32x4 b = wq[slot];
                f32x4 b2 = {0.0f, 0.0f, 0.0f, 0.0f};
                if (GATE) b2 = wq2[slot];
                const float *src = s4 + AHEAD < GROUPS ? ws + (int64_t)(s4 + AHEAD) * 256 : wn + (int64_t)(s4 + AHEAD - GROUPS) * 256;
                wq[slot] = *reinterpret_cast<const f32x4 *>(src);
                if (GATE) wq2[slot] = *reinterpret_cast<const f32x4 *>(src + block_floats);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * s4 + 0], b.x, acc, 0, 0, 0);
                if (GATE) acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * s4 + 0], b2.x, acc2, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * s4 + 1], b.y, acc, 0, 0, 0);
                if (GATE) acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * s4 + 1], b2.y, acc2, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * s4 + 2], b.z, acc, 0, 0, 0);
                if (GATE) acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * s4 + 2], b2.z, acc2, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * s4 + 3], b.w, acc, 0, 0, 0);
                if (GATE) acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4 * s4 + 3], b2.w, acc2, 0, 0, 0);
                // keep the request for group s4 + AHEAD in front of group s4's products: left to itself the
                // scheduler sinks the loads until just before their use and the matrix cores wait for L2
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // ---- epilogue: the lane holds feature 32 ob + m of rows 8 i + 4 half + j ----
        const int feat = ob * 32 + m;
        const float bv = bias != nullptr ? bias[feat] : 0.0f;
        float res[16];
        if (resid != nullptr) {
            // all sixteen requests first: one round trip instead of sixteen
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int64_t r = row0 + 8 * (v >> 2) + 4 * half + (v & 3);
                res[v] = resid[(r < R ? r : R - 1) * resid_stride + feat];
            }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            float o = acc[v] + bv;
            if (GATE) o = gelu_erf_lf(o) * acc2[v];
            if (resid != nullptr) o += res[v];
            acc[v] = o;
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int64_t r = row0 + 8 * (v >> 2) + 4 * half + (v & 3);
            if (r < R) out[r * out_stride + feat] = acc[v];
        }
    }
}

template <bool NORM, bool MULGELU, bool GATE>
static int launch_linear_f32(const float *x, int64_t x_stride, const float *x2, int64_t x2_stride, const float *norm_w, float eps,
                             const float *w_packed, const float *bias, const float *resid, int64_t resid_stride, float *out,
                             int64_t out_stride, int64_t R, int K, int N, hipStream_t stream)
{
    const int n_blocks = N / 32;
    const int n_out_blocks = GATE ? n_blocks / 2 : n_blocks;
    const int64_t tiles = (R + 31) / 32;
    // split the features over enough waves to give every SIMD several tasks (1024 SIMDs) when the row count is small
    int per = n_out_blocks;
    while (per > 1 && tiles * ((n_out_blocks + per - 1) / per) < 8192) per = (per + 1) / 2;
    const int waves = (n_out_blocks + per - 1) / per;
    if (tiles * waves > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((linear_f32_kernel<NORM, MULGELU, GATE>), dim3((unsigned)(tiles * waves)), dim3(64), 0, stream,
                       x, x_stride, x2, x2_stride, norm_w, eps, w_packed, bias, resid, resid_stride, out, out_stride, R, K, n_blocks,
                       per);
    return (int)hipGetLastError();
}

}  // namespace bnb

extern "C" int bnb_linear_f32_fwd(const float *x, int64_t x_row_stride, const float *x2, int64_t x2_row_stride,
                                  const float *norm_weight, float eps, const float *weight_packed, const float *bias,
                                  const float *resid, int64_t resid_row_stride, float *out, int64_t out_row_stride, int64_t R,
                                  int K, int N, int gate, void *stream)
{
    using namespace bnb;
    if (R < 0 || K < 1 || N < 1) return BNB_ERR_BAD_SHAPE;
    if (K % 128 != 0 || N % 32 != 0 || (gate && N % 64 != 0)) return BNB_ERR_UNSUPPORTED;
    if (norm_weight != nullptr && (K != 128 || x2 != nullptr)) return BNB_ERR_UNSUPPORTED;
    if (gate && (bias != nullptr || x2 != nullptr)) return BNB_ERR_UNSUPPORTED;
    if (R == 0) return 0;
    if (!x || !weight_packed || !out) return BNB_ERR_NULL_POINTER;
    const int n_out = gate ? N / 2 : N;
    if (x_row_stride < K || out_row_stride < n_out || (x2 && x2_row_stride < K) || (resid && resid_row_stride < n_out))
        return BNB_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(weight_packed) || x_row_stride % 4 != 0 || (x2 && (!aligned16(x2) || x2_row_stride % 4 != 0)) ||
        (norm_weight && !aligned16(norm_weight)))
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    if (norm_weight != nullptr) {
        if (gate)
            return launch_linear_f32<true, false, true>(x, x_row_stride, nullptr, 0, norm_weight, eps, weight_packed, nullptr, resid,
                                                        resid_row_stride, out, out_row_stride, R, K, N, s);
        return launch_linear_f32<true, false, false>(x, x_row_stride, nullptr, 0, norm_weight, eps, weight_packed, bias, resid,
                                                     resid_row_stride, out, out_row_stride, R, K, N, s);
    }
    if (x2 != nullptr)
        return launch_linear_f32<false, true, false>(x, x_row_stride, x2, x2_row_stride, nullptr, eps, weight_packed, bias, resid,
                                                     resid_row_stride, out, out_row_stride, R, K, N, s);
    if (gate)
        return launch_linear_f32<false, false, true>(x, x_row_stride, nullptr, 0, nullptr, eps, weight_packed, nullptr, resid,
                                                     resid_row_stride, out, out_row_stride, R, K, N, s);
    return launch_linear_f32<false, false, false>(x, x_row_stride, nullptr, 0, nullptr, eps, weight_packed, bias, resid,
                                                  resid_row_stride, out, out_row_stride, R, K, N, s);
}
