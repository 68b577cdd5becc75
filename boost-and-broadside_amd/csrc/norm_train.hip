// RMSNorm backward for gfx950:  y = x * rsqrt(mean(x^2) + eps) * w
//   dx = rstd * (dy * w) - x * rstd^3 * mean(dy * w * x)   (+ grad_sum, the gradient arriving on the
//                                                           residual branch that bypasses the norm)
//   dw = sum over rows of dy * x * rstd
//
// What autograd runs for every nn.RMSNorm of the trunk during the PPO update (reference:
// train/rl/ppo.py:1417-1425 through models/yemong/attention.py:60,73,94-98 and
// griffin.py:238,246,269,284-285).  The library does it in two kernels over fp32 tensors, after
// a cast of the bf16 gradient to fp32 and before an add with the residual gradient; here one
// streaming pass reads x (fp32) and dy (bf16 or fp32) once and writes dx once.  rstd is
// recomputed from x, which is being read anyway.  Weight-gradient partial sums stay in
// registers across a work-group's rows, are combined through LDS in a fixed order and written
// one row per work-group; a second kernel adds those rows in a fixed order: no atomics, the
// result does not depend on timing.
// Bound: HBM.  8 channels per lane, 16-byte nontemporal accesses, fp32 arithmetic.

#include "common.h"

#include <mutex>

namespace bnb {

constexpr int kNbThreads = 256;
constexpr int kNbMaxBlocks = 1280;  // five work-groups per CU: what 80-98 registers per lane let run at once, so no work-group waits for a free slot

// Workspace of the entry point that allocates nothing (bnb_rmsnorm_bwd_static): the per-work-group
// partial weight gradients, kNbMaxBlocks rows of at most kNbStaticMaxD floats = 2.5 MiB.  Every GPU
// the library runs on holds its own copy at its own address until the process ends.  In host
// code this name is only a handle for hipGetSymbolAddress, never a device address.
constexpr int kNbStaticMaxD = 512;
static __device__ __align__(256) float scratch[kNbMaxBlocks * kNbStaticMaxD];

constexpr int kMaxDevices = 64;
static float *g_scratch_ptr[kMaxDevices];  // device address of `scratch` per device, looked up once
static std::mutex g_scratch_mutex;

// Device address of this device's `scratch`, resolved on the first call with that device current.
static int scratch_address(float **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return BNB_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        float *ptr = nullptr;
        e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (ptr == nullptr) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

template <int LANES, typename GT, bool HAS_SUM>
__global__ __launch_bounds__(kNbThreads) void rmsnorm_bwd_kernel(
    const float *__restrict__ x, int64_t x_stride, const GT *__restrict__ dy, int64_t dy_stride,
    const float *__restrict__ weight, float eps, const float *__restrict__ grad_sum, float *__restrict__ dx,
    uint16_t *__restrict__ dx_bf16, float *__restrict__ partials, int64_t R)
{
    constexpr int D = LANES * 8;
    constexpr int ROWS = kNbThreads / LANES;
    __shared__ float s_dw[ROWS * D];

    const int local_row = threadIdx.x / LANES;
    // a lane's eight channels are two runs of four, d0 .. d0 + 3 and D/2 + d0 ..: each access of a row's lanes is
    // then one dense run of bytes (eight consecutive float32 channels per lane put the lanes of an instruction 32
    // bytes apart, which streams at two thirds of the rate)
    const int d0 = (threadIdx.x - local_row * LANES) << 2;
    constexpr int gap = D / 2;
    const int64_t step = (int64_t)gridDim.x * ROWS;
    const Row8 w = load8_split<false>(weight + d0, gap);
    float dw[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};

    // every lane of a row group walks the same number of iterations (the butterflies need all of them)
    int64_t row = (int64_t)blockIdx.x * ROWS + local_row;
    int64_t r = row < R ? row : R - 1;
    Row8 xn = load8_split<true>(x + r * x_stride + d0, gap), gn = load8_split<true>(dy + r * dy_stride + d0, gap);
    Row8 sn = xn;  // the bypass gradient travels with the other two rows, one iteration ahead
    if (HAS_SUM) sn = load8_split<true>(grad_sum + r * D + d0, gap);
    for (int64_t base = (int64_t)blockIdx.x * ROWS; base < R; base += step) {
        const Row8 xv = xn, gv = gn, sv = sn;
        const int64_t cur = row;
        const bool valid = cur < R;
        row += step;
        if (base + step < R) {
            r = row < R ? row : R - 1;
            xn = load8_split<true>(x + r * x_stride + d0, gap), gn = load8_split<true>(dy + r * dy_stride + d0, gap);
            if (HAS_SUM) sn = load8_split<true>(grad_sum + r * D + d0, gap);
        }
        float ss = 0.0f, dot = 0.0f;
        Row8 g;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            g.v[e] = gv.v[e] * w.v[e];
            ss = fmaf(xv.v[e], xv.v[e], ss);
            dot = fmaf(g.v[e], xv.v[e], dot);
        }
#pragma unroll
        for (int off = 1; off < LANES; off <<= 1) {
            ss += __shfl_xor(ss, off);
            dot += __shfl_xor(dot, off);
        }
        if (!valid) continue;
        const float rstd = rsqrtf(ss * (1.0f / D) + eps);
        const float coef = dot * (1.0f / D) * rstd * rstd * rstd;
        Row8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            o.v[e] = g.v[e] * rstd - xv.v[e] * coef;
            dw[e] = fmaf(gv.v[e] * rstd, xv.v[e], dw[e]);
        }
        if (HAS_SUM) {
#pragma unroll
            for (int e = 0; e < 8; ++e) o.v[e] += sv.v[e];
        }
        store8_split<true>(dx + cur * D + d0, gap, o);
        // an ordinary store: as a third nontemporal stream this copy cost 50 us more on some allocations
        if (dx_bf16 != nullptr) store8_split<false>(dx_bf16 + cur * D + d0, gap, o);
    }

#pragma unroll
    for (int e = 0; e < 8; ++e) s_dw[local_row * D + d0 + (e & 3) + (e >> 2) * gap] = dw[e];
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += kNbThreads) {
        float t = 0.0f;
#pragma unroll
        for (int j = 0; j < ROWS; ++j) t += s_dw[j * D + d];
        partials[(int64_t)blockIdx.x * D + d] = t;
    }
}

template <int LANES, typename GT>
static int launch_norm_bwd(const float *x, int64_t x_stride, const void *dy, int64_t dy_stride, const float *weight, float eps,
                           const float *grad_sum, float *dx, uint16_t *dx_bf16, float *partials, int blocks, float *dw,
                           int64_t R, hipStream_t stream)
{
    const dim3 g((unsigned)blocks), t(kNbThreads);
    if (grad_sum)
        hipLaunchKernelGGL((rmsnorm_bwd_kernel<LANES, GT, true>), g, t, 0, stream, x, x_stride, (const GT *)dy, dy_stride, weight,
                           eps, grad_sum, dx, dx_bf16, partials, R);
    else
        hipLaunchKernelGGL((rmsnorm_bwd_kernel<LANES, GT, false>), g, t, 0, stream, x, x_stride, (const GT *)dy, dy_stride, weight,
                           eps, grad_sum, dx, dx_bf16, partials, R);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return launch_sum_slices(partials, dw, LANES * 8, blocks, 0, stream);
}

template <typename GT>
static int dispatch_norm_bwd(int D, const float *x, int64_t x_stride, const void *dy, int64_t dy_stride, const float *weight,
                             float eps, const float *grad_sum, float *dx, uint16_t *dx_bf16, float *partials, int blocks,
                             float *dw, int64_t R, hipStream_t s)
{
    switch (D) {
        case 64: return launch_norm_bwd<8, GT>(x, x_stride, dy, dy_stride, weight, eps, grad_sum, dx, dx_bf16, partials, blocks, dw, R, s);
        case 128: return launch_norm_bwd<16, GT>(x, x_stride, dy, dy_stride, weight, eps, grad_sum, dx, dx_bf16, partials, blocks, dw, R, s);
        case 256: return launch_norm_bwd<32, GT>(x, x_stride, dy, dy_stride, weight, eps, grad_sum, dx, dx_bf16, partials, blocks, dw, R, s);
        case 512: return launch_norm_bwd<64, GT>(x, x_stride, dy, dy_stride, weight, eps, grad_sum, dx, dx_bf16, partials, blocks, dw, R, s);
        default: return BNB_ERR_UNSUPPORTED;
    }
}

}  // namespace bnb

extern "C" int bnb_rmsnorm_bwd_blocks(int64_t R, int D)
{
    if (R <= 0 || D < 8) return 1;
    const int rows = bnb::kNbThreads / (D / 8) > 0 ? bnb::kNbThreads / (D / 8) : 1;
    const int64_t need = (R + rows - 1) / rows;
    return (int)(need < bnb::kNbMaxBlocks ? need : bnb::kNbMaxBlocks);
}

extern "C" int bnb_rmsnorm_bwd(const float *x, int64_t x_row_stride, const void *dy, int dy_dtype, int64_t dy_row_stride,
                               const float *weight, float eps, const float *grad_sum, float *dx, void *dx_bf16,
                               float *partials, int blocks, float *dw, int64_t R, int D, void *stream)
{
    using namespace bnb;
    if (R < 0 || D < 1 || x_row_stride < D || dy_row_stride < D) return BNB_ERR_BAD_SHAPE;
    if (D != 64 && D != 128 && D != 256 && D != 512) return BNB_ERR_UNSUPPORTED;
    if (dy_dtype != BNB_F32 && dy_dtype != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (!weight || !dw || !partials || (R > 0 && (!x || !dy || !dx))) return BNB_ERR_NULL_POINTER;
    if (blocks < 1 || blocks > kNbMaxBlocks) return BNB_ERR_BAD_SHAPE;
    if (!aligned16(weight) || !aligned16(dw) || !aligned16(partials) ||
        (R > 0 && (!aligned16(x) || !aligned16(dy) || !aligned16(dx) || (grad_sum && !aligned16(grad_sum)) ||
                   (dx_bf16 && !aligned16(dx_bf16)))) ||
        x_row_stride % 4 != 0 || dy_row_stride % 8 != 0)
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    if (R == 0) return launch_sum_slices(partials, dw, D, 0, 0, s);  // no rows: the weight gradient is zero
    if (dy_dtype == BNB_BF16)
        return dispatch_norm_bwd<uint16_t>(D, x, x_row_stride, dy, dy_row_stride, weight, eps, grad_sum, dx, (uint16_t *)dx_bf16,
                                           partials, blocks, dw, R, s);
    return dispatch_norm_bwd<float>(D, x, x_row_stride, dy, dy_row_stride, weight, eps, grad_sum, dx, (uint16_t *)dx_bf16, partials,
                                    blocks, dw, R, s);
}

extern "C" int64_t bnb_rmsnorm_bwd_static_limit(void) { return (int64_t)bnb::kNbMaxBlocks * bnb::kNbStaticMaxD * (int64_t)sizeof(float); }

extern "C" int bnb_rmsnorm_bwd_static(const float *x, int64_t x_row_stride, const void *dy, int dy_dtype, int64_t dy_row_stride,
                                      const float *weight, float eps, const float *grad_sum, float *dx, void *dx_bf16,
                                      float *dw, int64_t R, int D, void *stream)
{
    using namespace bnb;
    if (D > kNbStaticMaxD) return BNB_ERR_SCRATCH_LIMIT;
    const int blocks = bnb_rmsnorm_bwd_blocks(R, D);
    if ((int64_t)blocks * D > (int64_t)kNbMaxBlocks * kNbStaticMaxD) return BNB_ERR_SCRATCH_LIMIT;
    float *partials = nullptr;
    const int rc = scratch_address(&partials);
    if (rc != 0) return rc;
    // every partial row that is summed is written by this launch first: nothing to clear
    return bnb_rmsnorm_bwd(x, x_row_stride, dy, dy_dtype, dy_row_stride, weight, eps, grad_sum, dx, dx_bf16, partials, blocks, dw,
                           R, D, stream);
}
