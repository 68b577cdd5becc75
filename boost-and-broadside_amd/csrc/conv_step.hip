// Causal depthwise conv tap sum + conv-buffer shift for one timestep, for gfx950.
//
// Per row (reference: models/yemong/griffin.py:275-277 with the tap loop of :127-139 at T = 1):
//   padded = [p0, p1, p2, b1]            p* = the three previous linear1 outputs, oldest first
//   v      = sum_k padded[k] * w[:, k] + bias
//   new buffer = [p1, p2, b1]
// The previous buffer is read from, and the new one written into, the conv columns of a
// packed (.., 4D) state row (models/yemong/policy.py:323-324, :346-354), so neither the
// `cat` that builds `padded`, the eight element-wise tap kernels, nor the `cat` that repacks
// the state exist any more.  Pure HBM streaming: 8 channels of one row per lane, 16-byte
// nontemporal accesses, fp32 arithmetic in the reference's order (taps 0..3, then the bias).

#include "common.h"

namespace bnb {

constexpr int kConvThreads = 256;
constexpr int kConvBigThreads = 1024;
constexpr int kTaps = 4;

template <int THREADS, typename BT>
__global__ __launch_bounds__(THREADS) void conv_step_vec8_kernel(
    const BT *__restrict__ b1, const float *conv_in, int64_t conv_in_stride, const float *__restrict__ weight,
    const float *__restrict__ bias, const uint8_t *__restrict__ reset, int rows_per_env, float *__restrict__ v_out,
    uint16_t *__restrict__ v_bf16_out, float *conv_out, int64_t conv_out_stride, int64_t R, int D, int rows_per_block,
    int64_t b1_group_stride, int64_t b1_row_stride)
{
    extern __shared__ float s_wb[];  // D*4 tap weights (as stored: [d][k]) then D biases
    for (int i = threadIdx.x; i < D * kTaps; i += THREADS) s_wb[i] = weight[i];
    for (int i = threadIdx.x; i < D; i += THREADS) s_wb[D * kTaps + i] = bias != nullptr ? bias[i] : 0.0f;
    __syncthreads();

    const int vecs_per_row = D >> 3;
    const int local_row = threadIdx.x / vecs_per_row;
    const int64_t row = (int64_t)blockIdx.x * rows_per_block + local_row;
    if (local_row >= rows_per_block || row >= R) return;
    // the lane's eight channels are two runs of four, d0..d0+3 and gap+d0..gap+d0+3: every access of a row's lanes
    // is then one dense run of bytes (8 consecutive fp32 channels per lane stream a third slower on MI355X)
    const int d0 = (threadIdx.x - local_row * vecs_per_row) << 2;
    const int gap = D >> 1;

    // environment of the row: for the reset flag and for inputs laid out per environment
    // (groups of rows_per_env rows, b1_group_stride elements apart)
    const int64_t env = (reset != nullptr || b1_group_stride != 0) ? row / rows_per_env : 0;
    const int64_t b1_off =
        b1_group_stride != 0 ? env * b1_group_stride + (row - env * rows_per_env) * b1_row_stride : row * b1_row_stride;
    const Row8 cur = load8_split<true>(b1 + b1_off + d0, gap);
    const float *pin = conv_in + row * conv_in_stride + d0;
    Row8 p0 = load8_split<true>(pin, gap), p1 = load8_split<true>(pin + D, gap), p2 = load8_split<true>(pin + 2 * D, gap);
    if (reset != nullptr && reset[env]) {
        // the environment was reset before this step: its stored inputs read as zero
#pragma unroll
        for (int e = 0; e < 8; ++e) p0.v[e] = p1.v[e] = p2.v[e] = 0.0f;
    }

    Row8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float *w = s_wb + (d0 + (e & 3) + (e >> 2) * gap) * kTaps;
        float acc = p0.v[e] * w[0];
        acc += p1.v[e] * w[1];
        acc += p2.v[e] * w[2];
        acc += cur.v[e] * w[3];
        v.v[e] = acc + s_wb[D * kTaps + d0 + (e & 3) + (e >> 2) * gap];
    }
    store8_split<true>(v_out + row * D + d0, gap, v);
    if (v_bf16_out != nullptr) store8_split<true>(v_bf16_out + row * D + d0, gap, v);
    float *pout = conv_out + row * conv_out_stride + d0;
    store8_split<true>(pout, gap, p1);
    store8_split<true>(pout + D, gap, p2);
    store8_split<true>(pout + 2 * D, gap, cur);
}

// Any D, any alignment: one lane per element.
template <typename BT>
__global__ __launch_bounds__(kConvThreads) void conv_step_scalar_kernel(
    const BT *__restrict__ b1, const float *conv_in, int64_t conv_in_stride, const float *__restrict__ weight,
    const float *__restrict__ bias, const uint8_t *__restrict__ reset, int rows_per_env, float *__restrict__ v_out,
    uint16_t *__restrict__ v_bf16_out, float *conv_out, int64_t conv_out_stride, int64_t R, int D,
    int64_t b1_group_stride, int64_t b1_row_stride)
{
    const int64_t idx = (int64_t)blockIdx.x * kConvThreads + threadIdx.x;
    if (idx >= R * D) return;
    const int64_t row = idx / D;
    const int d = (int)(idx - row * D);
    const int64_t env = (reset != nullptr || b1_group_stride != 0) ? row / rows_per_env : 0;
    const int64_t b1_off =
        b1_group_stride != 0 ? env * b1_group_stride + (row - env * rows_per_env) * b1_row_stride : row * b1_row_stride;
    const bool zero = reset != nullptr && reset[env];
    const float *pin = conv_in + row * conv_in_stride + d;
    const float p0 = zero ? 0.0f : pin[0], p1 = zero ? 0.0f : pin[D], p2 = zero ? 0.0f : pin[2 * D];
    const float cur = load1(b1 + b1_off + d);
    const float *w = weight + (int64_t)d * kTaps;
    float acc = p0 * w[0];
    acc += p1 * w[1];
    acc += p2 * w[2];
    acc += cur * w[3];
    const float v = acc + (bias != nullptr ? bias[d] : 0.0f);
    v_out[idx] = v;
    if (v_bf16_out != nullptr) store1(v_bf16_out + idx, v);
    float *pout = conv_out + row * conv_out_stride + d;
    pout[0] = p1;
    pout[D] = p2;
    pout[2 * D] = cur;
}

template <typename BT>
static int launch_conv(const void *b1, const float *conv_in, int64_t conv_in_stride, const float *weight,
                       const float *bias, const uint8_t *reset, int rows_per_env, float *v_out, uint16_t *v_bf16_out,
                       float *conv_out, int64_t conv_out_stride, int64_t R, int D, int64_t b1_group_stride,
                       int64_t b1_row_stride, hipStream_t stream)
{
    const bool vec = (D % 8 == 0) && (D / 8 <= kConvThreads) && aligned16(b1) && (b1_row_stride % 8 == 0) && aligned16(conv_in) &&
                     aligned16(conv_out) && aligned16(v_out) && aligned16(v_bf16_out) && (conv_in_stride % 4 == 0) &&
                     (conv_out_stride % 4 == 0) && (size_t)D * (kTaps + 1) * sizeof(float) <= 48 * 1024;
    if (vec) {
        const int vecs_per_row = D / 8;
        const bool big = R * vecs_per_row >= (int64_t)kConvBigThreads * 2048;
        const int threads = big ? kConvBigThreads : kConvThreads;
        const int rows_per_block = threads / vecs_per_row;
        const int64_t blocks = (R + rows_per_block - 1) / rows_per_block;
        if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
        const size_t lds = (size_t)D * (kTaps + 1) * sizeof(float);
        if (big)
            hipLaunchKernelGGL((conv_step_vec8_kernel<kConvBigThreads, BT>), dim3((unsigned)blocks), dim3(threads), lds,
                               stream, (const BT *)b1, conv_in, conv_in_stride, weight, bias, reset, rows_per_env,
                               v_out, v_bf16_out, conv_out, conv_out_stride, R, D, rows_per_block, b1_group_stride, b1_row_stride);
        else
            hipLaunchKernelGGL((conv_step_vec8_kernel<kConvThreads, BT>), dim3((unsigned)blocks), dim3(threads), lds,
                               stream, (const BT *)b1, conv_in, conv_in_stride, weight, bias, reset, rows_per_env,
                               v_out, v_bf16_out, conv_out, conv_out_stride, R, D, rows_per_block, b1_group_stride, b1_row_stride);
    } else {
        const int64_t blocks = (R * D + kConvThreads - 1) / kConvThreads;
        if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((conv_step_scalar_kernel<BT>), dim3((unsigned)blocks), dim3(kConvThreads), 0, stream,
                           (const BT *)b1, conv_in, conv_in_stride, weight, bias, reset, rows_per_env, v_out,
                           v_bf16_out, conv_out, conv_out_stride, R, D, b1_group_stride, b1_row_stride);
    }
    return (int)hipGetLastError();
}

}  // namespace bnb

extern "C" int bnb_conv_step_rows_fwd(const void *b1, int b1_dtype, int64_t b1_group_stride, int64_t b1_row_stride,
                                      const float *conv_in,
                                      int64_t conv_in_row_stride, const float *weight, const float *bias,
                                      const uint8_t *reset, int rows_per_env, float *v_out, void *v_bf16_out,
                                      float *conv_out, int64_t conv_out_row_stride, int64_t R, int D, void *stream)
{
    using namespace bnb;
    if (R < 0 || D < 1) return BNB_ERR_BAD_SHAPE;
    if (R == 0) return 0;
    if (!b1 || !conv_in || !weight || !v_out || !conv_out) return BNB_ERR_NULL_POINTER;
    if (b1_dtype != BNB_F32 && b1_dtype != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (conv_in_row_stride < 3 * (int64_t)D || conv_out_row_stride < 3 * (int64_t)D) return BNB_ERR_BAD_SHAPE;
    if ((reset != nullptr || b1_group_stride != 0) && rows_per_env < 1) return BNB_ERR_BAD_SHAPE;
    if (b1_row_stride == 0) b1_row_stride = D;
    if (b1_row_stride < D) return BNB_ERR_BAD_SHAPE;
    if (b1_group_stride != 0 && (b1_group_stride < (int64_t)rows_per_env * b1_row_stride || b1_group_stride % 8 != 0))
        return BNB_ERR_BAD_SHAPE;
    if ((reinterpret_cast<uintptr_t>(conv_in) | reinterpret_cast<uintptr_t>(conv_out) |
         reinterpret_cast<uintptr_t>(v_out) | reinterpret_cast<uintptr_t>(weight) |
         reinterpret_cast<uintptr_t>(bias)) & 3u)
        return BNB_ERR_MISALIGNED;
    if (reinterpret_cast<uintptr_t>(v_bf16_out) & 1u) return BNB_ERR_MISALIGNED;
    if (reset == nullptr && b1_group_stride == 0) rows_per_env = 1;
    hipStream_t s = (hipStream_t)stream;
    if (b1_dtype == BNB_BF16)
        return launch_conv<uint16_t>(b1, conv_in, conv_in_row_stride, weight, bias, reset, rows_per_env, v_out,
                                     (uint16_t *)v_bf16_out, conv_out, conv_out_row_stride, R, D, b1_group_stride,
                                     b1_row_stride, s);
    return launch_conv<float>(b1, conv_in, conv_in_row_stride, weight, bias, reset, rows_per_env, v_out,
                              (uint16_t *)v_bf16_out, conv_out, conv_out_row_stride, R, D, b1_group_stride,
                                     b1_row_stride, s);
}

extern "C" int bnb_conv_step_fwd(const void *b1, int b1_dtype, const float *conv_in, int64_t conv_in_row_stride,
                                 const float *weight, const float *bias, const uint8_t *reset, int rows_per_env,
                                 float *v_out, void *v_bf16_out, float *conv_out, int64_t conv_out_row_stride,
                                 int64_t R, int D, void *stream)
{
    return bnb_conv_step_rows_fwd(b1, b1_dtype, 0, 0, conv_in, conv_in_row_stride, weight, bias, reset, rows_per_env,
                                  v_out, v_bf16_out, conv_out, conv_out_row_stride, R, D, stream);
}
