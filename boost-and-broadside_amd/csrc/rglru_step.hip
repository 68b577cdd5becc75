// RG-LRU recurrence step for gfx950: one coalesced pass over the entity rows.
//
// Per element (reference: models/yemong/griffin.py:179-185):
//   r = sigmoid(ga), i = sigmoid(gx), a = sigmoid(lambda)^(c r),
//   h' = a h + sqrt(max((1-a)(1+a), 1e-6)) (i x)
// The kernel is bound by HBM traffic (x, two gate pre-activations and the old state in,
// the new state and its optional low-precision copy out), so the design is a plain
// streaming pass: every lane owns 8 consecutive channels of ONE row, moves them with
// 16-byte accesses (nontemporal once the launch outgrows the last-level cache) and keeps
// everything between load and store in registers.
// Measured on MI355X, one row per lane in large blocks streams faster than several rows in
// flight per lane (more, shorter waves beat deeper per-lane unrolling on this memory system),
// and what matters most is that each memory instruction of a wave covers one dense run of bytes
// (rglru_step_dense_kernel below, the form taken for the widths where it applies).

#include "common.h"
#include "rglru_math.h"

namespace bnb {

constexpr int kRglruThreads = 256;     // scalar path, and the vector path on small inputs
constexpr int kRglruBigThreads = 1024;  // vector path once the grid is large enough to fill the chip

template <int THREADS, typename XT, typename GT, typename YT, bool HAS_Y, bool STREAM>
__global__ __launch_bounds__(THREADS) void rglru_step_vec8_kernel(
    const XT *__restrict__ x, const GT *__restrict__ gates, const float *__restrict__ log_lambda, float c,
    const float *h_in, int64_t h_in_stride, float *h_out, int64_t h_out_stride, YT *__restrict__ y,
    int64_t R, int D, int rows_per_block, const uint8_t *__restrict__ reset, int rows_per_env,
    int64_t y_group_stride)
{
    extern __shared__ float s_l2sig[];  // D entries
    for (int d = threadIdx.x; d < D; d += THREADS) s_l2sig[d] = log2_sigmoid(log_lambda[d]);
    __syncthreads();

    const int vecs_per_row = D >> 3;
    const int local_row = threadIdx.x / vecs_per_row;
    const int64_t row = (int64_t)blockIdx.x * rows_per_block + local_row;
    if (local_row >= rows_per_block || row >= R) return;
    // two runs of four channels per lane (d0.. and gap + d0..): every access of a row's lanes is one dense run
    const int d0 = (threadIdx.x - local_row * vecs_per_row) << 2;
    const int gap = D >> 1;

    // STREAM: nontemporal accesses, best once the rows no longer fit the last-level cache; below
    // that size cached accesses let the producer's output be picked up on chip
    const Row8 xv = load8_split<STREAM>(x + row * D + d0, gap);
    const Row8 ga = load8_split<STREAM>(gates + row * 2 * D + d0, gap);
    const Row8 gx = load8_split<STREAM>(gates + row * 2 * D + D + d0, gap);
    Row8 hv = load8_split<STREAM>(h_in + row * h_in_stride + d0, gap);
    // environment of the row: for the reset flag and for an output laid out per environment
    const int64_t env = (reset != nullptr || y_group_stride != 0) ? row / rows_per_env : 0;
    if (reset != nullptr && reset[env]) {
        // the environment was reset before this step: its previous state reads as zero
#pragma unroll
        for (int e = 0; e < 8; ++e) hv.v[e] = 0.0f;
    }

    Row8 out;
#pragma unroll
    for (int e = 0; e < 8; ++e)
        out.v[e] = rglru_element<is_bf16<GT>::value, is_bf16<XT>::value>(xv.v[e], ga.v[e], gx.v[e],
                                                                          s_l2sig[d0 + (e & 3) + (e >> 2) * gap], c, hv.v[e]);
    store8_split<STREAM>(h_out + row * h_out_stride + d0, gap, out);
    if (HAS_Y) {
        // y rows either back to back or in groups of rows_per_env, y_group_stride elements apart
        const int64_t y_off = y_group_stride != 0 ? env * y_group_stride + (row - env * rows_per_env) * D : row * D;
        store8_split<STREAM>(y + y_off + d0, gap, out);
    }
}

// The same pass with a lane -> channel map under which EVERY memory instruction of a wave covers one
// dense run of bytes.  With 8 channels per lane the fp32 state moves as two 16-byte accesses whose
// lanes sit 32 bytes apart, so each instruction touches every other 16-byte piece of 2 KB: a plain
// copy with that pattern streams at 3.9-4.4 TB/s on MI355X against 6.4-6.5 TB/s for dense
// instructions (measured).  Here a wave spans 512 consecutive elements of the flattened (row, channel)
// index space and lane l owns elements 4l..4l+3 and 256+4l..256+4l+3: bf16 streams move as two dense
// 8-byte instructions (512 B each), fp32 streams as two dense 16-byte instructions (1 KB each).
template <int THREADS, typename XT, typename GT, typename YT, bool HAS_Y, bool STREAM>
__global__ __launch_bounds__(THREADS) void rglru_step_dense_kernel(
    const XT *__restrict__ x, const GT *__restrict__ gates, const float *__restrict__ log_lambda, float c,
    const float *h_in, int64_t h_in_stride, float *h_out, int64_t h_out_stride, YT *__restrict__ y,
    int64_t R, int D, int log2_d, const uint8_t *__restrict__ reset, int rows_per_env, int64_t y_group_stride)
{
    extern __shared__ float s_l2sig[];  // D entries
    for (int d = threadIdx.x; d < D; d += THREADS) s_l2sig[d] = log2_sigmoid(log_lambda[d]);
    __syncthreads();

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t first = ((int64_t)blockIdx.x * (THREADS >> 6) + wave) * 512 + 4 * lane;  // flattened element index
#pragma unroll
    for (int part = 0; part < 2; ++part) {
        const int64_t e = first + 256 * part;
        const int64_t row = e >> log2_d;  // D divides 512: a power of two
        if (row >= R) continue;
        const int d0 = (int)e & (D - 1);
        const Row4 xv = load4<STREAM>(x + row * D + d0);
        const Row4 ga = load4<STREAM>(gates + row * 2 * D + d0);
        const Row4 gx = load4<STREAM>(gates + row * 2 * D + D + d0);
        Row4 hv = load4<STREAM>(h_in + row * h_in_stride + d0);
        // rows fit 32 bits wherever a packed state of that many rows exists at all: one 32-bit division
        const int64_t env = (reset != nullptr || y_group_stride != 0)
                                ? (row <= 0xffffffffLL ? (int64_t)((uint32_t)row / (uint32_t)rows_per_env) : row / rows_per_env)
                                : 0;
        if (reset != nullptr && reset[env]) {
#pragma unroll
            for (int k = 0; k < 4; ++k) hv.v[k] = 0.0f;
        }
        Row4 out;
#pragma unroll
        for (int k = 0; k < 4; ++k)
            out.v[k] = rglru_element<is_bf16<GT>::value, is_bf16<XT>::value>(xv.v[k], ga.v[k], gx.v[k], s_l2sig[d0 + k], c, hv.v[k]);
        store4<STREAM>(h_out + row * h_out_stride + d0, out);
        if (HAS_Y) {
            const int64_t y_off = y_group_stride != 0 ? env * y_group_stride + (row - env * rows_per_env) * D : row * D;
            store4<STREAM>(y + y_off + d0, out);
        }
    }
}

// Any D, any alignment: one lane per element.
template <typename XT, typename GT, typename YT, bool HAS_Y>
__global__ __launch_bounds__(kRglruThreads) void rglru_step_scalar_kernel(
    const XT *__restrict__ x, const GT *__restrict__ gates, const float *__restrict__ log_lambda, float c,
    const float *h_in, int64_t h_in_stride, float *h_out, int64_t h_out_stride, YT *__restrict__ y,
    int64_t R, int D, const uint8_t *__restrict__ reset, int rows_per_env, int64_t y_group_stride)
{
    const int64_t idx = (int64_t)blockIdx.x * kRglruThreads + threadIdx.x;
    if (idx >= R * D) return;
    const int64_t row = idx / D;
    const int d = (int)(idx - row * D);
    const int64_t env = (reset != nullptr || y_group_stride != 0) ? row / rows_per_env : 0;
    const float h_prev = (reset != nullptr && reset[env]) ? 0.0f : h_in[row * h_in_stride + d];
    const float out = rglru_element<is_bf16<GT>::value, is_bf16<XT>::value>(
        load1(x + idx), load1(gates + row * 2 * D + d), load1(gates + row * 2 * D + D + d),
        log2_sigmoid(log_lambda[d]), c, h_prev);
    h_out[row * h_out_stride + d] = out;
    if (HAS_Y) {
        const int64_t y_off = y_group_stride != 0 ? env * y_group_stride + (row - env * rows_per_env) * D : row * D;
        store1(y + y_off + d, out);
    }
}

template <typename XT, typename GT, typename YT, bool HAS_Y>
static int launch_rglru(const void *x, const void *gates, const float *log_lambda, float c, const float *h_in,
                        int64_t h_in_stride, float *h_out, int64_t h_out_stride, void *y, int64_t R, int D,
                        const uint8_t *reset, int rows_per_env, int64_t y_group_stride, hipStream_t stream)
{
    const bool vec = (D % 8 == 0) && (D / 8 <= kRglruThreads) && aligned16(x) && aligned16(gates) &&
                     aligned16(h_in) && aligned16(h_out) && (!HAS_Y || aligned16(y)) &&
                     (h_in_stride % 4 == 0) && (h_out_stride % 4 == 0);
    if (vec) {
        const int vecs_per_row = D / 8;
        // big blocks amortise the per-block log2 sigmoid(lambda) table; keep small inputs spread out
        const bool big = vecs_per_row <= kRglruBigThreads && R * vecs_per_row >= (int64_t)kRglruBigThreads * 2048;
        const int threads = big ? kRglruBigThreads : kRglruThreads;
        const int rows_per_block = threads / vecs_per_row;
        const int64_t blocks = (R + rows_per_block - 1) / rows_per_block;
        if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
        // bytes the launch touches; MI355X keeps up to 256 MB in its last-level cache
        const size_t bytes = (size_t)R * D * (sizeof(XT) + 2 * sizeof(GT) + 2 * sizeof(float) + (HAS_Y ? sizeof(YT) : 0));
        const bool stream_hint = bytes > ((size_t)192 << 20);
#define BNB_RGLRU_LAUNCH(T, S)                                                                                        \
    hipLaunchKernelGGL((rglru_step_vec8_kernel<T, XT, GT, YT, HAS_Y, S>), dim3((unsigned)blocks), dim3(threads),         \
                       (size_t)D * sizeof(float), stream, (const XT *)x, (const GT *)gates, log_lambda, c, h_in,         \
                       h_in_stride, h_out, h_out_stride, (YT *)y, R, D, rows_per_block, reset, rows_per_env,             \
                       y_group_stride)
        // dense lane map (every wave spans 512 elements) whenever 512 is a whole number of rows: D = 128, 256, 512.
        // Measured at D = 128 bf16, 622,592 rows: 216 -> 202 us; 256-thread blocks are as fast as 1024-thread ones
        // there and faster on mid-sized inputs (327,680 rows: 107 against 111 us).
        if (512 % D == 0) {
            const int64_t waves = (R * (int64_t)D + 511) / 512;
            int log2_d = 0;
            while ((1 << log2_d) < D) ++log2_d;
            const int64_t dblocks = (waves + (kRglruThreads >> 6) - 1) / (kRglruThreads >> 6);
            if (dblocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
            if (stream_hint)
                hipLaunchKernelGGL((rglru_step_dense_kernel<kRglruThreads, XT, GT, YT, HAS_Y, true>), dim3((unsigned)dblocks),
                                   dim3(kRglruThreads), (size_t)D * sizeof(float), stream, (const XT *)x, (const GT *)gates,
                                   log_lambda, c, h_in, h_in_stride, h_out, h_out_stride, (YT *)y, R, D, log2_d, reset, rows_per_env,
                                   y_group_stride);
            else
                hipLaunchKernelGGL((rglru_step_dense_kernel<kRglruThreads, XT, GT, YT, HAS_Y, false>), dim3((unsigned)dblocks),
                                   dim3(kRglruThreads), (size_t)D * sizeof(float), stream, (const XT *)x, (const GT *)gates,
                                   log_lambda, c, h_in, h_in_stride, h_out, h_out_stride, (YT *)y, R, D, log2_d, reset, rows_per_env,
                                   y_group_stride);
            return (int)hipGetLastError();
        }
        if (big && stream_hint) BNB_RGLRU_LAUNCH(kRglruBigThreads, true);
        else if (big) BNB_RGLRU_LAUNCH(kRglruBigThreads, false);
        else if (stream_hint) BNB_RGLRU_LAUNCH(kRglruThreads, true);
        else BNB_RGLRU_LAUNCH(kRglruThreads, false);
#undef BNB_RGLRU_LAUNCH
    } else {
        const int64_t blocks = (R * D + kRglruThreads - 1) / kRglruThreads;
        if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((rglru_step_scalar_kernel<XT, GT, YT, HAS_Y>), dim3((unsigned)blocks),
                           dim3(kRglruThreads), 0, stream, (const XT *)x, (const GT *)gates, log_lambda, c,
                           h_in, h_in_stride, h_out, h_out_stride, (YT *)y, R, D, reset, rows_per_env, y_group_stride);
    }
    return (int)hipGetLastError();
}

template <typename XT, typename GT>
static int dispatch_y(const void *x, const void *gates, const float *log_lambda, float c, const float *h_in,
                      int64_t h_in_stride, float *h_out, int64_t h_out_stride, void *y, int y_dtype, int64_t R,
                      int D, const uint8_t *reset, int rows_per_env, int64_t y_group_stride, hipStream_t stream)
{
    if (y == nullptr)
        return launch_rglru<XT, GT, float, false>(x, gates, log_lambda, c, h_in, h_in_stride, h_out,
                                                  h_out_stride, nullptr, R, D, reset, rows_per_env, 0, stream);
    if (y_dtype == BNB_F32)
        return launch_rglru<XT, GT, float, true>(x, gates, log_lambda, c, h_in, h_in_stride, h_out,
                                                 h_out_stride, y, R, D, reset, rows_per_env, y_group_stride, stream);
    return launch_rglru<XT, GT, uint16_t, true>(x, gates, log_lambda, c, h_in, h_in_stride, h_out,
                                                h_out_stride, y, R, D, reset, rows_per_env, y_group_stride, stream);
}

}  // namespace bnb

extern "C" int bnb_rglru_step_rows_fwd(const void *x, int x_dtype, const void *gates_pre, int g_dtype,
                                       const float *log_lambda, float c, const float *h_in,
                                       int64_t h_in_row_stride, float *h_out, int64_t h_out_row_stride, void *y,
                                       int y_dtype, int64_t y_group_stride, const uint8_t *reset,
                                       int rows_per_env, int64_t R, int D, void *stream)
{
    using namespace bnb;
    if (R < 0 || D < 1) return BNB_ERR_BAD_SHAPE;
    if (R == 0) return 0;
    if (!x || !gates_pre || !log_lambda || !h_in || !h_out) return BNB_ERR_NULL_POINTER;
    if ((x_dtype != BNB_F32 && x_dtype != BNB_BF16) || (g_dtype != BNB_F32 && g_dtype != BNB_BF16) ||
        (y && y_dtype != BNB_F32 && y_dtype != BNB_BF16))
        return BNB_ERR_BAD_DTYPE;
    if (h_in_row_stride < D || h_out_row_stride < D) return BNB_ERR_BAD_SHAPE;
    if ((reset != nullptr || y_group_stride != 0) && rows_per_env < 1) return BNB_ERR_BAD_SHAPE;
    if (y_group_stride != 0 && (!y || y_group_stride < (int64_t)rows_per_env * D || y_group_stride % 8 != 0))
        return BNB_ERR_BAD_SHAPE;
    if ((reinterpret_cast<uintptr_t>(h_in) | reinterpret_cast<uintptr_t>(h_out) |
         reinterpret_cast<uintptr_t>(log_lambda)) & 3u)
        return BNB_ERR_MISALIGNED;
    if (reset == nullptr && y_group_stride == 0) rows_per_env = 1;
    hipStream_t s = (hipStream_t)stream;
    const bool xb = x_dtype == BNB_BF16, gb = g_dtype == BNB_BF16;
    if (!xb && !gb)
        return dispatch_y<float, float>(x, gates_pre, log_lambda, c, h_in, h_in_row_stride, h_out,
                                        h_out_row_stride, y, y_dtype, R, D, reset, rows_per_env, y_group_stride, s);
    if (xb && gb)
        return dispatch_y<uint16_t, uint16_t>(x, gates_pre, log_lambda, c, h_in, h_in_row_stride, h_out,
                                              h_out_row_stride, y, y_dtype, R, D, reset, rows_per_env, y_group_stride, s);
    if (!xb && gb)
        return dispatch_y<float, uint16_t>(x, gates_pre, log_lambda, c, h_in, h_in_row_stride, h_out,
                                           h_out_row_stride, y, y_dtype, R, D, reset, rows_per_env, y_group_stride, s);
    return dispatch_y<uint16_t, float>(x, gates_pre, log_lambda, c, h_in, h_in_row_stride, h_out,
                                       h_out_row_stride, y, y_dtype, R, D, reset, rows_per_env, y_group_stride, s);
}

extern "C" int bnb_rglru_step_reset_fwd(const void *x, int x_dtype, const void *gates_pre, int g_dtype,
                                        const float *log_lambda, float c, const float *h_in,
                                        int64_t h_in_row_stride, float *h_out, int64_t h_out_row_stride,
                                        void *y, int y_dtype, const uint8_t *reset, int rows_per_env, int64_t R,
                                        int D, void *stream)
{
    return bnb_rglru_step_rows_fwd(x, x_dtype, gates_pre, g_dtype, log_lambda, c, h_in, h_in_row_stride, h_out,
                                   h_out_row_stride, y, y_dtype, 0, reset, rows_per_env, R, D, stream);
}

extern "C" int bnb_rglru_step_fwd(const void *x, int x_dtype, const void *gates_pre, int g_dtype,
                                  const float *log_lambda, float c, const float *h_in,
                                  int64_t h_in_row_stride, float *h_out, int64_t h_out_row_stride, void *y,
                                  int y_dtype, int64_t R, int D, void *stream)
{
    return bnb_rglru_step_reset_fwd(x, x_dtype, gates_pre, g_dtype, log_lambda, c, h_in, h_in_row_stride, h_out,
                                    h_out_row_stride, y, y_dtype, nullptr, 1, R, D, stream);
}
