// Fused element-wise pieces of the trunk layers around the projections, for gfx950.
//
//   add_rmsnorm   s = x (+ delta);  n = s * rsqrt(mean(s^2) + eps) * weight
//                 one pass instead of: residual add, RMSNorm, and the fp32 -> bf16 cast that
//                 autocast inserts in front of the next Linear
//                 (reference: models/yemong/attention.py:97-98, models/yemong/griffin.py:269,
//                 284-285; nn.RMSNorm with eps = finfo(float32).eps)
//   gelu_mul      out = gelu(a) * b, exact (erf) GELU
//                 (reference: GatedMLP, attention.py:36-37; the gate branch of the temporal
//                 block, griffin.py:281-282)
//
// Both are pure streaming kernels: 8 channels per lane, nontemporal accesses, fp32
// arithmetic, roundings placed where torch's type promotion places them.

#include "common.h"

namespace bnb {

constexpr int kEwThreads = 256;

// ---- s = x (+ delta), n = rmsnorm(s) ------------------------------------------------------
// LANES = lanes per row (D / 8), a power of two <= 64, so the sum of squares is a butterfly
// inside the wavefront.
template <int LANES, typename DT, typename OT, bool HAS_DELTA, bool HAS_SUM>
__global__ __launch_bounds__(kEwThreads) void add_rmsnorm_kernel(
    const float *__restrict__ x, int64_t x_stride, const DT *__restrict__ delta, const float *__restrict__ weight,
    float eps, float *__restrict__ sum_out, OT *__restrict__ norm_out, int64_t R)
{
    constexpr int D = LANES * 8;
    constexpr int ROWS = kEwThreads / LANES;
    const int local_row = threadIdx.x / LANES;
    // a lane's eight channels are two runs of four, d0 .. d0 + 3 and D/2 + d0 ..: every access of a row's lanes is one
    // dense run of bytes
    const int d0 = (threadIdx.x - local_row * LANES) << 2;
    constexpr int gap = D / 2;
    const int64_t row = (int64_t)blockIdx.x * ROWS + local_row;
    const bool valid = row < R;  // keep every lane in the butterfly
    const int64_t r = valid ? row : R - 1;

    Row8 s = load8_split<true>(x + r * x_stride + d0, gap);
    if (HAS_DELTA) {
        const Row8 dl = load8_split<true>(delta + r * D + d0, gap);
#pragma unroll
        for (int e = 0; e < 8; ++e) s.v[e] += dl.v[e];
    }
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = fmaf(s.v[e], s.v[e], ss);
#pragma unroll
    for (int off = 1; off < LANES; off <<= 1) ss += __shfl_xor(ss, off);
    const float rstd = rsqrtf(ss * (1.0f / D) + eps);

    if (!valid) return;
    if (HAS_SUM) store8_split<true>(sum_out + row * D + d0, gap, s);
    const Row8 w = load8_split<false>(weight + d0, gap);
    Row8 n;
#pragma unroll
    for (int e = 0; e < 8; ++e) n.v[e] = (s.v[e] * rstd) * w.v[e];
    store8_split<true>(norm_out + row * D + d0, gap, n);
}

// ---- out = gelu(a) * b -----------------------------------------------------------------------
template <typename AT, typename BT, typename OT>
__global__ __launch_bounds__(kEwThreads) void gelu_mul_kernel(const AT *__restrict__ a, int64_t a_stride,
                                                              const BT *__restrict__ b, int64_t b_stride,
                                                              OT *__restrict__ out, int64_t R, int H)
{
    const int vecs_per_row = H >> 3;
    const int64_t idx = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
    if (idx >= R * vecs_per_row) return;
    const int64_t row = idx / vecs_per_row;
    const int c0 = (int)(idx - row * vecs_per_row) << 3;
    const Row8 av = load8_stream(a + row * a_stride + c0);
    const Row8 bv = load8_stream(b + row * b_stride + c0);
    Row8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float g = gelu_erf(av.v[e]);
        if (is_bf16<AT>::value) g = round_to_bf16(g);  // F.gelu returns its input's dtype
        o.v[e] = g * bv.v[e];
    }
    store8_stream(out + row * H + c0, o);
}

// ---- backward of out = gelu(a) * b:  da = dout * b * gelu'(a),  db = dout * gelu(a) -----------
// gelu'(v) = Phi(v) + v * phi(v); gelu(a) is rounded to a's dtype first, as the forward does.
template <typename AT, typename BT, typename OT>
__global__ __launch_bounds__(kEwThreads) void gelu_mul_bwd_kernel(const AT *__restrict__ a, int64_t a_stride,
                                                                  const BT *__restrict__ b, int64_t b_stride,
                                                                  const OT *__restrict__ dout, AT *__restrict__ da,
                                                                  int64_t da_stride, BT *__restrict__ db, int64_t db_stride,
                                                                  int64_t R, int H)
{
    const int vecs_per_row = H >> 3;
    const int64_t idx = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
    if (idx >= R * vecs_per_row) return;
    const int64_t row = idx / vecs_per_row;
    const int c0 = (int)(idx - row * vecs_per_row) << 3;
    const Row8 av = load8_stream(a + row * a_stride + c0);
    const Row8 bv = load8_stream(b + row * b_stride + c0);
    const Row8 gv = load8_stream(dout + row * H + c0);
    Row8 ga, gb;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float v = av.v[e];
        const float cdf = 0.5f * (1.0f + erff(v * 0.70710678118654752f));
        const float pdf = 0.3989422804014327f * __expf(-0.5f * v * v);
        float g = v * cdf;
        if (is_bf16<AT>::value) g = round_to_bf16(g);
        ga.v[e] = gv.v[e] * bv.v[e] * (cdf + v * pdf);
        gb.v[e] = gv.v[e] * g;
    }
    store8_stream(da + row * da_stride + c0, ga);
    store8_stream(db + row * db_stride + c0, gb);
}

template <int LANES, typename DT, typename OT>
static int launch_norm(const float *x, int64_t x_stride, const void *delta, const float *weight, float eps,
                       float *sum_out, void *norm_out, int64_t R, hipStream_t stream)
{
    constexpr int ROWS = kEwThreads / LANES;
    const int64_t blocks = (R + ROWS - 1) / ROWS;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    const dim3 g((unsigned)blocks), t(kEwThreads);
    const DT *dp = (const DT *)delta;
    OT *np = (OT *)norm_out;
    if (delta && sum_out)
        hipLaunchKernelGGL((add_rmsnorm_kernel<LANES, DT, OT, true, true>), g, t, 0, stream, x, x_stride, dp, weight, eps, sum_out, np, R);
    else if (delta)
        hipLaunchKernelGGL((add_rmsnorm_kernel<LANES, DT, OT, true, false>), g, t, 0, stream, x, x_stride, dp, weight, eps, sum_out, np, R);
    else
        hipLaunchKernelGGL((add_rmsnorm_kernel<LANES, DT, OT, false, false>), g, t, 0, stream, x, x_stride, dp, weight, eps, sum_out, np, R);
    return (int)hipGetLastError();
}

template <typename DT, typename OT>
static int dispatch_norm_lanes(int D, const float *x, int64_t x_stride, const void *delta, const float *weight,
                               float eps, float *sum_out, void *norm_out, int64_t R, hipStream_t stream)
{
    switch (D) {
        case 8: return launch_norm<1, DT, OT>(x, x_stride, delta, weight, eps, sum_out, norm_out, R, stream);
        case 16: return launch_norm<2, DT, OT>(x, x_stride, delta, weight, eps, sum_out, norm_out, R, stream);
        case 32: return launch_norm<4, DT, OT>(x, x_stride, delta, weight, eps, sum_out, norm_out, R, stream);
        case 64: return launch_norm<8, DT, OT>(x, x_stride, delta, weight, eps, sum_out, norm_out, R, stream);
        case 128: return launch_norm<16, DT, OT>(x, x_stride, delta, weight, eps, sum_out, norm_out, R, stream);
        case 256: return launch_norm<32, DT, OT>(x, x_stride, delta, weight, eps, sum_out, norm_out, R, stream);
        case 512: return launch_norm<64, DT, OT>(x, x_stride, delta, weight, eps, sum_out, norm_out, R, stream);
        default: return BNB_ERR_UNSUPPORTED;
    }
}

template <typename AT, typename BT, typename OT>
static int launch_gelu_mul(const void *a, int64_t a_stride, const void *b, int64_t b_stride, void *out, int64_t R,
                           int H, hipStream_t stream)
{
    const int64_t blocks = (R * (H / 8) + kEwThreads - 1) / kEwThreads;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((gelu_mul_kernel<AT, BT, OT>), dim3((unsigned)blocks), dim3(kEwThreads), 0, stream,
                       (const AT *)a, a_stride, (const BT *)b, b_stride, (OT *)out, R, H);
    return (int)hipGetLastError();
}

template <typename AT, typename BT, typename OT>
static int launch_gelu_mul_bwd(const void *a, int64_t a_stride, const void *b, int64_t b_stride, const void *dout, void *da,
                               int64_t da_stride, void *db, int64_t db_stride, int64_t R, int H, hipStream_t stream)
{
    const int64_t blocks = (R * (H / 8) + kEwThreads - 1) / kEwThreads;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((gelu_mul_bwd_kernel<AT, BT, OT>), dim3((unsigned)blocks), dim3(kEwThreads), 0, stream, (const AT *)a,
                       a_stride, (const BT *)b, b_stride, (const OT *)dout, (AT *)da, da_stride, (BT *)db, db_stride, R, H);
    return (int)hipGetLastError();
}

}  // namespace bnb

extern "C" int bnb_add_rmsnorm_fwd(const float *x, int64_t x_row_stride, const void *delta, int delta_dtype,
                                   const float *weight, float eps, float *sum_out, void *norm_out, int out_dtype,
                                   int64_t R, int D, void *stream)
{
    using namespace bnb;
    if (R < 0 || D < 1 || x_row_stride < D) return BNB_ERR_BAD_SHAPE;
    if (R == 0) return 0;
    if (!x || !weight || !norm_out) return BNB_ERR_NULL_POINTER;
    if (sum_out && !delta) return BNB_ERR_BAD_SHAPE;  // the sum is x itself without a delta
    if ((out_dtype != BNB_F32 && out_dtype != BNB_BF16) || (delta && delta_dtype != BNB_F32 && delta_dtype != BNB_BF16))
        return BNB_ERR_BAD_DTYPE;
    if (!aligned16(x) || !aligned16(norm_out) || !aligned16(weight) || (delta && !aligned16(delta)) ||
        (sum_out && !aligned16(sum_out)) || (x_row_stride % 4) != 0)
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    const bool db = delta && delta_dtype == BNB_BF16, ob = out_dtype == BNB_BF16;
    if (db && ob) return dispatch_norm_lanes<uint16_t, uint16_t>(D, x, x_row_stride, delta, weight, eps, sum_out, norm_out, R, s);
    if (db) return dispatch_norm_lanes<uint16_t, float>(D, x, x_row_stride, delta, weight, eps, sum_out, norm_out, R, s);
    if (ob) return dispatch_norm_lanes<float, uint16_t>(D, x, x_row_stride, delta, weight, eps, sum_out, norm_out, R, s);
    return dispatch_norm_lanes<float, float>(D, x, x_row_stride, delta, weight, eps, sum_out, norm_out, R, s);
}

extern "C" int bnb_gelu_mul_fwd(const void *a, int a_dtype, int64_t a_row_stride, const void *b, int b_dtype,
                                int64_t b_row_stride, void *out, int out_dtype, int64_t R, int H, void *stream)
{
    using namespace bnb;
    if (R < 0 || H < 1 || a_row_stride < H || b_row_stride < H) return BNB_ERR_BAD_SHAPE;
    if (R == 0) return 0;
    if (!a || !b || !out) return BNB_ERR_NULL_POINTER;
    for (int dt : {a_dtype, b_dtype, out_dtype})
        if (dt != BNB_F32 && dt != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (H % 8) return BNB_ERR_UNSUPPORTED;
    const int64_t ea = a_dtype == BNB_BF16 ? 2 : 4, eb = b_dtype == BNB_BF16 ? 2 : 4;
    if (!aligned16(a) || !aligned16(b) || !aligned16(out) || (a_row_stride * ea) % 16 || (b_row_stride * eb) % 16)
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    const int key = (a_dtype << 2) | (b_dtype << 1) | out_dtype;
    switch (key) {
        case 0: return launch_gelu_mul<float, float, float>(a, a_row_stride, b, b_row_stride, out, R, H, s);
        case 1: return launch_gelu_mul<float, float, uint16_t>(a, a_row_stride, b, b_row_stride, out, R, H, s);
        case 2: return launch_gelu_mul<float, uint16_t, float>(a, a_row_stride, b, b_row_stride, out, R, H, s);
        case 3: return launch_gelu_mul<float, uint16_t, uint16_t>(a, a_row_stride, b, b_row_stride, out, R, H, s);
        case 4: return launch_gelu_mul<uint16_t, float, float>(a, a_row_stride, b, b_row_stride, out, R, H, s);
        case 5: return launch_gelu_mul<uint16_t, float, uint16_t>(a, a_row_stride, b, b_row_stride, out, R, H, s);
        case 6: return launch_gelu_mul<uint16_t, uint16_t, float>(a, a_row_stride, b, b_row_stride, out, R, H, s);
        default: return launch_gelu_mul<uint16_t, uint16_t, uint16_t>(a, a_row_stride, b, b_row_stride, out, R, H, s);
    }
}

extern "C" int bnb_gelu_mul_bwd(const void *a, int a_dtype, int64_t a_row_stride, const void *b, int b_dtype,
                                int64_t b_row_stride, const void *dout, int out_dtype, void *da, int64_t da_row_stride,
                                void *db, int64_t db_row_stride, int64_t R, int H, void *stream)
{
    using namespace bnb;
    if (R < 0 || H < 1 || a_row_stride < H || b_row_stride < H || da_row_stride < H || db_row_stride < H) return BNB_ERR_BAD_SHAPE;
    if (R == 0) return 0;
    if (!a || !b || !dout || !da || !db) return BNB_ERR_NULL_POINTER;
    for (int dt : {a_dtype, b_dtype, out_dtype})
        if (dt != BNB_F32 && dt != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (H % 8) return BNB_ERR_UNSUPPORTED;
    const int64_t ea = a_dtype == BNB_BF16 ? 2 : 4, eb = b_dtype == BNB_BF16 ? 2 : 4;
    if (!aligned16(a) || !aligned16(b) || !aligned16(dout) || !aligned16(da) || !aligned16(db) || (a_row_stride * ea) % 16 ||
        (b_row_stride * eb) % 16 || (da_row_stride * ea) % 16 || (db_row_stride * eb) % 16)
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
#define BNB_GMB(AT, BT, OT) \
    return launch_gelu_mul_bwd<AT, BT, OT>(a, a_row_stride, b, b_row_stride, dout, da, da_row_stride, db, db_row_stride, R, H, s)
    const int key = (a_dtype << 2) | (b_dtype << 1) | out_dtype;
    switch (key) {
        case 0: BNB_GMB(float, float, float);
        case 1: BNB_GMB(float, float, uint16_t);
        case 2: BNB_GMB(float, uint16_t, float);
        case 3: BNB_GMB(float, uint16_t, uint16_t);
        case 4: BNB_GMB(uint16_t, float, float);
        case 5: BNB_GMB(uint16_t, float, uint16_t);
        case 6: BNB_GMB(uint16_t, uint16_t, float);
        default: BNB_GMB(uint16_t, uint16_t, uint16_t);
    }
#undef BNB_GMB
}
