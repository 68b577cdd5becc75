// Temporal sublayer over a whole sequence for gfx950: the causal depthwise conv and the
// RG-LRU recurrence, each as ONE pass over (rows, T, D).
//
// Reference: models/yemong/griffin.py:96-140 (tap loop with episode-aware validity,
// :67-93) and :188-219 (gates, decay, Hillis-Steele scan :25-64).  The reference evaluates
// h_t = a_t h_{t-1} + b_t with a log-depth scan, log2(T) rounds of full-tensor element-wise
// kernels over padded copies of a and b; here every lane owns 8 channels of one row and
// simply walks t = 0..T-1 with the state in registers: x and the gate pre-activations are
// read once, y is written once, a and b never exist in memory.  `done[r, t]` ends an episode
// at t: step t+1 starts from a zero state (:213-218) and its conv taps do not reach back
// across the boundary (:67-93).  Loads for several timesteps are issued before the
// dependent arithmetic, so the sequential recurrence does not serialise the memory traffic.
// The recurrence also has a backward kernel (reverse-time walk) so that the update path of
// training can use it.

#include "common.h"
#include "rglru_math.h"

namespace bnb {

constexpr int kSeqThreads = 256;
constexpr int kSeqTaps = 4;
constexpr int kSeqAhead = 4;  // timesteps whose operands are in flight together
constexpr int kScalarAhead = 16;  // the same for the forward one-lane-per-channel forms (few waves per SIMD there: more steps per lane)

// A time-major tensor may hold this call's rows inside a wider token tensor (T, environments * pitch, D): the rows of
// environment b are then rows b * pitch .. b * pitch + group - 1 of every step (group == 0: the tensor holds this
// call's rows only).  The update path keeps ship and field tokens of a sublayer in one tensor that way.
__device__ __forceinline__ int64_t placed_row(int64_t row, int group, int pitch)
{
    if (group <= 0) return row;
    const int64_t b = row / group;
    return b * pitch + (row - b * group);
}

// ------------------------------------------------------------------------------------
// RG-LRU over T steps
// ------------------------------------------------------------------------------------

template <typename XT, typename GT, typename YT>
__global__ __launch_bounds__(kSeqThreads) void rglru_scan_vec8_kernel(
    const XT *__restrict__ x, const GT *__restrict__ gates, const float *__restrict__ log_lambda, float c,
    const float *__restrict__ h0, int64_t h0_stride, const uint8_t *__restrict__ done, YT *__restrict__ y,
    float *__restrict__ h_last, int64_t h_last_stride, int64_t R, int T, int D, int64_t rs, int64_t ts, int rows_per_block,
    int y_group, int y_pitch, int64_t ts_y)
{
    extern __shared__ float s_l2sig[];  // D entries
    for (int d = threadIdx.x; d < D; d += kSeqThreads) s_l2sig[d] = log2_sigmoid(log_lambda[d]);
    __syncthreads();

    const int vecs_per_row = D >> 3;
    const int local_row = threadIdx.x / vecs_per_row;
    const int64_t row = (int64_t)blockIdx.x * rows_per_block + local_row;
    if (local_row >= rows_per_block || row >= R) return;
    const int d0 = (threadIdx.x - local_row * vecs_per_row) << 2;  // first of the lane's two runs of four channels
    const int gap = D >> 1;        // the second run starts here: every access of a row's lanes is one dense run

    float l2[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) l2[e] = s_l2sig[d0 + (e & 3) + (e >> 2) * gap];
    Row8 h = load8_split<false>(h0 + row * h0_stride + d0, gap);
    const XT *xp = x + row * rs + d0;
    const GT *gp = gates + row * 2 * rs + d0;
    YT *yp = y + placed_row(row, y_group, y_pitch) * rs + d0;
    const uint8_t *dn = done == nullptr ? nullptr : done + row * T;

    for (int t0 = 0; t0 < T; t0 += kSeqAhead) {
        Row8 xv[kSeqAhead], ga[kSeqAhead], gx[kSeqAhead];
        uint32_t cut[kSeqAhead];
#pragma unroll
        for (int u = 0; u < kSeqAhead; ++u) {
            // past the end: re-read the last step (discarded) so the loads stay branch-free
            const int t = t0 + u < T ? t0 + u : T - 1;
            xv[u] = load8_split<true>(xp + t * ts, gap);
            ga[u] = load8_split<true>(gp + t * 2 * ts, gap);
            gx[u] = load8_split<true>(gp + t * 2 * ts + D, gap);
            cut[u] = 0;
            if (dn != nullptr) cut[u] = dn[t > 0 ? t - 1 : 0];
            if (t == 0) cut[u] = 0;  // the first step continues the stored state
        }
#pragma unroll
        for (int u = 0; u < kSeqAhead; ++u) {
            if (t0 + u < T) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float prev = cut[u] ? 0.0f : h.v[e];
                    h.v[e] = rglru_element<is_bf16<GT>::value, is_bf16<XT>::value>(xv[u].v[e], ga[u].v[e], gx[u].v[e],
                                                                                    l2[e], c, prev);
                }
                store8_split<true>(yp + (t0 + u) * ts_y, gap, h);
            }
        }
    }
    store8_split<false>(h_last + row * h_last_stride + d0, gap, h);
}

// Any D, any alignment, and small inputs (eight times the lanes): one lane per (row, channel).
template <typename XT, typename GT, typename YT>
__global__ __launch_bounds__(kSeqThreads) void rglru_scan_scalar_kernel(
    const XT *__restrict__ x, const GT *__restrict__ gates, const float *__restrict__ log_lambda, float c,
    const float *__restrict__ h0, int64_t h0_stride, const uint8_t *__restrict__ done, YT *__restrict__ y,
    float *__restrict__ h_last, int64_t h_last_stride, int64_t R, int T, int D, int64_t rs, int64_t ts, int y_group,
    int y_pitch, int64_t ts_y)
{
    const int64_t idx = (int64_t)blockIdx.x * kSeqThreads + threadIdx.x;
    if (idx >= R * D) return;
    const int64_t row = idx / D;
    const int d = (int)(idx - row * D);
    const float l2 = log2_sigmoid(log_lambda[d]);
    float h = h0[row * h0_stride + d];
    const XT *xp = x + row * rs + d;
    const GT *gp = gates + row * 2 * rs + d;
    YT *yp = y + placed_row(row, y_group, y_pitch) * rs + d;
    const uint8_t *dn = done == nullptr ? nullptr : done + row * T;
    for (int t0 = 0; t0 < T; t0 += kScalarAhead) {
        float xv[kScalarAhead], ga[kScalarAhead], gx[kScalarAhead];
        uint32_t cut[kScalarAhead];
#pragma unroll
        for (int u = 0; u < kScalarAhead; ++u) {
            const int t = t0 + u < T ? t0 + u : T - 1;
            xv[u] = load1(xp + t * ts);
            ga[u] = load1(gp + t * 2 * ts);
            gx[u] = load1(gp + t * 2 * ts + D);
            cut[u] = 0;
            if (dn != nullptr) cut[u] = dn[t > 0 ? t - 1 : 0];
            if (t == 0) cut[u] = 0;
        }
#pragma unroll
        for (int u = 0; u < kScalarAhead; ++u) {
            if (t0 + u < T) {
                h = rglru_element<is_bf16<GT>::value, is_bf16<XT>::value>(xv[u], ga[u], gx[u], l2, c,
                                                                          cut[u] ? 0.0f : h);
                store1(yp + (t0 + u) * ts_y, h);
            }
        }
    }
    h_last[row * h_last_stride + d] = h;
}

template <typename XT, typename GT, typename YT>
static int launch_scan(const void *x, const void *gates, const float *log_lambda, float c, const float *h0,
                       int64_t h0_stride, const uint8_t *done, void *y, float *h_last, int64_t h_last_stride,
                       int64_t R, int T, int D, int time_major, int y_group, int y_pitch, hipStream_t stream)
{
    // element strides of one row / one timestep: (R, T, D) or (T, R, D)
    const int64_t rs = time_major ? D : (int64_t)T * D, ts = time_major ? R * D : D;
    const int64_t ts_y = y_group > 0 ? R / y_group * y_pitch * D : ts;
    const bool vec_ok = (D % 8 == 0) && (D / 8 <= kSeqThreads) && aligned16(x) && aligned16(gates) && aligned16(h0) &&
                        aligned16(h_last) && aligned16(y) && (h0_stride % 4 == 0) && (h_last_stride % 4 == 0);
    // the wide lanes need enough rows to fill the chip; below that one lane per channel
    const bool vec = vec_ok && R * (D / 8) >= (int64_t)256 * kSeqThreads * 2;
    if (vec) {
        const int rows_per_block = kSeqThreads / (D / 8);
        const int64_t blocks = (R + rows_per_block - 1) / rows_per_block;
        if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((rglru_scan_vec8_kernel<XT, GT, YT>), dim3((unsigned)blocks), dim3(kSeqThreads),
                           (size_t)D * sizeof(float), stream, (const XT *)x, (const GT *)gates, log_lambda, c, h0,
                           h0_stride, done, (YT *)y, h_last, h_last_stride, R, T, D, rs, ts, rows_per_block, y_group, y_pitch,
                           ts_y);
    } else {
        const int64_t blocks = (R * D + kSeqThreads - 1) / kSeqThreads;
        if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((rglru_scan_scalar_kernel<XT, GT, YT>), dim3((unsigned)blocks), dim3(kSeqThreads), 0,
                           stream, (const XT *)x, (const GT *)gates, log_lambda, c, h0, h0_stride, done, (YT *)y,
                           h_last, h_last_stride, R, T, D, rs, ts, y_group, y_pitch, ts_y);
    }
    return (int)hipGetLastError();
}

template <typename XT, typename GT>
static int scan_dispatch_y(const void *x, const void *gates, const float *log_lambda, float c, const float *h0,
                           int64_t h0_stride, const uint8_t *done, void *y, int y_dtype, float *h_last,
                           int64_t h_last_stride, int64_t R, int T, int D, int time_major, int y_group, int y_pitch,
                           hipStream_t stream)
{
    if (y_dtype == BNB_F32)
        return launch_scan<XT, GT, float>(x, gates, log_lambda, c, h0, h0_stride, done, y, h_last, h_last_stride, R,
                                          T, D, time_major, y_group, y_pitch, stream);
    return launch_scan<XT, GT, uint16_t>(x, gates, log_lambda, c, h0, h0_stride, done, y, h_last, h_last_stride, R, T,
                                         D, time_major, y_group, y_pitch, stream);
}

// ------------------------------------------------------------------------------------
// RG-LRU over T steps, backward
// ------------------------------------------------------------------------------------
//
// Reverse-time walk with the running state gradient in registers:
//   G_t   = dy_t + a'_{t+1} G_{t+1}            (a' = 0 across an episode boundary)
//   da_t  = G_t h_{t-1}  (0 at a boundary)  -  [s_t > 1e-6] G_t (i x)_t a_t / g_t
//   d(ix) = G_t g_t,  dx = d(ix) i,  di = d(ix) x
//   d ga  = da a ln(sigmoid(lambda)) c r (1 - r),   d gx = di i (1 - i)
//   d lambda += da a (c r) (1 - sigmoid(lambda))
// r, i, a, g are recomputed from the saved inputs exactly as the forward computed them
// (roundings included); h_{t-1} is read from the saved states.

struct RglruGrad {
    float dx, dga, dgx, dlam, carry;
};

template <bool G_BF16, bool X_BF16>
__device__ __forceinline__ RglruGrad rglru_element_bwd(float x, float ga, float gx, float l2sig, float one_minus_sig,
                                                        float c, float h_prev, float G)
{
    float r = fast_sigmoid(ga);
    float i = fast_sigmoid(gx);
    float cr = c * r;
    if (G_BF16) {
        r = round_to_bf16(r);
        i = round_to_bf16(i);
        cr = round_to_bf16(c * r);
    }
    const float a = __builtin_amdgcn_exp2f(cr * l2sig);
    const float s = (1.0f - a) * (1.0f + a);
    const float gate = __builtin_amdgcn_sqrtf(fmaxf(s, 1e-6f));
    float ix = i * x;
    if (G_BF16 && X_BF16) ix = round_to_bf16(ix);
    float da = G * h_prev;
    if (s > 1e-6f) da -= G * ix * a * __builtin_amdgcn_rcpf(gate);
    const float dix = G * gate;
    RglruGrad out;
    out.dx = dix * i;
    out.dgx = dix * x * i * (1.0f - i);
    const float da_a = da * a;
    out.dga = da_a * (l2sig * 0.6931471805599453f) * c * r * (1.0f - r);
    out.dlam = da_a * cr * one_minus_sig;
    out.carry = a * G;
    return out;
}

// 1 - sigmoid(lambda) = sigmoid(-lambda)
__device__ __forceinline__ float sigmoid_neg(float lam) { return 1.0f / (1.0f + expf(lam)); }

template <typename XT, typename GT, typename YT>
__global__ __launch_bounds__(kSeqThreads) void rglru_scan_bwd_scalar_kernel(
    const XT *__restrict__ x, const GT *__restrict__ gates, const float *__restrict__ log_lambda, float c,
    const float *__restrict__ h0, int64_t h0_stride, const uint8_t *__restrict__ done, const YT *__restrict__ y,
    const YT *__restrict__ dy, const float *__restrict__ dh_last, int64_t dh_last_stride, XT *__restrict__ dx,
    GT *__restrict__ dgates, float *__restrict__ dh0, float *__restrict__ dlam_rows, int64_t R, int T, int D,
    int64_t rs, int64_t ts, int y_group, int y_pitch, int64_t ts_y)
{
    const int64_t idx = (int64_t)blockIdx.x * kSeqThreads + threadIdx.x;
    if (idx >= R * D) return;
    const int64_t row = idx / D;
    const int d = (int)(idx - row * D);
    const float lam = log_lambda[d];
    const float l2 = log2_sigmoid(lam), oms = sigmoid_neg(lam);
    const XT *xp = x + row * rs + d;
    const GT *gp = gates + row * 2 * rs + d;
    const int64_t at_y = placed_row(row, y_group, y_pitch) * rs;  // y and dy: possibly rows of a wider token tensor
    const YT *yp = y + at_y + d;
    const YT *dyp = dy == nullptr ? nullptr : dy + at_y + d;
    XT *dxp = dx + row * rs + d;
    GT *dgp = dgates + row * 2 * rs + d;
    const uint8_t *dn = done == nullptr ? nullptr : done + row * T;
    const float h_first = h0[row * h0_stride + d];
    float carry = dh_last == nullptr ? 0.0f : dh_last[row * dh_last_stride + d];
    float dlam = 0.0f;
    for (int t1 = T; t1 > 0; t1 -= kSeqAhead) {
        float xv[kSeqAhead], ga[kSeqAhead], gx[kSeqAhead], dyv[kSeqAhead], hp[kSeqAhead];
        uint32_t cut[kSeqAhead];
#pragma unroll
        for (int u = 0; u < kSeqAhead; ++u) {
            const int t = t1 - 1 - u > 0 ? t1 - 1 - u : 0;  // before the start: re-read step 0 (discarded)
            xv[u] = load1(xp + t * ts);
            ga[u] = load1(gp + t * 2 * ts);
            gx[u] = load1(gp + t * 2 * ts + D);
            dyv[u] = dyp == nullptr ? 0.0f : load1(dyp + t * ts_y);
            hp[u] = load1(yp + (t > 0 ? t - 1 : 0) * ts_y);
            cut[u] = 0;
            if (dn != nullptr) cut[u] = dn[t > 0 ? t - 1 : 0];
            if (t == 0) {
                cut[u] = 0;
                hp[u] = h_first;
            }
        }
#pragma unroll
        for (int u = 0; u < kSeqAhead; ++u) {
            const int t = t1 - 1 - u;
            if (t >= 0) {
                const float G = dyv[u] + carry;
                const RglruGrad g = rglru_element_bwd<is_bf16<GT>::value, is_bf16<XT>::value>(
                    xv[u], ga[u], gx[u], l2, oms, c, cut[u] ? 0.0f : hp[u], G);
                store1(dxp + t * ts, g.dx);
                store1(dgp + t * 2 * ts, g.dga);
                store1(dgp + t * 2 * ts + D, g.dgx);
                dlam += g.dlam;
                carry = cut[u] ? 0.0f : g.carry;
            }
        }
    }
    dh0[row * D + d] = carry;
    dlam_rows[row * D + d] = dlam;
}

template <typename XT, typename GT, typename YT>
__global__ __launch_bounds__(kSeqThreads) void rglru_scan_bwd_vec8_kernel(
    const XT *__restrict__ x, const GT *__restrict__ gates, const float *__restrict__ log_lambda, float c,
    const float *__restrict__ h0, int64_t h0_stride, const uint8_t *__restrict__ done, const YT *__restrict__ y,
    const YT *__restrict__ dy, const float *__restrict__ dh_last, int64_t dh_last_stride, XT *__restrict__ dx,
    GT *__restrict__ dgates, float *__restrict__ dh0, float *__restrict__ dlam_rows, int64_t R, int T, int D,
    int64_t rs, int64_t ts, int rows_per_block, int y_group, int y_pitch, int64_t ts_y)
{
    extern __shared__ float s_lam[];  // D entries of log2 sigmoid(lambda), then D of 1 - sigmoid(lambda)
    for (int d = threadIdx.x; d < D; d += kSeqThreads) {
        const float lam = log_lambda[d];
        s_lam[d] = log2_sigmoid(lam);
        s_lam[D + d] = sigmoid_neg(lam);
    }
    __syncthreads();

    const int vecs_per_row = D >> 3;
    const int local_row = threadIdx.x / vecs_per_row;
    const int64_t row = (int64_t)blockIdx.x * rows_per_block + local_row;
    if (local_row >= rows_per_block || row >= R) return;
    const int d0 = (threadIdx.x - local_row * vecs_per_row) << 2;  // first of the lane's two runs of four channels
    const int gap = D >> 1;        // the second run starts here: every access of a row's lanes is one dense run

    float l2[8], oms[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        l2[e] = s_lam[d0 + (e & 3) + (e >> 2) * gap];
        oms[e] = s_lam[D + d0 + (e & 3) + (e >> 2) * gap];
    }
    const XT *xp = x + row * rs + d0;
    const GT *gp = gates + row * 2 * rs + d0;
    const int64_t at_y = placed_row(row, y_group, y_pitch) * rs;  // y and dy: possibly rows of a wider token tensor
    const YT *yp = y + at_y + d0;
    const YT *dyp = dy == nullptr ? nullptr : dy + at_y + d0;
    XT *dxp = dx + row * rs + d0;
    GT *dgp = dgates + row * 2 * rs + d0;
    const uint8_t *dn = done == nullptr ? nullptr : done + row * T;
    const Row8 h_first = load8_split<false>(h0 + row * h0_stride + d0, gap);
    Row8 carry, dlam;
#pragma unroll
    for (int e = 0; e < 8; ++e) carry.v[e] = dlam.v[e] = 0.0f;
    if (dh_last != nullptr) carry = load8_split<false>(dh_last + row * dh_last_stride + d0, gap);

    constexpr int AHEAD = 2;  // five operand rows per step: keep the register footprint moderate
    for (int t1 = T; t1 > 0; t1 -= AHEAD) {
        Row8 xv[AHEAD], ga[AHEAD], gx[AHEAD], dyv[AHEAD], hp[AHEAD];
        uint32_t cut[AHEAD];
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            const int t = t1 - 1 - u > 0 ? t1 - 1 - u : 0;
            xv[u] = load8_split<true>(xp + t * ts, gap);
            ga[u] = load8_split<true>(gp + t * 2 * ts, gap);
            gx[u] = load8_split<true>(gp + t * 2 * ts + D, gap);
            if (dyp != nullptr) {
                dyv[u] = load8_split<true>(dyp + t * ts_y, gap);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) dyv[u].v[e] = 0.0f;
            }
            hp[u] = load8_split<false>(yp + (t > 0 ? t - 1 : 0) * ts_y, gap);
            cut[u] = 0;
            if (dn != nullptr) cut[u] = dn[t > 0 ? t - 1 : 0];
            if (t == 0) {
                cut[u] = 0;
                hp[u] = h_first;
            }
        }
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            const int t = t1 - 1 - u;
            if (t >= 0) {
                Row8 ox, oa, og;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float G = dyv[u].v[e] + carry.v[e];
                    const RglruGrad g = rglru_element_bwd<is_bf16<GT>::value, is_bf16<XT>::value>(
                        xv[u].v[e], ga[u].v[e], gx[u].v[e], l2[e], oms[e], c, cut[u] ? 0.0f : hp[u].v[e], G);
                    ox.v[e] = g.dx;
                    oa.v[e] = g.dga;
                    og.v[e] = g.dgx;
                    dlam.v[e] += g.dlam;
                    carry.v[e] = cut[u] ? 0.0f : g.carry;
                }
                store8_split<true>(dxp + t * ts, gap, ox);
                store8_split<true>(dgp + t * 2 * ts, gap, oa);
                store8_split<true>(dgp + t * 2 * ts + D, gap, og);
            }
        }
    }
    store8_split<false>(dh0 + row * D + d0, gap, carry);
    store8_split<false>(dlam_rows + row * D + d0, gap, dlam);
}

template <typename XT, typename GT, typename YT>
static int launch_scan_bwd(const void *x, const void *gates, const float *log_lambda, float c, const float *h0,
                           int64_t h0_stride, const uint8_t *done, const void *y, const void *dy,
                           const float *dh_last, int64_t dh_last_stride, void *dx, void *dgates, float *dh0,
                           float *dlam_rows, int64_t R, int T, int D, int time_major, int y_group, int y_pitch,
                           hipStream_t stream)
{
    const int64_t rs = time_major ? D : (int64_t)T * D, ts = time_major ? R * D : D;
    const int64_t ts_y = y_group > 0 ? R / y_group * y_pitch * D : ts;
    const bool vec_ok = (D % 8 == 0) && (D / 8 <= kSeqThreads) && aligned16(x) && aligned16(gates) && aligned16(h0) &&
                        aligned16(y) && aligned16(dy) && aligned16(dh_last) && aligned16(dx) && aligned16(dgates) &&
                        aligned16(dh0) && aligned16(dlam_rows) && (h0_stride % 4 == 0) && (dh_last_stride % 4 == 0);
    const bool vec = vec_ok && R * (D / 8) >= (int64_t)256 * kSeqThreads * 2;
    if (vec) {
        const int rows_per_block = kSeqThreads / (D / 8);
        const int64_t blocks = (R + rows_per_block - 1) / rows_per_block;
        if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((rglru_scan_bwd_vec8_kernel<XT, GT, YT>), dim3((unsigned)blocks), dim3(kSeqThreads),
                           (size_t)2 * D * sizeof(float), stream, (const XT *)x, (const GT *)gates, log_lambda, c, h0,
                           h0_stride, done, (const YT *)y, (const YT *)dy, dh_last, dh_last_stride, (XT *)dx,
                           (GT *)dgates, dh0, dlam_rows, R, T, D, rs, ts, rows_per_block, y_group, y_pitch, ts_y);
    } else {
        const int64_t blocks = (R * D + kSeqThreads - 1) / kSeqThreads;
        if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((rglru_scan_bwd_scalar_kernel<XT, GT, YT>), dim3((unsigned)blocks), dim3(kSeqThreads), 0,
                           stream, (const XT *)x, (const GT *)gates, log_lambda, c, h0, h0_stride, done,
                           (const YT *)y, (const YT *)dy, dh_last, dh_last_stride, (XT *)dx, (GT *)dgates, dh0,
                           dlam_rows, R, T, D, rs, ts, y_group, y_pitch, ts_y);
    }
    return (int)hipGetLastError();
}

template <typename XT, typename GT>
static int scan_bwd_dispatch_y(const void *x, const void *gates, const float *log_lambda, float c, const float *h0,
                               int64_t h0_stride, const uint8_t *done, const void *y, int y_dtype, const void *dy,
                               const float *dh_last, int64_t dh_last_stride, void *dx, void *dgates, float *dh0,
                               float *dlam_rows, int64_t R, int T, int D, int time_major, int y_group, int y_pitch,
                               hipStream_t stream)
{
    if (y_dtype == BNB_F32)
        return launch_scan_bwd<XT, GT, float>(x, gates, log_lambda, c, h0, h0_stride, done, y, dy, dh_last, dh_last_stride,
                                              dx, dgates, dh0, dlam_rows, R, T, D, time_major, y_group, y_pitch, stream);
    return launch_scan_bwd<XT, GT, uint16_t>(x, gates, log_lambda, c, h0, h0_stride, done, y, dy, dh_last, dh_last_stride,
                                             dx, dgates, dh0, dlam_rows, R, T, D, time_major, y_group, y_pitch, stream);
}

// ------------------------------------------------------------------------------------
// causal depthwise conv over T steps
// ------------------------------------------------------------------------------------

// `hist` counts how many of the three previous inputs belong to the running episode: the
// stored buffer belongs to the episode running at t = 0, a boundary clears the history.
template <typename BT>
__global__ __launch_bounds__(kSeqThreads) void conv_seq_vec8_kernel(
    const BT *__restrict__ b1, const float *__restrict__ conv_in, int64_t conv_in_stride,
    const float *__restrict__ weight, const float *__restrict__ bias, const uint8_t *__restrict__ done,
    float *__restrict__ v_out, uint16_t *__restrict__ v_bf16_out, float *__restrict__ conv_out,
    int64_t conv_out_stride, int64_t R, int T, int D, int64_t rs, int64_t ts, int rows_per_block, int b_group, int b_pitch,
    int64_t ts_b)
{
    const int vecs_per_row = D >> 3;
    const int local_row = threadIdx.x / vecs_per_row;
    const int64_t row = (int64_t)blockIdx.x * rows_per_block + local_row;
    if (local_row >= rows_per_block || row >= R) return;
    const int d0 = (threadIdx.x - local_row * vecs_per_row) << 2;  // first of the lane's two runs of four channels
    const int gap = D >> 1;        // the second run starts here: every access of a row's lanes is one dense run

    float w[8][kSeqTaps], bs[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const f32x4 wv = *reinterpret_cast<const f32x4 *>(weight + (int64_t)(d0 + (e & 3) + (e >> 2) * gap) * kSeqTaps);
        w[e][0] = wv.x;
        w[e][1] = wv.y;
        w[e][2] = wv.z;
        w[e][3] = wv.w;
        bs[e] = bias != nullptr ? bias[d0 + (e & 3) + (e >> 2) * gap] : 0.0f;
    }
    const float *pin = conv_in + row * conv_in_stride + d0;
    Row8 p0 = load8_split<false>(pin, gap), p1 = load8_split<false>(pin + D, gap), p2 = load8_split<false>(pin + 2 * D, gap);
    const BT *bp = b1 + placed_row(row, b_group, b_pitch) * rs + d0;
    const uint8_t *dn = done == nullptr ? nullptr : done + row * T;
    int hist = 3;

    for (int t0 = 0; t0 < T; t0 += kSeqAhead) {
        Row8 cur[kSeqAhead];
        uint32_t cut[kSeqAhead];
#pragma unroll
        for (int u = 0; u < kSeqAhead; ++u) {
            const int t = t0 + u < T ? t0 + u : T - 1;
            cur[u] = load8_split<true>(bp + t * ts_b, gap);
            cut[u] = 0;
            if (dn != nullptr) cut[u] = dn[t > 0 ? t - 1 : 0];
            if (t == 0) cut[u] = 0;
        }
#pragma unroll
        for (int u = 0; u < kSeqAhead; ++u) {
            if (t0 + u < T) {
                if (cut[u]) hist = 0;
                Row8 v;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    // inputs from before the boundary read as zero; the reference's order:
                    // taps 0..3 (oldest input first), then the bias
                    float acc = (hist >= 3 ? p0.v[e] : 0.0f) * w[e][0];
                    acc += (hist >= 2 ? p1.v[e] : 0.0f) * w[e][1];
                    acc += (hist >= 1 ? p2.v[e] : 0.0f) * w[e][2];
                    acc += cur[u].v[e] * w[e][3];
                    v.v[e] = acc + bs[e];
                }
                const int64_t off = row * rs + (t0 + u) * ts + d0;
                store8_split<true>(v_out + off, gap, v);
                if (v_bf16_out != nullptr) store8_split<true>(v_bf16_out + off, gap, v);
                p0 = p1;
                p1 = p2;
                p2 = cur[u];
                hist = hist < 3 ? hist + 1 : 3;
            }
        }
    }
    // the last three inputs, whatever episode they belong to (griffin.py:277)
    float *pout = conv_out + row * conv_out_stride + d0;
    store8_split<false>(pout, gap, p0);
    store8_split<false>(pout + D, gap, p1);
    store8_split<false>(pout + 2 * D, gap, p2);
}

template <typename BT>
__global__ __launch_bounds__(kSeqThreads) void conv_seq_scalar_kernel(
    const BT *__restrict__ b1, const float *__restrict__ conv_in, int64_t conv_in_stride,
    const float *__restrict__ weight, const float *__restrict__ bias, const uint8_t *__restrict__ done,
    float *__restrict__ v_out, uint16_t *__restrict__ v_bf16_out, float *__restrict__ conv_out,
    int64_t conv_out_stride, int64_t R, int T, int D, int64_t rs, int64_t ts, int b_group, int b_pitch, int64_t ts_b)
{
    const int64_t idx = (int64_t)blockIdx.x * kSeqThreads + threadIdx.x;
    if (idx >= R * D) return;
    const int64_t row = idx / D;
    const int d = (int)(idx - row * D);
    const float *wp = weight + (int64_t)d * kSeqTaps;
    const float w0 = wp[0], w1 = wp[1], w2 = wp[2], w3 = wp[3];
    const float bs = bias != nullptr ? bias[d] : 0.0f;
    const float *pin = conv_in + row * conv_in_stride + d;
    float p0 = pin[0], p1 = pin[D], p2 = pin[2 * D];
    const BT *bp = b1 + placed_row(row, b_group, b_pitch) * rs + d;
    const uint8_t *dn = done == nullptr ? nullptr : done + row * T;
    int hist = 3;
    for (int t0 = 0; t0 < T; t0 += kScalarAhead) {
        float in[kScalarAhead];
        uint32_t cut[kScalarAhead];
#pragma unroll
        for (int u = 0; u < kScalarAhead; ++u) {
            const int t = t0 + u < T ? t0 + u : T - 1;  // past the end: re-read the last step (discarded)
            in[u] = load1(bp + t * ts_b);
            cut[u] = (dn != nullptr && t > 0) ? dn[t - 1] : 0;
        }
#pragma unroll
        for (int u = 0; u < kScalarAhead; ++u) {
            const int t = t0 + u;
            if (t < T) {
                const float cur = in[u];
                if (cut[u]) hist = 0;
                float acc = (hist >= 3 ? p0 : 0.0f) * w0;
                acc += (hist >= 2 ? p1 : 0.0f) * w1;
                acc += (hist >= 1 ? p2 : 0.0f) * w2;
                acc += cur * w3;
                const float v = acc + bs;
                v_out[row * rs + t * ts + d] = v;
                if (v_bf16_out != nullptr) store1(v_bf16_out + row * rs + t * ts + d, v);
                p0 = p1;
                p1 = p2;
                p2 = cur;
                hist = hist < 3 ? hist + 1 : 3;
            }
        }
    }
    float *pout = conv_out + row * conv_out_stride + d;
    pout[0] = p0;
    pout[D] = p1;
    pout[2 * D] = p2;
}

template <typename BT>
static int launch_conv_seq(const void *b1, const float *conv_in, int64_t conv_in_stride, const float *weight,
                           const float *bias, const uint8_t *done, float *v_out, uint16_t *v_bf16_out,
                           float *conv_out, int64_t conv_out_stride, int64_t R, int T, int D, int time_major,
                           int b_group, int b_pitch, hipStream_t stream)
{
    const int64_t rs = time_major ? D : (int64_t)T * D, ts = time_major ? R * D : D;
    const int64_t ts_b = b_group > 0 ? R / b_group * b_pitch * D : ts;
    const bool vec_ok = (D % 8 == 0) && (D / 8 <= kSeqThreads) && aligned16(b1) && aligned16(conv_in) &&
                        aligned16(conv_out) && aligned16(v_out) && aligned16(v_bf16_out) && aligned16(weight) &&
                        (conv_in_stride % 4 == 0) && (conv_out_stride % 4 == 0);
    const bool vec = vec_ok && R * (D / 8) >= (int64_t)256 * kSeqThreads * 2;
    if (vec) {
        const int rows_per_block = kSeqThreads / (D / 8);
        const int64_t blocks = (R + rows_per_block - 1) / rows_per_block;
        if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((conv_seq_vec8_kernel<BT>), dim3((unsigned)blocks), dim3(kSeqThreads), 0, stream,
                           (const BT *)b1, conv_in, conv_in_stride, weight, bias, done, v_out, v_bf16_out, conv_out,
                           conv_out_stride, R, T, D, rs, ts, rows_per_block, b_group, b_pitch, ts_b);
    } else {
        const int64_t blocks = (R * D + kSeqThreads - 1) / kSeqThreads;
        if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((conv_seq_scalar_kernel<BT>), dim3((unsigned)blocks), dim3(kSeqThreads), 0, stream,
                           (const BT *)b1, conv_in, conv_in_stride, weight, bias, done, v_out, v_bf16_out, conv_out,
                           conv_out_stride, R, T, D, rs, ts, b_group, b_pitch, ts_b);
    }
    return (int)hipGetLastError();
}

// ------------------------------------------------------------------------------------
// backward of the causal depthwise conv over T steps
// ------------------------------------------------------------------------------------
//
// With in[s] = stored input s + 3 for s in -3..-1 and b1[s] for s >= 0, the forward is
//   v[t] = bias + sum_j w[3 - j] * in[t - j] * [no episode end in t-j .. t-1],   j = 0..3,
// so every input's gradient depends on four output gradients only,
//   d_in[s] = dv[s] w3 + m1 dv[s+1] w2 + m2 dv[s+2] w1 + m3 dv[s+3] w0,
//   m1 = !done[s], m2 = m1 && !done[s+1], m3 = m2 && !done[s+2]   (done[s < 0] = false, dv[t >= T] = 0),
// and the same products pair in[s] with the taps' gradients.  No recurrence: a work item is
// (a group of rows, 16 consecutive s), a work-group walks items in a grid-stride loop with the
// tap and bias gradients in registers, then adds its rows through LDS and writes one partial
// row; the partial rows are added in a fixed order by sum_slices.
constexpr int kCbChunk = 16;
constexpr int kCbMaxBlocks = 2048;

template <typename BT>
__global__ __launch_bounds__(kSeqThreads) void conv_seq_bwd_kernel(
    const BT *__restrict__ b1, const float *__restrict__ conv_in, int64_t conv_in_stride, const float *__restrict__ weight,
    const uint8_t *__restrict__ done, const float *__restrict__ dv, const uint16_t *__restrict__ dv_lp,
    const float *__restrict__ dconv_out, BT *__restrict__ db1, float *__restrict__ dconv_in, float *__restrict__ partials,
    int64_t R, int T, int D, int64_t rs, int64_t ts, int chunks, int64_t items, int b_group, int b_pitch, int64_t ts_b)
{
    __shared__ float s_red[kSeqThreads * 8];
    const int vecs = D >> 3;
    const int rows_per_block = kSeqThreads / vecs;
    const int local_row = threadIdx.x / vecs;
    const int d0 = (threadIdx.x - local_row * vecs) << 2;  // first of the lane's two runs of four channels
    const int gap = D >> 1;        // the second run starts here: every access of a row's lanes is one dense run

    float w[8][kSeqTaps], dw[8][kSeqTaps], db[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const f32x4 wv = *reinterpret_cast<const f32x4 *>(weight + (int64_t)(d0 + (e & 3) + (e >> 2) * gap) * kSeqTaps);
        w[e][0] = wv.x, w[e][1] = wv.y, w[e][2] = wv.z, w[e][3] = wv.w;
        dw[e][0] = dw[e][1] = dw[e][2] = dw[e][3] = 0.0f;
        db[e] = 0.0f;
    }
    const Row8 zero = {{0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f}};

    for (int64_t item = blockIdx.x; item < items; item += gridDim.x) {
        const int64_t group = item / chunks;
        const int s0 = (int)(item - group * chunks) * kCbChunk - (kSeqTaps - 1);  // uniform over the work-group
        const int64_t row = group * rows_per_block + local_row;
        if (row >= R) continue;
        const float *dvp = dv + row * rs + d0;
        const uint16_t *dlp = dv_lp == nullptr ? nullptr : dv_lp + row * rs + d0;
        const int64_t at_b = placed_row(row, b_group, b_pitch) * rs;  // b1 and db1: possibly rows of a wider token tensor
        const BT *bp = b1 + at_b + d0;
        const uint8_t *dn = done == nullptr ? nullptr : done + row * T;
        // the output's gradient: the float32 part plus, when the output also went out in bfloat16, that copy's
        auto grad_row = [&](int t) -> Row8 {
            if (t < 0 || t >= T) return zero;
            Row8 g = load8_split<true>(dvp + t * ts, gap);
            if (dlp != nullptr) {
                const Row8 l = load8_split<true>(dlp + t * ts, gap);
#pragma unroll
                for (int e = 0; e < 8; ++e) g.v[e] += l.v[e];
            }
            return g;
        };
        auto ended = [&](int t) -> bool { return dn != nullptr && t >= 0 && t < T && dn[t] != 0; };

        Row8 g0 = grad_row(s0), g1 = grad_row(s0 + 1), g2 = grad_row(s0 + 2);
        bool f0 = ended(s0), f1 = ended(s0 + 1);
        for (int u0 = 0; u0 < kCbChunk && s0 + u0 < T; u0 += kSeqAhead) {
            Row8 gn[kSeqAhead], in[kSeqAhead];
            bool fn[kSeqAhead];
#pragma unroll
            for (int u = 0; u < kSeqAhead; ++u) {
                const int s = s0 + u0 + u;
                gn[u] = grad_row(s + 3);
                fn[u] = ended(s + 2);
                if (s < 0)
                    in[u] = load8_split<false>(conv_in + row * conv_in_stride + (int64_t)(s + 3) * D + d0, gap);
                else
                    in[u] = s < T ? load8_split<true>(bp + s * ts_b, gap) : zero;
            }
#pragma unroll
            for (int u = 0; u < kSeqAhead; ++u) {
                const int s = s0 + u0 + u;
                if (s < T) {
                    const Row8 g3 = gn[u];
                    const bool f2 = fn[u];
                    const float m1 = f0 ? 0.0f : 1.0f, m2 = (f0 || f1) ? 0.0f : 1.0f, m3 = (f0 || f1 || f2) ? 0.0f : 1.0f;
                    Row8 o;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float a1 = m1 * g1.v[e], a2 = m2 * g2.v[e], a3 = m3 * g3.v[e];
                        o.v[e] = g0.v[e] * w[e][3] + a1 * w[e][2] + a2 * w[e][1] + a3 * w[e][0];
                        const float x = in[u].v[e];
                        dw[e][3] = fmaf(x, g0.v[e], dw[e][3]);
                        dw[e][2] = fmaf(x, a1, dw[e][2]);
                        dw[e][1] = fmaf(x, a2, dw[e][1]);
                        dw[e][0] = fmaf(x, a3, dw[e][0]);
                        db[e] += g0.v[e];
                    }
                    if (dconv_out != nullptr && s >= T - 3) {
                        // this input is also entry s - (T - 3) of the stored inputs handed on
                        const Row8 h = load8_split<false>(dconv_out + row * 3 * (int64_t)D + (int64_t)(s - (T - 3)) * D + d0, gap);
#pragma unroll
                        for (int e = 0; e < 8; ++e) o.v[e] += h.v[e];
                    }
                    if (s < 0)
                        store8_split<false>(dconv_in + row * 3 * (int64_t)D + (int64_t)(s + 3) * D + d0, gap, o);
                    else
                        store8_split<true>(db1 + at_b + s * ts_b + d0, gap, o);
                    g0 = g1, g1 = g2, g2 = g3;
                    f0 = f1, f1 = f2;
                }
            }
        }
    }

    // this work-group's tap and bias gradients: rows added in order, one partial row
    // [ (d, tap) for all d | bias ] per work-group
    float *part = partials + (int64_t)blockIdx.x * 5 * D;
#pragma unroll
    for (int q = 0; q < 5; ++q) {
#pragma unroll
        for (int e = 0; e < 8; ++e) s_red[local_row * D + d0 + (e & 3) + (e >> 2) * gap] = q < 4 ? dw[e][q < 4 ? q : 0] : db[e];
        __syncthreads();
        for (int d = threadIdx.x; d < D; d += kSeqThreads) {
            float t = 0.0f;
            for (int j = 0; j < rows_per_block; ++j) t += s_red[j * D + d];
            part[q < 4 ? d * kSeqTaps + q : 4 * D + d] = t;
        }
        __syncthreads();
    }
}

template <typename BT>
static int launch_conv_seq_bwd(const void *b1, const float *conv_in, int64_t conv_in_stride, const float *weight,
                               const uint8_t *done, const float *dv, const uint16_t *dv_lp, const float *dconv_out, void *db1,
                               float *dconv_in, float *partials, int blocks, float *dwb, int64_t R, int T, int D,
                               int time_major, int b_group, int b_pitch, hipStream_t stream)
{
    const int64_t rs = time_major ? D : (int64_t)T * D, ts = time_major ? R * D : D;
    const int64_t ts_b = b_group > 0 ? R / b_group * b_pitch * D : ts;
    const int rows_per_block = kSeqThreads / (D / 8);
    const int chunks = (T + (kSeqTaps - 1) + kCbChunk - 1) / kCbChunk;
    const int64_t items = (R + rows_per_block - 1) / rows_per_block * chunks;
    hipLaunchKernelGGL((conv_seq_bwd_kernel<BT>), dim3((unsigned)blocks), dim3(kSeqThreads), 0, stream, (const BT *)b1, conv_in,
                       conv_in_stride, weight, done, dv, dv_lp, dconv_out, (BT *)db1, dconv_in, partials, R, T, D, rs, ts, chunks,
                       items, b_group, b_pitch, ts_b);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return launch_sum_slices(partials, dwb, 5 * (int64_t)D, blocks, 0, stream);
}

// rows_per_env / env_row_pitch of the entry points below: both zero, or a time-major call whose rows are the first
// rows_per_env of every env_row_pitch rows of a wider tensor
static int check_token_rows(int64_t R, int time_major, int rows_per_env, int env_row_pitch)
{
    if (rows_per_env == 0 && env_row_pitch == 0) return 0;
    if (rows_per_env < 1 || env_row_pitch < rows_per_env || !time_major || R % rows_per_env != 0) return BNB_ERR_BAD_SHAPE;
    return 0;
}

}  // namespace bnb

extern "C" int bnb_rglru_scan_fwd(const void *x, int x_dtype, const void *gates_pre, int g_dtype,
                                  const float *log_lambda, float c, const float *h0, int64_t h0_row_stride,
                                  const uint8_t *done, void *y, int y_dtype, float *h_last,
                                  int64_t h_last_row_stride, int64_t R, int T, int D, int time_major, int rows_per_env,
                                  int env_row_pitch, void *stream)
{
    using namespace bnb;
    if (R < 0 || T < 0 || D < 1) return BNB_ERR_BAD_SHAPE;
    if (check_token_rows(R, time_major, rows_per_env, env_row_pitch)) return BNB_ERR_BAD_SHAPE;
    if (R == 0) return 0;
    if (!log_lambda || !h0 || !h_last) return BNB_ERR_NULL_POINTER;
    if (h0_row_stride < D || h_last_row_stride < D) return BNB_ERR_BAD_SHAPE;
    if ((x_dtype != BNB_F32 && x_dtype != BNB_BF16) || (g_dtype != BNB_F32 && g_dtype != BNB_BF16) ||
        (y_dtype != BNB_F32 && y_dtype != BNB_BF16))
        return BNB_ERR_BAD_DTYPE;
    if ((reinterpret_cast<uintptr_t>(h0) | reinterpret_cast<uintptr_t>(h_last) |
         reinterpret_cast<uintptr_t>(log_lambda)) & 3u)
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    if (T == 0) {  // nothing to advance: the state passes through
        if (h0 == h_last && h0_row_stride == h_last_row_stride) return 0;
        return (int)hipMemcpy2DAsync(h_last, (size_t)h_last_row_stride * sizeof(float), h0,
                                     (size_t)h0_row_stride * sizeof(float), (size_t)D * sizeof(float), (size_t)R,
                                     hipMemcpyDeviceToDevice, s);
    }
    if (!x || !gates_pre || !y) return BNB_ERR_NULL_POINTER;
    const bool xb = x_dtype == BNB_BF16, gb = g_dtype == BNB_BF16;
    if (!xb && !gb)
        return scan_dispatch_y<float, float>(x, gates_pre, log_lambda, c, h0, h0_row_stride, done, y, y_dtype, h_last,
                                             h_last_row_stride, R, T, D, time_major != 0, rows_per_env, env_row_pitch, s);
    if (xb && gb)
        return scan_dispatch_y<uint16_t, uint16_t>(x, gates_pre, log_lambda, c, h0, h0_row_stride, done, y, y_dtype,
                                                   h_last, h_last_row_stride, R, T, D, time_major != 0, rows_per_env, env_row_pitch, s);
    if (!xb && gb)
        return scan_dispatch_y<float, uint16_t>(x, gates_pre, log_lambda, c, h0, h0_row_stride, done, y, y_dtype,
                                                h_last, h_last_row_stride, R, T, D, time_major != 0, rows_per_env, env_row_pitch, s);
    return scan_dispatch_y<uint16_t, float>(x, gates_pre, log_lambda, c, h0, h0_row_stride, done, y, y_dtype, h_last,
                                            h_last_row_stride, R, T, D, time_major != 0, rows_per_env, env_row_pitch, s);
}

extern "C" int bnb_rglru_scan_bwd(const void *x, int x_dtype, const void *gates_pre, int g_dtype,
                                  const float *log_lambda, float c, const float *h0, int64_t h0_row_stride,
                                  const uint8_t *done, const void *y, int y_dtype, const void *dy,
                                  const float *dh_last, int64_t dh_last_row_stride, void *dx, void *dgates,
                                  float *dh0, float *dlam_rows, int64_t R, int T, int D, int time_major,
                                  int rows_per_env, int env_row_pitch, void *stream)
{
    using namespace bnb;
    if (R < 0 || T < 1 || D < 1) return BNB_ERR_BAD_SHAPE;
    if (check_token_rows(R, time_major, rows_per_env, env_row_pitch)) return BNB_ERR_BAD_SHAPE;
    if (R == 0) return 0;
    if (!x || !gates_pre || !log_lambda || !h0 || !y || !dx || !dgates || !dh0 || !dlam_rows)
        return BNB_ERR_NULL_POINTER;
    if (h0_row_stride < D || (dh_last && dh_last_row_stride < D)) return BNB_ERR_BAD_SHAPE;
    if ((x_dtype != BNB_F32 && x_dtype != BNB_BF16) || (g_dtype != BNB_F32 && g_dtype != BNB_BF16) ||
        (y_dtype != BNB_F32 && y_dtype != BNB_BF16))
        return BNB_ERR_BAD_DTYPE;
    if ((reinterpret_cast<uintptr_t>(h0) | reinterpret_cast<uintptr_t>(dh_last) | reinterpret_cast<uintptr_t>(dh0) |
         reinterpret_cast<uintptr_t>(dlam_rows) | reinterpret_cast<uintptr_t>(log_lambda)) & 3u)
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    const bool xb = x_dtype == BNB_BF16, gb = g_dtype == BNB_BF16;
    if (!xb && !gb)
        return scan_bwd_dispatch_y<float, float>(x, gates_pre, log_lambda, c, h0, h0_row_stride, done, y, y_dtype, dy,
                                                 dh_last, dh_last_row_stride, dx, dgates, dh0, dlam_rows, R, T, D,
                                                 time_major != 0, rows_per_env, env_row_pitch, s);
    if (xb && gb)
        return scan_bwd_dispatch_y<uint16_t, uint16_t>(x, gates_pre, log_lambda, c, h0, h0_row_stride, done, y,
                                                       y_dtype, dy, dh_last, dh_last_row_stride, dx, dgates, dh0,
                                                       dlam_rows, R, T, D, time_major != 0, rows_per_env, env_row_pitch, s);
    if (!xb && gb)
        return scan_bwd_dispatch_y<float, uint16_t>(x, gates_pre, log_lambda, c, h0, h0_row_stride, done, y, y_dtype,
                                                    dy, dh_last, dh_last_row_stride, dx, dgates, dh0, dlam_rows, R, T,
                                                    D, time_major != 0, rows_per_env, env_row_pitch, s);
    return scan_bwd_dispatch_y<uint16_t, float>(x, gates_pre, log_lambda, c, h0, h0_row_stride, done, y, y_dtype, dy,
                                                dh_last, dh_last_row_stride, dx, dgates, dh0, dlam_rows, R, T, D,
                                                time_major != 0, rows_per_env, env_row_pitch, s);
}

extern "C" int bnb_conv_seq_fwd(const void *b1, int b1_dtype, const float *conv_in, int64_t conv_in_row_stride,
                                const float *weight, const float *bias, const uint8_t *done, float *v_out,
                                void *v_bf16_out, float *conv_out, int64_t conv_out_row_stride, int64_t R, int T,
                                int D, int time_major, int rows_per_env, int env_row_pitch, void *stream)
{
    using namespace bnb;
    if (R < 0 || T < 1 || D < 1) return BNB_ERR_BAD_SHAPE;
    if (check_token_rows(R, time_major, rows_per_env, env_row_pitch)) return BNB_ERR_BAD_SHAPE;
    if (R == 0) return 0;
    if (!b1 || !conv_in || !weight || !v_out || !conv_out) return BNB_ERR_NULL_POINTER;
    if (b1_dtype != BNB_F32 && b1_dtype != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (conv_in_row_stride < 3 * (int64_t)D || conv_out_row_stride < 3 * (int64_t)D) return BNB_ERR_BAD_SHAPE;
    if ((reinterpret_cast<uintptr_t>(conv_in) | reinterpret_cast<uintptr_t>(conv_out) |
         reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(v_out) |
         reinterpret_cast<uintptr_t>(bias)) & 3u)
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    if (b1_dtype == BNB_BF16)
        return launch_conv_seq<uint16_t>(b1, conv_in, conv_in_row_stride, weight, bias, done, v_out,
                                         (uint16_t *)v_bf16_out, conv_out, conv_out_row_stride, R, T, D, time_major != 0,
                                         rows_per_env, env_row_pitch, s);
    return launch_conv_seq<float>(b1, conv_in, conv_in_row_stride, weight, bias, done, v_out, (uint16_t *)v_bf16_out,
                                  conv_out, conv_out_row_stride, R, T, D, time_major != 0, rows_per_env, env_row_pitch, s);
}

extern "C" int bnb_conv_seq_bwd_blocks(int64_t R, int T, int D)
{
    if (R <= 0 || T < 1 || D < 8) return 1;
    const int rows_per_block = bnb::kSeqThreads / (D / 8) > 0 ? bnb::kSeqThreads / (D / 8) : 1;
    const int64_t items = (R + rows_per_block - 1) / rows_per_block * ((T + 3 + bnb::kCbChunk - 1) / bnb::kCbChunk);
    return (int)(items < bnb::kCbMaxBlocks ? items : bnb::kCbMaxBlocks);
}

extern "C" int bnb_conv_seq_bwd(const void *b1, int b1_dtype, const float *conv_in, int64_t conv_in_row_stride,
                                const float *weight, const uint8_t *done, const float *dv, const void *dv_bf16,
                                const float *dconv_out, void *db1, float *dconv_in, float *partials, int blocks, float *dwb,
                                int64_t R, int T, int D, int time_major, int rows_per_env, int env_row_pitch, void *stream)
{
    using namespace bnb;
    if (R < 0 || T < 1 || D < 1) return BNB_ERR_BAD_SHAPE;
    if (check_token_rows(R, time_major, rows_per_env, env_row_pitch)) return BNB_ERR_BAD_SHAPE;
    if (D != 64 && D != 128 && D != 256 && D != 512) return BNB_ERR_UNSUPPORTED;
    if (b1_dtype != BNB_F32 && b1_dtype != BNB_BF16) return BNB_ERR_BAD_DTYPE;
    if (!weight || !partials || !dwb || (R > 0 && (!b1 || !conv_in || !dv || !db1 || !dconv_in))) return BNB_ERR_NULL_POINTER;
    if (conv_in_row_stride < 3 * (int64_t)D || blocks < 1 || blocks > kCbMaxBlocks) return BNB_ERR_BAD_SHAPE;
    if (!aligned16(weight) || !aligned16(partials) || !aligned16(dwb) ||
        (R > 0 && (!aligned16(b1) || !aligned16(conv_in) || !aligned16(dv) || !aligned16(db1) || !aligned16(dconv_in) ||
                   (dconv_out && !aligned16(dconv_out)) || (dv_bf16 && !aligned16(dv_bf16)))) ||
        conv_in_row_stride % 4 != 0)
        return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
    if (R == 0) return launch_sum_slices(partials, dwb, 5 * (int64_t)D, 0, 0, s);
    if (b1_dtype == BNB_BF16)
        return launch_conv_seq_bwd<uint16_t>(b1, conv_in, conv_in_row_stride, weight, done, dv, (const uint16_t *)dv_bf16,
                                             dconv_out, db1, dconv_in, partials, blocks, dwb, R, T, D, time_major != 0,
                                             rows_per_env, env_row_pitch, s);
    return launch_conv_seq_bwd<float>(b1, conv_in, conv_in_row_stride, weight, done, dv, (const uint16_t *)dv_bf16, dconv_out,
                                      db1, dconv_in, partials, blocks, dwb, R, T, D, time_major != 0, rows_per_env,
                                      env_row_pitch, s);
}
