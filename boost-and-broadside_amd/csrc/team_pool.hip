// Pooling by multi-head attention over each team's ships, for gfx950 (fp32, d_model 128).
//
// Reference: TeamPMA.forward, models/yemong/policy.py:94-120.  Per environment and team t in
// {0, 1} one learned seed is the only query of a bias-free multi-head attention over the ship
// rows x (B, N, D), keys restricted to the alive ships of team t; the result goes through
// out_proj and RMSNorm, a team without an alive ship pools to zero, and every ship receives the
// pooled vector of team clamp(team_id, 0, 1).
//
// Because the query is a constant of the model, the K and V projections of all N ships (the
// bulk of the reference's work, done twice) fold away:
//   score_j(t, h) = x_j . u(t, h),     u(t, h) = W_k[h]^T (W_q seed_t)[h] / sqrt(dh)      (2H vectors)
//   out_t         = sum_h M_h z(t, h),  z(t, h) = sum_j softmax_j(score) x_j,  M_h = W_o[:, h] W_v[h, :]
// so x is read from HBM exactly once and everything per ship is 2H dot products and 2H scaled
// adds of a 128-vector.  Three steps:
//   team_attend_kernel          x -> z (B, 2, H, 128); HBM-bound on x
//   one plain fp32 library GEMM (B*2, H*128) x (H*128, 128) with [M_0 | .. | M_{H-1}] (the caller's)
//   team_norm_broadcast_kernel  RMSNorm, then every ship receives its team's vector; HBM-bound
//                               on the (B, N, 128) result
// All arithmetic is fp32 on the vector ALUs, which keeps the fp32 parity bar (the op also
// serves evaluation without autocast).
//
// team_attend_kernel: ships come in chunks of 64 rows staged in LDS (the next chunk is already
// in flight in registers):
//   scores                    lane = ship, wave = a quarter of the channels, all heads of the
//                             ship's own team (the other team's heads would be masked)
//   online softmax            lane = ship, wave = head; the running maximum and sum of both
//                             teams live in the wave's registers
//   pooling                   thread = (channel, team): z(t, h)[d] for the H heads of its team

#include "common.h"

namespace bnb {

constexpr int kTpD = 128;
constexpr int kTpThreads = 256;
constexpr int kTpChunk = 64;           // ship rows staged at a time
constexpr int kTpPitch = kTpD + 4;     // floats per staged row: 16-byte aligned, bank-spread
constexpr int kTpEnvs = 4;             // environments per work-group of the norm + hand-out kernel

// max / sum over aligned groups of SEG lanes (SEG = 64: the whole wave)
template <int SEG>
__device__ __forceinline__ float seg_max(float v)
{
#pragma unroll
    for (int o = SEG / 2; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

template <int SEG>
__device__ __forceinline__ float seg_sum(float v)
{
#pragma unroll
    for (int o = SEG / 2; o >= 1; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// SEG = lanes (staged rows) per environment in the score phase: 64 = one environment per
// work-group, any number of ships in chunks of 64; 16 = four environments of up to 16 ships
// side by side.  Writes z (B, 2, H, 128): the softmax-weighted mean of the ship rows per
// (team, head), zero for a team without an alive ship.
template <int H, int SEG>
__global__ __launch_bounds__(kTpThreads) void team_attend_kernel(
    const float *__restrict__ x, int64_t x_env_stride, int64_t x_row_stride, const int32_t *__restrict__ team_id,
    int64_t team_env_stride, const uint8_t *__restrict__ alive, int64_t alive_env_stride,
    const float *__restrict__ score_vec, float *__restrict__ z_out, int B, int N)
{
    constexpr int NC = 2 * H;            // (team, head) pairs
    constexpr int EPP = kTpChunk / SEG;  // environments per work-group
    __shared__ __align__(16) float s_x[kTpChunk * kTpPitch];
    constexpr int kTeamPitch = H * kTpD + 4;  // team 1's vectors start 16 bytes off team 0's banks
    __shared__ __align__(16) float s_u[2 * kTeamPitch];
    __shared__ __align__(16) float s_p[kTpChunk * NC];  // softmax numerators; 0 under the other team's heads
    __shared__ __align__(16) float s_part[4 * kTpChunk * H];  // per channel quarter: partial scores
    __shared__ float s_alpha[EPP * NC], s_l[EPP * NC];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int d = tid & (kTpD - 1);  // pooling phase: channel
    const int tm = wave >> 1;        // and team (wave-uniform)
    for (int i = tid; i < NC * kTpD; i += kTpThreads) s_u[(i / (H * kTpD)) * kTeamPitch + i % (H * kTpD)] = score_vec[i];

    const int env_first = blockIdx.x * EPP;
    const int seg = lane / SEG;      // environment of this lane inside the work-group
    const int srow = lane % SEG;     // its ship inside the chunk
    const int env_lane = env_first + seg;
    float run_max[2] = {-INFINITY, -INFINITY}, run_sum[2] = {0.0f, 0.0f};  // of head `wave`, per team
    float z[EPP][H];
#pragma unroll
    for (int q = 0; q < EPP; ++q)
#pragma unroll
        for (int k = 0; k < H; ++k) z[q][k] = 0.0f;

    // A thread's share of a chunk: 8 pieces of 16 bytes.  The next chunk is requested before the
    // current one is worked on, so its latency hides under the arithmetic.
    constexpr int kPieces = kTpChunk * (kTpD / 4) / kTpThreads;
    f32x4 stage[kPieces];
    auto fetch = [&](int c0) {
        const int rows = N - c0 < SEG ? N - c0 : SEG;
#pragma unroll
        for (int it = 0; it < kPieces; ++it) {
            const int idx = tid + it * kTpThreads;
            const int q4 = (idx & 31) * 4;
            const int rr = idx >> 5;  // staged row: q * SEG + r
            const int q = rr / SEG, r = rr % SEG;
            const bool on = r < rows && env_first + q < B;
            const int64_t off = on ? (int64_t)(env_first + q) * x_env_stride + (int64_t)(c0 + r) * x_row_stride + q4 : 0;
            stage[it] = *reinterpret_cast<const f32x4 *>(x + off);
        }
    };
    auto stash = [&](int c0) {
        const int rows = N - c0 < SEG ? N - c0 : SEG;
#pragma unroll
        for (int it = 0; it < kPieces; ++it) {
            const int idx = tid + it * kTpThreads;
            const int q4 = (idx & 31) * 4;
            const int rr = idx >> 5;
            if (rr % SEG < rows) *reinterpret_cast<f32x4 *>(s_x + rr * kTpPitch + q4) = stage[it];
        }
    };

    if (N > 0) fetch(0);
    for (int c0 = 0; c0 < N; c0 += SEG) {
        const int rows = N - c0 < SEG ? N - c0 : SEG;
        __syncthreads();  // previous chunk is done with s_x, s_p, s_alpha
        stash(c0);
        if (c0 + SEG < N) fetch(c0 + SEG);
        __syncthreads();

        // ---- scores of this lane's ship under the heads of ITS team (the other team's heads
        //      would be masked anyway).  Each wave covers a quarter of the channels, so the
        //      staged rows are read from LDS once, not once per head. ----
        const bool present = srow < rows && env_lane < B;
        const int ship_team = present ? team_id[(int64_t)env_lane * team_env_stride + c0 + srow] : -1;
        const bool key = present && alive[(int64_t)env_lane * alive_env_stride + c0 + srow] != 0 &&
                         (ship_team == 0 || ship_team == 1);
        {
            float part[H];
#pragma unroll
            for (int k = 0; k < H; ++k) part[k] = 0.0f;
            const float *xr = s_x + (present ? lane : 0) * kTpPitch + 32 * wave;
            const float *ur = s_u + (key ? ship_team : 0) * kTeamPitch + 32 * wave;
#pragma unroll
            for (int i = 0; i < 32; i += 4) {
                const f32x4 xv = *reinterpret_cast<const f32x4 *>(xr + i);
#pragma unroll
                for (int k = 0; k < H; ++k) {
                    const f32x4 uv = *reinterpret_cast<const f32x4 *>(ur + k * kTpD + i);
                    part[k] += xv.x * uv.x + xv.y * uv.y + xv.z * uv.z + xv.w * uv.w;
                }
            }
#pragma unroll
            for (int k = 0; k < H; ++k) s_part[(wave * H + k) * kTpChunk + lane] = part[k];
        }
        __syncthreads();

        // ---- online softmax per environment and team: wave = head ----
        if (wave < H) {
            const int head = wave;
            float dot = 0.0f;
#pragma unroll
            for (int qw = 0; qw < 4; ++qw) dot += s_part[(qw * H + head) * kTpChunk + lane];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const bool mine = key && ship_team == t;
                const float sc = mine ? dot : -INFINITY;
                const float new_max = fmaxf(run_max[t], seg_max<SEG>(sc));
                const bool none = new_max == -INFINITY;  // no key of this team so far
                const float pt = none ? 0.0f : __builtin_amdgcn_exp2f(sc - new_max);
                const float alpha = none ? 1.0f : __builtin_amdgcn_exp2f(run_max[t] - new_max);
                run_sum[t] = run_sum[t] * alpha + seg_sum<SEG>(pt);
                run_max[t] = new_max;
                s_p[lane * NC + t * H + head] = mine ? pt : 0.0f;
                if (srow == 0) s_alpha[seg * NC + t * H + head] = alpha;
            }
        }
        __syncthreads();

        // ---- z(t, h)[d] = alpha z + sum_j p_j x_j[d] for the H heads of team tm.  Eight rows per
        //      step, all their LDS reads issued before the arithmetic (the loop is bound by LDS
        //      latency otherwise); rows past the chunk were never written and carry p = 0 only
        //      if they are cleared, so the tail is done row by row. ----
#pragma unroll
        for (int q = 0; q < EPP; ++q) {
#pragma unroll
            for (int k = 0; k < H; ++k) z[q][k] *= s_alpha[q * NC + tm * H + k];
            const float *xq = s_x + q * SEG * kTpPitch + d;
            const float *pq = s_p + q * SEG * NC + tm * H;
            int j = 0;
            for (; j + 8 <= rows; j += 8) {
                float xv[8], pv[8][H];
#pragma unroll
                for (int jj = 0; jj < 8; ++jj) {
                    xv[jj] = xq[(j + jj) * kTpPitch];
#pragma unroll
                    for (int k = 0; k < H; ++k) pv[jj][k] = pq[(j + jj) * NC + k];
                }
#pragma unroll
                for (int jj = 0; jj < 8; ++jj)
#pragma unroll
                    for (int k = 0; k < H; ++k) z[q][k] += pv[jj][k] * xv[jj];
            }
            for (; j < rows; ++j) {
                const float xv = xq[j * kTpPitch];
#pragma unroll
                for (int k = 0; k < H; ++k) z[q][k] += pq[j * NC + k] * xv;
            }
        }
    }
    __syncthreads();
    if (srow == 0 && wave < H) {
#pragma unroll
        for (int t = 0; t < 2; ++t) s_l[seg * NC + t * H + wave] = run_sum[t];
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < EPP; ++q) {
        if (env_first + q >= B) break;
#pragma unroll
        for (int k = 0; k < H; ++k) {
            const float l = s_l[q * NC + tm * H + k];  // 0: no alive ship on this team
            z_out[((int64_t)(env_first + q) * NC + tm * H + k) * kTpD + d] = l > 0.0f ? z[q][k] / l : 0.0f;
        }
    }
}

// RMSNorm of the projected team vectors and the hand-out to the ships: `pre` (B, 2, 128) ->
// pool (B, 2, 128) and out[b, n] = pool[b, clamp(team_id[b, n], 0, 1)].  One work-group per
// kTpEnvs environments; a zero vector (empty team) stays zero.
__global__ __launch_bounds__(kTpThreads) void team_norm_broadcast_kernel(
    const float *__restrict__ pre, const float *__restrict__ norm_w, float eps, const int32_t *__restrict__ team_id,
    int64_t team_env_stride, float *__restrict__ pool, float *__restrict__ out, int64_t out_env_stride,
    int64_t out_row_stride, int B, int N)
{
    __shared__ __align__(16) float s_pool[kTpEnvs * 2 * kTpD];
    __shared__ float s_red[kTpEnvs * 4];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int d = tid & (kTpD - 1), tm = tid >> 7;
    const int env0 = blockIdx.x * kTpEnvs;
    float v[kTpEnvs];
#pragma unroll
    for (int g = 0; g < kTpEnvs; ++g) {
        v[g] = env0 + g < B ? pre[((int64_t)(env0 + g) * 2 + tm) * kTpD + d] : 0.0f;
        const float ss = seg_sum<64>(v[g] * v[g]);
        if (lane == 0) s_red[g * 4 + wave] = ss;
    }
    __syncthreads();
    const float nw = norm_w[d];
#pragma unroll
    for (int g = 0; g < kTpEnvs; ++g) {
        const float ms = (s_red[g * 4 + 2 * tm] + s_red[g * 4 + 2 * tm + 1]) * (1.0f / kTpD);
        const float r = v[g] * rsqrtf(ms + eps) * nw;
        s_pool[(g * 2 + tm) * kTpD + d] = r;
        if (env0 + g < B && pool != nullptr) pool[((int64_t)(env0 + g) * 2 + tm) * kTpD + d] = r;
    }
    __syncthreads();
    if (out == nullptr) return;
    for (int g = 0; g < kTpEnvs; ++g) {
        const int env = env0 + g;
        if (env >= B) break;
        const int32_t *te = team_id + (int64_t)env * team_env_stride;
        float *oe = out + (int64_t)env * out_env_stride;
        for (int idx = tid; idx < N * (kTpD / 4); idx += kTpThreads) {
            const int n = idx >> 5, q4 = (idx & 31) * 4;
            int t = te[n];
            t = t < 0 ? 0 : (t > 1 ? 1 : t);
            *reinterpret_cast<f32x4 *>(oe + (int64_t)n * out_row_stride + q4) =
                *reinterpret_cast<const f32x4 *>(s_pool + (g * 2 + t) * kTpD + q4);
        }
    }
}

template <int H, int SEG>
static int launch_team_attend(const float *x, int64_t x_env_stride, int64_t x_row_stride, const int32_t *team_id,
                              int64_t team_env_stride, const uint8_t *alive, int64_t alive_env_stride,
                              const float *score_vectors, float *z, int B, int N, hipStream_t s)
{
    constexpr int EPP = kTpChunk / SEG;
    const int64_t blocks = ((int64_t)B + EPP - 1) / EPP;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((team_attend_kernel<H, SEG>), dim3((unsigned)blocks), dim3(kTpThreads), 0, s, x, x_env_stride,
                       x_row_stride, team_id, team_env_stride, alive, alive_env_stride, score_vectors, z, B, N);
    return (int)hipGetLastError();
}

}  // namespace bnb

extern "C" int bnb_team_attend_fwd(const float *x, int64_t x_env_stride, int64_t x_row_stride, const int32_t *team_id,
                                   int64_t team_env_stride, const uint8_t *alive, int64_t alive_env_stride,
                                   const float *score_vectors, float *z, int B, int N, int H, int D, void *stream)
{
    using namespace bnb;
    if (B < 0 || N < 0 || H < 1) return BNB_ERR_BAD_SHAPE;
    if (D != kTpD || (H != 2 && H != 4)) return BNB_ERR_UNSUPPORTED;
    if (B == 0) return 0;
    if (!x || !team_id || !alive || !score_vectors || !z) return BNB_ERR_NULL_POINTER;
    if (x_row_stride < D || x_env_stride < (int64_t)N * D || team_env_stride < N || alive_env_stride < N)
        return BNB_ERR_BAD_SHAPE;
    if (!aligned16(x) || (x_row_stride % 4) != 0 || (x_env_stride % 4) != 0) return BNB_ERR_MISALIGNED;
    hipStream_t s = (hipStream_t)stream;
#define BNB_TP_ARGS x, x_env_stride, x_row_stride, team_id, team_env_stride, alive, alive_env_stride, score_vectors, z, B, N, s
    // up to 16 ships: four environments share a work-group; otherwise one environment each
    if (H == 4) return N <= 16 ? launch_team_attend<4, 16>(BNB_TP_ARGS) : launch_team_attend<4, 64>(BNB_TP_ARGS);
    return N <= 16 ? launch_team_attend<2, 16>(BNB_TP_ARGS) : launch_team_attend<2, 64>(BNB_TP_ARGS);
#undef BNB_TP_ARGS
}

extern "C" int bnb_team_norm_broadcast_fwd(const float *pre, const float *norm_weight, float eps, const int32_t *team_id,
                                           int64_t team_env_stride, float *pool, float *out, int64_t out_env_stride,
                                           int64_t out_row_stride, int B, int N, int D, void *stream)
{
    using namespace bnb;
    if (B < 0 || N < 0) return BNB_ERR_BAD_SHAPE;
    if (D != kTpD) return BNB_ERR_UNSUPPORTED;
    if (B == 0) return 0;
    if (!pre || !norm_weight || (!pool && !out) || (out && !team_id)) return BNB_ERR_NULL_POINTER;
    if (out && (out_row_stride < D || out_env_stride < (int64_t)N * D || team_env_stride < N)) return BNB_ERR_BAD_SHAPE;
    if (out && (!aligned16(out) || (out_row_stride % 4) != 0 || (out_env_stride % 4) != 0)) return BNB_ERR_MISALIGNED;
    const int64_t blocks = ((int64_t)B + kTpEnvs - 1) / kTpEnvs;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(team_norm_broadcast_kernel, dim3((unsigned)blocks), dim3(kTpThreads), 0, (hipStream_t)stream, pre,
                       norm_weight, eps, team_id, team_env_stride, pool, out, out_env_stride, out_row_stride, B, N);
    return (int)hipGetLastError();
}
