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
#include "common.h"

namespace bnb {

constexpr int kTpD = 128;
constexpr int kTpThreads = 256;
constexpr int kTaRows = 16;            // ship rows a wave stages at a time
constexpr int kTaWaves = 4;            // waves (environments) per work-group of the attend kernel
constexpr int kTpPitch = kTpD + 4;     // floats per staged row: 16-byte aligned, bank-spread
constexpr int kTpEnvs = 4;             // environments per work-group of the norm + hand-out kernel

// All-reduce over the aligned group of 16 lanes a lane belongs to, on the data-parallel
// primitives (no LDS round trips): swap inside pairs, pairs inside quads, then mirror inside 8
// and inside 16 (after the first two steps a quad is uniform, so mirroring exchanges quads).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

__device__ __forceinline__ float row16_max(float v)
{
    v = fmaxf(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_move<0x141>(v));  // row_half_mirror
    return fmaxf(v, dpp_move<0x140>(v));  // row_mirror
}

__device__ __forceinline__ float row16_sum(float v)
{
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    return v + dpp_move<0x140>(v);
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// One wavefront per environment, four per work-group, each on its own: after the score vectors
// are in LDS no work-group barrier is left, only hand-overs inside the wave, so a CU keeps 16
// independent waves busy.  Ships come in chunks of 16 rows through the wave's private LDS tile
// (the next chunk is already in flight in registers).  Writes z (B, 2, H, 128): the
// softmax-weighted mean of the ship rows per (team, head), zero for a team without an alive ship.
//   scores     lane = (channel quarter g, ship s): partial dot products of ship s with the H
//              score vectors of ITS team (the other team's would be masked) over channels
//              32g .. 32g+31, summed over g with two cross-lane steps
//   softmax    lane (g, s) keeps head g: online maximum / sum over the 16-lane group of head g,
//              separately for the two teams
//   pooling    lane l = channels 2l, 2l+1 of all 2H weighted sums
template <int H>
__global__ __launch_bounds__(kTaWaves * kWave) void team_attend_kernel(
    const float *__restrict__ x, int64_t x_env_stride, int64_t x_row_stride, const int32_t *__restrict__ team_id,
    int64_t team_env_stride, const uint8_t *__restrict__ alive, int64_t alive_env_stride,
    const float *__restrict__ score_vec, float *__restrict__ z_out, int B, int N)
{
    constexpr int NC = 2 * H;                  // (team, head) pairs
    constexpr int kTeamPitch = H * kTpD + 4;   // team 1's vectors start 16 bytes off team 0's banks
    __shared__ __align__(16) float s_u[2 * kTeamPitch];
    __shared__ __align__(16) float s_x[kTaWaves][kTaRows * kTpPitch];
    __shared__ __align__(16) float s_p[kTaWaves][kTaRows * NC];  // softmax numerators; 0 under the other team's heads
    __shared__ float s_scale[kTaWaves][2 * NC];                   // per pair: rescale factor, then the final sum

    const int tid = threadIdx.x;
    for (int i = tid; i < NC * kTpD; i += kTaWaves * kWave)
        s_u[(i / (H * kTpD)) * kTeamPitch + i % (H * kTpD)] = score_vec[i];
    __syncthreads();

    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int env = blockIdx.x * kTaWaves + wave;
    if (env >= B) return;
    float *tile = s_x[wave];
    float *ptile = s_p[wave];
    float *scale = s_scale[wave];
    const int g = lane >> 4;   // channel quarter in the score phase, head in the softmax
    const int ship = lane & 15;
    const float *xe = x + (int64_t)env * x_env_stride;
    const int32_t *te = team_id + (int64_t)env * team_env_stride;
    const uint8_t *ae = alive + (int64_t)env * alive_env_stride;

    float run_max[2] = {-INFINITY, -INFINITY}, run_sum[2] = {0.0f, 0.0f};  // head g, per team
    float z[NC][2];
#pragma unroll
    for (int c = 0; c < NC; ++c) z[c][0] = z[c][1] = 0.0f;

    // a lane's share of a chunk: 8 pieces of 16 bytes (piece = lane + 64*it: row piece/32)
    constexpr int kPieces = kTaRows * (kTpD / 4) / kWave;
    f32x4 stage[kPieces];
    int stage_team = -1, stage_alive = 0;  // of ship `ship` of the chunk in flight
    auto fetch = [&](int c0) {
        const int rows = N - c0 < kTaRows ? N - c0 : kTaRows;
        const int sr = ship < rows ? ship : rows - 1;
        stage_team = te[c0 + sr];
        stage_alive = ae[c0 + sr];
#pragma unroll
        for (int it = 0; it < kPieces; ++it) {
            const int idx = lane + it * kWave;
            const int r = idx >> 5, q4 = (idx & 31) * 4;
            const int rr = r < rows ? r : rows - 1;  // rows past the end re-read the last one and are zeroed below
            stage[it] = *reinterpret_cast<const f32x4 *>(xe + (int64_t)(c0 + rr) * x_row_stride + q4);
        }
    };

    if (N > 0) fetch(0);
    for (int c0 = 0; c0 < N; c0 += kTaRows) {
        const int rows = N - c0 < kTaRows ? N - c0 : kTaRows;
        // absent rows are stored as zeros: their weight is 0 and 0 * finite keeps the sums clean
#pragma unroll
        for (int it = 0; it < kPieces; ++it) {
            const int idx = lane + it * kWave;
            const int r = idx >> 5, q4 = (idx & 31) * 4;
            *reinterpret_cast<f32x4 *>(tile + r * kTpPitch + q4) = r < rows ? stage[it] : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
        const bool present = ship < rows;
        const int ship_team = present ? stage_team : -1;
        const bool key = present && stage_alive != 0 && (ship_team == 0 || ship_team == 1);
        if (c0 + kTaRows < N) fetch(c0 + kTaRows);
        wave_lds_handover();

        // ---- partial scores over this lane's channel quarter, all heads of the ship's team ----
        float part[H];
#pragma unroll
        for (int k = 0; k < H; ++k) part[k] = 0.0f;
        {
            const float *xr = tile + ship * kTpPitch + 32 * g;
            const float *ur = s_u + (key ? ship_team : 0) * kTeamPitch + 32 * g;
#pragma unroll
            for (int i = 0; i < 32; i += 4) {
                const f32x4 xv = *reinterpret_cast<const f32x4 *>(xr + i);
#pragma unroll
                for (int k = 0; k < H; ++k) {
                    const f32x4 uv = *reinterpret_cast<const f32x4 *>(ur + k * kTpD + i);
                    part[k] += xv.x * uv.x + xv.y * uv.y + xv.z * uv.z + xv.w * uv.w;
                }
            }
        }
        // sum over the four channel quarters (lanes l, l^16, l^32, l^48); lane (g, s) keeps head g
        float dot = 0.0f;
#pragma unroll
        for (int k = 0; k < H; ++k) {
            float v = part[k];
            v += __shfl_xor(v, 16);
            v += __shfl_xor(v, 32);
            if (k == g) dot = v;
        }

        // ---- online softmax of head g over the 16 ships, per team ----
        if (g < H) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const bool mine = key && ship_team == t;
                const float sc = mine ? dot : -INFINITY;
                const float new_max = fmaxf(run_max[t], row16_max(sc));
                const bool none = new_max == -INFINITY;  // no key of this team so far
                const float pt = none ? 0.0f : __builtin_amdgcn_exp2f(sc - new_max);
                const float alpha = none ? 1.0f : __builtin_amdgcn_exp2f(run_max[t] - new_max);
                run_sum[t] = run_sum[t] * alpha + row16_sum(pt);
                run_max[t] = new_max;
                ptile[ship * NC + t * H + g] = mine ? pt : 0.0f;
                if (ship == 0) scale[t * H + g] = alpha;
            }
        }
        wave_lds_handover();

        // ---- z(t, h)[2l, 2l+1] = alpha z + sum_j p_j x_j ----
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const float a = scale[c];
            z[c][0] *= a, z[c][1] *= a;
        }
#pragma unroll 4
        for (int j = 0; j < kTaRows; ++j) {
            const f32x2 xv = *reinterpret_cast<const f32x2 *>(tile + j * kTpPitch + 2 * lane);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const float pv = ptile[j * NC + c];
                z[c][0] += pv * xv.x, z[c][1] += pv * xv.y;
            }
        }
        wave_lds_handover();  // the tile is rewritten by the next chunk
    }
    if (g < H && ship == 0) {
#pragma unroll
        for (int t = 0; t < 2; ++t) scale[NC + t * H + g] = run_sum[t];
    }
    wave_lds_handover();
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const float l = scale[NC + c];  // 0: no alive ship on this team
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        const f32x2 r = {z[c][0] * inv, z[c][1] * inv};
        *reinterpret_cast<f32x2 *>(z_out + ((int64_t)env * NC + c) * kTpD + 2 * lane) = r;
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
        const float ss = wave_sum(v[g] * v[g]);
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

// Backward of team_attend_kernel for the update path.  With p = softmax over the team's alive
// ships of the base-2 scores x_j . u(t, h) and z(t, h) = sum_j p_j x_j:
//   dp_j = x_j . dz(t, h),   delta(t, h) = sum_j p_j dp_j = z(t, h) . dz(t, h)   (z is the forward's result),
//   ds_j = ln2 p_j (dp_j - delta),   dx_j = sum_h p_j dz(t_j, h) + ds_j u(t_j, h),   du(t, h) = sum_j ds_j x_j.
// Same layout as the forward: one wave per environment, ships in chunks of 16 through the wave's
// LDS tile, lane = (channel quarter, ship).  Pass 1 repeats the online maximum / sum, pass 2 forms p,
// ds and dx.  The ds values go out as a (B*N, 2H) matrix (zero under the other team's heads), so
// that du is a plain product with x, formed by team_du_kernel in a fixed order.
template <int H>
__global__ __launch_bounds__(kTaWaves * kWave) void team_attend_bwd_kernel(
    const float *__restrict__ x, int64_t x_env_stride, int64_t x_row_stride, const int32_t *__restrict__ team_id,
    int64_t team_env_stride, const uint8_t *__restrict__ alive, int64_t alive_env_stride,
    const float *__restrict__ score_vec, const float *__restrict__ z, const float *__restrict__ dz,
    float *__restrict__ dx, float *__restrict__ ds_out, int B, int N)
{
    constexpr int NC = 2 * H;
    constexpr int kTeamPitch = H * kTpD + 4;
    constexpr int kPerPair = kWave / NC;          // lanes that share one (team, head) pair in the delta step
    constexpr int kSpan = kTpD / kPerPair;        // channels of such a lane
    __shared__ __align__(16) float s_u[2 * kTeamPitch];
    __shared__ __align__(16) float s_x[kTaWaves][kTaRows * kTpPitch];
    __shared__ __align__(16) float s_dz[kTaWaves][2 * kTeamPitch];
    __shared__ float s_stat[kTaWaves][3 * NC];  // per pair: maximum, 1 / sum, delta

    const int tid = threadIdx.x;
    for (int i = tid; i < NC * kTpD; i += kTaWaves * kWave)
        s_u[(i / (H * kTpD)) * kTeamPitch + i % (H * kTpD)] = score_vec[i];
    __syncthreads();

    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int env = blockIdx.x * kTaWaves + wave;
    if (env >= B) return;
    float *tile = s_x[wave];
    float *dzt = s_dz[wave];
    float *stat = s_stat[wave];
    const int g = lane >> 4, ship = lane & 15;
    const float *xe = x + (int64_t)env * x_env_stride;
    const int32_t *te = team_id + (int64_t)env * team_env_stride;
    const uint8_t *ae = alive + (int64_t)env * alive_env_stride;

    // dz of the environment into LDS, and delta = z . dz per pair
    {
        const int pair = lane / kPerPair, c0 = (lane % kPerPair) * kSpan;
        const float *zp = z + ((int64_t)env * NC + pair) * kTpD + c0;
        const float *dp = dz + ((int64_t)env * NC + pair) * kTpD + c0;
        float *dst = dzt + (pair / H) * kTeamPitch + (pair % H) * kTpD + c0;
        float d = 0.0f;
#pragma unroll
        for (int i = 0; i < kSpan; i += 4) {
            const f32x4 zv = *reinterpret_cast<const f32x4 *>(zp + i);
            const f32x4 dv = *reinterpret_cast<const f32x4 *>(dp + i);
            *reinterpret_cast<f32x4 *>(dst + i) = dv;
            d += zv.x * dv.x + zv.y * dv.y + zv.z * dv.z + zv.w * dv.w;
        }
#pragma unroll
        for (int o = 1; o < kPerPair; o <<= 1) d += __shfl_xor(d, o);
        if (lane % kPerPair == 0) stat[2 * NC + pair] = d;
    }

    constexpr int kPieces = kTaRows * (kTpD / 4) / kWave;
    // stage a chunk of ship rows (absent rows as zeros) and return this lane's ship's key status
    auto stage_chunk = [&](int c0, int &ship_team, bool &key) {
        const int rows = N - c0 < kTaRows ? N - c0 : kTaRows;
#pragma unroll
        for (int it = 0; it < kPieces; ++it) {
            const int idx = lane + it * kWave;
            const int r = idx >> 5, q4 = (idx & 31) * 4;
            const int rr = r < rows ? r : rows - 1;
            const f32x4 v = *reinterpret_cast<const f32x4 *>(xe + (int64_t)(c0 + rr) * x_row_stride + q4);
            *reinterpret_cast<f32x4 *>(tile + r * kTpPitch + q4) = r < rows ? v : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
        const bool present = ship < rows;
        const int sr = present ? ship : rows - 1;
        ship_team = present ? te[c0 + sr] : -1;
        key = present && ae[c0 + sr] != 0 && (ship_team == 0 || ship_team == 1);
    };
    // scores of the lane's ship with the H vectors of `vecs` for its team, summed over the channel quarters
    auto dots = [&](const float *vecs, int team, float (&out)[H]) {
        const float *xr = tile + ship * kTpPitch + 32 * g;
        const float *ur = vecs + team * kTeamPitch + 32 * g;
#pragma unroll
        for (int k = 0; k < H; ++k) out[k] = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; i += 4) {
            const f32x4 xv = *reinterpret_cast<const f32x4 *>(xr + i);
#pragma unroll
            for (int k = 0; k < H; ++k) {
                const f32x4 uv = *reinterpret_cast<const f32x4 *>(ur + k * kTpD + i);
                out[k] += xv.x * uv.x + xv.y * uv.y + xv.z * uv.z + xv.w * uv.w;
            }
        }
#pragma unroll
        for (int k = 0; k < H; ++k) {
            out[k] += __shfl_xor(out[k], 16);
            out[k] += __shfl_xor(out[k], 32);
        }
    };

    // ---- pass 1: maximum and sum per (team, head); lane (g, ship) keeps head g ----
    float run_max[2] = {-INFINITY, -INFINITY}, run_sum[2] = {0.0f, 0.0f};
    for (int c0 = 0; c0 < N; c0 += kTaRows) {
        int ship_team;
        bool key;
        stage_chunk(c0, ship_team, key);
        wave_lds_handover();
        float sc[H];
        dots(s_u, key ? ship_team : 0, sc);
        float dot = 0.0f;
#pragma unroll
        for (int k = 0; k < H; ++k)
            if (k == g) dot = sc[k];
        if (g < H) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const bool mine = key && ship_team == t;
                const float v = mine ? dot : -INFINITY;
                const float new_max = fmaxf(run_max[t], row16_max(v));
                const bool none = new_max == -INFINITY;
                const float pt = none ? 0.0f : __builtin_amdgcn_exp2f(v - new_max);
                const float alpha = none ? 1.0f : __builtin_amdgcn_exp2f(run_max[t] - new_max);
                run_sum[t] = run_sum[t] * alpha + row16_sum(pt);
                run_max[t] = new_max;
            }
        }
        wave_lds_handover();  // the tile is rewritten by the next chunk
    }
    if (g < H && ship == 0) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            stat[t * H + g] = run_max[t];
            stat[NC + t * H + g] = run_sum[t] > 0.0f ? 1.0f / run_sum[t] : 0.0f;
        }
    }
    wave_lds_handover();

    // ---- pass 2: p, ds, dx ----
    for (int c0 = 0; c0 < N; c0 += kTaRows) {
        int ship_team;
        bool key;
        stage_chunk(c0, ship_team, key);
        wave_lds_handover();
        const int t = key ? ship_team : 0;
        float sc[H], dp[H], p[H], ds[H];
        dots(s_u, t, sc);
        dots(dzt, t, dp);
#pragma unroll
        for (int k = 0; k < H; ++k) {
            p[k] = key ? __builtin_amdgcn_exp2f(sc[k] - stat[t * H + k]) * stat[NC + t * H + k] : 0.0f;
            ds[k] = 0.6931471805599453f * p[k] * (dp[k] - stat[2 * NC + t * H + k]);
        }
        if (c0 + ship < N) {
            float *dxr = dx + ((int64_t)env * N + c0 + ship) * kTpD + 32 * g;
            const float *ur = s_u + t * kTeamPitch + 32 * g;
            const float *dr = dzt + t * kTeamPitch + 32 * g;
#pragma unroll
            for (int i = 0; i < 32; i += 4) {
                f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int k = 0; k < H; ++k) {
                    const f32x4 uv = *reinterpret_cast<const f32x4 *>(ur + k * kTpD + i);
                    const f32x4 dv = *reinterpret_cast<const f32x4 *>(dr + k * kTpD + i);
                    acc.x += p[k] * dv.x + ds[k] * uv.x, acc.y += p[k] * dv.y + ds[k] * uv.y;
                    acc.z += p[k] * dv.z + ds[k] * uv.z, acc.w += p[k] * dv.w + ds[k] * uv.w;
                }
                *reinterpret_cast<f32x4 *>(dxr + i) = acc;
            }
            if (g == 0) {
                float *row = ds_out + ((int64_t)env * N + c0 + ship) * NC;
#pragma unroll
                for (int c = 0; c < NC; ++c) row[c] = (c / H == t) ? ds[c % H] : 0.0f;
            }
        }
        wave_lds_handover();
    }
}

// Backward of the hand-out: dpool(b, t) = sum of dout over the ships that hold team t's vector
// (clamp(team_id, 0, 1) == t), zero for a team without an alive ship of its own (its vector is the
// constant zero).  One thread per (environment, 4 channels).
__global__ __launch_bounds__(256) void team_gather_bwd_kernel(const float *__restrict__ dout, const int32_t *__restrict__ team_id,
                                                              int64_t team_env_stride, const uint8_t *__restrict__ alive,
                                                              int64_t alive_env_stride, float *__restrict__ dpool, int B, int N)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t env = idx >> 5;
    if (env >= B) return;
    const int q4 = (int)(idx & 31) * 4;
    const int32_t *te = team_id + env * team_env_stride;
    const uint8_t *ae = alive + env * alive_env_stride;
    const float *de = dout + env * N * kTpD + q4;
    f32x4 a0 = {0.0f, 0.0f, 0.0f, 0.0f}, a1 = a0;
    bool has0 = false, has1 = false;
    for (int n = 0; n < N; ++n) {
        const int t = te[n];
        const bool al = ae[n] != 0;
        has0 |= al && t == 0;
        has1 |= al && t == 1;
        const f32x4 v = *reinterpret_cast<const f32x4 *>(de + (int64_t)n * kTpD);
        if (t >= 1) a1.x += v.x, a1.y += v.y, a1.z += v.z, a1.w += v.w;
        else a0.x += v.x, a0.y += v.y, a0.z += v.z, a0.w += v.w;
    }
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    *reinterpret_cast<f32x4 *>(dpool + (env * 2 + 0) * kTpD + q4) = has0 ? a0 : zero;
    *reinterpret_cast<f32x4 *>(dpool + (env * 2 + 1) * kTpD + q4) = has1 ? a1 : zero;
}

// du(pair) = sum over all ship rows of ds(row, pair) * x(row): rows dealt to the work-groups in
// contiguous runs, a thread per (channel, half of the pairs), partial sums per work-group, then
// sum_slices in a fixed order.
constexpr int kDuBlocks = 2048;  // measured: 1280 (all resident at once) is 10 % slower

__global__ __launch_bounds__(256) void team_du_kernel(const float *__restrict__ x, int64_t x_env_stride, int64_t x_row_stride,
                                                      const float *__restrict__ ds, float *__restrict__ partials, int64_t rows,
                                                      int N, int NC)
{
    // thread = (row lane 0..7, 4 channels); rows of the work-group's run are taken 8 at a time
    __shared__ __align__(16) float s_acc[8][8 * kTpD];
    const int q4 = (threadIdx.x & 31) * 4, rl = threadIdx.x >> 5;
    const int64_t per = (rows + gridDim.x - 1) / gridDim.x;
    const int64_t r0 = (int64_t)blockIdx.x * per, r1 = r0 + per < rows ? r0 + per : rows;
    f32x4 acc[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 4
    for (int64_t r = r0 + rl; r < r1; r += 8) {
        const uint32_t r32 = (uint32_t)r;  // B * N < 2^31: 32-bit division
        const uint32_t env = r32 / (uint32_t)N;
        const uint32_t n = r32 - env * (uint32_t)N;
        const f32x4 xv = *reinterpret_cast<const f32x4 *>(x + (int64_t)env * x_env_stride + (int64_t)n * x_row_stride + q4);
        const float *d = ds + r * NC;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if (c < NC) {
                const float w = d[c];
                acc[c].x = fmaf(w, xv.x, acc[c].x), acc[c].y = fmaf(w, xv.y, acc[c].y);
                acc[c].z = fmaf(w, xv.z, acc[c].z), acc[c].w = fmaf(w, xv.w, acc[c].w);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < 8; ++c)
        if (c < NC) *reinterpret_cast<f32x4 *>(&s_acc[rl][c * kTpD + q4]) = acc[c];
    __syncthreads();
    for (int i = threadIdx.x; i < NC * kTpD; i += 256) {
        float t = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) t += s_acc[j][i];
        partials[(int64_t)blockIdx.x * NC * kTpD + i] = t;
    }
}

template <int H>
static int launch_team_attend(const float *x, int64_t x_env_stride, int64_t x_row_stride, const int32_t *team_id,
                              int64_t team_env_stride, const uint8_t *alive, int64_t alive_env_stride,
                              const float *score_vectors, float *z, int B, int N, hipStream_t s)
{
    const int64_t blocks = ((int64_t)B + kTaWaves - 1) / kTaWaves;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((team_attend_kernel<H>), dim3((unsigned)blocks), dim3(kTaWaves * kWave), 0, s, x, x_env_stride,
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
    if (H == 4)
        return launch_team_attend<4>(x, x_env_stride, x_row_stride, team_id, team_env_stride, alive, alive_env_stride,
                                     score_vectors, z, B, N, s);
    return launch_team_attend<2>(x, x_env_stride, x_row_stride, team_id, team_env_stride, alive, alive_env_stride,
                                 score_vectors, z, B, N, s);
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

extern "C" int bnb_team_attend_bwd(const float *x, int64_t x_env_stride, int64_t x_row_stride, const int32_t *team_id,
                                   int64_t team_env_stride, const uint8_t *alive, int64_t alive_env_stride,
                                   const float *score_vectors, const float *z, const float *dz, float *dx, float *ds,
                                   float *partials, float *du, int B, int N, int H, int D, void *stream)
{
    using namespace bnb;
    if (B < 0 || N < 0 || H < 1) return BNB_ERR_BAD_SHAPE;
    if (D != kTpD || (H != 2 && H != 4)) return BNB_ERR_UNSUPPORTED;
    if (!du || !partials) return BNB_ERR_NULL_POINTER;
    hipStream_t s = (hipStream_t)stream;
    const int NC = 2 * H;
    if (B == 0 || N == 0) return launch_sum_slices(partials, du, (int64_t)NC * kTpD, 0, 0, s);
    if ((int64_t)B * N >= (1LL << 31)) return BNB_ERR_UNSUPPORTED;
    if (!x || !team_id || !alive || !score_vectors || !z || !dz || !dx || !ds) return BNB_ERR_NULL_POINTER;
    if (x_row_stride < D || x_env_stride < (int64_t)N * D || team_env_stride < N || alive_env_stride < N)
        return BNB_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(z) || !aligned16(dz) || !aligned16(dx) || !aligned16(partials) || !aligned16(du) ||
        (x_row_stride % 4) != 0 || (x_env_stride % 4) != 0)
        return BNB_ERR_MISALIGNED;
    const int64_t blocks = ((int64_t)B + kTaWaves - 1) / kTaWaves;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    if (H == 4)
        hipLaunchKernelGGL((team_attend_bwd_kernel<4>), dim3((unsigned)blocks), dim3(kTaWaves * kWave), 0, s, x, x_env_stride,
                           x_row_stride, team_id, team_env_stride, alive, alive_env_stride, score_vectors, z, dz, dx, ds, B, N);
    else
        hipLaunchKernelGGL((team_attend_bwd_kernel<2>), dim3((unsigned)blocks), dim3(kTaWaves * kWave), 0, s, x, x_env_stride,
                           x_row_stride, team_id, team_env_stride, alive, alive_env_stride, score_vectors, z, dz, dx, ds, B, N);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(team_du_kernel, dim3(kDuBlocks), dim3(256), 0, s, x, x_env_stride, x_row_stride, ds, partials,
                       (int64_t)B * N, N, NC);
    e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return launch_sum_slices(partials, du, (int64_t)NC * kTpD, kDuBlocks, 0, s);
}

extern "C" int bnb_team_attend_bwd_partial_rows(void) { return bnb::kDuBlocks; }

extern "C" int bnb_team_gather_bwd(const float *dout, const int32_t *team_id, int64_t team_env_stride, const uint8_t *alive,
                                   int64_t alive_env_stride, float *dpool, int B, int N, int D, void *stream)
{
    using namespace bnb;
    if (B < 0 || N < 0) return BNB_ERR_BAD_SHAPE;
    if (D != kTpD) return BNB_ERR_UNSUPPORTED;
    if (B == 0) return 0;
    if (!dpool || (N > 0 && (!dout || !team_id || !alive))) return BNB_ERR_NULL_POINTER;
    if (team_env_stride < N || alive_env_stride < N) return BNB_ERR_BAD_SHAPE;
    if (!aligned16(dout) || !aligned16(dpool)) return BNB_ERR_MISALIGNED;
    const int64_t blocks = ((int64_t)B * 32 + 255) / 256;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(team_gather_bwd_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, dout, team_id,
                       team_env_stride, alive, alive_env_stride, dpool, B, N);
    return (int)hipGetLastError();
}
