// The bullet read in float32 on the fp32 matrix cores, for gfx950.
//
// Entity queries read a second set of key/value rows (models/yemong/attention.py:149-166) when the
// policy runs without autocast (evaluation, crossover: evaluation/agents.py:214-219).  Same
// mathematics as the bf16 bullet read: only active keys take part, an environment without an active
// key contributes exactly zero (the reference's any_active gate), the result is added to the
// self-attention output.  True fp32 products (v_mfma_f32_32x32x2_f32), so the 1e-5 bar holds.
//
// One work-group per (environment, head), one wave per 32 queries.  The work-group first lists the
// active slots of its environment in LDS (ascending), then walks that list in tiles of 32 keys per
// wave: K and V rows of a tile are staged in LDS, every wave forms S^T = K Q^T for its queries and
// carries an online softmax (running maximum, sum, rescaled O^T) from tile to tile.  Operand
// layouts are those of the fp32 self-attention kernel: keys on the M axis so a lane holds 16
// scores of ONE query; the k index of K Q^T walks channel 16*half + s, the k index of V^T P^T walks
// key 8(s/4) + 4*half + s%4, the key whose score sits in accumulator register s, so P never moves
// and V is read from LDS as stored.  Positions past the last active key are zero rows whose scores
// are forced to -inf.

#include "common.h"

namespace bnb {

constexpr float kLog2eC = 1.4426950408889634f;
constexpr int kCDh = 32;
constexpr int kCKeyPitch = kCDh + 1;   // floats per K row in LDS: odd, so 32 rows hit 32 banks
constexpr int kCrossF32MaxKeys = 4096;  // slots per environment the index list holds

__global__ __launch_bounds__(1024) void sdpa_cross_f32_kernel(
    const float *__restrict__ q, int64_t q_stride, const float *__restrict__ k, const float *__restrict__ v,
    int64_t kv_stride, const uint8_t *__restrict__ key_mask, const float *accum, float *out, int B, int NQ, int NK, int H,
    float scale_log2e)
{
    extern __shared__ __align__(16) float s_c32[];
    const int nwaves = blockDim.x >> 6;
    const int TK = nwaves * 32;  // keys per tile
    float *s_k = s_c32;                                      // [TK][33]
    float *s_v = s_k + TK * kCKeyPitch;                      // [TK][32]
    uint16_t *s_idx = reinterpret_cast<uint16_t *>(s_v + TK * kCDh);  // [kCrossF32MaxKeys]
    int *s_wcnt = reinterpret_cast<int *>(s_idx + kCrossF32MaxKeys);  // [nwaves]

    const int chunk = gridDim.x >> 3;
    const int logical = (blockIdx.x & 7) * chunk + (blockIdx.x >> 3);
    if (logical >= B * H) return;
    const int env = logical / H;
    const int head = logical - env * H;
    const int D = H * kCDh;
    const int tid = threadIdx.x;
    const int NT = blockDim.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 31;
    const int half = lane >> 5;

    // this lane's query values: channels 16*half .. +15 of query 32*wave + m, in flight during the scan
    const int qrow = wave * 32 + m;
    const float *qp = q + ((int64_t)env * NQ + (qrow < NQ ? qrow : NQ - 1)) * q_stride + head * kCDh + 16 * half;
    f32x4 qv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) qv[i] = *reinterpret_cast<const f32x4 *>(qp + 4 * i);

    // ---- ascending list of the active slots: wave w scans slots [w*J*64, (w+1)*J*64), 64 per ballot ----
    const uint8_t *mask_env = key_mask == nullptr ? nullptr : key_mask + (int64_t)env * NK;
    const int J = (NK + NT - 1) / NT;  // <= 64 because NK <= kCrossF32MaxKeys and NT >= 64
    const int key0 = wave * J * 64 + lane;
    uint64_t bits = 0;
    int mine = 0;
    for (int j = 0; j < J; ++j) {
        const int key = key0 + j * 64;
        bool on = key < NK;
        if (on && mask_env != nullptr) on = mask_env[key] != 0;
        bits |= (on ? 1ull : 0ull) << j;
        mine += (int)__popcll(__ballot(on));
    }
    if (lane == 0) s_wcnt[wave] = mine;
    __syncthreads();
    int base = 0, cnt = 0;
    for (int w = 0; w < nwaves; ++w) {
        const int c = s_wcnt[w];
        if (w < wave) base += c;
        cnt += c;
    }
    for (int j = 0; j < J; ++j) {
        const bool a = (bits >> j) & 1ull;
        const uint64_t mask = __ballot(a);
        if (a) s_idx[base + (int)__popcll(mask & ((1ull << lane) - 1ull))] = (uint16_t)(key0 + j * 64);
        base += (int)__popcll(mask);
    }
    __syncthreads();

    float qf[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) qf[4 * i + 0] = qv[i].x, qf[4 * i + 1] = qv[i].y, qf[4 * i + 2] = qv[i].z, qf[4 * i + 3] = qv[i].w;

    const float *k_env = k + (int64_t)env * NK * kv_stride + head * kCDh;
    const float *v_env = v + (int64_t)env * NK * kv_stride + head * kCDh;
    float run_max = -INFINITY, sum = 0.0f;
    f32x16 o = {0.0f};
    const int ntiles = (cnt + TK - 1) / TK;
    for (int t = 0; t < ntiles; ++t) {
        if (t) __syncthreads();  // every wave is done with the previous tile
        // ---- stage the tile: thread -> (position, 8 channels) ----
        const int left = cnt - t * TK;                    // active keys from this tile on
        const int nb = ((left < TK ? left : TK) + 31) >> 5;  // key blocks of this tile
        for (int item = tid; item < nb * 32 * 4; item += NT) {
            const int pos = item >> 2;
            const int c8 = (item & 3) * 8;
            f32x4 k0 = {0.0f, 0.0f, 0.0f, 0.0f}, k1 = k0, v0 = k0, v1 = k0;
            if (pos < left) {
                const int64_t off = (int64_t)s_idx[t * TK + pos] * kv_stride + c8;
                k0 = *reinterpret_cast<const f32x4 *>(k_env + off);
                k1 = *reinterpret_cast<const f32x4 *>(k_env + off + 4);
                v0 = *reinterpret_cast<const f32x4 *>(v_env + off);
                v1 = *reinterpret_cast<const f32x4 *>(v_env + off + 4);
            }
            float *kd = s_k + pos * kCKeyPitch + c8;
            kd[0] = k0.x, kd[1] = k0.y, kd[2] = k0.z, kd[3] = k0.w;
            kd[4] = k1.x, kd[5] = k1.y, kd[6] = k1.z, kd[7] = k1.w;
            *reinterpret_cast<f32x4 *>(s_v + pos * kCDh + c8) = v0;
            *reinterpret_cast<f32x4 *>(s_v + pos * kCDh + c8 + 4) = v1;
        }
        __syncthreads();
        if (wave * 32 >= NQ) continue;  // a wave without queries only helps staging (it still meets the barriers)
        for (int kb = 0; kb < nb; ++kb) {
            f32x16 z = {0.0f};
            const float *kp = s_k + (kb * 32 + m) * kCKeyPitch + 16 * half;
#pragma unroll
            for (int st = 0; st < 16; ++st) z = __builtin_amdgcn_mfma_f32_32x32x2f32(kp[st], qf[st], z, 0, 0, 0);
            const int valid = left - kb * 32;  // positions of this block that hold a key (>= 1)
            if (valid < 32) {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    if (8 * (e >> 2) + 4 * half + (e & 3) >= valid) z[e] = -INFINITY;
            }
            float bmax = z[0];
#pragma unroll
            for (int e = 1; e < 16; ++e) bmax = fmaxf(bmax, z[e]);
            bmax = fmaxf(bmax, __shfl_xor(bmax, 32));
            const float new_max = fmaxf(run_max, bmax);  // finite: position 0 of every block holds a key
            const float alpha = __builtin_amdgcn_exp2f((run_max - new_max) * scale_log2e);
            run_max = new_max;
            const float mc = new_max * scale_log2e;
            sum *= alpha;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                o[e] *= alpha;
                z[e] = __builtin_amdgcn_exp2f(fmaf(z[e], scale_log2e, -mc));
                sum += z[e];
            }
            const float *vp = s_v + (kb * 32 + 4 * half) * kCDh + m;
#pragma unroll
            for (int st = 0; st < 16; ++st)
                o = __builtin_amdgcn_mfma_f32_32x32x2f32(vp[(8 * (st >> 2) + (st & 3)) * kCDh], z[st], o, 0, 0, 0);
        }
    }
    if (wave * 32 >= NQ || qrow >= NQ) return;
    sum += __shfl_xor(sum, 32);
    const float inv = cnt == 0 ? 0.0f : 1.0f / sum;  // nothing active: the read contributes exactly zero
    // the lane holds channels 8a + 4*half + b (a, b = 0..3) of its query: four 16-byte pieces
    const int64_t o_off = ((int64_t)env * NQ + qrow) * D + head * kCDh + 4 * half;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        f32x4 r = {o[4 * a + 0] * inv, o[4 * a + 1] * inv, o[4 * a + 2] * inv, o[4 * a + 3] * inv};
        if (accum != nullptr) {
            const f32x4 acc = *reinterpret_cast<const f32x4 *>(accum + o_off + 8 * a);
            r = f32x4{acc.x + r.x, acc.y + r.y, acc.z + r.z, acc.w + r.w};
        }
        *reinterpret_cast<f32x4 *>(out + o_off + 8 * a) = r;
    }
}

int launch_cross_f32(const void *q, int64_t q_stride, const void *k, const void *v, int64_t kv_stride, const uint8_t *key_mask,
                     const void *accum, void *out, int B, int NQ, int NK, int H, hipStream_t stream)
{
    if (NK > kCrossF32MaxKeys || NQ > 512) return BNB_ERR_UNSUPPORTED;
    const int nwaves = (NQ + 31) / 32;
    const size_t lds = (size_t)nwaves * 32 * (kCKeyPitch + kCDh) * sizeof(float) + (size_t)kCrossF32MaxKeys * sizeof(uint16_t) +
                       (size_t)nwaves * sizeof(int);
    if (lds > 160 * 1024) return BNB_ERR_UNSUPPORTED;
    if (lds > 64 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(sdpa_cross_f32_kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return (int)e;
    }
    const int64_t pairs = (int64_t)B * H;
    const int64_t blocks = (pairs + 7) / 8 * 8;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(sdpa_cross_f32_kernel, dim3((unsigned)blocks), dim3(nwaves * kWave), lds, stream, (const float *)q,
                       q_stride, (const float *)k, (const float *)v, kv_stride, key_mask, (const float *)accum, (float *)out, B,
                       NQ, NK, H, kLog2eC / sqrtf((float)kCDh));
    return (int)hipGetLastError();
}

}  // namespace bnb
