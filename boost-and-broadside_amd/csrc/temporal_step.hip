// One timestep of the temporal sublayer's state path as a single kernel, for gfx950:
// causal conv taps + buffer shift, the two RG-LRU gate projections, and the recurrence.
//
// Per ship row (reference: models/yemong/griffin.py:275-277 with the taps of :127-139 at T = 1,
// then :179-185 with the projections of :166-167), under bfloat16 autocast:
//   v        = p0 w[:,0] + p1 w[:,1] + p2 w[:,2] + b1 w[:,3] + beta        fp32
//   buffer'  = [p1, p2, b1]
//   [ga|gx]  = bf16( bf16(v) [Wa|Wx]^T + bf16([ba|bx]) )                   matrix cores, fp32 accumulate
//   h'       = RG-LRU(x = v, ga, gx, h)                                     fp32, y = bf16(h')
// As three kernels (conv, library GEMM, recurrence) the row costs 7168 bytes of HBM traffic:
// v goes out in fp32 and bf16 and comes back twice, the gate pre-activations go out and come
// back.  Here v and the gates never leave the CU: 4608 bytes per row (b1 in; p0..p2 and h in;
// the shifted buffer and h' out; y out), which is what bounds the kernel.
//
// Layout of the work.  A work-group keeps the packed gate weights (64 KB) in LDS for its whole
// life and its 8 waves walk over tiles of 32 rows independently (no work-group barrier inside
// the loop).  A wave alternates between two thread-to-data mappings and exchanges only the small
// operands through its private 8.5 KB LDS tile:
//   * row mapping (global memory side): 8 lanes cover 64 consecutive channels of a row, each lane
//     two runs of four channels 32 apart, so that every 16-byte (fp32) or 8-byte (bf16) access
//     instruction covers dense 128-byte / 64-byte runs, 8 rows per instruction; conv, buffer
//     shift and the recurrence run here, v stays in registers between them;
//   * matrix-core mapping: G^T = W v^T per 32 gate features x 32 rows, v^T read from the LDS
//     tile as the B operand, W as the A operand straight from the packed stream; the result
//     (bias added, rounded to bf16 like the library GEMM's output) goes back through the same
//     LDS tile, 64 channels of both gates at a time, to the row mapping.

#include "common.h"
#include "rglru_math.h"

namespace bnb {

constexpr int kTsD = 128;
constexpr int kTsMaxWaves = 8;                    // waves of a work-group; fewer when there are few rows
constexpr int kTsRows = 32;                       // rows of one wave's tile
constexpr int kTsPitch = kTsD + 8;                // halfs per row of a wave's LDS tile: 272 bytes
constexpr int kTsWeightHalfs = 2 * kTsD * kTsD;   // [Wa | Wx] in bf16: 64 KB
constexpr int kTsTileHalfs = kTsRows * kTsPitch;
constexpr int kTsTableFloats = kTsD * 4 + kTsD + 2 * kTsD + kTsD;  // conv taps, conv bias, gate bias, log2 sigmoid(lambda)

static size_t ts_lds_bytes(int waves)
{
    return (size_t)kTsWeightHalfs * 2 + (size_t)kTsTableFloats * sizeof(float) + (size_t)waves * kTsTileHalfs * 2;
}

__global__ __launch_bounds__(kTsMaxWaves * kWave) __attribute__((amdgpu_waves_per_eu(2, 2))) void temporal_step_kernel(
    const uint16_t *__restrict__ b1, int64_t b1_group_stride, int64_t b1_row_stride, const float *conv_in,
    int64_t conv_in_stride, float *conv_out, int64_t conv_out_stride, const float *h_in, int64_t h_in_stride,
    float *h_out, int64_t h_out_stride, const float *__restrict__ conv_weight, const float *__restrict__ conv_bias,
    const uint16_t *__restrict__ gate_weight_packed, const float *__restrict__ gate_bias,
    const float *__restrict__ log_lambda, float c, uint16_t *__restrict__ y, int64_t y_group_stride,
    int64_t y_row_stride, const uint8_t *__restrict__ reset, int rows_per_env, int64_t R, int64_t full_rounds, int tail_rows_per_wave)
{
    extern __shared__ __align__(16) unsigned char s_raw[];
    uint16_t *s_w = reinterpret_cast<uint16_t *>(s_raw);
    float *s_conv_w = reinterpret_cast<float *>(s_w + kTsWeightHalfs);  // [d][k], as stored
    float *s_conv_b = s_conv_w + kTsD * 4;
    float *s_gate_b = s_conv_b + kTsD;  // [ba | bx], rounded to bf16 as autocast hands them to the GEMM
    float *s_l2sig = s_gate_b + 2 * kTsD;
    uint16_t *s_tiles = reinterpret_cast<uint16_t *>(s_l2sig + kTsD);

    const int tid = threadIdx.x;
    const int threads = blockDim.x;
    for (int i = tid; i < kTsWeightHalfs / 8; i += threads)
        reinterpret_cast<u32x4 *>(s_w)[i] = reinterpret_cast<const u32x4 *>(gate_weight_packed)[i];
    for (int i = tid; i < kTsD * 4; i += threads) s_conv_w[i] = conv_weight[i];
    for (int i = tid; i < kTsD; i += threads) s_conv_b[i] = conv_bias != nullptr ? conv_bias[i] : 0.0f;
    for (int i = tid; i < 2 * kTsD; i += threads) s_gate_b[i] = round_to_bf16(gate_bias[i]);
    for (int i = tid; i < kTsD; i += threads) s_l2sig[i] = log2_sigmoid(log_lambda[i]);
    __syncthreads();

    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint16_t *tile = s_tiles + wave * kTsTileHalfs;
    // row mapping
    const int sub = lane >> 3;       // row inside a pass of 8 rows
    // The lane's 8 channels inside a half of 64 are two runs of four, c4 .. c4+3 and 32+c4 .. 32+c4+3, so that the
    // eight lanes of a row cover 128 contiguous bytes of fp32 with EACH 16-byte access (64 bytes of bf16 with each
    // 8-byte access): a 16-byte access whose lanes sit 32 bytes apart streams a third slower on this memory system.
    const int c4 = (lane & 7) * 4;
    auto ch = [&](int e) { return c4 + (e & 3) + 32 * (e >> 2); };  // channel of element e inside the half
    auto ld8 = [&](auto *half_base) -> Row8 {
        const Row4 a = load4<false>(half_base + c4), b = load4<false>(half_base + c4 + 32);
        return Row8{{a.v[0], a.v[1], a.v[2], a.v[3], b.v[0], b.v[1], b.v[2], b.v[3]}};
    };
    auto st8 = [&](auto *half_base, const Row8 &r) {
        store4<false>(half_base + c4, Row4{{r.v[0], r.v[1], r.v[2], r.v[3]}});
        store4<false>(half_base + c4 + 32, Row4{{r.v[4], r.v[5], r.v[6], r.v[7]}});
    };
    // matrix-core mapping
    const int m = lane & 31;
    const int half = lane >> 5;

    float l2s[2][8];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int e = 0; e < 8; ++e) l2s[hf][e] = s_l2sig[64 * hf + ch(e)];

    // Rounds of whole tiles are dealt to the waves of the grid in turn (at any time the grid works
    // on one compact window of rows); what is left after the last whole round is split evenly
    // between all waves in pieces of 8, 16 or 24 rows, so no wave has a whole tile more to do
    // than another and a small input still spreads over the chip.
    const int64_t grid_waves = (int64_t)gridDim.x * (threads >> 6);
    const int64_t wave_global = (int64_t)blockIdx.x * (threads >> 6) + wave;
    for (int64_t round = 0; round <= full_rounds; ++round) {
        int64_t t0, t_end;
        if (round < full_rounds) {
            t0 = (round * grid_waves + wave_global) * kTsRows;
            t_end = t0 + kTsRows;
        } else {
            t0 = full_rounds * grid_waves * kTsRows + wave_global * tail_rows_per_wave;
            t_end = t0 + tail_rows_per_wave < R ? t0 + tail_rows_per_wave : R;
            if (t0 >= t_end) break;
        }
        const int tile_rows = (int)(t_end - t0);  // wave-uniform
        // ---- the lane's four rows (rows past the end repeat the last row and store nothing) ----
        int64_t row[4], env[4];
        bool valid[4], zero[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int64_t r = t0 + 8 * p + sub;
            valid[p] = r < t_end;
            row[p] = valid[p] ? r : t_end - 1;
            env[p] = (int64_t)((uint32_t)row[p] / (uint32_t)rows_per_env);  // R < 2^31, checked by the launcher
            zero[p] = reset != nullptr && reset[env[p]] != 0;
        }

        // ---- conv taps, buffer shift; bf16(v) into the LDS tile ----
        float v[2][4][8];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int d0 = 64 * hf;  // first channel of the half
            float w[8][4], beta[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const f32x4 q = *reinterpret_cast<const f32x4 *>(s_conv_w + (d0 + ch(e)) * 4);
                w[e][0] = q.x, w[e][1] = q.y, w[e][2] = q.z, w[e][3] = q.w;
                beta[e] = s_conv_b[d0 + ch(e)];
            }
            // two rows at a time: all loads of the pair, then arithmetic and stores
#pragma unroll
            for (int pg = 0; pg < 2; ++pg) {
                if (16 * pg >= tile_rows) break;  // short tile: nothing in this pair of passes
                Row8 p0[2], p1[2], p2[2], cur[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int p = 2 * pg + i;
                    const int64_t b1_off = b1_group_stride != 0
                                               ? env[p] * b1_group_stride + (row[p] - env[p] * rows_per_env) * b1_row_stride
                                               : row[p] * b1_row_stride;
                    cur[i] = ld8(b1 + b1_off + d0);
                    const float *pin = conv_in + row[p] * conv_in_stride + d0;
                    p0[i] = ld8(pin);
                    p1[i] = ld8(pin + kTsD);
                    p2[i] = ld8(pin + 2 * kTsD);
                }
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int p = 2 * pg + i;
                    if (zero[p]) {
                        // the environment was reset before this step: its stored inputs read as zero
#pragma unroll
                        for (int e = 0; e < 8; ++e) p0[i].v[e] = p1[i].v[e] = p2[i].v[e] = 0.0f;
                    }
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        float acc = p0[i].v[e] * w[e][0];
                        acc += p1[i].v[e] * w[e][1];
                        acc += p2[i].v[e] * w[e][2];
                        acc += cur[i].v[e] * w[e][3];
                        v[hf][p][e] = acc + beta[e];
                    }
                    if (valid[p]) {
                        float *pout = conv_out + row[p] * conv_out_stride + d0;
                        st8(pout, p1[i]);
                        st8(pout + kTsD, p2[i]);
                        st8(pout + 2 * kTsD, cur[i]);
                    }
                    const float *vv = v[hf][p];
                    uint16_t *tp = tile + (8 * p + sub) * kTsPitch + d0 + c4;
                    *reinterpret_cast<u32x2 *>(tp) = u32x2{pack_bf16x2(vv[0], vv[1]), pack_bf16x2(vv[2], vv[3])};
                    *reinterpret_cast<u32x2 *>(tp + 32) = u32x2{pack_bf16x2(vv[4], vv[5]), pack_bf16x2(vv[6], vv[7])};
                }
            }
        }
        wave_lds_handover();

        // ---- v^T as the B operand of all 8 k-steps: lane = row m, k-slots 8*half .. +7 ----
        bf16x8 vb[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
            vb[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(tile + m * kTsPitch + 16 * ks + 8 * half));
        wave_lds_handover();

#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int d0 = 64 * hf;
            // previous state of this half's channels: in flight while the matrix cores work
            Row8 hv[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) hv[p] = ld8(h_in + row[p] * h_in_stride + d0);

            // ---- gate pre-activations of channels 64*hf .. +63: blocks q = 0,1 of Wa, 2,3 of Wx ----
            // A lane ends up with 16 consecutive channels per block: 32*(q%2) + 16*half + 0..15.
            // Two blocks at a time (one gate): two independent accumulator chains keep the matrix
            // cores issuing back to back without holding all four results in registers.
#pragma unroll
            for (int gate = 0; gate < 2; ++gate) {
                f32x16 acc[2];
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const float *bp = s_gate_b + gate * kTsD + 64 * hf + 32 * j + 16 * half;
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x4 b4 = *reinterpret_cast<const f32x4 *>(bp + 4 * g);
                        acc[j][4 * g + 0] = b4.x, acc[j][4 * g + 1] = b4.y, acc[j][4 * g + 2] = b4.z, acc[j][4 * g + 3] = b4.w;
                    }
                }
#pragma unroll
                for (int ks = 0; ks < 8; ++ks) {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const int q = 2 * gate + j;
                        const u32x4 a = *reinterpret_cast<const u32x4 *>(s_w + ((((hf * 4 + q) * 8 + ks) * 64 + lane) * 8));
                        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), vb[ks], acc[j], 0, 0, 0);
                    }
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    uint16_t *gp = tile + m * kTsPitch + 64 * gate + 32 * j + 16 * half;
#pragma unroll
                    for (int g = 0; g < 2; ++g)
                        *reinterpret_cast<u32x4 *>(gp + 8 * g) =
                            u32x4{pack_bf16x2(acc[j][8 * g + 0], acc[j][8 * g + 1]), pack_bf16x2(acc[j][8 * g + 2], acc[j][8 * g + 3]),
                                  pack_bf16x2(acc[j][8 * g + 4], acc[j][8 * g + 5]), pack_bf16x2(acc[j][8 * g + 6], acc[j][8 * g + 7])};
                }
            }
            wave_lds_handover();

            // ---- recurrence on the row mapping ----
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                if (8 * p >= tile_rows) break;
                const uint16_t *gp = tile + (8 * p + sub) * kTsPitch;
                const Row8 ga = ld8(gp);
                const Row8 gx = ld8(gp + 64);
                Row8 out;
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    out.v[e] = rglru_element<true, false>(v[hf][p][e], ga.v[e], gx.v[e], l2s[hf][e], c,
                                                          zero[p] ? 0.0f : hv[p].v[e]);
                if (valid[p]) {
                    st8(h_out + row[p] * h_out_stride + d0, out);
                    const int64_t y_off = y_group_stride != 0
                                              ? env[p] * y_group_stride + (row[p] - env[p] * rows_per_env) * y_row_stride
                                              : row[p] * y_row_stride;
                    st8(y + y_off + d0, out);
                }
            }
            wave_lds_handover();
        }
    }
}

static int ts_cu_count()
{
    // compute units of the current device, looked up once per device
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

}  // namespace bnb

extern "C" int bnb_temporal_step_fwd(const void *b1, int64_t b1_group_stride, int64_t b1_row_stride,
                                     const float *conv_in, int64_t conv_in_row_stride, float *conv_out,
                                     int64_t conv_out_row_stride, const float *h_in, int64_t h_in_row_stride,
                                     float *h_out, int64_t h_out_row_stride, const float *conv_weight,
                                     const float *conv_bias, const void *gate_weight_packed, const float *gate_bias,
                                     const float *log_lambda, float c, void *y, int64_t y_group_stride,
                                     int64_t y_row_stride, const uint8_t *reset, int rows_per_env, int64_t R, int D, void *stream)
{
    using namespace bnb;
    if (R < 0 || rows_per_env < 1) return BNB_ERR_BAD_SHAPE;
    if (D != kTsD) return BNB_ERR_UNSUPPORTED;
    if (R == 0) return 0;
    if (R > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    if (!b1 || !conv_in || !conv_out || !h_in || !h_out || !conv_weight || !gate_weight_packed || !gate_bias ||
        !log_lambda || !y)
        return BNB_ERR_NULL_POINTER;
    if (y_row_stride == 0) y_row_stride = D;
    if (y_row_stride < D) return BNB_ERR_BAD_SHAPE;
    if (conv_in_row_stride < 3 * D || conv_out_row_stride < 3 * D || h_in_row_stride < D || h_out_row_stride < D ||
        b1_row_stride < D)
        return BNB_ERR_BAD_SHAPE;
    if ((b1_group_stride != 0 || y_group_stride != 0 || reset != nullptr) && R % rows_per_env != 0)
        return BNB_ERR_BAD_SHAPE;
    if (!aligned16(b1) || !aligned16(conv_in) || !aligned16(conv_out) || !aligned16(h_in) || !aligned16(h_out) ||
        !aligned16(y) || !aligned16(conv_weight) || !aligned16(gate_weight_packed) || (b1_row_stride % 8) != 0 ||
        (b1_group_stride % 8) != 0 || (y_group_stride % 8) != 0 || (y_row_stride % 8) != 0 || (conv_in_row_stride % 4) != 0 ||
        (conv_out_row_stride % 4) != 0 || (h_in_row_stride % 4) != 0 || (h_out_row_stride % 4) != 0)
        return BNB_ERR_MISALIGNED;
    // One work-group per CU at most (LDS), 8 waves each, every wave at least 8 rows.
    const int cus = ts_cu_count();
    const int waves = kTsMaxWaves;
    int64_t blocks = (R + (int64_t)waves * 8 - 1) / ((int64_t)waves * 8);
    if (blocks > cus) blocks = cus;
    const int64_t grid_waves = blocks * waves;
    const int64_t full_rounds = R / (grid_waves * kTsRows);
    const int64_t tail = R - full_rounds * grid_waves * kTsRows;
    const int tail_rows_per_wave = (int)(((tail + grid_waves - 1) / grid_waves + 7) / 8 * 8);
    const size_t lds = ts_lds_bytes(waves);
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(temporal_step_kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)ts_lds_bytes(kTsMaxWaves));
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(temporal_step_kernel, dim3((unsigned)blocks), dim3(waves * kWave), lds, (hipStream_t)stream,
                       (const uint16_t *)b1, b1_group_stride, b1_row_stride, conv_in, conv_in_row_stride, conv_out,
                       conv_out_row_stride, h_in, h_in_row_stride, h_out, h_out_row_stride, conv_weight, conv_bias,
                       (const uint16_t *)gate_weight_packed, gate_bias, log_lambda, c, (uint16_t *)y, y_group_stride,
                       y_row_stride, reset, rows_per_env, R, full_rounds, tail_rows_per_wave);
    return (int)hipGetLastError();
}
