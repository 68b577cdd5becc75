// Issue-rate yardstick of libbnb_amd.so: how one SIMD's instruction issue is shared between the matrix cores and
// the vector ALU.  The gated-MLP and attention kernels of this library are bound by exactly that sum, so the
// benchmark measures it beside them, as it measures a plain copy beside the bandwidth-bound kernels.

#include "common.h"

namespace bnb {

// `iters` rounds of four slots, a slot being one 32x32x16 bf16 matrix product (MFMA true) followed by M independent
// vector instructions: fused multiply-adds, every fifth one an exp2 with TRANS.  The order is pinned, so the
// stream the hardware sees is the one written here.  Nothing is loaded or stored except a never-taken result store.
template <int M, bool MFMA, bool TRANS>
__global__ __launch_bounds__(256) void issue_probe_kernel(float *sink, int iters, float seed)
{
    f32x16 acc[4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[a][v] = seed * (float)(a + v);
    bf16x8 A, B;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        A[e] = (__bf16)(seed + (float)(e + (int)threadIdx.x));
        B[e] = (__bf16)(seed * (float)e);
    }
    float f[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) f[i] = seed + (float)(i + (int)threadIdx.x);
    const float k1 = seed * 1.0001f, k2 = seed * 0.5f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            if (MFMA) acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A, B, acc[a], 0, 0, 0);
#pragma unroll
            for (int j = 0; j < M; ++j) {
                float &x = f[(a * M + j) & 15];
                x = (TRANS && (j % 5) == 4) ? __builtin_amdgcn_exp2f(x) : __builtin_fmaf(x, k1, k2);
            }
            if (MFMA) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (M > 0) __builtin_amdgcn_sched_group_barrier(0x002, M, 0);
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int v = 0; v < 16; ++v) s += acc[a][v];
#pragma unroll
    for (int i = 0; i < 16; ++i) s += f[i];
    if (s == 12345.678f) sink[threadIdx.x] = s;  // keeps the arithmetic alive; never true for the seeds used
}

template <int M>
static int launch_probe(bool mfma, bool trans, float *sink, int iters, int blocks, hipStream_t s)
{
    if (mfma && trans) hipLaunchKernelGGL((issue_probe_kernel<M, true, true>), dim3(blocks), dim3(256), 0, s, sink, iters, 1.0f);
    else if (mfma) hipLaunchKernelGGL((issue_probe_kernel<M, true, false>), dim3(blocks), dim3(256), 0, s, sink, iters, 1.0f);
    else if (trans) hipLaunchKernelGGL((issue_probe_kernel<M, false, true>), dim3(blocks), dim3(256), 0, s, sink, iters, 1.0f);
    else hipLaunchKernelGGL((issue_probe_kernel<M, false, false>), dim3(blocks), dim3(256), 0, s, sink, iters, 1.0f);
    return (int)hipGetLastError();
}

}  // namespace bnb

extern "C" int bnb_issue_probe(int valu_per_mfma, int with_mfma, int with_transcendentals, int waves_per_simd, int iters,
                               float *sink, void *stream)
{
    using namespace bnb;
    if (iters < 0 || waves_per_simd < 1 || waves_per_simd > 2) return BNB_ERR_BAD_SHAPE;
    if (!sink) return BNB_ERR_NULL_POINTER;
    if (!with_mfma && valu_per_mfma == 0) return BNB_ERR_BAD_SHAPE;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        return BNB_ERR_UNSUPPORTED;
    // a work-group of 256 lanes is one wave on each SIMD of a compute unit (128 registers per lane: at most two per unit)
    const int blocks = cus * waves_per_simd;
    hipStream_t s = (hipStream_t)stream;
    const bool mf = with_mfma != 0, tr = with_transcendentals != 0;
    switch (valu_per_mfma) {
        case 0: return launch_probe<0>(mf, tr, sink, iters, blocks, s);
        case 2: return launch_probe<2>(mf, tr, sink, iters, blocks, s);
        case 4: return launch_probe<4>(mf, tr, sink, iters, blocks, s);
        case 8: return launch_probe<8>(mf, tr, sink, iters, blocks, s);
        case 10: return launch_probe<10>(mf, tr, sink, iters, blocks, s);
        case 12: return launch_probe<12>(mf, tr, sink, iters, blocks, s);
        case 16: return launch_probe<16>(mf, tr, sink, iters, blocks, s);
        default: return BNB_ERR_UNSUPPORTED;
    }
}
