// Element-wise RG-LRU update shared by the single-step and the sequence kernels.
#pragma once

#include "common.h"

namespace bnb {

constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float fast_sigmoid(float v)
{
    // 1 / (1 + 2^(-v log2 e)); v_exp_f32 and v_rcp_f32 are 1-ulp approximations
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-kLog2e * v));
}

// log2(sigmoid(lambda)) computed with the precise library routines (once per block).
__device__ __forceinline__ float log2_sigmoid(float lam) { return -log1pf(expf(-lam)) * kLog2e; }

template <bool G_BF16, bool X_BF16>
__device__ __forceinline__ float rglru_element(float x, float ga, float gx, float l2sig, float c, float h)
{
    float r = fast_sigmoid(ga);
    float i = fast_sigmoid(gx);
    float cr = c * r;
    if (G_BF16) {
        // autocast keeps the sigmoid outputs and the python-scalar product c*r in bf16
        r = round_to_bf16(r);
        i = round_to_bf16(i);
        cr = round_to_bf16(c * r);
    }
    const float a = __builtin_amdgcn_exp2f(cr * l2sig);
    const float gate = __builtin_amdgcn_sqrtf(fmaxf((1.0f - a) * (1.0f + a), 1e-6f));
    float ix = i * x;
    if (G_BF16 && X_BF16) ix = round_to_bf16(ix);
    return a * h + gate * ix;
}

}  // namespace bnb
