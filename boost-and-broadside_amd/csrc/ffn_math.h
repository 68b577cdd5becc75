// Scalar pieces shared by the gated-MLP kernels (forward tail and its backward).
#pragma once

#include "common.h"

namespace bnb {

constexpr int kFfnD = 128;
constexpr int kFfnHidden = 512;
constexpr int kFfnChunks = kFfnHidden / 32;

// The normal distribution function as Phi(v) ~ 1 / (1 + 2^(-v p(v^2))), p a quadratic fitted (minimax
// over |v| <= 9): |error of v * Phi(v)| <= 2.6e-5, two orders of magnitude below the bf16 rounding of
// the product that follows.  v^2 is clamped at 64, beyond which the quadratic would turn over (there
// Phi is 0 or 1 to 1e-15 anyway).
__device__ __forceinline__ float normal_cdf_fit(float v)
{
    const float v2 = fminf(v * v, 64.0f);
    const float p = fmaf(fmaf(v2, -0.0010142630628405414f, 0.10677572405393032f), v2, 2.3011213393619663f);
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-(p * v)));
}

// erf-GELU as v * Phi(v): eight vector-ALU instructions per element, two of them transcendental; the
// three-term Abramowitz-Stegun erfc form used before had the same error at eleven.
__device__ __forceinline__ float gelu_phi(float v) { return v * normal_cdf_fit(v); }

// The normal density exp(-v^2 / 2) / sqrt(2 pi): gelu'(v) = Phi(v) + v * pdf(v).
__device__ __forceinline__ float normal_pdf(float v)
{
    return 0.3989422804014327f * __builtin_amdgcn_exp2f(v * v * -0.7213475204444817f);
}

}  // namespace bnb
