// Shared device helpers for the gfx950 kernels: raw bf16 handling and vector types.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bnb_amd.h"

namespace bnb {

constexpr int kWave = 64;  // CDNA wavefront width

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// bf16 is carried as raw 16-bit patterns outside the MFMA operands.
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// Round-to-nearest-even fp32 -> bf16, the rounding torch applies when it stores bf16.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float v)
{
    __bf16 b = (__bf16)v;  // v_cvt_pk_bf16_f32 on gfx950
    return (uint32_t)__builtin_bit_cast(uint16_t, b);
}

__device__ __forceinline__ float round_to_bf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// Two fp32 -> one dword of two bf16 (lo in bits 0..15): a single v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}

// Eight consecutive channels of one row, widened to fp32.
struct Row8 {
    float v[8];
};

__device__ __forceinline__ Row8 load8(const float *p)
{
    const f32x4 a = *reinterpret_cast<const f32x4 *>(p);
    const f32x4 b = *reinterpret_cast<const f32x4 *>(p + 4);
    return Row8{{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w}};
}

__device__ __forceinline__ Row8 load8(const uint16_t *p)
{
    const u32x4 w = *reinterpret_cast<const u32x4 *>(p);
    Row8 r;
    r.v[0] = __uint_as_float(w.x << 16);
    r.v[1] = __uint_as_float(w.x & 0xffff0000u);
    r.v[2] = __uint_as_float(w.y << 16);
    r.v[3] = __uint_as_float(w.y & 0xffff0000u);
    r.v[4] = __uint_as_float(w.z << 16);
    r.v[5] = __uint_as_float(w.z & 0xffff0000u);
    r.v[6] = __uint_as_float(w.w << 16);
    r.v[7] = __uint_as_float(w.w & 0xffff0000u);
    return r;
}

__device__ __forceinline__ void store8(float *p, const Row8 &r)
{
    *reinterpret_cast<f32x4 *>(p) = f32x4{r.v[0], r.v[1], r.v[2], r.v[3]};
    *reinterpret_cast<f32x4 *>(p + 4) = f32x4{r.v[4], r.v[5], r.v[6], r.v[7]};
}

__device__ __forceinline__ void store8(uint16_t *p, const Row8 &r)
{
    *reinterpret_cast<u32x4 *>(p) = u32x4{pack_bf16x2(r.v[0], r.v[1]), pack_bf16x2(r.v[2], r.v[3]),
                                          pack_bf16x2(r.v[4], r.v[5]), pack_bf16x2(r.v[6], r.v[7])};
}

// Streaming variants: nontemporal accesses for data that is touched once per launch.
__device__ __forceinline__ Row8 load8_stream(const float *p)
{
    const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p));
    const f32x4 b = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p + 4));
    return Row8{{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w}};
}

__device__ __forceinline__ Row8 load8_stream(const uint16_t *p)
{
    const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    Row8 r;
    r.v[0] = __uint_as_float(w.x << 16);
    r.v[1] = __uint_as_float(w.x & 0xffff0000u);
    r.v[2] = __uint_as_float(w.y << 16);
    r.v[3] = __uint_as_float(w.y & 0xffff0000u);
    r.v[4] = __uint_as_float(w.z << 16);
    r.v[5] = __uint_as_float(w.z & 0xffff0000u);
    r.v[6] = __uint_as_float(w.w << 16);
    r.v[7] = __uint_as_float(w.w & 0xffff0000u);
    return r;
}

__device__ __forceinline__ void store8_stream(float *p, const Row8 &r)
{
    __builtin_nontemporal_store(f32x4{r.v[0], r.v[1], r.v[2], r.v[3]}, reinterpret_cast<f32x4 *>(p));
    __builtin_nontemporal_store(f32x4{r.v[4], r.v[5], r.v[6], r.v[7]}, reinterpret_cast<f32x4 *>(p + 4));
}

__device__ __forceinline__ void store8_stream(uint16_t *p, const Row8 &r)
{
    __builtin_nontemporal_store(u32x4{pack_bf16x2(r.v[0], r.v[1]), pack_bf16x2(r.v[2], r.v[3]),
                                      pack_bf16x2(r.v[4], r.v[5]), pack_bf16x2(r.v[6], r.v[7])},
                                reinterpret_cast<u32x4 *>(p));
}

// Four consecutive channels of one row, widened to fp32 (an 8-byte access in bf16, 16 bytes in fp32).
struct Row4 {
    float v[4];
};

template <bool STREAM>
__device__ __forceinline__ Row4 load4(const float *p)
{
    const f32x4 a = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p)) : *reinterpret_cast<const f32x4 *>(p);
    return Row4{{a.x, a.y, a.z, a.w}};
}

template <bool STREAM>
__device__ __forceinline__ Row4 load4(const uint16_t *p)
{
    const u32x2 w = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p)) : *reinterpret_cast<const u32x2 *>(p);
    return Row4{{__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16),
                 __uint_as_float(w.y & 0xffff0000u)}};
}

template <bool STREAM>
__device__ __forceinline__ void store4(float *p, const Row4 &r)
{
    const f32x4 v = {r.v[0], r.v[1], r.v[2], r.v[3]};
    if (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(p));
    else *reinterpret_cast<f32x4 *>(p) = v;
}

template <bool STREAM>
__device__ __forceinline__ void store4(uint16_t *p, const Row4 &r)
{
    const u32x2 v = {pack_bf16x2(r.v[0], r.v[1]), pack_bf16x2(r.v[2], r.v[3])};
    if (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<u32x2 *>(p));
    else *reinterpret_cast<u32x2 *>(p) = v;
}

// Eight channels of one row as two runs of four, `gap` elements apart (p points at the first run): with
// lane j of a row on channels 4j..4j+3 and gap + 4j..gap + 4j+3, every access instruction of the lanes
// of a row covers one dense run of bytes, which streams markedly faster than eight consecutive
// channels per lane (two 16-byte accesses whose lanes sit 32 bytes apart).
template <bool STREAM, typename T>
__device__ __forceinline__ Row8 load8_split(const T *p, int gap)
{
    const Row4 a = load4<STREAM>(p), b = load4<STREAM>(p + gap);
    return Row8{{a.v[0], a.v[1], a.v[2], a.v[3], b.v[0], b.v[1], b.v[2], b.v[3]}};
}

template <bool STREAM, typename T>
__device__ __forceinline__ void store8_split(T *p, int gap, const Row8 &r)
{
    store4<STREAM>(p, Row4{{r.v[0], r.v[1], r.v[2], r.v[3]}});
    store4<STREAM>(p + gap, Row4{{r.v[4], r.v[5], r.v[6], r.v[7]}});
}

__device__ __forceinline__ float load1(const float *p) { return *p; }
__device__ __forceinline__ float load1(const uint16_t *p) { return bf16_bits_to_f32(*p); }
__device__ __forceinline__ void store1(float *p, float v) { *p = v; }
__device__ __forceinline__ void store1(uint16_t *p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }

template <typename T>
struct is_bf16 {
    static constexpr bool value = false;
};
template <>
struct is_bf16<uint16_t> {
    static constexpr bool value = true;
};

// Exact (erf) GELU, as torch's default F.gelu.
__device__ __forceinline__ float gelu_erf(float v) { return 0.5f * v * (1.0f + erff(v * 0.70710678118654752f)); }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// LDS traffic between lanes of ONE wave: LDS operations of a wave complete in issue order, so
// only the compiler has to be kept from moving accesses across the hand-over point.
__device__ __forceinline__ void wave_lds_handover()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// out[i] (+)= sum over s of partials[s * elems + i], slices added in a fixed order (defined in
// linear_wgrad.hip).  elems must be a multiple of 64; slices == 0 writes zeros (or leaves out alone
// when accumulating).
int launch_sum_slices(const float *partials, float *out, int64_t elems, int slices, int accumulate, hipStream_t stream);

}  // namespace bnb
