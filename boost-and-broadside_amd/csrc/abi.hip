// Library identification, error names and the copy yardstick of libbnb_amd.so.

#include "common.h"

namespace bnb {

constexpr int kCopyThreads = 256;

// One 16-byte nontemporal move per lane: the fastest plain copy measured on MI355X
// (deeper per-lane unrolling and grid-stride loops both stream slower).
__global__ __launch_bounds__(kCopyThreads) void copy16_kernel(const u32x4 *__restrict__ src,
                                                              u32x4 *__restrict__ dst, int64_t n16)
{
    const int64_t i = (int64_t)blockIdx.x * kCopyThreads + threadIdx.x;
    if (i < n16) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

}  // namespace bnb

extern "C" int bnb_abi_version(void) { return BNB_ABI_VERSION; }

extern "C" const char *bnb_build_arch(void) { return "gfx950"; }

extern "C" const char *bnb_error_string(int code)
{
    switch (code) {
        case 0: return "success";
        case BNB_ERR_NULL_POINTER: return "a required pointer is NULL";
        case BNB_ERR_BAD_DTYPE: return "dtype is neither BNB_F32 nor BNB_BF16";
        case BNB_ERR_BAD_SHAPE: return "negative size, inconsistent dimensions or a stride smaller than a row";
        case BNB_ERR_UNSUPPORTED: return "shape or path outside what the kernels cover";
        case BNB_ERR_MISALIGNED: return "pointer or stride breaks the required alignment";
        case BNB_ERR_SCRATCH_LIMIT: return "the call needs more workspace than the library's built-in buffer holds";
        default: return hipGetErrorString((hipError_t)code);
    }
}

extern "C" int bnb_copy_bytes(const void *src, void *dst, int64_t bytes, void *stream)
{
    using namespace bnb;
    if (bytes < 0 || (bytes & 15)) return BNB_ERR_BAD_SHAPE;
    if (bytes == 0) return 0;
    if (!src || !dst) return BNB_ERR_NULL_POINTER;
    if (!aligned16(src) || !aligned16(dst)) return BNB_ERR_MISALIGNED;
    const int64_t n16 = bytes >> 4;
    const int64_t blocks = (n16 + kCopyThreads - 1) / kCopyThreads;
    if (blocks > 0x7fffffffLL) return BNB_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(copy16_kernel, dim3((unsigned)blocks), dim3(kCopyThreads), 0, (hipStream_t)stream,
                       (const u32x4 *)src, (u32x4 *)dst, n16);
    return (int)hipGetLastError();
}
