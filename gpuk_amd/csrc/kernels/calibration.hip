// Calibration kernels.
//
// 1. A plain streaming copy of a known number of bytes.  Its achieved GB/s is the
// practical HBM ceiling of the machine, and its FETCH_SIZE / WRITE_SIZE counter readings give the factor
// by which to scale those counters for the fused kernels.  Same purpose as the reference's
// test/cpp/global_memory_bandwidth.cpp:95-114 (1 GB vectorised copy).
//
// 2. data[i] += 1 over a small array: the cost of launching and draining a kernel that does next to nothing,
// which is the floor under every decode-sized call.  Same purpose as the reference's
// test/cpp/test_small_kernel.cpp:85-126 (increment kernel, many launches inside one captured graph).
#include <hip/hip_runtime.h>

#include "../../../include/gpuk_amd.h"
#include "host_utils.h"

namespace gpuk {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Each workgroup copies a contiguous 16 KiB tile: 256 lanes x 4 x 16 bytes, all four loads issued first.
__global__ void __launch_bounds__(256) copy_tiles(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, int64_t n16) {
    const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
    u32x4 v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (base + i * 256 < n16) v[i] = __builtin_nontemporal_load(src + base + i * 256);
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (base + i * 256 < n16) __builtin_nontemporal_store(v[i], dst + base + i * 256);
}

typedef float f32x4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(256) increment_floats(float *data, int64_t n) {
    const int64_t first = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (first + 4 <= n) {
        f32x4 v = *reinterpret_cast<f32x4 *>(data + first);
        v += 1.0f;
        *reinterpret_cast<f32x4 *>(data + first) = v;
    } else {
        for (int64_t i = first; i < n; ++i) data[i] += 1.0f;
    }
}

}  // namespace
}  // namespace gpuk

extern "C" int gpuk_increment_floats(float *data, int64_t n, void *stream) {
    using namespace gpuk;
    if (n < 0) return GPUK_ERR_INVALID_ARG;
    if (n == 0) return GPUK_OK;
    if (!data) return GPUK_ERR_INVALID_ARG;
    if (!aligned16(data)) return GPUK_ERR_MISALIGNED;
    const int64_t blocks = (n + 1023) / 1024;
    if (blocks > 0x7fffffffLL) return GPUK_ERR_UNSUPPORTED;
    increment_floats<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(data, n);
    return hip_status(hipGetLastError());
}

extern "C" int gpuk_copy_bytes(void *dst, const void *src, int64_t nbytes, void *stream) {
    using namespace gpuk;
    if (nbytes < 0 || (nbytes & 15)) return GPUK_ERR_INVALID_ARG;
    if (nbytes == 0) return GPUK_OK;
    if (!dst || !src) return GPUK_ERR_INVALID_ARG;
    if (!aligned16(dst) || !aligned16(src)) return GPUK_ERR_MISALIGNED;
    const int64_t n16 = nbytes / 16;
    const int64_t blocks = (n16 + 1023) / 1024;
    if (blocks > 0x7fffffffLL) return GPUK_ERR_UNSUPPORTED;
    copy_tiles<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const u32x4 *>(src), static_cast<u32x4 *>(dst), n16);
    return hip_status(hipGetLastError());
}
