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
//
// 3. The two halves of the copy on their own: a kernel that only reads and one that only writes, same tiles and
// streaming accesses.  A kernel that reads R bytes and writes W bytes is priced against R / (read-only rate) +
// W / (write-only rate): the memory system serves one direction at a time.
//
// 4. A grid of workgroups that return at once: what launching, placing and draining a grid of a given shape costs
// before any byte moves -- the part of a short kernel's duration that its memory traffic does not explain.
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

// The reading half of copy_tiles.  The loaded values are folded and stored only if the fold hits a value that random
// data never produces in practice, so the loads stay and (almost) nothing is written.
__global__ void __launch_bounds__(256) read_tiles(const u32x4 *__restrict__ src, uint32_t *__restrict__ sink, int64_t n16) {
    const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
    u32x4 v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = base + i * 256 < n16 ? __builtin_nontemporal_load(src + base + i * 256) : u32x4{0, 0, 0, 0};
    const u32x4 f = v[0] ^ v[1] ^ v[2] ^ v[3];
    if ((f[0] ^ f[1]) == 0x9e3779b9u && (f[2] ^ f[3]) == 0x7f4a7c15u) sink[0] = f[0];
}

// The writing half: every lane stores a value that depends on its place, 16 KiB per workgroup.
__global__ void __launch_bounds__(256) fill_tiles(u32x4 *__restrict__ dst, int64_t n16, uint32_t seed) {
    const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
    const uint32_t w = seed + (uint32_t)base;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (base + i * 256 < n16) __builtin_nontemporal_store(u32x4{w, w + i, w ^ seed, seed}, dst + base + i * 256);
}

// A grid whose workgroups do nothing.  `lds` is touched so that the dynamic allocation is real.
__global__ void __launch_bounds__(1024) empty_grid(uint32_t *never_written, int never) {
    extern __shared__ uint32_t lds[];
    if (never) never_written[threadIdx.x] = lds[threadIdx.x];
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

extern "C" int gpuk_read_bytes(const void *src, int64_t nbytes, void *sink, void *stream) {
    using namespace gpuk;
    if (nbytes < 0 || (nbytes & 15)) return GPUK_ERR_INVALID_ARG;
    if (nbytes == 0) return GPUK_OK;
    if (!src || !sink) return GPUK_ERR_INVALID_ARG;
    if (!aligned16(src) || (reinterpret_cast<uintptr_t>(sink) & 3u)) return GPUK_ERR_MISALIGNED;
    const int64_t n16 = nbytes / 16;
    const int64_t blocks = (n16 + 1023) / 1024;
    if (blocks > 0x7fffffffLL) return GPUK_ERR_UNSUPPORTED;
    read_tiles<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const u32x4 *>(src), static_cast<uint32_t *>(sink), n16);
    return hip_status(hipGetLastError());
}

extern "C" int gpuk_fill_bytes(void *dst, int64_t nbytes, uint32_t seed, void *stream) {
    using namespace gpuk;
    if (nbytes < 0 || (nbytes & 15)) return GPUK_ERR_INVALID_ARG;
    if (nbytes == 0) return GPUK_OK;
    if (!dst) return GPUK_ERR_INVALID_ARG;
    if (!aligned16(dst)) return GPUK_ERR_MISALIGNED;
    const int64_t n16 = nbytes / 16;
    const int64_t blocks = (n16 + 1023) / 1024;
    if (blocks > 0x7fffffffLL) return GPUK_ERR_UNSUPPORTED;
    fill_tiles<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<u32x4 *>(dst), n16, seed);
    return hip_status(hipGetLastError());
}

extern "C" int gpuk_empty_grid(int64_t workgroups, int lanes_per_workgroup, int lds_bytes, void *stream) {
    using namespace gpuk;
    if (workgroups < 0 || lanes_per_workgroup <= 0 || lanes_per_workgroup > 1024 || lanes_per_workgroup % 64 ||
        lds_bytes < 0 || lds_bytes > 65536)
        return GPUK_ERR_INVALID_ARG;
    if (workgroups == 0) return GPUK_OK;
    if (workgroups > 0x7fffffffLL) return GPUK_ERR_UNSUPPORTED;
    empty_grid<<<(unsigned)workgroups, lanes_per_workgroup, lds_bytes, static_cast<hipStream_t>(stream)>>>(nullptr, 0);
    return hip_status(hipGetLastError());
}
