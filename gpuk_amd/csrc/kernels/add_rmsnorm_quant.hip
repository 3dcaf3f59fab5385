// residual-add -> RMSNorm -> (optional) FP8 e4m3fn quantisation, one workgroup per token row.
//
// This is the one-GPU share of the reference's all-reduce-fusion epilogue: the residual add at
// src/impl/all_reduce_fusion_impl.h:256-265 followed by epilogue<>() at :202-228 (rms_norm :159-181,
// reduce_abs_max :183-200, convert_to_fp8 :148-157), reached through the allreduce_rms host op
// (src/ops/all_reduce_fusion.cpp:363-396).  There is no all-reduce here.
//
// Numerics follow the reference's torch oracle (gpuk/__init__.py:147-164) op by op, *not* the
// reference kernel (which keeps fp32 until the fp8 cast):
//     res  = rT(x + r)                       rT = round-to-nearest-even into the 16-bit type
//     var  = sum(res^2) / H ; rstd = 1 / sqrt(var + eps)          (correctly rounded sqrt and divide)
//     n1   = rT(res * rstd) ; n2 = rT(gamma * n1)
//     scale = amax|n2| / fp8_max  (1 when the row is all zero, as the reference kernel: :217)
//     code = e4m3fn_rne(clamp(n2 / scale, +-fp8_max))             (fp32 IEEE quotient)
//
// Data movement per element: 2 B x + 2 B residual in, 2 B residual out, 1 B code (7 B); the row lives
// in registers between the three phases, so HBM sees each byte once.  Lane `t` of the workgroup owns
// 16-byte chunk `i*blockDim + t` of the row for i < NCHUNK: every wave load/store instruction covers
// 1 KiB (loads) or 512 B (codes) of contiguous memory.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "../../../include/gpuk_amd.h"
#include "device_utils.h"
#include "host_utils.h"

namespace gpuk {

namespace {

constexpr int kMaxThreads = 1024;
constexpr int kMaxWaves = kMaxThreads / 64;

template <typename V>
__device__ __forceinline__ V load_stream(const V *p) { return __builtin_nontemporal_load(p); }
template <typename V>
__device__ __forceinline__ void store_stream(V *p, V v) { __builtin_nontemporal_store(v, p); }

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// The scale reciprocal is usable by div_by_rcp when scale is comfortably normal.
__device__ __forceinline__ bool scale_in_fast_range(float s) {
    return s >= 0x1p-60f && s <= 0x1p60f;
}

// max(m, |a|, |b|) in one instruction.  Written in assembly: the inputs come out of integer-typed conversions and
// the compiler turns fabs() of such a value into a separate v_and instead of a source modifier.  NaNs are dropped
// (callers track them apart).
__device__ __forceinline__ float max3_abs(float m, float a, float b) {
    float r;
    asm("v_max3_f32 %0, |%1|, |%2|, %3" : "=v"(r) : "v"(a), "v"(b), "v"(m));
    return r;
}

// a / b for finite a and b > 0 comfortably normal, given rcp = RN(1/b): the correctly rounded quotient by one
// multiply and two fused multiply-adds (Markstein), arranged so that a = -0 gives -0: with e = q*b - a the last step
// fma(-e, rcp, q) adds two negative zeros, where the usual fma(a - q*b, rcp, q) adds +0 and -0.
__device__ __forceinline__ float div_by_rcp_finite(float a, float b, float rcp) {
    const float q = a * rcp;
    const float e = __builtin_fmaf(q, b, -a);
    return __builtin_fmaf(-e, rcp, q);
}

// The codes of one chunk by plain IEEE division, for scales so small or large (or not a number) that a reciprocal
// leaves the normal range.  Kept out of line: it is long (eight expanded divisions and clamps), it is almost never
// taken, and inlined it sat between the kernel's last two stretches of common-path code, which a wave then reached
// by a jump into instructions no prefetch had brought in.
typedef float f32x8 __attribute__((ext_vector_type(8)));
__device__ __attribute__((noinline)) u32x2 codes_by_division(f32x8 n, float scale, float fp8_max) {  // by value: in registers
    float q[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = clamp_sym(n[j] / scale, fp8_max);
    return u32x2{cvt4_e4m3fn(q[0], q[1], q[2], q[3]), cvt4_e4m3fn(q[4], q[5], q[6], q[7])};
}

// EXACT: lanes x NCHUNK equals the chunks of a row, so every lane owns NCHUNK live chunks and nothing is masked
// (true for every power-of-two row and for 7168 elements; it removes a sixth of the kernel's instructions, which is
// what a decode-sized batch waits for: with at most one row per compute unit the run time is the row's arithmetic).
template <typename T, int NCHUNK, int QUANT, bool EXACT, bool GATED>
__global__ void __launch_bounds__(kMaxThreads) __attribute__((amdgpu_waves_per_eu(GATED && NCHUNK <= 4 ? 8 : 4)))
add_rmsnorm_quant_rows(const u32x4 *x, const u32x4 *residual_in, int chunks_per_row, int remap_end,
                       uint32_t lanes_and_shift, uint32_t gate, const u32x4 *__restrict__ gamma, u32x4 *residual_out,
                       void *norm_out, float *__restrict__ scale_io, float hidden_f, float rcp_hidden, int hidden_pow2,
                       float eps, float fp8_max, float rcp_fp8_max) {
    // The arguments are ordered by when a wave needs them: the first fourteen dwords (up to norm_out) are handed to
    // the wave in scalar registers at launch (-amdgpu-kernarg-preload-count), so the loads of the row are issued
    // without a round trip for the argument block; lanes_and_shift holds the workgroup size (bits 0-15), passed so
    // that it need not be fetched from the dispatch packet either, and the row-run shift (bits 16-31).
    const int nthreads = (int)(lanes_and_shift & 0xffffu), group_shift = (int)(lanes_and_shift >> 16);
    using P = Pack16<T>;
    __shared__ float s_sum[kReduceSlots];
    __shared__ float s_max[kReduceSlots];
    GPUK_STAMPS_BEGIN();  // profiling build only
    // GATED (batches whose rows are all resident at once): no store before `gate` ticks of 10 ns after the wave's
    // entry, the time the launch's reads take; the chip then reads in the first part of the launch and writes in the
    // second instead of mixing the two, which the memory system charges for.  The residual is stored with the codes.
    // (A template parameter: as a run-time choice the branches around the early stores cost the large batches 1 %.)
    const uint64_t entry = GATED ? __builtin_amdgcn_s_memrealtime() : 0;

    const int tid = threadIdx.x;
    const int num_waves = nthreads >> 6;
    // Workgroup ids are handed to the 8 XCDs round-robin.  Below remap_end the rows are dealt out in runs of
    // 2^group_shift consecutive rows per XCD instead of one row each (which rows run concurrently stays the same;
    // which XCD's L2 and fabric port each row goes through changes).
    int row = blockIdx.x;
    if (row < remap_end) {
        const int xcd = row & 7, idx = row >> 3;
        row = ((((idx >> group_shift) << 3) | xcd) << group_shift) | (idx & ((1 << group_shift) - 1));
    }
    const int64_t row_base = (int64_t)row * chunks_per_row;

    // ---- phase 0: issue every load of the row before touching any of them.  The row is loaded whole before any of
    // it is stored, so residual_out may be the same buffer as residual_in or x.
    u32x4 xv[NCHUNK], rv[NCHUNK], gv[NCHUNK];
    bool live[NCHUNK];
#pragma unroll
    for (int i = 0; i < NCHUNK; ++i) {
        const int c = i * nthreads + tid;
        live[i] = EXACT || c < chunks_per_row;
        if (live[i]) {
            xv[i] = load_stream(x + row_base + c);
            rv[i] = load_stream(residual_in + row_base + c);
        } else {
            xv[i] = u32x4{0, 0, 0, 0};
            rv[i] = u32x4{0, 0, 0, 0};
        }
    }
#pragma unroll
    for (int i = 0; i < NCHUNK; ++i) {
        const int c = i * nthreads + tid;
        gv[i] = live[i] ? gamma[c] : u32x4{0, 0, 0, 0};
    }
    // The arguments beyond the preloaded ones are fetched here, behind the row's loads and while those are in flight:
    // left to itself the compiler fetches them where they are first used, after the first barrier, and every wave of
    // the row then waits there for the scalar cache (0.1-0.15 us of a decode-sized call).
    asm volatile("" ::"s"(hidden_f), "s"(rcp_hidden), "s"(hidden_pow2), "s"(eps), "s"(fp8_max), "s"(rcp_fp8_max));
    // ... and so is the static scale, which the kernel only reads (asked for here, needed in phase 3: fetched where it
    // is first used it put a round trip through the scalar cache between the last two phases)
    float static_scale = 0.f;
    if constexpr (QUANT == GPUK_QUANT_FP8_STATIC) static_scale = *(const __attribute__((address_space(4))) float *)scale_io;
    GPUK_STAMP(1);          // every load issued
    GPUK_STAMP_DRAINED(2);  // ... and landed

    // ---- phase 1: res = rT(x + r), stored once; sum of squares of the *rounded* residual.  Waves in this phase
    // are given issue priority over the arithmetic of phases 2-3 so that their residual stores leave early (+0.4 %).
    __builtin_amdgcn_s_setprio(1);
    float ss0 = 0.f, ss1 = 0.f;
#pragma unroll
    for (int i = 0; i < NCHUNK; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t w = P::pack(P::lo(xv[i][j]) + P::lo(rv[i][j]), P::hi(xv[i][j]) + P::hi(rv[i][j]));
            xv[i][j] = w;  // xv now holds the residual
            if (j & 1) ss1 = P::add_squares(w, ss1);
            else ss0 = P::add_squares(w, ss0);
        }
        if (!GATED && live[i]) store_stream(residual_out + row_base + i * nthreads + tid, xv[i]);
    }
    if constexpr (GATED && NCHUNK == 4) {  // (the packed residual is what stays in registers, not the sums it was rounded from)
#pragma unroll
        for (int i = 0; i < NCHUNK; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(xv[i][j]));
    }
    float sumsq[1] = {ss0 + ss1};
    if constexpr (QUANT == GPUK_QUANT_FP8_STATIC) asm volatile("" ::"s"(static_scale));  // (it has arrived by now)
    GPUK_STAMP(3);  // residual stored, the lane's squares summed
    block_allreduce<SumOp, 1>(sumsq, s_sum, num_waves);
    __builtin_amdgcn_s_setprio(0);
    GPUK_STAMP(4);  // sum of squares of the row known to every wave

    // ---- phase 2: n2 = rT(gamma * rT(res * rstd)); row amax for the dynamic scale.
    // mean = sumsq / H as an exact IEEE quotient: a multiplication when H is a power of two (exact, and rounded like
    // the quotient when the result is subnormal), a division otherwise
    // Elsewhere the quotient by multiply and two fused multiply-adds (exact on the guarded range, see div_by_rcp) and
    // the short square root and reciprocal: every wave of the row walks this dependent chain before it can go on.
    float mean;
    if (hidden_pow2) mean = sumsq[0] * rcp_hidden;
    else if (__builtin_expect(__builtin_amdgcn_ballot_w64(!in_mid_range(sumsq[0])) == 0, 1)) mean = div_by_rcp_finite(sumsq[0], hidden_f, rcp_hidden);
    else mean = sumsq[0] / hidden_f;
    const float rstd = rsqrt_two_roundings(mean + eps);
    GPUK_STAMP(5);  // rstd
    if constexpr (QUANT == GPUK_QUANT_NONE) {
        u32x4 *out = reinterpret_cast<u32x4 *>(norm_out) + row_base;
        u32x4 normed[NCHUNK];
#pragma unroll
        for (int i = 0; i < NCHUNK; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float lo = P::lo(gv[i][j]) * P::round(P::lo(xv[i][j]) * rstd);
                const float hi = P::hi(gv[i][j]) * P::round(P::hi(xv[i][j]) * rstd);
                normed[i][j] = P::pack(lo, hi);
            }
            if (!GATED && live[i]) store_stream(out + i * nthreads + tid, normed[i]);
        }
        if constexpr (GATED) {
            // (the values to store are pinned down ahead of the wait: nothing ties the arithmetic to the clock, and the
            // compiler otherwise moves it behind the wait)
#pragma unroll
            for (int i = 0; i < NCHUNK; ++i) asm volatile("" ::"v"(normed[i]));
            while (__builtin_amdgcn_s_memrealtime() < entry + gate) __builtin_amdgcn_s_sleep(1);
#pragma unroll
            for (int i = 0; i < NCHUNK; ++i)
                if (live[i]) store_stream(residual_out + row_base + i * nthreads + tid, xv[i]);
#pragma unroll
            for (int i = 0; i < NCHUNK; ++i)
                if (live[i]) store_stream(out + i * nthreads + tid, normed[i]);
        }
        GPUK_STAMP(9);
        GPUK_STAMP_DRAINED(10);
        GPUK_STAMPS_WRITE(blockIdx.x * num_waves + (tid >> 6));
        return;
    } else {
        // the normed row stays in fp32 registers, every value already rounded to the 16-bit type.
        // v_max3_f32 drops NaNs where the reference's amax propagates them: they are tracked apart
        // (kPacked, the gated four-chunk form: as 16-bit pairs instead, half the registers, so that eight waves fit a
        // SIMD with the residual kept for the gate as well; unpacked again in phase 3)
        constexpr bool kPacked = GATED && NCHUNK == 4;
        float nv[kPacked ? 1 : NCHUNK][8];
        uint32_t nw[kPacked ? NCHUNK : 1][4];
        float m0 = 0.f, m1 = 0.f;
        bool any_nan = false;
#pragma unroll
        for (int i = 0; i < NCHUNK; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float lo, hi;
                if constexpr (kPacked) {
                    nw[i][j] = P::pack(P::lo(gv[i][j]) * P::round(P::lo(xv[i][j]) * rstd), P::hi(gv[i][j]) * P::round(P::hi(xv[i][j]) * rstd));
                    lo = P::lo(nw[i][j]);
                    hi = P::hi(nw[i][j]);
                } else {
                    lo = P::round(P::lo(gv[i][j]) * P::round(P::lo(xv[i][j]) * rstd));
                    hi = P::round(P::hi(gv[i][j]) * P::round(P::hi(xv[i][j]) * rstd));
                    nv[i][2 * j] = lo;
                    nv[i][2 * j + 1] = hi;
                }
                if constexpr (QUANT == GPUK_QUANT_FP8_DYNAMIC) {
                    if (j & 1) m1 = max3_abs(m1, lo, hi);
                    else m0 = max3_abs(m0, lo, hi);
                    any_nan |= __builtin_isunordered(lo, hi);
                }
            }
        }
        float scale;
        GPUK_STAMP(6);  // row normed, the lane's maximum known
        if constexpr (QUANT == GPUK_QUANT_FP8_DYNAMIC) {
            float amax[1] = {any_nan ? __builtin_nanf("") : __builtin_fmaxf(m0, m1)};
            block_allreduce<MaxOp, 1>(amax, s_max, num_waves);
            GPUK_STAMP(7);  // row maximum known to every wave
            // rcp_fp8_max is RN(1 / fp8_max) for the two maxima the quotient was checked for (448, 240), else 0
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(in_mid_range(amax[0]) && rcp_fp8_max != 0.f)) == 0, 1))
                scale = div_by_rcp_finite(amax[0], fp8_max, rcp_fp8_max);
            else
                scale = amax[0] == 0.f ? 1.f : amax[0] / fp8_max;
            if (tid == 0) scale_io[row] = scale;
        } else {
            scale = static_scale;
        }

        // ---- phase 3: code = e4m3fn(clamp(n2 / scale)), 8 codes per chunk.  With the dynamic scale every value is
        // finite and |n2 / scale| <= 448 * (1 + 2^-23), which the converter already rounds to 448: no clamp, and the
        // short form of the quotient.  The static scale may meet anything: clamp, and the form that restores what a
        // division gives for infinite and NaN numerators.
        constexpr bool kDynamic = QUANT == GPUK_QUANT_FP8_DYNAMIC;
        u32x2 *out = reinterpret_cast<u32x2 *>(norm_out) + row_base;
        if constexpr (kPacked) {  // (or the compiler keeps phase 2's unpacked copies alive instead)
#pragma unroll
            for (int i = 0; i < NCHUNK; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(nw[i][j]));
        }
        // (the scale is the same in every lane; deciding by ballot tells the compiler so, and the common path is
        // laid out as straight-line code with the other one out of the way)
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(!scale_in_fast_range(scale)) == 0, 1)) {
            float rcp;
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(mantissa_all_ones(scale)) == 0, 1)) rcp = rcp_rn_mid_range(scale);
            else rcp = 1.0f / scale;
            GPUK_STAMP(8);  // scale and its reciprocal
            u32x2 codes[NCHUNK];
#pragma unroll
            for (int i = 0; i < NCHUNK; ++i) {
                float q[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    float n;
                    if constexpr (kPacked) n = (j & 1) ? P::hi(nw[i][j >> 1]) : P::lo(nw[i][j >> 1]);
                    else n = nv[i][j];
                    q[j] = kDynamic ? div_by_rcp_finite(n, scale, rcp) : div_by_rcp(n, scale, rcp);
                }
                if constexpr (!kDynamic) clamp8_sym(q, fp8_max);
                codes[i] = u32x2{cvt4_e4m3fn(q[0], q[1], q[2], q[3]), cvt4_e4m3fn(q[4], q[5], q[6], q[7])};
                if (!GATED && live[i]) store_stream(out + i * nthreads + tid, codes[i]);
            }
            if constexpr (GATED) {
#pragma unroll
                for (int i = 0; i < NCHUNK; ++i) asm volatile("" ::"v"(codes[i]));  // computed ahead of the wait, as above
                while (__builtin_amdgcn_s_memrealtime() < entry + gate) __builtin_amdgcn_s_sleep(1);
#pragma unroll
                for (int i = 0; i < NCHUNK; ++i)
                    if (live[i]) store_stream(residual_out + row_base + i * nthreads + tid, xv[i]);
#pragma unroll
                for (int i = 0; i < NCHUNK; ++i)
                    if (live[i]) store_stream(out + i * nthreads + tid, codes[i]);
            }
        } else {
            if constexpr (GATED) {  // (no wait on this path: it is taken by rows whose scale is degenerate)
#pragma unroll
                for (int i = 0; i < NCHUNK; ++i)
                    if (live[i]) store_stream(residual_out + row_base + i * nthreads + tid, xv[i]);
            }
            // (unrolled like the common path: a runtime index into the register arrays would move them to scratch)
#pragma unroll
            for (int i = 0; i < NCHUNK; ++i) {
                f32x8 n;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    if constexpr (kPacked) n[j] = (j & 1) ? P::hi(nw[i][j >> 1]) : P::lo(nw[i][j >> 1]);
                    else n[j] = nv[i][j];
                }
                const u32x2 codes = codes_by_division(n, scale, fp8_max);
                if (live[i]) store_stream(out + i * nthreads + tid, codes);
            }
        }
        GPUK_STAMP(9);           // codes stored (issued)
        GPUK_STAMP_DRAINED(10);  // every store of the wave acknowledged
        GPUK_STAMPS_WRITE(blockIdx.x * num_waves + (tid >> 6));
    }
}

// Calibration: the memory traffic of add_rmsnorm_quant_rows without its arithmetic.  Same launch shape, lane-to-chunk
// mapping, row-to-workgroup mapping, streaming loads and stores and the same two workgroup barriers; the "residual"
// is x ^ r and the "codes" fold it to half its size.  What this kernel reaches is the ceiling of the access pattern.
template <int NCHUNK>
__global__ void __launch_bounds__(kMaxThreads)
add_rmsnorm_quant_traffic_only(const u32x4 *x, const u32x4 *residual_in, int chunks_per_row, int remap_end,
                               uint32_t lanes_and_shift, uint32_t gate, u32x4 *residual_out, u32x2 *codes,
                               float *__restrict__ scale_out) {
    const int nthreads = (int)(lanes_and_shift & 0xffffu), group_shift = (int)(lanes_and_shift >> 16);
    const uint64_t entry = __builtin_amdgcn_s_memrealtime();  // the kernel's store gate, see there
    const int tid = threadIdx.x;  // arguments in the order of add_rmsnorm_quant_rows: the same ones arrive in registers
    int row = blockIdx.x;
    if (row < remap_end) {
        const int xcd = row & 7, idx = row >> 3;
        row = ((((idx >> group_shift) << 3) | xcd) << group_shift) | (idx & ((1 << group_shift) - 1));
    }
    const int64_t row_base = (int64_t)row * chunks_per_row;
    u32x4 xv[NCHUNK], rv[NCHUNK];
    bool live[NCHUNK];
#pragma unroll
    for (int i = 0; i < NCHUNK; ++i) {
        const int c = i * nthreads + tid;
        live[i] = c < chunks_per_row;
        xv[i] = live[i] ? load_stream(x + row_base + c) : u32x4{0, 0, 0, 0};
        rv[i] = live[i] ? load_stream(residual_in + row_base + c) : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < NCHUNK; ++i) {
        xv[i] ^= rv[i];
        if (!gate && live[i]) store_stream(residual_out + row_base + i * nthreads + tid, xv[i]);
    }
    __syncthreads();
    __syncthreads();
    if (gate) {
        while (__builtin_amdgcn_s_memrealtime() < entry + gate) __builtin_amdgcn_s_sleep(1);
#pragma unroll
        for (int i = 0; i < NCHUNK; ++i)
            if (live[i]) store_stream(residual_out + row_base + i * nthreads + tid, xv[i]);
    }
    if (tid == 0) scale_out[row] = 1.0f;
#pragma unroll
    for (int i = 0; i < NCHUNK; ++i) {
        const u32x2 folded = {xv[i][0] + xv[i][1], xv[i][2] + xv[i][3]};
        if (live[i]) store_stream(codes + row_base + i * nthreads + tid, folded);
    }
}

// Rows too long to keep in registers (more than 8 chunks per lane at 1024 lanes, i.e. hidden > 65536):
// three sweeps over the row, re-reading what this same lane wrote to residual_out (L2-resident).
template <typename T, int QUANT>
__global__ void __launch_bounds__(kMaxThreads)
add_rmsnorm_quant_long_rows(const u32x4 *x, const u32x4 *residual_in,  // either may be residual_out: no __restrict__
                            const u32x4 *__restrict__ gamma, u32x4 *residual_out, void *norm_out,
                            float *__restrict__ scale_io, int chunks_per_row, float hidden_f, float eps,
                            float fp8_max) {
    using P = Pack16<T>;
    __shared__ float s_sum[kReduceSlots];
    __shared__ float s_max[kReduceSlots];
    const int tid = threadIdx.x;
    const int num_waves = blockDim.x >> 6;
    const int64_t row_base = (int64_t)blockIdx.x * chunks_per_row;

    float ss = 0.f;
    for (int c = tid; c < chunks_per_row; c += blockDim.x) {
        u32x4 xv = x[row_base + c], rv = residual_in[row_base + c];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t w = P::pack(P::lo(xv[j]) + P::lo(rv[j]), P::hi(xv[j]) + P::hi(rv[j]));
            xv[j] = w;
            ss = __builtin_fmaf(P::lo(w), P::lo(w), ss);
            ss = __builtin_fmaf(P::hi(w), P::hi(w), ss);
        }
        residual_out[row_base + c] = xv;
    }
    float sumsq[1] = {ss};
    block_allreduce<SumOp, 1>(sumsq, s_sum, num_waves);
    const float rstd = 1.0f / sqrtf(sumsq[0] / hidden_f + eps);

    auto normed = [&](int c) {
        u32x4 v = residual_out[row_base + c];  // written by this lane above
        const u32x4 g = gamma[c];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t n1 = P::pack(P::lo(v[j]) * rstd, P::hi(v[j]) * rstd);
            v[j] = P::pack(P::lo(g[j]) * P::lo(n1), P::hi(g[j]) * P::hi(n1));
        }
        return v;
    };

    if constexpr (QUANT == GPUK_QUANT_NONE) {
        u32x4 *out = reinterpret_cast<u32x4 *>(norm_out) + row_base;
        for (int c = tid; c < chunks_per_row; c += blockDim.x) out[c] = normed(c);
    } else {
        float scale;
        if constexpr (QUANT == GPUK_QUANT_FP8_DYNAMIC) {
            float amax = 0.f;
            for (int c = tid; c < chunks_per_row; c += blockDim.x) {
                const u32x4 v = normed(c);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    amax = MaxOp::apply(amax, __builtin_fabsf(P::lo(v[j])));  // keeps a NaN, like the reference's amax
                    amax = MaxOp::apply(amax, __builtin_fabsf(P::hi(v[j])));
                }
            }
            float am[1] = {amax};
            block_allreduce<MaxOp, 1>(am, s_max, num_waves);
            scale = am[0] == 0.f ? 1.f : am[0] / fp8_max;
            if (tid == 0) scale_io[blockIdx.x] = scale;
        } else {
            scale = scale_io[0];
        }
        u32x2 *out = reinterpret_cast<u32x2 *>(norm_out) + row_base;
        for (int c = tid; c < chunks_per_row; c += blockDim.x) {
            const u32x4 v = normed(c);
            float q[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                q[2 * j] = clamp_sym(P::lo(v[j]) / scale, fp8_max);
                q[2 * j + 1] = clamp_sym(P::hi(v[j]) / scale, fp8_max);
            }
            out[c] = u32x2{cvt4_e4m3fn(q[0], q[1], q[2], q[3]), cvt4_e4m3fn(q[4], q[5], q[6], q[7])};
        }
    }
}

// fp32 and fp64 activations: the reference dispatches them through the same template
// (AT_DISPATCH_FLOATING_TYPES_AND2, src/ops/all_reduce_fusion.cpp:375-378).  4 elements per chunk; a lane keeps its
// CPL chunks of the summed row in registers (rows of up to 4 x 1024 chunks), or, with CPL = 0, sweeps a longer row
// three times, reading back what it stored to residual_out.  Rounding to the activation type is the identity here, so
// the oracle's sequence is plain arithmetic in that type around an fp32 variance:
//   res = x + r;  rstd = 1/sqrt(mean(float(res)^2) + eps) in fp32;  n = gamma * (res * F(rstd));
//   scale = max|float(n)| / fp8_max in fp32;  code = e4m3fn(float(clamp(n / F(scale))))
// (for F = double torch promotes tensor * fp32-tensor products to double and casts double -> float -> fp8).
template <typename F>
using wide4 = F __attribute__((ext_vector_type(4)));

template <typename F, int QUANT, int CPL>
__global__ void __launch_bounds__(kMaxThreads)
add_rmsnorm_quant_wide_rows(const wide4<F> *x, const wide4<F> *residual_in,  // either may be residual_out
                            const wide4<F> *__restrict__ gamma, wide4<F> *residual_out, void *norm_out,
                            float *__restrict__ scale_io, int chunks_per_row, float hidden_f, float eps, float fp8_max) {
    __shared__ float s_sum[kReduceSlots];
    __shared__ float s_max[kReduceSlots];
    const int tid = threadIdx.x;
    const int num_waves = blockDim.x >> 6;
    const int64_t row_base = (int64_t)blockIdx.x * chunks_per_row;
    constexpr int KEPT = CPL ? CPL : 1;
    // streaming accesses where the row stays in registers: measured 6-12 % faster for fp32 and 12 % slower for fp64
    constexpr bool STREAM = CPL > 0 && sizeof(F) == 4;
    wide4<F> kept[KEPT];  // CPL > 0: chunk tid + i * blockDim.x of the summed row (and later of the normed row)

    // f(i, c) for every chunk c of the row this lane owns; i is its place in kept[]
    auto for_chunks = [&](auto f) {
        if constexpr (CPL > 0) {
#pragma unroll
            for (int i = 0; i < CPL; ++i) {
                const int c = tid + i * (int)blockDim.x;
                if (c < chunks_per_row) f(i, c);
            }
        } else {
            for (int c = tid; c < chunks_per_row; c += blockDim.x) f(0, c);
        }
    };

    float ss = 0.f;
    for_chunks([&](int i, int c) {
        wide4<F> res;
        if constexpr (STREAM) {
            res = __builtin_nontemporal_load(x + row_base + c) + __builtin_nontemporal_load(residual_in + row_base + c);
            __builtin_nontemporal_store(res, residual_out + row_base + c);
        } else {
            res = x[row_base + c] + residual_in[row_base + c];
            residual_out[row_base + c] = res;  // CPL = 0: read back below
        }
        kept[i] = res;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float r = (float)res[j];
            ss = __builtin_fmaf(r, r, ss);
        }
    });
    float sumsq[1] = {ss};
    block_allreduce<SumOp, 1>(sumsq, s_sum, num_waves);
    const F rstd = (F)(1.0f / sqrtf(sumsq[0] / hidden_f + eps));

    // the normed chunk; with CPL = 0 the summed chunk is read back (this lane wrote it above)
    auto normed = [&](int i, int c) {
        const wide4<F> v = CPL > 0 ? kept[i] : residual_out[row_base + c];
        return gamma[c] * (v * rstd);
    };

    if constexpr (QUANT == GPUK_QUANT_NONE) {
        wide4<F> *out = reinterpret_cast<wide4<F> *>(norm_out) + row_base;
        for_chunks([&](int i, int c) {
            if constexpr (STREAM) __builtin_nontemporal_store(normed(i, c), out + c);
            else out[c] = normed(i, c);
        });
    } else {
        float scale;
        if constexpr (QUANT == GPUK_QUANT_FP8_DYNAMIC) {
            float amax = 0.f;
            for_chunks([&](int i, int c) {
                const wide4<F> v = normed(i, c);
                if constexpr (CPL > 0) kept[i] = v;
#pragma unroll
                for (int j = 0; j < 4; ++j) amax = MaxOp::apply(amax, __builtin_fabsf((float)v[j]));
            });
            float am[1] = {amax};
            block_allreduce<MaxOp, 1>(am, s_max, num_waves);
            scale = am[0] == 0.f ? 1.f : am[0] / fp8_max;
            if (tid == 0) scale_io[blockIdx.x] = scale;
        } else {
            scale = scale_io[0];
        }
        const F wide_scale = (F)scale;
        uint32_t *out = reinterpret_cast<uint32_t *>(norm_out) + row_base;
        for_chunks([&](int i, int c) {
            wide4<F> n;
            if constexpr (CPL > 0 && QUANT == GPUK_QUANT_FP8_DYNAMIC) n = kept[i];
            else n = normed(i, c);
            const wide4<F> q = n / wide_scale;
            // clamping after the cast to fp32 equals the oracle's clamp before it: the bounds are fp32 numbers
            const uint32_t codes = cvt4_e4m3fn(clamp_sym((float)q[0], fp8_max), clamp_sym((float)q[1], fp8_max),
                                               clamp_sym((float)q[2], fp8_max), clamp_sym((float)q[3], fp8_max));
            if constexpr (STREAM) __builtin_nontemporal_store(codes, out + c);
            else out[c] = codes;
        });
    }
}

int g_force_nchunk = 0;   // 0 = heuristic; set through gpuk_set_tuning for sweeps
int g_force_threads = 0;  // 0 = heuristic
int g_row_group_shift = -1;  // -1 = heuristic, else log2 of the run of consecutive rows an XCD takes (0 = one row)
int g_gate = -1;             // store gate in ticks of 10 ns: -1 = built-in rule, 0 = none, > 0 = that many
int g_pieces = 0;            // launches per call: 0 = built-in rule, 1 = always one, 2 = two wherever each half fits one round
constexpr int kComputeUnits = 256;  // MI355X

// Rows resident at once, chip-wide, with `threads` lanes per row and `nchunk` chunks per lane: 2048 lanes per compute
// unit, eight waves per SIMD, which the gated instantiations of up to four chunks per lane are compiled for
// (amdgpu_waves_per_eu: at most 64 registers); with eight chunks per lane, up to 128 registers, half of that.
// Measured exception: of workgroups of 5 or 10 waves a compute unit takes 25 or 20 waves' worth, not 30 (1408 rows of
// 5120 elements, 5.5 per compute unit, run no faster gated than ungated, 1280 run 22 % faster; likewise 640 and 512
// rows of 10240), where 3, 6, 7, 9, 11-16 waves fill it as counted (30, 30, 28, 27, ... waves).
int64_t resident_rows(int threads, int nchunk) {
    const int waves = threads / 64;
    int waves_per_cu = nchunk >= 8 ? 16 : 32;
    if (waves == 5 || waves == 10) waves_per_cu = std::min(waves_per_cu, waves == 5 ? 25 : 20);
    return (int64_t)kComputeUnits * (waves_per_cu / waves);
}

// The store gate of a launch of 16-bit rows: for batches whose workgroups are all resident at once (2048 lanes per
// compute unit) the time their reads take at 7 TB/s, the rate of a read-only kernel on this part, plus a twentieth;
// 0 (stores as soon as they are ready) for larger batches, whose later workgroups read while earlier ones write
// whatever a wave does.  Measured per call at 7168 elements: 6.35 against 7.2 us at 512 rows, 7.6 against 9.5 at
// 768, 9.0 against 11.7 at 1024 (gate 1.0-1.1 times the read time; 10.2 with 0.9, 9.6 with 1.2), nothing gained and
// 0.1 us lost below a quarter of a round; at 4096 elements 6.2 against 7.7 us at 1024 rows, 10.2 against 12.4 at 2048; 20-45 % slower where the
// batch does not fit one round.
uint32_t store_gate(int64_t tokens, int64_t hidden, int threads, int nchunk) {
    if (g_gate >= 0) return (uint32_t)g_gate;
    const int64_t resident = resident_rows(threads, nchunk);
    if (tokens > resident || 4 * tokens < resident) return 0;
    // (four chunks per lane: the shape pick_shape takes to hold in one round what two chunks per lane cannot)
    const double ticks = (nchunk >= 4 ? 1.08 : 1.05) * (double)(4 * tokens * hidden) / 70000.0;  // 70,000 bytes per tick of 10 ns
    return (uint32_t)std::min(ticks, 5000.0);
}

// Lanes per row and chunks per lane.  Measured on MI355X over rows of 1024 .. 16384 elements: two chunks per lane
// on as many lanes as that needs (up to 1024) streams best or ties everywhere (1-6 % over one or four chunks per
// lane), unless rounding up to whole waves would idle more lanes that way; longer rows double the chunks per lane.
// Decode-sized batches are served best by the same shape (7168 elements, per call replayed from a graph: 3.3 us
// against 3.5 us with one chunk per lane at one row, 5.0 against 5.6 us at 256 rows).
void pick_shape(int64_t tokens, int chunks_per_row, int *threads, int *nchunk) {
    auto fits = [&](int n) { return (int64_t)n * kMaxThreads >= chunks_per_row; };
    int n;
    if (g_force_nchunk) {
        n = g_force_nchunk;
    } else {
        // one chunk per lane only where two would leave more lanes idle after rounding up to whole waves
        const int lanes1 = round_up(chunks_per_row, 64), lanes2 = round_up((chunks_per_row + 1) / 2, 64);
        n = (2 * lanes2 > lanes1 && lanes1 <= kMaxThreads) ? 1 : 2;
        while (n < 8 && chunks_per_row > kMaxThreads * n) n *= 2;
        // A batch that two chunks per lane cannot hold in one round but four can (half the lanes per row, so up to
        // 2048 rows of 7168 or 8192 elements instead of 1024) takes four: one round, with the store gate, against two
        // rounds of mixed reads and writes.  7168 elements: 10.8 against 12.8 us at 1100 rows, 10.9 against 14.3 at
        // 1280, 13.0 against 16.2 at 1536, 14.3 against 17.5 at 1700; 8192 elements: 12.4 against 15.5 us at 1280 rows,
        // 16.3 against 18.7 at 1700.  (That form keeps the normed row as 16-bit pairs between its last two phases:
        // with it in fp32 the kernel took 70 registers, seven waves per SIMD, 1792 rows.)
        if (n == 2 && !g_force_threads) {
            const int t2 = round_up((chunks_per_row + 1) / 2, 64), t4 = round_up((chunks_per_row + 3) / 4, 64);
            if (tokens > resident_rows(t2, 2) && tokens <= resident_rows(t4, 4)) n = 4;
        }
    }
    while (n < 8 && !fits(n)) n *= 2;
    if (!fits(n)) {
        *nchunk = 0;
        *threads = kMaxThreads;
        return;
    }
    int t = round_up((chunks_per_row + n - 1) / n, 64);
    if (g_force_threads && (int64_t)g_force_threads * n >= chunks_per_row) t = g_force_threads;
    *nchunk = n;
    *threads = t;
}

// Launches per call.  A batch of more than one round of workgroups and at most two runs as two launches of half the
// rows, each a round of its own with the store gate: a read phase and a write phase twice over instead of two rounds
// that mix the directions.
int launches_for(int64_t tokens, int chunks_per_row) {
    if (g_pieces == 1 || g_force_nchunk || g_force_threads || chunks_per_row > 2 * kMaxThreads) return 1;
    const int64_t round = resident_rows(round_up((chunks_per_row + 3) / 4, 64), 4);
    if (tokens <= round || tokens > 2 * round) return 1;
    if (g_pieces == 2) return 2;
    return 10 * tokens >= 11 * round ? 2 : 1;
}

// Rows of the first launch: the whole batch, or of two pieces the first, a whole number of rows per compute unit (half
// of what the batch needs, rounded down), so that neither piece pays for a partly filled last row of workgroups twice.
int64_t first_piece(int64_t tokens, int chunks_per_row) {
    if (launches_for(tokens, chunks_per_row) == 1) return tokens;
    return (tokens + kComputeUnits - 1) / kComputeUnits / 2 * kComputeUnits;
}

template <typename T, int QUANT>
int launch_rows(const void *x, const void *residual_in, const void *gamma, void *residual_out, void *norm_out,
                float *scale, int64_t tokens, int64_t hidden, float eps, float fp8_max, hipStream_t stream);

template <typename T, int QUANT>
int launch(const void *x, const void *residual_in, const void *gamma, void *residual_out, void *norm_out,
           float *scale, int64_t tokens, int64_t hidden, float eps, float fp8_max, hipStream_t stream) {
    const int64_t piece = first_piece(tokens, (int)(hidden / 8));
    for (int64_t first = 0; first < tokens; first = first ? tokens : piece) {
        const int64_t in_bytes = first * hidden * 2, out_bytes = first * hidden * (QUANT == GPUK_QUANT_NONE ? 2 : 1);
        const int rc = launch_rows<T, QUANT>(static_cast<const char *>(x) + in_bytes, static_cast<const char *>(residual_in) + in_bytes,
                                             gamma, static_cast<char *>(residual_out) + in_bytes, static_cast<char *>(norm_out) + out_bytes,
                                             QUANT == GPUK_QUANT_FP8_DYNAMIC ? scale + first : scale, first ? tokens - first : piece,
                                             hidden, eps, fp8_max, stream);
        if (rc != GPUK_OK) return rc;
    }
    return GPUK_OK;
}

template <typename T, int QUANT>
int launch_rows(const void *x, const void *residual_in, const void *gamma, void *residual_out, void *norm_out,
                float *scale, int64_t tokens, int64_t hidden, float eps, float fp8_max, hipStream_t stream) {
    const int chunks = (int)(hidden / 8);
    int threads, nchunk;
    pick_shape(tokens, chunks, &threads, &nchunk);
    const dim3 grid((unsigned)tokens);
    auto xs = static_cast<const u32x4 *>(x);
    auto rs = static_cast<const u32x4 *>(residual_in);
    auto gs = static_cast<const u32x4 *>(gamma);
    auto ro = static_cast<u32x4 *>(residual_out);
    const float hf = (float)hidden;
    if (nchunk == 0) {
        add_rmsnorm_quant_long_rows<T, QUANT><<<grid, kMaxThreads, 0, stream>>>(xs, rs, gs, ro, norm_out, scale, chunks, hf, eps, fp8_max);
        return hip_status(hipGetLastError());
    }
    const float rcp_hidden = 1.0f / hf;
    const int hidden_pow2 = (hidden & (hidden - 1)) == 0;
    const float rcp_fp8_max = (fp8_max == 448.0f || fp8_max == 240.0f) ? 1.0f / fp8_max : 0.0f;
    const uint32_t gate = store_gate(tokens, hidden, threads, nchunk);
    // Runs of 64 rows per XCD: measured +1.1 % for 16 KiB rows (8192 rows); neutral or 1-10 % slower for every other
    // row size tried (2, 3, 4, 8, 10, 14, 32 KiB) and for fewer rows, hence the narrow rule.
    const int64_t row_bytes = hidden * 2;
    int group_shift = row_bytes == 16384 && tokens >= 1024 ? 6 : 0;
    if (g_row_group_shift >= 0) group_shift = g_row_group_shift;
    const int remap_end = group_shift > 0 ? (int)((tokens >> (3 + group_shift)) << (3 + group_shift)) : 0;
    const bool exact = (int64_t)threads * nchunk == chunks;
#define GPUK_LAUNCH_NQ_AS(N, EXACT, GATED)                                                                              \
    add_rmsnorm_quant_rows<T, N, QUANT, EXACT, GATED><<<grid, threads, 0, stream>>>(                                    \
        xs, rs, chunks, remap_end, (uint32_t)threads | ((uint32_t)group_shift << 16), gate, gs, ro, norm_out, scale, hf, \
        rcp_hidden, hidden_pow2, eps, fp8_max, rcp_fp8_max)
#define GPUK_LAUNCH_NQ(N)                                                                                              \
    do {                                                                                                               \
        if (exact && gate) GPUK_LAUNCH_NQ_AS(N, true, true);                                                           \
        else if (exact) GPUK_LAUNCH_NQ_AS(N, true, false);                                                             \
        else if (gate) GPUK_LAUNCH_NQ_AS(N, false, true);                                                              \
        else GPUK_LAUNCH_NQ_AS(N, false, false);                                                                       \
    } while (0)
    switch (nchunk) {
        case 1: GPUK_LAUNCH_NQ(1); break;
        case 2: GPUK_LAUNCH_NQ(2); break;
        case 4: GPUK_LAUNCH_NQ(4); break;
        case 8: GPUK_LAUNCH_NQ(8); break;
        default: return GPUK_ERR_INTERNAL;
    }
#undef GPUK_LAUNCH_NQ
#undef GPUK_LAUNCH_NQ_AS
    return hip_status(hipGetLastError());
}

// Lanes and kept chunks per lane of the fp32 / fp64 kernel; 0 chunks kept = rows beyond 4096 chunks, swept.  fp32, as
// for the 16-bit kernel: two chunks per lane unless that leaves more lanes idle in the last wave (12 % ahead of one
// chunk at 32768 x 4096); fp64: one chunk (32 bytes) per lane up to 1024 lanes (6 % ahead of two).
void pick_wide_shape(int chunks, bool fp64, int *threads, int *cpl) {
    const int lanes1 = round_up(chunks, 64), lanes2 = round_up((chunks + 1) / 2, 64);
    int n = (fp64 || 2 * lanes2 > lanes1) && lanes1 <= kMaxThreads ? 1 : 2;
    while (n < 4 && chunks > n * kMaxThreads) n *= 2;
    if (chunks > n * kMaxThreads) {
        *cpl = 0;
        *threads = kMaxThreads;
        return;
    }
    *cpl = n;
    *threads = round_up((chunks + n - 1) / n, 64);
}

template <typename F, int QUANT>
int launch_wide(const void *x, const void *residual_in, const void *gamma, void *residual_out, void *norm_out,
                float *scale, int64_t tokens, int64_t hidden, float eps, float fp8_max, hipStream_t stream) {
    const int chunks = (int)(hidden / 4);
    int threads, cpl;
    pick_wide_shape(chunks, sizeof(F) == 8, &threads, &cpl);
#define GPUK_LAUNCH_WIDE(CPL)                                                                                          \
    add_rmsnorm_quant_wide_rows<F, QUANT, CPL><<<dim3((unsigned)tokens), threads, 0, stream>>>(                        \
        static_cast<const wide4<F> *>(x), static_cast<const wide4<F> *>(residual_in),                                  \
        static_cast<const wide4<F> *>(gamma), static_cast<wide4<F> *>(residual_out), norm_out, scale, chunks,          \
        (float)hidden, eps, fp8_max)
    switch (cpl) {
        case 1: GPUK_LAUNCH_WIDE(1); break;
        case 2: GPUK_LAUNCH_WIDE(2); break;
        case 4: GPUK_LAUNCH_WIDE(4); break;
        default: GPUK_LAUNCH_WIDE(0); break;
    }
#undef GPUK_LAUNCH_WIDE
    return hip_status(hipGetLastError());
}

template <typename F>
int launch_quant_wide(int quant_mode, const void *x, const void *residual_in, const void *gamma, void *residual_out,
                      void *norm_out, float *scale, int64_t tokens, int64_t hidden, float eps, float fp8_max,
                      hipStream_t stream) {
    switch (quant_mode) {
        case GPUK_QUANT_NONE:
            return launch_wide<F, GPUK_QUANT_NONE>(x, residual_in, gamma, residual_out, norm_out, scale, tokens, hidden, eps, fp8_max, stream);
        case GPUK_QUANT_FP8_DYNAMIC:
            return launch_wide<F, GPUK_QUANT_FP8_DYNAMIC>(x, residual_in, gamma, residual_out, norm_out, scale, tokens, hidden, eps, fp8_max, stream);
        case GPUK_QUANT_FP8_STATIC:
            return launch_wide<F, GPUK_QUANT_FP8_STATIC>(x, residual_in, gamma, residual_out, norm_out, scale, tokens, hidden, eps, fp8_max, stream);
        default:
            return GPUK_ERR_UNSUPPORTED;
    }
}

template <typename T>
int launch_quant(int quant_mode, const void *x, const void *residual_in, const void *gamma, void *residual_out,
                 void *norm_out, float *scale, int64_t tokens, int64_t hidden, float eps, float fp8_max,
                 hipStream_t stream) {
    switch (quant_mode) {
        case GPUK_QUANT_NONE:
            return launch<T, GPUK_QUANT_NONE>(x, residual_in, gamma, residual_out, norm_out, scale, tokens, hidden, eps, fp8_max, stream);
        case GPUK_QUANT_FP8_DYNAMIC:
            return launch<T, GPUK_QUANT_FP8_DYNAMIC>(x, residual_in, gamma, residual_out, norm_out, scale, tokens, hidden, eps, fp8_max, stream);
        case GPUK_QUANT_FP8_STATIC:
            return launch<T, GPUK_QUANT_FP8_STATIC>(x, residual_in, gamma, residual_out, norm_out, scale, tokens, hidden, eps, fp8_max, stream);
        default:
            return GPUK_ERR_UNSUPPORTED;
    }
}

}  // namespace

void set_norm_quant_tuning(int key, int value) {
    if (key == 0) g_force_nchunk = value;
    if (key == 1) g_force_threads = value;
    if (key == 5) g_row_group_shift = value;
    if (key == 6) g_gate = value;
    if (key == 7) g_pieces = value;
}

}  // namespace gpuk

// profiling build: where the kernels of this file write their phase stamps
GPUK_STAMPS_SETTER(gpuk_stamps_set_norm_quant)

extern "C" int gpuk_add_rmsnorm_quant_traffic_only(const void *x, const void *residual_in, void *residual_out,
                                                   void *codes, float *scale, int64_t tokens, int64_t hidden,
                                                   void *stream) {
    using namespace gpuk;
    if (tokens <= 0 || hidden <= 0 || hidden % 8 != 0 || tokens > 0x7fffffffLL) return GPUK_ERR_INVALID_ARG;
    if (!x || !residual_in || !residual_out || !codes || !scale) return GPUK_ERR_INVALID_ARG;
    if (!aligned16(x) || !aligned16(residual_in) || !aligned16(residual_out) || !aligned8(codes)) return GPUK_ERR_MISALIGNED;
    const int chunks = (int)(hidden / 8);
    if (const int64_t piece = first_piece(tokens, chunks); piece < tokens) {  // two launches where the op takes two
        const int rc = gpuk_add_rmsnorm_quant_traffic_only(x, residual_in, residual_out, codes, scale, piece, hidden, stream);
        if (rc != GPUK_OK) return rc;
        const int64_t wide = piece * hidden * 2, narrow = piece * hidden;
        return gpuk_add_rmsnorm_quant_traffic_only(static_cast<const char *>(x) + wide, static_cast<const char *>(residual_in) + wide,
                                                   static_cast<char *>(residual_out) + wide, static_cast<char *>(codes) + narrow,
                                                   scale + piece, tokens - piece, hidden, stream);
    }
    int threads, nchunk;
    pick_shape(tokens, chunks, &threads, &nchunk);
    if (nchunk == 0) return GPUK_ERR_UNSUPPORTED;  // rows that do not stay in registers
    int group_shift = hidden * 2 == 16384 && tokens >= 1024 ? 6 : 0;
    if (g_row_group_shift >= 0) group_shift = g_row_group_shift;
    const int remap_end = group_shift > 0 ? (int)((tokens >> (3 + group_shift)) << (3 + group_shift)) : 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    auto xs = static_cast<const u32x4 *>(x), rs = static_cast<const u32x4 *>(residual_in);
    auto ro = static_cast<u32x4 *>(residual_out);
    auto co = static_cast<u32x2 *>(codes);
    const dim3 grid((unsigned)tokens);
    const uint32_t gate = store_gate(tokens, hidden, threads, nchunk);
    const uint32_t shape = (uint32_t)threads | ((uint32_t)group_shift << 16);
    switch (nchunk) {
        case 1: add_rmsnorm_quant_traffic_only<1><<<grid, threads, 0, s>>>(xs, rs, chunks, remap_end, shape, gate, ro, co, scale); break;
        case 2: add_rmsnorm_quant_traffic_only<2><<<grid, threads, 0, s>>>(xs, rs, chunks, remap_end, shape, gate, ro, co, scale); break;
        case 4: add_rmsnorm_quant_traffic_only<4><<<grid, threads, 0, s>>>(xs, rs, chunks, remap_end, shape, gate, ro, co, scale); break;
        default: add_rmsnorm_quant_traffic_only<8><<<grid, threads, 0, s>>>(xs, rs, chunks, remap_end, shape, gate, ro, co, scale); break;
    }
    return hip_status(hipGetLastError());
}

extern "C" int gpuk_add_rmsnorm_quant_launch_shape(int64_t tokens, int64_t hidden, int dtype, int *lanes_per_row,
                                                   int *chunks_per_lane) {
    using namespace gpuk;
    if (tokens <= 0 || hidden <= 0 || !lanes_per_row || !chunks_per_lane) return GPUK_ERR_INVALID_ARG;
    if (dtype != GPUK_DTYPE_BF16 && dtype != GPUK_DTYPE_FP16 && dtype != GPUK_DTYPE_F32 && dtype != GPUK_DTYPE_F64) return GPUK_ERR_UNSUPPORTED;
    const bool wide = dtype == GPUK_DTYPE_F32 || dtype == GPUK_DTYPE_F64;
    if (hidden % 8 != 0) return GPUK_ERR_UNSUPPORTED;  // the rule of gpuk_add_rmsnorm_quant, for every dtype
    if (wide) {  // the fp32 / fp64 kernel: 4-element chunks, 0 = rows swept three times
        pick_wide_shape((int)(hidden / 4), dtype == GPUK_DTYPE_F64, lanes_per_row, chunks_per_lane);
        return GPUK_OK;
    }
    pick_shape(first_piece(tokens, (int)(hidden / 8)), (int)(hidden / 8), lanes_per_row, chunks_per_lane);
    return GPUK_OK;
}

extern "C" int gpuk_add_rmsnorm_quant(const void *x, const void *residual_in, const void *gamma, void *residual_out,
                                      void *norm_out, float *scale, int64_t tokens, int64_t hidden, float eps,
                                      int dtype, int quant_mode, float fp8_max, void *stream) {
    using namespace gpuk;
    if (tokens < 0 || hidden <= 0) return GPUK_ERR_INVALID_ARG;
    if (hidden % 8 != 0) return GPUK_ERR_UNSUPPORTED;           // rows are moved in 16-byte chunks
    if (tokens > 0x7fffffffLL || hidden / 8 > 0x7fffffffLL) return GPUK_ERR_UNSUPPORTED;
    if (!(fp8_max > 0.f) && quant_mode != GPUK_QUANT_NONE) return GPUK_ERR_INVALID_ARG;
    if (quant_mode == GPUK_QUANT_FP8_E4M3FNUZ) return GPUK_ERR_UNSUPPORTED;  // gfx950 encodes OCP e4m3fn only
    if (tokens == 0) return GPUK_OK;
    if (!x || !residual_in || !gamma || !residual_out || !norm_out) return GPUK_ERR_INVALID_ARG;
    if (quant_mode != GPUK_QUANT_NONE && !scale) return GPUK_ERR_INVALID_ARG;
    if (!aligned16(x) || !aligned16(residual_in) || !aligned16(gamma) || !aligned16(residual_out)) return GPUK_ERR_MISALIGNED;
    if (!(quant_mode == GPUK_QUANT_NONE ? aligned16(norm_out) : aligned8(norm_out))) return GPUK_ERR_MISALIGNED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case GPUK_DTYPE_BF16:
            return launch_quant<BF16>(quant_mode, x, residual_in, gamma, residual_out, norm_out, scale, tokens, hidden, eps, fp8_max, s);
        case GPUK_DTYPE_FP16:
            return launch_quant<FP16>(quant_mode, x, residual_in, gamma, residual_out, norm_out, scale, tokens, hidden, eps, fp8_max, s);
        case GPUK_DTYPE_F32:
            return launch_quant_wide<float>(quant_mode, x, residual_in, gamma, residual_out, norm_out, scale, tokens, hidden, eps, fp8_max, s);
        case GPUK_DTYPE_F64:
            return launch_quant_wide<double>(quant_mode, x, residual_in, gamma, residual_out, norm_out, scale, tokens, hidden, eps, fp8_max, s);
        default:
            return GPUK_ERR_UNSUPPORTED;
    }
}
