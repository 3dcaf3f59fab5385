// Device-side building blocks shared by the gfx950 kernels: 16-bit float pack/unpack on the
// hardware converters, wave64 DPP reductions, and the OCP e4m3fn packed converter.
//
// Replaces the reference's src/common/kernel_utils.h (vec_t, 32-wide shuffle reductions,
// block_reduce with WARP_SIZE hard-coded to 32: kernel_utils.h:29-53) and src/common/float8.h
// (software fp32->fp8 encoder: float8.h:17-150) with wave64 / hardware equivalents.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gpuk {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

struct BF16 {};  // tag types: the 16-bit storage format of activations
struct FP16 {};

// Two 16-bit floats packed in one dword <-> two fp32 values.  Packing rounds to nearest even
// (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32).
template <typename T> struct Pack16;

template <> struct Pack16<BF16> {
    static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        f32x2 v = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
    }
    // rT(a) as a float: the high half of a pair whose low half is zero is the float's own bit pattern, so one
    // conversion instruction rounds without a separate unpack
    static __device__ __forceinline__ float round(float a) { return __builtin_bit_cast(float, pack(0.0f, a)); }
    // acc + lo(w)^2 + hi(w)^2 in one v_dot2c_f32_bf16 (products exact, fp32 accumulate)
    static __device__ __forceinline__ float add_squares(uint32_t w, float acc) {
        const bf16x2_t v = __builtin_bit_cast(bf16x2_t, w);
        return __builtin_amdgcn_fdot2_f32_bf16(v, v, acc, false);
    }
    static __device__ __forceinline__ float from_bits16(uint32_t h) { return __builtin_bit_cast(float, h << 16); }
};

template <> struct Pack16<FP16> {
    static __device__ __forceinline__ float lo(uint32_t w) {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
    }
    static __device__ __forceinline__ float hi(uint32_t w) {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
    }
    // The empty asm statements keep the fp32 value a result of its own: where the compiler sees a product or a
    // fused multiply-add feeding the conversion it emits v_fma_mixlo_f16, which rounds the exact result once, to
    // half precision -- not the fp32 rounding followed by the half rounding of the sequence being reproduced
    // (they differ when the fp32 rounding lands on a half-precision tie).
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        asm("" : "+v"(a));
        asm("" : "+v"(b));
        const uint32_t l = __builtin_bit_cast(uint16_t, (_Float16)a);
        const uint32_t h = __builtin_bit_cast(uint16_t, (_Float16)b);
        return l | (h << 16);
    }
    static __device__ __forceinline__ float round(float a) {
        asm("" : "+v"(a));
        return (float)(_Float16)a;
    }
    static __device__ __forceinline__ float add_squares(uint32_t w, float acc) {
        const float a = lo(w), b = hi(w);
        return __builtin_fmaf(b, b, __builtin_fmaf(a, a, acc));
    }
    static __device__ __forceinline__ float from_bits16(uint32_t h) {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
    }
};

// ---- DPP lane exchange.  CTRL encodings: quad_perm[a,b,c,d] = a|b<<2|c<<4|d<<6,
// row_half_mirror = 0x141, row_mirror = 0x140 (both reverse within 8 / 16 lanes).
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(float,
                              __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

constexpr int DPP_QUAD_XOR1 = 0xB1;       // quad_perm [1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;       // quad_perm [2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;

struct SumOp {
    static __device__ __forceinline__ float apply(float a, float b) { return a + b; }
    static __device__ __forceinline__ float identity() { return 0.f; }
};
struct MaxOp {  // used on magnitudes only, so 0 is the identity.  Compared as bit patterns: for non-negative floats
                // these order like the values, and a (positive) NaN beats everything, as in the reference's amax
    static __device__ __forceinline__ float apply(float a, float b) {
        const uint32_t x = __builtin_bit_cast(uint32_t, a), y = __builtin_bit_cast(uint32_t, b);
        return __builtin_bit_cast(float, __builtin_elementwise_max(x, y));
    }
    static __device__ __forceinline__ float identity() { return 0.f; }
};

// All-reduce over aligned groups of LANES consecutive lanes (LANES in {2, 4, 8, 16}): every lane
// ends with its group's result.  One DPP row is 16 lanes, so these never leave the row.
template <typename Op, int LANES>
__device__ __forceinline__ float group_allreduce(float v) {
    static_assert(LANES == 2 || LANES == 4 || LANES == 8 || LANES == 16, "group must fit in one DPP row");
    v = Op::apply(v, dpp_f32<DPP_QUAD_XOR1>(v));
    if constexpr (LANES >= 4) v = Op::apply(v, dpp_f32<DPP_QUAD_XOR2>(v));
    if constexpr (LANES >= 8) v = Op::apply(v, dpp_f32<DPP_ROW_HALF_MIRROR>(v));
    if constexpr (LANES >= 16) v = Op::apply(v, dpp_f32<DPP_ROW_MIRROR>(v));
    return v;
}

// All-reduce over the 64 lanes of a wave; the result is wave-uniform.  Four row results are
// combined in a fixed order (rows 0,1,2,3), so the value does not depend on lane.
template <typename Op>
__device__ __forceinline__ float wave_allreduce(float v) {
    v = group_allreduce<Op, 16>(v);
    int b = __builtin_bit_cast(int, v);
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return Op::apply(Op::apply(r0, r1), Op::apply(r2, r3));
}

// Workgroup all-reduce of N independent values: wave results meet in LDS (N x 16 floats, at most 16 waves), one
// barrier, then every wave reads the per-wave results into its lanes (lane l takes wave l mod 16) and folds them with
// four DPP steps, so the result is the same in every lane of the workgroup.  `slots` must be private to this call
// site so that two consecutive reductions need only one barrier each.
constexpr int kReduceSlots = 16;
template <typename Op, int N>
__device__ __forceinline__ void block_allreduce(float (&v)[N], float *slots, int num_waves) {
#pragma unroll
    for (int n = 0; n < N; ++n) v[n] = wave_allreduce<Op>(v[n]);
    if (num_waves == 1) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
#pragma unroll
        for (int n = 0; n < N; ++n) slots[n * kReduceSlots + wave] = v[n];
    }
    __syncthreads();
    const int src = lane & (kReduceSlots - 1);
#pragma unroll
    for (int n = 0; n < N; ++n) {
        const float s = slots[n * kReduceSlots + src];
        v[n] = group_allreduce<Op, 16>(src < num_waves ? s : Op::identity());
    }
}

// Four fp32 -> four OCP e4m3fn codes in one dword (two v_cvt_pk_fp8_f32).  Inputs must already be
// clamped to the finite range; rounding is to nearest even.
__device__ __forceinline__ uint32_t cvt4_e4m3fn(float a, float b, float c, float d) {
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
    return (uint32_t)w;
}

// clamp to [-bound, bound]; a NaN stays a NaN (v_med3_f32 alone would turn it into one of the bounds)
__device__ __forceinline__ float clamp_sym(float v, float bound) {
    const float c = __builtin_amdgcn_fmed3f(v, -bound, bound);
    return v != v ? v : c;
}

// clamp_sym over 8 values, done only if one of them is out of range (rare): the test costs four v_max3_f32, the
// clamps 24 instructions.  A NaN does not trigger the clamp (fmax drops it) and needs none: the fp8 converter maps
// NaN to NaN.
__device__ __forceinline__ void clamp8_sym(float (&q)[8], float bound) {
    const float m01 = __builtin_fmaxf(__builtin_fabsf(q[0]), __builtin_fabsf(q[1]));
    const float m23 = __builtin_fmaxf(__builtin_fabsf(q[2]), __builtin_fabsf(q[3]));
    const float m45 = __builtin_fmaxf(__builtin_fabsf(q[4]), __builtin_fabsf(q[5]));
    const float m67 = __builtin_fmaxf(__builtin_fabsf(q[6]), __builtin_fabsf(q[7]));
    const float m = __builtin_fmaxf(__builtin_fmaxf(m01, m23), __builtin_fmaxf(m45, m67));
    if (__builtin_expect(m > bound, 0)) {
#pragma unroll
        for (int j = 0; j < 8; ++j) q[j] = clamp_sym(q[j], bound);
    }
}

// Correctly rounded fp32 quotient a/b given rcp = RN(1/b): one multiply and two fused
// multiply-adds (Markstein's correction step).  Valid while a/b, the residual and rcp stay in the
// normal range and b > 0; callers guard the range of b once per row and fall back to `/` outside it.
// The correction step alone turns a quotient of -0 into +0 and an infinite one into NaN; v_div_fixup_f32 puts
// back the sign and the zero / infinity / NaN a division gives for such numerators.
__device__ __forceinline__ float div_by_rcp(float a, float b, float rcp) {
    float q = a * rcp;
    float e = __builtin_fmaf(-q, b, a);
    return __builtin_amdgcn_div_fixupf(__builtin_fmaf(e, rcp, q), b, a);
}

// ---- Correctly rounded square root and reciprocal by short sequences.  The compiler's expansions of sqrtf() and of
// 1.0f / x are correct for every operand and pay for it with rescaling and fix-up steps (about 20 and 11 dependent
// instructions); on operands in the middle of the exponent range those steps do nothing.  These start from
// v_sqrt_f32 / v_rcp_f32 (1 ULP) and correct the result; oracle/gpuk_oracle.c holds the same sequences and
// tests/test_oracle_norm_quant.py runs them over every mantissa from every first guess within one ULP: they return the
// correctly rounded value except the reciprocal of a number whose mantissa bits are all ones, which callers exclude.
__device__ __forceinline__ float sqrt_rn_mid_range(float v) {  // v in [2^-95, 2^97)
    const float s = __builtin_amdgcn_sqrtf(v);
    const float dn = __builtin_bit_cast(float, __builtin_bit_cast(int32_t, s) - 1);
    const float up = __builtin_bit_cast(float, __builtin_bit_cast(int32_t, s) + 1);
    const float r_dn = __builtin_fmaf(-dn, s, v), r_up = __builtin_fmaf(-up, s, v);
    const float t = r_dn <= 0.0f ? dn : s;
    return r_up > 0.0f ? up : t;
}
__device__ __forceinline__ float rcp_rn_mid_range(float s) {  // s in [2^-60, 2^60], mantissa not all ones
    float y = __builtin_amdgcn_rcpf(s);
    y = __builtin_fmaf(__builtin_fmaf(-s, y, 1.0f), y, y);
    return __builtin_fmaf(__builtin_fmaf(-s, y, 1.0f), y, y);
}
__device__ __forceinline__ bool in_mid_range(float v) {  // [2^-60, 2^60): one subtraction and one unsigned compare
    return __builtin_bit_cast(uint32_t, v) - 0x21800000u < 0x3c000000u;
}
__device__ __forceinline__ bool mantissa_all_ones(float v) {
    return (__builtin_bit_cast(uint32_t, v) & 0x7fffffu) == 0x7fffffu;
}
// 1 / sqrt(v), both steps correctly rounded, as `1.0f / sqrtf(v)`.  The choice between the short and the general
// sequence is made for the whole wave, so the common case has no divergent branch.
__device__ __forceinline__ float rsqrt_two_roundings(float v) {
    const float s = sqrt_rn_mid_range(v);
    const bool ok = in_mid_range(v) && !mantissa_all_ones(s);
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(!ok) == 0, 1)) return rcp_rn_mid_range(s);
    return 1.0f / sqrtf(v);
}

// ---- Phase stamps (profiling build only: -DGPUK_STAMPS, `python -m gpuk_amd.build --stamps`).  A wave reads the
// shader clock at named points of a kernel and keeps the readings in scalar registers; at its end lane 0 writes them,
// with the 100 MHz wall clock at entry and exit and the wave's place on the chip, to a host-provided buffer of
// kStampSlots 64-bit words per wave.  In the product build every macro below expands to nothing.
constexpr int kStampSlots = 16;
#ifdef GPUK_STAMPS
static __device__ uint64_t *g_stamp_buffer;   // one copy per translation unit, set by that unit's gpuk_stamps_* entry
static __device__ uint32_t g_stamp_waves;     // waves the buffer has room for
struct Stamps {
    uint64_t t[kStampSlots - 3];
    uint64_t wall0;
    __device__ __forceinline__ static uint64_t cycles() {
        uint64_t v;
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v)::"memory");
        __builtin_amdgcn_sched_barrier(0);
        return v;
    }
    __device__ __forceinline__ static uint64_t wall() {
        uint64_t v;
        asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v)::"memory");
        return v;
    }
    __device__ __forceinline__ void begin() {
#pragma unroll
        for (int i = 0; i < kStampSlots - 3; ++i) t[i] = 0;
        wall0 = wall();
        t[0] = cycles();
    }
    // every vector memory operation of the wave has completed: loads have landed, stores are acknowledged
    __device__ __forceinline__ static void drain() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
    __device__ __forceinline__ void write(uint32_t wave_index) const {
        const uint64_t wall1 = wall();
        uint32_t hw_id, xcc_id;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw_id));
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc_id));
        if (g_stamp_buffer && wave_index < g_stamp_waves && (threadIdx.x & 63) == 0) {
            uint64_t *out = g_stamp_buffer + (uint64_t)wave_index * kStampSlots;
#pragma unroll
            for (int i = 0; i < kStampSlots - 3; ++i) out[i] = t[i];
            out[kStampSlots - 3] = wall0;
            out[kStampSlots - 2] = wall1;
            out[kStampSlots - 1] = ((uint64_t)(xcc_id & 0xf) << 32) | hw_id;
        }
    }
};
#define GPUK_STAMPS_BEGIN() gpuk::Stamps stamps_; stamps_.begin()
#define GPUK_STAMP(slot) (stamps_.t[slot] = gpuk::Stamps::cycles())
#define GPUK_STAMP_DRAINED(slot) (gpuk::Stamps::drain(), stamps_.t[slot] = gpuk::Stamps::cycles())
#define GPUK_STAMPS_WRITE(wave_index) stamps_.write(wave_index)
#define GPUK_STAMPS_SETTER(name)                                                                                     \
    extern "C" int name(void *buffer, uint32_t waves) {                                                                \
        uint64_t *b = static_cast<uint64_t *>(buffer);                                                                 \
        if (hipMemcpyToSymbol(HIP_SYMBOL(gpuk::g_stamp_buffer), &b, sizeof(b)) != hipSuccess) return GPUK_ERR_INTERNAL; \
        if (hipMemcpyToSymbol(HIP_SYMBOL(gpuk::g_stamp_waves), &waves, sizeof(waves)) != hipSuccess) return GPUK_ERR_INTERNAL; \
        return GPUK_OK;                                                                                                \
    }
#else
#define GPUK_STAMPS_BEGIN() ((void)0)
#define GPUK_STAMP(slot) ((void)0)
#define GPUK_STAMP_DRAINED(slot) ((void)0)
#define GPUK_STAMPS_WRITE(wave_index) ((void)0)
#define GPUK_STAMPS_SETTER(name)
#endif

}  // namespace gpuk
