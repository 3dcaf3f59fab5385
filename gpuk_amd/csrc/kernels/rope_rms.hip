// Per-head RMSNorm of Q and K + rotary embedding (RoPE / 3-axis mRoPE), written in place or scattered
// to q_out and a paged KV cache.
//
// Stands behind the reference's fused_rope_rms, fused_mrope_3d_rms and fused_mrope_3d_rms_set_kv
// (host ops src/ops/fused_rope.cpp:19-166, kernels src/impl/rope_rms_impl.h:157-466, launchers :468-610).
// The reference maps one 32-lane group to one head with D/32 elements per lane, fetches the rotation
// partner with two vector shuffles and gathers cos/sin element by element, per head, with 64-bit modulo
// arithmetic.  Here a head is D/16 lanes of a wave64 and every lane owns two 16-byte chunks that already
// contain both members of each rotation pair, so the rotation needs no cross-lane traffic and the sum of
// squares is reduced with 2-4 DPP steps inside one 16-lane row.
//
// Work decomposition: Q and K heads of a token form one index space of Hq+Hk heads; one wave takes 64/(D/16)
// consecutive heads of one token (2 KiB of contiguous qkv at D=128), whether they are Q, K or a mix (the norm
// weights and the destination are chosen per lane).  With a KV cache, the waves of a token also share out the
// token's V row, one 16-byte chunk per lane, so no wave exists only to copy.
//
// Numerics follow the reference's torch oracle (test/test_fused_rope_rms.py:8-34,
// test/test_fused_mrope_rms_set_kv.py:62-130), rT = round-to-nearest-even into the 16-bit type:
//     n   = rT(w * rT(x * rstd)),  rstd = 1/sqrt(mean(x^2) + eps)   (fp32, correctly rounded)
//     o1  = rT(rT(n1*cos) - rT(n2*sin)) ;  o2 = rT(rT(n2*cos) + rT(n1*sin))
//     fp8 cache: code = e4m3fn(rT(o / scale)), saturating at +-448
#include <hip/hip_runtime.h>

#include <algorithm>

#include "../../../include/gpuk_amd.h"
#include "device_utils.h"
#include "host_utils.h"

namespace gpuk {

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr float kE4M3Max = 448.0f;

struct RopeArgs {
    const void *qkv_in;
    void *qkv_out;  // == qkv_in for the in-place form, unused for set_kv
    const void *qw, *kw, *cos_sin;
    const int64_t *positions;
    int64_t ps_axis, ps_token;
    void *q_out, *k_cache, *v_cache;
    const int64_t *kv_loc;
    // one wave per unit = (token, group of heads); units_per_token = ceil((hq + hk) / heads per wave)
    uint32_t total_units, units_per_token;
    uint32_t upt_magic;  // ceil(2^32 / units_per_token), or 0 when units_per_token is 1: unit / units_per_token is
                         // mulhi(unit, magic) for every unit the host admits
    int hq, hk, hv;
    float eps, k_scale, v_scale;
    // mRoPE: bit f of axis1 / axis2 set when rotary frequency f takes its position from axis 1 / 2
    uint32_t axis1[4], axis2[4];
};

// dword mask selecting the 16-bit halves whose bit is set in a 2-bit field
__device__ __forceinline__ uint32_t halves_mask(uint32_t two_bits) {
    return ((two_bits & 1u) ? 0x0000ffffu : 0u) | ((two_bits & 2u) ? 0xffff0000u : 0u);
}
__device__ __forceinline__ uint32_t bitselect(uint32_t mask, uint32_t a, uint32_t b) {  // mask ? a : b
    return (a & mask) | (b & ~mask);
}

template <typename T>
__device__ __forceinline__ float elem(const u32x4 &v, int e) {  // element e (0..7) of a packed chunk
    return (e & 1) ? Pack16<T>::hi(v[e >> 1]) : Pack16<T>::lo(v[e >> 1]);
}

// A lane's two chunks sit at elements 8*sub and D/2 + 8*sub of its head in both styles, so that every load and store
// instruction of a wave covers whole 128-byte lines.  NeoX: the chunks hold x1 and x2 of rotary frequencies
// 8*sub .. 8*sub+7.  GPT-J: each dword is an (x1, x2) pair; the first chunk holds frequencies 4*sub .. 4*sub+3, the
// second D/4 + 4*sub .. D/4 + 4*sub+3.  The cos (or sin) values of the lane's 8 frequencies, first chunk's first:
template <int D, bool NEOX>
__device__ __forceinline__ u32x4 load_trig(const uint16_t *row, int sub) {  // row = cos (or sin) half of a table row
    if constexpr (NEOX) {
        return *reinterpret_cast<const u32x4 *>(row + 8 * sub);
    } else {
        const u32x2 lo = *reinterpret_cast<const u32x2 *>(row + 4 * sub);
        const u32x2 hi = *reinterpret_cast<const u32x2 *>(row + D / 4 + 4 * sub);
        return u32x4{lo[0], lo[1], hi[0], hi[1]};
    }
}
// ... and the matching 8 bits of a frequency bitmap (bit f = frequency f)
template <int D, bool NEOX>
__device__ __forceinline__ uint32_t trig_bits(const uint32_t (&bitmap)[4], int sub) {
    if constexpr (NEOX) {
        const int f = 8 * sub;
        return (bitmap[f >> 5] >> (f & 31)) & 0xffu;
    } else {
        const int f0 = 4 * sub, f1 = D / 4 + 4 * sub;
        return ((bitmap[f0 >> 5] >> (f0 & 31)) & 0xfu) | (((bitmap[f1 >> 5] >> (f1 & 31)) & 0xfu) << 4);
    }
}

// 8 codes = e4m3fn(clamp(rT(v / scale))) for one chunk; `rcp` is RN(1/scale) and is used when FAST
template <typename T, bool FAST>
__device__ __forceinline__ u32x2 quantize_chunk(const u32x4 &v, float scale, float rcp) {
    using P = Pack16<T>;
    float q[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float a = FAST ? div_by_rcp(P::lo(v[j]), scale, rcp) : P::lo(v[j]) / scale;
        const float b = FAST ? div_by_rcp(P::hi(v[j]), scale, rcp) : P::hi(v[j]) / scale;
        const uint32_t w = P::pack(a, b);
        q[2 * j] = P::lo(w);
        q[2 * j + 1] = P::hi(w);
    }
    clamp8_sym(q, kE4M3Max);
    return u32x2{cvt4_e4m3fn(q[0], q[1], q[2], q[3]), cvt4_e4m3fn(q[4], q[5], q[6], q[7])};
}
__device__ __forceinline__ bool scale_is_fast(float s) { return s >= 0x1p-60f && s <= 0x1p60f; }

// RMSNorm of one head (D/16 lanes x two chunks) followed by the rotation, for the lane's two chunks.
//   NeoX : chunk a holds x1 for the lane's 8 frequencies, chunk b the matching x2.
//   GPT-J: each dword is one (x1, x2) pair; chunk a uses cos/sin values 0-3 of the lane, chunk b values 4-7.
template <typename T, int D, bool NEOX>
__device__ __forceinline__ void norm_rotate(const u32x4 &xa, const u32x4 &xb, const u32x4 &wa, const u32x4 &wb,
                                            const u32x4 &cosv, const u32x4 &sinv, float eps, u32x4 &oa, u32x4 &ob) {
    using P = Pack16<T>;
    constexpr int LPH = D / 16;
    float ss0 = 0.f, ss1 = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        ss0 = P::add_squares(xa[j], ss0);
        ss1 = P::add_squares(xb[j], ss1);
    }
    const float sumsq = group_allreduce<SumOp, LPH>(ss0 + ss1);
    const float rstd = 1.0f / sqrtf(sumsq * (1.0f / D) + eps);  // D is a power of two: the product is exact

    // normed values stay in fp32 registers, each already rounded to the 16-bit type
    float na[8], nb[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        na[2 * j] = P::round(P::lo(wa[j]) * P::round(P::lo(xa[j]) * rstd));
        na[2 * j + 1] = P::round(P::hi(wa[j]) * P::round(P::hi(xa[j]) * rstd));
        nb[2 * j] = P::round(P::lo(wb[j]) * P::round(P::lo(xb[j]) * rstd));
        nb[2 * j + 1] = P::round(P::hi(wb[j]) * P::round(P::hi(xb[j]) * rstd));
    }

    if constexpr (NEOX) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float x1l = na[2 * j], x1h = na[2 * j + 1], x2l = nb[2 * j], x2h = nb[2 * j + 1];
            const float cl = P::lo(cosv[j]), ch = P::hi(cosv[j]), sl = P::lo(sinv[j]), sh = P::hi(sinv[j]);
            oa[j] = P::pack(P::round(x1l * cl) - P::round(x2l * sl), P::round(x1h * ch) - P::round(x2h * sh));
            ob[j] = P::pack(P::round(x2l * cl) + P::round(x1l * sl), P::round(x2h * ch) + P::round(x1h * sh));
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            {
                const float x1 = na[2 * e], x2 = na[2 * e + 1];
                const float c = elem<T>(cosv, e), s = elem<T>(sinv, e);
                oa[e] = P::pack(P::round(x1 * c) - P::round(x2 * s), P::round(x2 * c) + P::round(x1 * s));
            }
            {
                const float x1 = nb[2 * e], x2 = nb[2 * e + 1];
                const float c = elem<T>(cosv, 4 + e), s = elem<T>(sinv, 4 + e);
                ob[e] = P::pack(P::round(x1 * c) - P::round(x2 * s), P::round(x2 * c) + P::round(x1 * s));
            }
        }
    }
}

// What one wave keeps about one unit (= one group of 64/(D/16) consecutive Q/K heads of one token, plus its share
// of the token's V row) between issuing the unit's loads and finishing it.
struct UnitState {
    uint32_t t, u;
    int head;
    bool live, active, is_q;
    int64_t slot, p0, p1, p2;
    const uint16_t *token_in;
    u32x4 xa, xb, wa, wb, cosv, sinv, vchunk;
};

// AXES: 1 = RoPE, 3 = mRoPE.  SETKV: false = in place, true = scatter to q_out / caches.
template <typename T, int D, bool NEOX, int AXES, bool SETKV, bool KVFP8>
struct RopeUnit {
    using P = Pack16<T>;
    static constexpr int LPH = D / 16;    // lanes per head
    static constexpr int HPW = 64 / LPH;  // heads per wave
    static constexpr int HALF = D / 2;

    // element offsets of a lane's two chunks inside a head
    static __device__ __forceinline__ int c0(int sub) { return 8 * sub; }
    static __device__ __forceinline__ int c1(int sub) { return HALF + 8 * sub; }

    // Issues every load of the unit; nothing is waited for.
    static __device__ __forceinline__ void issue_loads(const RopeArgs &a, uint32_t unit, int lane, UnitState &st) {
        st.live = unit < a.total_units;  // wave-uniform
        if (!st.live) return;
        st.t = a.upt_magic ? __umulhi(unit, a.upt_magic) : unit;
        st.u = unit - st.t * a.units_per_token;
        const int sub = lane % LPH, hl = lane / LPH;
        const int heads_qk = a.hq + a.hk, heads_all = heads_qk + a.hv;
        st.token_in = static_cast<const uint16_t *>(a.qkv_in) + (int64_t)st.t * heads_all * D;

        // lanes past the last head re-read the last head (nothing of theirs is stored): no branch around the loads
        const int head_raw = st.u * HPW + hl;
        st.active = head_raw < heads_qk;
        st.head = min(head_raw, heads_qk - 1);
        st.is_q = st.head < a.hq;
        const uint16_t *src = st.token_in + (int64_t)st.head * D;
        // streamed when the results go elsewhere; in place the same lines are written a moment later, and keeping
        // them in L2 measured 2 % faster
        if constexpr (SETKV) {
            st.xa = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + c0(sub)));
            st.xb = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + c1(sub)));
        } else {
            st.xa = *reinterpret_cast<const u32x4 *>(src + c0(sub));
            st.xb = *reinterpret_cast<const u32x4 *>(src + c1(sub));
        }

        // this wave's share of the token's V row: chunk u*64 + lane (and further strides of units_per_token*64)
        if constexpr (SETKV) {
            st.slot = a.kv_loc[st.t];
            const int v_first = st.u * 64 + lane;
            if (v_first < a.hv * (D / 8))
                st.vchunk = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(st.token_in + (int64_t)heads_qk * D + 8 * v_first));
        }

        const uint16_t *wsrc = static_cast<const uint16_t *>(st.is_q ? a.qw : a.kw);
        st.wa = *reinterpret_cast<const u32x4 *>(wsrc + c0(sub));
        st.wb = *reinterpret_cast<const u32x4 *>(wsrc + c1(sub));

        st.p0 = a.positions[(int64_t)st.t * a.ps_token];
        if constexpr (AXES == 3) {
            st.p1 = a.positions[a.ps_axis + (int64_t)st.t * a.ps_token];
            st.p2 = a.positions[2 * a.ps_axis + (int64_t)st.t * a.ps_token];
        }
    }

    // The cos/sin loads, whose addresses wait for the positions.
    static __device__ __forceinline__ void issue_table_loads(const RopeArgs &a, int lane, UnitState &st) {
        if (!st.live) return;
        const int sub = lane % LPH;
        const uint16_t *table = static_cast<const uint16_t *>(a.cos_sin);
        const int64_t p0 = st.p0;
        st.cosv = load_trig<D, NEOX>(table + p0 * D, sub);
        st.sinv = load_trig<D, NEOX>(table + p0 * D + HALF, sub);
        if constexpr (AXES == 3) {
            const int64_t p1 = st.p1, p2 = st.p2;
            if (p1 != p0 || p2 != p0) {  // wave-uniform; text tokens carry three equal positions
                const u32x4 cos1 = load_trig<D, NEOX>(table + p1 * D, sub);
                const u32x4 sin1 = load_trig<D, NEOX>(table + p1 * D + HALF, sub);
                const u32x4 cos2 = load_trig<D, NEOX>(table + p2 * D, sub);
                const u32x4 sin2 = load_trig<D, NEOX>(table + p2 * D + HALF, sub);
                // the axis bits of the lane's 8 frequencies, in the order of the loaded values
                const uint32_t b1 = trig_bits<D, NEOX>(a.axis1, sub), b2 = trig_bits<D, NEOX>(a.axis2, sub);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t m1 = halves_mask(b1 >> (2 * j)), m2 = halves_mask(b2 >> (2 * j));
                    st.cosv[j] = bitselect(m2, cos2[j], bitselect(m1, cos1[j], st.cosv[j]));
                    st.sinv[j] = bitselect(m2, sin2[j], bitselect(m1, sin1[j], st.sinv[j]));
                }
            }
        }
    }

    // Norm, rotation and all stores of the unit.
    static __device__ __forceinline__ void finish(const RopeArgs &a, int lane, UnitState &st) {
        if (!st.live) return;
        const int sub = lane % LPH;
        const int heads_qk = a.hq + a.hk, heads_all = heads_qk + a.hv;
        const u32x4 &xa = st.xa, &xb = st.xb, &wa = st.wa, &wb = st.wb, &cosv = st.cosv, &sinv = st.sinv;

        u32x4 oa, ob;
        norm_rotate<T, D, NEOX>(xa, xb, wa, wb, cosv, sinv, a.eps, oa, ob);

        // A negative slot marks a token that has no place in the cache (padding in a fixed-size decode batch): its Q
        // row is still produced, its K and V rows are dropped.  The reference would write out of bounds.
        const bool slot_ok = !SETKV || st.slot >= 0;  // wave-uniform
        const int head = st.head;
        if (st.active && (st.is_q || slot_ok)) {
            if constexpr (!SETKV) {
                uint16_t *dst = static_cast<uint16_t *>(a.qkv_out) + ((int64_t)st.t * heads_all + head) * D;
                *reinterpret_cast<u32x4 *>(dst + c0(sub)) = oa;
                *reinterpret_cast<u32x4 *>(dst + c1(sub)) = ob;
            } else if (KVFP8 && !st.is_q) {
                uint8_t *dst = static_cast<uint8_t *>(a.k_cache) + (st.slot * a.hk + (head - a.hq)) * D;
                const float s = a.k_scale, rcp = 1.0f / s;
                if (scale_is_fast(s)) {
                    *reinterpret_cast<u32x2 *>(dst + c0(sub)) = quantize_chunk<T, true>(oa, s, rcp);
                    *reinterpret_cast<u32x2 *>(dst + c1(sub)) = quantize_chunk<T, true>(ob, s, rcp);
                } else {
                    *reinterpret_cast<u32x2 *>(dst + c0(sub)) = quantize_chunk<T, false>(oa, s, rcp);
                    *reinterpret_cast<u32x2 *>(dst + c1(sub)) = quantize_chunk<T, false>(ob, s, rcp);
                }
            } else {
                // q_out row or (16-bit) K cache row of the slot: one store sequence, destination chosen per lane
                uint16_t *dst = st.is_q ? static_cast<uint16_t *>(a.q_out) + ((int64_t)st.t * a.hq + head) * D
                                        : static_cast<uint16_t *>(a.k_cache) + (st.slot * a.hk + (head - a.hq)) * D;
                *reinterpret_cast<u32x4 *>(dst + c0(sub)) = oa;
                *reinterpret_cast<u32x4 *>(dst + c1(sub)) = ob;
            }
        }

        if constexpr (SETKV) {
            // V: copied (16-bit cache) or quantised (fp8 cache), chunk by chunk
            const int v_chunks = a.hv * (D / 8), v_first = st.u * 64 + lane;
            const int stride = a.units_per_token * 64;
            const float s = a.v_scale, rcp = 1.0f / s;
            const bool fast = scale_is_fast(s);
            u32x4 vchunk = st.vchunk;
            for (int c = v_first; slot_ok && c < v_chunks; c += stride) {
                if (c != v_first)
                    vchunk = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(st.token_in + (int64_t)heads_qk * D + 8 * c));
                const int64_t off = st.slot * a.hv * D + 8 * (int64_t)c;
                if constexpr (!KVFP8) {
                    *reinterpret_cast<u32x4 *>(static_cast<uint16_t *>(a.v_cache) + off) = vchunk;
                } else {
                    *reinterpret_cast<u32x2 *>(static_cast<uint8_t *>(a.v_cache) + off) =
                        fast ? quantize_chunk<T, true>(vchunk, s, rcp) : quantize_chunk<T, false>(vchunk, s, rcp);
                }
            }
        }
    }
};

template <typename T, int D, bool NEOX, int AXES, bool SETKV, bool KVFP8>
__global__ void __launch_bounds__(512) rope_rms_kernel(const RopeArgs a) {
    using Unit = RopeUnit<T, D, NEOX, AXES, SETKV, KVFP8>;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t unit = blockIdx.x * (blockDim.x >> 6) + wave;
    if (unit >= a.total_units) return;
    const int lane = threadIdx.x & 63;
    UnitState st;
    Unit::issue_loads(a, unit, lane, st);
    Unit::issue_table_loads(a, lane, st);
    // Every load of the wave is in flight before the first use of any of them: without this fence the scheduler
    // moves arithmetic above later loads and the wave pays several memory round trips in a row.
    __builtin_amdgcn_sched_barrier(0);
    Unit::finish(a, lane, st);
}

// ---------------------------------------------------------------------------------------------------------------
// fp32 activations: the reference dispatches them through the same templates (src/ops/fused_rope.cpp:27-30, :108-111).
// A compatibility path, not a tuned one: one wave per (token, head), lane l owns rotation pairs l, l+64, ...;
// with a KV cache the V heads get waves of their own that copy or quantise.  Rounding to the activation type is the
// identity, so the oracle's sequence is plain fp32 arithmetic with every product rounded before the add.
template <int D, bool NEOX, int AXES, bool SETKV, bool KVFP8>
__global__ void __launch_bounds__(256) rope_rms_f32_kernel(const RopeArgs a) {
    constexpr int HALF = D / 2;
    constexpr int PPL = (HALF + 63) / 64;  // pairs per lane
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t unit = blockIdx.x * (blockDim.x >> 6) + wave;
    if (unit >= a.total_units) return;
    const int lane = threadIdx.x & 63;
    const uint32_t t = a.upt_magic ? __umulhi(unit, a.upt_magic) : unit;
    const int h = (int)(unit - t * a.units_per_token);  // head index inside the token's qkv row
    const int heads_qk = a.hq + a.hk, heads_all = heads_qk + a.hv;
    const float *src = static_cast<const float *>(a.qkv_in) + ((int64_t)t * heads_all + h) * D;

    if (h >= heads_qk) {  // a V head: only reached with a KV cache
        if constexpr (SETKV) {
            const int64_t slot = a.kv_loc[t];
            if (slot < 0) return;  // token without a cache slot
            const int64_t row = (slot * a.hv + (h - heads_qk)) * D;
            for (int e = lane; e < D; e += 64) {
                const float v = src[e];
                if constexpr (KVFP8) {
                    static_cast<uint8_t *>(a.v_cache)[row + e] =
                        (uint8_t)cvt4_e4m3fn(clamp_sym(v / a.v_scale, kE4M3Max), 0.f, 0.f, 0.f);
                } else {
                    static_cast<float *>(a.v_cache)[row + e] = v;
                }
            }
        }
        return;
    }

    const bool is_q = h < a.hq;
    const float *w = static_cast<const float *>(is_q ? a.qw : a.kw);
    float x1[PPL], x2[PPL];
    int i1[PPL], i2[PPL];
    bool live[PPL];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < PPL; ++k) {
        const int p = lane + 64 * k;
        live[k] = p < HALF;
        const int pc = live[k] ? p : 0;
        i1[k] = NEOX ? pc : 2 * pc;
        i2[k] = NEOX ? pc + HALF : 2 * pc + 1;
        x1[k] = live[k] ? src[i1[k]] : 0.f;
        x2[k] = live[k] ? src[i2[k]] : 0.f;
        ss = __builtin_fmaf(x1[k], x1[k], ss);
        ss = __builtin_fmaf(x2[k], x2[k], ss);
    }
    ss = wave_allreduce<SumOp>(ss);
    const float rstd = 1.0f / sqrtf(ss * (1.0f / D) + a.eps);

    const float *table = static_cast<const float *>(a.cos_sin);
    const int64_t p0 = a.positions[(int64_t)t * a.ps_token];
    int64_t p1 = p0, p2 = p0;
    if constexpr (AXES == 3) {
        p1 = a.positions[a.ps_axis + (int64_t)t * a.ps_token];
        p2 = a.positions[2 * a.ps_axis + (int64_t)t * a.ps_token];
    }
    float *dst;
    uint8_t *dst8 = nullptr;
    if constexpr (!SETKV) {
        dst = static_cast<float *>(a.qkv_out) + ((int64_t)t * heads_all + h) * D;
    } else if (is_q) {
        dst = static_cast<float *>(a.q_out) + ((int64_t)t * a.hq + h) * D;
    } else {
        const int64_t slot = a.kv_loc[t];
        if (slot < 0) return;  // token without a cache slot: nothing of a K head is kept
        const int64_t row = (slot * a.hk + (h - a.hq)) * D;
        dst = static_cast<float *>(a.k_cache) + row;          // used when the cache is fp32
        dst8 = static_cast<uint8_t *>(a.k_cache) + row;       // used when it is fp8
    }
#pragma unroll
    for (int k = 0; k < PPL; ++k) {
        if (!live[k]) continue;
        const int f = lane + 64 * k;  // rotary frequency of this pair
        int64_t pos = p0;
        if constexpr (AXES == 3) {
            const bool on1 = (a.axis1[f >> 5] >> (f & 31)) & 1u, on2 = (a.axis2[f >> 5] >> (f & 31)) & 1u;
            pos = on2 ? p2 : (on1 ? p1 : p0);
        }
        const float c = table[pos * D + f], s = table[pos * D + HALF + f];
        const float n1 = w[i1[k]] * (x1[k] * rstd), n2 = w[i2[k]] * (x2[k] * rstd);
        const float o1 = n1 * c - n2 * s, o2 = n2 * c + n1 * s;
        if (SETKV && KVFP8 && !is_q) {
            dst8[i1[k]] = (uint8_t)cvt4_e4m3fn(clamp_sym(o1 / a.k_scale, kE4M3Max), 0.f, 0.f, 0.f);
            dst8[i2[k]] = (uint8_t)cvt4_e4m3fn(clamp_sym(o2 / a.k_scale, kE4M3Max), 0.f, 0.f, 0.f);
        } else {
            dst[i1[k]] = o1;
            dst[i2[k]] = o2;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Two token streams with their own norm weights and per-token cos/sin rows, outputs concatenated along the token
// axis (reference: fused_rope_rms_2way, src/ops/fused_rope.cpp:168-227 -> src/impl/rope_rms_impl.h:612-857).
// Per batch entry there are four segments of heads, each a contiguous [tokens, heads, D] block:
//   0: q0 -> out_q[:, 0:T0]   1: k0 -> out_k[:, 0:T0]   2: q1 -> out_q[:, T0:T0+T1]   3: k1 -> out_k[:, T0:T0+T1]
// A wave takes 64/(D/16) consecutive heads of one segment (they may belong to several tokens, so the cos/sin row
// is chosen per lane); blockIdx.y is the batch entry.
struct TwoWayArgs {
    const void *in[4];     // q0, k0, q1, k1
    const void *w[4];      // w_q0, w_k0, w_q1, w_k1
    const void *cos_sin[2];
    void *out[2];          // out_q01, out_k01
    uint32_t unit_end[4];  // prefix sums of the segments' unit counts
    uint32_t rows[4];      // tokens * heads of each segment
    uint32_t heads[2];     // Hq, Hk
    uint32_t heads_magic[2];  // ceil(2^32 / heads), 0 for heads == 1
    int tokens0, tokens1;
    float eps;
};

template <typename T, int D, bool NEOX>
__global__ void __launch_bounds__(256) rope_rms_2way_kernel(const TwoWayArgs a) {
    constexpr int LPH = D / 16, HPW = 64 / LPH, HALF = D / 2;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t unit = blockIdx.x * (blockDim.x >> 6) + wave;
    if (unit >= a.unit_end[3]) return;
    const int seg = (unit >= a.unit_end[0]) + (unit >= a.unit_end[1]) + (unit >= a.unit_end[2]);  // wave-uniform
    const uint32_t unit_in_seg = unit - (seg ? a.unit_end[seg - 1] : 0u);
    const int kind = seg & 1, stream_id = seg >> 1;  // q|k, stream 0|1
    const uint32_t heads = a.heads[kind], rows = a.rows[seg];
    const int batch = blockIdx.y;

    const int lane = threadIdx.x & 63, sub = lane % LPH, hl = lane / LPH;
    const uint32_t row_raw = unit_in_seg * HPW + hl;
    const bool active = row_raw < rows;
    const uint32_t row = min(row_raw, rows - 1);  // (token, head) flattened inside the segment
    const uint32_t token = a.heads_magic[kind] ? __umulhi(row, a.heads_magic[kind]) : row;
    const uint32_t head = row - token * heads;

    const int c0 = 8 * sub, c1 = HALF + 8 * sub;
    const uint16_t *src = static_cast<const uint16_t *>(a.in[seg]) + ((int64_t)batch * rows + row) * D;
    const u32x4 xa = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + c0));
    const u32x4 xb = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + c1));
    const uint16_t *wsrc = static_cast<const uint16_t *>(a.w[seg]);
    const u32x4 wa = *reinterpret_cast<const u32x4 *>(wsrc + c0);
    const u32x4 wb = *reinterpret_cast<const u32x4 *>(wsrc + c1);
    const uint16_t *table = static_cast<const uint16_t *>(a.cos_sin[stream_id]) + (int64_t)token * D;
    const u32x4 cosv = load_trig<D, NEOX>(table, sub);
    const u32x4 sinv = load_trig<D, NEOX>(table + HALF, sub);
    __builtin_amdgcn_sched_barrier(0);

    u32x4 oa, ob;
    norm_rotate<T, D, NEOX>(xa, xb, wa, wb, cosv, sinv, a.eps, oa, ob);
    if (active) {
        const int64_t out_token = (int64_t)batch * (a.tokens0 + a.tokens1) + (stream_id ? a.tokens0 : 0) + token;
        uint16_t *dst = static_cast<uint16_t *>(a.out[kind]) + (out_token * heads + head) * D;
        *reinterpret_cast<u32x4 *>(dst + c0) = oa;
        *reinterpret_cast<u32x4 *>(dst + c1) = ob;
    }
}

// fp32 form of the two-stream op (the reference dispatches float here too: src/ops/fused_rope.cpp:197-200): one wave
// per (token, head) row of a segment, lane l owns rotation pairs l, l+64, ...; plain fp32 arithmetic, every product
// rounded before the add.  The host counts one unit per row for this kernel.
template <int D, bool NEOX>
__global__ void __launch_bounds__(256) rope_rms_2way_f32_kernel(const TwoWayArgs a) {
    constexpr int HALF = D / 2;
    constexpr int PPL = (HALF + 63) / 64;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t unit = blockIdx.x * (blockDim.x >> 6) + wave;
    if (unit >= a.unit_end[3]) return;
    const int seg = (unit >= a.unit_end[0]) + (unit >= a.unit_end[1]) + (unit >= a.unit_end[2]);
    const uint32_t row = unit - (seg ? a.unit_end[seg - 1] : 0u);
    const int kind = seg & 1, stream_id = seg >> 1;
    const uint32_t heads = a.heads[kind], rows = a.rows[seg];
    const int batch = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const uint32_t token = a.heads_magic[kind] ? __umulhi(row, a.heads_magic[kind]) : row;
    const uint32_t head = row - token * heads;

    const float *src = static_cast<const float *>(a.in[seg]) + ((int64_t)batch * rows + row) * D;
    const float *w = static_cast<const float *>(a.w[seg]);
    const float *table = static_cast<const float *>(a.cos_sin[stream_id]) + (int64_t)token * D;
    const int64_t out_token = (int64_t)batch * (a.tokens0 + a.tokens1) + (stream_id ? a.tokens0 : 0) + token;
    float *dst = static_cast<float *>(a.out[kind]) + (out_token * heads + head) * D;

    float x1[PPL], x2[PPL];
    int i1[PPL], i2[PPL];
    bool live[PPL];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < PPL; ++k) {
        const int p = lane + 64 * k;
        live[k] = p < HALF;
        const int pc = live[k] ? p : 0;
        i1[k] = NEOX ? pc : 2 * pc;
        i2[k] = NEOX ? pc + HALF : 2 * pc + 1;
        x1[k] = live[k] ? src[i1[k]] : 0.f;
        x2[k] = live[k] ? src[i2[k]] : 0.f;
        ss = __builtin_fmaf(x1[k], x1[k], ss);
        ss = __builtin_fmaf(x2[k], x2[k], ss);
    }
    ss = wave_allreduce<SumOp>(ss);
    const float rstd = 1.0f / sqrtf(ss * (1.0f / D) + a.eps);
#pragma unroll
    for (int k = 0; k < PPL; ++k) {
        if (!live[k]) continue;
        const int f = lane + 64 * k;
        const float c = table[f], s = table[HALF + f];
        const float n1 = w[i1[k]] * (x1[k] * rstd), n2 = w[i2[k]] * (x2[k] * rstd);
        dst[i1[k]] = n1 * c - n2 * s;
        dst[i2[k]] = n2 * c + n1 * s;
    }
}

template <typename T, int D>
int launch_2way(const TwoWayArgs &a, bool neox, unsigned batch, hipStream_t stream) {
    const dim3 grid((a.unit_end[3] + 3) / 4, batch);
    if (neox) rope_rms_2way_kernel<T, D, true><<<grid, 256, 0, stream>>>(a);
    else rope_rms_2way_kernel<T, D, false><<<grid, 256, 0, stream>>>(a);
    return hip_status(hipGetLastError());
}

template <int D>
int launch_2way_f32(const TwoWayArgs &a, bool neox, unsigned batch, hipStream_t stream) {
    const dim3 grid((a.unit_end[3] + 3) / 4, batch);
    if (neox) rope_rms_2way_f32_kernel<D, true><<<grid, 256, 0, stream>>>(a);
    else rope_rms_2way_f32_kernel<D, false><<<grid, 256, 0, stream>>>(a);
    return hip_status(hipGetLastError());
}

int launch_2way_f32_head_size(const TwoWayArgs &a, int64_t D, bool neox, unsigned batch, hipStream_t stream) {
    switch (D) {
        case 64: return launch_2way_f32<64>(a, neox, batch, stream);
        case 128: return launch_2way_f32<128>(a, neox, batch, stream);
        case 256: return launch_2way_f32<256>(a, neox, batch, stream);
        default: return GPUK_ERR_UNSUPPORTED;
    }
}

template <typename T>
int launch_2way_head_size(const TwoWayArgs &a, int64_t D, bool neox, unsigned batch, hipStream_t stream) {
    switch (D) {
        case 64: return launch_2way<T, 64>(a, neox, batch, stream);
        case 128: return launch_2way<T, 128>(a, neox, batch, stream);
        case 256: return launch_2way<T, 256>(a, neox, batch, stream);
        default: return GPUK_ERR_UNSUPPORTED;
    }
}

int g_block_threads = 0;    // 0 = default

template <typename T, int D, bool NEOX, int AXES, bool SETKV, bool KVFP8>
int launch_one(const RopeArgs &a, hipStream_t stream) {
    const int threads = g_block_threads ? g_block_threads : 256;
    const uint32_t units_per_block = threads / 64;
    const uint32_t blocks = (a.total_units + units_per_block - 1) / units_per_block;
    rope_rms_kernel<T, D, NEOX, AXES, SETKV, KVFP8><<<blocks, threads, 0, stream>>>(a);
    return hip_status(hipGetLastError());
}

template <typename T, int D, bool NEOX, int AXES>
int launch_mode(const RopeArgs &a, bool set_kv, bool kv_fp8, hipStream_t stream) {
    if (!set_kv) return launch_one<T, D, NEOX, AXES, false, false>(a, stream);
    if (kv_fp8) return launch_one<T, D, NEOX, AXES, true, true>(a, stream);
    return launch_one<T, D, NEOX, AXES, true, false>(a, stream);
}

template <typename T, int D>
int launch_style(const RopeArgs &a, bool neox, int n_axes, bool set_kv, bool kv_fp8, hipStream_t stream) {
    if (neox) {
        return n_axes == 3 ? launch_mode<T, D, true, 3>(a, set_kv, kv_fp8, stream)
                           : launch_mode<T, D, true, 1>(a, set_kv, kv_fp8, stream);
    }
    return n_axes == 3 ? launch_mode<T, D, false, 3>(a, set_kv, kv_fp8, stream)
                       : launch_mode<T, D, false, 1>(a, set_kv, kv_fp8, stream);
}

template <int D, bool NEOX, int AXES>
int launch_f32_mode(const RopeArgs &a, bool set_kv, bool kv_fp8, hipStream_t stream) {
    const uint32_t blocks = (a.total_units + 3) / 4;
    if (!set_kv) rope_rms_f32_kernel<D, NEOX, AXES, false, false><<<blocks, 256, 0, stream>>>(a);
    else if (kv_fp8) rope_rms_f32_kernel<D, NEOX, AXES, true, true><<<blocks, 256, 0, stream>>>(a);
    else rope_rms_f32_kernel<D, NEOX, AXES, true, false><<<blocks, 256, 0, stream>>>(a);
    return hip_status(hipGetLastError());
}

template <int D>
int launch_f32_style(const RopeArgs &a, bool neox, int n_axes, bool set_kv, bool kv_fp8, hipStream_t stream) {
    if (neox) {
        return n_axes == 3 ? launch_f32_mode<D, true, 3>(a, set_kv, kv_fp8, stream)
                           : launch_f32_mode<D, true, 1>(a, set_kv, kv_fp8, stream);
    }
    return n_axes == 3 ? launch_f32_mode<D, false, 3>(a, set_kv, kv_fp8, stream)
                       : launch_f32_mode<D, false, 1>(a, set_kv, kv_fp8, stream);
}

int launch_f32_head_size(const RopeArgs &a, int64_t head_size, bool neox, int n_axes, bool set_kv, bool kv_fp8,
                         hipStream_t stream) {
    switch (head_size) {
        case 64: return launch_f32_style<64>(a, neox, n_axes, set_kv, kv_fp8, stream);
        case 128: return launch_f32_style<128>(a, neox, n_axes, set_kv, kv_fp8, stream);
        case 256: return launch_f32_style<256>(a, neox, n_axes, set_kv, kv_fp8, stream);
        default: return GPUK_ERR_UNSUPPORTED;
    }
}

template <typename T>
int launch_head_size(const RopeArgs &a, int64_t head_size, bool neox, int n_axes, bool set_kv, bool kv_fp8,
                     hipStream_t stream) {
    switch (head_size) {
        case 64: return launch_style<T, 64>(a, neox, n_axes, set_kv, kv_fp8, stream);
        case 128: return launch_style<T, 128>(a, neox, n_axes, set_kv, kv_fp8, stream);
        case 256: return launch_style<T, 256>(a, neox, n_axes, set_kv, kv_fp8, stream);
        default: return GPUK_ERR_UNSUPPORTED;
    }
}

// Frequency -> axis map of mRoPE as two bitmaps.  Interleaved (rope_rms_impl.h:127-138): axis a = f mod 3
// when a >= 1 and f < section[a]*3, else axis 0.  Chunked (:139-151): first a with f < section[0..a] summed.
void build_axis_bitmaps(const int64_t *section, bool interleaved, int half, uint32_t *axis1, uint32_t *axis2) {
    for (int i = 0; i < 4; ++i) axis1[i] = axis2[i] = 0;
    for (int f = 0; f < half; ++f) {
        int axis;
        if (interleaved) {
            const int m = f % 3;
            axis = (m >= 1 && f < section[m] * 3) ? m : 0;
        } else {
            axis = f < section[0] ? 0 : (f < section[0] + section[1] ? 1 : 2);
        }
        if (axis == 1) axis1[f >> 5] |= 1u << (f & 31);
        if (axis == 2) axis2[f >> 5] |= 1u << (f & 31);
    }
}

int rope_common(const void *qkv_in, void *qkv_out, const void *qw, const void *kw, const void *cos_sin,
                const int64_t *positions, int64_t ps_axis, int64_t ps_token, int n_axes, int64_t T, int64_t hq,
                int64_t hk, int64_t hv, int64_t D, int neox, const int64_t *section, int interleaved, float eps,
                int dtype, bool set_kv, void *q_out, void *k_cache, void *v_cache, const int64_t *kv_loc,
                float k_scale, float v_scale, int kv_dtype, void *stream) {
    if (T < 0 || hq < 0 || hk < 0 || hv < 0) return GPUK_ERR_INVALID_ARG;
    if (n_axes != 1 && n_axes != 3) return GPUK_ERR_INVALID_ARG;
    if (D != 64 && D != 128 && D != 256) return GPUK_ERR_UNSUPPORTED;
    if (dtype != GPUK_DTYPE_BF16 && dtype != GPUK_DTYPE_FP16 && dtype != GPUK_DTYPE_F32) return GPUK_ERR_UNSUPPORTED;
    if (set_kv && kv_dtype != GPUK_KV_SAME && kv_dtype != GPUK_KV_E4M3FN) return GPUK_ERR_UNSUPPORTED;
    if (hq > 0x7fffff || hk > 0x7fffff || hv > 0x7fffff) return GPUK_ERR_UNSUPPORTED;
    RopeArgs a{};
    if (n_axes == 3) {
        if (!section) return GPUK_ERR_INVALID_ARG;
        if (section[0] < 0 || section[1] < 0 || section[2] < 0 || section[0] + section[1] + section[2] != D / 2)
            return GPUK_ERR_INVALID_ARG;
        build_axis_bitmaps(section, interleaved != 0, (int)(D / 2), a.axis1, a.axis2);
    }
    if (T == 0 || hq + hk + (set_kv ? hv : 0) == 0) return GPUK_OK;
    if (!qkv_in || !qw || !kw || !cos_sin || !positions) return GPUK_ERR_INVALID_ARG;
    if (!aligned16(qkv_in) || !aligned16(qw) || !aligned16(kw) || !aligned16(cos_sin)) return GPUK_ERR_MISALIGNED;
    const bool kv_fp8 = set_kv && kv_dtype == GPUK_KV_E4M3FN;
    if (set_kv) {
        // a buffer may be absent (or empty) when no head of its kind exists
        if ((hq > 0 && !q_out) || (hk > 0 && !k_cache) || (hv > 0 && !v_cache) || !kv_loc) return GPUK_ERR_INVALID_ARG;
        if (!aligned16(q_out) || !aligned16(k_cache) || !aligned16(v_cache)) return GPUK_ERR_MISALIGNED;
        if (kv_fp8 && !(k_scale > 0.f && v_scale > 0.f)) return GPUK_ERR_INVALID_ARG;
    }
    // one wave per group of 64/(D/16) consecutive Q/K heads of a token; with a KV cache and no Q/K heads at all the
    // token still gets the waves its V row needs
    const int64_t hpw = 64 / (D / 16);
    int64_t upt = (hq + hk + hpw - 1) / hpw;
    if (upt == 0) upt = (hv * (D / 8) + 63) / 64;
    if (hq + hk == 0) return GPUK_ERR_UNSUPPORTED;  // a qkv row without Q and K heads has nothing to rotate
    if (dtype == GPUK_DTYPE_F32) upt = hq + hk + (set_kv ? hv : 0);  // the fp32 path: one wave per head
    // mulhi(unit, ceil(2^32/upt)) equals unit / upt while unit * upt < 2^32
    if (upt * T >= 0x7fffffffLL || upt * T * upt >= (1LL << 32)) return GPUK_ERR_UNSUPPORTED;
    a.qkv_in = qkv_in;
    a.qkv_out = qkv_out;
    a.qw = qw;
    a.kw = kw;
    a.cos_sin = cos_sin;
    a.positions = positions;
    a.ps_axis = ps_axis;
    a.ps_token = ps_token;
    a.q_out = q_out;
    a.k_cache = k_cache;
    a.v_cache = v_cache;
    a.kv_loc = kv_loc;
    a.total_units = (uint32_t)(upt * T);
    a.units_per_token = (uint32_t)upt;
    a.upt_magic = upt == 1 ? 0u : (uint32_t)(((1ull << 32) + (uint64_t)upt - 1) / (uint64_t)upt);
    a.hq = (int)hq;
    a.hk = (int)hk;
    a.hv = (int)hv;
    a.eps = eps;
    a.k_scale = k_scale;
    a.v_scale = v_scale;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == GPUK_DTYPE_F32) return launch_f32_head_size(a, D, neox != 0, n_axes, set_kv, kv_fp8, s);
    if (dtype == GPUK_DTYPE_BF16) return launch_head_size<BF16>(a, D, neox != 0, n_axes, set_kv, kv_fp8, s);
    return launch_head_size<FP16>(a, D, neox != 0, n_axes, set_kv, kv_fp8, s);
}

}  // namespace

void set_rope_tuning(int key, int value) {
    if (key == 0) g_block_threads = value;
}

}  // namespace gpuk

extern "C" int gpuk_rope_rms(void *qkv, const void *qw, const void *kw, const void *cos_sin, const int64_t *positions,
                             int64_t pos_stride_axis, int64_t pos_stride_token, int n_axes, int64_t num_tokens,
                             int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v, int64_t head_size,
                             int is_neox_style, const int64_t *mrope_section, int is_interleaved, float eps,
                             int dtype, void *stream) {
    return gpuk::rope_common(qkv, qkv, qw, kw, cos_sin, positions, pos_stride_axis, pos_stride_token, n_axes,
                             num_tokens, num_heads_q, num_heads_k, num_heads_v, head_size, is_neox_style,
                             mrope_section, is_interleaved, eps, dtype, false, nullptr, nullptr, nullptr, nullptr,
                             1.f, 1.f, GPUK_KV_SAME, stream);
}

extern "C" int gpuk_rope_rms_set_kv(const void *qkv, const void *qw, const void *kw, const void *cos_sin,
                                    const int64_t *positions, int64_t pos_stride_axis, int64_t pos_stride_token,
                                    int n_axes, int64_t num_tokens, int64_t num_heads_q, int64_t num_heads_k,
                                    int64_t num_heads_v, int64_t head_size, int is_neox_style,
                                    const int64_t *mrope_section, int is_interleaved, float eps, int dtype,
                                    void *q_out, void *k_cache, void *v_cache, const int64_t *kv_loc, float k_scale,
                                    float v_scale, int kv_dtype, void *stream) {
    return gpuk::rope_common(qkv, nullptr, qw, kw, cos_sin, positions, pos_stride_axis, pos_stride_token, n_axes,
                             num_tokens, num_heads_q, num_heads_k, num_heads_v, head_size, is_neox_style,
                             mrope_section, is_interleaved, eps, dtype, true, q_out, k_cache, v_cache, kv_loc,
                             k_scale, v_scale, kv_dtype, stream);
}

extern "C" int gpuk_rope_rms_2way(const void *q0, const void *k0, const void *q1, const void *k1, const void *w_q0,
                                  const void *w_k0, const void *w_q1, const void *w_k1, const void *cos_sin0,
                                  const void *cos_sin1, int64_t batch_size, int64_t num_tokens0, int64_t num_tokens1,
                                  int64_t num_heads_q, int64_t num_heads_k, int64_t head_size, int is_interleaved,
                                  float eps, int dtype, void *out_q01, void *out_k01, void *stream) {
    using namespace gpuk;
    if (batch_size < 0 || num_tokens0 < 0 || num_tokens1 < 0 || num_heads_q < 0 || num_heads_k < 0) return GPUK_ERR_INVALID_ARG;
    if (head_size != 64 && head_size != 128 && head_size != 256) return GPUK_ERR_UNSUPPORTED;
    if (dtype != GPUK_DTYPE_BF16 && dtype != GPUK_DTYPE_FP16 && dtype != GPUK_DTYPE_F32) return GPUK_ERR_UNSUPPORTED;
    if (batch_size > 65535) return GPUK_ERR_UNSUPPORTED;  // grid.y
    const int64_t hpw = dtype == GPUK_DTYPE_F32 ? 1 : 64 / (head_size / 16);  // rows (heads) per wave
    const int64_t rows[4] = {num_tokens0 * num_heads_q, num_tokens0 * num_heads_k, num_tokens1 * num_heads_q,
                             num_tokens1 * num_heads_k};
    const void *ins[4] = {q0, k0, q1, k1};
    const void *ws[4] = {w_q0, w_k0, w_q1, w_k1};
    TwoWayArgs a{};
    int64_t end = 0;
    for (int s = 0; s < 4; ++s) {
        if (rows[s] >= (1LL << 31)) return GPUK_ERR_UNSUPPORTED;
        if (rows[s] > 0 && (!ins[s] || !ws[s] || !aligned16(ins[s]) || !aligned16(ws[s])))
            return !ins[s] || !ws[s] ? GPUK_ERR_INVALID_ARG : GPUK_ERR_MISALIGNED;
        end += (rows[s] + hpw - 1) / hpw;
        a.in[s] = ins[s];
        a.w[s] = ws[s];
        a.unit_end[s] = (uint32_t)end;
        a.rows[s] = (uint32_t)rows[s];
    }
    if (end >= (1LL << 31)) return GPUK_ERR_UNSUPPORTED;
    if (batch_size == 0 || end == 0) return GPUK_OK;
    if ((num_tokens0 > 0 && !cos_sin0) || (num_tokens1 > 0 && !cos_sin1)) return GPUK_ERR_INVALID_ARG;
    if ((rows[0] + rows[2] > 0 && !out_q01) || (rows[1] + rows[3] > 0 && !out_k01)) return GPUK_ERR_INVALID_ARG;
    if (!aligned16(cos_sin0) || !aligned16(cos_sin1) || !aligned16(out_q01) || !aligned16(out_k01)) return GPUK_ERR_MISALIGNED;
    a.cos_sin[0] = cos_sin0;
    a.cos_sin[1] = cos_sin1;
    a.out[0] = out_q01;
    a.out[1] = out_k01;
    const int64_t heads[2] = {num_heads_q, num_heads_k};
    for (int k = 0; k < 2; ++k) {
        a.heads[k] = (uint32_t)heads[k];
        // mulhi(row, ceil(2^32/heads)) == row / heads while row * heads < 2^32
        if (heads[k] > 1 && std::max(rows[k], rows[k + 2]) * heads[k] >= (1LL << 32)) return GPUK_ERR_UNSUPPORTED;
        a.heads_magic[k] = heads[k] <= 1 ? 0u : (uint32_t)(((1ull << 32) + (uint64_t)heads[k] - 1) / (uint64_t)heads[k]);
    }
    a.tokens0 = (int)num_tokens0;
    a.tokens1 = (int)num_tokens1;
    a.eps = eps;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool neox = !is_interleaved;  // reference: fused_rope.cpp:168-227 dispatches the NeoX kernel when !is_interleaved
    if (dtype == GPUK_DTYPE_F32) return launch_2way_f32_head_size(a, head_size, neox, (unsigned)batch_size, s);
    if (dtype == GPUK_DTYPE_BF16) return launch_2way_head_size<BF16>(a, head_size, neox, (unsigned)batch_size, s);
    return launch_2way_head_size<FP16>(a, head_size, neox, (unsigned)batch_size, s);
}
