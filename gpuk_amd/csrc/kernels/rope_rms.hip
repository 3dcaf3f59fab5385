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
    const int64_t *positions;
    const int64_t *kv_loc;
    // one wave per unit = (token, group of heads); units_per_token = ceil((hq + hk) / heads per wave)
    uint32_t total_units, units_per_token;
    uint32_t upt_magic;  // ceil(2^32 / units_per_token), or 0 when units_per_token is 1: unit / units_per_token is
                         // mulhi(unit, magic) for every unit the host admits
    int hq, hk, hv;
    int64_t ps_axis, ps_token;
    void *qkv_out;  // == qkv_in for the in-place form, unused for set_kv
    const void *qw, *kw, *cos_sin;
    void *q_out, *k_cache, *v_cache;
    float eps, k_scale, v_scale;
    // mRoPE: bit f of axis1 / axis2 set when rotary frequency f takes its position from axis 1 / 2
    uint32_t axis1[4], axis2[4];
    uint32_t num_tokens;
    uint32_t stream_rows;  // 1: q_out / K rows / in-place rows are stored past the L2 (calls that move more than a few MB)
    uint32_t merge_rows;   // mRoPE: every aligned group of 8 frequencies takes one axis: each lane loads from that axis's row
    uint32_t gate;         // ticks of 10 ns after a wave's entry before which it stores nothing (0 = no gate)
};

// A pointer read from the argument block by hand is a generic one to the compiler; these say what it points at, so
// that the accesses through it are global (not flat) ones, and scalar ones where the address is the same in every lane.
template <typename P>
__device__ __forceinline__ P *as_global(P *p) {
    return (P *)(__attribute__((address_space(1))) P *)p;
}
template <typename P>
__device__ __forceinline__ P load_unchanging(const P *p) {  // memory no kernel of the launch writes
    return *(const __attribute__((address_space(4))) P *)p;
}

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
// Word f / 32 of a frequency bitmap for a lane-dependent f.  The bitmaps are kernel arguments: indexed per lane they
// would be fetched from the argument segment with a vector load, one more memory round trip between a wave's
// positions and its table loads.  The words are pinned in scalar registers instead and picked with selects.
template <int D>
__device__ __forceinline__ uint32_t bitmap_word(const uint32_t (&bitmap)[4], int f) {
    uint32_t w0 = bitmap[0], w1 = bitmap[1], w2 = bitmap[2], w3 = bitmap[3];
    if constexpr (D / 2 <= 32) {
        asm("" : "+s"(w0));
        return w0;
    } else if constexpr (D / 2 <= 64) {
        asm("" : "+s"(w0), "+s"(w1));
        return f < 32 ? w0 : w1;
    } else {
        asm("" : "+s"(w0), "+s"(w1), "+s"(w2), "+s"(w3));
        return f < 64 ? (f < 32 ? w0 : w1) : (f < 96 ? w2 : w3);
    }
}
template <int D, bool NEOX>
__device__ __forceinline__ uint32_t trig_bits(const uint32_t (&bitmap)[4], int sub) {
    if constexpr (NEOX) {
        const int f = 8 * sub;
        return (bitmap_word<D>(bitmap, f) >> (f & 31)) & 0xffu;
    } else {
        const int f0 = 4 * sub, f1 = D / 4 + 4 * sub;
        return ((bitmap_word<D>(bitmap, f0) >> (f0 & 31)) & 0xfu) | (((bitmap_word<D>(bitmap, f1) >> (f1 & 31)) & 0xfu) << 4);
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
    const float rstd = rsqrt_two_roundings(sumsq * (1.0f / D) + eps);  // D is a power of two: the product is exact

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

// A pair of 16-byte stores OFFSET bytes apart, streamed past the L2 (nt) or left to it.  The streaming form is
// written in assembly: as two arms of a run-time choice, the compiler merges a non-temporal and a plain store into
// one plain store.
template <int OFFSET>
__device__ __forceinline__ void store_pair(void *p, const u32x4 &a, const u32x4 &b, bool nt) {
    if (nt) {
        // the trailing s_nop: a store wider than 64 bits needs one wait state before its data registers may be
        // overwritten, and the compiler's hazard pass does not look inside an asm statement
        asm volatile("global_store_dwordx4 %0, %1, off nt\n\tglobal_store_dwordx4 %0, %2, off offset:%3 nt\n\ts_nop 0" ::"v"(p), "v"(a), "v"(b), "n"(OFFSET) : "memory");
    } else {
        *reinterpret_cast<u32x4 *>(p) = a;
        *reinterpret_cast<u32x4 *>(static_cast<char *>(p) + OFFSET) = b;
    }
}
// What one wave keeps about one unit (= one group of 64/(D/16) consecutive Q/K heads of one token, plus its share
// of the token's V row) between issuing the unit's loads and finishing it.
struct UnitState {
    uint32_t t, u;
    int head;
    bool active, is_q;
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

    // Issues the loads of the unit that need nothing but the kernel's leading parameters (which a wave finds in its
    // registers): the activations, the unit's share of the V row, the position(s).  Nothing is waited for.
    static __device__ __forceinline__ void issue_early_loads(const RopeArgs &a, uint32_t unit, int lane, UnitState &st) {
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
        // streamed, in place too (the lines are written a moment later, but past the L2: keeping them there cost 2-17 %
        // from 512 tokens on once the stores were streamed)
        st.xa = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + c0(sub)));
        st.xb = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + c1(sub)));

        // this wave's share of the token's V row: chunk u*64 + lane (and further strides of units_per_token*64)
        if constexpr (SETKV) {
            const int v_first = st.u * 64 + lane;
            if (v_first < a.hv * (D / 8))
                st.vchunk = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(st.token_in + (int64_t)heads_qk * D + 8 * v_first));
        }
        // (read as memory that no kernel of the launch writes: scalar loads whatever else the kernel contains)
        st.p0 = load_unchanging(a.positions + (int64_t)st.t * a.ps_token);
        if constexpr (AXES == 3) {
            st.p1 = load_unchanging(a.positions + a.ps_axis + (int64_t)st.t * a.ps_token);
            st.p2 = load_unchanging(a.positions + 2 * a.ps_axis + (int64_t)st.t * a.ps_token);
        }
    }

    // The loads reached through pointers of the argument block: the token's cache slot and the norm weights.
    static __device__ __forceinline__ void issue_late_loads(const RopeArgs &a, int lane, UnitState &st) {
        // With three position axes both weight pointers are pinned in scalar registers: the select between the two
        // kernel arguments is otherwise turned into a per-lane load of the pointer from the argument segment in those
        // instantiations, and the weights wait for that round trip.  The one-axis instantiations keep the pointers in
        // scalar registers by themselves and lose 2-7 % to the pin.
        const void *qw = a.qw, *kw = a.kw;
        if constexpr (AXES == 3) asm("" : "+s"(qw), "+s"(kw));
        const int sub = lane % LPH;
        if constexpr (SETKV) st.slot = load_unchanging(a.kv_loc + st.t);
        typedef const __attribute__((address_space(1))) u32x4 *GlobalChunk;
        const uint16_t *wsrc = static_cast<const uint16_t *>(st.is_q ? qw : kw);
        st.wa = *(GlobalChunk)(wsrc + c0(sub));
        st.wb = *(GlobalChunk)(wsrc + c1(sub));
    }

    // The cos/sin loads, whose addresses wait for the positions.
    static __device__ __forceinline__ void issue_table_loads(const RopeArgs &a, int lane, UnitState &st) {
        const int sub = lane % LPH;
        const uint16_t *table = static_cast<const uint16_t *>(a.cos_sin);
        const int64_t p0 = st.p0;
        if constexpr (AXES == 3) {
            const int64_t p1 = st.p1, p2 = st.p2;
            if (a.merge_rows && (p1 != p0 || p2 != p0)) {
                // every aligned group of 8 frequencies takes one axis: each lane reads its pieces from that axis's row
                const uint32_t b1 = trig_bits<D, NEOX>(a.axis1, sub), b2 = trig_bits<D, NEOX>(a.axis2, sub);
                const int64_t pa = (b2 & 1u) ? p2 : ((b1 & 1u) ? p1 : p0);
                if constexpr (NEOX) {
                    st.cosv = load_trig<D, NEOX>(table + pa * D, sub);
                    st.sinv = load_trig<D, NEOX>(table + pa * D + HALF, sub);
                } else {
                    const int64_t pb = (b2 & 16u) ? p2 : ((b1 & 16u) ? p1 : p0);
                    const u32x2 cl = *reinterpret_cast<const u32x2 *>(table + pa * D + 4 * sub);
                    const u32x2 ch = *reinterpret_cast<const u32x2 *>(table + pb * D + D / 4 + 4 * sub);
                    const u32x2 sl = *reinterpret_cast<const u32x2 *>(table + pa * D + HALF + 4 * sub);
                    const u32x2 sh = *reinterpret_cast<const u32x2 *>(table + pb * D + HALF + D / 4 + 4 * sub);
                    st.cosv = u32x4{cl[0], cl[1], ch[0], ch[1]};
                    st.sinv = u32x4{sl[0], sl[1], sh[0], sh[1]};
                }
                return;
            }
        }
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

    // Norm, rotation and all stores of the unit.  GATED: no store before a.gate ticks after `entry`, the wave's entry
    // time (a template parameter: as a run-time choice the check cost the launches without a gate 2-6 %).
    template <bool GATED>
    static __device__ __forceinline__ void finish(const RopeArgs &a, int lane, UnitState &st, uint64_t entry) {
        const int sub = lane % LPH;
        const int heads_qk = a.hq + a.hk, heads_all = heads_qk + a.hv;
        const u32x4 &xa = st.xa, &xb = st.xb, &wa = st.wa, &wb = st.wb, &cosv = st.cosv, &sinv = st.sinv;

        u32x4 oa, ob;
        norm_rotate<T, D, NEOX>(xa, xb, wa, wb, cosv, sinv, a.eps, oa, ob);
        // batches whose waves are all resident at once: no store before the launch's reads are through (the rotated
        // rows are pinned down ahead of the wait: nothing ties the arithmetic to the clock, and the compiler
        // otherwise moves it behind the wait)
        if constexpr (GATED) {
            asm volatile("" ::"v"(oa), "v"(ob));
            while (__builtin_amdgcn_s_memrealtime() < entry + a.gate) __builtin_amdgcn_s_sleep(1);
        }

        // A negative slot marks a token that has no place in the cache (padding in a fixed-size decode batch): its Q
        // row is still produced, its K and V rows are dropped.  The reference would write out of bounds.
        const bool slot_ok = !SETKV || st.slot >= 0;  // wave-uniform
        const int head = st.head;
        if (st.active && (st.is_q || slot_ok)) {
            if constexpr (!SETKV) {
                uint16_t *dst = static_cast<uint16_t *>(a.qkv_out) + ((int64_t)st.t * heads_all + head) * D;
                store_pair<HALF * 2>(dst + c0(sub), oa, ob, a.stream_rows != 0);
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
                store_pair<HALF * 2>(dst + c0(sub), oa, ob, a.stream_rows != 0);
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

// What a wave needs to ask for its activations and its position(s) comes as 14 dwords of leading scalar parameters,
// which are handed to the wave in scalar registers at launch (-amdgpu-kernarg-preload-count=14): those requests
// leave without a round trip for the argument block, which under load costs a wave of this kernel a third of its
// life; the block (weights, table, outputs, slots) is fetched beside the position, and everything that depends on
// either is asked for one round trip after entry.  hv_and_waves: hv in bits 0-23, log2 of the waves per workgroup above.
// (The three-axis instantiations take 66 registers per lane, one wave short of the eight a SIMD can hold; held to 64
// with amdgpu_waves_per_eu they fit without spilling and run 1-4 % slower: 26.9 against 26.6 us at 8192 tokens of
// 28+4+4 heads, 51.3 against 49.1 at 16384.)
// The leading parameters of the kernel below as the argument segment lays them out; the block follows them.
struct UnitKernelLead {
    const void *qkv_in;
    const int64_t *positions;
    uint32_t total_units, units_per_token, upt_magic;
    int hq, hk;
    uint32_t hv_and_waves;
    int64_t ps_token, ps_axis;
};
static_assert(sizeof(UnitKernelLead) == 56 && sizeof(UnitKernelLead) % alignof(RopeArgs) == 0, "offset of the block");

template <typename T, int D, bool NEOX, int AXES, bool SETKV, bool KVFP8, bool GATED>
__global__ void __launch_bounds__(512)
rope_rms_kernel(const void *qkv_in, const int64_t *positions, uint32_t total_units, uint32_t units_per_token,
                uint32_t upt_magic, int hq, int hk, uint32_t hv_and_waves, int64_t ps_token, int64_t ps_axis,
                const RopeArgs rest) {
    using Unit = RopeUnit<T, D, NEOX, AXES, SETKV, KVFP8>;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t unit = (blockIdx.x << (hv_and_waves >> 24)) + wave;
    if (unit >= total_units) return;
    const uint64_t entry = GATED ? __builtin_amdgcn_s_memrealtime() : 0;
    RopeArgs a;
    a.qkv_in = qkv_in;
    a.positions = positions;
    a.total_units = total_units;
    a.units_per_token = units_per_token;
    a.upt_magic = upt_magic;
    a.hq = hq;
    a.hk = hk;
    a.hv = (int)(hv_and_waves & 0xffffffu);
    a.ps_token = ps_token;
    a.ps_axis = ps_axis;
    GPUK_STAMPS_BEGIN();  // profiling build only
    const int lane = threadIdx.x & 63;
    UnitState st;
    Unit::issue_early_loads(a, unit, lane, st);
    // The rest of the arguments is fetched from the argument block only now, behind the requests above.  (Left to
    // the compiler the fetch is the kernel's first instruction, and the first vector load then waits for it: in one
    // instantiation for a register the fetch is about to overwrite, in another for the pinned weight pointers.)
    // (`rest` is read through the argument segment's own address: taking the parameter's address would have the
    // whole block copied to the stack.  It follows the 14 leading dwords.)
    typedef const __attribute__((address_space(4))) RopeArgs *BlockPtr;
    BlockPtr block = (BlockPtr)((const __attribute__((address_space(4))) char *)__builtin_amdgcn_kernarg_segment_ptr() +
                                sizeof(UnitKernelLead));
    asm volatile("" : "+s"(block));
    a.kv_loc = as_global(block->kv_loc);
    a.qkv_out = as_global(block->qkv_out);
    a.qw = as_global(block->qw);
    a.kw = as_global(block->kw);
    a.cos_sin = as_global(block->cos_sin);
    a.q_out = as_global(block->q_out);
    a.k_cache = as_global(block->k_cache);
    a.v_cache = as_global(block->v_cache);
    a.eps = block->eps;
    a.k_scale = block->k_scale;
    a.v_scale = block->v_scale;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a.axis1[i] = block->axis1[i];
        a.axis2[i] = block->axis2[i];
    }
    a.stream_rows = block->stream_rows;
    a.merge_rows = block->merge_rows;
    a.gate = block->gate;
    // ... all of it in one go (the compiler otherwise fetches each field where it is first used, the output pointers
    // after the arithmetic, and the wave waits for the scalar cache once more before it can store)
    asm volatile("" ::"s"(a.kv_loc), "s"(a.qkv_out), "s"(a.qw), "s"(a.kw), "s"(a.cos_sin), "s"(a.q_out), "s"(a.k_cache),
                 "s"(a.v_cache), "s"(a.eps), "s"(a.k_scale), "s"(a.v_scale), "s"(a.stream_rows), "s"(a.merge_rows),
                 "s"(a.gate));
    Unit::issue_late_loads(a, lane, st);
    GPUK_STAMP(1);  // activations, weights, position and slot requested
    Unit::issue_table_loads(a, lane, st);
    // (the slot is asked for here and not where the rows are stored, for the same reason)
    if constexpr (SETKV) asm volatile("" ::"s"((uint32_t)st.slot), "s"((uint32_t)(st.slot >> 32)));
    GPUK_STAMP(2);  // position known, cos/sin requested
    // Every load of the wave is in flight before the first use of any of them: without this fence the scheduler
    // moves arithmetic above later loads and the wave pays several memory round trips in a row.
    __builtin_amdgcn_sched_barrier(0);
    GPUK_STAMP_DRAINED(3);  // everything landed
    Unit::template finish<GATED>(a, lane, st, entry);
    GPUK_STAMP(4);          // rows stored (issued)
    GPUK_STAMP_DRAINED(5);  // ... and acknowledged
    GPUK_STAMPS_WRITE(unit);
}

// ---------------------------------------------------------------------------------------------------------------
// One wave per token -- or per two tokens --, for batches that the chip holds in one round (a cache write, up to
// kTokenWaveCapacity waves).  The memory system serves reads and writes one direction at a time, and a kernel of this
// size (tens of MB each way, 15-25 us) spends a fifth of its time paying for the mix; here the launch is arranged so
// that there is hardly any: every wave is resident from the start and asks for everything it will read -- all UPT
// units of its token, its token's V row, the weights, then the table row -- before it computes anything, the
// rotated rows replace the activations in the wave's registers, and no store is issued before `gate` ticks (10 ns)
// after the wave's entry, the time the launch's reads take at the read-only rate (the host computes it from the
// bytes of the call).  The chip thus reads for the first half of the launch and writes for the second.
// TWO: the wave takes a second token (the one num_waves further on), whose activations and V row travel from global
// memory straight into the wave's 9 KB of LDS (global_load_lds_dwordx4: no register is the destination) during the
// same read phase, and are taken into the first token's registers once that one is stored.  Registers and LDS
// together hold 8192 tokens of up to 32 Q and K heads and 4 V heads: twice the batch, still one round.
// The arithmetic is norm_rotate's, as in the kernel above.
constexpr uint32_t kTokenWaveCapacity = 4096;  // 4 waves per SIMD: the 100-odd registers a wave of this kernel takes
// The gate: 0.97 of the time the launch's reads take at 7 TB/s, the rate of a read-only kernel on this part (4096
// tokens of 32+8+8 heads: 15.6-15.8 us with 0.95 to 1.0 of that time, 16.0 with 0.9, 17.0 with 0.85, 16.5 with 1.05,
// 19-20 with no gate at all; the kernel above: 18.2).
constexpr double kGateBytesPerTick = 70000.0 / 0.97;

// The leading parameters of the kernel below as the argument segment lays them out; the block follows them.
struct TokenKernelLead {
    const void *qkv_in;
    const int64_t *positions;
    uint32_t num_tokens, gate;
    int hq, hk, hv;
    uint32_t num_waves;
    int64_t ps_token, ps_axis;
};
static_assert(sizeof(TokenKernelLead) == 56 && sizeof(TokenKernelLead) % alignof(RopeArgs) == 0, "offset of the block");

// One 16-byte piece per lane from global memory into LDS at lds_byte_offset + 16 * lane; the address is the lane's
// own.  M0 carries the LDS offset: one wait state after writing it, and it is named as clobbered so that the compiler
// never keeps a value of its own there across the transfer (its warning that M0 is reserved is silenced: reserved
// means it allocates nothing there, which is the point).  Counted by vmcnt like a load.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void lds_fill16(uint32_t lds_byte_offset, const void *lane_address) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 1\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(lds_byte_offset), "v"(lane_address) : "memory", "m0");
}
#pragma clang diagnostic pop

// cos and sin pieces of a lane for a token at positions (p0, p1, p2): with three axes every aligned group of 8
// frequencies takes one axis (the host checks the sections), so each lane reads its pieces from that axis's row
template <int D, bool NEOX, int AXES>
__device__ __forceinline__ void load_trig_by_axis(const uint16_t *table, int64_t p0, int64_t p1, int64_t p2,
                                                  const uint32_t (&axis1)[4], const uint32_t (&axis2)[4], int sub,
                                                  u32x4 &cosv, u32x4 &sinv) {
    constexpr int HALF = D / 2;
    if constexpr (AXES == 1) {
        cosv = load_trig<D, NEOX>(table + p0 * D, sub);
        sinv = load_trig<D, NEOX>(table + p0 * D + HALF, sub);
    } else {
        const uint32_t b1 = trig_bits<D, NEOX>(axis1, sub), b2 = trig_bits<D, NEOX>(axis2, sub);
        const int64_t pa = (b2 & 1u) ? p2 : ((b1 & 1u) ? p1 : p0);
        if constexpr (NEOX) {
            cosv = load_trig<D, NEOX>(table + pa * D, sub);
            sinv = load_trig<D, NEOX>(table + pa * D + HALF, sub);
        } else {
            const int64_t pb = (b2 & 16u) ? p2 : ((b1 & 16u) ? p1 : p0);
            const u32x2 cl = *reinterpret_cast<const u32x2 *>(table + pa * D + 4 * sub);
            const u32x2 ch = *reinterpret_cast<const u32x2 *>(table + pb * D + D / 4 + 4 * sub);
            const u32x2 sl = *reinterpret_cast<const u32x2 *>(table + pa * D + HALF + 4 * sub);
            const u32x2 sh = *reinterpret_cast<const u32x2 *>(table + pb * D + HALF + D / 4 + 4 * sub);
            cosv = u32x4{cl[0], cl[1], ch[0], ch[1]};
            sinv = u32x4{sl[0], sl[1], sh[0], sh[1]};
        }
    }
}

// Norm and rotation of a token's units, in place.
template <typename T, int D, bool NEOX, int UPT>
__device__ __forceinline__ void token_rotate(u32x4 (&xa)[UPT], u32x4 (&xb)[UPT], const u32x4 &qwa, const u32x4 &qwb,
                                             const u32x4 &kwa, const u32x4 &kwb, const u32x4 &cosv, const u32x4 &sinv,
                                             float eps, int hq, int hl) {
    constexpr int HPW = 64 / (D / 16);
#pragma unroll
    for (int u = 0; u < UPT; ++u) {
        const int h0 = u * HPW;
        u32x4 wa, wb;
        if (h0 + HPW <= hq) {  // wave-uniform: a unit of Q heads, of K heads, or of both
            wa = qwa, wb = qwb;
        } else if (h0 >= hq) {
            wa = kwa, wb = kwb;
        } else {
            const bool is_q = h0 + hl < hq;
#pragma unroll
            for (int j = 0; j < 4; ++j) wa[j] = is_q ? qwa[j] : kwa[j], wb[j] = is_q ? qwb[j] : kwb[j];
        }
        u32x4 oa, ob;
        norm_rotate<T, D, NEOX>(xa[u], xb[u], wa, wb, cosv, sinv, eps, oa, ob);
        xa[u] = oa, xb[u] = ob;
    }
}

// The stores of a token: q_out rows, the K and V rows of its slot (dropped for a negative slot); in place (!SETKV)
// the rotated Q and K heads back where they came from.
template <typename T, int D, int UPT, bool SETKV, bool KVFP8, int VN>
__device__ __forceinline__ void token_store(const RopeArgs &a, uint32_t t, int64_t slot, const u32x4 (&xa)[UPT],
                                            const u32x4 (&xb)[UPT], const u32x4 (&v)[VN], int hq, int hk, int hv, int lane) {
    constexpr int LPH = D / 16, HPW = 64 / LPH, HALF = D / 2;
    const int sub = lane % LPH, hl = lane / LPH, heads_qk = hq + hk, v_chunks = hv * (D / 8);
    if constexpr (!SETKV) {
#pragma unroll
        for (int u = 0; u < UPT; ++u) {
            const int head = u * HPW + hl;
            if (head < heads_qk) {
                uint16_t *dst = static_cast<uint16_t *>(a.qkv_out) + ((int64_t)t * (heads_qk + hv) + head) * D + 8 * sub;
                store_pair<HALF * 2>(dst, xa[u], xb[u], true);
            }
        }
        return;
    }
    const bool slot_ok = slot >= 0;  // a negative slot: no place in the cache, the K and V rows are dropped
#pragma unroll
    for (int u = 0; u < UPT; ++u) {
        const int head = u * HPW + hl;
        if (head < hq) {
            uint16_t *dst = static_cast<uint16_t *>(a.q_out) + ((int64_t)t * hq + head) * D + 8 * sub;
            store_pair<HALF * 2>(dst, xa[u], xb[u], true);
        } else if (head < heads_qk && slot_ok) {
            const int64_t at = (slot * hk + (head - hq)) * D + 8 * sub;
            if constexpr (KVFP8) {
                uint8_t *dst = static_cast<uint8_t *>(a.k_cache) + at;
                const float s = a.k_scale, rcp = 1.0f / s;
                if (scale_is_fast(s)) {
                    *reinterpret_cast<u32x2 *>(dst) = quantize_chunk<T, true>(xa[u], s, rcp);
                    *reinterpret_cast<u32x2 *>(dst + HALF) = quantize_chunk<T, true>(xb[u], s, rcp);
                } else {
                    *reinterpret_cast<u32x2 *>(dst) = quantize_chunk<T, false>(xa[u], s, rcp);
                    *reinterpret_cast<u32x2 *>(dst + HALF) = quantize_chunk<T, false>(xb[u], s, rcp);
                }
            } else {
                store_pair<HALF * 2>(static_cast<uint16_t *>(a.k_cache) + at, xa[u], xb[u], true);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < VN; ++j) {
        const int c = lane + 64 * j;
        if (slot_ok && c < v_chunks) {
            const int64_t off = slot * hv * D + 8 * (int64_t)c;
            if constexpr (KVFP8) {
                const float s = a.v_scale, rcp = 1.0f / s;
                *reinterpret_cast<u32x2 *>(static_cast<uint8_t *>(a.v_cache) + off) =
                    scale_is_fast(s) ? quantize_chunk<T, true>(v[j], s, rcp) : quantize_chunk<T, false>(v[j], s, rcp);
            } else {
                *reinterpret_cast<u32x4 *>(static_cast<uint16_t *>(a.v_cache) + off) = v[j];
            }
        }
    }
}

constexpr int token_kernel_lds_bytes_per_wave(int upt, bool set_kv) { return (2 * upt + (set_kv ? 1 : 0)) * 1024; }  // TWO: a token's units and 64 V chunks

template <typename T, int D, bool NEOX, int UPT, bool SETKV, bool KVFP8, int AXES, bool TWO>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4)))
rope_rms_token_kernel(const void *qkv_in, const int64_t *positions, uint32_t num_tokens, uint32_t gate, int hq, int hk,
                      int hv, uint32_t num_waves, int64_t ps_token, int64_t ps_axis, const RopeArgs rest) {
    constexpr int LPH = D / 16, HPW = 64 / LPH, HALF = D / 2;
    constexpr int VN = TWO ? 1 : 2;  // V chunks per lane: the host admits 64 chunks per token with TWO, else 128
    extern __shared__ __attribute__((aligned(16))) char token_lds[];  // TWO: 4 waves x token_kernel_lds_bytes_per_wave()
    const uint64_t entry = __builtin_amdgcn_s_memrealtime();
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t w = blockIdx.x * 4 + wave;
    if (w >= num_waves) return;
    // The wave's token(s).  TWO: the tokens beyond num_waves (a multiple of 1024 wherever there are any: a whole
    // number of waves on every SIMD) ride as second tokens, dealt out evenly over the compute units -- workgroup g runs
    // on compute unit g mod 256 while the launch is one round, so the waves of a compute unit are w = 4 (cu + 256 l) + i,
    // ranked l, i here, and the first extra / 256 of each rank order take one (the remainder: one more on the first units).
    // (Any other num_waves: wave w takes token w + num_waves as well, where there is one.)
    const uint32_t t = w;
    uint32_t t2 = num_tokens;
    if constexpr (TWO) {
        if (num_waves & 1023u) {
            t2 = w + num_waves;
        } else {
            const uint32_t extra = num_tokens - num_waves, each = extra >> 8, more = extra & 255u;
            const uint32_t cu = (w >> 2) & 255u, layer = w >> 10, rank = (layer << 2) | (w & 3u);
            // (in wave order as far as whole layers of 1024 waves go -- neighbouring workgroups then take neighbouring
            // tokens, 1 % at 8192 tokens -- then the waves of the part layer, then the remainder)
            if (rank < each) t2 = num_waves + (layer < (each >> 2) ? w : (layer << 10) + cu * (each & 3u) + (w & 3u));
            else if (rank == each && cu < more) t2 = num_waves + (each << 8) + cu;
        }
    }
    const bool second = TWO && t2 < num_tokens;  // wave-uniform
    const int lane = threadIdx.x & 63, sub = lane % LPH, hl = lane / LPH;
    const int heads_qk = hq + hk, heads_all = heads_qk + hv, v_chunks = hv * (D / 8);
    const uint16_t *token_in = static_cast<const uint16_t *>(qkv_in) + (int64_t)t * heads_all * D;

    // ---- everything the wave reads, asked for at once (what needs only the leading parameters first)
    u32x4 xa[UPT], xb[UPT], v[VN];
#pragma unroll
    for (int u = 0; u < UPT; ++u) {
        const int head = min(u * HPW + hl, heads_qk - 1);  // lanes past the last head re-read it
        const uint16_t *src = token_in + (int64_t)head * D;
        xa[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + 8 * sub));
        xb[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + HALF + 8 * sub));
    }
    if constexpr (SETKV) {
#pragma unroll
        for (int j = 0; j < VN; ++j) {
            const int c = min(lane + 64 * j, v_chunks - 1);
            v[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(token_in + (int64_t)heads_qk * D + 8 * c));
        }
    }
    uint32_t lds_base = 0;
    if constexpr (TWO) {
        lds_base = (uint32_t)(uintptr_t)token_lds + wave * (uint32_t)token_kernel_lds_bytes_per_wave(UPT, SETKV);
        if (second) {
            const uint16_t *token2_in = static_cast<const uint16_t *>(qkv_in) + (int64_t)t2 * heads_all * D;
#pragma unroll
            for (int u = 0; u < UPT; ++u) {
                const int head = min(u * HPW + hl, heads_qk - 1);
                const uint16_t *src = token2_in + (int64_t)head * D;
                lds_fill16(lds_base + (2 * u) * 1024u, src + 8 * sub);
                lds_fill16(lds_base + (2 * u + 1) * 1024u, src + HALF + 8 * sub);
            }
            if constexpr (SETKV) {
                const int c = min(lane, v_chunks - 1);
                lds_fill16(lds_base + (2 * UPT) * 1024u, token2_in + (int64_t)heads_qk * D + 8 * c);
            }
        }
    }
    // (positions: read as memory that no kernel of the launch writes, scalar loads whatever else the kernel contains)
    int64_t p[3] = {0, 0, 0}, p2[3] = {0, 0, 0};
#pragma unroll
    for (int ax = 0; ax < AXES; ++ax) {
        p[ax] = load_unchanging(positions + ax * ps_axis + (int64_t)t * ps_token);
        if (second) p2[ax] = load_unchanging(positions + ax * ps_axis + (int64_t)t2 * ps_token);
    }
    // the rest of the arguments, fetched from the argument block behind the requests above (see rope_rms_kernel)
    typedef const __attribute__((address_space(4))) RopeArgs *BlockPtr;
    BlockPtr block = (BlockPtr)((const __attribute__((address_space(4))) char *)__builtin_amdgcn_kernarg_segment_ptr() +
                                sizeof(TokenKernelLead));
    asm volatile("" : "+s"(block));
    RopeArgs a;
    a.qw = as_global(block->qw);
    a.kw = as_global(block->kw);
    a.cos_sin = as_global(block->cos_sin);
    a.eps = block->eps;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a.axis1[i] = AXES == 3 ? block->axis1[i] : 0u;
        a.axis2[i] = AXES == 3 ? block->axis2[i] : 0u;
    }
    int64_t slot = 0, slot2 = 0;
    if constexpr (SETKV) {
        a.kv_loc = as_global(block->kv_loc);
        a.q_out = as_global(block->q_out);
        a.k_cache = as_global(block->k_cache);
        a.v_cache = as_global(block->v_cache);
        a.k_scale = block->k_scale;
        a.v_scale = block->v_scale;
        asm volatile("" ::"s"(a.kv_loc), "s"(a.qw), "s"(a.kw), "s"(a.cos_sin), "s"(a.q_out), "s"(a.k_cache), "s"(a.v_cache),
                     "s"(a.eps), "s"(a.k_scale), "s"(a.v_scale));
        slot = load_unchanging(a.kv_loc + t);
        slot2 = second ? load_unchanging(a.kv_loc + t2) : -1;
    } else {
        a.qkv_out = as_global(block->qkv_out);
        asm volatile("" ::"s"(a.qw), "s"(a.kw), "s"(a.cos_sin), "s"(a.qkv_out), "s"(a.eps));
    }
    const uint16_t *qw = static_cast<const uint16_t *>(a.qw), *kw = static_cast<const uint16_t *>(a.kw);
    const u32x4 qwa = *reinterpret_cast<const u32x4 *>(qw + 8 * sub), qwb = *reinterpret_cast<const u32x4 *>(qw + HALF + 8 * sub);
    const u32x4 kwa = *reinterpret_cast<const u32x4 *>(kw + 8 * sub), kwb = *reinterpret_cast<const u32x4 *>(kw + HALF + 8 * sub);
    const uint16_t *table = static_cast<const uint16_t *>(a.cos_sin);
    u32x4 cosv, sinv, cosv2 = {0, 0, 0, 0}, sinv2 = {0, 0, 0, 0};
    load_trig_by_axis<D, NEOX, AXES>(table, p[0], p[1], p[2], a.axis1, a.axis2, sub, cosv, sinv);
    if (second) load_trig_by_axis<D, NEOX, AXES>(table, p2[0], p2[1], p2[2], a.axis1, a.axis2, sub, cosv2, sinv2);
    // (the slots are asked for here and not where the rows are stored)
    if constexpr (SETKV)
        asm volatile("" ::"s"((uint32_t)slot), "s"((uint32_t)(slot >> 32)), "s"((uint32_t)slot2), "s"((uint32_t)(slot2 >> 32)));
    __builtin_amdgcn_sched_barrier(0);

    // ---- norm and rotation of the first token, unit by unit, in place
    token_rotate<T, D, NEOX, UPT>(xa, xb, qwa, qwb, kwa, kwb, cosv, sinv, a.eps, hq, hl);

    // (the rotated rows are pinned down here, ahead of the wait: nothing ties the arithmetic to the clock, and the
    // compiler otherwise moves it behind the wait, into the writing half)
#pragma unroll
    for (int u = 0; u < UPT; ++u) asm volatile("" ::"v"(xa[u]), "v"(xb[u]));

    // ---- the writing half of the launch
    while (__builtin_amdgcn_s_memrealtime() < entry + gate) __builtin_amdgcn_s_sleep(1);
    // (the transfers into LDS are not loads the compiler knows of; they landed long ago, and with nothing else of
    // the wave outstanding at this point the wait that says so to the hardware costs nothing)
    if constexpr (TWO) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    token_store<T, D, UPT, SETKV, KVFP8, VN>(a, t, slot, xa, xb, v, hq, hk, hv, lane);
    if constexpr (TWO) {
        if (second) {  // the second token takes the registers of the first
            const char *mine = token_lds + wave * token_kernel_lds_bytes_per_wave(UPT, SETKV) + lane * 16;
#pragma unroll
            for (int u = 0; u < UPT; ++u) {
                xa[u] = *reinterpret_cast<const u32x4 *>(mine + (2 * u) * 1024);
                xb[u] = *reinterpret_cast<const u32x4 *>(mine + (2 * u + 1) * 1024);
            }
            if constexpr (SETKV) v[0] = *reinterpret_cast<const u32x4 *>(mine + (2 * UPT) * 1024);
            token_rotate<T, D, NEOX, UPT>(xa, xb, qwa, qwb, kwa, kwb, cosv2, sinv2, a.eps, hq, hl);
            token_store<T, D, UPT, SETKV, KVFP8, VN>(a, t2, slot2, xa, xb, v, hq, hk, hv, lane);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// fp32 and fp64 activations: the reference dispatches them through the same templates (AT_DISPATCH_FLOATING_TYPES_AND2,
// src/ops/fused_rope.cpp:27-30, :108-111).  The layout of the 16-bit kernel with chunks of 4 elements: a head is D/8
// lanes, a lane owns the chunks at elements 4*sub and D/2 + 4*sub of its head (NeoX: x1 and x2 of frequencies
// 4*sub .. 4*sub+3; GPT-J: the pairs of frequencies 2*sub, 2*sub+1 and D/4 + 2*sub, D/4 + 2*sub+1), a wave takes 512/D
// consecutive Q/K heads of a token; with a KV cache further waves of the token copy or quantise its V row, 128 chunks
// each.  Rounding to the activation type F is the identity, so the oracle's sequence is plain arithmetic in F with
// every product rounded before the add, around an fp32 variance and rstd (torch promotes x * rstd to F); an fp8
// cache takes float(o / F(scale)).
constexpr int kWideChunksPerValueUnit = 128;
template <int D> constexpr int wide_heads_per_wave() { return 512 / D; }

template <typename F, int D, bool NEOX, int AXES, bool SETKV, bool KVFP8>
__global__ void __launch_bounds__(256) rope_rms_wide_kernel(const RopeArgs a) {
    typedef F V4 __attribute__((ext_vector_type(4), aligned(16)));
    constexpr int HALF = D / 2, LPH = D / 8, HPW = wide_heads_per_wave<D>();
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t unit = blockIdx.x * (blockDim.x >> 6) + wave;
    if (unit >= a.total_units) return;
    const int lane = threadIdx.x & 63, sub = lane % LPH, hl = lane / LPH;
    const uint32_t t = a.upt_magic ? __umulhi(unit, a.upt_magic) : unit;
    const int u = (int)(unit - t * a.units_per_token);  // unit inside the token
    const int heads_qk = a.hq + a.hk, heads_all = heads_qk + a.hv;
    const int qk_units = (heads_qk + HPW - 1) / HPW;
    const F *token_row = static_cast<const F *>(a.qkv_in) + (int64_t)t * heads_all * D;

    if (u >= qk_units) {  // a share of the token's V row: only reached with a KV cache
        if constexpr (SETKV) {
            const int64_t slot = a.kv_loc[t];
            if (slot < 0) return;  // token without a cache slot
            const int v_chunks = a.hv * (D / 4);
#pragma unroll
            for (int k = 0; k < kWideChunksPerValueUnit / 64; ++k) {
                const int chunk = (u - qk_units) * kWideChunksPerValueUnit + 64 * k + lane;
                if (chunk >= v_chunks) continue;
                const V4 v = __builtin_nontemporal_load(reinterpret_cast<const V4 *>(token_row + (int64_t)heads_qk * D + 4 * chunk));
                const int64_t off = slot * a.hv * D + 4 * (int64_t)chunk;
                if constexpr (KVFP8) {
                    const V4 q = v / (F)a.v_scale;
                    *reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(a.v_cache) + off) =
                        cvt4_e4m3fn(clamp_sym((float)q[0], kE4M3Max), clamp_sym((float)q[1], kE4M3Max),
                                    clamp_sym((float)q[2], kE4M3Max), clamp_sym((float)q[3], kE4M3Max));
                } else {
                    *reinterpret_cast<V4 *>(static_cast<F *>(a.v_cache) + off) = v;
                }
            }
        }
        return;
    }

    const int head_raw = u * HPW + hl;
    const bool active = head_raw < heads_qk;
    const int head = active ? head_raw : heads_qk - 1;  // idle lanes of a token's last unit repeat its last head
    const bool is_q = head < a.hq;
    const int e0 = 4 * sub, e1 = HALF + 4 * sub;

    // every load of the wave is issued before the first use: positions and slot (wave-uniform), then x, the weights
    // and the cos/sin values, whose rows depend on the positions
    const F *table = static_cast<const F *>(a.cos_sin);
    const int64_t p0 = a.positions[(int64_t)t * a.ps_token];
    int64_t p1 = p0, p2 = p0;
    if constexpr (AXES == 3) {
        p1 = a.positions[a.ps_axis + (int64_t)t * a.ps_token];
        p2 = a.positions[2 * a.ps_axis + (int64_t)t * a.ps_token];
    }
    int64_t slot = 0;
    if constexpr (SETKV) slot = a.kv_loc[t];
    const F *src = token_row + (int64_t)head * D;
    const V4 xa = __builtin_nontemporal_load(reinterpret_cast<const V4 *>(src + e0));
    const V4 xb = __builtin_nontemporal_load(reinterpret_cast<const V4 *>(src + e1));
    const void *qw = a.qw, *kw = a.kw;
    if constexpr (AXES == 3) asm("" : "+s"(qw), "+s"(kw));  // a select between kernel arguments: see RopeUnit::issue_loads
    const F *w = static_cast<const F *>(is_q ? qw : kw);
    const V4 wa = *reinterpret_cast<const V4 *>(w + e0), wb = *reinterpret_cast<const V4 *>(w + e1);
    // the lane's four rotary frequencies, in the order the chunks' elements use them
    int freq[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) freq[j] = NEOX ? 4 * sub + j : (j < 2 ? 2 * sub + j : D / 4 + 2 * sub + (j - 2));
    V4 c, s;
    if (AXES == 1 || (p0 == p1 && p1 == p2)) {  // wave-uniform: one row, whole pieces of it
        const F *row = table + p0 * D;
        if constexpr (NEOX) {
            c = *reinterpret_cast<const V4 *>(row + freq[0]);
            s = *reinterpret_cast<const V4 *>(row + HALF + freq[0]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                c[j] = row[freq[j]];
                s[j] = row[HALF + freq[j]];
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int f = freq[j];
            const bool on1 = (bitmap_word<D>(a.axis1, f) >> (f & 31)) & 1u, on2 = (bitmap_word<D>(a.axis2, f) >> (f & 31)) & 1u;
            const int64_t pos = on2 ? p2 : (on1 ? p1 : p0);
            c[j] = table[pos * D + f];
            s[j] = table[pos * D + HALF + f];
        }
    }

    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float fa = (float)xa[j], fb = (float)xb[j];
        ss = __builtin_fmaf(fa, fa, ss);
        ss = __builtin_fmaf(fb, fb, ss);
    }
    ss = group_allreduce<SumOp, LPH < 16 ? LPH : 16>(ss);
    if constexpr (LPH == 32) ss += __shfl_xor(ss, 16);
    const F rstd = (F)(1.0f / sqrtf(ss * (1.0f / D) + a.eps));

    const V4 na = wa * (xa * rstd), nb = wb * (xb * rstd);
    V4 oa, ob;
    if constexpr (NEOX) {
        oa = na * c - nb * s;
        ob = nb * c + na * s;
    } else {
        oa = V4{na[0] * c[0] - na[1] * s[0], na[1] * c[0] + na[0] * s[0], na[2] * c[1] - na[3] * s[1], na[3] * c[1] + na[2] * s[1]};
        ob = V4{nb[0] * c[2] - nb[1] * s[2], nb[1] * c[2] + nb[0] * s[2], nb[2] * c[3] - nb[3] * s[3], nb[3] * c[3] + nb[2] * s[3]};
    }
    if (!active) return;
    // rotated rows are stored past the L2 (as the 16-bit kernel does from a few MB per call on; smaller calls are
    // bound by their launch either way)
    if constexpr (!SETKV) {
        F *dst = static_cast<F *>(a.qkv_out) + ((int64_t)t * heads_all + head) * D;
        __builtin_nontemporal_store(oa, reinterpret_cast<V4 *>(dst + e0));
        __builtin_nontemporal_store(ob, reinterpret_cast<V4 *>(dst + e1));
    } else if (is_q) {
        F *dst = static_cast<F *>(a.q_out) + ((int64_t)t * a.hq + head) * D;
        __builtin_nontemporal_store(oa, reinterpret_cast<V4 *>(dst + e0));
        __builtin_nontemporal_store(ob, reinterpret_cast<V4 *>(dst + e1));
    } else {
        if (slot < 0) return;  // token without a cache slot: nothing of a K head is kept
        const int64_t row = (slot * a.hk + (head - a.hq)) * D;
        if constexpr (KVFP8) {
            const V4 qa = oa / (F)a.k_scale, qb = ob / (F)a.k_scale;
            uint8_t *dst = static_cast<uint8_t *>(a.k_cache) + row;
            *reinterpret_cast<uint32_t *>(dst + e0) =
                cvt4_e4m3fn(clamp_sym((float)qa[0], kE4M3Max), clamp_sym((float)qa[1], kE4M3Max),
                            clamp_sym((float)qa[2], kE4M3Max), clamp_sym((float)qa[3], kE4M3Max));
            *reinterpret_cast<uint32_t *>(dst + e1) =
                cvt4_e4m3fn(clamp_sym((float)qb[0], kE4M3Max), clamp_sym((float)qb[1], kE4M3Max),
                            clamp_sym((float)qb[2], kE4M3Max), clamp_sym((float)qb[3], kE4M3Max));
        } else {
            F *dst = static_cast<F *>(a.k_cache) + row;
            __builtin_nontemporal_store(oa, reinterpret_cast<V4 *>(dst + e0));
            __builtin_nontemporal_store(ob, reinterpret_cast<V4 *>(dst + e1));
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
    uint32_t stream;  // 1: the output rows are stored past the L2 (calls that move more than a few MB)
};

// The leading parameters of the kernel below as the argument segment lays them out; the block follows them.
struct TwoWayKernelLead {
    const void *q0, *k0, *q1, *k1;
    uint32_t tokens0, tokens1, heads_q, heads_k, stream;
    uint32_t pad_;
};
static_assert(sizeof(TwoWayKernelLead) == 56 && sizeof(TwoWayKernelLead) % alignof(TwoWayArgs) == 0, "offset of the block");

// As in rope_rms_kernel, what a wave needs to find and request its activations -- the four input pointers, the token
// and head counts -- are leading scalar parameters that arrive in scalar registers at launch; segment bounds and
// row counts are products and sums of those, not loads.  (With everything in the argument block and the per-segment
// values picked by index, a wave went through five dependent fetches of the block before its first request.)  The
// block (weights, tables, outputs, the division constants) is fetched behind the activations, in one batch.
template <typename T, int D, bool NEOX>
__global__ void __launch_bounds__(256)
rope_rms_2way_kernel(const void *q0, const void *k0, const void *q1, const void *k1, uint32_t tokens0, uint32_t tokens1,
                     uint32_t heads_q, uint32_t heads_k, uint32_t stream, const TwoWayArgs rest) {
    constexpr int LPH = D / 16, HPW = 64 / LPH, HALF = D / 2;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t unit = blockIdx.x * 4 + wave;
    const uint32_t rows0 = tokens0 * heads_q, rows1 = tokens0 * heads_k, rows2 = tokens1 * heads_q, rows3 = tokens1 * heads_k;
    const uint32_t end0 = (rows0 + HPW - 1) / HPW, end1 = end0 + (rows1 + HPW - 1) / HPW, end2 = end1 + (rows2 + HPW - 1) / HPW,
                   end3 = end2 + (rows3 + HPW - 1) / HPW;
    if (unit >= end3) return;
    const int seg = (unit >= end0) + (unit >= end1) + (unit >= end2);  // wave-uniform
    const uint32_t unit_in_seg = unit - (seg == 0 ? 0u : seg == 1 ? end0 : seg == 2 ? end1 : end2);
    const int kind = seg & 1, stream_id = seg >> 1;  // q|k, stream 0|1
    const uint32_t heads = kind ? heads_k : heads_q;
    const uint32_t rows = seg == 0 ? rows0 : seg == 1 ? rows1 : seg == 2 ? rows2 : rows3;
    const void *in = seg == 0 ? q0 : seg == 1 ? k0 : seg == 2 ? q1 : k1;
    const int batch = blockIdx.y;

    const int lane = threadIdx.x & 63, sub = lane % LPH, hl = lane / LPH;
    const uint32_t row_raw = unit_in_seg * HPW + hl;
    const bool active = row_raw < rows;
    const uint32_t row = min(row_raw, rows - 1);  // (token, head) flattened inside the segment

    const int c0 = 8 * sub, c1 = HALF + 8 * sub;
    const uint16_t *src = static_cast<const uint16_t *>(in) + ((int64_t)batch * rows + row) * D;
    const u32x4 xa = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + c0));
    const u32x4 xb = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + c1));

    typedef const __attribute__((address_space(4))) TwoWayArgs *BlockPtr;
    BlockPtr block = (BlockPtr)((const __attribute__((address_space(4))) char *)__builtin_amdgcn_kernarg_segment_ptr() +
                                sizeof(TwoWayKernelLead));
    asm volatile("" : "+s"(block));
    const void *w0 = as_global(block->w[0]), *w1 = as_global(block->w[1]), *w2 = as_global(block->w[2]), *w3 = as_global(block->w[3]);
    const void *table0 = as_global(block->cos_sin[0]), *table1 = as_global(block->cos_sin[1]);
    void *out_q = as_global(block->out[0]), *out_k = as_global(block->out[1]);
    const uint32_t magic_q = block->heads_magic[0], magic_k = block->heads_magic[1];
    const float eps = block->eps;
    asm volatile("" ::"s"(w0), "s"(w1), "s"(w2), "s"(w3), "s"(table0), "s"(table1), "s"(out_q), "s"(out_k), "s"(magic_q),
                 "s"(magic_k), "s"(eps));
    const uint32_t magic = kind ? magic_k : magic_q;
    const uint32_t token = magic ? __umulhi(row, magic) : row;
    const uint32_t head = row - token * heads;
    const uint16_t *wsrc = static_cast<const uint16_t *>(seg == 0 ? w0 : seg == 1 ? w1 : seg == 2 ? w2 : w3);
    const u32x4 wa = *reinterpret_cast<const u32x4 *>(wsrc + c0);
    const u32x4 wb = *reinterpret_cast<const u32x4 *>(wsrc + c1);
    const uint16_t *table = static_cast<const uint16_t *>(stream_id ? table1 : table0) + (int64_t)token * D;
    const u32x4 cosv = load_trig<D, NEOX>(table, sub);
    const u32x4 sinv = load_trig<D, NEOX>(table + HALF, sub);
    __builtin_amdgcn_sched_barrier(0);

    u32x4 oa, ob;
    norm_rotate<T, D, NEOX>(xa, xb, wa, wb, cosv, sinv, eps, oa, ob);
    if (active) {
        const int64_t out_token = (int64_t)batch * (tokens0 + tokens1) + (stream_id ? tokens0 : 0u) + token;
        uint16_t *dst = static_cast<uint16_t *>(kind ? out_k : out_q) + (out_token * heads + head) * D;
        store_pair<HALF * 2>(dst + c0, oa, ob, stream != 0);
    }
}

// fp32 / fp64 form of the two-stream op (the reference dispatches float and double here too:
// src/ops/fused_rope.cpp:197-200): one wave per (token, head) row of a segment, lane l owns rotation pairs l, l+64, ...;
// plain arithmetic in the activation type F around an fp32 variance, every product rounded before the add.  The host
// counts one unit per row for this kernel.
template <typename F, int D, bool NEOX>
__global__ void __launch_bounds__(256) rope_rms_2way_wide_kernel(const TwoWayArgs a) {
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

    const F *src = static_cast<const F *>(a.in[seg]) + ((int64_t)batch * rows + row) * D;
    const F *w = static_cast<const F *>(a.w[seg]);
    const F *table = static_cast<const F *>(a.cos_sin[stream_id]) + (int64_t)token * D;
    const int64_t out_token = (int64_t)batch * (a.tokens0 + a.tokens1) + (stream_id ? a.tokens0 : 0) + token;
    F *dst = static_cast<F *>(a.out[kind]) + (out_token * heads + head) * D;

    F x1[PPL], x2[PPL];
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
        x1[k] = live[k] ? src[i1[k]] : (F)0;
        x2[k] = live[k] ? src[i2[k]] : (F)0;
        const float f1 = (float)x1[k], f2 = (float)x2[k];
        ss = __builtin_fmaf(f1, f1, ss);
        ss = __builtin_fmaf(f2, f2, ss);
    }
    ss = wave_allreduce<SumOp>(ss);
    const F rstd = (F)(1.0f / sqrtf(ss * (1.0f / D) + a.eps));
#pragma unroll
    for (int k = 0; k < PPL; ++k) {
        if (!live[k]) continue;
        const int f = lane + 64 * k;
        const F c = table[f], s = table[HALF + f];
        const F n1 = w[i1[k]] * (x1[k] * rstd), n2 = w[i2[k]] * (x2[k] * rstd);
        dst[i1[k]] = n1 * c - n2 * s;
        dst[i2[k]] = n2 * c + n1 * s;
    }
}

template <typename T, int D>
int launch_2way(const TwoWayArgs &a, bool neox, unsigned batch, hipStream_t stream) {
    const dim3 grid((a.unit_end[3] + 3) / 4, batch);
#define GPUK_LAUNCH_2WAY(NEOX)                                                                                         \
    rope_rms_2way_kernel<T, D, NEOX><<<grid, 256, 0, stream>>>(a.in[0], a.in[1], a.in[2], a.in[3], (uint32_t)a.tokens0,  \
                                                               (uint32_t)a.tokens1, a.heads[0], a.heads[1], a.stream, a)
    if (neox) GPUK_LAUNCH_2WAY(true);
    else GPUK_LAUNCH_2WAY(false);
#undef GPUK_LAUNCH_2WAY
    return hip_status(hipGetLastError());
}

template <typename F, int D>
int launch_2way_wide(const TwoWayArgs &a, bool neox, unsigned batch, hipStream_t stream) {
    const dim3 grid((a.unit_end[3] + 3) / 4, batch);
    if (neox) rope_rms_2way_wide_kernel<F, D, true><<<grid, 256, 0, stream>>>(a);
    else rope_rms_2way_wide_kernel<F, D, false><<<grid, 256, 0, stream>>>(a);
    return hip_status(hipGetLastError());
}

template <typename F>
int launch_2way_wide_head_size(const TwoWayArgs &a, int64_t D, bool neox, unsigned batch, hipStream_t stream) {
    switch (D) {
        case 64: return launch_2way_wide<F, 64>(a, neox, batch, stream);
        case 128: return launch_2way_wide<F, 128>(a, neox, batch, stream);
        case 256: return launch_2way_wide<F, 256>(a, neox, batch, stream);
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

int g_block_threads = 0;  // 0 = default
int g_stream_rows = 0;    // output rows stored past the L2: 0 = built-in rule, 1 = never, 2 = always
int g_merge_rows = 0;     // mRoPE rows merged on load where the sections allow: 0 = yes, 1 = never
int g_token_waves = 0;    // one-wave-per-token kernel: 0 = built-in rule, 1 = never, 2 = wherever it fits, 3 = likewise, two tokens per wave where that fits
int g_token_gate = -1;    // its gate in ticks of 10 ns; -1 = from the bytes of the call
int g_unit_gate = -1;     // gate of the kernel with one wave per unit: -1 = built-in rule, 0 = none, > 0 = ticks
constexpr uint32_t kResidentUnits = 8192;  // waves of the one-wave-per-unit kernel the chip holds at once (8 per SIMD)

// Streaming stores, measured on MI355X (32/8/8, 28/4/4 and 64/8/8 heads, head sizes 64-256, random slots): q_out /
// K rows / in-place rows written past the L2 are ahead from about 10 MB per call on (64+8 heads, fp8 cache: 5.9
// against 7.0 us at 512 tokens, 16.0 against 18.1 at 2048; 40 heads: 19.0 against 21.1 us at 4096 tokens, 65.2 against
// 80.2 at 16384; level at 5 MB and below) -- what a kernel leaves dirty in the L2 is written back at its end.
constexpr int64_t kStreamFromBytes = 8'000'000;

// What a call of the 16-bit rope kernel launches: its grid, and whether the output rows go past the L2.
struct RopePlan {
    uint32_t threads, blocks;  // workgroup size and count of the launch
    bool stream;               // q_out / K rows / in-place rows stored past the L2
    bool token_waves;          // the one-wave-per-token kernel
    bool two_tokens;           // ... with two tokens per wave, the second through LDS
    uint32_t token_wave_count; // its waves
    uint32_t gate;             // its gate: ticks of 10 ns before which no wave stores
    uint32_t unit_gate;        // the same for the kernel with one wave per unit (0 = none)
};

RopePlan plan_rope(const RopeArgs &a, int D, int axes, bool set_kv, bool kv_fp8) {
    RopePlan p{};
    // One wave per token (or per two) where the whole batch is resident at once and large enough for its traffic to
    // matter: head size 128, 4 or 5 units (25-40 Q and K heads) and at most 128 chunks of V per token, a cache; with
    // three position axes only where every aligned group of 8 frequencies takes one axis, and not with an fp8 cache.
    const int64_t read_bytes = 2 * (int64_t)a.num_tokens * (a.hq + a.hk + (set_kv ? a.hv : 0)) * D;
    const bool shape = D == 128 && a.units_per_token >= 4 && a.units_per_token <= 5 &&
                       (!set_kv || (a.hv * (D / 8) <= 128 && a.hv > 0)) && (axes == 1 || (axes == 3 && a.merge_rows && !kv_fp8));
    const bool one = shape && a.num_tokens <= kTokenWaveCapacity;
    // Two tokens per wave, the second through LDS (4 units and 64 V chunks per token: 9 KB of the 160 KB of a compute
    // unit for each of its 16 waves), for up to twice that many tokens.
    const bool two_shape = shape && a.units_per_token == 4 && (!set_kv || a.hv * (D / 8) <= 64) && !kv_fp8 &&
                           a.num_tokens <= 2 * kTokenWaveCapacity;
    const bool two = two_shape && (g_token_waves == 3 || !one);
    // ... and clearly too large for the kernel above to hold all of its waves at once (from 10240 units, five quarters
    // of what it holds; below that the kernel above, gated, is ahead or level: 8.3 against 9.7 us at 1536 tokens of
    // 32+8+8 heads, 9.1 against 9.5 at 2100 tokens of 28+4+4; from there on this one is: 32+8+8 heads 10.3 against
    // 11.1 us at 2048 tokens, 13.6 against 14.8 at 3000, 16.6 against 17.3 at 3700, 16.2 against 18.2 at 4096; 28+4+4
    // heads with three axes 10.0 against 11.7 us at 3000 tokens, 12.2 against 14.5 at 4096).
    // With two tokens per wave from there to twice that many tokens: 4096 waves, four on every SIMD, one token each and
    // the others dealt out evenly.  The SIMD with the most tokens sets the time (the rotation arithmetic of its waves
    // is two thirds of the launch), so the time goes up in steps of 1024 tokens where the kernel above is linear; this
    // one is ahead or level everywhere (graph replays, 28+4+4 heads, one axis / three: 16.1 / 16.4 against 17.2 / 17.5 us
    // at 4800 tokens, 18.2 / 18.5 against 18.4 / 18.8 at 5200, 19.1 / 19.6 against 21.1 / 21.5 at 6144, 21.7 / 21.7 against
    // 23.5 / 23.7 at 7000, 24.2 / 24.4 against 24.7 / 25.3 at 7500, 25.3 / 25.3 against 26.8 / 27.3 at 8192; level below
    // 4608 tokens, where the kernel above stays).  Half as many waves with two tokens each were behind that: 20.0 at 6144 tokens.
    // (in place, with no V row and no scatter, the kernel above holds out a little longer: 9.0 against 9.5 us at 2048
    // tokens of 32+8 heads, then 11.9 against 11.2 at 3000, 15.4 against 13.7 at 4096; 28+4 heads with three axes 10.7
    // against 9.5 at 3000 tokens, 13.2 against 11.5 at 4096, 18.4 against 17.4 at 6144 and 23.2 against 21.6 at 8192 with
    // two tokens per wave)
    const bool large = a.total_units >= (set_kv ? kResidentUnits + kResidentUnits / 4 : kResidentUnits + 2 * kResidentUnits / 5);
    // (with an fp8 cache the conversions lengthen the wave and the gate hardly matters; one token per wave is still
    // ahead once the batch is large: 28+4+4 heads 10.8 against 11.9 us at 3000 tokens, 13.3 against 14.2 at 4096; 32+8+8
    // heads 16.8 against 17.6 at 4096, level at 3000, behind at 2560)
    const bool large_fp8 = a.total_units >= (a.units_per_token == 4 ? kResidentUnits + kResidentUnits / 4 : 7 * kResidentUnits / 4);
    const bool extra_enough = a.num_tokens >= kTokenWaveCapacity + kTokenWaveCapacity / 8;  // (level or 1 % behind below: 15.4 against 15.2 us at 4100 tokens)
    const bool by_rule = g_token_waves == 0 && (two ? extra_enough : (kv_fp8 ? large_fp8 : large));
    p.token_waves = (one || two) && (g_token_waves >= 2 || by_rule);
    p.two_tokens = p.token_waves && two;
    // (with two tokens per wave the full read time: 24.4 us at 8192 tokens of 28+4+4 heads with three axes, against 25.4
    // with 0.95 of it, 24.8 with 1.05, 27.2 with 0.9 -- opening early, into the last reads, costs more than waiting)
    const double gate = g_token_gate >= 0 ? (double)g_token_gate : (double)read_bytes / (two ? 70000.0 : kGateBytesPerTick);
    p.gate = (uint32_t)std::min(gate, 5000.0);
    // The kernel with one wave per unit gates its stores in the same way where its waves are all resident at once
    // (8192 of them, eight per SIMD) and fill at least half of that round.
    // The gate is 1.15 to 1.2 times the read time at 7 TB/s (its waves enter over a few microseconds, and the gate
    // counts from each wave's own entry); from two thirds of a round on the launch is made of four-wave workgroups
    // whatever the head count, because 8192 single-wave workgroups take so long to place that the last waves' reads
    // fall into the first waves' writes.  Measured (us, ungated single-wave workgroups / gated as chosen here): 32+8+8
    // heads 6.6 / 5.9 at 1024 tokens, 7.9 / 7.0 at 1280, 9.1 / 7.7 at 1536, 9.5 / 8.0 at 1638; 64+8+8 heads 5.9 / 5.5 at
    // 512 tokens, 7.4 / 6.6 at 700, 8.9 / 7.4 at 900; 28+4+4 heads 5.8 / 5.4 at 1024 tokens, 7.1 / 6.4 at 1536, 9.1 / 7.5
    // at 2048.  With an fp8 cache (half the bytes to write) or three position axes only from two thirds of a round on:
    // 64+8+8 heads, fp8, 7.6 / 7.4 at 700 tokens, 8.8 / 8.1 at 900; 28+4+4 heads with three axes 7.2 / 6.6 at 1536 tokens,
    // 9.2 / 7.7 at 2048 (5.5 / 5.7 at 1024).  The in-place ops alike: 32+8 heads 5.9 / 5.5 at 1024 tokens, 7.3 / 6.4 at 1400,
    // 8.2 / 7.0 at 1638; 28+4 heads with three axes 6.8 / 6.2 at 1536 tokens, 8.5 / 7.1 at 2048.  Nothing to gain below
    // half a round, 15-35 % slower one unit beyond a round.
    p.unit_gate = 0;
    const bool two_thirds = 3 * a.total_units > 2 * kResidentUnits;
    const bool gated_by_rule = g_unit_gate < 0 && a.total_units <= kResidentUnits &&
                               (two_thirds || (axes == 1 && !kv_fp8 && a.total_units >= kResidentUnits / 2));
    const bool fuller = gated_by_rule && two_thirds;
    if (g_unit_gate > 0) p.unit_gate = (uint32_t)g_unit_gate;
    else if (gated_by_rule) p.unit_gate = (uint32_t)std::min((fuller ? 1.2 : 1.15) * (double)read_bytes / 70000.0, 5000.0);
    // bytes the call moves: every Q/K/V element in, Q (and K) elements out, the cache rows
    const int64_t elems_qk = (int64_t)a.num_tokens * (a.hq + a.hk) * D, elems_v = (int64_t)a.num_tokens * a.hv * D;
    const int64_t call_bytes = set_kv ? 2 * (elems_qk + elems_v) + 2 * (int64_t)a.num_tokens * a.hq * D +
                                            (kv_fp8 ? 1 : 2) * ((int64_t)a.num_tokens * a.hk * D + elems_v)
                                      : 4 * elems_qk;
    p.stream = g_stream_rows == 2 || (g_stream_rows == 0 && call_bytes >= kStreamFromBytes);
    // Workgroup size, swept over 64/128/256/512 lanes and one workgroup per token for 2-9 units per token: four
    // waves where a workgroup then holds whole tokens (its waves share the token's position and table row in the
    // CU's caches: 3-15 % ahead at 28+4 heads) and for large batches (1-3 % ahead from 4096 tokens on), single
    // waves for small batches of other head counts (2-6 % ahead at 64+8 heads with an fp8 cache up to 512 tokens,
    // within 1-3 % either way for 3, 5 and 6 units per token); 128 lanes is the slowest in most cases.
    p.threads = g_block_threads ? (uint32_t)g_block_threads : (a.units_per_token % 4 == 0 || a.total_units > 8192 || fuller ? 256u : 64u);
    const uint32_t units_per_block = p.threads / 64;
    p.blocks = (a.total_units + units_per_block - 1) / units_per_block;
    if (p.token_waves) {
        p.threads = 256;
        // (two tokens per wave: every SIMD's four waves take one token each and the rest are dealt out over them; a
        // batch that two tokens per wave are forced onto although one would do is halved instead)
        p.token_wave_count = !p.two_tokens ? a.num_tokens : a.num_tokens > kTokenWaveCapacity ? kTokenWaveCapacity : (a.num_tokens + 1) / 2;
        p.blocks = (p.token_wave_count + 3) / 4;
        p.stream = true;
    }
    return p;
}

template <typename T, int D, bool NEOX, int AXES, bool SETKV, bool KVFP8>
int launch_one(const RopeArgs &a, hipStream_t stream) {
    const RopePlan p = plan_rope(a, D, AXES, SETKV, KVFP8);
    RopeArgs b = a;
    b.stream_rows = p.stream ? 1u : 0u;
    b.gate = p.unit_gate;
    if constexpr (D == 128 && (AXES == 1 || !KVFP8)) {
        if (p.token_waves) {
#define GPUK_LAUNCH_TOKEN(UPT, TWO)                                                                                    \
    rope_rms_token_kernel<T, D, NEOX, UPT, SETKV, KVFP8, AXES, TWO>                                                    \
        <<<p.blocks, 256, TWO ? 4 * token_kernel_lds_bytes_per_wave(UPT, SETKV) : 0, stream>>>(                        \
            a.qkv_in, a.positions, a.num_tokens, p.gate, a.hq, a.hk, a.hv, p.token_wave_count, a.ps_token, a.ps_axis, b)
            if (p.two_tokens) {
                if constexpr (!KVFP8) {
                    if (a.units_per_token != 4) return GPUK_ERR_INTERNAL;
                    GPUK_LAUNCH_TOKEN(4, true);
                } else {
                    return GPUK_ERR_INTERNAL;
                }
            } else {
                switch (a.units_per_token) {
                    case 4: GPUK_LAUNCH_TOKEN(4, false); break;
                    case 5: GPUK_LAUNCH_TOKEN(5, false); break;
                    default: return GPUK_ERR_INTERNAL;
                }
            }
#undef GPUK_LAUNCH_TOKEN
            return hip_status(hipGetLastError());
        }
    }
    const uint32_t log2_waves = p.threads == 64 ? 0u : p.threads == 128 ? 1u : p.threads == 256 ? 2u : 3u;
#define GPUK_LAUNCH_UNITS(GATED)                                                                                        \
    rope_rms_kernel<T, D, NEOX, AXES, SETKV, KVFP8, GATED><<<p.blocks, p.threads, 0, stream>>>(                         \
        a.qkv_in, a.positions, a.total_units, a.units_per_token, a.upt_magic, a.hq, a.hk,                               \
        (uint32_t)a.hv | (log2_waves << 24), a.ps_token, a.ps_axis, b)
    if (b.gate) GPUK_LAUNCH_UNITS(true);
    else GPUK_LAUNCH_UNITS(false);
#undef GPUK_LAUNCH_UNITS
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

template <typename F, int D, bool NEOX, int AXES>
int launch_wide_mode(const RopeArgs &a, bool set_kv, bool kv_fp8, hipStream_t stream) {
    const uint32_t blocks = (a.total_units + 3) / 4;
    if (!set_kv) rope_rms_wide_kernel<F, D, NEOX, AXES, false, false><<<blocks, 256, 0, stream>>>(a);
    else if (kv_fp8) rope_rms_wide_kernel<F, D, NEOX, AXES, true, true><<<blocks, 256, 0, stream>>>(a);
    else rope_rms_wide_kernel<F, D, NEOX, AXES, true, false><<<blocks, 256, 0, stream>>>(a);
    return hip_status(hipGetLastError());
}

template <typename F, int D>
int launch_wide_style(const RopeArgs &a, bool neox, int n_axes, bool set_kv, bool kv_fp8, hipStream_t stream) {
    if (neox) {
        return n_axes == 3 ? launch_wide_mode<F, D, true, 3>(a, set_kv, kv_fp8, stream)
                           : launch_wide_mode<F, D, true, 1>(a, set_kv, kv_fp8, stream);
    }
    return n_axes == 3 ? launch_wide_mode<F, D, false, 3>(a, set_kv, kv_fp8, stream)
                       : launch_wide_mode<F, D, false, 1>(a, set_kv, kv_fp8, stream);
}

template <typename F>
int launch_wide_head_size(const RopeArgs &a, int64_t head_size, bool neox, int n_axes, bool set_kv, bool kv_fp8,
                          hipStream_t stream) {
    switch (head_size) {
        case 64: return launch_wide_style<F, 64>(a, neox, n_axes, set_kv, kv_fp8, stream);
        case 128: return launch_wide_style<F, 128>(a, neox, n_axes, set_kv, kv_fp8, stream);
        case 256: return launch_wide_style<F, 256>(a, neox, n_axes, set_kv, kv_fp8, stream);
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

// Waves per token of the fp32 / fp64 kernel: 512/D consecutive Q/K heads each, then 128 chunks of the V row each.
int64_t wide_units_per_token(int64_t hq, int64_t hk, int64_t hv, int64_t D, bool set_kv) {
    const int64_t hpw = 512 / D, v_chunks = set_kv ? hv * (D / 4) : 0;
    return (hq + hk + hpw - 1) / hpw + (v_chunks + kWideChunksPerValueUnit - 1) / kWideChunksPerValueUnit;
}

int rope_common(const void *qkv_in, void *qkv_out, const void *qw, const void *kw, const void *cos_sin,
                const int64_t *positions, int64_t ps_axis, int64_t ps_token, int n_axes, int64_t T, int64_t hq,
                int64_t hk, int64_t hv, int64_t D, int neox, const int64_t *section, int interleaved, float eps,
                int dtype, bool set_kv, void *q_out, void *k_cache, void *v_cache, const int64_t *kv_loc,
                float k_scale, float v_scale, int kv_dtype, void *stream) {
    if (T < 0 || hq < 0 || hk < 0 || hv < 0) return GPUK_ERR_INVALID_ARG;
    if (n_axes != 1 && n_axes != 3) return GPUK_ERR_INVALID_ARG;
    if (D != 64 && D != 128 && D != 256) return GPUK_ERR_UNSUPPORTED;
    if (dtype != GPUK_DTYPE_BF16 && dtype != GPUK_DTYPE_FP16 && dtype != GPUK_DTYPE_F32 && dtype != GPUK_DTYPE_F64) return GPUK_ERR_UNSUPPORTED;
    if (set_kv && kv_dtype != GPUK_KV_SAME && kv_dtype != GPUK_KV_E4M3FN) return GPUK_ERR_UNSUPPORTED;
    if (hq > 0x7fffff || hk > 0x7fffff || hv > 0x7fffff) return GPUK_ERR_UNSUPPORTED;
    RopeArgs a{};
    if (n_axes == 3) {
        if (!section) return GPUK_ERR_INVALID_ARG;
        if (section[0] < 0 || section[1] < 0 || section[2] < 0 || section[0] + section[1] + section[2] != D / 2)
            return GPUK_ERR_INVALID_ARG;
        build_axis_bitmaps(section, interleaved != 0, (int)(D / 2), a.axis1, a.axis2);
        a.merge_rows = 1;
        for (int f = 0; f < D / 2; f += 8) {
            const uint32_t g1 = (a.axis1[f >> 5] >> (f & 31)) & 0xffu, g2 = (a.axis2[f >> 5] >> (f & 31)) & 0xffu;
            if ((g1 != 0 && g1 != 0xffu) || (g2 != 0 && g2 != 0xffu)) a.merge_rows = 0;
        }
        if (g_merge_rows == 1) a.merge_rows = 0;
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
    // one wave per group of 64/(D/16) consecutive Q/K heads of a token
    const int64_t hpw = 64 / (D / 16);
    int64_t upt = (hq + hk + hpw - 1) / hpw;
    if (hq + hk == 0) return GPUK_ERR_UNSUPPORTED;  // a qkv row without Q and K heads has nothing to rotate
    const bool wide = dtype == GPUK_DTYPE_F32 || dtype == GPUK_DTYPE_F64;
    if (wide) upt = wide_units_per_token(hq, hk, hv, D, set_kv);
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
    a.num_tokens = (uint32_t)T;
    a.units_per_token = (uint32_t)upt;
    a.upt_magic = upt == 1 ? 0u : (uint32_t)(((1ull << 32) + (uint64_t)upt - 1) / (uint64_t)upt);
    a.hq = (int)hq;
    a.hk = (int)hk;
    a.hv = (int)hv;
    a.eps = eps;
    a.k_scale = k_scale;
    a.v_scale = v_scale;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == GPUK_DTYPE_F32) return launch_wide_head_size<float>(a, D, neox != 0, n_axes, set_kv, kv_fp8, s);
    if (dtype == GPUK_DTYPE_F64) return launch_wide_head_size<double>(a, D, neox != 0, n_axes, set_kv, kv_fp8, s);
    if (dtype == GPUK_DTYPE_BF16) return launch_head_size<BF16>(a, D, neox != 0, n_axes, set_kv, kv_fp8, s);
    return launch_head_size<FP16>(a, D, neox != 0, n_axes, set_kv, kv_fp8, s);
}

int rope_launch_shape(int64_t T, int64_t hq, int64_t hk, int64_t hv, int64_t D, int n_axes, int dtype, bool set_kv,
                      int kv_dtype, int *workgroups, int *lanes, int *streamed, int *token_waves) {
    if (T <= 0 || hq < 0 || hk < 0 || hv < 0 || hq + hk == 0 || (n_axes != 1 && n_axes != 3)) return GPUK_ERR_INVALID_ARG;
    if (D != 64 && D != 128 && D != 256) return GPUK_ERR_UNSUPPORTED;
    if (!workgroups || !lanes || !streamed || !token_waves) return GPUK_ERR_INVALID_ARG;
    *token_waves = 0;
    if (dtype != GPUK_DTYPE_BF16 && dtype != GPUK_DTYPE_FP16 && dtype != GPUK_DTYPE_F32 && dtype != GPUK_DTYPE_F64) return GPUK_ERR_UNSUPPORTED;
    const bool wide = dtype == GPUK_DTYPE_F32 || dtype == GPUK_DTYPE_F64;
    const int64_t hpw = 64 / (D / 16);
    const int64_t upt = wide ? wide_units_per_token(hq, hk, hv, D, set_kv) : (hq + hk + hpw - 1) / hpw;
    if (upt * T >= 0x7fffffffLL || upt * T * upt >= (1LL << 32)) return GPUK_ERR_UNSUPPORTED;
    RopeArgs a{};
    a.total_units = (uint32_t)(upt * T);
    a.num_tokens = (uint32_t)T;
    a.units_per_token = (uint32_t)upt;
    a.hq = (int)hq;
    a.hk = (int)hk;
    a.hv = (int)hv;
    a.merge_rows = g_merge_rows == 1 ? 0u : 1u;  // (three axes: the answer is for sections that split at multiples of 8 frequencies)
    if (wide) {
        *workgroups = (int)((a.total_units + 3) / 4);
        *lanes = 256;
        *streamed = 1;  // the fp32 / fp64 kernel always stores its rotated rows past the L2
        return GPUK_OK;
    }
    const RopePlan p = plan_rope(a, (int)D, n_axes, set_kv, set_kv && kv_dtype == GPUK_KV_E4M3FN);
    *workgroups = (int)p.blocks;
    *lanes = (int)p.threads;
    *streamed = p.stream ? 1 : 0;
    *token_waves = p.token_waves ? (p.two_tokens ? 2 : 1) : 0;
    return GPUK_OK;
}

}  // namespace

void set_rope_tuning(int key, int value) {
    if (key == 0) g_block_threads = value;
    if (key == 6) g_unit_gate = value;
    if (key == 1) g_token_waves = value;
    if (key == 2) g_token_gate = value;
    if (key == 3) g_stream_rows = value;
    if (key == 4) g_merge_rows = value;
}

}  // namespace gpuk

// profiling build: where the kernels of this file write their phase stamps
GPUK_STAMPS_SETTER(gpuk_stamps_set_rope)

extern "C" int gpuk_rope_rms_launch_shape(int64_t num_tokens, int64_t num_heads_q, int64_t num_heads_k,
                                          int64_t num_heads_v, int64_t head_size, int n_axes, int dtype, int set_kv,
                                          int kv_dtype, int *workgroups, int *lanes_per_workgroup,
                                          int *streamed, int *token_waves) {
    return gpuk::rope_launch_shape(num_tokens, num_heads_q, num_heads_k, num_heads_v, head_size, n_axes, dtype,
                                   set_kv != 0, kv_dtype, workgroups, lanes_per_workgroup, streamed, token_waves);
}

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
    if (dtype != GPUK_DTYPE_BF16 && dtype != GPUK_DTYPE_FP16 && dtype != GPUK_DTYPE_F32 && dtype != GPUK_DTYPE_F64) return GPUK_ERR_UNSUPPORTED;
    if (batch_size > 65535) return GPUK_ERR_UNSUPPORTED;  // grid.y
    const bool wide = dtype == GPUK_DTYPE_F32 || dtype == GPUK_DTYPE_F64;
    const int64_t hpw = wide ? 1 : 64 / (head_size / 16);  // rows (heads) per wave
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
    {   // as in the one-wave-per-unit rope kernel: streamed stores are ahead from about 10 MB per call on
        const int64_t call_bytes = 4 * batch_size * (num_tokens0 + num_tokens1) * (num_heads_q + num_heads_k) * head_size;
        a.stream = g_stream_rows == 2 || (g_stream_rows == 0 && call_bytes >= kStreamFromBytes) ? 1u : 0u;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool neox = !is_interleaved;  // reference: fused_rope.cpp:168-227 dispatches the NeoX kernel when !is_interleaved
    if (dtype == GPUK_DTYPE_F32) return launch_2way_wide_head_size<float>(a, head_size, neox, (unsigned)batch_size, s);
    if (dtype == GPUK_DTYPE_F64) return launch_2way_wide_head_size<double>(a, head_size, neox, (unsigned)batch_size, s);
    if (dtype == GPUK_DTYPE_BF16) return launch_2way_head_size<BF16>(a, head_size, neox, (unsigned)batch_size, s);
    return launch_2way_head_size<FP16>(a, head_size, neox, (unsigned)batch_size, s);
}
