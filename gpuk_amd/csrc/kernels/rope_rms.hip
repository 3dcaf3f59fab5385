// Per-head RMSNorm of Q and K + rotary embedding (RoPE / 3-axis mRoPE), written in place or scattered
// to q_out and a paged KV cache.
//
// Stands behind the reference's fused_rope_rms, fused_mrope_3d_rms and fused_mrope_3d_rms_set_kv
// (host ops src/ops/fused_rope.cpp:19-166, kernels src/impl/rope_rms_impl.h:157-466, launchers :468-610).
// The reference maps one 32-lane group to one head with D/32 elements per lane, fetches the rotation
// partner with two vector shuffles and re-gathers cos/sin element by element for every head.  Here a head
// is D/32 lanes of a wave64 and every lane owns four 16-byte chunks (32 elements) that already contain
// both members of each rotation pair, so the rotation needs no cross-lane traffic, the sum of squares is
// reduced inside one DPP quad or row, and the per-head scalar work (rstd) is shared by twice as many
// elements.  A wave covers 64/(D/32) heads per round and loops over rounds of the same token and kind,
// so the position lookup, the mRoPE axis selection and the cos/sin and weight loads happen once per wave.
//
// Numerics follow the reference's torch oracle (test/test_fused_rope_rms.py:8-34,
// test/test_fused_mrope_rms_set_kv.py:62-130), rT = round-to-nearest-even into the 16-bit type:
//     n   = rT(w * rT(x * rstd)),  rstd = 1/sqrt(mean(x^2) + eps)   (fp32, correctly rounded)
//     o1  = rT(rT(n1*cos) - rT(n2*sin)) ;  o2 = rT(rT(n2*cos) + rT(n1*sin))
//     fp8 cache: code = e4m3fn(rT(o / scale)), saturating at +-448
#include <hip/hip_runtime.h>

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
    // work decomposition: a unit is (token, kind q|k|v, block of `rounds_per_wave` rounds); one wave per unit
    uint32_t total_units, units_per_token, units_q, units_k, rounds_per_wave;
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

// Divides by a scale that is the same for the whole launch; `rcp` is RN(1/scale) when `fast`.
struct Divider {
    float scale, rcp;
    bool fast;
    __device__ __forceinline__ explicit Divider(float s)
        : scale(s), rcp(1.0f / s), fast(s >= 0x1p-60f && s <= 0x1p60f) {}
    __device__ __forceinline__ float operator()(float a) const {
        return fast ? div_by_rcp(a, scale, rcp) : a / scale;
    }
};

// 8 codes = e4m3fn(clamp(rT(v / scale))) for one chunk
template <typename T, bool FAST>
__device__ __forceinline__ u32x2 quantize_chunk(const u32x4 &v, const Divider &d) {
    using P = Pack16<T>;
    float q[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float a = FAST ? div_by_rcp(P::lo(v[j]), d.scale, d.rcp) : P::lo(v[j]) / d.scale;
        const float b = FAST ? div_by_rcp(P::hi(v[j]), d.scale, d.rcp) : P::hi(v[j]) / d.scale;
        const uint32_t w = P::pack(a, b);
        q[2 * j] = clamp_sym(P::lo(w), kE4M3Max);
        q[2 * j + 1] = clamp_sym(P::hi(w), kE4M3Max);
    }
    return u32x2{cvt4_e4m3fn(q[0], q[1], q[2], q[3]), cvt4_e4m3fn(q[4], q[5], q[6], q[7])};
}

// Chunk ids (units of 8 elements inside a head) owned by lane `sub` of the head's LPH = D/(8*CPL) lanes, for
// CPL = 2 or 4 chunks per lane.  HC = chunks per half head.
//   NeoX  : the first CPL/2 slots come from the first half of the head, slot i + CPL/2 is the chunk D/2 elements
//           further, so slot i pairs with slot i + CPL/2 under table chunk i.
//   GPT-J : runs of two adjacent chunks {2sub, 2sub+1} (and {2sub+HC, 2sub+1+HC} for CPL 4); pairs sit inside a
//           chunk, and a run of two chunks uses one table chunk.
// In both styles the lane's rotary frequencies are the table chunks {sub} (CPL 2) or {sub, sub+LPH} (CPL 4) of
// the cos half and of the sin half.
template <int D, bool NEOX, int CPL>
__device__ __forceinline__ void chunk_ids(int sub, int (&c)[CPL]) {
    constexpr int HC = D / 16, LPH = D / (8 * CPL);
    if constexpr (NEOX) {
#pragma unroll
        for (int i = 0; i < CPL / 2; ++i) {
            c[i] = sub + i * LPH;
            c[i + CPL / 2] = HC + sub + i * LPH;
        }
    } else {
#pragma unroll
        for (int i = 0; i < CPL / 2; ++i) {
            c[2 * i] = 2 * sub + i * HC;
            c[2 * i + 1] = 2 * sub + 1 + i * HC;
        }
    }
}

// Keeps the compiler from hoisting the unpacking of a loop-invariant packed dword out of the round loop
// (the unpacked copies would double the register count and halve the occupancy).
__device__ __forceinline__ uint32_t opaque(uint32_t v) {
    asm volatile("" : "+v"(v));
    return v;
}

// AXES: 1 = RoPE, 3 = mRoPE.  SETKV: false = in place, true = scatter to q_out / caches.
// CPL: 16-byte chunks per lane and head (2 or 4).
template <typename T, int D, bool NEOX, int AXES, bool SETKV, bool KVFP8, int CPL>
__global__ void __launch_bounds__(512) rope_rms_kernel(const RopeArgs a) {
    using P = Pack16<T>;
    constexpr int LPH = D / (8 * CPL);  // lanes per head
    constexpr int HPW = 64 / LPH;       // heads per wave and round
    constexpr int HALF = D / 2;
    constexpr int NT = CPL / 2;         // table chunks (of cos and of sin) per lane

    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t unit = blockIdx.x * (blockDim.x >> 6) + wave;
    if (unit >= a.total_units) return;
    const uint32_t t = unit / a.units_per_token;
    const uint32_t u = unit - t * a.units_per_token;

    const int lane = threadIdx.x & 63;
    const int sub = lane % LPH;
    const int hl = lane / LPH;
    const int heads_all = a.hq + a.hk + a.hv;
    const uint16_t *token_in = static_cast<const uint16_t *>(a.qkv_in) + (int64_t)t * heads_all * D;

    if (u < a.units_q + a.units_k) {
        // ------------------------------------------------------------------ Q or K heads
        const bool is_q = u < a.units_q;
        const int heads_kind = is_q ? a.hq : a.hk;
        const int head_base = is_q ? 0 : a.hq;  // first head of this kind inside the token
        const int round0 = (is_q ? u : u - a.units_q) * a.rounds_per_wave;
        const int rounds_kind = (heads_kind + HPW - 1) / HPW;
        const int round1 = min(round0 + (int)a.rounds_per_wave, rounds_kind);

        int cid[CPL];
        chunk_ids<D, NEOX, CPL>(sub, cid);
        // Lanes past the last head of the kind re-read the last head (their results are never stored): the load
        // needs no branch, which keeps the compiler's wait counters exact inside the round loop.
        auto load_head = [&](int round, u32x4(&x)[CPL]) {
            const int head = min(round * HPW + hl, heads_kind - 1);
            const uint16_t *src = token_in + (int64_t)(head_base + head) * D;
#pragma unroll
            for (int i = 0; i < CPL; ++i) x[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + 8 * cid[i]));
        };
        u32x4 cur[CPL], nxt[CPL];
        load_head(round0, cur);

        // per-wave constants: norm weights of the lane's chunks, cos / sin of the lane's frequencies
        const uint16_t *wsrc = static_cast<const uint16_t *>(is_q ? a.qw : a.kw);
        u32x4 w[CPL];
#pragma unroll
        for (int i = 0; i < CPL; ++i) w[i] = *reinterpret_cast<const u32x4 *>(wsrc + 8 * cid[i]);

        const uint16_t *table = static_cast<const uint16_t *>(a.cos_sin);
        const int64_t p0 = a.positions[(int64_t)t * a.ps_token];
        u32x4 cosv[NT], sinv[NT];
#pragma unroll
        for (int k = 0; k < NT; ++k) {
            const int f = 8 * (sub + k * LPH);  // first frequency of the lane's table chunk k
            cosv[k] = *reinterpret_cast<const u32x4 *>(table + p0 * D + f);
            sinv[k] = *reinterpret_cast<const u32x4 *>(table + p0 * D + HALF + f);
        }
        if constexpr (AXES == 3) {
            const int64_t p1 = a.positions[a.ps_axis + (int64_t)t * a.ps_token];
            const int64_t p2 = a.positions[2 * a.ps_axis + (int64_t)t * a.ps_token];
            if (p1 != p0 || p2 != p0) {  // wave-uniform; text tokens carry three equal positions
#pragma unroll
                for (int k = 0; k < NT; ++k) {
                    const int f = 8 * (sub + k * LPH);
                    const u32x4 cos1 = *reinterpret_cast<const u32x4 *>(table + p1 * D + f);
                    const u32x4 sin1 = *reinterpret_cast<const u32x4 *>(table + p1 * D + HALF + f);
                    const u32x4 cos2 = *reinterpret_cast<const u32x4 *>(table + p2 * D + f);
                    const u32x4 sin2 = *reinterpret_cast<const u32x4 *>(table + p2 * D + HALF + f);
                    // 8 axis bits for frequencies f .. f+7 (f is a multiple of 8, so they share a word)
                    const uint32_t b1 = (a.axis1[f >> 5] >> (f & 31)) & 0xffu;
                    const uint32_t b2 = (a.axis2[f >> 5] >> (f & 31)) & 0xffu;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t m1 = halves_mask(b1 >> (2 * j)), m2 = halves_mask(b2 >> (2 * j));
                        cosv[k][j] = bitselect(m2, cos2[j], bitselect(m1, cos1[j], cosv[k][j]));
                        sinv[k][j] = bitselect(m2, sin2[j], bitselect(m1, sin1[j], sinv[k][j]));
                    }
                }
            }
        }

        int64_t slot = 0;
        if constexpr (SETKV) {
            if (!is_q) slot = a.kv_loc[t];
        }
        const Divider kdiv(a.k_scale);
        // row of head 0 of this kind in the 16-bit destination (in place / q_out / k_cache slot)
        uint16_t *out_row;
        if constexpr (!SETKV) out_row = static_cast<uint16_t *>(a.qkv_out) + ((int64_t)t * heads_all + head_base) * D;
        else out_row = is_q ? static_cast<uint16_t *>(a.q_out) + (int64_t)t * a.hq * D
                            : static_cast<uint16_t *>(a.k_cache) + slot * a.hk * D;

        // All set-up loads (weights, cos/sin, first round) have to land before the loop: the waits the compiler
        // would otherwise place inside it also cover the prefetch of the next round and serialise the rounds.
        if (round1 - round0 > 1) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
#pragma unroll 1
        for (int round = round0; round < round1; ++round) {
            if (round + 1 < round1) load_head(round + 1, nxt);

            // RMSNorm over the head: LPH lanes x 8*CPL elements
            float ss0 = 0.f, ss1 = 0.f;
#pragma unroll
            for (int i = 0; i < CPL; ++i) {
                ss0 = P::add_squares(cur[i][0], ss0);
                ss1 = P::add_squares(cur[i][1], ss1);
                ss0 = P::add_squares(cur[i][2], ss0);
                ss1 = P::add_squares(cur[i][3], ss1);
            }
            const float sumsq = group_allreduce<SumOp, LPH>(ss0 + ss1);
            const float rstd = 1.0f / sqrtf(sumsq * (1.0f / D) + a.eps);  // D is a power of two: exact

            u32x4 n[CPL];
#pragma unroll
            for (int i = 0; i < CPL; ++i) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t wj = opaque(w[i][j]);
                    const uint32_t s = P::pack(P::lo(cur[i][j]) * rstd, P::hi(cur[i][j]) * rstd);
                    n[i][j] = P::pack(P::lo(wj) * P::lo(s), P::hi(wj) * P::hi(s));
                }
            }

            u32x4 o[CPL];
            if constexpr (NEOX) {
                // slot i holds x1 and slot i + CPL/2 the matching x2 for the 8 frequencies of table chunk i
#pragma unroll
                for (int i = 0; i < NT; ++i) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t cj = opaque(cosv[i][j]), sj = opaque(sinv[i][j]);
                        const float x1l = P::lo(n[i][j]), x1h = P::hi(n[i][j]);
                        const float x2l = P::lo(n[i + NT][j]), x2h = P::hi(n[i + NT][j]);
                        const float cl = P::lo(cj), ch = P::hi(cj), sl = P::lo(sj), sh = P::hi(sj);
                        const uint32_t t1 = P::pack(x1l * cl, x1h * ch), t2 = P::pack(x2l * sl, x2h * sh);
                        const uint32_t t3 = P::pack(x2l * cl, x2h * ch), t4 = P::pack(x1l * sl, x1h * sh);
                        o[i][j] = P::pack(P::lo(t1) - P::lo(t2), P::hi(t1) - P::hi(t2));
                        o[i + NT][j] = P::pack(P::lo(t3) + P::lo(t4), P::hi(t3) + P::hi(t4));
                    }
                }
            } else {
                // each dword is one (x1, x2) pair; slots 2k, 2k+1 use elements 0-3 and 4-7 of table chunk k
#pragma unroll
                for (int i = 0; i < CPL; ++i) {
                    u32x4 ck, sk;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        ck[j] = opaque(cosv[i >> 1][j]);
                        sk[j] = opaque(sinv[i >> 1][j]);
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float x1 = P::lo(n[i][e]), x2 = P::hi(n[i][e]);
                        const float c = elem<T>(ck, 4 * (i & 1) + e), s = elem<T>(sk, 4 * (i & 1) + e);
                        const uint32_t tc = P::pack(x1 * c, x2 * c), ts = P::pack(x2 * s, x1 * s);
                        o[i][e] = P::pack(P::lo(tc) - P::lo(ts), P::hi(tc) + P::hi(ts));
                    }
                }
            }

            // The prefetch has had the whole round to land.  Waiting for it here, while it is the youngest
            // outstanding access, keeps this round's stores out of the wait.
            if (round + 1 < round1) {
                __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
#pragma unroll
                for (int i = 0; i < CPL; ++i) cur[i] = nxt[i];
            }
            const int head = round * HPW + hl;
            if (head < heads_kind) {
                if (KVFP8 && !is_q) {
                    uint8_t *dst = static_cast<uint8_t *>(a.k_cache) + (slot * a.hk + head) * D;
                    if (kdiv.fast) {
#pragma unroll
                        for (int i = 0; i < CPL; ++i)
                            *reinterpret_cast<u32x2 *>(dst + 8 * cid[i]) = quantize_chunk<T, true>(o[i], kdiv);
                    } else {
#pragma unroll 1
                        for (int i = 0; i < CPL; ++i)
                            *reinterpret_cast<u32x2 *>(dst + 8 * cid[i]) = quantize_chunk<T, false>(o[i], kdiv);
                    }
                } else {
                    // one store sequence for every 16-bit destination; `out_row` is wave-uniform
#pragma unroll
                    for (int i = 0; i < CPL; ++i) *reinterpret_cast<u32x4 *>(out_row + (int64_t)head * D + 8 * cid[i]) = o[i];
                }
            }
        }
    } else {
        // ------------------------------------------------------------------ V heads (set_kv only): copy or quantise
        if constexpr (SETKV) {
            const int round0 = (u - a.units_q - a.units_k) * a.rounds_per_wave;
            const int rounds_kind = (a.hv + HPW - 1) / HPW;
            const int round1 = min(round0 + (int)a.rounds_per_wave, rounds_kind);
            const int64_t slot = a.kv_loc[t];
            const Divider vdiv(a.v_scale);
            for (int round = round0; round < round1; ++round) {
                const int head = round * HPW + hl;
                if (head >= a.hv) continue;
                const uint16_t *src = token_in + (int64_t)(a.hq + a.hk + head) * D;
                const int64_t off = (slot * a.hv + head) * D;
                if constexpr (!KVFP8) {
                    // chunk i*LPH + sub: every load / store instruction covers LPH*16 contiguous bytes per head
                    u32x4 v[CPL];
#pragma unroll
                    for (int i = 0; i < CPL; ++i)
                        v[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + 8 * (i * LPH + sub)));
                    uint16_t *dst = static_cast<uint16_t *>(a.v_cache) + off;
#pragma unroll
                    for (int i = 0; i < CPL; ++i) *reinterpret_cast<u32x4 *>(dst + 8 * (i * LPH + sub)) = v[i];
                } else {
                    // adjacent chunk pairs {2sub, 2sub+1} (+ 2*LPH per further pair): 16 codes leave as one 16-byte store
                    u32x4 v[CPL];
#pragma unroll
                    for (int i = 0; i < CPL; ++i)
                        v[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + 8 * (2 * sub + (i & 1) + (i >> 1) * 2 * LPH)));
                    uint8_t *dst = static_cast<uint8_t *>(a.v_cache) + off;
                    if (vdiv.fast) {
#pragma unroll
                        for (int h = 0; h < CPL / 2; ++h) {
                            const u32x2 qa = quantize_chunk<T, true>(v[2 * h], vdiv), qb = quantize_chunk<T, true>(v[2 * h + 1], vdiv);
                            *reinterpret_cast<u32x4 *>(dst + 8 * (2 * sub + h * 2 * LPH)) = u32x4{qa[0], qa[1], qb[0], qb[1]};
                        }
                    } else {
#pragma unroll 1
                        for (int h = 0; h < CPL / 2; ++h) {
                            const u32x2 qa = quantize_chunk<T, false>(v[2 * h], vdiv), qb = quantize_chunk<T, false>(v[2 * h + 1], vdiv);
                            *reinterpret_cast<u32x4 *>(dst + 8 * (2 * sub + h * 2 * LPH)) = u32x4{qa[0], qa[1], qb[0], qb[1]};
                        }
                    }
                }
            }
        }
    }
}

int g_block_threads = 0;    // 0 = default
int g_rounds_per_wave = 0;  // 0 = heuristic
int g_chunks_per_lane = 2;  // 2 or 4

template <typename T, int D, bool NEOX, int AXES, bool SETKV, bool KVFP8>
int launch_one(const RopeArgs &a, hipStream_t stream) {
    const int threads = g_block_threads ? g_block_threads : 256;
    const uint32_t waves_per_block = threads / 64;
    const uint32_t blocks = (a.total_units + waves_per_block - 1) / waves_per_block;
    if (g_chunks_per_lane == 4)
        rope_rms_kernel<T, D, NEOX, AXES, SETKV, KVFP8, 4><<<blocks, threads, 0, stream>>>(a);
    else
        rope_rms_kernel<T, D, NEOX, AXES, SETKV, KVFP8, 2><<<blocks, threads, 0, stream>>>(a);
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
    if (dtype != GPUK_DTYPE_BF16 && dtype != GPUK_DTYPE_FP16) return GPUK_ERR_UNSUPPORTED;
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
        if (!q_out || !k_cache || !v_cache || !kv_loc) return GPUK_ERR_INVALID_ARG;
        if (!aligned16(q_out) || !aligned16(k_cache) || !aligned16(v_cache)) return GPUK_ERR_MISALIGNED;
        if (kv_fp8 && !(k_scale > 0.f && v_scale > 0.f)) return GPUK_ERR_INVALID_ARG;
    }
    // Heads per wave-round, rounds per kind, and how many rounds one wave takes on.  One round per wave
    // measured fastest at every size tried (more waves in flight hide the position -> cos/sin dependent loads
    // better than a longer wave with a one-round prefetch does); larger values stay selectable for tuning.
    const int64_t hpw = 64 / (D / (8 * g_chunks_per_lane));
    const int64_t rq = (hq + hpw - 1) / hpw, rk = (hk + hpw - 1) / hpw, rv = set_kv ? (hv + hpw - 1) / hpw : 0;
    const int64_t rpw = g_rounds_per_wave ? g_rounds_per_wave : 1;
    const int64_t uq = (rq + rpw - 1) / rpw, uk = (rk + rpw - 1) / rpw, uv = (rv + rpw - 1) / rpw;
    const int64_t upt = uq + uk + uv;
    if (upt * T >= 0x7fffffffLL) return GPUK_ERR_UNSUPPORTED;
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
    a.units_q = (uint32_t)uq;
    a.units_k = (uint32_t)uk;
    a.rounds_per_wave = (uint32_t)rpw;
    a.hq = (int)hq;
    a.hk = (int)hk;
    a.hv = (int)hv;
    a.eps = eps;
    a.k_scale = k_scale;
    a.v_scale = v_scale;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == GPUK_DTYPE_BF16) return launch_head_size<BF16>(a, D, neox != 0, n_axes, set_kv, kv_fp8, s);
    return launch_head_size<FP16>(a, D, neox != 0, n_axes, set_kv, kv_fp8, s);
}

}  // namespace

void set_rope_tuning(int key, int value) {
    if (key == 0) g_block_threads = value;
    if (key == 1) g_rounds_per_wave = value;
    if (key == 2) g_chunks_per_lane = value;
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
