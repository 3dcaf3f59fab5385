// Per-head RMSNorm of Q and K + rotary embedding (RoPE / 3-axis mRoPE), written in place or scattered
// to q_out and a paged KV cache.
//
// Stands behind the reference's fused_rope_rms, fused_mrope_3d_rms and fused_mrope_3d_rms_set_kv
// (host ops src/ops/fused_rope.cpp:19-166, kernels src/impl/rope_rms_impl.h:157-466, launchers :468-610).
// The reference maps one 32-lane group to one head with D/32 elements per lane and re-gathers cos/sin
// element by element; here a head is D/16 lanes of a wave64, each lane owning two 16-byte chunks that
// already contain both members of every rotation pair, so no cross-lane exchange is needed for the
// rotation and the sum of squares is reduced inside one 16-lane DPP row.
//
// Numerics follow the reference's torch oracle (test/test_fused_rope_rms.py:8-34,
// test/test_fused_mrope_rms_set_kv.py:62-130), rT = round-to-nearest-even into the 16-bit type:
//     n   = rT(w * rT(x * rstd)),  rstd = 1/sqrt(mean(x^2) + eps)   (fp32, correctly rounded)
//     o1  = rT(rT(n1*cos) - rT(n2*sin)) ;  o2 = rT(rT(n2*cos) + rT(n1*sin))
//     fp8 cache: code = e4m3fn(rT(o / scale)), saturating at +-448
//
// Work decomposition: one wave per (token, head kind q|k|v, group of 64/(D/16) heads).  A wave's lanes
// read 2 KiB of contiguous qkv; K and V rows of a token are contiguous in the cache slot.
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
    uint32_t total_units, units_per_token, groups_q, groups_k;
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

// code = e4m3fn(clamp(rT(v / scale)))
template <typename T>
__device__ __forceinline__ u32x2 quantize_chunk(const u32x4 &v, float scale, float rcp, bool fast) {
    using P = Pack16<T>;
    float q[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float a = P::lo(v[j]), b = P::hi(v[j]);
        if (fast) {
            a = div_by_rcp(a, scale, rcp);
            b = div_by_rcp(b, scale, rcp);
        } else {
            a = a / scale;
            b = b / scale;
        }
        const uint32_t w = P::pack(a, b);
        q[2 * j] = clamp_sym(P::lo(w), kE4M3Max);
        q[2 * j + 1] = clamp_sym(P::hi(w), kE4M3Max);
    }
    return u32x2{cvt4_e4m3fn(q[0], q[1], q[2], q[3]), cvt4_e4m3fn(q[4], q[5], q[6], q[7])};
}

// AXES: 1 = RoPE, 3 = mRoPE.  SETKV: false = in place, true = scatter to q_out / caches.
template <typename T, int D, bool NEOX, int AXES, bool SETKV, bool KVFP8>
__global__ void __launch_bounds__(512) rope_rms_kernel(const RopeArgs a) {
    using P = Pack16<T>;
    constexpr int LPH = D / 16;    // lanes per head
    constexpr int HPW = 64 / LPH;  // heads per wave
    constexpr int HALF = D / 2;

    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t unit = blockIdx.x * (blockDim.x >> 6) + wave;
    if (unit >= a.total_units) return;
    const uint32_t t = unit / a.units_per_token;
    const uint32_t u = unit - t * a.units_per_token;

    const int lane = threadIdx.x & 63;
    const int sub = lane % LPH;
    const int hl = lane / LPH;
    // element offsets of this lane's two chunks inside a head, and of its cos / sin chunks in a table row
    const int c0 = NEOX ? 8 * sub : 16 * sub;
    const int c1 = NEOX ? HALF + 8 * sub : 16 * sub + 8;
    const int fc = 8 * sub;

    const int heads_all = a.hq + a.hk + a.hv;
    const T *dummy = nullptr;
    (void)dummy;

    if (u < a.groups_q + a.groups_k) {
        // ------------------------------------------------------------------ Q or K heads
        const bool is_q = u < a.groups_q;
        const int head = (is_q ? u : u - a.groups_q) * HPW + hl;
        const bool active = head < (is_q ? a.hq : a.hk);
        const int head_in_token = is_q ? head : a.hq + head;
        const int64_t in_off = ((int64_t)t * heads_all + head_in_token) * D;
        const uint16_t *src = static_cast<const uint16_t *>(a.qkv_in) + in_off;
        const uint16_t *w = static_cast<const uint16_t *>(is_q ? a.qw : a.kw);

        u32x4 xa = {0, 0, 0, 0}, xb = {0, 0, 0, 0};
        if (active) {
            xa = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + c0));
            xb = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + c1));
        }
        const u32x4 wa = *reinterpret_cast<const u32x4 *>(w + c0);
        const u32x4 wb = *reinterpret_cast<const u32x4 *>(w + c1);

        const uint16_t *table = static_cast<const uint16_t *>(a.cos_sin);
        const int64_t p0 = a.positions[(int64_t)t * a.ps_token];
        u32x4 cosv = *reinterpret_cast<const u32x4 *>(table + p0 * D + fc);
        u32x4 sinv = *reinterpret_cast<const u32x4 *>(table + p0 * D + HALF + fc);
        if constexpr (AXES == 3) {
            const int64_t p1 = a.positions[a.ps_axis + (int64_t)t * a.ps_token];
            const int64_t p2 = a.positions[2 * a.ps_axis + (int64_t)t * a.ps_token];
            if (p1 != p0 || p2 != p0) {  // wave-uniform; text tokens carry three equal positions
                const u32x4 cos1 = *reinterpret_cast<const u32x4 *>(table + p1 * D + fc);
                const u32x4 sin1 = *reinterpret_cast<const u32x4 *>(table + p1 * D + HALF + fc);
                const u32x4 cos2 = *reinterpret_cast<const u32x4 *>(table + p2 * D + fc);
                const u32x4 sin2 = *reinterpret_cast<const u32x4 *>(table + p2 * D + HALF + fc);
                // 8 axis bits for frequencies fc .. fc+7 (fc is a multiple of 8, so they share a word)
                const uint32_t b1 = (a.axis1[fc >> 5] >> (fc & 31)) & 0xffu;
                const uint32_t b2 = (a.axis2[fc >> 5] >> (fc & 31)) & 0xffu;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t m1 = halves_mask(b1 >> (2 * j)), m2 = halves_mask(b2 >> (2 * j));
                    cosv[j] = bitselect(m2, cos2[j], bitselect(m1, cos1[j], cosv[j]));
                    sinv[j] = bitselect(m2, sin2[j], bitselect(m1, sin1[j], sinv[j]));
                }
            }
        }

        // RMSNorm over the head: D/16 lanes x 16 elements
        float ss0 = 0.f, ss1 = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            ss0 = __builtin_fmaf(P::lo(xa[j]), P::lo(xa[j]), ss0);
            ss1 = __builtin_fmaf(P::hi(xa[j]), P::hi(xa[j]), ss1);
            ss0 = __builtin_fmaf(P::lo(xb[j]), P::lo(xb[j]), ss0);
            ss1 = __builtin_fmaf(P::hi(xb[j]), P::hi(xb[j]), ss1);
        }
        const float sumsq = group_allreduce<SumOp, LPH>(ss0 + ss1);
        const float rstd = 1.0f / sqrtf(sumsq / (float)D + a.eps);

        u32x4 na, nb;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t ta = P::pack(P::lo(xa[j]) * rstd, P::hi(xa[j]) * rstd);
            const uint32_t tb = P::pack(P::lo(xb[j]) * rstd, P::hi(xb[j]) * rstd);
            na[j] = P::pack(P::lo(wa[j]) * P::lo(ta), P::hi(wa[j]) * P::hi(ta));
            nb[j] = P::pack(P::lo(wb[j]) * P::lo(tb), P::hi(wb[j]) * P::hi(tb));
        }

        u32x4 oa, ob;
        if constexpr (NEOX) {
            // chunk a holds x1 for frequencies fc..fc+7, chunk b the matching x2
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float x1l = P::lo(na[j]), x1h = P::hi(na[j]), x2l = P::lo(nb[j]), x2h = P::hi(nb[j]);
                const float cl = P::lo(cosv[j]), ch = P::hi(cosv[j]), sl = P::lo(sinv[j]), sh = P::hi(sinv[j]);
                const uint32_t t1 = P::pack(x1l * cl, x1h * ch), t2 = P::pack(x2l * sl, x2h * sh);
                const uint32_t t3 = P::pack(x2l * cl, x2h * ch), t4 = P::pack(x1l * sl, x1h * sh);
                oa[j] = P::pack(P::lo(t1) - P::lo(t2), P::hi(t1) - P::hi(t2));
                ob[j] = P::pack(P::lo(t3) + P::lo(t4), P::hi(t3) + P::hi(t4));
            }
        } else {
            // each dword is one (x1, x2) pair; chunk a uses frequencies fc..fc+3, chunk b fc+4..fc+7
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                {
                    const float x1 = P::lo(na[e]), x2 = P::hi(na[e]);
                    const float c = elem<T>(cosv, e), s = elem<T>(sinv, e);
                    const uint32_t tc = P::pack(x1 * c, x2 * c), ts = P::pack(x2 * s, x1 * s);
                    oa[e] = P::pack(P::lo(tc) - P::lo(ts), P::hi(tc) + P::hi(ts));
                }
                {
                    const float x1 = P::lo(nb[e]), x2 = P::hi(nb[e]);
                    const float c = elem<T>(cosv, 4 + e), s = elem<T>(sinv, 4 + e);
                    const uint32_t tc = P::pack(x1 * c, x2 * c), ts = P::pack(x2 * s, x1 * s);
                    ob[e] = P::pack(P::lo(tc) - P::lo(ts), P::hi(tc) + P::hi(ts));
                }
            }
        }

        if (!active) return;
        if constexpr (!SETKV) {
            uint16_t *dst = static_cast<uint16_t *>(a.qkv_out) + in_off;
            *reinterpret_cast<u32x4 *>(dst + c0) = oa;
            *reinterpret_cast<u32x4 *>(dst + c1) = ob;
        } else {
            if (is_q) {
                uint16_t *dst = static_cast<uint16_t *>(a.q_out) + ((int64_t)t * a.hq + head) * D;
                *reinterpret_cast<u32x4 *>(dst + c0) = oa;
                *reinterpret_cast<u32x4 *>(dst + c1) = ob;
            } else {
                const int64_t slot = a.kv_loc[t];
                const int64_t off = (slot * a.hk + head) * D;
                if constexpr (!KVFP8) {
                    uint16_t *dst = static_cast<uint16_t *>(a.k_cache) + off;
                    *reinterpret_cast<u32x4 *>(dst + c0) = oa;
                    *reinterpret_cast<u32x4 *>(dst + c1) = ob;
                } else {
                    uint8_t *dst = static_cast<uint8_t *>(a.k_cache) + off;
                    const float s = a.k_scale;
                    const bool fast = s >= 0x1p-60f && s <= 0x1p60f;
                    const float rcp = 1.0f / s;
                    *reinterpret_cast<u32x2 *>(dst + c0) = quantize_chunk<T>(oa, s, rcp, fast);
                    *reinterpret_cast<u32x2 *>(dst + c1) = quantize_chunk<T>(ob, s, rcp, fast);
                }
            }
        }
    } else {
        // ------------------------------------------------------------------ V heads (set_kv only)
        if constexpr (SETKV) {
            const int head = (u - a.groups_q - a.groups_k) * HPW + hl;
            if (head >= a.hv) return;
            const int64_t in_off = ((int64_t)t * heads_all + a.hq + a.hk + head) * D;
            const uint16_t *src = static_cast<const uint16_t *>(a.qkv_in) + in_off;
            const int v0 = 16 * sub, v1 = 16 * sub + 8;
            const u32x4 va = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + v0));
            const u32x4 vb = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + v1));
            const int64_t slot = a.kv_loc[t];
            const int64_t off = (slot * a.hv + head) * D;
            if constexpr (!KVFP8) {
                uint16_t *dst = static_cast<uint16_t *>(a.v_cache) + off;
                *reinterpret_cast<u32x4 *>(dst + v0) = va;
                *reinterpret_cast<u32x4 *>(dst + v1) = vb;
            } else {
                uint8_t *dst = static_cast<uint8_t *>(a.v_cache) + off;
                const float s = a.v_scale;
                const bool fast = s >= 0x1p-60f && s <= 0x1p60f;
                const float rcp = 1.0f / s;
                const u32x2 qa = quantize_chunk<T>(va, s, rcp, fast), qb = quantize_chunk<T>(vb, s, rcp, fast);
                *reinterpret_cast<u32x4 *>(dst + v0) = u32x4{qa[0], qa[1], qb[0], qb[1]};
            }
        }
    }
}

int g_block_threads = 0;  // 0 = default

template <typename T, int D, bool NEOX, int AXES, bool SETKV, bool KVFP8>
int launch_one(const RopeArgs &a, hipStream_t stream) {
    const int threads = g_block_threads ? g_block_threads : 256;
    const uint32_t waves_per_block = threads / 64;
    const uint32_t blocks = (a.total_units + waves_per_block - 1) / waves_per_block;
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
    const int64_t hpw = 64 / (D / 16);
    const int64_t gq = (hq + hpw - 1) / hpw, gk = (hk + hpw - 1) / hpw, gv = set_kv ? (hv + hpw - 1) / hpw : 0;
    const int64_t upt = gq + gk + gv;
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
    a.groups_q = (uint32_t)gq;
    a.groups_k = (uint32_t)gk;
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
