// TEST INFRASTRUCTURE ONLY -- never linked into or loaded by the product.
//
// C entry points around the reference's own rope kernels, built from the reference's headers where they lie
// (-I/root/reference/src/impl -I/root/reference/src/common; nothing of them is copied here):
//   rope_rms::fused_rope_rms<T>                 src/impl/rope_rms_impl.h:468-503
//   rope_rms::fused_mrope_rms<T, 3>             src/impl/rope_rms_impl.h:505-555
//   rope_rms::fused_mrope_rms_set_kv<T, 3, KVT> src/impl/rope_rms_impl.h:557-610
//   rope_rms::fused_rope_rms_2way<T>            src/impl/rope_rms_impl.h:820-857
// called the way the reference's host ops call them (src/ops/fused_rope.cpp:19-227).  The library that results
// (oracle/_ref/libgpuk_ref.so) lets the GPU tests run the reference's kernels and this repository's kernels on the
// same inputs on the same MI355X, and lets the benchmark time them side by side.  bf16 only.
#include "rope_rms_impl.h"

#include <array>
#include <cstdint>

namespace {
using T = __bfloat16;
inline int last_error() { return (int)hipGetLastError(); }
inline bool head_size_ok(int64_t d) { return d == 64 || d == 128 || d == 256; }  // the launchers only assert this
}  // namespace

// n_axes 1: positions [T], ps0 unused (the host op passes 0), ps1 = its stride.  n_axes 3: positions [3, T] with
// strides (ps0, ps1), section[3] summing to head_size / 2.
extern "C" int gpuk_ref_rope_rms(void *qkv, const void *qw, const void *kw, const void *cos_sin, const int64_t *positions,
                                 int64_t ps0, int64_t ps1, int n_axes, int64_t num_tokens, int64_t hq, int64_t hk,
                                 int64_t hv, int64_t head_size, int is_neox, const int64_t *section, int is_interleaved,
                                 double eps, void *stream) {
    if (!head_size_ok(head_size) || num_tokens <= 0 || hq + hk <= 0) return -1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (n_axes == 1) {
        rope_rms::fused_rope_rms<T>(static_cast<T *>(qkv), static_cast<const T *>(qw), static_cast<const T *>(kw),
                                    static_cast<const T *>(cos_sin), positions, 0, ps1, num_tokens, hq, hk, hv, head_size,
                                    is_neox != 0, eps, s);
    } else if (n_axes == 3) {
        if (!section || section[0] + section[1] + section[2] != head_size / 2) return -1;
        const std::array<int64_t, 3> sec = {section[0], section[1], section[2]};
        rope_rms::fused_mrope_rms<T, 3>(static_cast<T *>(qkv), static_cast<const T *>(qw), static_cast<const T *>(kw),
                                        static_cast<const T *>(cos_sin), positions, ps0, ps1, num_tokens, hq, hk, hv,
                                        head_size, is_neox != 0, eps, sec, is_interleaved != 0, s);
    } else {
        return -1;
    }
    return last_error();
}

// positions [3, T] with strides (ps0, ps1); a 1-D position vector is passed as its expansion to three equal rows
// (ps0 = 0).  kv_fp8: the caches hold the reference's 1-byte fp8e4m3fn, else bf16.
extern "C" int gpuk_ref_mrope_rms_set_kv(void *qkv, const void *qw, const void *kw, const void *cos_sin,
                                         const int64_t *positions, int64_t ps0, int64_t ps1, int64_t num_tokens,
                                         int64_t hq, int64_t hk, int64_t hv, int64_t head_size, int is_neox,
                                         const int64_t *section, int is_interleaved, double eps, void *q, void *k_cache,
                                         void *v_cache, int64_t *kv_loc, float k_scale, float v_scale, int kv_fp8,
                                         void *stream) {
    if (!head_size_ok(head_size) || num_tokens <= 0 || hq + hk + hv <= 0) return -1;
    if (!section || section[0] + section[1] + section[2] != head_size / 2) return -1;
    const std::array<int64_t, 3> sec = {section[0], section[1], section[2]};
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (kv_fp8) {
        rope_rms::fused_mrope_rms_set_kv<T, 3, fp8e4m3fn>(
            static_cast<T *>(qkv), static_cast<const T *>(qw), static_cast<const T *>(kw), static_cast<const T *>(cos_sin),
            positions, ps0, ps1, num_tokens, hq, hk, hv, head_size, is_neox != 0, eps, sec, is_interleaved != 0,
            static_cast<T *>(q), static_cast<fp8e4m3fn *>(k_cache), static_cast<fp8e4m3fn *>(v_cache), kv_loc, k_scale,
            v_scale, s);
    } else {
        rope_rms::fused_mrope_rms_set_kv<T, 3, T>(
            static_cast<T *>(qkv), static_cast<const T *>(qw), static_cast<const T *>(kw), static_cast<const T *>(cos_sin),
            positions, ps0, ps1, num_tokens, hq, hk, hv, head_size, is_neox != 0, eps, sec, is_interleaved != 0,
            static_cast<T *>(q), static_cast<T *>(k_cache), static_cast<T *>(v_cache), kv_loc, k_scale, v_scale, s);
    }
    return last_error();
}

extern "C" int gpuk_ref_rope_rms_2way(const void *q0, const void *k0, const void *q1, const void *k1, const void *w_q0,
                                      const void *w_k0, const void *w_q1, const void *w_k1, const void *cos_sin0,
                                      const void *cos_sin1, int64_t batch_size, int64_t num_tokens0, int64_t num_tokens1,
                                      int64_t hq, int64_t hk, int64_t head_size, int is_interleaved, double eps,
                                      void *out_q01, void *out_k01, void *stream) {
    if (!head_size_ok(head_size) || batch_size <= 0 || num_tokens0 + num_tokens1 <= 0 || hq + hk <= 0) return -1;
    rope_rms::fused_rope_rms_2way<T>(
        static_cast<const T *>(q0), static_cast<const T *>(k0), static_cast<const T *>(q1), static_cast<const T *>(k1),
        static_cast<const T *>(w_q0), static_cast<const T *>(w_k0), static_cast<const T *>(w_q1),
        static_cast<const T *>(w_k1), static_cast<const T *>(cos_sin0), static_cast<const T *>(cos_sin1), batch_size,
        num_tokens0, num_tokens1, hq, hk, head_size, is_interleaved != 0, eps, static_cast<T *>(out_q01),
        static_cast<T *>(out_k01), static_cast<hipStream_t>(stream));
    return last_error();
}
