// fused_rope_rms / fused_mrope_3d_rms / fused_mrope_3d_rms_set_kv (+ the additive fused_rope_rms_set_kv).
// Mirrors the host ops at src/ops/fused_rope.cpp:19-166: same argument order, contiguity checks, positions
// passed by stride, KV-cache dtype decided by comparing it with qkv's dtype (:114).
#include "ops.h"

namespace gpuk_ops {

namespace {

struct RopeCall {
    const char *op;
    int n_axes;
    const int64_t *section;
    bool interleaved;
};

void check_common(const char *op, const Tensor &qkv, const Tensor &qw, const Tensor &kw, const Tensor &cos_sin,
                  const Tensor &positions, int n_axes, int64_t num_tokens, int64_t hq, int64_t hk, int64_t hv,
                  int64_t head_size) {
    TORCH_CHECK(qkv.is_contiguous() && qw.is_contiguous() && kw.is_contiguous() && cos_sin.is_contiguous());
    TORCH_CHECK(positions.dim() == (n_axes == 1 ? 1 : 2), op, ": positions must be ", n_axes == 1 ? "1-D [T]" : "2-D [3, T]");
    TORCH_CHECK(positions.scalar_type() == at::kLong, op, ": positions must be int64");
    TORCH_CHECK(head_size == 64 || head_size == 128 || head_size == 256, op, ": head_size must be 64, 128 or 256");
    TORCH_CHECK(num_tokens >= 0 && hq >= 0 && hk >= 0 && hv >= 0, op, ": negative size");
    TORCH_CHECK(qkv.numel() == num_tokens * (hq + hk + hv) * head_size, op, ": qkv does not hold num_tokens*(hq+hk+hv)*head_size elements");
    TORCH_CHECK(qw.numel() == head_size && kw.numel() == head_size, op, ": qw and kw must hold head_size elements");
    TORCH_CHECK(cos_sin.numel() % head_size == 0, op, ": cos_sin must be [max_positions, head_size]");
    TORCH_CHECK(positions.size(-1) >= num_tokens && (n_axes == 1 || positions.size(0) == 3), op, ": positions shape");
    const auto act = qkv.scalar_type();
    TORCH_CHECK(qw.scalar_type() == act && kw.scalar_type() == act && cos_sin.scalar_type() == act, op,
                ": qw, kw and cos_sin must share qkv's dtype");
    TORCH_CHECK(qkv.is_cuda(), op, ": tensors must live on the GPU");
    const auto dev = qkv.device();
    TORCH_CHECK(qw.device() == dev && kw.device() == dev && cos_sin.device() == dev && positions.device() == dev, op,
                ": all tensors must be on the same device");
}

void run_inplace(const RopeCall &c, Tensor &qkv, Tensor &qw, Tensor &kw, Tensor &cos_sin, Tensor &positions,
                 int64_t num_tokens, int64_t hq, int64_t hk, int64_t hv, int64_t head_size, bool is_neox, double eps) {
    check_common(c.op, qkv, qw, kw, cos_sin, positions, c.n_axes, num_tokens, hq, hk, hv, head_size);
    const int dtype = activation_dtype(qkv, c.op);
    const auto st = positions.strides();
    DeviceGuard guard(qkv.device());
    const int status = gpuk_rope_rms(qkv.data_ptr(), qw.data_ptr(), kw.data_ptr(), cos_sin.data_ptr(),
                                     positions.data_ptr<int64_t>(), c.n_axes == 3 ? st[0] : 0, st[c.n_axes == 3 ? 1 : 0],
                                     c.n_axes, num_tokens, hq, hk, hv, head_size, is_neox, c.section, c.interleaved,
                                     (float)eps, dtype, current_stream());
    check_status(status, c.op);
}

void run_set_kv(const RopeCall &c, Tensor &qkv, Tensor &qw, Tensor &kw, Tensor &cos_sin, Tensor &positions,
                int64_t num_tokens, int64_t hq, int64_t hk, int64_t hv, int64_t head_size, bool is_neox, double eps,
                Tensor &q, Tensor &k_cache, Tensor &v_cache, Tensor &kv_loc, double k_scale, double v_scale) {
    check_common(c.op, qkv, qw, kw, cos_sin, positions, c.n_axes, num_tokens, hq, hk, hv, head_size);
    TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && kv_loc.is_contiguous());
    TORCH_CHECK(q.is_contiguous(), c.op, ": q must be contiguous");
    TORCH_CHECK(q.scalar_type() == qkv.scalar_type() && q.numel() == num_tokens * hq * head_size, c.op,
                ": q must be [num_tokens, num_heads_q, head_size] of qkv's dtype");
    TORCH_CHECK(kv_loc.scalar_type() == at::kLong && kv_loc.numel() >= num_tokens, c.op, ": kv_loc must be int64 [num_tokens]");
    TORCH_CHECK(k_cache.scalar_type() == v_cache.scalar_type(), c.op, ": k_cache and v_cache must share a dtype");
    const bool same = k_cache.scalar_type() == qkv.scalar_type();
    TORCH_CHECK(same || k_cache.element_size() == 1, c.op, ": the KV cache must have qkv's dtype or a 1-byte fp8 dtype");
    TORCH_CHECK(k_cache.numel() % std::max<int64_t>(hk * head_size, 1) == 0 && v_cache.numel() % std::max<int64_t>(hv * head_size, 1) == 0,
                c.op, ": caches must be [slots, heads, head_size]");
    const auto dev = qkv.device();
    TORCH_CHECK(q.device() == dev && k_cache.device() == dev && v_cache.device() == dev && kv_loc.device() == dev, c.op,
                ": all tensors must be on the same device");
    const int dtype = activation_dtype(qkv, c.op);
    const auto st = positions.strides();
    DeviceGuard guard(dev);
    const int status = gpuk_rope_rms_set_kv(
        qkv.data_ptr(), qw.data_ptr(), kw.data_ptr(), cos_sin.data_ptr(), positions.data_ptr<int64_t>(),
        c.n_axes == 3 ? st[0] : 0, st[c.n_axes == 3 ? 1 : 0], c.n_axes, num_tokens, hq, hk, hv, head_size, is_neox,
        c.section, c.interleaved, (float)eps, dtype, q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
        kv_loc.data_ptr<int64_t>(), (float)k_scale, (float)v_scale, same ? GPUK_KV_SAME : GPUK_KV_E4M3FN, current_stream());
    check_status(status, c.op);
}

}  // namespace

void fused_rope_rms(Tensor &qkv, Tensor &qw, Tensor &kw, Tensor &cos_sin, Tensor &positions, int64_t num_tokens,
                    int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v, int64_t head_size,
                    bool is_neox_style, double eps) {
    run_inplace({"fused_rope_rms", 1, nullptr, false}, qkv, qw, kw, cos_sin, positions, num_tokens, num_heads_q,
                num_heads_k, num_heads_v, head_size, is_neox_style, eps);
}

void fused_mrope_3d_rms(Tensor &qkv, Tensor &qw, Tensor &kw, Tensor &cos_sin, Tensor &positions, int64_t num_tokens,
                        int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v, int64_t head_size,
                        bool is_neox_style, std::vector<int64_t> mrope_section_, bool is_interleaved, double eps) {
    TORCH_CHECK(mrope_section_.size() == 3);
    run_inplace({"fused_mrope_3d_rms", 3, mrope_section_.data(), is_interleaved}, qkv, qw, kw, cos_sin, positions,
                num_tokens, num_heads_q, num_heads_k, num_heads_v, head_size, is_neox_style, eps);
}

void fused_mrope_3d_rms_set_kv(Tensor &qkv, Tensor &qw, Tensor &kw, Tensor &cos_sin, Tensor &positions,
                               int64_t num_tokens, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                               int64_t head_size, bool is_neox_style, std::vector<int64_t> mrope_section_,
                               bool is_interleaved, double eps, Tensor &q, Tensor &k_cache, Tensor &v_cache,
                               Tensor &kv_loc, double k_scale, double v_scale) {
    TORCH_CHECK(mrope_section_.size() == 3);
    run_set_kv({"fused_mrope_3d_rms_set_kv", 3, mrope_section_.data(), is_interleaved}, qkv, qw, kw, cos_sin, positions,
               num_tokens, num_heads_q, num_heads_k, num_heads_v, head_size, is_neox_style, eps, q, k_cache, v_cache,
               kv_loc, k_scale, v_scale);
}

void fused_rope_rms_set_kv(Tensor &qkv, Tensor &qw, Tensor &kw, Tensor &cos_sin, Tensor &positions, int64_t num_tokens,
                           int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v, int64_t head_size,
                           bool is_neox_style, double eps, Tensor &q, Tensor &k_cache, Tensor &v_cache, Tensor &kv_loc,
                           double k_scale, double v_scale) {
    run_set_kv({"fused_rope_rms_set_kv", 1, nullptr, false}, qkv, qw, kw, cos_sin, positions, num_tokens, num_heads_q,
               num_heads_k, num_heads_v, head_size, is_neox_style, eps, q, k_cache, v_cache, kv_loc, k_scale, v_scale);
}

// fused_rope_rms_2way: shape inference shared by the Meta and the GPU kernel (src/ops/fused_rope.cpp:168-182).
std::tuple<Tensor, Tensor> fused_rope_rms_2way_meta(Tensor &q0, Tensor &k0, Tensor &q1, Tensor &k1, Tensor &w_q0,
                                                    Tensor &w_k0, Tensor &w_q1, Tensor &w_k1, Tensor &cos_sin0,
                                                    Tensor &cos_sin1, int64_t batch_size, int64_t num_tokens0,
                                                    int64_t num_tokens1, int64_t num_heads_q, int64_t num_heads_k,
                                                    int64_t head_size, bool is_interleaved, double eps) {
    TORCH_CHECK(q0.is_contiguous() && k0.is_contiguous() && q1.is_contiguous() && k1.is_contiguous());
    TORCH_CHECK(w_q0.is_contiguous() && w_k0.is_contiguous() && w_q1.is_contiguous() && w_k1.is_contiguous());
    TORCH_CHECK(cos_sin0.is_contiguous() && cos_sin1.is_contiguous());
    Tensor out_q01 = at::empty({batch_size, num_tokens0 + num_tokens1, num_heads_q, head_size}, q0.options());
    Tensor out_k01 = at::empty({batch_size, num_tokens0 + num_tokens1, num_heads_k, head_size}, k0.options());
    return std::make_tuple(std::move(out_q01), std::move(out_k01));
}

std::tuple<Tensor, Tensor> fused_rope_rms_2way(Tensor &q0, Tensor &k0, Tensor &q1, Tensor &k1, Tensor &w_q0, Tensor &w_k0,
                                               Tensor &w_q1, Tensor &w_k1, Tensor &cos_sin0, Tensor &cos_sin1,
                                               int64_t batch_size, int64_t num_tokens0, int64_t num_tokens1,
                                               int64_t num_heads_q, int64_t num_heads_k, int64_t head_size,
                                               bool is_interleaved, double eps) {
    const char *op = "fused_rope_rms_2way";
    auto outs = fused_rope_rms_2way_meta(q0, k0, q1, k1, w_q0, w_k0, w_q1, w_k1, cos_sin0, cos_sin1, batch_size,
                                         num_tokens0, num_tokens1, num_heads_q, num_heads_k, head_size, is_interleaved, eps);
    TORCH_CHECK(head_size == 64 || head_size == 128 || head_size == 256, op, ": head_size must be 64, 128 or 256");
    TORCH_CHECK(q0.numel() == batch_size * num_tokens0 * num_heads_q * head_size &&
                    k0.numel() == batch_size * num_tokens0 * num_heads_k * head_size &&
                    q1.numel() == batch_size * num_tokens1 * num_heads_q * head_size &&
                    k1.numel() == batch_size * num_tokens1 * num_heads_k * head_size,
                op, ": q0/k0/q1/k1 must be [batch, tokens, heads, head_size]");
    TORCH_CHECK(w_q0.numel() == head_size && w_k0.numel() == head_size && w_q1.numel() == head_size &&
                    w_k1.numel() == head_size, op, ": the norm weights must hold head_size elements");
    TORCH_CHECK(cos_sin0.numel() == num_tokens0 * head_size && cos_sin1.numel() == num_tokens1 * head_size, op,
                ": cos_sin0/1 must be [num_tokens, head_size]");
    const auto act = q0.scalar_type();
    for (const Tensor *t : {&k0, &q1, &k1, &w_q0, &w_k0, &w_q1, &w_k1, &cos_sin0, &cos_sin1}) {
        TORCH_CHECK(t->scalar_type() == act, op, ": all tensors must share q0's dtype");
        TORCH_CHECK(t->device() == q0.device(), op, ": all tensors must be on the same device");
    }
    TORCH_CHECK(q0.is_cuda(), op, ": tensors must live on the GPU");
    const int dtype = activation_dtype(q0, op);
    DeviceGuard guard(q0.device());
    const int status = gpuk_rope_rms_2way(q0.data_ptr(), k0.data_ptr(), q1.data_ptr(), k1.data_ptr(), w_q0.data_ptr(),
                                          w_k0.data_ptr(), w_q1.data_ptr(), w_k1.data_ptr(), cos_sin0.data_ptr(),
                                          cos_sin1.data_ptr(), batch_size, num_tokens0, num_tokens1, num_heads_q,
                                          num_heads_k, head_size, is_interleaved, (float)eps, dtype,
                                          std::get<0>(outs).data_ptr(), std::get<1>(outs).data_ptr(), current_stream());
    check_status(status, op);
    return outs;
}

}  // namespace gpuk_ops
