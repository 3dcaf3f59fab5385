// Host operators of the `gpuk` torch library: argument checks, device guard, current stream, then a
// call into the C ABI (include/gpuk_amd.h).  No kernels and no device code in this layer.
//
// Same role as the reference's src/ops/ops.h:23-65; only the operators of the two fused paths are
// declared, plus three additive ones (fused_rope_rms_set_kv, set_fp8_max, get_fp8_max).
#pragma once

#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <tuple>
#include <vector>

#include "../../../include/gpuk_amd.h"

namespace gpuk_ops {

using at::Tensor;

// HIP tensors carry the CUDA device type on PyTorch-ROCm, hence the "masquerading" guard and stream.
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;

// The stream torch would launch on for the device that is current under the caller's guard.
inline void *current_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

inline int activation_dtype(const Tensor &t, const char *op) {
    switch (t.scalar_type()) {
        case at::kBFloat16: return GPUK_DTYPE_BF16;
        case at::kHalf: return GPUK_DTYPE_FP16;
        case at::kFloat: return GPUK_DTYPE_F32;
        case at::kDouble: return GPUK_DTYPE_F64;
        default: TORCH_CHECK(false, op, ": activations must be bfloat16, float16, float32 or float64, got ", t.scalar_type());
    }
}

inline void check_status(int status, const char *op) {
    TORCH_CHECK(status == GPUK_OK, op, ": ", gpuk_status_string(status), " (status ", status, ")");
}

void allreduce_rms(int64_t fptr, Tensor &allreduce_in, Tensor &residual_in, Tensor &rms_gamma, Tensor &residual_out,
                   Tensor &norm_out, Tensor &scale_out, double eps, int64_t quant_type);
void set_fp8_max(double value);
double get_fp8_max();

void fused_rope_rms(Tensor &qkv, Tensor &qw, Tensor &kw, Tensor &cos_sin, Tensor &positions, int64_t num_tokens,
                    int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v, int64_t head_size,
                    bool is_neox_style, double eps);
void fused_mrope_3d_rms(Tensor &qkv, Tensor &qw, Tensor &kw, Tensor &cos_sin, Tensor &positions, int64_t num_tokens,
                        int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v, int64_t head_size,
                        bool is_neox_style, std::vector<int64_t> mrope_section_, bool is_interleaved, double eps);
void fused_mrope_3d_rms_set_kv(Tensor &qkv, Tensor &qw, Tensor &kw, Tensor &cos_sin, Tensor &positions,
                               int64_t num_tokens, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                               int64_t head_size, bool is_neox_style, std::vector<int64_t> mrope_section_,
                               bool is_interleaved, double eps, Tensor &q, Tensor &k_cache, Tensor &v_cache,
                               Tensor &kv_loc, double k_scale, double v_scale);
void fused_rope_rms_set_kv(Tensor &qkv, Tensor &qw, Tensor &kw, Tensor &cos_sin, Tensor &positions,
                           int64_t num_tokens, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                           int64_t head_size, bool is_neox_style, double eps, Tensor &q, Tensor &k_cache,
                           Tensor &v_cache, Tensor &kv_loc, double k_scale, double v_scale);

// Two token streams, outputs concatenated along the token axis (functional op with a Meta kernel, as in the
// reference: src/ops/ops.h:52-65).
std::tuple<Tensor, Tensor> fused_rope_rms_2way_meta(Tensor &q0, Tensor &k0, Tensor &q1, Tensor &k1, Tensor &w_q0,
                                                    Tensor &w_k0, Tensor &w_q1, Tensor &w_k1, Tensor &cos_sin0,
                                                    Tensor &cos_sin1, int64_t batch_size, int64_t num_tokens0,
                                                    int64_t num_tokens1, int64_t num_heads_q, int64_t num_heads_k,
                                                    int64_t head_size, bool is_interleaved, double eps);
std::tuple<Tensor, Tensor> fused_rope_rms_2way(Tensor &q0, Tensor &k0, Tensor &q1, Tensor &k1, Tensor &w_q0, Tensor &w_k0,
                                               Tensor &w_q1, Tensor &w_k1, Tensor &cos_sin0, Tensor &cos_sin1,
                                               int64_t batch_size, int64_t num_tokens0, int64_t num_tokens1,
                                               int64_t num_heads_q, int64_t num_heads_k, int64_t head_size,
                                               bool is_interleaved, double eps);

}  // namespace gpuk_ops
