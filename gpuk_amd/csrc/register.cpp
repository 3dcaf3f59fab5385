// Operator registration of the `gpuk` torch library for the two fused paths.
//
// The five schema strings marked "reference" are the reference's own (src/register.cpp:37-39, :42-44,
// :47-49, :52-55, :58-61), so `torch.ops.gpuk.<name>(...)` call sites keep working unchanged.  Compute ops are
// registered for the CUDA dispatch key, which is the key HIP tensors carry on PyTorch-ROCm.
//
// Each in-place operator also has an overload `.mut` with the same arguments whose schema declares which tensors
// it writes (`Tensor(a!)`), and a Meta kernel that does nothing: the reference's schemas carry no alias
// annotations, which eager mode tolerates but functionalisation (torch.compile, AOT autograd) needs in order to
// keep the writes.  `torch.ops.gpuk.<name>(...)` resolves to the reference's schema; `torch.ops.gpuk.<name>.mut`
// is the one to trace.
#include "ops/ops.h"

namespace {
// A function with the signature of F that does nothing: the Meta kernel of an operator that only writes into
// tensors the caller allocated.
template <auto F> struct NoOpLike;
template <typename... A, void (*F)(A...)> struct NoOpLike<F> {
    static void call(A...) {}
};
}  // namespace

TORCH_LIBRARY(gpuk, m) {
    using namespace gpuk_ops;

    // reference: src/register.cpp:37-40
    m.def("allreduce_rms(SymInt fptr, Tensor allreduce_in, Tensor residual_in, Tensor rms_gamma, Tensor residual_out, "
          "Tensor norm_out, Tensor scale_out, float eps, SymInt quant_type) -> ()");
    m.impl("allreduce_rms", c10::DispatchKey::CUDA, &allreduce_rms);
    m.def("allreduce_rms.mut(SymInt fptr, Tensor allreduce_in, Tensor residual_in, Tensor rms_gamma, "
          "Tensor(a!) residual_out, Tensor(b!) norm_out, Tensor(c!) scale_out, float eps, SymInt quant_type) -> ()");
    m.impl("allreduce_rms.mut", c10::DispatchKey::CUDA, &allreduce_rms);
    m.impl("allreduce_rms.mut", c10::DispatchKey::Meta, &NoOpLike<&allreduce_rms>::call);

    // reference: src/register.cpp:42-45
    m.def("fused_rope_rms(Tensor qkv, Tensor qw, Tensor kw, Tensor cos_sin, Tensor positions, SymInt num_tokens, "
          "SymInt num_heads_q, SymInt num_heads_k, SymInt num_heads_v, SymInt head_size, bool is_neox_style, "
          "float eps) -> ()");
    m.impl("fused_rope_rms", c10::DispatchKey::CUDA, &fused_rope_rms);
    m.def("fused_rope_rms.mut(Tensor(a!) qkv, Tensor qw, Tensor kw, Tensor cos_sin, Tensor positions, "
          "SymInt num_tokens, SymInt num_heads_q, SymInt num_heads_k, SymInt num_heads_v, SymInt head_size, "
          "bool is_neox_style, float eps) -> ()");
    m.impl("fused_rope_rms.mut", c10::DispatchKey::CUDA, &fused_rope_rms);
    m.impl("fused_rope_rms.mut", c10::DispatchKey::Meta, &NoOpLike<&fused_rope_rms>::call);

    // reference: src/register.cpp:47-50
    m.def("fused_mrope_3d_rms(Tensor qkv, Tensor qw, Tensor kw, Tensor cos_sin, Tensor positions, SymInt num_tokens, "
          "SymInt num_heads_q, SymInt num_heads_k, SymInt num_heads_v, SymInt head_size, bool is_neox_style, "
          "int[] mrope_section_, bool is_interleaved, float eps) -> ()");
    m.impl("fused_mrope_3d_rms", c10::DispatchKey::CUDA, &fused_mrope_3d_rms);
    m.def("fused_mrope_3d_rms.mut(Tensor(a!) qkv, Tensor qw, Tensor kw, Tensor cos_sin, Tensor positions, "
          "SymInt num_tokens, SymInt num_heads_q, SymInt num_heads_k, SymInt num_heads_v, SymInt head_size, "
          "bool is_neox_style, int[] mrope_section_, bool is_interleaved, float eps) -> ()");
    m.impl("fused_mrope_3d_rms.mut", c10::DispatchKey::CUDA, &fused_mrope_3d_rms);
    m.impl("fused_mrope_3d_rms.mut", c10::DispatchKey::Meta, &NoOpLike<&fused_mrope_3d_rms>::call);

    // reference: src/register.cpp:52-56
    m.def("fused_mrope_3d_rms_set_kv(Tensor qkv, Tensor qw, Tensor kw, Tensor cos_sin, Tensor positions, "
          "SymInt num_tokens, SymInt num_heads_q, SymInt num_heads_k, SymInt num_heads_v, SymInt head_size, "
          "bool is_neox_style, int[] mrope_section_, bool is_interleaved, float eps, Tensor q, Tensor k_cache, "
          "Tensor v_cache, Tensor kv_loc, float k_scale, float v_scale) -> ()");
    m.impl("fused_mrope_3d_rms_set_kv", c10::DispatchKey::CUDA, &fused_mrope_3d_rms_set_kv);
    m.def("fused_mrope_3d_rms_set_kv.mut(Tensor qkv, Tensor qw, Tensor kw, Tensor cos_sin, Tensor positions, "
          "SymInt num_tokens, SymInt num_heads_q, SymInt num_heads_k, SymInt num_heads_v, SymInt head_size, "
          "bool is_neox_style, int[] mrope_section_, bool is_interleaved, float eps, Tensor(a!) q, "
          "Tensor(b!) k_cache, Tensor(c!) v_cache, Tensor kv_loc, float k_scale, float v_scale) -> ()");
    m.impl("fused_mrope_3d_rms_set_kv.mut", c10::DispatchKey::CUDA, &fused_mrope_3d_rms_set_kv);
    m.impl("fused_mrope_3d_rms_set_kv.mut", c10::DispatchKey::Meta, &NoOpLike<&fused_mrope_3d_rms_set_kv>::call);

    // additive: plain-RoPE form of the KV-writing op (1-D positions)
    m.def("fused_rope_rms_set_kv(Tensor qkv, Tensor qw, Tensor kw, Tensor cos_sin, Tensor positions, "
          "SymInt num_tokens, SymInt num_heads_q, SymInt num_heads_k, SymInt num_heads_v, SymInt head_size, "
          "bool is_neox_style, float eps, Tensor q, Tensor k_cache, Tensor v_cache, Tensor kv_loc, float k_scale, "
          "float v_scale) -> ()");
    m.impl("fused_rope_rms_set_kv", c10::DispatchKey::CUDA, &fused_rope_rms_set_kv);
    m.def("fused_rope_rms_set_kv.mut(Tensor qkv, Tensor qw, Tensor kw, Tensor cos_sin, Tensor positions, "
          "SymInt num_tokens, SymInt num_heads_q, SymInt num_heads_k, SymInt num_heads_v, SymInt head_size, "
          "bool is_neox_style, float eps, Tensor(a!) q, Tensor(b!) k_cache, Tensor(c!) v_cache, Tensor kv_loc, "
          "float k_scale, float v_scale) -> ()");
    m.impl("fused_rope_rms_set_kv.mut", c10::DispatchKey::CUDA, &fused_rope_rms_set_kv);
    m.impl("fused_rope_rms_set_kv.mut", c10::DispatchKey::Meta, &NoOpLike<&fused_rope_rms_set_kv>::call);

    // reference: src/register.cpp:58-63 (functional op with a Meta kernel for shape inference)
    m.def("fused_rope_rms_2way(Tensor q0, Tensor k0, Tensor q1, Tensor k1, Tensor w_q0, Tensor w_k0, Tensor w_q1, "
          "Tensor w_k1, Tensor cos_sin0, Tensor cos_sin1, SymInt batch_size, SymInt num_tokens0, SymInt num_tokens1, "
          "SymInt num_heads_q, SymInt num_heads_k, SymInt head_size, bool is_interleaved, float eps) -> "
          "(Tensor out_q01, Tensor out_k01)");
    m.impl("fused_rope_rms_2way", c10::DispatchKey::CUDA, &fused_rope_rms_2way);
    m.impl("fused_rope_rms_2way", c10::DispatchKey::Meta, &fused_rope_rms_2way_meta);

    // additive: amax divisor / clamp bound of the fp8 modes of allreduce_rms (448 OCP default, 240 reference)
    m.def("set_fp8_max(float value) -> ()");
    m.impl("set_fp8_max", &set_fp8_max);
    m.def("get_fp8_max() -> float");
    m.impl("get_fp8_max", &get_fp8_max);
}
