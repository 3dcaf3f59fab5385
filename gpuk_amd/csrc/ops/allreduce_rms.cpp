// allreduce_rms for one GPU: the residual-add + RMSNorm + FP8 epilogue without the all-reduce.
// Mirrors the host op at src/ops/all_reduce_fusion.cpp:363-396 (same argument order and checks);
// the IPC workspace behind a non-zero `fptr` belongs to the multi-GPU path and is not built here.
#include <atomic>

#include "ops.h"

namespace gpuk_ops {

namespace {
// amax divisor / clamp bound of the fp8 modes.  448 = OCP e4m3fn (gfx950 hardware); 240 reproduces
// the reference's fp8e4m3fn::max_value (src/common/float8.h:216-218, gpuk/__init__.py:42-46).
// One value for the whole process: it changes the numerics of every later allreduce_rms call from any thread (the
// store itself is atomic).  Set it once at start-up, not around individual calls.
std::atomic<double> g_fp8_max{448.0};
}  // namespace

void set_fp8_max(double value) {
    TORCH_CHECK(value > 0.0 && value <= 448.0, "set_fp8_max: value must be in (0, 448], got ", value);
    g_fp8_max.store(value);
}

double get_fp8_max() { return g_fp8_max.load(); }

void allreduce_rms(int64_t fptr, Tensor &allreduce_in, Tensor &residual_in, Tensor &rms_gamma, Tensor &residual_out,
                   Tensor &norm_out, Tensor &scale_out, double eps, int64_t quant_type) {
    TORCH_CHECK(fptr == 0,
                "allreduce_rms: this build is the single-GPU share of the op; pass fptr=0 (no all-reduce workspace)");
    TORCH_CHECK(allreduce_in.is_contiguous() && residual_in.is_contiguous() && rms_gamma.is_contiguous());
    TORCH_CHECK(residual_out.is_contiguous() && norm_out.is_contiguous() && scale_out.is_contiguous());
    TORCH_CHECK(allreduce_in.dim() >= 1, "allreduce_rms: allreduce_in needs a hidden dimension");
    const int64_t hidden = allreduce_in.size(-1);
    const int64_t size = allreduce_in.numel();
    const int64_t tokens = hidden > 0 ? size / hidden : 0;
    TORCH_CHECK(hidden > 0 && hidden % 8 == 0, "allreduce_rms: hidden must be a positive multiple of 8, got ", hidden);
    TORCH_CHECK(residual_in.numel() == size && residual_out.numel() == size && norm_out.numel() == size,
                "allreduce_rms: residual_in, residual_out and norm_out must have allreduce_in's element count");
    TORCH_CHECK(rms_gamma.numel() == hidden, "allreduce_rms: rms_gamma must have `hidden` elements");
    const auto act = allreduce_in.scalar_type();
    TORCH_CHECK(residual_in.scalar_type() == act && rms_gamma.scalar_type() == act && residual_out.scalar_type() == act,
                "allreduce_rms: residual_in, rms_gamma and residual_out must share allreduce_in's dtype");
    const int dtype = activation_dtype(allreduce_in, "allreduce_rms");
    TORCH_CHECK(quant_type != GPUK_QUANT_FP8_E4M3FNUZ,
                "allreduce_rms: quant_type 2 (e4m3fnuz) is the MI300 encoding; gfx950 encodes OCP e4m3fn (quant_type 1)");
    TORCH_CHECK(quant_type == GPUK_QUANT_NONE || quant_type == GPUK_QUANT_FP8_DYNAMIC || quant_type == GPUK_QUANT_FP8_STATIC,
                "allreduce_rms: unknown quant_type ", quant_type);
    float *scale_ptr = nullptr;
    if (quant_type == GPUK_QUANT_NONE) {
        TORCH_CHECK(norm_out.scalar_type() == act, "allreduce_rms: norm_out must have the activation dtype when quant_type is 0");
    } else {
        TORCH_CHECK(norm_out.element_size() == 1, "allreduce_rms: norm_out must be a 1-byte fp8 tensor when quant_type is ", quant_type);
        TORCH_CHECK(scale_out.scalar_type() == at::kFloat, "allreduce_rms: scale_out must be float32");
        TORCH_CHECK(scale_out.numel() >= (quant_type == GPUK_QUANT_FP8_DYNAMIC ? tokens : 1),
                    "allreduce_rms: scale_out is too small");
        scale_ptr = scale_out.data_ptr<float>();
    }
    TORCH_CHECK(allreduce_in.is_cuda(), "allreduce_rms: tensors must live on the GPU");
    const auto dev = allreduce_in.device();
    TORCH_CHECK(residual_in.device() == dev && rms_gamma.device() == dev && residual_out.device() == dev &&
                    norm_out.device() == dev && (quant_type == GPUK_QUANT_NONE || scale_out.device() == dev),
                "allreduce_rms: all tensors must be on the same device");
    DeviceGuard guard(dev);
    const int status = gpuk_add_rmsnorm_quant(allreduce_in.data_ptr(), residual_in.data_ptr(), rms_gamma.data_ptr(),
                                              residual_out.data_ptr(), norm_out.data_ptr(), scale_ptr, tokens, hidden,
                                              (float)eps, dtype, (int)quant_type, (float)g_fp8_max.load(),
                                              current_stream());
    check_status(status, "allreduce_rms");
}

}  // namespace gpuk_ops
