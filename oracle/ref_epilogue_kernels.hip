// TEST INFRASTRUCTURE ONLY -- never linked into or loaded by the product.
//
// The reference's residual-add + RMSNorm + FP8 epilogue cannot run as the reference launches it on one GPU: its
// kernels start with a cross-GPU flag barrier and read the peers' buffers (src/impl/all_reduce_fusion_impl.h:230-270,
// dispatch for 2/4/8 ranks only).  What can run is the reference's own epilogue device code,
//   epilogue<T, VEC, STORE, BLOCK, QUANT>()  src/impl/all_reduce_fusion_impl.h:202-228
//   (rms_norm :159-181, reduce_abs_max :183-200, convert_to_fp8 :148-157, software fp8 types src/common/float8.h),
// compiled from the reference's headers where they lie, under a caller written here that does what the 1-stage
// kernel does around it without the communication part: one workgroup of hidden/8 lanes per token, fp32 add of the
// input and the residual, one rounding, store, then epilogue() (:251-267).  So this is the reference's arithmetic and
// its launch shape, not the reference's kernel; it is used to compare results and time on the same MI355X.
// bf16 only; hidden in {1024, 2048, 4096, 8192} (the reference's block_reduce needs hidden/256 to be a power of two;
// its own launchers stop at 4096).
#include "all_reduce_fusion_impl.h"

#include <cstdint>

namespace {

template <typename T, int BLOCK_SIZE, int QUANT_TYPE>
__global__ void __launch_bounds__(BLOCK_SIZE, 1) epilogue_rows(AllReduceFusionParams<T> params) {
    static constexpr int VEC_SIZE = details::kBytesPerAccess / sizeof(T);
    using vec_t_ = vec_t<T, VEC_SIZE>;
    const int tidx = blockIdx.x;
    const int access_id_in_token = threadIdx.x * VEC_SIZE;
    const int idx = tidx * params.hidden_dim + access_id_in_token;
    vec_t_ vec = *reinterpret_cast<vec_t_ *>(reinterpret_cast<T *>(params.allreduce_in) + idx);
    const vec_t_ res = *reinterpret_cast<vec_t_ *>(reinterpret_cast<T *>(params.residual_in) + idx);
#pragma unroll
    for (int v = 0; v < VEC_SIZE; ++v) vec.data[v] = (T)((float)vec.data[v] + (float)res.data[v]);
    *reinterpret_cast<vec_t_ *>(reinterpret_cast<T *>(params.residual_out) + idx) = vec;
    vec_t_ gamma = *reinterpret_cast<vec_t_ *>(reinterpret_cast<T *>(params.rms_gamma) + access_id_in_token);
    epilogue<T, VEC_SIZE, false, BLOCK_SIZE, QUANT_TYPE>(params, vec, gamma, idx, tidx);
}

template <typename T, int HIDDEN>
int launch(const AllReduceFusionParams<T> &p, int tokens, int quant, hipStream_t s) {
    constexpr int BLOCK = HIDDEN / (details::kBytesPerAccess / sizeof(T));
    if (quant == 0) epilogue_rows<T, BLOCK, QuantType::NONE><<<tokens, BLOCK, 0, s>>>(p);
    else epilogue_rows<T, BLOCK, QuantType::FP8E4M3FN><<<tokens, BLOCK, 0, s>>>(p);
    return (int)hipGetLastError();
}

}  // namespace

// quant 0: norm_out bf16; quant 1: norm_out = the reference's fp8e4m3fn codes (maximum 240, clipped), scale_out [tokens].
extern "C" int gpuk_ref_epilogue_rows(void *x, void *residual_in, void *gamma, void *residual_out, void *norm_out,
                                      float *scale_out, int64_t tokens, int64_t hidden, float eps, int quant, void *stream) {
    using T = __bfloat16;
    if (tokens <= 0 || tokens * hidden >= (1LL << 31) || (quant != 0 && quant != 1)) return -1;
    AllReduceFusionParams<T> p{};
    p.nranks = 1;
    p.rank = 0;
    p.size = (int)(tokens * hidden);
    p.hidden_dim = (int)hidden;
    p.allreduce_in = x;
    p.residual_in = residual_in;
    p.residual_out = residual_out;
    p.norm_out = norm_out;
    p.rms_gamma = gamma;
    p.rms_eps = eps;
    p.quant_type = quant ? QuantType::FP8E4M3FN : QuantType::NONE;
    p.scale_out = scale_out;
    p.allreduce_out = nullptr;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (hidden) {
        case 1024: return launch<T, 1024>(p, (int)tokens, quant, s);
        case 2048: return launch<T, 2048>(p, (int)tokens, quant, s);
        case 4096: return launch<T, 4096>(p, (int)tokens, quant, s);
        case 8192: return launch<T, 8192>(p, (int)tokens, quant, s);
        default: return -1;
    }
}
