/*
 * gpuk_amd.h -- C ABI of libgpuk_amd.so: gfx950 (MI355X) kernels for gpuk's memory-bound fused
 * inference ops.  Plain pointers and sizes, no torch types, no exceptions, no ownership transfer:
 * every buffer is borrowed for the duration of the enqueued kernel.  All entry points are
 * asynchronous on `stream` (a hipStream_t passed as void*; NULL = the default stream), allocate
 * nothing and never synchronise, so they can be recorded into a HIP graph.
 *
 * Each function returns GPUK_OK (0) or a gpuk_status; gpuk_status_string() names it.
 * Device pointers must be 16-byte aligned (8-byte for fp8 code buffers) as noted per argument.
 *
 * The reference interface each entry point stands behind is cited as <file>:<lines> in the
 * reference repository (xytpai/gpuk).
 */
#ifndef GPUK_AMD_H_
#define GPUK_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GPUK_AMD_ABI_VERSION 2

typedef enum gpuk_status {
    GPUK_OK = 0,
    GPUK_ERR_INVALID_ARG = 1,  /* null pointer, negative size, inconsistent sections ...        */
    GPUK_ERR_UNSUPPORTED = 2,  /* a shape / dtype / mode this build has no kernel for            */
    GPUK_ERR_MISALIGNED = 3,   /* a pointer misses the alignment the vector accesses need         */
    GPUK_ERR_LAUNCH = 4,       /* hipGetLastError() reported a launch failure                     */
    GPUK_ERR_INTERNAL = 5
} gpuk_status;

/* Activation formats (the reference dispatches on at::ScalarType:
 * src/ops/all_reduce_fusion.cpp:375, src/ops/fused_rope.cpp:27-31). */
typedef enum gpuk_dtype {
    GPUK_DTYPE_BF16 = 0,
    GPUK_DTYPE_FP16 = 1,
    GPUK_DTYPE_F32 = 2, /* compatibility paths (the reference dispatches float and double too: */
    GPUK_DTYPE_F64 = 3  /* AT_DISPATCH_FLOATING_TYPES_AND2); not tuned like the 16-bit types */
} gpuk_dtype;

/* quant_type of the allreduce_rms op.  0/1/2 are the reference's QuantType
 * (src/impl/all_reduce_fusion_impl.h:13-17); 3 is additive. */
typedef enum gpuk_quant {
    GPUK_QUANT_NONE = 0,         /* norm_out holds the activation dtype                                   */
    GPUK_QUANT_FP8_DYNAMIC = 1,  /* e4m3fn codes, per-token scale written to scale[tokens]                */
    GPUK_QUANT_FP8_E4M3FNUZ = 2, /* MI300 fnuz encoding: rejected with GPUK_ERR_UNSUPPORTED on gfx950     */
    GPUK_QUANT_FP8_STATIC = 3    /* e4m3fn codes, one per-tensor scale read from scale[0]                 */
} gpuk_quant;

/* Storage format of the paged KV cache. */
typedef enum gpuk_kv_dtype {
    GPUK_KV_SAME = 0,   /* cache holds the activation dtype; K/V are stored unscaled
                           (src/impl/rope_rms_impl.h:213-214,225-226)                                    */
    GPUK_KV_E4M3FN = 1  /* cache holds e4m3fn codes of x / scale (src/impl/rope_rms_impl.h:109-118,215-217) */
} gpuk_kv_dtype;

const char *gpuk_status_string(int status);
int gpuk_abi_version(void);

/*
 * residual_out = x + residual_in ; norm_out = quant(RMSNorm(residual_out) * gamma).
 *
 * Stands behind the allreduce_rms op for the one-GPU case (no all-reduce):
 * host op src/ops/all_reduce_fusion.cpp:363-396, launcher src/impl/all_reduce_fusion_impl.h:424-469,
 * device code :256-265 (residual add) + :202-228 (epilogue).  Rounding follows the reference's torch
 * oracle gpuk/__init__.py:147-164.
 *
 *   x, residual_in, residual_out : [tokens, hidden] contiguous, `dtype`, 16-byte aligned
 *   gamma                        : [hidden] `dtype`, 16-byte aligned
 *   norm_out                     : [tokens, hidden]; `dtype` (16-byte aligned) for GPUK_QUANT_NONE,
 *                                  else one byte per element (8-byte aligned)
 *   scale                        : fp32; written [tokens] for FP8_DYNAMIC, read [1] for FP8_STATIC,
 *                                  ignored (may be NULL) for NONE
 *   hidden                       : multiple of 8 (the reference supports 1024/2048/4096 only:
 *                                  all_reduce_fusion_impl.h:389-401)
 *   fp8_max                      : clamp bound and amax divisor; 448 (OCP e4m3fn) or 240 (the
 *                                  reference's fp8e4m3fn::max_value, src/common/float8.h:216-218)
 *
 * residual_out may be the same buffer as residual_in or as x (the usual in-place residual stream): every row is read
 * whole before any of it is written.  Partial overlap, and norm_out overlapping an input, are not allowed.
 */
int gpuk_add_rmsnorm_quant(const void *x, const void *residual_in, const void *gamma, void *residual_out,
                           void *norm_out, float *scale, int64_t tokens, int64_t hidden, float eps, int dtype,
                           int quant_mode, float fp8_max, void *stream);

/*
 * Per-head RMSNorm of Q and K, then rotary embedding, written back in place; V is not touched.
 *
 * Stands behind fused_rope_rms (src/ops/fused_rope.cpp:19-49 -> src/impl/rope_rms_impl.h:468-503)
 * with n_axes == 1 and behind fused_mrope_3d_rms (fused_rope.cpp:51-89 -> rope_rms_impl.h:505-555)
 * with n_axes == 3.  Rounding follows test/test_fused_rope_rms.py:8-34.
 *
 *   qkv        : [num_tokens, hq+hk+hv, head_size] contiguous `dtype`, 16-byte aligned, in/out
 *   qw, kw     : [head_size] `dtype`
 *   cos_sin    : [max_positions, head_size] `dtype`; row p = cos(p*f_0..f_{D/2-1}) | sin(...)
 *   positions  : int64; element (axis a, token t) at positions[a*pos_stride_axis + t*pos_stride_token]
 *   n_axes     : 1 (RoPE) or 3 (mRoPE; mrope_section is a HOST pointer to 3 values that sum to
 *                head_size/2; it is read during the call and may be NULL when n_axes == 1)
 *   interleaved: mRoPE frequency->axis map; 0 chunked, 1 interleaved (rope_rms_impl.h:120-153)
 *   head_size  : 64, 128 or 256 (rope_rms_impl.h:473)
 */
int gpuk_rope_rms(void *qkv, const void *qw, const void *kw, const void *cos_sin, const int64_t *positions,
                  int64_t pos_stride_axis, int64_t pos_stride_token, int n_axes, int64_t num_tokens,
                  int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v, int64_t head_size,
                  int is_neox_style, const int64_t *mrope_section, int is_interleaved, float eps, int dtype,
                  void *stream);

/*
 * Same arithmetic, results scattered: q -> q_out[t,h,:], k -> k_cache[kv_loc[t],h,:],
 * v -> v_cache[kv_loc[t],h,:]; qkv is read only.
 *
 * Stands behind fused_mrope_3d_rms_set_kv (src/ops/fused_rope.cpp:91-166 ->
 * src/impl/rope_rms_impl.h:557-610, kernels :157-301) with n_axes == 3; n_axes == 1 is the additive
 * fused_rope_rms_set_kv.  Rounding follows test/test_fused_mrope_rms_set_kv.py:62-130.
 *
 *   q_out            : [num_tokens, hq, head_size] `dtype`, 16-byte aligned
 *   k_cache, v_cache : [slots, hk|hv, head_size]; `dtype` or e4m3fn bytes per kv_dtype; slots not named
 *                      by kv_loc are left bit-identical
 *   kv_loc           : [num_tokens] int64 slot per token.  Tokens that name the same slot race: every aligned group of
 *                      8 elements of the slot's K and V rows comes whole from one of them, the rows may mix.  A negative slot
 *                      marks a token with no place in the cache (padding): its q_out row is written, its K and V
 *                      rows are dropped (an addition: the reference would write out of bounds)
 *   k_scale, v_scale : used only with GPUK_KV_E4M3FN: code = e4m3fn(rT(x / scale)), saturating at +-448
 */
int gpuk_rope_rms_set_kv(const void *qkv, const void *qw, const void *kw, const void *cos_sin,
                         const int64_t *positions, int64_t pos_stride_axis, int64_t pos_stride_token, int n_axes,
                         int64_t num_tokens, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                         int64_t head_size, int is_neox_style, const int64_t *mrope_section, int is_interleaved,
                         float eps, int dtype, void *q_out, void *k_cache, void *v_cache, const int64_t *kv_loc,
                         float k_scale, float v_scale, int kv_dtype, void *stream);

/*
 * Two token streams (e.g. text and image) with their own norm weights and per-token cos/sin rows: per-head RMSNorm
 * and rotation of q0/k0 with cos_sin0 and of q1/k1 with cos_sin1, outputs concatenated along the token axis.
 *
 * Stands behind fused_rope_rms_2way (src/ops/fused_rope.cpp:168-227 -> src/impl/rope_rms_impl.h:612-857).
 * Rounding follows test/test_fused_rope_rms_2way.py:37-81.
 *
 *   q0, q1          : [batch, num_tokens{0,1}, num_heads_q, head_size] contiguous `dtype`, 16-byte aligned
 *   k0, k1          : [batch, num_tokens{0,1}, num_heads_k, head_size]
 *   w_q0 .. w_k1    : [head_size]
 *   cos_sin0, 1     : [num_tokens{0,1}, head_size]; row t = cos | sin for token t of that stream
 *   out_q01, out_k01: [batch, num_tokens0 + num_tokens1, num_heads_{q,k}, head_size]; stream 0 first
 *   is_interleaved  : 1 rotates adjacent pairs (GPT-J style), 0 pairs element i with i + head_size/2 (NeoX style)
 */
int gpuk_rope_rms_2way(const void *q0, const void *k0, const void *q1, const void *k1, const void *w_q0,
                       const void *w_k0, const void *w_q1, const void *w_k1, const void *cos_sin0,
                       const void *cos_sin1, int64_t batch_size, int64_t num_tokens0, int64_t num_tokens1,
                       int64_t num_heads_q, int64_t num_heads_k, int64_t head_size, int is_interleaved, float eps,
                       int dtype, void *out_q01, void *out_k01, void *stream);

/*
 * Roofline calibration: dst[0..nbytes) = src[0..nbytes) with a plain streaming copy kernel (nbytes a
 * multiple of 16, both pointers 16-byte aligned).  Moves exactly 2*nbytes of HBM traffic; used to measure
 * the practical bandwidth ceiling and to scale the profiler's FETCH_SIZE / WRITE_SIZE readings.
 * Counterpart of the reference's micro-benchmark test/cpp/global_memory_bandwidth.cpp:95-114.
 */
int gpuk_copy_bytes(void *dst, const void *src, int64_t nbytes, void *stream);

/*
 * Roofline calibration, one direction at a time: gpuk_read_bytes reads src[0..nbytes) with the copy kernel's tiles
 * and streaming loads and writes nothing (`sink`, 4 bytes of device memory, receives a word only if a fold of the
 * data hits one fixed value); gpuk_fill_bytes writes dst[0..nbytes) with the copy kernel's streaming stores and
 * reads nothing.  A kernel that reads R and writes W bytes is priced against R / read-only rate + W / write-only
 * rate.  nbytes a multiple of 16, pointers 16-byte aligned.  The reference's micro-benchmark measures the copy
 * only (test/cpp/global_memory_bandwidth.cpp:95-114); these are its two halves.
 */
int gpuk_read_bytes(const void *src, int64_t nbytes, void *sink, void *stream);
int gpuk_fill_bytes(void *dst, int64_t nbytes, uint32_t seed, void *stream);

/*
 * Launch-cost calibration for a grid shape: `workgroups` workgroups of `lanes_per_workgroup` lanes (a multiple of 64,
 * at most 1024) with `lds_bytes` of dynamic LDS each (at most 65536) that return at once.  Its duration is what
 * launching, placing and draining that grid costs before any byte moves.  Same purpose as the reference's
 * test/cpp/test_small_kernel.cpp:98-178, for a full-size grid.
 */
int gpuk_empty_grid(int64_t workgroups, int lanes_per_workgroup, int lds_bytes, void *stream);

/*
 * Roofline calibration: the memory traffic of gpuk_add_rmsnorm_quant (16-bit activations, fp8 output, per-token
 * scale) without its arithmetic: same launch shape, lane-to-data mapping, streaming loads and stores and barriers;
 * residual_out receives x ^ residual_in, codes a fold of it, scale 1.0 per token.  Its duration is the ceiling of the
 * access pattern, to be read beside the real kernel's.  x, residual_in, residual_out: [tokens, hidden] 16-bit;
 * codes: [tokens, hidden] bytes; scale: [tokens] fp32; hidden a multiple of 8 and at most 65536.
 * Not part of the reference (its micro-benchmarks are test/cpp/global_memory_bandwidth.cpp).
 */
int gpuk_add_rmsnorm_quant_traffic_only(const void *x, const void *residual_in, void *residual_out, void *codes,
                                        float *scale, int64_t tokens, int64_t hidden, void *stream);

/*
 * The launch shape gpuk_add_rmsnorm_quant picks for a batch: lanes per token row (= workgroup size; one workgroup
 * per row) and chunks per lane (8 elements of a 16-bit type, 4 of fp32 / fp64; 0: rows too long for registers, swept
 * three times); of a batch that runs as two launches, the first one's.  For reports.
 */
int gpuk_add_rmsnorm_quant_launch_shape(int64_t tokens, int64_t hidden, int dtype, int *lanes_per_row,
                                        int *chunks_per_lane);

/*
 * The launch gpuk_rope_rms_set_kv (set_kv != 0) or gpuk_rope_rms (set_kv == 0) makes for a batch: the grid as
 * workgroups x lanes per workgroup; *streamed = 1 when the rotated rows are stored past the L2; *token_waves = 1 for
 * the kernel in which a wave of 64 lanes takes a whole token (batches the chip holds in one round), 2 where it takes
 * two tokens, the second through LDS, 0 for the kernel in which a wave takes a group of heads of a token.  Computed
 * on the host from the sizes and the tuning keys (with three position axes: for sections that split at multiples of
 * 8 frequencies, which the call itself checks); the four outputs are host pointers.  For reports.  Not part of the
 * reference.
 */
int gpuk_rope_rms_launch_shape(int64_t num_tokens, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                               int64_t head_size, int n_axes, int dtype, int set_kv, int kv_dtype, int *workgroups,
                               int *lanes_per_workgroup, int *streamed, int *token_waves);

/*
 * Launch-cost calibration: data[i] += 1 for i in [0, n) (data 16-byte aligned).  With a small n the call costs
 * what launching and draining any kernel costs, the floor under decode-sized calls.
 * Counterpart of the reference's micro-benchmark test/cpp/test_small_kernel.cpp:85-126.
 */
int gpuk_increment_floats(float *data, int64_t n, void *stream);

/* Launch-shape knobs for sweeps and for the tests that show the results do not depend on them; value 0 restores
 * the built-in choice.  Keys: "norm_quant_nchunk" (1/2/4/8 16-byte chunks per lane), "norm_quant_threads" (lanes
 * per row), "norm_quant_row_group_shift" (log2 of the run of consecutive rows one XCD takes; -1, not 0, restores the
 * built-in rule), "norm_quant_gate" (how long, in ticks of 10 ns after a wave's entry, the stores of the norm-quant
 * kernel are held back so that the reads of a batch the chip holds at once go first: -1 the built-in rule, 0 never),
 * "norm_quant_launches" (1: a call is always one launch; 2: two, of half the rows each, wherever the batch is more
 * than one round of workgroups and at most two),
 * "rope_block_threads" (64/128/256/512 lanes per workgroup of the rope kernel), "rope_stream_rows" (output rows of
 * the rope kernels stored past the L2: 1 never, 2 always), "rope_merge_rows" (1: never let the lanes of an mRoPE
 * token load their cos/sin pieces straight from the row of their axis), "rope_token_waves" (the kernel in which one
 * wave takes a whole token: 1 never, 2 wherever the shape fits it, 3 likewise with two tokens per wave where that fits), "rope_token_gate" and "rope_unit_gate" (the
 * store gate of the two rope kernels, in ticks as above: -1 the built-in rule, 0 never).  The results do not depend
 * on any of them.  Unknown keys or values return GPUK_ERR_INVALID_ARG.  The settings are process-global plain
 * variables read at launch: set them from one thread while no other thread is launching.  Not part of the
 * reference. */
int gpuk_set_tuning(const char *key, int value);

#ifdef __cplusplus
}
#endif

#endif /* GPUK_AMD_H_ */
