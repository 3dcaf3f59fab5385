"""gpuk_amd -- MI355X (gfx950) implementation of gpuk's memory-bound fused inference ops.

Mirrors the reference's Python shim (gpuk/__init__.py): importing the package loads the torch
library `gpuk` and binds the operator names as module attributes, so

    import gpuk_amd as gpuk
    gpuk.fused_rope_rms(qkv, qw, kw, cos_sin, positions, T, Hq, Hk, Hv, D, True, 1e-6)
    env = gpuk.GPUKDistEnv(device_id=0); env.allreduce_add_rms_fused(x, residual, gamma, eps, fp8_out=True)

works as with the reference (gpuk/__init__.py:18-35, :54-205).  Only the operators of the two fused
paths exist here; there is no CPU or pure-torch fallback: if the built libraries are missing the
import raises.
"""
from __future__ import annotations

import os
from contextlib import contextmanager
from typing import Optional

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_PKG_DIR, "lib")
KERNEL_LIB = os.path.join(LIB_DIR, "libgpuk_amd.so")   # C ABI, include/gpuk_amd.h
TORCH_LIB = os.path.join(LIB_DIR, "libgpuk.so")        # TORCH_LIBRARY(gpuk, ...)

if not (os.path.exists(KERNEL_LIB) and os.path.exists(TORCH_LIB)):
    raise ImportError(
        f"gpuk_amd: {KERNEL_LIB} / {TORCH_LIB} not built; run `python -m gpuk_amd.build` "
        "(hipcc cross-compiles gfx950 without a GPU). There is no fallback path.")

torch.ops.load_library(TORCH_LIB)

allreduce_rms = torch.ops.gpuk.allreduce_rms
fused_rope_rms = torch.ops.gpuk.fused_rope_rms
fused_mrope_3d_rms = torch.ops.gpuk.fused_mrope_3d_rms
fused_mrope_3d_rms_set_kv = torch.ops.gpuk.fused_mrope_3d_rms_set_kv
fused_rope_rms_2way = torch.ops.gpuk.fused_rope_rms_2way
fused_rope_rms_set_kv = torch.ops.gpuk.fused_rope_rms_set_kv       # additive: 1-D positions + KV write
set_fp8_max = torch.ops.gpuk.set_fp8_max                           # additive
get_fp8_max = torch.ops.gpuk.get_fp8_max                           # additive


class _Traceable:
    """The in-place operators under schemas that declare their writes (`Tensor(a!)`), each with a Meta kernel:
    the overloads to call from code that goes through torch.compile / functionalisation.  Same arguments, same
    kernels as the names above, whose schemas are the reference's and carry no alias annotations."""
    allreduce_rms = torch.ops.gpuk.allreduce_rms.mut
    fused_rope_rms = torch.ops.gpuk.fused_rope_rms.mut
    fused_mrope_3d_rms = torch.ops.gpuk.fused_mrope_3d_rms.mut
    fused_mrope_3d_rms_set_kv = torch.ops.gpuk.fused_mrope_3d_rms_set_kv.mut
    fused_rope_rms_set_kv = torch.ops.gpuk.fused_rope_rms_set_kv.mut
    fused_rope_rms_2way = torch.ops.gpuk.fused_rope_rms_2way.default   # functional already


traceable = _Traceable

# gfx950 encodes OCP e4m3fn.  The reference defaults to the MI300-only e4m3fnuz (gpuk/__init__.py:38)
# and uses 240 as e4m3fn's maximum (:42-46); 448 is the OCP maximum.  `set_fp8_max(240)` restores the
# reference's divisor (codes up to 240 are identical in both encodings).
fp8 = torch.float8_e4m3fn
fp8_max_val_ = {torch.float8_e4m3fn: 448}
fp8_max_val = fp8_max_val_[fp8]
fp8_policy_id_ = {torch.float8_e4m3fn: 1}
fp8_policy_id = fp8_policy_id_[fp8]

QUANT_NONE = 0
QUANT_FP8_DYNAMIC = 1
QUANT_FP8_STATIC = 3   # additive: one per-tensor scale, read from scale_out[0]


class GPUKDistEnv:
    """Single-GPU counterpart of the reference's GPUKDistEnv (gpuk/__init__.py:54-205).

    The reference returns early with `fptr = None` at world size 1 and cannot run the fused op there
    (:72-73); here world size 1 is the supported case: `fptr` is 0 and `allreduce_add_rms_fused` runs
    residual-add + RMSNorm + quant with `allreduce_in` taken as the already-reduced activation.
    A larger world size raises: the IPC workspace and the all-reduce kernels are not part of this build.
    """

    _SUPPORTED_WORLD_SIZES = [1]

    def __init__(self, group=None, device_id: Optional[int] = None, max_size_in_bytes=16384 * 16384,
                 comm_ptrs_buf_len=1024 * 256, dtype: torch.dtype = torch.bfloat16) -> None:
        import torch.distributed as dist

        self.group = group
        self.device_id = device_id if device_id is not None else torch.cuda.current_device()
        if dist.is_available() and dist.is_initialized():
            self.rank = dist.get_rank(group=self.group)
            self.world_size = dist.get_world_size(group=self.group)
        else:
            self.rank, self.world_size = 0, 1
        if self.world_size not in GPUKDistEnv._SUPPORTED_WORLD_SIZES:
            raise NotImplementedError(
                f"GPUKDistEnv: world size {self.world_size} needs the cross-GPU all-reduce workspace, "
                "which this single-GPU build does not contain")
        self.fptr = 0
        self.disabled = False
        self._IS_CAPTURING = False
        self._IS_CAPTURED = False
        torch.cuda.set_device(self.device_id)

    def barrier(self):
        torch.cuda.set_device(self.device_id)
        torch.cuda.synchronize(self.device_id)

    def consume_capture(self):
        """No peer pointers to exchange at world size 1 (reference: gpuk/__init__.py:98-110)."""
        self.barrier()

    @contextmanager
    def capture(self):
        """Wraps a stream capture (gpuk/__init__.py:112-120).  The fused op allocates nothing and launches on the
        current stream, so at world size 1 a captured graph needs no pointer registration afterwards."""
        try:
            self._IS_CAPTURING = True
            yield
        finally:
            self._IS_CAPTURING = False
            # consume_capture() synchronises the device, which is not allowed while the stream is still capturing
            if not self.disabled and not torch.cuda.is_current_stream_capturing():
                self.consume_capture()

    def capture_(self, input: torch.Tensor):
        """Per-call bookkeeping of the reference (gpuk/__init__.py:122-129): remember that a capture happened, and
        after it ended do what consume_capture does."""
        if torch.compiler.is_compiling():
            return
        if torch.cuda.is_current_stream_capturing():
            self._IS_CAPTURED = True
        elif self._IS_CAPTURED:
            self.consume_capture()
            self._IS_CAPTURED = False

    def allreduce_native(self, allreduce_in):
        return allreduce_in.clone()

    def allreduce(self, allreduce_in):
        return allreduce_in.clone()

    def allreduce_add_rms_native(self, allreduce_in, residual_in, rms_weight, eps, fp8_out=False):
        """The unfused torch sequence the reference keeps beside the fused op (gpuk/__init__.py:147-173), minus the
        all-reduce: a handful of torch kernels on the tensors' device, for comparison and timing only."""
        residual_out = allreduce_in + residual_in
        variance = residual_out.float().pow(2).mean(-1, keepdim=True)
        norm_out = rms_weight * (residual_out * torch.rsqrt(variance + eps)).to(residual_out.dtype)
        if fp8_out:
            limit = float(get_fp8_max())
            scale = norm_out.float().abs().max(dim=-1, keepdim=True)[0] / limit
            norm_out = (norm_out / scale).clamp_(min=-limit, max=limit).to(fp8)
            return residual_out, norm_out, scale
        scale_out = torch.empty(allreduce_in.shape[0], 1, dtype=torch.float32, device=allreduce_in.device)
        return residual_out, norm_out, scale_out

    def allreduce_add_rms_fused(self, allreduce_in, residual_in, rms_weight, eps, fp8_out=False, static_scale=None):
        """gpuk/__init__.py:175-205.  Returns (residual_out, norm_out, scale_out).

        `static_scale` (additive): a 1-element fp32 tensor on the activations' device; selects per-tensor static
        quantisation.
        """
        self.capture_(allreduce_in)
        residual_out = torch.empty_like(residual_in)
        if fp8_out:
            norm_out = torch.empty_like(allreduce_in, dtype=fp8)
            if static_scale is not None:
                # read by the kernel as it is: a copy or cast made here would be a hidden transfer inside the call,
                # which a stream capture rejects
                if static_scale.device != allreduce_in.device or static_scale.dtype != torch.float32 or static_scale.numel() != 1:
                    raise ValueError("static_scale must be a 1-element fp32 tensor on the device of the activations")
                scale_out = static_scale.reshape(1)
                quant = QUANT_FP8_STATIC
            else:
                scale_out = torch.empty(allreduce_in.shape[0], 1, dtype=torch.float32, device=allreduce_in.device)
                quant = fp8_policy_id
        else:
            norm_out = torch.empty_like(allreduce_in)
            scale_out = torch.empty(1, dtype=torch.float32, device=allreduce_in.device)
            quant = QUANT_NONE
        # the overload whose schema declares the three writes: same kernel, and the call survives tracing
        traceable.allreduce_rms(self.fptr, allreduce_in, residual_in, rms_weight, residual_out, norm_out, scale_out,
                                eps, quant)
        return residual_out, norm_out, scale_out
