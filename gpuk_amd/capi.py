"""ctypes binding of the C ABI (include/gpuk_amd.h) for callers that hold raw device pointers.

Takes torch tensors only to read `data_ptr()`; the launches go on torch's current stream unless a
stream handle is given.  Raises GpukError on a non-zero status.  No fallback of any kind.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Sequence

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libgpuk_amd.so")

EXPORTS = ("gpuk_status_string", "gpuk_abi_version", "gpuk_add_rmsnorm_quant", "gpuk_rope_rms",
           "gpuk_rope_rms_set_kv", "gpuk_rope_rms_2way", "gpuk_copy_bytes", "gpuk_increment_floats", "gpuk_set_tuning",
           "gpuk_add_rmsnorm_quant_traffic_only", "gpuk_add_rmsnorm_quant_launch_shape",
           "gpuk_rope_rms_launch_shape", "gpuk_read_bytes", "gpuk_fill_bytes", "gpuk_empty_grid")

DTYPE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2, torch.float64: 3}
QUANT_NONE, QUANT_FP8_DYNAMIC, QUANT_FP8_E4M3FNUZ, QUANT_FP8_STATIC = 0, 1, 2, 3
KV_SAME, KV_E4M3FN = 0, 1


class GpukError(RuntimeError):
    def __init__(self, status: int, what: str):
        self.status = status
        super().__init__(f"{what}: {lib().gpuk_status_string(status).decode()} (status {status})")


_lib = None


def use_library(path: str) -> None:
    """Bind this module to another build of the C ABI (the profiling build libgpuk_amd_stamps.so) from here on."""
    global _lib, _LIB_PATH
    _LIB_PATH, _lib = path, None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(f"{_LIB_PATH} not built; run `python -m gpuk_amd.build`")
        L = C.CDLL(_LIB_PATH)
        L.gpuk_status_string.restype = C.c_char_p
        L.gpuk_status_string.argtypes = [C.c_int]
        L.gpuk_abi_version.restype = C.c_int
        L.gpuk_set_tuning.restype = C.c_int
        L.gpuk_set_tuning.argtypes = [C.c_char_p, C.c_int]
        L.gpuk_add_rmsnorm_quant.restype = C.c_int
        L.gpuk_add_rmsnorm_quant.argtypes = [C.c_void_p] * 6 + [C.c_int64, C.c_int64, C.c_float, C.c_int, C.c_int,
                                                               C.c_float, C.c_void_p]
        rope_head = [C.c_void_p] * 5 + [C.c_int64, C.c_int64, C.c_int] + [C.c_int64] * 5 + [
            C.c_int, C.POINTER(C.c_int64), C.c_int, C.c_float, C.c_int]
        L.gpuk_rope_rms.restype = C.c_int
        L.gpuk_rope_rms.argtypes = rope_head + [C.c_void_p]
        L.gpuk_rope_rms_set_kv.restype = C.c_int
        L.gpuk_rope_rms_set_kv.argtypes = rope_head + [C.c_void_p] * 4 + [C.c_float, C.c_float, C.c_int, C.c_void_p]
        L.gpuk_rope_rms_2way.restype = C.c_int
        L.gpuk_rope_rms_2way.argtypes = [C.c_void_p] * 10 + [C.c_int64] * 6 + [C.c_int, C.c_float, C.c_int,
                                                                             C.c_void_p, C.c_void_p, C.c_void_p]
        L.gpuk_increment_floats.restype = C.c_int
        L.gpuk_increment_floats.argtypes = [C.c_void_p, C.c_int64, C.c_void_p]
        L.gpuk_add_rmsnorm_quant_traffic_only.restype = C.c_int
        L.gpuk_add_rmsnorm_quant_traffic_only.argtypes = [C.c_void_p] * 5 + [C.c_int64, C.c_int64, C.c_void_p]
        L.gpuk_add_rmsnorm_quant_launch_shape.restype = C.c_int
        L.gpuk_add_rmsnorm_quant_launch_shape.argtypes = [C.c_int64, C.c_int64, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        L.gpuk_rope_rms_launch_shape.restype = C.c_int
        L.gpuk_rope_rms_launch_shape.argtypes = [C.c_int64] * 5 + [C.c_int] * 4 + [C.POINTER(C.c_int)] * 4
        L.gpuk_copy_bytes.restype = C.c_int
        L.gpuk_copy_bytes.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
        L.gpuk_read_bytes.restype = C.c_int
        L.gpuk_read_bytes.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]
        L.gpuk_fill_bytes.restype = C.c_int
        L.gpuk_fill_bytes.argtypes = [C.c_void_p, C.c_int64, C.c_uint32, C.c_void_p]
        L.gpuk_empty_grid.restype = C.c_int
        L.gpuk_empty_grid.argtypes = [C.c_int64, C.c_int, C.c_int, C.c_void_p]
        _lib = L
    return _lib


def _stream(stream) -> int:
    if stream is None:
        return torch.cuda.current_stream().cuda_stream
    return getattr(stream, "cuda_stream", stream)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def set_tuning(key: str, value: int) -> None:
    rc = lib().gpuk_set_tuning(key.encode(), value)
    if rc:
        raise GpukError(rc, f"gpuk_set_tuning({key})")


def add_rmsnorm_quant(x, residual_in, gamma, residual_out, norm_out, scale, eps: float, quant: int,
                      fp8_max: float = 448.0, stream=None) -> None:
    tokens = x.numel() // x.shape[-1] if x.shape[-1] else 0
    rc = lib().gpuk_add_rmsnorm_quant(_ptr(x), _ptr(residual_in), _ptr(gamma), _ptr(residual_out), _ptr(norm_out),
                                      _ptr(scale), tokens, x.shape[-1], eps, DTYPE[x.dtype], quant, fp8_max,
                                      _stream(stream))
    if rc:
        raise GpukError(rc, "gpuk_add_rmsnorm_quant")


def add_rmsnorm_quant_traffic_only(x, residual_in, residual_out, codes, scale, stream=None) -> None:
    tokens = x.numel() // x.shape[-1]
    rc = lib().gpuk_add_rmsnorm_quant_traffic_only(_ptr(x), _ptr(residual_in), _ptr(residual_out), _ptr(codes), _ptr(scale),
                                                   tokens, x.shape[-1], _stream(stream))
    if rc:
        raise GpukError(rc, "gpuk_add_rmsnorm_quant_traffic_only")


def add_rmsnorm_quant_launch_shape(tokens: int, hidden: int, dtype=torch.bfloat16):
    """(lanes per row, 16-byte chunks per lane) of the launch gpuk_add_rmsnorm_quant makes for this batch."""
    lanes, chunks = C.c_int(0), C.c_int(0)
    rc = lib().gpuk_add_rmsnorm_quant_launch_shape(tokens, hidden, DTYPE[dtype], C.byref(lanes), C.byref(chunks))
    if rc:
        raise GpukError(rc, "gpuk_add_rmsnorm_quant_launch_shape")
    return lanes.value, chunks.value


def rope_rms_launch_shape(num_tokens: int, num_heads_q: int, num_heads_k: int, num_heads_v: int, head_size: int,
                          n_axes: int = 1, dtype=torch.bfloat16, set_kv: bool = True, kv_fp8: bool = False):
    """(workgroups, lanes per workgroup, streamed, tokens per wave) of the launch the rope entry points make; tokens
    per wave is 0 for the kernel in which a wave takes a group of heads, 1 or 2 for the one in which it takes tokens."""
    out = [C.c_int(0) for _ in range(4)]
    rc = lib().gpuk_rope_rms_launch_shape(num_tokens, num_heads_q, num_heads_k, num_heads_v, head_size, n_axes,
                                          DTYPE[dtype], int(set_kv), 1 if kv_fp8 else 0, *(C.byref(o) for o in out))
    if rc:
        raise GpukError(rc, "gpuk_rope_rms_launch_shape")
    return out[0].value, out[1].value, bool(out[2].value), out[3].value


def _pos_args(positions):
    if positions.dim() == 1:
        return 0, positions.stride(0), 1
    return positions.stride(0), positions.stride(1), 3


def _section(mrope_section: Optional[Sequence[int]]):
    if mrope_section is None:
        return None
    return (C.c_int64 * 3)(*[int(v) for v in mrope_section])


def rope_rms(qkv, qw, kw, cos_sin, positions, T, Hq, Hk, Hv, D, is_neox, eps, mrope_section=None,
             is_interleaved=False, stream=None) -> None:
    psa, pst, n_axes = _pos_args(positions)
    rc = lib().gpuk_rope_rms(_ptr(qkv), _ptr(qw), _ptr(kw), _ptr(cos_sin), _ptr(positions), psa, pst, n_axes,
                             T, Hq, Hk, Hv, D, int(is_neox), _section(mrope_section), int(is_interleaved), eps,
                             DTYPE[qkv.dtype], _stream(stream))
    if rc:
        raise GpukError(rc, "gpuk_rope_rms")


def rope_rms_set_kv(qkv, qw, kw, cos_sin, positions, T, Hq, Hk, Hv, D, is_neox, eps, q_out, k_cache, v_cache, kv_loc,
                    k_scale=1.0, v_scale=1.0, mrope_section=None, is_interleaved=False, stream=None) -> None:
    psa, pst, n_axes = _pos_args(positions)
    kv = KV_SAME if k_cache.dtype == qkv.dtype else KV_E4M3FN
    rc = lib().gpuk_rope_rms_set_kv(_ptr(qkv), _ptr(qw), _ptr(kw), _ptr(cos_sin), _ptr(positions), psa, pst, n_axes,
                                    T, Hq, Hk, Hv, D, int(is_neox), _section(mrope_section), int(is_interleaved), eps,
                                    DTYPE[qkv.dtype], _ptr(q_out), _ptr(k_cache), _ptr(v_cache), _ptr(kv_loc),
                                    k_scale, v_scale, kv, _stream(stream))
    if rc:
        raise GpukError(rc, "gpuk_rope_rms_set_kv")


def increment_floats(data, n: int, stream=None) -> None:
    rc = lib().gpuk_increment_floats(_ptr(data), n, _stream(stream))
    if rc:
        raise GpukError(rc, "gpuk_increment_floats")


def copy_bytes(dst, src, nbytes: int, stream=None) -> None:
    rc = lib().gpuk_copy_bytes(_ptr(dst), _ptr(src), nbytes, _stream(stream))
    if rc:
        raise GpukError(rc, "gpuk_copy_bytes")


def read_bytes(src, nbytes: int, sink, stream=None) -> None:
    rc = lib().gpuk_read_bytes(_ptr(src), nbytes, _ptr(sink), _stream(stream))
    if rc:
        raise GpukError(rc, "gpuk_read_bytes")


def fill_bytes(dst, nbytes: int, seed: int = 1, stream=None) -> None:
    rc = lib().gpuk_fill_bytes(_ptr(dst), nbytes, seed & 0xFFFFFFFF, _stream(stream))
    if rc:
        raise GpukError(rc, "gpuk_fill_bytes")


def empty_grid(workgroups: int, lanes: int, lds_bytes: int = 0, stream=None) -> None:
    rc = lib().gpuk_empty_grid(workgroups, lanes, lds_bytes, _stream(stream))
    if rc:
        raise GpukError(rc, "gpuk_empty_grid")


def rope_rms_2way(q0, k0, q1, k1, w_q0, w_k0, w_q1, w_k1, cos_sin0, cos_sin1, batch_size, T0, T1, Hq, Hk, D,
                  is_interleaved, eps, out_q01, out_k01, stream=None) -> None:
    rc = lib().gpuk_rope_rms_2way(_ptr(q0), _ptr(k0), _ptr(q1), _ptr(k1), _ptr(w_q0), _ptr(w_k0), _ptr(w_q1),
                                  _ptr(w_k1), _ptr(cos_sin0), _ptr(cos_sin1), batch_size, T0, T1, Hq, Hk, D,
                                  int(is_interleaved), eps, DTYPE[q0.dtype], _ptr(out_q01), _ptr(out_k01),
                                  _stream(stream))
    if rc:
        raise GpukError(rc, "gpuk_rope_rms_2way")
