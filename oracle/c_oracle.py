"""ctypes loader for oracle/libgpuk_oracle.so (the plain-C CPU checker).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py, never by the product package.  Takes CPU torch tensors,
passes raw pointers; nothing here computes.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional, Sequence

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libgpuk_oracle.so")
_lib = None

DT = {torch.bfloat16: 0, torch.float16: 1}


def build(force: bool = False) -> str:
    """Compile the checker with gcc (a checker build, not a use of it)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.gpuk_oracle_f32_to_bf16.restype = C.c_uint16
        L.gpuk_oracle_f32_to_bf16.argtypes = [C.c_float]
        L.gpuk_oracle_f32_to_fp16.restype = C.c_uint16
        L.gpuk_oracle_f32_to_fp16.argtypes = [C.c_float]
        L.gpuk_oracle_fp16_to_f32.restype = C.c_float
        L.gpuk_oracle_fp16_to_f32.argtypes = [C.c_uint16]
        L.gpuk_oracle_f32_to_e4m3fn.restype = C.c_uint8
        L.gpuk_oracle_f32_to_e4m3fn.argtypes = [C.c_float]
        L.gpuk_oracle_e4m3fn_to_f32.restype = C.c_float
        L.gpuk_oracle_e4m3fn_to_f32.argtypes = [C.c_uint8]
        L.gpuk_oracle_e4m3fn_table_bf16.restype = None
        L.gpuk_oracle_e4m3fn_table_bf16.argtypes = [C.c_void_p]
        L.gpuk_oracle_add_rmsnorm_quant.restype = C.c_int
        L.gpuk_oracle_add_rmsnorm_quant.argtypes = [C.c_void_p] * 6 + [C.c_int64, C.c_int64, C.c_float, C.c_int, C.c_int, C.c_float]
        L.gpuk_oracle_rope_rms.restype = C.c_int
        L.gpuk_oracle_rope_rms.argtypes = (
            [C.c_void_p] * 5 + [C.c_int64, C.c_int64, C.c_int] + [C.c_int64] * 5 +
            [C.c_int, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_int] + [C.c_void_p] * 4 +
            [C.c_float, C.c_float, C.c_int])
        L.gpuk_oracle_rope_rms_2way.restype = C.c_int
        L.gpuk_oracle_rope_rms_2way.argtypes = (
            [C.c_void_p] * 10 + [C.c_int64] * 6 + [C.c_int, C.c_float, C.c_int, C.c_void_p, C.c_void_p])
        L.gpuk_oracle_count_div_rcp_mismatch.restype = C.c_int64
        L.gpuk_oracle_count_div_rcp_mismatch.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        for name in ("gpuk_oracle_count_short_sqrt_mismatch", "gpuk_oracle_count_short_rcp_mismatch"):
            getattr(L, name).restype = C.c_int64
            getattr(L, name).argtypes = [C.c_uint32, C.c_int64, C.c_int]
        _lib = L
    return _lib


def _p(t: Optional[torch.Tensor]):
    if t is None:
        return None
    assert t.device.type == "cpu" and t.is_contiguous()
    return t.data_ptr()


def e4m3fn_table_bf16() -> torch.Tensor:
    out = torch.empty(65536, dtype=torch.uint8)
    lib().gpuk_oracle_e4m3fn_table_bf16(out.data_ptr())
    return out


def add_rmsnorm_quant(x, residual_in, gamma, eps, quant, fp8_max=448.0, static_scale=None):
    """Returns (residual_out, norm_out, scale); norm_out is uint8 codes for quant 1/3."""
    T, H = x.shape
    res_out = torch.empty_like(x)
    if quant == 0:
        norm = torch.empty_like(x)
        scale = torch.empty(1, dtype=torch.float32)
    elif quant == 1:
        norm = torch.empty((T, H), dtype=torch.uint8)
        scale = torch.empty((T, 1), dtype=torch.float32)
    else:
        norm = torch.empty((T, H), dtype=torch.uint8)
        scale = static_scale.reshape(1).float().clone()
    rc = lib().gpuk_oracle_add_rmsnorm_quant(_p(x), _p(residual_in), _p(gamma), _p(res_out), _p(norm), _p(scale),
                                             T, H, eps, DT[x.dtype], quant, fp8_max)
    assert rc == 0, rc
    return res_out, norm, (None if quant == 0 else scale)


def rope_rms(qkv, qw, kw, cos_sin, positions, T, Hq, Hk, Hv, D, is_neox, eps,
             mrope_section: Optional[Sequence[int]] = None, is_interleaved: bool = False,
             q_out=None, k_cache=None, v_cache=None, kv_loc=None, k_scale=1.0, v_scale=1.0):
    """In place on qkv when q_out is None, else the set_kv form.  positions [T] or [3,T] (any strides)."""
    if positions.dim() == 1:
        n_axes, ps_axis, ps_token = 1, 0, positions.stride(0)
    else:
        n_axes, ps_axis, ps_token = 3, positions.stride(0), positions.stride(1)
    sec = torch.tensor(list(mrope_section) if mrope_section is not None else [0, 0, 0], dtype=torch.int64)
    set_kv = q_out is not None
    kv_fp8 = bool(set_kv and k_cache.dtype != qkv.dtype)
    rc = lib().gpuk_oracle_rope_rms(
        _p(qkv), _p(qw), _p(kw), _p(cos_sin), positions.data_ptr(), ps_axis, ps_token, n_axes,
        T, Hq, Hk, Hv, D, int(is_neox), _p(sec), int(is_interleaved), eps, DT[qkv.dtype],
        int(set_kv), _p(q_out), _p(k_cache), _p(v_cache), _p(kv_loc), k_scale, v_scale, int(kv_fp8))
    assert rc == 0, rc


def rope_rms_2way(q0, k0, q1, k1, wq0, wk0, wq1, wk1, cs0, cs1, B, T0, T1, Hq, Hk, D, is_interleaved, eps):
    out_q = torch.empty((B, T0 + T1, Hq, D), dtype=q0.dtype)
    out_k = torch.empty((B, T0 + T1, Hk, D), dtype=k0.dtype)
    rc = lib().gpuk_oracle_rope_rms_2way(_p(q0), _p(k0), _p(q1), _p(k1), _p(wq0), _p(wk0), _p(wq1), _p(wk1),
                                         _p(cs0), _p(cs1), B, T0, T1, Hq, Hk, D, int(is_interleaved), eps,
                                         DT[q0.dtype], _p(out_q), _p(out_k))
    assert rc == 0, rc
    return out_q, out_k


def count_div_rcp_mismatch(a: torch.Tensor, b: torch.Tensor) -> int:
    """a, b: fp32 CPU tensors of equal length; see gpuk_oracle_count_div_rcp_mismatch."""
    assert a.dtype == torch.float32 and b.dtype == torch.float32 and a.numel() == b.numel()
    return lib().gpuk_oracle_count_div_rcp_mismatch(_p(a.contiguous()), _p(b.contiguous()), a.numel())


def count_short_sqrt_mismatch(first_bits: int, n: int, first_guess_ulp: int) -> int:
    """See gpuk_oracle_count_short_sqrt_mismatch: fp32 bit patterns first_bits .. first_bits + n - 1."""
    return lib().gpuk_oracle_count_short_sqrt_mismatch(first_bits, n, first_guess_ulp)


def count_short_rcp_mismatch(first_bits: int, n: int, first_guess_ulp: int) -> int:
    """See gpuk_oracle_count_short_rcp_mismatch."""
    return lib().gpuk_oracle_count_short_rcp_mismatch(first_bits, n, first_guess_ulp)
