"""ctypes loader for oracle/_ref/libgpuk_ref.so: the reference repository's own kernels for this path, compiled for
gfx950 from the reference's headers (recipe: `make -C oracle ref`; sources oracle/ref_rope_kernels.hip and
oracle/ref_epilogue_kernels.hip say exactly which reference code runs).

TEST INFRASTRUCTURE ONLY: used by tests/ and by the reference-timing leg of bench.py, never by the product package.
The library exists only where it was built from a checkout of the reference; `available()` says whether it does.
Takes torch tensors on the GPU, passes raw pointers, launches on torch's current stream.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional, Sequence

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_ref", "libgpuk_ref.so")
REFERENCE_ROOT = "/root/reference"
_lib = None


def can_build() -> bool:
    return os.path.isdir(os.path.join(REFERENCE_ROOT, "src", "impl"))


def build(force: bool = False) -> Optional[str]:
    """Compile the reference's kernels (a checker build).  Returns None where the reference is not present."""
    if not can_build():
        return None
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean-ref"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE, "ref"], stdout=subprocess.DEVNULL)
    return LIB_PATH


def available() -> bool:
    return os.path.exists(LIB_PATH)


def lib():
    global _lib
    if _lib is None:
        L = C.CDLL(LIB_PATH)
        i64, vp = C.c_int64, C.c_void_p
        L.gpuk_ref_rope_rms.restype = C.c_int
        L.gpuk_ref_rope_rms.argtypes = [vp] * 5 + [i64, i64, C.c_int] + [i64] * 5 + [C.c_int, vp, C.c_int, C.c_double, vp]
        L.gpuk_ref_mrope_rms_set_kv.restype = C.c_int
        L.gpuk_ref_mrope_rms_set_kv.argtypes = ([vp] * 5 + [i64] * 7 + [C.c_int, vp, C.c_int, C.c_double] + [vp] * 4 +
                                               [C.c_float, C.c_float, C.c_int, vp])
        L.gpuk_ref_rope_rms_2way.restype = C.c_int
        L.gpuk_ref_rope_rms_2way.argtypes = [vp] * 10 + [i64] * 6 + [C.c_int, C.c_double, vp, vp, vp]
        L.gpuk_ref_epilogue_rows.restype = C.c_int
        L.gpuk_ref_epilogue_rows.argtypes = [vp] * 6 + [i64, i64, C.c_float, C.c_int, vp]
        _lib = L
    return _lib


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc: int, what: str):
    if rc:
        raise RuntimeError(f"{what}: the reference launcher was refused or failed (status {rc})")


def _bf16_cuda(*tensors):
    for t in tensors:
        assert t.is_cuda and t.is_contiguous() and t.dtype == torch.bfloat16, (t.device, t.dtype, t.is_contiguous())


def _section(section: Optional[Sequence[int]]):
    return None if section is None else (C.c_int64 * 3)(*section)


def _in_range(index: torch.Tensor, bound: int) -> bool:
    return int(index.min()) >= 0 and int(index.max()) < bound   # synchronises: skipped by timing loops (check_values=False)


def rope_rms(qkv, qw, kw, cos_sin, positions, T, hq, hk, hv, D, is_neox, eps, mrope_section=None, is_interleaved=False,
             check_values=True):
    """In place on qkv [T, hq+hk+hv, D].  positions [T] (rope) or [3, T] (mrope), int64, values below cos_sin's rows."""
    _bf16_cuda(qkv, qw, kw, cos_sin)
    assert qkv.numel() == T * (hq + hk + hv) * D and qw.numel() == D and kw.numel() == D and cos_sin.shape[-1] == D
    assert positions.dtype == torch.int64 and positions.is_cuda
    assert not check_values or _in_range(positions, cos_sin.shape[0])
    if mrope_section is None:
        assert positions.dim() == 1 and positions.numel() == T
        ps0, ps1, n_axes = 0, positions.stride(0), 1
    else:
        assert positions.dim() == 2 and positions.shape == (3, T)
        ps0, ps1, n_axes = positions.stride(0), positions.stride(1), 3
    _check(lib().gpuk_ref_rope_rms(qkv.data_ptr(), qw.data_ptr(), kw.data_ptr(), cos_sin.data_ptr(), positions.data_ptr(),
                                   ps0, ps1, n_axes, T, hq, hk, hv, D, int(is_neox), _section(mrope_section),
                                   int(is_interleaved), eps, _stream()), "gpuk_ref_rope_rms")


def mrope_rms_set_kv(qkv, qw, kw, cos_sin, positions, T, hq, hk, hv, D, is_neox, eps, q, k_cache, v_cache, kv_loc,
                     k_scale, v_scale, mrope_section=None, is_interleaved=False, check_values=True):
    """positions [T] is passed as three equal rows (stride 0 over the axes) with one section covering D/2, which is
    how the reference's set_kv kernel does plain RoPE."""
    _bf16_cuda(qkv, qw, kw, cos_sin, q)
    assert qkv.numel() == T * (hq + hk + hv) * D and q.numel() == T * hq * D and cos_sin.shape[-1] == D
    assert k_cache.is_cuda and v_cache.is_cuda and k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_cache.dtype == v_cache.dtype and k_cache.dtype in (torch.bfloat16, torch.float8_e4m3fn)
    slots = k_cache.shape[0]
    assert k_cache.numel() == slots * hk * D and v_cache.numel() == slots * hv * D
    assert kv_loc.dtype == torch.int64 and kv_loc.is_cuda and kv_loc.numel() >= T
    assert positions.dtype == torch.int64 and positions.is_cuda
    assert not check_values or (_in_range(kv_loc[:T], slots) and _in_range(positions, cos_sin.shape[0]))
    if mrope_section is None:
        assert positions.dim() == 1 and positions.numel() == T
        ps0, ps1, section = 0, positions.stride(0), [D // 2, 0, 0]
    else:
        assert positions.shape == (3, T)
        ps0, ps1, section = positions.stride(0), positions.stride(1), list(mrope_section)
    _check(lib().gpuk_ref_mrope_rms_set_kv(qkv.data_ptr(), qw.data_ptr(), kw.data_ptr(), cos_sin.data_ptr(),
                                           positions.data_ptr(), ps0, ps1, T, hq, hk, hv, D, int(is_neox),
                                           _section(section), int(is_interleaved), eps, q.data_ptr(), k_cache.data_ptr(),
                                           v_cache.data_ptr(), kv_loc.data_ptr(), k_scale, v_scale,
                                           int(k_cache.dtype == torch.float8_e4m3fn), _stream()),
           "gpuk_ref_mrope_rms_set_kv")


def rope_rms_2way(q0, k0, q1, k1, w_q0, w_k0, w_q1, w_k1, cos_sin0, cos_sin1, B, T0, T1, hq, hk, D, is_interleaved, eps,
                  out_q01, out_k01):
    _bf16_cuda(q0, k0, q1, k1, w_q0, w_k0, w_q1, w_k1, cos_sin0, cos_sin1, out_q01, out_k01)
    assert q0.numel() == B * T0 * hq * D and k0.numel() == B * T0 * hk * D
    assert q1.numel() == B * T1 * hq * D and k1.numel() == B * T1 * hk * D
    assert cos_sin0.numel() == T0 * D and cos_sin1.numel() == T1 * D
    assert out_q01.numel() == B * (T0 + T1) * hq * D and out_k01.numel() == B * (T0 + T1) * hk * D
    _check(lib().gpuk_ref_rope_rms_2way(q0.data_ptr(), k0.data_ptr(), q1.data_ptr(), k1.data_ptr(), w_q0.data_ptr(),
                                        w_k0.data_ptr(), w_q1.data_ptr(), w_k1.data_ptr(), cos_sin0.data_ptr(),
                                        cos_sin1.data_ptr(), B, T0, T1, hq, hk, D, int(is_interleaved), eps,
                                        out_q01.data_ptr(), out_k01.data_ptr(), _stream()), "gpuk_ref_rope_rms_2way")


def epilogue_rows(x, residual_in, gamma, residual_out, norm_out, scale_out, eps, quant):
    """The reference's epilogue device code under a one-GPU caller (see oracle/ref_epilogue_kernels.hip).
    quant 0: norm_out bf16; quant 1: norm_out 1-byte codes of the reference's fp8e4m3fn (maximum 240), scale_out [T]."""
    _bf16_cuda(x, residual_in, gamma, residual_out)
    T, H = x.shape
    assert H in (1024, 2048, 4096, 8192) and gamma.numel() == H
    assert residual_in.shape == x.shape and residual_out.shape == x.shape
    assert norm_out.is_cuda and norm_out.is_contiguous() and norm_out.numel() == T * H
    assert norm_out.element_size() == (1 if quant else 2)
    if quant:
        assert scale_out.is_cuda and scale_out.dtype == torch.float32 and scale_out.numel() >= T
    _check(lib().gpuk_ref_epilogue_rows(x.data_ptr(), residual_in.data_ptr(), gamma.data_ptr(), residual_out.data_ptr(),
                                        norm_out.data_ptr(), scale_out.data_ptr() if quant else None, T, H, eps, quant,
                                        _stream()), "gpuk_ref_epilogue_rows")
