"""CPU restatement of the reference's torch oracles for the two fused paths.

TEST INFRASTRUCTURE ONLY.  Nothing in the product path (gpuk_amd/, the C-ABI
library, the torch extension) may import this module; it is imported by
tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg as the
checker / the timed CPU baseline, never as a fallback.

Every function follows the reference's own pure-torch reference code
op by op, so that the rounding sequence (which torch op rounds to bf16 where)
is identical.  Citations are into the reference repository.

Deliberate, documented deviations from the reference's torch code (both follow
the reference's *kernel* where the torch code and the kernel disagree or the
torch code is undefined):

* all-zero rows in add_rmsnorm_quant: the torch code yields scale 0 and 0/0 =
  NaN codes; the kernel sets scale = 1 (src/impl/all_reduce_fusion_impl.h:217,221).
  We follow the kernel.
* a KV cache whose dtype equals the qkv dtype: the kernel stores K/V unscaled
  (src/impl/rope_rms_impl.h:213-214,225-226) while the torch test code divides by
  k_scale/v_scale (test/test_fused_mrope_rms_set_kv.py:127-128, only ever run
  with an fp8 cache).  `scale_same_dtype_cache=False` (default) follows the kernel.

Parity pinning (see tests/test_oracle_*.py): e4m3fn encode against an
exhaustive torch-CPU table over all 65536 bf16 patterns; RMSNorm against an fp64
brute force and scale invariances; the double bf16 rounding against a
single-rounding discriminator; RoPE against rotation identities and an fp64
rotation; mRoPE selection against three independent index formulas; KV scatter
against permutation invariants; and, on the GPU, against the reference's own
kernels built into oracle/_ref (tests/test_gpu_reference_kernels.py holds them to
this restatement at the reference tests' allclose bar).  The reference ships no
golden vectors for this path.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch
from torch import Tensor

FP8_DTYPE = torch.float8_e4m3fn
FP8_MAX_OCP = 448.0      # OCP e4m3fn finite maximum (what gfx950 hardware encodes)
FP8_MAX_REFERENCE = 240.0  # the reference's software fp8e4m3fn::max_value (src/common/float8.h:216-218)

QUANT_NONE = 0       # norm_out in the activation dtype                 (all_reduce_fusion_impl.h:13-17)
QUANT_DYNAMIC = 1    # per-token e4m3fn, scale_out[T,1] written
QUANT_STATIC = 3     # per-tensor e4m3fn, scale[1] read  (additive mode, no reference counterpart)


def rms_norm_forward(x: Tensor, weight: Tensor, eps: float, rstd_ulp_offset: int = 0) -> Tensor:
    """gpuk/__init__.py:150-155 and test/test_fused_rope_rms.py:8-13.

    variance in fp32; x*rstd is a (low-precision tensor) x (fp32 tensor) product and
    so is evaluated and rounded in fp32, then rounded to the input dtype; the final
    weight*x is evaluated in the input dtype (one more rounding).

    `rstd_ulp_offset` (test aid, 0 in the reference): move rstd by that many fp32 ULPs, to
    show that an output row is bit-exact up to the summation order of the variance.
    """
    input_dtype = x.dtype
    variance = x.float().pow(2).mean(-1, keepdim=True)
    rstd = torch.rsqrt(variance + eps)
    if rstd_ulp_offset:
        rstd = (rstd.view(torch.int32) + rstd_ulp_offset).view(torch.float32)
    x = x * rstd
    x = x.to(input_dtype)
    return weight * x


def add_rmsnorm_quant_ref(
    allreduce_in: Tensor,
    residual_in: Tensor,
    rms_weight: Tensor,
    eps: float,
    quant: int = QUANT_DYNAMIC,
    fp8_max: float = FP8_MAX_OCP,
    static_scale: Optional[Tensor] = None,
    rstd_ulp_offset: int = 0,
) -> Tuple[Tensor, Tensor, Optional[Tensor]]:
    """gpuk/__init__.py:147-173 (allreduce_add_rms_native) without the dist.all_reduce.

    Returns (residual_out, norm_out, scale).  `quant`:
      QUANT_NONE    -> norm_out in the input dtype, scale None          (:165-173)
      QUANT_DYNAMIC -> per-token scale = amax/fp8_max, codes e4m3fn      (:158-164)
      QUANT_STATIC  -> codes = e4m3fn(clamp(norm/static_scale))          (additive)
    """
    residual_out = allreduce_in + residual_in
    norm_out = rms_norm_forward(residual_out, rms_weight, eps, rstd_ulp_offset)
    if quant == QUANT_NONE:
        return residual_out, norm_out, None
    if quant == QUANT_DYNAMIC:
        scale, _ = norm_out.float().abs().max(dim=-1, keepdim=True)
        scale = scale / fp8_max
        # kernel semantics for an all-zero row (all_reduce_fusion_impl.h:217)
        scale = torch.where(scale == 0, torch.ones_like(scale), scale)
    elif quant == QUANT_STATIC:
        assert static_scale is not None and static_scale.numel() == 1
        scale = static_scale.reshape(1).float()
    else:
        raise ValueError(f"unsupported quant mode {quant}")
    q = norm_out / scale                      # low-precision / fp32 -> fp32 true division
    q.clamp_(min=-fp8_max, max=fp8_max)
    q = q.to(FP8_DTYPE)
    return residual_out, q, scale


def static_scale_for(allreduce_in: Tensor, residual_in: Tensor, rms_weight: Tensor, eps: float,
                     fp8_max: float = FP8_MAX_OCP) -> Tensor:
    """Per-tensor scale 'computed once' for the static configuration: amax(normed)/fp8_max."""
    _, n, _ = add_rmsnorm_quant_ref(allreduce_in, residual_in, rms_weight, eps, QUANT_NONE)
    return (n.float().abs().max() / fp8_max).reshape(1)


def apply_rotary_emb(x: Tensor, cos: Tensor, sin: Tensor, is_neox_style: bool) -> Tensor:
    """test/test_fused_rope_rms.py:16-34.  x [T, heads, D]; cos, sin [T, D/2].

    Everything is evaluated in x.dtype: each product and the sum/difference round.
    """
    cos = cos.unsqueeze(-2).to(x.dtype)
    sin = sin.unsqueeze(-2).to(x.dtype)
    if is_neox_style:
        x1, x2 = torch.chunk(x, 2, dim=-1)
    else:
        x1 = x[..., ::2]
        x2 = x[..., 1::2]
    o1 = x1 * cos - x2 * sin
    o2 = x2 * cos + x1 * sin
    if is_neox_style:
        return torch.cat((o1, o2), dim=-1)
    return torch.stack((o1, o2), dim=-1).flatten(-2)


def mrope_select(x: Tensor, mrope_section: Sequence[int], is_interleaved: bool) -> Tensor:
    """Pick, per rotary frequency, which of the 3 position axes supplies cos (or sin).

    x [3, T, D/2].  Interleaved: test/test_fused_mrope_rms_set_kv.py:16-24.
    Chunked: test/test_fused_mrope_rms_set_kv.py:108-115.
    """
    if is_interleaved:
        x_t = x[0].clone()
        x_t[..., 1:mrope_section[1] * 3:3] = x[1, ..., 1:mrope_section[1] * 3:3]
        x_t[..., 2:mrope_section[2] * 3:3] = x[2, ..., 2:mrope_section[2] * 3:3]
        return x_t
    return torch.cat([m[i] for i, m in enumerate(x.split(list(mrope_section), dim=-1))], dim=-1)


def gather_cos_sin(cos_sin: Tensor, positions: Tensor, head_size: int,
                   mrope_section: Optional[Sequence[int]], is_interleaved: bool) -> Tuple[Tensor, Tensor]:
    """cos, sin [T, D/2] for 1-D positions (test_fused_rope_rms.py:80-82) or 3xT mRoPE
    positions (test_fused_mrope_rms_set_kv.py:98-115)."""
    cos_sin = cos_sin.view(-1, head_size)
    cs = cos_sin[positions]
    cos, sin = cs.chunk(2, dim=-1)
    if positions.dim() == 2:
        assert mrope_section is not None
        cos = mrope_select(cos, mrope_section, is_interleaved)
        sin = mrope_select(sin, mrope_section, is_interleaved)
    return cos, sin


def rope_rms_ref(
    qkv: Tensor, qw: Tensor, kw: Tensor, cos_sin: Tensor, positions: Tensor,
    num_tokens: int, num_heads_q: int, num_heads_k: int, num_heads_v: int, head_size: int,
    is_neox_style: bool, eps: float,
    mrope_section: Optional[Sequence[int]] = None, is_interleaved: bool = False,
    rstd_ulp_offset: int = 0,
) -> Tuple[Tensor, Tensor, Tensor]:
    """test/test_fused_rope_rms.py:52-94 (1-D positions) and
    test/test_fused_mrope_rms.py:62-130 (3xT positions).  Returns (q, k, v) as
    [T, heads, D]; v is the untouched input slice.  `rstd_ulp_offset` (test aid, 0 in the
    reference) moves every head's rstd by that many fp32 ULPs, see rms_norm_forward."""
    q_size = num_heads_q * head_size
    k_size = num_heads_k * head_size
    v_size = num_heads_v * head_size
    qkv = qkv.view(num_tokens, q_size + k_size + v_size)
    q, k, v = qkv.split([q_size, k_size, v_size], dim=-1)
    q = rms_norm_forward(q.reshape(num_tokens, num_heads_q, head_size), qw, eps, rstd_ulp_offset)
    k = rms_norm_forward(k.reshape(num_tokens, num_heads_k, head_size), kw, eps, rstd_ulp_offset)
    cos, sin = gather_cos_sin(cos_sin, positions, head_size, mrope_section, is_interleaved)
    q = apply_rotary_emb(q, cos, sin, is_neox_style)
    k = apply_rotary_emb(k, cos, sin, is_neox_style)
    return q, k, v.reshape(num_tokens, num_heads_v, head_size)


def rope_rms_set_kv_ref(
    qkv: Tensor, qw: Tensor, kw: Tensor, cos_sin: Tensor, positions: Tensor,
    num_tokens: int, num_heads_q: int, num_heads_k: int, num_heads_v: int, head_size: int,
    is_neox_style: bool, eps: float,
    q_out: Tensor, k_cache: Tensor, v_cache: Tensor, kv_loc: Tensor,
    k_scale: float, v_scale: float,
    mrope_section: Optional[Sequence[int]] = None, is_interleaved: bool = False,
    scale_same_dtype_cache: bool = False, rstd_ulp_offset: int = 0,
) -> None:
    """test/test_fused_mrope_rms_set_kv.py:62-130.  Mutates q_out, k_cache, v_cache.

    fp8 cache: (k / k_scale) is a bf16 tensor divided by a python float, evaluated as
    float(k)/float(scale) and rounded to bf16, then cast to e4m3fn (:127-128).
    """
    q, k, v = rope_rms_ref(qkv, qw, kw, cos_sin, positions, num_tokens, num_heads_q, num_heads_k,
                           num_heads_v, head_size, is_neox_style, eps, mrope_section, is_interleaved, rstd_ulp_offset)
    if k_cache.dtype != qkv.dtype or scale_same_dtype_cache:
        k = k / k_scale
        v = v / v_scale
    # a negative slot marks a token without a place in the cache (this build's extension; the reference's code would
    # index out of range): its K and V are dropped
    keep = kv_loc[:num_tokens] >= 0
    k_cache[kv_loc[:num_tokens][keep]] = k.to(k_cache.dtype)[keep]
    v_cache[kv_loc[:num_tokens][keep]] = v.to(v_cache.dtype)[keep]
    q_out.copy_(q.reshape(q_out.shape))


def rope_rms_2way_ref(
    q0: Tensor, k0: Tensor, q1: Tensor, k1: Tensor,
    w_q0: Tensor, w_k0: Tensor, w_q1: Tensor, w_k1: Tensor,
    cos_sin0: Tensor, cos_sin1: Tensor,
    batch_size: int, num_tokens0: int, num_tokens1: int, num_heads_q: int, num_heads_k: int,
    head_size: int, is_interleaved: bool, eps: float, rstd_ulp_offset: int = 0,
) -> Tuple[Tensor, Tensor]:
    """test/test_fused_rope_rms_2way.py:37-81: two token streams with their own norm
    weights and per-token cos/sin rows, concatenated along the token axis."""
    is_neox_style = not is_interleaved
    q0n = rms_norm_forward(q0.view(batch_size, num_tokens0, num_heads_q, head_size), w_q0, eps, rstd_ulp_offset)
    k0n = rms_norm_forward(k0.view(batch_size, num_tokens0, num_heads_k, head_size), w_k0, eps, rstd_ulp_offset)
    q1n = rms_norm_forward(q1.view(batch_size, num_tokens1, num_heads_q, head_size), w_q1, eps, rstd_ulp_offset)
    k1n = rms_norm_forward(k1.view(batch_size, num_tokens1, num_heads_k, head_size), w_k1, eps, rstd_ulp_offset)
    cos0, sin0 = cos_sin0.view(num_tokens0, head_size).chunk(2, dim=-1)
    cos1, sin1 = cos_sin1.view(num_tokens1, head_size).chunk(2, dim=-1)
    q0o = apply_rotary_emb(q0n, cos0, sin0, is_neox_style)
    k0o = apply_rotary_emb(k0n, cos0, sin0, is_neox_style)
    q1o = apply_rotary_emb(q1n, cos1, sin1, is_neox_style)
    k1o = apply_rotary_emb(k1n, cos1, sin1, is_neox_style)
    return torch.cat([q0o, q1o], dim=1), torch.cat([k0o, k1o], dim=1)
