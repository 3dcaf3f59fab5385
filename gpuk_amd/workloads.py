"""Seeded synthetic inputs for the five benchmark configurations.

All draws come from one CPU `torch.Generator().manual_seed(seed)` per configuration, in
the order listed in each function, so the CPU checker and the GPU run see identical
bytes.  Tensors are returned on the CPU; callers move them to the device.

Shapes follow the reference's operator contracts:
  add+RMSNorm+quant : allreduce_in/residual_in [T,H], rms_gamma [H]   (src/ops/all_reduce_fusion.cpp:363-396)
  rope              : qkv [T, Hq+Hk+Hv, D], qw/kw [D], cos_sin [max_pos, D] (cos | sin halves),
                      positions [T] or [3,T] int64, k_cache/v_cache [slots, H, D], kv_loc [T] int64
                                                                       (src/ops/fused_rope.cpp:91-166)
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import torch

DECODE_TOKENS = (1, 8, 32, 128, 512)          # the benchmark definition's decode sweep
DECODE_TOKENS_WIDE = (1, 8, 32, 128, 256, 512, 1024, 2048)   # the same with the mid-range filled in


@dataclass
class NormQuantInputs:
    x: torch.Tensor
    residual: torch.Tensor
    gamma: torch.Tensor
    eps: float = 1e-6

    @property
    def tokens(self) -> int:
        return self.x.shape[0]

    @property
    def hidden(self) -> int:
        return self.x.shape[1]


@dataclass
class RopeInputs:
    qkv: torch.Tensor
    qw: torch.Tensor
    kw: torch.Tensor
    cos_sin: torch.Tensor
    positions: torch.Tensor
    kv_loc: torch.Tensor
    num_tokens: int
    num_heads_q: int
    num_heads_k: int
    num_heads_v: int
    head_size: int
    num_slots: int
    is_neox: bool = True
    eps: float = 1e-6
    mrope_section: Optional[List[int]] = None
    is_interleaved: bool = False
    kv_dtype: torch.dtype = torch.bfloat16
    k_scale: float = 1.0
    v_scale: float = 1.0
    block_size: int = 16
    extra: dict = field(default_factory=dict)

    def new_cache(self, fill_seed: int = 1234):
        """K and V caches pre-filled with a recognisable byte pattern, so that a write to a
        slot that should stay untouched is visible."""
        g = torch.Generator().manual_seed(fill_seed)
        shape_k = (self.num_slots, self.num_heads_k, self.head_size)
        shape_v = (self.num_slots, self.num_heads_v, self.head_size)
        if self.kv_dtype == torch.float8_e4m3fn:
            # finite codes only (avoid 0x7f / 0xff NaN patterns so equality checks are plain)
            k = torch.randint(0, 0x7E, shape_k, generator=g, dtype=torch.uint8).view(torch.float8_e4m3fn)
            v = torch.randint(0, 0x7E, shape_v, generator=g, dtype=torch.uint8).view(torch.float8_e4m3fn)
        elif self.kv_dtype in (torch.float32, torch.float64):
            k = (torch.randn(shape_k, generator=g) * 1000.0).to(self.kv_dtype)
            v = (torch.randn(shape_v, generator=g) * 1000.0).to(self.kv_dtype)
        else:
            k = torch.randint(-30000, 30000, shape_k, generator=g, dtype=torch.int16).view(self.kv_dtype)
            v = torch.randint(-30000, 30000, shape_v, generator=g, dtype=torch.int16).view(self.kv_dtype)
        return k, v


def norm_quant_inputs(tokens: int, hidden: int, seed: int = 0, res_sigma: float = 1.0,
                      outlier_frac: float = 0.0, outlier_mag: float = 50.0,
                      dtype: torch.dtype = torch.bfloat16) -> NormQuantInputs:
    """x ~ N(0,1), residual ~ N(0, res_sigma^2), gamma ~ N(1, 0.1^2); optionally a fraction of x
    replaced by +-outlier_mag (Bernoulli mask, then random sign, from the same generator)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((tokens, hidden), generator=g, dtype=torch.float32)
    r = torch.randn((tokens, hidden), generator=g, dtype=torch.float32) * res_sigma
    gamma = 1.0 + 0.1 * torch.randn((hidden,), generator=g, dtype=torch.float32)
    if outlier_frac > 0:
        mask = torch.rand((tokens, hidden), generator=g) < outlier_frac
        sign = torch.randint(0, 2, (tokens, hidden), generator=g, dtype=torch.int8).float() * 2 - 1
        x = torch.where(mask, sign * outlier_mag, x)
    return NormQuantInputs(x.to(dtype), r.to(dtype), gamma.to(dtype))


def config1() -> NormQuantInputs:
    """Static per-tensor quant: tokens=128, hidden=4096, x,res ~ N(0,1), seed 0."""
    return norm_quant_inputs(128, 4096, seed=0)


def config2(tokens: int = 8192, hidden: int = 8192) -> NormQuantInputs:
    """Dynamic per-token quant: 8192x8192, x ~ N(0,1), residual ~ N(0, sigma=2), 1% of x = +-50."""
    return norm_quant_inputs(tokens, hidden, seed=0, res_sigma=2.0, outlier_frac=0.01)


def config5_norm(tokens: int) -> NormQuantInputs:
    """Decode sweep: hidden 7168, x,res ~ N(0,1)."""
    return norm_quant_inputs(tokens, 7168, seed=5)


def rope_table(max_pos: int, head_size: int, base: float = 1e6, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """cos_sin [max_pos, D]: cos(p*f_i) | sin(p*f_i), f_i = base^(-2i/D), evaluated in fp32 then cast."""
    half = head_size // 2
    inv_freq = 1.0 / (base ** (torch.arange(0, half, dtype=torch.float32) * 2.0 / head_size))
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * inv_freq[None, :]
    return torch.cat([ang.cos(), ang.sin()], dim=-1).to(dtype).contiguous()


def rope_inputs(num_tokens: int, hq: int, hk: int, hv: int, head_size: int, seed: int,
                max_pos: int = 32768, num_slots: Optional[int] = None, base: float = 1e6,
                kv_dtype: torch.dtype = torch.bfloat16, k_scale: float = 1.0, v_scale: float = 1.0,
                dtype: torch.dtype = torch.bfloat16, is_neox: bool = True, random_table: bool = False) -> RopeInputs:
    g = torch.Generator().manual_seed(seed)
    qkv = torch.randn((num_tokens, hq + hk + hv, head_size), generator=g, dtype=torch.float32).to(dtype)
    qw = (1.0 + 0.1 * torch.randn((head_size,), generator=g)).to(dtype)
    kw = (1.0 + 0.1 * torch.randn((head_size,), generator=g)).to(dtype)
    if random_table:   # the reference's own tests use a random table (test_fused_rope_rms.py:154)
        cos_sin = torch.randn((max_pos, head_size), generator=g).to(dtype)
    else:
        cos_sin = rope_table(max_pos, head_size, base, dtype)
    positions = torch.randint(0, max_pos, (num_tokens,), generator=g, dtype=torch.int64)
    if num_slots is None:
        num_slots = max(num_tokens, 16)
    kv_loc = torch.randperm(num_slots, generator=g)[:num_tokens].to(torch.int64).contiguous()
    return RopeInputs(qkv, qw, kw, cos_sin, positions, kv_loc, num_tokens, hq, hk, hv, head_size, num_slots,
                      is_neox=is_neox, kv_dtype=kv_dtype, k_scale=k_scale, v_scale=v_scale)


def config3(num_tokens: int = 4096) -> RopeInputs:
    """Qwen3-8B-like: Hq=32, Hk=Hv=8, D=128, NeoX, base 1e6, positions U[0,32768),
    cache 4096 blocks x 16 slots (bf16), distinct random slots."""
    return rope_inputs(num_tokens, 32, 8, 8, 128, seed=3, max_pos=32768, num_slots=4096 * 16)


def vl_positions(num_tokens: int, text_run: int = 1024, grid: int = 32) -> torch.Tensor:
    """3 x T (t,h,w) positions: runs of text (all three axes equal, increasing) alternating with
    grid x grid image segments (t constant, h = row, w = column, all offset by the running start;
    the following text resumes at max+1), truncated to num_tokens."""
    rows = [[], [], []]
    nxt = 0
    n = 0
    while n < num_tokens:
        m = min(text_run, num_tokens - n)
        for a in range(3):
            rows[a].extend(range(nxt, nxt + m))
        nxt += m
        n += m
        if n >= num_tokens:
            break
        m = min(grid * grid, num_tokens - n)
        idx = torch.arange(m)
        rows[0].extend([nxt] * m)
        rows[1].extend((nxt + idx // grid).tolist())
        rows[2].extend((nxt + idx % grid).tolist())
        nxt += grid
        n += m
    return torch.tensor(rows, dtype=torch.int64).contiguous()


def config4(num_tokens: int = 8192, is_interleaved: bool = False, text_only: bool = False) -> RopeInputs:
    """Qwen2-VL-like mRoPE: Hq=28, Hk=Hv=4, D=128, sections [16,24,24], text + 32x32 image segments
    (text_only: one run of text, the three position rows equal)."""
    inp = rope_inputs(num_tokens, 28, 4, 4, 128, seed=4, max_pos=32768, num_slots=max(num_tokens, 16) * 2)
    inp.positions = vl_positions(num_tokens, text_run=num_tokens if text_only else 1024)
    inp.mrope_section = [16, 24, 24]
    inp.is_interleaved = is_interleaved
    return inp


def config5_rope(num_tokens: int) -> RopeInputs:
    """Decode sweep: Hq=64, Hk=Hv=8, D=128, e4m3fn KV cache with static per-tensor k/v scales."""
    return rope_inputs(num_tokens, 64, 8, 8, 128, seed=50 + num_tokens, max_pos=32768, num_slots=4096 * 16,
                       kv_dtype=torch.float8_e4m3fn, k_scale=0.05, v_scale=0.02)


# ---------------------------------------------------------------- algorithmic bytes (compulsory traffic)

def norm_quant_bytes(tokens: int, hidden: int, quant: int, elem: int = 2) -> int:
    """x + residual_in + residual_out at `elem` bytes, codes 1 B (or norm_out at `elem`), gamma, scale."""
    if quant == 0:
        return 4 * elem * tokens * hidden + elem * hidden
    per = (3 * elem + 1) * tokens * hidden + elem * hidden
    return per + (4 * tokens if quant == 1 else 4)


def rope_set_kv_bytes(T: int, hq: int, hk: int, hv: int, D: int, n_axes: int, kv_elem: int, elem: int = 2) -> int:
    per = elem * D * (hq + hk + hv) + elem * D * hq + kv_elem * D * (hk + hv) + elem * D + 8 * n_axes + 8
    return per * T + 2 * elem * D


def rope_inplace_bytes(T: int, hq: int, hk: int, D: int, n_axes: int = 1, elem: int = 2) -> int:
    return (2 * elem * D * (hq + hk) + elem * D + 8 * n_axes) * T + 2 * elem * D
