"""A caller of the two fused paths: one decoder block with a paged KV cache.

The reference's own model (model/transformer_model.py) is plain torch: `RMSNorm` (:68-80), `Attention` with
per-head q/k norms, rotary embedding and a dense `[batch, heads, seq, head]` cache (:52-66, :82-156),
`FeedForward` (:170-180) and `TransformerBlock.forward` = `x + attn(norm(x))` then `x + ffn(norm(x))` (:235-242).
This module is that block with the memory-bound glue replaced by the fused operators:

    residual add + attention_norm / ffn_norm      -> gpuk.allreduce_rms (quant_type 0; world size 1: no all-reduce)
    q_norm, k_norm, rotary embedding, cache write -> gpuk.fused_rope_rms_set_kv (paged cache, slot per token)

and, beside it, `forward_unfused`: the same weights driven through the reference's torch sequence, which the
tests compare against and the benchmark times next to the fused path.  The GEMMs and the attention itself are
torch's in both paths; nothing here is a kernel.

Conventions that differ from the reference's model, because the fused operators need them:
  * the three projections are one weight `wqkv` whose output rows are `[q heads | k heads | v heads]`, which is
    the `qkv [T, Hq+Hk+Hv, D]` layout the operator reads (src/ops/fused_rope.cpp:91-113);
  * rotation is the NeoX form (`rope_interval_split=False` in the reference's `apply_rotary_emb`, :118-128),
    with the cos|sin table rounded to the activation type as the operator's tests do
    (test/test_fused_rope_rms.py:80-82);
  * the cache is paged: `[num_blocks * block_size, Hk, D]`, a sequence owning the blocks its table lists;
  * a block takes and returns the pair (sublayer output, residual stream) so that each residual add fuses with
    the norm that follows it.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

import gpuk_amd


@dataclass
class BlockArgs:
    """The subset of the reference's ModelArgs (model/transformer_model.py:23-49) a block needs."""
    dim: int = 4096
    n_heads: int = 32
    n_kv_heads: int = 8
    head_dim: int = 128
    ffn_dim: int = 12288
    norm_eps: float = 1e-6
    rope_theta: float = 1e6
    max_positions: int = 32768
    dtype: torch.dtype = torch.bfloat16


class PagedKVCache:
    """`num_blocks` blocks of `block_size` token slots; slot s = block * block_size + offset holds one token's
    K (and V) heads: `k_cache[s]` is `[Hk, D]`.  The layout the KV-writing operator scatters into
    (src/impl/rope_rms_impl.h:208-231)."""

    def __init__(self, num_blocks: int, block_size: int, n_kv_heads: int, head_dim: int, dtype, device):
        self.block_size = block_size
        self.num_slots = num_blocks * block_size
        self.k_cache = torch.zeros((self.num_slots, n_kv_heads, head_dim), dtype=dtype, device=device)
        self.v_cache = torch.zeros_like(self.k_cache)

    def slots(self, block_table: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Slot of each (sequence, position): block_table [B, blocks], positions [B, L] -> int64 [B, L]."""
        block = torch.gather(block_table, 1, positions // self.block_size)
        return block * self.block_size + positions % self.block_size


def rope_table(head_dim: int, max_positions: int, theta: float, dtype, device) -> torch.Tensor:
    """[max_positions, head_dim] = cos | sin of position * theta^(-2i/head_dim), computed in fp32
    (model/transformer_model.py:110-116), stored in the activation type."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    ang = torch.outer(torch.arange(max_positions, dtype=torch.float32), inv)
    return torch.cat([ang.cos(), ang.sin()], dim=-1).to(dtype).to(device)


def _rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNorm.forward of the reference (model/transformer_model.py:75-80)."""
    variance = x.float().pow(2).mean(-1, keepdim=True)
    return weight * (x * torch.rsqrt(variance + eps)).to(x.dtype)


class TransformerBlock(nn.Module):
    def __init__(self, args: BlockArgs, device):
        super().__init__()
        a = self.args = args
        kw = dict(bias=False, dtype=a.dtype, device=device)
        self.wqkv = nn.Linear(a.dim, (a.n_heads + 2 * a.n_kv_heads) * a.head_dim, **kw)
        self.wo = nn.Linear(a.n_heads * a.head_dim, a.dim, **kw)
        self.w1 = nn.Linear(a.dim, a.ffn_dim, **kw)
        self.w3 = nn.Linear(a.dim, a.ffn_dim, **kw)
        self.w2 = nn.Linear(a.ffn_dim, a.dim, **kw)
        ones = lambda n: nn.Parameter(torch.ones(n, dtype=a.dtype, device=device))
        self.attention_norm, self.ffn_norm = ones(a.dim), ones(a.dim)
        self.q_norm, self.k_norm = ones(a.head_dim), ones(a.head_dim)
        self.register_buffer("cos_sin", rope_table(a.head_dim, a.max_positions, a.rope_theta, a.dtype, device),
                             persistent=False)

    # ---- the part both paths share: attention over the cache, output projection, feed-forward -------------------
    def _attend(self, q: torch.Tensor, cache: PagedKVCache, context_slots: torch.Tensor,
                attn_mask: torch.Tensor) -> torch.Tensor:
        """q [B, Lq, Hq, D]; context_slots [B, Lk] slots of every cached position of each sequence;
        attn_mask [B, 1, Lq, Lk] bool."""
        a = self.args
        rep = a.n_heads // a.n_kv_heads
        k = cache.k_cache[context_slots].transpose(1, 2).repeat_interleave(rep, dim=1)   # [B, Hq, Lk, D]
        v = cache.v_cache[context_slots].transpose(1, 2).repeat_interleave(rep, dim=1)
        out = F.scaled_dot_product_attention(q.transpose(1, 2), k, v, attn_mask=attn_mask)
        return self.wo(out.transpose(1, 2).reshape(q.shape[0] * q.shape[1], a.n_heads * a.head_dim))

    def _feed_forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.w2(F.silu(self.w1(h)) * self.w3(h))

    # ---- fused path ----------------------------------------------------------------------------------------------
    def forward(self, hidden: torch.Tensor, residual: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                cache: PagedKVCache, context_slots: torch.Tensor, attn_mask: torch.Tensor
                ) -> Tuple[torch.Tensor, torch.Tensor]:
        """hidden, residual [T, dim] (T = B * Lq tokens, sequence-major); positions, slots [T] int64.
        Returns (feed-forward output, residual stream); the next block adds them."""
        a = self.args
        T = hidden.shape[0]
        ops = gpuk_amd.traceable
        residual1, h, unused_scale = torch.empty_like(hidden), torch.empty_like(hidden), hidden.new_empty(1, dtype=torch.float32)
        ops.allreduce_rms(0, hidden, residual, self.attention_norm, residual1, h, unused_scale, a.norm_eps, 0)
        qkv = self.wqkv(h)
        q = torch.empty((T, a.n_heads, a.head_dim), dtype=a.dtype, device=hidden.device)
        ops.fused_rope_rms_set_kv(qkv, self.q_norm, self.k_norm, self.cos_sin, positions, T, a.n_heads, a.n_kv_heads,
                                  a.n_kv_heads, a.head_dim, True, a.norm_eps, q, cache.k_cache, cache.v_cache, slots,
                                  1.0, 1.0)
        B = context_slots.shape[0]
        attn = self._attend(q.view(B, T // B, a.n_heads, a.head_dim), cache, context_slots, attn_mask)
        residual2, h2 = torch.empty_like(hidden), torch.empty_like(hidden)
        ops.allreduce_rms(0, attn, residual1, self.ffn_norm, residual2, h2, unused_scale, a.norm_eps, 0)
        return self._feed_forward(h2), residual2

    # ---- the reference's torch sequence on the same weights ----------------------------------------------------
    def forward_unfused(self, hidden, residual, positions, slots, cache: PagedKVCache, context_slots, attn_mask):
        a = self.args
        T = hidden.shape[0]
        x = hidden + residual
        h = _rms_norm(x, self.attention_norm, a.norm_eps)
        qkv = self.wqkv(h).view(T, a.n_heads + 2 * a.n_kv_heads, a.head_dim)
        xq, xk, xv = qkv.split([a.n_heads, a.n_kv_heads, a.n_kv_heads], dim=1)
        xq, xk = _rms_norm(xq, self.q_norm, a.norm_eps), _rms_norm(xk, self.k_norm, a.norm_eps)
        cos, sin = self.cos_sin[positions].unsqueeze(1).chunk(2, dim=-1)                  # [T, 1, D/2] each

        def rotate(t):   # apply_rotary_emb with rope_interval_split=False (model/transformer_model.py:118-128)
            t1, t2 = torch.chunk(t.float(), 2, dim=-1)
            return torch.cat((t1 * cos - t2 * sin, t2 * cos + t1 * sin), dim=-1).type_as(t)

        xq, xk = rotate(xq), rotate(xk)
        cache.k_cache[slots] = xk
        cache.v_cache[slots] = xv
        B = context_slots.shape[0]
        attn = self._attend(xq.reshape(B, T // B, a.n_heads, a.head_dim), cache, context_slots, attn_mask)
        x = attn + x
        return self._feed_forward(_rms_norm(x, self.ffn_norm, a.norm_eps)), x


def decode_batch(cache: PagedKVCache, block_table: torch.Tensor, context_len: torch.Tensor, new_tokens: int = 1):
    """Index tensors for a step in which each of B sequences appends `new_tokens` tokens to a context that then
    holds `context_len[b]` positions: (positions [B*Lq], slots [B*Lq], context_slots [B, Lk], attn_mask
    [B, 1, Lq, Lk]); Lk = max context, causal inside the new tokens."""
    B = block_table.shape[0]
    dev = block_table.device
    Lk = int(context_len.max().item())
    new_pos = context_len[:, None] - new_tokens + torch.arange(new_tokens, device=dev)[None, :]      # [B, Lq]
    all_pos = torch.arange(Lk, device=dev)[None, :].expand(B, Lk)
    context_slots = cache.slots(block_table, all_pos.clamp(max=block_table.shape[1] * cache.block_size - 1))
    attn_mask = (all_pos[:, None, :] <= new_pos[:, :, None])[:, None]                                # [B,1,Lq,Lk]
    return new_pos.reshape(-1), cache.slots(block_table, new_pos).reshape(-1), context_slots, attn_mask
