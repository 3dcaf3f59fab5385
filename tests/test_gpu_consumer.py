"""GPU: the decoder block that calls the fused operators (gpuk_amd/consumer.py) against the same block driven
through the reference model's torch sequence (model/transformer_model.py:68-156, :235-242) on the same weights.

The two differ where the operators' oracle differs from the model's code: the model rotates in fp32 and rounds
once, the operators round each product to bf16 (test/test_fused_rope_rms.py:16-34).  The comparison therefore uses
the reference tests' own bar (allclose, rtol 1e-2 / atol 5e-2: test/test_fused_rope_rms.py:191-193) on the cache
rows and a relative bar on the block outputs."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def make_block(device, seed=0):
    from gpuk_amd.consumer import BlockArgs, TransformerBlock

    torch.manual_seed(seed)
    args = BlockArgs(dim=512, n_heads=4, n_kv_heads=2, head_dim=128, ffn_dim=1024, max_positions=4096)
    block = TransformerBlock(args, device)
    with torch.no_grad():   # norm weights away from 1 so that a missing or misplaced weight shows
        for w in (block.attention_norm, block.ffn_norm, block.q_norm, block.k_norm):
            w.copy_((1 + 0.2 * torch.randn(w.shape, device=device)).to(w.dtype))
    return args, block


def rel_err(a, b):
    return ((a.float() - b.float()).abs().max() / b.float().abs().max().clamp_min(1e-6)).item()


@torch.no_grad()
def test_prefill_then_decode_matches_unfused_block(device):
    from gpuk_amd.consumer import PagedKVCache, decode_batch

    args, block = make_block(device)
    block_size, blocks_per_seq = 16, 8
    prompt = [37, 64, 5]
    B = len(prompt)
    # each sequence owns a shuffled set of blocks
    perm = torch.randperm(B * blocks_per_seq, generator=torch.Generator().manual_seed(1)).view(B, blocks_per_seq).to(device)
    cache_f = PagedKVCache(B * blocks_per_seq, block_size, args.n_kv_heads, args.head_dim, args.dtype, device)
    cache_u = PagedKVCache(B * blocks_per_seq, block_size, args.n_kv_heads, args.head_dim, args.dtype, device)

    for b, n in enumerate(prompt):                      # prefill, one sequence at a time
        print(f"case consumer prefill seq={b} tokens={n}", flush=True)
        hidden = torch.randn((n, args.dim), device=device).to(args.dtype)
        residual = torch.randn((n, args.dim), device=device).to(args.dtype)
        table = perm[b:b + 1]
        idx = decode_batch(cache_f, table, torch.tensor([n], device=device), new_tokens=n)
        out_f, res_f = block(hidden, residual, *idx[:2], cache_f, *idx[2:])
        out_u, res_u = block.forward_unfused(hidden, residual, *idx[:2], cache_u, *idx[2:])
        assert torch.equal(res_f, res_u.to(res_f.dtype)) or rel_err(res_f, res_u) < 1e-2
        assert rel_err(out_f, out_u) < 3e-2, rel_err(out_f, out_u)
        slots = idx[1]
        assert torch.allclose(cache_f.k_cache[slots].float(), cache_u.k_cache[slots].float(), rtol=1e-2, atol=5e-2)
        assert torch.equal(cache_f.v_cache[slots], cache_u.v_cache[slots])    # V is copied, bit for bit

    # slots no sequence wrote are still zero in both caches
    written = torch.zeros(cache_f.num_slots, dtype=torch.bool, device=device)
    for b, n in enumerate(prompt):
        written[cache_f.slots(perm[b:b + 1], torch.arange(n, device=device)[None])[0]] = True
    assert not cache_f.k_cache[~written].any() and not cache_f.v_cache[~written].any()

    print("case consumer decode step", flush=True)
    context = torch.tensor(prompt, device=device) + 1   # every sequence appends one token
    hidden = torch.randn((B, args.dim), device=device).to(args.dtype)
    residual = torch.randn((B, args.dim), device=device).to(args.dtype)
    idx = decode_batch(cache_f, perm, context)
    out_f, res_f = block(hidden, residual, *idx[:2], cache_f, *idx[2:])
    out_u, res_u = block.forward_unfused(hidden, residual, *idx[:2], cache_u, *idx[2:])
    assert rel_err(res_f, res_u) < 1e-2
    assert rel_err(out_f, out_u) < 3e-2, rel_err(out_f, out_u)
    assert torch.allclose(cache_f.k_cache[idx[1]].float(), cache_u.k_cache[idx[1]].float(), rtol=1e-2, atol=5e-2)


@torch.no_grad()
def test_block_under_graph_replay(device):
    """A decode step of the fused block captured in a HIP graph: replays with new inputs copied into the captured
    buffers match eager calls on the same inputs and cache state."""
    from gpuk_amd.consumer import PagedKVCache, decode_batch

    args, block = make_block(device, seed=3)
    B, block_size, blocks_per_seq = 4, 16, 4
    table = torch.arange(B * blocks_per_seq, device=device).view(B, blocks_per_seq)
    cache_g = PagedKVCache(B * blocks_per_seq, block_size, args.n_kv_heads, args.head_dim, args.dtype, device)
    cache_e = PagedKVCache(B * blocks_per_seq, block_size, args.n_kv_heads, args.head_dim, args.dtype, device)
    context = torch.tensor([9, 17, 1, 30], device=device)
    pos, slots, ctx_slots, mask = decode_batch(cache_g, table, context)
    s_hidden = torch.zeros((B, args.dim), dtype=args.dtype, device=device)
    s_resid = torch.zeros_like(s_hidden)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        block(s_hidden, s_resid, pos, slots, cache_g, ctx_slots, mask)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out, g_res = block(s_hidden, s_resid, pos, slots, cache_g, ctx_slots, mask)
    for rep in range(3):
        hidden = torch.randn((B, args.dim), device=device).to(args.dtype)
        resid = torch.randn((B, args.dim), device=device).to(args.dtype)
        s_hidden.copy_(hidden)
        s_resid.copy_(resid)
        graph.replay()
        torch.cuda.synchronize()
        e_out, e_res = block(hidden, resid, pos, slots, cache_e, ctx_slots, mask)
        torch.cuda.synchronize()
        assert torch.equal(g_res, e_res), rep
        assert torch.equal(cache_g.k_cache[slots], cache_e.k_cache[slots]), rep
        assert rel_err(g_out, e_out) < 1e-3, rep     # the GEMM library may pick another algorithm under capture
