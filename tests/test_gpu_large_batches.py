"""Batches whose tensors pass 2^31 elements / 2^32 bytes: the index arithmetic of both kernels at sizes no other test
reaches.  The inputs are made on the GPU; the oracle, which works a token (or row) at a time, is run on windows of the
batch -- its first rows, the rows around the 2^31-element / 2^32-byte mark, its last rows -- and the whole batch is held
to what the rows do not depend on: the rope kernel gives the same bits when the batch is cut into eight calls, whose
index arithmetic stays small; no cache slot outside the named ones changes.
"""
import pytest
import torch

from gpuk_amd import workloads
from oracle import torch_oracle as O
from tests.test_gpu_norm_quant import check as check_norm_quant
from tests.util import assert_bits_equal, assert_heads_explained

pytestmark = pytest.mark.gpu


def windows(n, mark, width=96):
    half = width // 2
    return [range(0, width), range(mark - half, mark + half), range(n - width, n)]


def test_rope_set_kv_past_4_gib(device):
    from gpuk_amd import capi

    T, hq, hk, hv, D = 360_000, 32, 8, 8, 128       # qkv: 4.42 GB, its 2^32nd byte inside token 349,525
    slots, max_pos = 400_000, 4096
    print(f"case large rope T={T}", flush=True)
    g = torch.Generator(device=device).manual_seed(5)
    qkv = torch.randn((T, hq + hk + hv, D), device=device, generator=g, dtype=torch.float32).to(torch.bfloat16)
    qw = (1 + 0.1 * torch.randn(D, device=device, generator=g)).to(torch.bfloat16)
    kw = (1 + 0.1 * torch.randn(D, device=device, generator=g)).to(torch.bfloat16)
    cos_sin = torch.randn((max_pos, D), device=device, generator=g).to(torch.bfloat16)
    positions = torch.randint(0, max_pos, (T,), device=device, generator=g, dtype=torch.int64)
    kv_loc = torch.randperm(slots, device=device, generator=g)[:T].contiguous()
    k0 = torch.randint(-30000, 30000, (slots, hk, D), device=device, generator=g, dtype=torch.int16).view(torch.bfloat16)
    v0 = torch.randint(-30000, 30000, (slots, hv, D), device=device, generator=g, dtype=torch.int16).view(torch.bfloat16)

    qa = torch.empty((T, hq, D), dtype=torch.bfloat16, device=device)
    ka, va = k0.clone(), v0.clone()
    capi.rope_rms_set_kv(qkv, qw, kw, cos_sin, positions, T, hq, hk, hv, D, True, 1e-6, qa, ka, va, kv_loc, 1.0, 1.0,
                         None, False)
    torch.cuda.synchronize()
    # the same batch in eight calls of 45,000 tokens: every call's offsets stay far below 2^31
    qb = torch.empty_like(qa)
    kb, vb = k0.clone(), v0.clone()
    step = T // 8
    for lo in range(0, T, step):
        hi = lo + step
        capi.rope_rms_set_kv(qkv[lo:hi], qw, kw, cos_sin, positions[lo:hi], step, hq, hk, hv, D, True, 1e-6, qb[lo:hi],
                             kb, vb, kv_loc[lo:hi], 1.0, 1.0, None, False)
    torch.cuda.synchronize()
    assert torch.equal(qa.view(torch.int16), qb.view(torch.int16)), "q_out: one call and eight calls differ"
    assert torch.equal(ka.view(torch.int16), kb.view(torch.int16)), "k_cache: one call and eight calls differ"
    assert torch.equal(va.view(torch.int16), vb.view(torch.int16)), "v_cache: one call and eight calls differ"
    # V rows are copies; slots no token names keep their content
    assert torch.equal(va[kv_loc].view(torch.int16), qkv[:, hq + hk:].view(torch.int16))
    untouched = torch.ones(slots, dtype=torch.bool, device=device)
    untouched[kv_loc] = False
    assert torch.equal(ka[untouched].view(torch.int16), k0[untouched].view(torch.int16))
    assert torch.equal(va[untouched].view(torch.int16), v0[untouched].view(torch.int16))

    mark = (1 << 32) // (2 * (hq + hk + hv) * D)   # the token that holds qkv's 2^32nd byte
    for w in windows(T, mark):
        idx = torch.tensor(list(w), device=device)
        n = len(w)
        small = workloads.RopeInputs(qkv[idx].cpu(), qw.cpu(), kw.cpu(), cos_sin.cpu(), positions[idx].cpu(),
                                     torch.arange(n), n, hq, hk, hv, D, n)
        q_ref = torch.empty((n, hq, D), dtype=torch.bfloat16)
        k_ref = torch.zeros((n, hk, D), dtype=torch.bfloat16)
        v_ref = torch.zeros((n, hv, D), dtype=torch.bfloat16)

        def want(off):
            q, k, v = q_ref.clone(), k_ref.clone(), v_ref.clone()
            O.rope_rms_set_kv_ref(small.qkv, small.qw, small.kw, small.cos_sin, small.positions, n, hq, hk, hv, D, True,
                                  1e-6, q, k, v, small.kv_loc, 1.0, 1.0, None, False, rstd_ulp_offset=off)
            return q, k

        cache = {}
        at = lambda off, i: cache.setdefault(off, want(off))[i]
        assert_heads_explained(qa[idx].cpu(), lambda off: at(off, 0), f"[large rope, tokens {w.start}..] q_out", D)
        assert_heads_explained(ka[kv_loc[idx]].cpu(), lambda off: at(off, 1), f"[large rope, tokens {w.start}..] k rows", D)


def test_norm_quant_past_2_31_elements(device):
    from gpuk_amd import capi

    T, H = 270_000, 8192          # 2.21e9 elements per tensor; element 2^31 opens row 262,144
    print(f"case large norm-quant {T}x{H}", flush=True)
    g = torch.Generator(device=device).manual_seed(6)
    x = torch.empty((T, H), dtype=torch.bfloat16, device=device)
    r = torch.empty((T, H), dtype=torch.bfloat16, device=device)
    step = 30_000                 # filled in slices: the fp32 draws of the whole batch would take 9 GB each
    for lo in range(0, T, step):
        hi = min(T, lo + step)
        x[lo:hi] = torch.randn((hi - lo, H), device=device, generator=g)
        r[lo:hi] = 2.0 * torch.randn((hi - lo, H), device=device, generator=g)
    gamma = (1 + 0.1 * torch.randn(H, device=device, generator=g)).to(torch.bfloat16)
    res = torch.empty_like(x)
    codes = torch.empty((T, H), dtype=torch.float8_e4m3fn, device=device)
    scale = torch.full((T, 1), -1.0, dtype=torch.float32, device=device)
    capi.add_rmsnorm_quant(x, r, gamma, res, codes, scale, 1e-6, 1)
    torch.cuda.synchronize()
    assert (scale > 0).all(), "a row was not written"
    for w in windows(T, (1 << 31) // H):
        rows = slice(w.start, w.stop)
        small = workloads.NormQuantInputs(x[rows].cpu(), r[rows].cpu(), gamma.cpu())
        check_norm_quant(small, 1, (res[rows], codes[rows], scale[rows]), tag=f"[large norm-quant, rows {w.start}..]")
    # the residual of the whole batch, on the GPU: one bf16 add
    assert torch.equal(res.view(torch.int16), (x + r).view(torch.int16))
