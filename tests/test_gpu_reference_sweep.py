"""The rest of the reference's own test sweeps, at their sizes.

test/test_fused_rope_rms.py:196-217 and test/test_fused_mrope_rms_set_kv.py:274-307 run token counts
513 / 1257 / 127 / 778 / 10024 / 3 with 32 and 64 heads of each kind (q = k = v), head sizes 64 / 128 / 256, NeoX and
GPT-J style, chunked and interleaved sections, a random table, an fp8 cache with k_scale 1.5 / v_scale 2.0.
tests/test_gpu_rope.py covers 513 / 127 / 3 with 32 heads; this file covers 1257 / 778 / 10024 with 64 heads, with
distinct cache slots so that the result is deterministic.

test/test_all_reduce_fusion.py:166-212 runs the norm-quant op with fp8 output on tokens x hidden = 1 x 4096 (bf16),
{128, 129} x 1024 (fp32, fp16, bf16) and 32768 x 4096 (bf16), inputs uniform in (-1, 1), weights uniform in
(-2/hidden, 2/hidden), five samples each (:138-148).  One GPU here: the all-reduce input is one tensor.
"""
import pytest
import torch

from oracle import torch_oracle as O
from tests.test_gpu_rope import check_inplace, check_set_kv, make, run_inplace, run_set_kv
from tests.util import assert_bits_equal, assert_codes_close, assert_scales_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("head_size", [64, 128, 256])
@pytest.mark.parametrize("tokens", [1257, 778, 10024])
def test_rope_sweep_64_heads(device, tokens, head_size):
    """Every variant the reference scripts run on one input: plain RoPE in place, mRoPE in place, mRoPE with the
    cache write (fp8 cache), each NeoX and GPT-J, the mRoPE ones chunked and interleaved."""
    import copy

    base = make(tokens, 64, head_size, True, seed=tokens + head_size, mrope=True, fp8=True)
    positions3 = base.positions
    for neox in (True, False):
        print(f"case reference sweep T={tokens} D={head_size} neox={neox}", flush=True)
        inp = copy.copy(base)
        inp.is_neox = neox
        inp.positions, inp.mrope_section = positions3[0].contiguous(), None
        check_inplace(inp, run_inplace(inp, device), f"[rope T={tokens} D={head_size} neox={neox}]")
        for interleaved in (True, False):
            inp = copy.copy(base)
            inp.is_neox, inp.is_interleaved = neox, interleaved
            if tokens < 10000 or interleaved:   # the largest size: one of the two in place, both with the cache
                check_inplace(inp, run_inplace(inp, device), f"[mrope T={tokens} D={head_size} neox={neox} il={interleaved}]")
            check_set_kv(inp, run_set_kv(inp, device), f"[set_kv T={tokens} D={head_size} neox={neox} il={interleaved}]")


def uniform_inputs(tokens, hidden, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.rand((tokens, hidden), generator=g) * 2 - 1).to(dtype)
    r = (torch.rand((tokens, hidden), generator=g) * 2 - 1).to(dtype)
    w = ((torch.rand((hidden,), generator=g) * 2 - 1) * (2.0 / hidden)).to(dtype)
    return x, r, w


@pytest.mark.parametrize("tokens,hidden,dtype", [(1, 4096, torch.bfloat16),
                                                 (129, 1024, torch.float32), (129, 1024, torch.bfloat16), (129, 1024, torch.float16),
                                                 (128, 1024, torch.float32), (128, 1024, torch.float16), (128, 1024, torch.bfloat16),
                                                 (32768, 4096, torch.bfloat16)])
def test_norm_quant_sweep(device, tokens, hidden, dtype):
    import gpuk_amd as gpuk

    env = gpuk.GPUKDistEnv(device_id=0)
    for sample in range(5 if tokens < 30000 else 2):
        print(f"case reference norm-quant {tokens}x{hidden} {dtype} sample {sample}", flush=True)
        x, r, w = uniform_inputs(tokens, hidden, dtype, seed=1000 * sample + tokens + hidden)
        res, codes, scale = env.allreduce_add_rms_fused(x.to(device), r.to(device), w.to(device), 1e-6, True)
        torch.cuda.synchronize()
        res_ref, codes_ref, scale_ref = O.add_rmsnorm_quant_ref(x, r, w, 1e-6, O.QUANT_DYNAMIC)
        tag = f"[{tokens}x{hidden} {dtype} #{sample}]"
        assert_bits_equal(res.cpu().view(torch.uint8), res_ref.view(torch.uint8), f"{tag} residual_out")
        assert_scales_close(scale, scale_ref, f"{tag} scale_out")
        assert_codes_close(codes, codes_ref, f"{tag} codes")
        # the reference's own bar on the dequantised values (rtol = atol = 1e-2)
        got, want = codes.cpu().float() * scale.cpu(), codes_ref.float() * scale_ref
        assert torch.allclose(got, want, rtol=1e-2, atol=1e-2), f"{tag} dequantised norm_out"
