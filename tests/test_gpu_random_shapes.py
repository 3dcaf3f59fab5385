"""GPU parity on seeded random shapes: token counts, row lengths, head mixes and head sizes drawn at random (fixed
seeds), so that ragged sizes nobody thought of listing are exercised: rows that do not fill the last wave, token counts
around the workgroup-to-row remapping thresholds, head counts that leave waves partly filled, V rows longer or
shorter than the Q/K waves cover.  Each case is checked like the listed cases of the other GPU test files."""
import random

import pytest
import torch

from gpuk_amd import workloads
from oracle import torch_oracle as O
from tests.test_gpu_norm_quant import check as check_norm_quant, run_capi as run_norm_quant
from tests.test_gpu_rope import check_inplace, check_set_kv, run_inplace, run_set_kv

pytestmark = pytest.mark.gpu


def norm_quant_cases(n=36):
    rng = random.Random(2024)
    cases = []
    for i in range(n):
        hidden = 8 * rng.choice([1, 2, 3, 7, 16, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 640, 896, 1000,
                                 1023, 1024, 1025, 2047, 2048, 2049, 4096, 4100, 8191])
        budget = 3_000_000 // hidden
        tokens = rng.choice([1, 2, 3, 17, 255, 256, 257, 1023, 1024, 1025, 1100, 1536, 2047, 2049, 3000])
        cases.append((min(tokens, max(1, budget)), hidden, rng.choice([0, 1, 3]), rng.choice([torch.bfloat16, torch.float16])))
    return cases


@pytest.mark.parametrize("tokens,hidden,quant,dtype", norm_quant_cases())
def test_norm_quant_random_shapes(device, tokens, hidden, quant, dtype):
    print(f"case random norm-quant tokens={tokens} hidden={hidden} quant={quant} dtype={dtype}", flush=True)
    inp = workloads.norm_quant_inputs(tokens, hidden, seed=tokens * 31 + hidden, res_sigma=1.5, outlier_frac=0.01, dtype=dtype)
    static = O.static_scale_for(inp.x, inp.residual, inp.gamma, inp.eps) if quant == 3 else None
    check_norm_quant(inp, quant, run_norm_quant(inp, quant, device, static_scale=static), static_scale=static,
                     tag=f"[{tokens}x{hidden} q{quant}]")


def norm_quant_round_cases(n=14):
    """Batches of a fifth of a round of workgroups to two and a half: the store gate, four chunks per lane, two
    launches per call and plain several-round launches, whichever the launcher's rules pick."""
    rng = random.Random(4242)
    cases = []
    for i in range(n):
        hidden = 8 * rng.choice([128, 256, 320, 384, 512, 640, 768, 896, 1024, 1280, 2048])
        waves4 = -(-(hidden // 8) // 4 // 64)                # waves per row at four chunks per lane
        round_rows = 256 * (32 // waves4)
        tokens = max(1, min(int(round_rows * rng.uniform(0.2, 2.5)), 20_000_000 // hidden))
        cases.append((tokens, hidden, rng.choice([0, 1, 3]), rng.choice([torch.bfloat16, torch.float16])))
    return cases


@pytest.mark.parametrize("tokens,hidden,quant,dtype", norm_quant_round_cases())
def test_norm_quant_random_batches_around_a_round(device, tokens, hidden, quant, dtype):
    from gpuk_amd import capi

    print(f"case random norm-quant around a round tokens={tokens} hidden={hidden} quant={quant} dtype={dtype} "
          f"shape={capi.add_rmsnorm_quant_launch_shape(tokens, hidden, dtype)}", flush=True)
    inp = workloads.norm_quant_inputs(tokens, hidden, seed=tokens * 13 + hidden, res_sigma=1.5, outlier_frac=0.01, dtype=dtype)
    static = O.static_scale_for(inp.x, inp.residual, inp.gamma, inp.eps) if quant == 3 else None
    check_norm_quant(inp, quant, run_norm_quant(inp, quant, device, static_scale=static), static_scale=static,
                     tag=f"[{tokens}x{hidden} q{quant}]")


def rope_cases(n=36):
    rng = random.Random(77)
    cases = []
    for i in range(n):
        head_size = rng.choice([64, 128, 256])
        hq, hk, hv = rng.randint(1, 20), rng.randint(1, 9), rng.randint(0, 24)
        tokens = rng.choice([1, 2, 5, 31, 64, 100, 257, 400])
        mrope = rng.random() < 0.5
        cases.append((tokens, hq, hk, hv, head_size, rng.random() < 0.5, mrope, mrope and rng.random() < 0.5,
                      rng.random() < 0.5))
    return cases


@pytest.mark.parametrize("tokens,hq,hk,hv,head_size,neox,mrope,interleaved,fp8", rope_cases())
def test_rope_random_shapes(device, tokens, hq, hk, hv, head_size, neox, mrope, interleaved, fp8):
    from tests.test_gpu_rope import make

    print(f"case random rope T={tokens} heads={hq},{hk},{hv} D={head_size} neox={neox} mrope={mrope} il={interleaved} "
          f"fp8={fp8}", flush=True)
    inp = make(tokens, hq, head_size, neox, seed=tokens + 100 * hq + hk, mrope=mrope, interleaved=interleaved, fp8=fp8,
               hk=hk, hv=hv)
    check_set_kv(inp, run_set_kv(inp, device), f"[random set_kv {tokens} {hq},{hk},{hv} D={head_size}]")
    check_inplace(inp, run_inplace(inp, device), "in place")
