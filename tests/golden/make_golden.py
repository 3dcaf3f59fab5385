#!/usr/bin/env python3
"""Writes the fixtures under tests/golden/ (run from the repository root: python tests/golden/make_golden.py).

The reference repository holds no golden vectors for these paths (its tests compare against a torch
reference computed on the spot), so the fixtures are produced here from torch-CPU library routines and
from this repository's restatement of the reference's torch code:

  e4m3fn_from_bf16.bin   65536 bytes: torch's own float8_e4m3fn cast of every bf16 bit pattern
                         (a library routine, independent of any code in this repository)
  bf16_round_cases.npz   fp32 bit patterns around rounding boundaries with torch's bf16/fp16 casts
  small_cases.npz        tiny seeded inputs with the outputs of oracle/torch_oracle.py under the torch
                         build named in small_cases.meta.json; they freeze the restated oracle so that a
                         later edit of it, or a different torch build, shows up as a diff

No file of the reference repository is imported, read or executed.
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from gpuk_amd import workloads  # noqa: E402
from oracle import torch_oracle as O  # noqa: E402


def bits16(t):
    return t.contiguous().view(torch.int16).numpy().copy()


def main():
    # every bf16 pattern through torch's e4m3fn cast
    allbf = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    table = allbf.float().to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    table.tofile(os.path.join(HERE, "e4m3fn_from_bf16.bin"))

    # fp32 patterns: ties and their neighbours for bf16, plus a seeded random sample
    g = torch.Generator().manual_seed(0)
    hi = torch.randint(0, 1 << 16, (4096,), generator=g, dtype=torch.int64)
    lows = torch.tensor([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=torch.int64)
    pats = ((hi[:, None] << 16) | lows[None, :]).flatten()
    rnd = torch.randint(0, 1 << 32, (8192,), generator=g, dtype=torch.int64)
    pats = torch.cat([pats, rnd])
    pats = torch.where(pats >= (1 << 31), pats - (1 << 32), pats).to(torch.int32)
    f = pats.view(torch.float32)
    keep = ~torch.isnan(f)
    pats, f = pats[keep], f[keep]
    np.savez_compressed(os.path.join(HERE, "bf16_round_cases.npz"), fp32_bits=pats.numpy(),
                        bf16_bits=bits16(f.to(torch.bfloat16)), fp16_bits=bits16(f.to(torch.float16)))

    out = {}
    # add + RMSNorm + quant: three tiny cases
    for name, (T, H, quant) in {"nq_dynamic": (5, 64, 1), "nq_none": (3, 40, 0), "nq_static": (4, 128, 3)}.items():
        inp = workloads.norm_quant_inputs(T, H, seed=7, res_sigma=2.0, outlier_frac=0.05)
        st = O.static_scale_for(inp.x, inp.residual, inp.gamma, inp.eps) if quant == 3 else None
        res, norm, scale = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, quant, static_scale=st)
        out[name + "_x"], out[name + "_r"], out[name + "_g"] = bits16(inp.x), bits16(inp.residual), bits16(inp.gamma)
        out[name + "_res"] = bits16(res)
        out[name + "_norm"] = bits16(norm) if quant == 0 else norm.view(torch.uint8).numpy().copy()
        if scale is not None:
            out[name + "_scale"] = scale.numpy().copy()
    # rope: NeoX + chunked mRoPE + fp8 cache, GPT-J + interleaved + bf16 cache
    for name, (neox, il, fp8) in {"rope_a": (True, False, True), "rope_b": (False, True, False)}.items():
        r = workloads.rope_inputs(6, 3, 2, 2, 64, seed=11, max_pos=64, num_slots=16, is_neox=neox, random_table=True,
                                  kv_dtype=torch.float8_e4m3fn if fp8 else torch.bfloat16,
                                  k_scale=1.5 if fp8 else 1.0, v_scale=2.0 if fp8 else 1.0)
        r.positions = torch.randint(0, 64, (3, 6), generator=torch.Generator().manual_seed(12), dtype=torch.int64)
        sec = [12, 10, 10]
        k, v = r.new_cache()
        q = torch.empty((6, 3, 64), dtype=torch.bfloat16)
        out[name + "_k0"], out[name + "_v0"] = k.view(torch.uint8).numpy().copy(), v.view(torch.uint8).numpy().copy()
        O.rope_rms_set_kv_ref(r.qkv, r.qw, r.kw, r.cos_sin, r.positions, 6, 3, 2, 2, 64, neox, r.eps, q, k, v, r.kv_loc,
                              r.k_scale, r.v_scale, sec, il)
        for key, t in (("qkv", r.qkv), ("qw", r.qw), ("kw", r.kw), ("cos_sin", r.cos_sin), ("q", q)):
            out[name + "_" + key] = bits16(t)
        out[name + "_pos"], out[name + "_loc"] = r.positions.numpy().copy(), r.kv_loc.numpy().copy()
        out[name + "_k"], out[name + "_v"] = k.view(torch.uint8).numpy().copy(), v.view(torch.uint8).numpy().copy()
    np.savez_compressed(os.path.join(HERE, "small_cases.npz"), **out)
    with open(os.path.join(HERE, "small_cases.meta.json"), "w") as fh:
        json.dump({"torch": torch.__version__, "numpy": np.__version__}, fh)
    print("wrote fixtures to", HERE)


if __name__ == "__main__":
    main()
