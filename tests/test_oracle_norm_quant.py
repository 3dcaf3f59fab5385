"""Pins the restated add + RMSNorm + FP8 quant oracle (oracle/torch_oracle.py and oracle/gpuk_oracle.c).

No reference file holds vectors for this path, so the checks are the ones the mathematics fixes:
closed forms, invariances, an fp64 brute force on small rows, a discriminator that a single-rounding
implementation fails, and agreement between the two independently written restatements.
"""
import os

import numpy as np
import pytest
import torch

from gpuk_amd import workloads
from oracle import c_oracle, torch_oracle as O
from tests.util import assert_bits_equal, ulp8, ulp16

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def bf(t):
    return torch.from_numpy(t.copy()).view(torch.bfloat16)


def test_residual_add_is_the_correctly_rounded_sum():
    """bf16(x + r) must be the bf16 nearest (ties to even) to the exact sum, which fp64 holds exactly."""
    inp = workloads.norm_quant_inputs(16, 512, seed=3, res_sigma=2.0)
    res, _, _ = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, O.QUANT_NONE)
    exact = inp.x.double() + inp.residual.double()
    ok = res.float().abs() > 1e-30          # bit-pattern neighbours are only taken away from zero
    bits = res.view(torch.int16)
    lo = (bits - 1).view(torch.bfloat16).double()
    hi = (bits + 1).view(torch.bfloat16).double()
    err = (res.double() - exact).abs()
    # the rounded value is at least as close to the exact sum as both of its bf16 neighbours ...
    assert ((err <= (lo - exact).abs()) | ~ok).all() and ((err <= (hi - exact).abs()) | ~ok).all()
    # ... and on an exact tie the even mantissa wins
    tie = ok & ((err == (lo - exact).abs()) | (err == (hi - exact).abs())) & (err > 0)
    assert ((bits[tie] & 1) == 0).all()
    assert ok.float().mean().item() > 0.99


def test_rmsnorm_against_fp64_brute_force():
    inp = workloads.norm_quant_inputs(8, 256, seed=4, res_sigma=1.0)
    res, norm, _ = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, O.QUANT_NONE)
    r64 = res.double()
    want = r64 / torch.sqrt((r64 * r64).mean(-1, keepdim=True) + inp.eps) * inp.gamma.double()
    # two bf16 roundings, each within half an ULP (2^-8 relative at worst): below 2 * 2^-8 plus a hair
    rel = ((norm.double() - want).abs() / want.abs().clamp_min(1e-3)).max().item()
    assert rel < 2 ** -7 * 1.01, rel


def test_rmsnorm_invariances():
    inp = workloads.norm_quant_inputs(8, 1024, seed=5)
    one = torch.ones_like(inp.gamma)
    zero = torch.zeros_like(inp.x)
    # gamma = 1: unit RMS up to bf16 rounding
    n = O.add_rmsnorm_quant_ref(inp.x, zero, one, 0.0, O.QUANT_NONE)[1].double()
    assert ((n * n).mean(-1).sqrt() - 1).abs().max().item() < 4e-3
    # scaling the input by a power of two changes nothing when eps is 0 (exact in binary floating point)
    n4 = O.add_rmsnorm_quant_ref(inp.x * 4, zero, one, 0.0, O.QUANT_NONE)[1]
    assert_bits_equal(n4, O.add_rmsnorm_quant_ref(inp.x, zero, one, 0.0, O.QUANT_NONE)[1], "norm(4x) vs norm(x)")
    # negating the input negates the output
    nn = O.add_rmsnorm_quant_ref(-inp.x, zero, inp.gamma, inp.eps, O.QUANT_NONE)[1]
    assert_bits_equal(nn, -O.add_rmsnorm_quant_ref(inp.x, zero, inp.gamma, inp.eps, O.QUANT_NONE)[1], "norm(-x)")
    # a constant row of value c has rms |c|: the normed value is sign(c) * gamma up to rounding
    c = torch.full((1, 64), 3.0, dtype=torch.bfloat16)
    g = (1 + 0.1 * torch.randn(64, generator=torch.Generator().manual_seed(0))).bfloat16()
    nc = O.add_rmsnorm_quant_ref(c, torch.zeros_like(c), g, 0.0, O.QUANT_NONE)[1]
    assert_bits_equal(nc[0], g, "norm of a constant row equals gamma")


def test_double_rounding_is_what_the_oracle_does():
    """A single-rounding evaluation (fp32 all the way to the fp8 cast, as the reference's own kernel does:
    all_reduce_fusion_impl.h:214-218) must be distinguishable: it changes a visible share of the scales and
    codes, while the op-by-op restatement in C reproduces the torch restatement bit for bit."""
    inp = workloads.norm_quant_inputs(256, 2048, seed=6, res_sigma=2.0, outlier_frac=0.01)
    res, codes, scale = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, O.QUANT_DYNAMIC)
    r = res.float()
    rstd = torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + inp.eps)
    single = r * rstd * inp.gamma.float()
    s1 = single.abs().amax(-1, keepdim=True) / 448.0
    c1 = (single / s1).clamp(-448, 448).to(torch.float8_e4m3fn)
    frac_codes = (ulp8(c1, codes) != 0).float().mean().item()
    rel_scale = ((s1 - scale).abs() / scale).max().item()
    assert frac_codes > 5e-3 and rel_scale > 1e-4, (frac_codes, rel_scale)
    c_res, c_codes, c_scale = c_oracle.add_rmsnorm_quant(inp.x, inp.residual, inp.gamma, inp.eps, 1)
    assert_bits_equal(c_res, res, "C residual")
    assert (c_codes == codes.view(torch.uint8)).all() and (c_scale == scale).all()


@pytest.mark.parametrize("fp8_max,top", [(448.0, 0x7E), (240.0, 0x77)])
def test_dynamic_scale_closed_form(fp8_max, top):
    """scale = amax / fp8_max exactly (fp32 division) and the row's largest element encodes to fp8_max."""
    inp = workloads.norm_quant_inputs(64, 512, seed=7, res_sigma=2.0, outlier_frac=0.02)
    _, n, _ = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, O.QUANT_NONE)
    _, codes, scale = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, O.QUANT_DYNAMIC, fp8_max=fp8_max)
    want = (n.float().abs().amax(-1, keepdim=True).numpy().astype(np.float32) / np.float32(fp8_max))
    assert (scale.numpy() == want).all()
    assert ((codes.view(torch.uint8) & 0x7F).amax(-1) == top).all()
    # dequantised codes stay within half an fp8 step of the normed values
    deq = codes.float() * scale
    assert ((deq - n.float()).abs() <= 0.0625 * n.float().abs() + scale * 2 ** -10 * 1.0001).all()


def test_static_scale_and_clamp():
    inp = workloads.config1()
    st = O.static_scale_for(inp.x, inp.residual, inp.gamma, inp.eps)
    _, codes, _ = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, O.QUANT_STATIC, static_scale=st)
    assert (codes.view(torch.uint8) & 0x7F).max().item() == 0x7E
    # a scale 8 times too small saturates instead of overflowing to NaN
    _, sat, _ = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, O.QUANT_STATIC, static_scale=st / 8)
    assert ((sat.view(torch.uint8) & 0x7F) != 0x7F).all()
    c = c_oracle.add_rmsnorm_quant(inp.x, inp.residual, inp.gamma, inp.eps, 3, static_scale=st / 8)[1]
    assert (c == sat.view(torch.uint8)).all()


def test_zero_rows_follow_the_reference_kernel():
    inp = workloads.norm_quant_inputs(4, 64, seed=8)
    inp.x[2].zero_(); inp.residual[2].zero_()
    for impl in ("torch", "c"):
        if impl == "torch":
            _, codes, scale = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, O.QUANT_DYNAMIC)
            codes = codes.view(torch.uint8)
        else:
            _, codes, scale = c_oracle.add_rmsnorm_quant(inp.x, inp.residual, inp.gamma, inp.eps, 1)
        assert scale[2].item() == 1.0 and (codes[2] == 0).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tokens,hidden", [(1, 8), (7, 520), (64, 4096), (3, 7168)])
def test_c_and_torch_restatements_agree(dtype, tokens, hidden):
    inp = workloads.norm_quant_inputs(tokens, hidden, seed=hidden, res_sigma=2.0, outlier_frac=0.01, dtype=dtype)
    for quant in (0, 1, 3):
        st = O.static_scale_for(inp.x, inp.residual, inp.gamma, inp.eps) if quant == 3 else None
        res, norm, scale = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, quant, static_scale=st)
        c_res, c_norm, c_scale = c_oracle.add_rmsnorm_quant(inp.x, inp.residual, inp.gamma, inp.eps, quant, static_scale=st)
        assert_bits_equal(c_res, res, "residual")
        if quant == 0:
            d = ulp16(c_norm, norm)   # the C sum is accumulated in double: rstd may differ by an fp32 ULP
            assert d.max().item() <= 2 and (d != 0).float().mean().item() < 1e-3
        else:
            d = ulp8(c_norm, norm)
            assert d.max().item() <= 1 and (d != 0).float().mean().item() < 1e-3
            if quant == 1:
                assert ((c_scale - scale).abs() / scale).max().item() < 2 ** -7


def test_small_golden_cases():
    z = np.load(os.path.join(GOLD, "small_cases.npz"))
    for name, quant in (("nq_dynamic", 1), ("nq_none", 0), ("nq_static", 3)):
        x, r, g = bf(z[name + "_x"]), bf(z[name + "_r"]), bf(z[name + "_g"])
        st = O.static_scale_for(x, r, g, 1e-6) if quant == 3 else None
        res, norm, scale = O.add_rmsnorm_quant_ref(x, r, g, 1e-6, quant, static_scale=st)
        assert (res.view(torch.int16).numpy() == z[name + "_res"]).all()
        got = norm.view(torch.int16).numpy() if quant == 0 else norm.view(torch.uint8).numpy()
        assert (got == z[name + "_norm"]).all()
        if quant:
            assert (scale.numpy() == z[name + "_scale"]).all()
        c_res, c_norm, c_scale = c_oracle.add_rmsnorm_quant(x, r, g, 1e-6, quant, static_scale=st)
        assert (c_res.view(torch.int16).numpy() == z[name + "_res"]).all()
        c_got = c_norm.view(torch.int16).numpy() if quant == 0 else c_norm.numpy()
        assert (c_got == z[name + "_norm"]).all()


def test_reciprocal_quotient_model_is_exact():
    """The kernels divide by a per-row scale with one multiply and two fused multiply-adds.  On the guarded
    range (scale in [2^-60, 2^60], quotients that matter for fp8 are >= 2^-10) the result equals the IEEE
    quotient for every bf16 numerator tried and for random fp32 scales."""
    g = torch.Generator().manual_seed(9)
    allbf = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    finite = allbf[torch.isfinite(allbf) & (allbf.abs() < 1e30) & (allbf.abs() > 1e-30)]
    bad = 0
    for _ in range(24):
        s = float(torch.exp(torch.randn((), generator=g) * 4).item())
        b = torch.full_like(finite, s)
        keep = (finite / b).abs() >= 2 ** -12
        bad += c_oracle.count_div_rcp_mismatch(finite[keep].contiguous(), b[keep].contiguous())
    a = torch.randn(2_000_000, generator=g).bfloat16().float() * 8
    b = torch.exp(torch.randn(2_000_000, generator=g) * 3).float()
    keep = (a / b).abs() >= 2 ** -12
    bad += c_oracle.count_div_rcp_mismatch(a[keep].contiguous(), b[keep].contiguous())
    # zeros of either sign, infinities and NaN as numerators: the quotient keeps sign and class
    special = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan")])
    for s in (2.0 ** -60, 0.0123, 1.0, 2.0 ** 60):
        bad += c_oracle.count_div_rcp_mismatch(special, torch.full_like(special, s))
    assert bad == 0


def test_short_sqrt_and_reciprocal_models_are_exact():
    """The kernels take sqrt and 1/x by v_sqrt_f32 / v_rcp_f32 (1 ULP) plus correction steps instead of the compiler's
    general expansions.  The same sequences in C, started from every value within one ULP of the true result, give
    the correctly rounded result for every mantissa (square root: both exponent parities), except the reciprocal of a
    number whose mantissa bits are all ones, which the kernels send to the general division."""
    import struct

    bits = lambda f: struct.unpack("<I", struct.pack("<f", f))[0]
    for first_guess in (-1, 0, 1):
        for lo in (1.0, 2.0, 2.0 ** -41, 2.0 ** 58):
            assert c_oracle.count_short_sqrt_mismatch(bits(lo), 1 << 23, first_guess) == 0, (lo, first_guess)
        for lo in (1.0, 2.0 ** -30, 2.0 ** 29):
            bad = c_oracle.count_short_rcp_mismatch(bits(lo), (1 << 23) - 1, first_guess)   # all but the all-ones mantissa
            assert bad == 0, (lo, first_guess, bad)
    assert c_oracle.count_short_rcp_mismatch(bits(1.0) + (1 << 23) - 1, 1, 1) == 1   # the excluded case does fail


def test_quotients_by_row_length_and_by_fp8_max_are_exact():
    """mean = sum / H and scale = amax / fp8_max are taken as one multiply and two fused multiply-adds with the
    reciprocal rounded on the host: equal to the IEEE quotient for every row length that is a multiple of 8 up to
    65536 (random sums on the guarded range) and for every positive bf16 amax on that range with 448 and 240."""
    g = torch.Generator().manual_seed(21)
    hs = torch.arange(8, 65536 + 8, 8, dtype=torch.float32)
    bad = 0
    for _ in range(40):
        sums = torch.exp2(torch.rand(hs.numel(), generator=g) * 100 - 50).float()
        bad += c_oracle.count_div_rcp_mismatch(sums.contiguous(), hs.contiguous())
    for h in (7168.0, 5120.0, 12288.0, 1032.0, 65528.0):
        sums = torch.exp2(torch.rand(1_000_000, generator=g) * 119 - 59.5).float()
        bad += c_oracle.count_div_rcp_mismatch(sums, torch.full_like(sums, h))
    allbf = torch.arange(1, 0x7F80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    amax = allbf[(allbf >= 2.0 ** -60) & (allbf < 2.0 ** 60)]
    for fp8_max in (448.0, 240.0):
        bad += c_oracle.count_div_rcp_mismatch(amax.contiguous(), torch.full_like(amax, fp8_max))
    assert bad == 0
