"""Comparison helpers shared by the parity tests: distances in units in the last place for 16-bit
floats and fp8 codes, and the acceptance bars the benchmark definition states."""
from __future__ import annotations

import torch

# Acceptance bars: normed 16-bit outputs within 1 ULP; fp8 codes bit-exact for >= 99.9 % of elements and
# at most 1 fp8 ULP otherwise; per-token scales within 1e-6 relative; untouched cache slots bit-exact.
MIN_EXACT_FRACTION = 0.999
SCALE_RTOL = 1e-6


def ordered16(t: torch.Tensor) -> torch.Tensor:
    """Map bf16/fp16 bit patterns to integers whose order is the numeric order (-0 == +0)."""
    b = t.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
    mag = b & 0x7FFF
    return torch.where((b & 0x8000) != 0, -mag, mag)


def ulp16(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return (ordered16(a.cpu()) - ordered16(b.cpu())).abs()


def ordered8(t: torch.Tensor) -> torch.Tensor:
    b = t.contiguous().view(torch.uint8).to(torch.int32)
    mag = b & 0x7F
    return torch.where((b & 0x80) != 0, -mag, mag)


def ulp8(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return (ordered8(a.cpu()) - ordered8(b.cpu())).abs()


def assert_bits_equal(a: torch.Tensor, b: torch.Tensor, what: str):
    a, b = a.cpu().contiguous(), b.cpu().contiguous()
    assert a.shape == b.shape and a.dtype == b.dtype, (what, a.shape, b.shape, a.dtype, b.dtype)
    va = a.view(torch.uint8) if a.element_size() == 1 else a.view(torch.int16)
    vb = b.view(torch.uint8) if b.element_size() == 1 else b.view(torch.int16)
    bad = (va != vb).sum().item()
    assert bad == 0, f"{what}: {bad} of {va.numel()} elements differ bitwise"


def assert_close_ulp16(got, want, what: str, max_ulp: int = 1, min_exact: float = MIN_EXACT_FRACTION,
                       rare_ulp: int = 2, rare_fraction: float = 1e-4):
    """Normed 16-bit outputs: bit-exact for >= min_exact of the elements and within `max_ulp` ULP, except
    that at most `rare_fraction` of them may sit `rare_ulp` ULP away.  The exception exists because the
    oracle rounds twice (rT(x*rstd), then rT(gamma*.)): when the fp32 sum of squares is accumulated in a
    different order, rstd can move by one fp32 ULP, which flips about 2^-16 of the first roundings, and the
    second rounding turns such a 1-ULP step into 2 ULP whenever gamma*n lands in a lower binade.
    tests/test_gpu_norm_quant.py::test_rows_explained_by_rstd_ulp shows every such row is bit-exact for a
    neighbouring rstd."""
    d = ulp16(got, want)
    n = d.numel()
    if n == 0:
        return
    exact = (d == 0).sum().item() / n
    worst = d.max().item()
    beyond = (d > max_ulp).sum().item()
    assert worst <= rare_ulp, f"{what}: worst distance {worst} ULP (> {rare_ulp}); exact fraction {exact:.6f}"
    assert beyond <= max(1, int(rare_fraction * n)), f"{what}: {beyond} of {n} elements beyond {max_ulp} ULP"
    assert exact >= min_exact, f"{what}: only {exact:.6f} of elements bit-exact (< {min_exact})"


def assert_codes_close(got, want, what: str, min_exact: float = MIN_EXACT_FRACTION):
    n = got.numel()
    if n == 0:
        return
    # NaN codes (0x7f / 0xff) must sit in the same places: next to 0x7e they would otherwise count as one step
    g8, w8 = got.cpu().contiguous().view(torch.uint8), want.cpu().contiguous().view(torch.uint8)
    g_nan, w_nan = (g8 & 0x7F) == 0x7F, (w8 & 0x7F) == 0x7F
    assert torch.equal(g_nan, w_nan), f"{what}: NaN codes in different places ({int(g_nan.sum())} vs {int(w_nan.sum())})"
    d = ulp8(got, want)
    exact = (d == 0).sum().item() / n
    worst = d.max().item()
    assert worst <= 1, f"{what}: worst fp8 distance {worst} ULP; exact fraction {exact:.6f}"
    assert exact >= min_exact, f"{what}: only {exact:.6f} of fp8 codes bit-exact (< {min_exact})"


def assert_scales_close(got, want, what: str, rtol: float = SCALE_RTOL):
    got, want = got.detach().cpu().double().flatten(), want.detach().cpu().double().flatten()
    rel = ((got - want).abs() / want.abs().clamp_min(1e-30)).max().item() if got.numel() else 0.0
    assert rel <= rtol, f"{what}: worst relative scale error {rel:.3e} (> {rtol})"


def _raw(t: torch.Tensor) -> torch.Tensor:
    t = t.cpu().contiguous()
    return t.view(torch.uint8) if t.element_size() == 1 else t.view(torch.int16)


def assert_heads_explained(got, want_at, what: str, head_size: int, min_exact: float = MIN_EXACT_FRACTION,
                           offsets=(0, -1, 1, -2, 2)):
    """Rotation outputs (16-bit values or fp8 codes), head by head, with no tolerance: every head of `got` must be
    bit-identical to the oracle evaluated with that head's rstd at most two fp32 ULPs away (`want_at(offset)` returns
    the oracle's output with every rstd moved by `offset` ULPs; at most one head in a thousand may need the second
    ULP), and at least `min_exact` of all elements must be bit-identical to the unmoved oracle.  The order in which
    the squares of a head are summed is the one thing the kernels do not reproduce; it moves the fp32 sum by an ULP
    or two and rstd with it, which flips about 2^-16 of the first roundings.  Prints what was found.  Returns
    (heads, heads identical at offset 0, worst 16-bit ULP distance from the unmoved oracle)."""
    g = _raw(got).reshape(-1, head_size)
    n_heads = g.shape[0]
    if n_heads == 0:
        return 0, 0, 0
    ok = torch.zeros(n_heads, dtype=torch.bool)
    at0 = exact_elems = worst = None
    within1 = 0
    for off in offsets:
        want = want_at(off)
        w = _raw(want).reshape(-1, head_size)
        assert w.shape == g.shape, (what, tuple(got.shape), tuple(want.shape))
        eq = g == w
        if off == 0:
            at0 = int(eq.all(dim=1).sum())
            exact_elems = eq.float().mean().item()
            worst = int((ulp16(got, want) if got.element_size() == 2 else ulp8(got, want)).max())
        ok |= eq.all(dim=1)
        if abs(off) <= 1:
            within1 = int(ok.sum())
        if bool(ok.all()):
            break
    explained = int(ok.sum())
    print(f"{what}: {n_heads} heads, {at0} bit-identical to the oracle, {within1 - at0} more at rstd -/+ 1 ULP, "
          f"{explained - within1} at -/+ 2 ULP, {n_heads - explained} unexplained; elements identical to the unmoved oracle "
          f"{exact_elems:.6f}, worst distance from it {worst} ULP", flush=True)
    assert explained == n_heads, f"{what}: {n_heads - explained} of {n_heads} heads match the oracle at no rstd within 2 ULP"
    assert explained - within1 <= max(1, n_heads // 1000), f"{what}: {explained - within1} of {n_heads} heads need rstd 2 ULP away"
    assert exact_elems >= min_exact, f"{what}: only {exact_elems:.6f} of elements bit-exact (< {min_exact})"
    return n_heads, at0, worst


def assert_rotated_close(got, want, what: str, min_exact: float = MIN_EXACT_FRACTION, atol: float = 0.05, rtol: float = 1e-2):
    """For comparisons where the oracle cannot be re-evaluated at a neighbouring rstd (one CPU restatement against
    the other, the smoke check): at least `min_exact` of all elements bit-identical, the rest within the reference
    tests' allclose bar (rtol 1e-2, atol 0.05: test/test_fused_rope_rms.py:191-193).  The GPU parity tests use
    assert_heads_explained, which has no tolerance."""
    g, w = got.cpu(), want.cpu()
    d = ulp16(g, w)
    n = d.numel()
    if n == 0:
        return
    exact = (d == 0).sum().item() / n
    assert exact >= min_exact, f"{what}: only {exact:.6f} of elements bit-exact (< {min_exact})"
    gf, wf = g.float(), w.float()
    bad = ((gf - wf).abs() > atol + rtol * wf.abs()).sum().item()
    assert bad == 0, f"{what}: {bad} elements outside rtol={rtol}, atol={atol}"
