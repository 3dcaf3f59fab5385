"""How far the kernels' outputs sit from the *unmoved* oracle, element by element, at the benchmark configurations'
full sizes -- the figures behind the parity table of the design notes.  The benchmark definition's bars are stated
per element (normed 16-bit outputs within 1 ULP, fp8 codes bit-exact for >= 99.9 % and within 1 fp8 ULP, scales within
1e-6); the other GPU tests hold every row / head bit-identical to the oracle at an rstd a few fp32 ULPs away, which is
stricter but is not the bar as written.  Here both views meet: the histogram of distances is printed (`pytest -s`),
every element that is not bit-identical must lie in a row / head that needed a moved rstd, and the counts beyond 1 ULP
are bounded by twice what was measured when these bounds were written."""
import pytest
import torch

from gpuk_amd import workloads
from oracle import torch_oracle as O
from tests.test_gpu_norm_quant import run_capi
from tests.test_gpu_rope import oracle_set_kv, run_set_kv
from tests.util import ulp16, ulp8

pytestmark = pytest.mark.gpu


def histogram(d):
    n = d.numel()
    return n, int((d == 0).sum()), int((d == 1).sum()), int((d == 2).sum()), int((d > 2).sum()), int(d.max()) if n else 0


def report(name, d, groups_off, group_len):
    """d: distances [groups, group_len] (rows or heads); groups_off: groups not bit-identical to the unmoved oracle."""
    n, d0, d1, d2, dmore, worst = histogram(d)
    print(f"[ULP] {name}: {n} elements; 0 ULP {d0} ({d0 / max(n, 1):.7f}), 1 ULP {d1}, 2 ULP {d2}, more {dmore}, worst {worst}; "
          f"{int(groups_off.sum())} of {groups_off.numel()} rows/heads differ from the unmoved oracle", flush=True)
    # an element off the unmoved oracle lies in a row / head that is not bit-identical to it (which the parity tests
    # show to be bit-identical to the oracle at a neighbouring rstd)
    stray = (d.reshape(-1, group_len) != 0).any(dim=1) & ~groups_off
    assert not stray.any()
    return d2 + dmore, worst


# beyond-1-ULP element counts measured at these sizes when the bounds were written (one element of C2's 67 million)
NORM_CASES = [("C1 128x4096", lambda: workloads.config1(), 0), ("C2 8192x8192", lambda: workloads.config2(), 1),
              ("C5 512x7168", lambda: workloads.config5_norm(512), 0)]


@pytest.mark.parametrize("case", range(len(NORM_CASES)))
def test_norm_quant_distances_from_the_unmoved_oracle(device, case):
    """Kernel A with quant NONE (the normed 16-bit row itself) and with the dynamic scale (codes, scales)."""
    name, make_inputs, seen_beyond_1 = NORM_CASES[case]
    inp = make_inputs()
    H = inp.x.shape[1]
    res_ref, norm_ref, _ = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, 0)
    _, norm, _ = run_capi(inp, 0, device)
    d = ulp16(norm, norm_ref)
    rows_off = (d != 0).any(dim=1)
    beyond, worst = report(f"kernel A {name}, normed bf16 output (quant none)", d, rows_off, H)
    assert worst <= 2 and beyond <= max(2 * seen_beyond_1, 8), (beyond, worst)
    assert (d <= 1).float().mean().item() >= 1 - 1e-6          # "within 1 bf16 ULP" holds for all but a handful
    _, codes_ref, scale_ref = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, 1)
    _, codes, scale = run_capi(inp, 1, device)
    d8 = ulp8(codes, codes_ref)
    rows_off8 = (d8 != 0).any(dim=1) | (scale.cpu().flatten() != scale_ref.flatten())
    beyond8, worst8 = report(f"kernel A {name}, fp8 codes (dynamic scale)", d8, rows_off8, H)
    rel = ((scale.cpu().double() - scale_ref.double()).abs() / scale_ref.double()).max().item()
    print(f"[ULP] kernel A {name}, scales: worst relative difference {rel:.3e}; "
          f"{int((scale.cpu().flatten() != scale_ref.flatten()).sum())} of {scale.numel()} not bit-identical", flush=True)
    assert worst8 <= 1 and (d8 == 0).float().mean().item() >= 0.999 and rel <= 1e-6


# (name, inputs, elements beyond 1 ULP seen in q_out, in the K rows) when the bounds were written
ROPE_CASES = [("C3", lambda: workloads.config3(), 15, 2), ("C4", lambda: workloads.config4(), 37, 1),
              ("C5 T=512", lambda: workloads.config5_rope(512), 14, 0)]


@pytest.mark.parametrize("case", range(len(ROPE_CASES)))
def test_rope_distances_from_the_unmoved_oracle(device, case):
    """Kernel B: q_out and the written K rows (16-bit values, or fp8 codes for the decode configuration).  A head whose
    rstd moved by an fp32 ULP flips a first rounding here and there, and the rotation, which subtracts two products
    of nearly equal size, can turn that into several ULPs of the (small) result: such elements exist, they are few,
    and each lies in a head that the parity tests show to be bit-identical to the oracle at the neighbouring rstd."""
    name, make_inputs, seen_q, seen_k = ROPE_CASES[case]
    inp = make_inputs()
    D = inp.head_size
    q_out, kc, vc, (k0, v0) = run_set_kv(inp, device)
    q_ref, k_ref, v_ref = oracle_set_kv(inp, k0, v0)
    loc = inp.kv_loc[inp.kv_loc >= 0]
    dq = ulp16(q_out, q_ref).reshape(-1, D)
    beyond_q, worst_q = report(f"kernel B {name}, q_out", dq, (dq != 0).any(dim=1), D)
    fp8 = kc.element_size() == 1
    dk = (ulp8 if fp8 else ulp16)(kc.cpu()[loc], k_ref[loc]).reshape(-1, D)
    beyond_k, worst_k = report(f"kernel B {name}, K rows ({'fp8 codes' if fp8 else 'bf16'})", dk, (dk != 0).any(dim=1), D)
    assert (dq == 0).float().mean().item() >= 0.999 and (dk == 0).float().mean().item() >= 0.999
    assert (dq <= 1).float().mean().item() >= 1 - 2e-5 and (dk <= 1).float().mean().item() >= 1 - 2e-5
    assert beyond_q <= max(2 * seen_q, 8) and beyond_k <= max(2 * seen_k, 8), (beyond_q, beyond_k)
    # ... and every element, however small, lies within 2 ULPs *of its head's largest value* of the unmoved oracle: an
    # rstd one fp32 ULP away moves a normed value by at most one ULP of itself, the rotation adds two of those
    qf, rf = q_out.cpu().float().reshape(-1, D), q_ref.float().reshape(-1, D)
    head_ulp = torch.exp2(torch.floor(torch.log2(rf.abs().amax(dim=1, keepdim=True).clamp_min(1e-30))) - 7)
    worst_abs = ((qf - rf).abs() / head_ulp).max().item()
    print(f"[ULP] kernel B {name}, q_out: worst distance in ULPs of the head's largest value {worst_abs:.3f}; "
          f"worst in ULPs of the element itself {worst_q}", flush=True)
    assert worst_abs <= 2.0 and worst_q <= 64
    if fp8:
        assert worst_k <= 1
    else:
        assert worst_k <= 64
    assert torch.equal(vc.cpu()[loc].view(torch.uint8), v_ref[loc].view(torch.uint8))
