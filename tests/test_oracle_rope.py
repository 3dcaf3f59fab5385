"""Pins the restated QK-RMSNorm + RoPE / mRoPE + KV-write oracle.

The reference holds no vectors for this path.  Checks: rotation identities with closed-form answers, an
fp64 rotation as an independent statement (the form of test/cpp/test_rope_rms.cpp:71-97), three independently
written frequency->axis maps for mRoPE that must agree, scatter invariants of the KV write, and
agreement between the torch restatement and the plain-C one.
"""
import os

import numpy as np
import pytest
import torch

from gpuk_amd import workloads
from oracle import c_oracle, torch_oracle as O
from tests.util import assert_bits_equal, assert_rotated_close

GOLD = os.path.join(os.path.dirname(__file__), "golden")
SECTIONS = {64: [12, 10, 10], 128: [24, 20, 20], 256: [48, 40, 40]}


def small(neox=True, D=64, T=9, hq=3, hk=2, hv=2, seed=0, table="random"):
    r = workloads.rope_inputs(T, hq, hk, hv, D, seed=seed, max_pos=128, num_slots=32, is_neox=neox,
                              random_table=(table == "random"))
    return r


def run(r, **kw):
    return O.rope_rms_ref(r.qkv, r.qw, r.kw, r.cos_sin, r.positions, r.num_tokens, r.num_heads_q, r.num_heads_k,
                          r.num_heads_v, r.head_size, r.is_neox, r.eps, **kw)


@pytest.mark.parametrize("neox", [True, False])
def test_rotation_identities(neox):
    r = small(neox)
    D, half = r.head_size, r.head_size // 2
    qn = O.rms_norm_forward(r.qkv[:, :3].clone(), r.qw, r.eps)
    # cos = 1, sin = 0: the rotation is the identity, the op reduces to the per-head RMSNorm
    r.cos_sin = torch.cat([torch.ones(128, half), torch.zeros(128, half)], -1).bfloat16()
    q, k, v = run(r)
    assert_bits_equal(q, qn, "identity rotation")
    assert_bits_equal(v, r.qkv[:, 5:], "v passes through")
    # cos = 0, sin = 1: (x1, x2) -> (-x2, x1)
    r.cos_sin = torch.cat([torch.zeros(128, half), torch.ones(128, half)], -1).bfloat16()
    q, _, _ = run(r)
    if neox:
        want = torch.cat([-qn[..., half:], qn[..., :half]], -1)
    else:
        want = torch.stack([-qn[..., 1::2], qn[..., ::2]], -1).flatten(-2)
    assert_bits_equal(q, want, "quarter turn")
    # position 0 of a real table is the identity as well
    r.cos_sin = workloads.rope_table(128, D)
    r.positions = torch.zeros_like(r.positions)
    q, _, _ = run(r)
    assert_bits_equal(q, qn, "position 0")


@pytest.mark.parametrize("neox", [True, False])
def test_against_fp64_rotation(neox):
    """Independent statement with double accumulation, as the reference's C++ CPU check does."""
    r = small(neox, D=128, table="real")
    q, k, _ = run(r)
    D, half = 128, 64
    x = r.qkv.double()
    cs = r.cos_sin[r.positions].double()
    cos, sin = cs[:, None, :half], cs[:, None, half:]

    def ref(xh, w):
        n = xh / torch.sqrt((xh * xh).mean(-1, keepdim=True) + r.eps) * w.double()
        if neox:
            x1, x2 = n[..., :half], n[..., half:]
            return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], -1)
        x1, x2 = n[..., ::2], n[..., 1::2]
        return torch.stack([x1 * cos - x2 * sin, x2 * cos + x1 * sin], -1).flatten(-2)

    for got, want in ((q, ref(x[:, :3], r.qw)), (k, ref(x[:, 3:5], r.kw))):
        # five bf16 roundings on values of magnitude ~|n|: absolute error a few bf16 ULPs of the head's scale
        assert (got.double() - want).abs().max().item() < 0.06
    # the rotation preserves the norm of every (x1, x2) pair up to rounding
    qn = O.rms_norm_forward(r.qkv[:, :3], r.qw, r.eps).double()
    if neox:
        n_in = qn[..., :half] ** 2 + qn[..., half:] ** 2
        n_out = q.double()[..., :half] ** 2 + q.double()[..., half:] ** 2
    else:
        n_in = qn[..., ::2] ** 2 + qn[..., 1::2] ** 2
        n_out = q.double()[..., ::2] ** 2 + q.double()[..., 1::2] ** 2
    assert ((n_out - n_in).abs() <= 0.05 * n_in + 1e-3).all()


def axis_kernel_formula(f, section, interleaved):
    """Index form of the reference kernel (src/impl/rope_rms_impl.h:126-152)."""
    if interleaved:
        m = f % 3
        return m if (m >= 1 and f < section[m] * 3) else 0
    end = 0
    for a in range(3):
        end += section[a]
        if f < end:
            return a
    raise AssertionError


def axis_cpp_test_formula(half, section, interleaved):
    """Loop form of the reference's C++ CPU check (test/cpp/test_mrope_rms.cpp:110-150)."""
    out = [0] * half
    if interleaved:
        for i in range(half):
            im = i % 3
            out[i] = im if (im >= 1 and i < section[im] * 3) else 0
    else:
        i = 0
        end = 0
        for mid in range(3):
            end += section[mid]
            while i < end:
                out[i] = mid
                i += 1
    return out


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("interleaved", [False, True])
def test_three_mrope_axis_maps_agree(D, interleaved):
    half = D // 2
    sections = [SECTIONS[D], [half, 0, 0], [0, half, 0], [half - 2, 1, 1]]
    if D == 128:
        sections.append([16, 24, 24])
    for sec in sections:
        # torch slicing form (the reference's python tests), probed with a tensor whose value is its axis
        probe = torch.arange(3.0)[:, None, None].expand(3, 1, half).contiguous()
        via_torch = O.mrope_select(probe, sec, interleaved)[0].long().tolist()
        via_kernel = [axis_kernel_formula(f, sec, interleaved) for f in range(half)]
        via_cpp = axis_cpp_test_formula(half, sec, interleaved)
        assert via_torch == via_kernel == via_cpp, (sec, interleaved)


def test_equal_position_rows_reduce_to_plain_rope():
    r = small(True, D=128)
    plain = run(r)
    pos3 = r.positions.unsqueeze(0).expand(3, -1).contiguous()
    for il in (False, True):
        q, k, v = O.rope_rms_ref(r.qkv, r.qw, r.kw, r.cos_sin, pos3, r.num_tokens, 3, 2, 2, 128, True, r.eps,
                                 SECTIONS[128], il)
        assert_bits_equal(q, plain[0], "q"); assert_bits_equal(k, plain[1], "k")


@pytest.mark.parametrize("fp8", [False, True])
def test_kv_scatter_invariants(fp8):
    r = workloads.rope_inputs(10, 3, 2, 2, 64, seed=3, max_pos=64, num_slots=40, random_table=True,
                              kv_dtype=torch.float8_e4m3fn if fp8 else torch.bfloat16,
                              k_scale=1.5 if fp8 else 1.0, v_scale=2.0 if fp8 else 1.0)
    k0, v0 = r.new_cache()
    k, v = k0.clone(), v0.clone()
    q = torch.empty((10, 3, 64), dtype=torch.bfloat16)
    O.rope_rms_set_kv_ref(r.qkv, r.qw, r.kw, r.cos_sin, r.positions, 10, 3, 2, 2, 64, True, r.eps, q, k, v, r.kv_loc,
                          r.k_scale, r.v_scale)
    qq, kk, vv = run(r)
    assert_bits_equal(q, qq, "q_out equals the rotated q")
    u8 = lambda t: t.view(torch.uint8)
    untouched = torch.ones(40, dtype=torch.bool); untouched[r.kv_loc] = False
    assert (u8(k)[untouched] == u8(k0)[untouched]).all() and (u8(v)[untouched] == u8(v0)[untouched]).all()
    if fp8:
        assert (u8(k)[r.kv_loc] == u8((kk / 1.5).to(torch.float8_e4m3fn))).all()
        assert (u8(v)[r.kv_loc] == u8((vv / 2.0).to(torch.float8_e4m3fn))).all()
    else:
        assert_bits_equal(k[r.kv_loc], kk, "k rows"); assert_bits_equal(v[r.kv_loc], vv, "v rows")
    # q_out does not depend on what the cache held
    k2, v2 = torch.zeros_like(k0), torch.zeros_like(v0)
    q2 = torch.empty_like(q)
    O.rope_rms_set_kv_ref(r.qkv, r.qw, r.kw, r.cos_sin, r.positions, 10, 3, 2, 2, 64, True, r.eps, q2, k2, v2, r.kv_loc,
                          r.k_scale, r.v_scale)
    assert_bits_equal(q2, q, "q independent of cache")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("neox", [True, False])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_c_and_torch_restatements_agree(dtype, neox, D):
    for mrope, il, fp8 in ((False, False, False), (True, False, True), (True, True, False), (True, True, True)):
        r = workloads.rope_inputs(21, 5, 3, 2, D, seed=D + il, max_pos=200, num_slots=50, is_neox=neox,
                                  random_table=True, dtype=dtype,
                                  kv_dtype=torch.float8_e4m3fn if fp8 else dtype,
                                  k_scale=1.5 if fp8 else 1.0, v_scale=2.0 if fp8 else 1.0)
        sec = None
        if mrope:
            r.positions = torch.randint(0, 200, (3, 21), generator=torch.Generator().manual_seed(1), dtype=torch.int64)
            sec = SECTIONS[D]
        k0, v0 = r.new_cache()
        q1 = torch.empty((21, 5, D), dtype=dtype); k1, v1 = k0.clone(), v0.clone()
        O.rope_rms_set_kv_ref(r.qkv, r.qw, r.kw, r.cos_sin, r.positions, 21, 5, 3, 2, D, neox, r.eps, q1, k1, v1,
                              r.kv_loc, r.k_scale, r.v_scale, sec, il)
        q2 = torch.empty_like(q1); k2, v2 = k0.clone(), v0.clone()
        c_oracle.rope_rms(r.qkv.clone(), r.qw, r.kw, r.cos_sin, r.positions, 21, 5, 3, 2, D, neox, r.eps, sec, il, q2,
                          k2.view(torch.uint8) if fp8 else k2, v2.view(torch.uint8) if fp8 else v2, r.kv_loc,
                          r.k_scale, r.v_scale)
        # the C sum of squares is accumulated in double, torch's in fp32: rstd can differ by one fp32 ULP, which
        # moves a rare element by one 16-bit ULP; everything else is bit-identical
        assert_rotated_close(q2, q1, "q", min_exact=0.999)
        assert (k1.view(torch.uint8) != k2.view(torch.uint8)).float().mean().item() < 1e-3
        assert (v1.view(torch.uint8) == v2.view(torch.uint8)).all()
        # in-place form
        qkv = r.qkv.clone()
        c_oracle.rope_rms(qkv, r.qw, r.kw, r.cos_sin, r.positions, 21, 5, 3, 2, D, neox, r.eps, sec, il)
        q, k, v = O.rope_rms_ref(r.qkv, r.qw, r.kw, r.cos_sin, r.positions, 21, 5, 3, 2, D, neox, r.eps, sec, il)
        assert_rotated_close(qkv, torch.cat([q, k, v], 1), "in place", min_exact=0.999)
        assert_bits_equal(qkv[:, 8:], v, "in place leaves v alone")


def test_strided_positions_in_c_checker():
    r = small(True, D=64)
    pos_t = torch.randint(0, 128, (9, 3), generator=torch.Generator().manual_seed(2), dtype=torch.int64)
    qkv = r.qkv.clone()
    c_oracle.rope_rms(qkv, r.qw, r.kw, r.cos_sin, pos_t.t(), 9, 3, 2, 2, 64, True, r.eps, SECTIONS[64], False)
    q, k, v = O.rope_rms_ref(r.qkv, r.qw, r.kw, r.cos_sin, pos_t.t().contiguous(), 9, 3, 2, 2, 64, True, r.eps,
                             SECTIONS[64], False)
    assert_bits_equal(qkv, torch.cat([q, k, v], 1), "strided positions")


def test_two_way_restatements_agree():
    g = torch.Generator().manual_seed(5)
    B, T0, T1, Hq, Hk, D = 2, 5, 3, 4, 2, 64
    mk = lambda *s: torch.randn(*s, generator=g).bfloat16()
    q0, k0, q1, k1 = mk(B, T0, Hq, D), mk(B, T0, Hk, D), mk(B, T1, Hq, D), mk(B, T1, Hk, D)
    ws = [mk(D) for _ in range(4)]
    cs0, cs1 = mk(T0, D), mk(T1, D)
    for il in (False, True):
        a = O.rope_rms_2way_ref(q0, k0, q1, k1, *ws, cs0, cs1, B, T0, T1, Hq, Hk, D, il, 1e-6)
        b = c_oracle.rope_rms_2way(q0, k0, q1, k1, *ws, cs0, cs1, B, T0, T1, Hq, Hk, D, il, 1e-6)
        assert_bits_equal(b[0], a[0], "q01"); assert_bits_equal(b[1], a[1], "k01")


def test_small_golden_cases():
    z = np.load(os.path.join(GOLD, "small_cases.npz"))
    bf = lambda a: torch.from_numpy(a.copy()).view(torch.bfloat16)
    for name, (neox, il, fp8) in {"rope_a": (True, False, True), "rope_b": (False, True, False)}.items():
        qkv, qw, kw, cs = (bf(z[f"{name}_{k}"]) for k in ("qkv", "qw", "kw", "cos_sin"))
        pos, loc = torch.from_numpy(z[name + "_pos"]), torch.from_numpy(z[name + "_loc"])
        kd = torch.float8_e4m3fn if fp8 else torch.bfloat16
        k = torch.from_numpy(z[name + "_k0"].copy()).view(kd); v = torch.from_numpy(z[name + "_v0"].copy()).view(kd)
        q = torch.empty((6, 3, 64), dtype=torch.bfloat16)
        ks, vs = (1.5, 2.0) if fp8 else (1.0, 1.0)
        for impl in ("torch", "c"):
            kk, vv, qq = k.clone(), v.clone(), q.clone()
            if impl == "torch":
                O.rope_rms_set_kv_ref(qkv, qw, kw, cs, pos, 6, 3, 2, 2, 64, neox, 1e-6, qq, kk, vv, loc, ks, vs, [12, 10, 10], il)
            else:
                c_oracle.rope_rms(qkv.clone(), qw, kw, cs, pos, 6, 3, 2, 2, 64, neox, 1e-6, [12, 10, 10], il, qq,
                                  kk.view(torch.uint8) if fp8 else kk, vv.view(torch.uint8) if fp8 else vv, loc, ks, vs)
            assert (qq.view(torch.int16).numpy() == z[name + "_q"]).all(), (name, impl)
            assert (kk.view(torch.uint8).numpy() == z[name + "_k"]).all(), (name, impl)
            assert (vv.view(torch.uint8).numpy() == z[name + "_v"]).all(), (name, impl)
