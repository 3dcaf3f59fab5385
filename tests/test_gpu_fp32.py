"""GPU parity of the fp32- and fp64-activation paths of both operators (the reference dispatches float and double
through the same templates, AT_DISPATCH_FLOATING_TYPES_AND2: src/ops/all_reduce_fusion.cpp:375-378,
src/ops/fused_rope.cpp:27-30, :64-67, :108-111) against the restated torch oracle on tensors of that type.

With these activations the oracle's roundings to the activation type are identities and its variance and rstd stay
fp32, so kernel and oracle differ only in the summation order of the variance (a relative 1e-7 on rstd, for double
too): values are compared with rtol 2e-6 (plus an atol for differences of nearly equal products in the rotation), fp8
codes to the same bar as the 16-bit paths (>= 99.9 % bit-exact, <= 1 fp8 ULP), scales within 1e-6 relative."""
import pytest
import torch

from gpuk_amd import workloads
from oracle import torch_oracle as O
from tests.util import assert_bits_equal, assert_codes_close, assert_scales_close

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-6, 2e-6


WIDE = [torch.float32, torch.float64]
INT_OF = {torch.float32: torch.int32, torch.float64: torch.int64}


def close32(got, want, what):
    g, w = got.cpu(), want.cpu()
    assert g.dtype == w.dtype and g.dtype in WIDE, what
    bad = ~torch.isclose(g, w, rtol=RTOL, atol=ATOL)
    assert not bad.any(), f"{what}: {bad.sum().item()} of {bad.numel()} beyond rtol {RTOL}; worst {(g - w).abs().max().item():.3e}"


@pytest.mark.parametrize("dtype", WIDE)
@pytest.mark.parametrize("tokens,hidden", [(33, 1024), (5, 8), (3, 16384), (64, 7168), (2, 20480), (7, 9000)])
@pytest.mark.parametrize("quant", [0, 1, 3])
def test_add_rmsnorm_quant_fp32(device, tokens, hidden, quant, dtype):
    from gpuk_amd import capi

    print(f"case {dtype} norm-quant tokens={tokens} hidden={hidden} quant={quant}", flush=True)
    inp = workloads.norm_quant_inputs(tokens, hidden, seed=tokens + hidden, res_sigma=1.5, outlier_frac=0.01,
                                      dtype=dtype)
    static = O.static_scale_for(inp.x, inp.residual, inp.gamma, inp.eps) if quant == 3 else None
    x, r, g = inp.x.to(device), inp.residual.to(device), inp.gamma.to(device)
    res = torch.empty_like(x)
    norm = torch.empty((tokens, hidden), dtype=dtype if quant == 0 else torch.float8_e4m3fn, device=device)
    scale = None if quant == 0 else (torch.full((tokens, 1), -1.0, device=device) if quant == 1
                                     else static.to(device).float().reshape(1))
    capi.add_rmsnorm_quant(x, r, g, res, norm, scale, inp.eps, quant)
    torch.cuda.synchronize()
    res_ref, norm_ref, scale_ref = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, quant, static_scale=static)
    assert_bits_equal(res.cpu().view(INT_OF[dtype]), res_ref.view(INT_OF[dtype]), "residual_out")   # one add: exact
    if quant == 0:
        close32(norm, norm_ref, "norm_out")
    else:
        assert_codes_close(norm, norm_ref, "codes")
        if quant == 1:
            assert_scales_close(scale, scale_ref, "scales")


@pytest.mark.parametrize("dtype", WIDE)
@pytest.mark.parametrize("alias", ["residual_in", "x"])
@pytest.mark.parametrize("quant", [0, 1, 3])
def test_residual_out_may_alias_an_input_fp32(device, alias, quant, dtype):
    """The in-place residual stream for fp32 / fp64 activations: residual_out is the same buffer as residual_in or x.
    Rows kept in registers (1, 2 and 4 chunks per lane) and rows swept three times, where a lane reads back what it
    stored (20480 elements), all give the results of separate buffers."""
    from gpuk_amd import capi

    for tokens, hidden in ((33, 1024), (9, 7168), (3, 16384), (4, 20480)):
        print(f"case {dtype} alias={alias} quant={quant} {tokens}x{hidden}", flush=True)
        inp = workloads.norm_quant_inputs(tokens, hidden, seed=hidden + quant, res_sigma=1.5, outlier_frac=0.01, dtype=dtype)
        static = O.static_scale_for(inp.x, inp.residual, inp.gamma, inp.eps) if quant == 3 else None
        x, r, g = inp.x.to(device), inp.residual.to(device), inp.gamma.to(device)
        norm = torch.empty((tokens, hidden), dtype=dtype if quant == 0 else torch.float8_e4m3fn, device=device)
        scale = None if quant == 0 else (torch.full((tokens, 1), -1.0, device=device) if quant == 1
                                         else static.to(device).float().reshape(1))
        res = r if alias == "residual_in" else x
        capi.add_rmsnorm_quant(x, r, g, res, norm, scale, inp.eps, quant)
        torch.cuda.synchronize()
        res_ref, norm_ref, scale_ref = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, quant, static_scale=static)
        assert_bits_equal(res.cpu().view(INT_OF[dtype]), res_ref.view(INT_OF[dtype]), "residual_out")
        if quant == 0:
            close32(norm, norm_ref, "norm_out")
        else:
            assert_codes_close(norm, norm_ref, "codes")
            if quant == 1:
                assert_scales_close(scale, scale_ref, "scales")


def test_torch_op_accepts_fp32(device):
    import gpuk_amd as gpuk

    inp = workloads.norm_quant_inputs(16, 2048, seed=3, dtype=torch.float32)
    x, r, g = inp.x.to(device), inp.residual.to(device), inp.gamma.to(device)
    env = gpuk.GPUKDistEnv(device_id=0)
    res, codes, scale = env.allreduce_add_rms_fused(x, r, g, inp.eps, fp8_out=True)
    res_ref, codes_ref, scale_ref = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, 1)
    assert_codes_close(codes, codes_ref, "codes through the op")
    assert_scales_close(scale, scale_ref, "scales through the op")
    res64, codes64, scale64 = env.allreduce_add_rms_fused(x.double(), r.double(), g.double(), inp.eps, fp8_out=True)
    ref64 = O.add_rmsnorm_quant_ref(inp.x.double(), inp.residual.double(), inp.gamma.double(), inp.eps, 1)
    assert res64.dtype == torch.float64
    assert_codes_close(codes64, ref64[1], "codes through the op, double")
    assert_scales_close(scale64, ref64[2], "scales through the op, double")
    with pytest.raises(RuntimeError):   # not a floating type the reference dispatches
        env.allreduce_add_rms_fused(x.to(torch.int32), r.to(torch.int32), g.to(torch.int32), inp.eps)


def rope_case(tokens, hq, hk, hv, head_size, neox, seed, mrope, interleaved, kv_dtype, dtype=torch.float32):
    inp = workloads.rope_inputs(tokens, hq, hk, hv, head_size, seed=seed, max_pos=5000, num_slots=max(2 * tokens, 64),
                                is_neox=neox, random_table=True, dtype=dtype, kv_dtype=kv_dtype,
                                k_scale=1.5 if kv_dtype == torch.float8_e4m3fn else 1.0,
                                v_scale=2.0 if kv_dtype == torch.float8_e4m3fn else 1.0)
    if mrope:
        g = torch.Generator().manual_seed(seed + 1)
        inp.positions = torch.randint(0, 5000, (3, tokens), generator=g, dtype=torch.int64)
        inp.mrope_section = {64: [12, 10, 10], 128: [24, 20, 20], 256: [48, 40, 40]}[head_size]
        inp.is_interleaved = interleaved
    return inp


@pytest.mark.parametrize("dtype", WIDE)
@pytest.mark.parametrize("head_size", [64, 128, 256])
@pytest.mark.parametrize("neox", [True, False])
@pytest.mark.parametrize("mrope,interleaved", [(False, False), (True, False), (True, True)])
def test_rope_inplace_fp32(device, head_size, neox, mrope, interleaved, dtype):
    from gpuk_amd import capi

    print(f"case {dtype} rope in place D={head_size} neox={neox} mrope={mrope} il={interleaved}", flush=True)
    inp = rope_case(37, 6, 3, 2, head_size, neox, head_size + 1, mrope, interleaved, dtype, dtype)
    qkv, qw, kw, cs, pos = (t.to(device) for t in (inp.qkv, inp.qw, inp.kw, inp.cos_sin, inp.positions))
    capi.rope_rms(qkv, qw, kw, cs, pos, 37, 6, 3, 2, head_size, neox, inp.eps, inp.mrope_section, inp.is_interleaved)
    torch.cuda.synchronize()
    q, k, v = O.rope_rms_ref(inp.qkv, inp.qw, inp.kw, inp.cos_sin, inp.positions, 37, 6, 3, 2, head_size, neox, inp.eps,
                             inp.mrope_section, inp.is_interleaved)
    close32(qkv[:, :6], q, "q")
    close32(qkv[:, 6:9], k, "k")
    assert_bits_equal(qkv[:, 9:].cpu().contiguous().view(INT_OF[dtype]), inp.qkv[:, 9:].contiguous().view(INT_OF[dtype]), "v untouched")


@pytest.mark.parametrize("dtype", WIDE)
@pytest.mark.parametrize("fp8_cache", [False, True])
@pytest.mark.parametrize("mrope", [False, True])
@pytest.mark.parametrize("D,neox", [(128, True), (128, False), (64, True), (256, False)])
def test_rope_set_kv_fp32(device, fp8_cache, mrope, dtype, D, neox):
    import gpuk_amd as gpuk

    kv_dtype = torch.float8_e4m3fn if fp8_cache else dtype
    print(f"case {dtype} rope set_kv cache={kv_dtype} mrope={mrope} D={D} neox={neox}", flush=True)
    T, hq, hk, hv = 45, 7, 2, 3     # a last Q/K wave with idle lanes; at D=256 a second, partly filled V wave
    inp = rope_case(T, hq, hk, hv, D, neox, 77 + D, mrope, False, kv_dtype, dtype)
    inp.kv_loc[3] = -1            # a padding token: q_out row written, K and V rows dropped
    qkv, qw, kw, cs, pos, loc = (t.to(device) for t in (inp.qkv, inp.qw, inp.kw, inp.cos_sin, inp.positions, inp.kv_loc))
    k0, v0 = inp.new_cache()
    kc, vc = k0.to(device), v0.to(device)
    q_out = torch.empty((T, hq, D), dtype=dtype, device=device)
    if mrope:
        gpuk.fused_mrope_3d_rms_set_kv(qkv, qw, kw, cs, pos, T, hq, hk, hv, D, neox, inp.mrope_section, False, inp.eps,
                                       q_out, kc, vc, loc, inp.k_scale, inp.v_scale)
    else:
        gpuk.fused_rope_rms_set_kv(qkv, qw, kw, cs, pos, T, hq, hk, hv, D, neox, inp.eps, q_out, kc, vc, loc,
                                   inp.k_scale, inp.v_scale)
    torch.cuda.synchronize()
    q_ref = torch.empty((T, hq, D), dtype=dtype)
    k_ref, v_ref = k0.clone(), v0.clone()
    O.rope_rms_set_kv_ref(inp.qkv, inp.qw, inp.kw, inp.cos_sin, inp.positions, T, hq, hk, hv, D, neox, inp.eps, q_ref,
                          k_ref, v_ref, inp.kv_loc, inp.k_scale, inp.v_scale, inp.mrope_section, False)
    close32(q_out, q_ref, "q_out")
    kc, vc = kc.cpu(), vc.cpu()
    sel = inp.kv_loc[inp.kv_loc >= 0]
    if not fp8_cache:
        close32(kc[sel], k_ref[sel], "k rows")
        assert_bits_equal(vc[sel].view(INT_OF[dtype]), v_ref[sel].view(INT_OF[dtype]), "v rows")
        raw = lambda t: t.view(INT_OF[dtype])
    else:
        assert_codes_close(kc[sel], k_ref[sel], "k codes")
        assert_codes_close(vc[sel], v_ref[sel], "v codes")
        raw = lambda t: t.view(torch.uint8)
    untouched = torch.ones(inp.num_slots, dtype=torch.bool)
    untouched[sel] = False
    assert_bits_equal(raw(kc[untouched]), raw(k0[untouched]), "untouched k slots")
    assert_bits_equal(raw(vc[untouched]), raw(v0[untouched]), "untouched v slots")
    assert torch.equal(qkv.cpu(), inp.qkv), "set_kv must not modify qkv"


@pytest.mark.parametrize("dtype", WIDE)
@pytest.mark.parametrize("head_size", [64, 128, 256])
@pytest.mark.parametrize("interleaved", [False, True])
def test_rope_2way_fp32(device, head_size, interleaved, dtype):
    import gpuk_amd as gpuk

    print(f"case {dtype} 2way D={head_size} il={interleaved}", flush=True)
    B, T0, T1, Hq, Hk = 2, 19, 45, 3, 5
    g = torch.Generator().manual_seed(head_size + interleaved)
    mk = lambda *shape: torch.randn(shape, generator=g, dtype=dtype)
    q0, k0, q1, k1 = mk(B, T0, Hq, head_size), mk(B, T0, Hk, head_size), mk(B, T1, Hq, head_size), mk(B, T1, Hk, head_size)
    ws = [1 + 0.2 * mk(head_size) for _ in range(4)]
    cs0, cs1 = mk(T0, head_size), mk(T1, head_size)
    dev = lambda t: t.to(device)
    out_q, out_k = gpuk.fused_rope_rms_2way(dev(q0), dev(k0), dev(q1), dev(k1), *(dev(w) for w in ws), dev(cs0), dev(cs1),
                                            B, T0, T1, Hq, Hk, head_size, interleaved, 1e-6)
    torch.cuda.synchronize()
    ref_q, ref_k = O.rope_rms_2way_ref(q0, k0, q1, k1, *ws, cs0, cs1, B, T0, T1, Hq, Hk, head_size, interleaved, 1e-6)
    close32(out_q, ref_q, "out_q01")
    close32(out_k, ref_k, "out_k01")
