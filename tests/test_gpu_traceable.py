"""GPU: the `.mut` overloads (schemas that declare the writes, Meta kernels) under torch's operator checks, under
torch.compile's functionalising front end, and GPUKDistEnv's capture path under HIP graph replay.

Reference: the in-place schemas without alias annotations (src/register.cpp:37-55), GPUKDistEnv.capture /
capture_ / consume_capture (gpuk/__init__.py:98-129), the fused call (gpuk/__init__.py:175-205)."""
import pytest
import torch

from gpuk_amd import workloads
from oracle import torch_oracle as O
from tests.util import assert_bits_equal, assert_codes_close, assert_scales_close

pytestmark = pytest.mark.gpu


def norm_quant_args(device, tokens=96, hidden=1024, quant=1, seed=11):
    inp = workloads.norm_quant_inputs(tokens, hidden, seed=seed, res_sigma=1.5, outlier_frac=0.01)
    x, r, g = inp.x.to(device), inp.residual.to(device), inp.gamma.to(device)
    res_out = torch.empty_like(x)
    norm = torch.empty((tokens, hidden), dtype=torch.float8_e4m3fn if quant else torch.bfloat16, device=device)
    scale = torch.empty((tokens, 1) if quant == 1 else (1,), dtype=torch.float32, device=device)
    return inp, (0, x, r, g, res_out, norm, scale, inp.eps, quant)


def rope_args(device, tokens=40, mrope=False):
    inp = workloads.rope_inputs(tokens, 8, 2, 2, 128, seed=5, max_pos=4096, num_slots=128)
    if mrope:
        g = torch.Generator().manual_seed(6)
        inp.positions = torch.randint(0, 4096, (3, tokens), generator=g, dtype=torch.int64)
        inp.mrope_section = [16, 24, 24]
    k0, v0 = inp.new_cache()
    qkv, qw, kw, cs, pos, loc = (t.to(device) for t in (inp.qkv, inp.qw, inp.kw, inp.cos_sin, inp.positions, inp.kv_loc))
    q = torch.empty((tokens, 8, 128), dtype=torch.bfloat16, device=device)
    return inp, qkv, qw, kw, cs, pos, loc, q, k0.to(device), v0.to(device)


def test_opcheck_schema_and_fake_tensor(device):
    """torch.library.opcheck runs the op and verifies that exactly the tensors the schema marks are written
    (test_schema) and that the Meta kernel agrees with the real one on output metadata (test_faketensor)."""
    import gpuk_amd
    from torch.library import opcheck

    checks = ("test_schema", "test_faketensor")
    _, args = norm_quant_args(device, quant=0)
    opcheck(gpuk_amd.traceable.allreduce_rms, args, test_utils=checks)
    _, args = norm_quant_args(device, quant=1)   # the schema checker's bookkeeping has no fp8 arithmetic
    opcheck(gpuk_amd.traceable.allreduce_rms, args, test_utils=("test_faketensor",))
    inp, qkv, qw, kw, cs, pos, loc, q, kc, vc = rope_args(device)
    opcheck(gpuk_amd.traceable.fused_rope_rms, (qkv.clone(), qw, kw, cs, pos, 40, 8, 2, 2, 128, True, inp.eps),
            test_utils=checks)
    opcheck(gpuk_amd.traceable.fused_rope_rms_set_kv,
            (qkv, qw, kw, cs, pos, 40, 8, 2, 2, 128, True, inp.eps, q, kc, vc, loc, 1.0, 1.0), test_utils=checks)
    inp, qkv, qw, kw, cs, pos, loc, q, kc, vc = rope_args(device, mrope=True)
    opcheck(gpuk_amd.traceable.fused_mrope_3d_rms,
            (qkv.clone(), qw, kw, cs, pos, 40, 8, 2, 2, 128, True, [16, 24, 24], False, inp.eps), test_utils=checks)
    opcheck(gpuk_amd.traceable.fused_mrope_3d_rms_set_kv,
            (qkv, qw, kw, cs, pos, 40, 8, 2, 2, 128, True, [16, 24, 24], False, inp.eps, q, kc, vc, loc, 1.0, 1.0),
            test_utils=checks)


def test_unannotated_schema_fails_the_schema_check(device):
    """The reference's schema string declares no write: the same check rejects it, which is why `.mut` exists."""
    from torch.library import opcheck

    _, args = norm_quant_args(device, quant=0)
    with pytest.raises(Exception, match="test_schema"):
        opcheck(torch.ops.gpuk.allreduce_rms.default, args, test_utils=("test_schema",))


def test_compiled_function_keeps_the_writes(device):
    """A function traced by torch.compile (functionalising `aot_eager` backend: no code generation involved) that
    allocates outputs, calls the fused ops and post-processes their results returns what eager mode returns."""
    import gpuk_amd

    env = gpuk_amd.GPUKDistEnv(device_id=device.index or 0)
    inp, args = norm_quant_args(device, tokens=64, hidden=2048)
    x, r, g = args[1], args[2], args[3]
    rinp, qkv, qw, kw, cs, pos, loc, q, kc, vc = rope_args(device)

    def step(x, r, g, qkv, kc, vc):
        res, codes, scale = env.allreduce_add_rms_fused(x, r, g, inp.eps, fp8_out=True)
        dequant = codes.float() * scale                       # consumer of the written tensors
        q_out = torch.empty((40, 8, 128), dtype=torch.bfloat16, device=x.device)
        gpuk_amd.traceable.fused_rope_rms_set_kv(qkv, qw, kw, cs, pos, 40, 8, 2, 2, 128, True, rinp.eps, q_out, kc, vc,
                                                 loc, 1.0, 1.0)
        return res, codes, scale, dequant.sum(dim=-1), q_out, kc[loc].float().sum(), vc[loc].float().sum()

    kc1, vc1 = kc.clone(), vc.clone()
    eager = step(x, r, g, qkv, kc1, vc1)
    compiled_step = torch.compile(step, backend="aot_eager", fullgraph=True)
    kc2, vc2 = kc.clone(), vc.clone()
    traced = compiled_step(x, r, g, qkv, kc2, vc2)
    torch.cuda.synchronize()
    for a, b, name in zip(eager, traced, ("res", "codes", "scale", "dequant", "q", "k sum", "v sum")):
        if a.dtype == torch.float8_e4m3fn:
            assert_bits_equal(a.view(torch.uint8), b.view(torch.uint8), name)
        else:
            assert torch.equal(a, b), name   # same kernels on the same inputs
    # the caches passed to the compiled function were written in place, like those of the eager call
    bits = lambda t: t.view(torch.int16)   # the cache pre-fill is a byte pattern that contains NaNs
    assert torch.equal(bits(kc2), bits(kc1)) and torch.equal(bits(vc2), bits(vc1))
    assert not torch.equal(bits(kc2), bits(kc)) and not torch.equal(bits(vc2), bits(vc))
    res_ref, codes_ref, scale_ref = O.add_rmsnorm_quant_ref(inp.x, inp.residual, inp.gamma, inp.eps, 1)
    assert_bits_equal(traced[0], res_ref, "compiled residual_out")
    assert_codes_close(traced[1], codes_ref, "compiled codes")
    assert_scales_close(traced[2], scale_ref, "compiled scales")


@pytest.mark.parametrize("tokens,hidden", [(32, 7168), (2048, 7168), (2600, 8192)])
def test_env_capture_replays(device, tokens, hidden):
    """GPUKDistEnv.capture() around a HIP graph capture of the fused call: every replay, with fresh inputs copied
    into the captured buffers and eager work in between, equals the eager result on the same inputs.  (32 rows: one
    ungated launch; 2048: one round of gated workgroups; 2600 x 8192: two gated launches recorded for the one call.)"""
    import gpuk_amd

    env = gpuk_amd.GPUKDistEnv(device_id=device.index or 0)
    static_x = torch.zeros((tokens, hidden), dtype=torch.bfloat16, device=device)
    static_r = torch.zeros_like(static_x)
    gamma = (1 + 0.1 * torch.randn(hidden, device=device)).bfloat16()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        env.allreduce_add_rms_fused(static_x, static_r, gamma, 1e-6, fp8_out=True)   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with env.capture():
        with torch.cuda.graph(graph):
            outs = env.allreduce_add_rms_fused(static_x, static_r, gamma, 1e-6, fp8_out=True)
    assert env._IS_CAPTURED
    for rep in range(4):
        g = torch.Generator(device=device).manual_seed(100 + rep)
        x = torch.randn((tokens, hidden), device=device, generator=g).bfloat16()
        r = torch.randn((tokens, hidden), device=device, generator=g).bfloat16()
        static_x.copy_(x)
        static_r.copy_(r)
        graph.replay()
        torch.cuda.synchronize()
        eager = env.allreduce_add_rms_fused(x, r, gamma, 1e-6, fp8_out=True)   # also clears the captured flag
        torch.cuda.synchronize()
        assert not env._IS_CAPTURED
        assert_bits_equal(outs[0], eager[0], f"replay {rep} residual_out")
        assert_bits_equal(outs[1].view(torch.uint8), eager[1].view(torch.uint8), f"replay {rep} codes")
        assert torch.equal(outs[2], eager[2]), f"replay {rep} scales"


def test_native_sequence_is_close_to_fused(device):
    """The unfused torch sequence kept for comparison agrees with the fused op to the reference test's own bar
    (test/test_all_reduce_fusion.py compares with allclose at 1e-2)."""
    import gpuk_amd

    env = gpuk_amd.GPUKDistEnv(device_id=device.index or 0)
    inp, args = norm_quant_args(device, tokens=64, hidden=4096, quant=0)
    x, r, g = args[1], args[2], args[3]
    fused = env.allreduce_add_rms_fused(x, r, g, inp.eps, fp8_out=False)
    native = env.allreduce_add_rms_native(x, r, g, inp.eps, fp8_out=False)
    assert torch.equal(fused[0], native[0])
    assert torch.allclose(fused[1].float(), native[1].float(), rtol=1e-2, atol=1e-2)
    fused8 = env.allreduce_add_rms_fused(x, r, g, inp.eps, fp8_out=True)
    native8 = env.allreduce_add_rms_native(x, r, g, inp.eps, fp8_out=True)
    assert torch.allclose(fused8[2], native8[2], rtol=1e-5)
    assert torch.allclose(fused8[1].float() * fused8[2], native8[1].float() * native8[2], rtol=0.13, atol=0.05)
