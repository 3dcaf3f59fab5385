"""CPU-only checks of the boundary: the C-ABI library loads and exports every symbol its header declares,
the torch library registers the reference's operator schemas, argument validation rejects what it must
without touching a GPU, and the host-side byte accounting matches the published per-configuration figures."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "gpuk_amd.h")


def declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(gpuk_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    from gpuk_amd import capi

    names = declared_functions()
    assert set(names) == set(capi.EXPORTS), (names, capi.EXPORTS)
    lib = ctypes.CDLL(os.path.join(ROOT, "gpuk_amd", "lib", "libgpuk_amd.so"))
    for n in names:
        assert getattr(lib, n) is not None
    assert capi.lib().gpuk_abi_version() == 2
    assert capi.lib().gpuk_status_string(0) == b"ok"
    assert b"unsupported" in capi.lib().gpuk_status_string(2)


def test_argument_validation_needs_no_gpu():
    """Bad arguments are rejected before any launch (status codes, not exceptions or aborts)."""
    from gpuk_amd import capi

    L = capi.lib()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p = (p + 15) & ~15
    f = L.gpuk_add_rmsnorm_quant
    assert f(p, p, p, p, p, p, -1, 1024, 1e-6, 0, 1, 448.0, None) == 1      # negative tokens
    assert f(p, p, p, p, p, p, 4, 1020, 1e-6, 0, 1, 448.0, None) == 2       # hidden % 8
    assert f(p, p, p, p, p, p, 4, 1024, 1e-6, 7, 1, 448.0, None) == 2       # unknown dtype
    assert f(p, p, p, p, p, p, 4, 1024, 1e-6, 0, 2, 448.0, None) == 2       # e4m3fnuz
    assert f(p, p, p, p, p, p, 4, 1024, 1e-6, 0, 9, 448.0, None) == 2       # unknown quant
    assert f(p, p, p, p, p, None, 4, 1024, 1e-6, 0, 1, 448.0, None) == 1    # dynamic quant needs scale
    assert f(p + 2, p, p, p, p, p, 4, 1024, 1e-6, 0, 1, 448.0, None) == 3   # misaligned
    assert f(p, p, p, p, p, p, 4, 1024, 1e-6, 0, 1, 0.0, None) == 1         # fp8_max must be positive
    assert f(None, None, None, None, None, None, 0, 1024, 1e-6, 0, 1, 448.0, None) == 0   # empty batch is a no-op
    sec = (ctypes.c_int64 * 3)(16, 16, 16)
    r = L.gpuk_rope_rms
    assert r(p, p, p, p, p, 0, 1, 3, 4, 2, 2, 2, 128, 1, sec, 0, 1e-6, 0, None) == 1     # sections sum to 48, not 64
    assert r(p, p, p, p, p, 0, 1, 1, 4, 2, 2, 2, 96, 1, None, 0, 1e-6, 0, None) == 2     # head size
    assert r(p, p, p, p, p, 0, 1, 2, 4, 2, 2, 2, 128, 1, None, 0, 1e-6, 0, None) == 1    # n_axes
    assert r(p, p, p, p, p, 0, 1, 3, 4, 2, 2, 2, 128, 1, None, 0, 1e-6, 0, None) == 1    # mRoPE without sections
    assert r(None, None, None, None, None, 0, 1, 1, 0, 2, 2, 2, 128, 1, None, 0, 1e-6, 0, None) == 0   # no tokens
    s = L.gpuk_rope_rms_set_kv
    assert s(p, p, p, p, p, 0, 1, 1, 4, 2, 2, 2, 128, 1, None, 0, 1e-6, 0, p, p, p, p, 1.0, 1.0, 5, None) == 2  # kv dtype
    assert s(p, p, p, p, p, 0, 1, 1, 4, 2, 2, 2, 128, 1, None, 0, 1e-6, 0, p, p, p, p, 0.0, 1.0, 1, None) == 1  # fp8 scale
    assert s(p, p, p, p, p, 0, 1, 1, 4, 2, 2, 2, 128, 1, None, 0, 1e-6, 0, None, p, p, p, 1.0, 1.0, 0, None) == 1
    w = L.gpuk_rope_rms_2way
    assert w(p, p, p, p, p, p, p, p, p, p, 1, 2, 2, 2, 2, 96, 0, 1e-6, 0, p, p, None) == 2     # head size
    assert w(p, p, p, p, p, p, p, p, p, p, 1, -2, 2, 2, 2, 128, 0, 1e-6, 0, p, p, None) == 1   # negative tokens
    assert w(p, p, p, p, p, p, p, p, p, p, 1, 2, 2, 2, 2, 128, 0, 1e-6, 0, None, p, None) == 1  # missing output
    assert w(p, p, p, p, p, p, p, p, p, p, 0, 2, 2, 2, 2, 128, 0, 1e-6, 0, p, p, None) == 0    # empty batch
    assert L.gpuk_copy_bytes(p, p, 24, None) == 1 and L.gpuk_copy_bytes(p, p, 0, None) == 0
    assert L.gpuk_read_bytes(p, 24, p, None) == 1 and L.gpuk_read_bytes(p, 0, p, None) == 0
    assert L.gpuk_read_bytes(p, 32, None, None) == 1 and L.gpuk_read_bytes(p + 4, 32, p, None) == 3
    assert L.gpuk_fill_bytes(p, 24, 1, None) == 1 and L.gpuk_fill_bytes(None, 32, 1, None) == 1
    assert L.gpuk_fill_bytes(p, 0, 1, None) == 0 and L.gpuk_fill_bytes(p + 8, 32, 1, None) == 3
    assert L.gpuk_empty_grid(4, 100, 0, None) == 1 and L.gpuk_empty_grid(4, 2048, 0, None) == 1
    assert L.gpuk_empty_grid(4, 256, 1 << 20, None) == 1 and L.gpuk_empty_grid(0, 256, 0, None) == 0
    assert L.gpuk_set_tuning(b"no_such_knob", 1) == 1 and L.gpuk_set_tuning(b"norm_quant_nchunk", 3) == 1
    assert L.gpuk_set_tuning(b"norm_quant_nchunk", 0) == 0
    assert L.gpuk_set_tuning(b"norm_quant_launches", 3) == 1 and L.gpuk_set_tuning(b"norm_quant_launches", 0) == 0


def test_torch_library_registers_reference_schemas():
    import gpuk_amd as gpuk

    def schema(name):
        return str(getattr(torch.ops.gpuk, name).default._schema)

    assert schema("allreduce_rms") == (
        "gpuk::allreduce_rms(SymInt fptr, Tensor allreduce_in, Tensor residual_in, Tensor rms_gamma, "
        "Tensor residual_out, Tensor norm_out, Tensor scale_out, float eps, SymInt quant_type) -> ()")
    assert schema("fused_rope_rms") == (
        "gpuk::fused_rope_rms(Tensor qkv, Tensor qw, Tensor kw, Tensor cos_sin, Tensor positions, SymInt num_tokens, "
        "SymInt num_heads_q, SymInt num_heads_k, SymInt num_heads_v, SymInt head_size, bool is_neox_style, "
        "float eps) -> ()")
    assert "int[] mrope_section_, bool is_interleaved, float eps) -> ()" in schema("fused_mrope_3d_rms")
    assert schema("fused_mrope_3d_rms_set_kv").endswith(
        "float eps, Tensor q, Tensor k_cache, Tensor v_cache, Tensor kv_loc, float k_scale, float v_scale) -> ()")
    for name in ("allreduce_rms", "fused_rope_rms", "fused_mrope_3d_rms", "fused_mrope_3d_rms_set_kv",
                 "fused_rope_rms_2way", "fused_rope_rms_set_kv", "set_fp8_max", "get_fp8_max"):
        assert hasattr(gpuk, name)
    assert gpuk.fp8 == torch.float8_e4m3fn and gpuk.fp8_max_val == 448 and gpuk.fp8_policy_id == 1


def test_two_way_op_has_a_meta_kernel():
    """Shape inference without a device, as the reference registers it (src/register.cpp:62-63)."""
    import gpuk_amd as gpuk

    m = lambda *s: torch.empty(*s, dtype=torch.bfloat16, device="meta")
    B, T0, T1, Hq, Hk, D = 2, 5, 7, 3, 2, 64
    q01, k01 = gpuk.fused_rope_rms_2way(m(B, T0, Hq, D), m(B, T0, Hk, D), m(B, T1, Hq, D), m(B, T1, Hk, D), m(D), m(D),
                                        m(D), m(D), m(T0, D), m(T1, D), B, T0, T1, Hq, Hk, D, False, 1e-6)
    assert q01.shape == (B, T0 + T1, Hq, D) and k01.shape == (B, T0 + T1, Hk, D)
    assert q01.device.type == "meta" and q01.dtype == torch.bfloat16
    assert str(torch.ops.gpuk.fused_rope_rms_2way.default._schema).endswith(
        "SymInt head_size, bool is_interleaved, float eps) -> (Tensor out_q01, Tensor out_k01)")


def test_fp8_max_setter_round_trip():
    import gpuk_amd as gpuk

    assert gpuk.get_fp8_max() == 448.0
    gpuk.set_fp8_max(240.0)
    try:
        assert gpuk.get_fp8_max() == 240.0
        with pytest.raises(RuntimeError):
            gpuk.set_fp8_max(0.0)
        with pytest.raises(RuntimeError):
            gpuk.set_fp8_max(1000.0)
    finally:
        gpuk.set_fp8_max(448.0)


def test_ops_refuse_cpu_tensors():
    """There is no CPU fallback: the compute ops exist for GPU tensors only."""
    import gpuk_amd as gpuk

    x = torch.zeros((2, 64), dtype=torch.bfloat16)
    with pytest.raises((RuntimeError, NotImplementedError)):
        gpuk.allreduce_rms(0, x, x, x[0], x.clone(), x.clone(), torch.zeros(2, 1), 1e-6, 0)
    with pytest.raises((RuntimeError, NotImplementedError)):
        gpuk.fused_rope_rms(torch.zeros((2, 3, 64), dtype=torch.bfloat16), x[0], x[0], torch.zeros((8, 64), dtype=torch.bfloat16),
                            torch.zeros(2, dtype=torch.int64), 2, 1, 1, 1, 64, True, 1e-6)


def test_algorithmic_byte_formulas():
    """Compulsory traffic per call, as published for the five configurations."""
    from gpuk_amd import workloads as W

    assert W.norm_quant_bytes(8192, 8192, 1) == 469_811_200
    assert W.norm_quant_bytes(128, 4096, 3) == 3_678_212
    assert [W.norm_quant_bytes(t, 7168, 1) for t in W.DECODE_TOKENS] == [64_516, 415_776, 1_620_096, 6_437_376, 25_706_496]
    assert W.rope_set_kv_bytes(4096, 32, 8, 8, 128, 1, 2) == 101_777_920
    assert W.rope_set_kv_bytes(8192, 28, 4, 4, 128, 3, 2) == 153_354_752
    assert W.rope_set_kv_bytes(1, 64, 8, 8, 128, 1, 1) == 39_696 and W.rope_set_kv_bytes(512, 64, 8, 8, 128, 1, 1) == 20_062_720
    # in-place form: the reference's own formula (test/cpp/test_rope_rms.cpp:184-188) plus the position read
    T, hq, hk, D = 513, 32, 32, 128
    ref = T * (hq + hk) * D * 2 + 2 * D * 2 + T * D * 2 + T * (hq + hk) * D * 2
    assert W.rope_inplace_bytes(T, hq, hk, D) == ref + 8 * T


def test_workload_generators_are_deterministic_and_shaped():
    from gpuk_amd import workloads as W

    a, b = W.config1(), W.config1()
    assert torch.equal(a.x, b.x) and a.x.shape == (128, 4096) and a.x.dtype == torch.bfloat16
    c2 = W.config2(64, 512)
    frac = (c2.x.abs() == 50).float().mean().item()
    assert 0.005 < frac < 0.015
    c3 = W.config3(256)
    assert c3.qkv.shape == (256, 48, 128) and c3.kv_loc.unique().numel() == 256 and c3.num_slots == 65536
    assert c3.cos_sin.shape == (32768, 128) and c3.cos_sin[0, :64].eq(1).all() and c3.cos_sin[0, 64:].eq(0).all()
    c4 = W.config4(4096)
    pos = c4.positions
    assert pos.shape == (3, 4096) and (pos[:, :1024] == torch.arange(1024)).all()
    img = pos[:, 1024:2048]
    assert (img[0] == 1024).all() and img[1].max() == 1024 + 31 and img[2].max() == 1024 + 31
    assert (pos[:, 2048] == 1024 + 32).all() and c4.mrope_section == [16, 24, 24]
    c5 = W.config5_rope(8)
    assert c5.kv_dtype == torch.float8_e4m3fn and c5.qkv.shape == (8, 80, 128)


def test_dist_env_rejects_multi_gpu_groups(monkeypatch):
    import torch.distributed as dist

    import gpuk_amd as gpuk

    monkeypatch.setattr(dist, "is_initialized", lambda: True)
    monkeypatch.setattr(dist, "get_rank", lambda group=None: 0)
    monkeypatch.setattr(dist, "get_world_size", lambda group=None: 2)
    monkeypatch.setattr(torch.cuda, "current_device", lambda: 0)
    with pytest.raises(NotImplementedError):
        gpuk.GPUKDistEnv(device_id=0)


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "single-GPU" in r.stderr


def test_mut_overloads_differ_from_reference_schemas_only_in_alias_annotations():
    """Every in-place operator has an overload `.mut` whose schema, with the `(x!)` annotations removed, is the
    reference's string (src/register.cpp:37-55), and which declares at least one written tensor."""
    import re

    import gpuk_amd  # noqa: F401  (loads the library)

    for name in ("allreduce_rms", "fused_rope_rms", "fused_mrope_3d_rms", "fused_mrope_3d_rms_set_kv",
                 "fused_rope_rms_set_kv"):
        packet = getattr(torch.ops.gpuk, name)
        assert packet.overloads() == ["default", "mut"], name
        plain, annotated = str(packet.default._schema), str(packet.mut._schema)
        assert "!)" in annotated and "!)" not in plain
        assert re.sub(r"\([a-z]!\)", "", annotated).replace(name + ".mut(", name + "(") == plain
    written = {a.name for a in torch.ops.gpuk.allreduce_rms.mut._schema.arguments if a.alias_info and a.alias_info.is_write}
    assert written == {"residual_out", "norm_out", "scale_out"}
    written = {a.name for a in torch.ops.gpuk.fused_mrope_3d_rms_set_kv.mut._schema.arguments
               if a.alias_info and a.alias_info.is_write}
    assert written == {"q", "k_cache", "v_cache"}
    written = {a.name for a in torch.ops.gpuk.fused_rope_rms.mut._schema.arguments if a.alias_info and a.alias_info.is_write}
    assert written == {"qkv"}


def test_mut_overloads_have_meta_kernels():
    """On meta tensors the `.mut` overloads run (and do nothing); the reference-schema overloads have no Meta
    kernel and refuse, as in the reference."""
    import gpuk_amd

    x = torch.empty((4, 64), dtype=torch.bfloat16, device="meta")
    g = torch.empty((64,), dtype=torch.bfloat16, device="meta")
    codes = torch.empty((4, 64), dtype=torch.float8_e4m3fn, device="meta")
    scale = torch.empty((4, 1), device="meta")
    assert gpuk_amd.traceable.allreduce_rms(0, x, x, g, x, codes, scale, 1e-6, 1) is None
    with pytest.raises(NotImplementedError):
        gpuk_amd.allreduce_rms(0, x, x, g, x, codes, scale, 1e-6, 1)
    qkv = torch.empty((4, 6, 64), dtype=torch.bfloat16, device="meta")
    pos = torch.empty((4,), dtype=torch.int64, device="meta")
    assert gpuk_amd.traceable.fused_rope_rms(qkv, g, g, x, pos, 4, 2, 2, 2, 64, True, 1e-6) is None


def test_reference_kernel_library_exports_its_entry_points():
    """oracle/_ref/libgpuk_ref.so (the reference's own kernels, compiled where a reference checkout exists) loads and
    exports the four entry points the GPU tests call.  Skipped where it was never built."""
    from oracle import ref_kernels

    if not ref_kernels.available():
        pytest.skip("oracle/_ref/libgpuk_ref.so not built")
    import torch  # noqa: F401  (its HIP runtime first, as for the product library)

    L = ref_kernels.lib()
    for name in ("gpuk_ref_rope_rms", "gpuk_ref_mrope_rms_set_kv", "gpuk_ref_rope_rms_2way", "gpuk_ref_epilogue_rows"):
        assert hasattr(L, name), name
    # argument refusal happens before any launch
    assert L.gpuk_ref_epilogue_rows(None, None, None, None, None, None, 0, 4096, 1e-6, 1, None) == -1
    assert L.gpuk_ref_rope_rms(None, None, None, None, None, 0, 1, 1, 4, 2, 2, 2, 96, 1, None, 0, 1e-6, None) == -1


def test_launch_shape_report():
    """gpuk_add_rmsnorm_quant_launch_shape computes on the host: lanes per row and 16-byte chunks per lane of the launch
    the norm-quant entry point would make (no GPU needed)."""
    from gpuk_amd import capi

    assert capi.add_rmsnorm_quant_launch_shape(8192, 8192) == (512, 2)
    assert capi.add_rmsnorm_quant_launch_shape(512, 7168) == (448, 2)
    # 1025-2048 rows of 7168: too many for one round at two chunks per lane, not at four (half the lanes per row)
    assert capi.add_rmsnorm_quant_launch_shape(1024, 7168) == (448, 2)
    assert capi.add_rmsnorm_quant_launch_shape(1025, 7168) == (256, 4)
    assert capi.add_rmsnorm_quant_launch_shape(2048, 8192) == (256, 4)
    assert capi.add_rmsnorm_quant_launch_shape(2049, 8192) == (512, 2)
    # from 1.1 rounds to two the call is two launches; the report is the first one's (1280 of 2600 rows, 1536 of 3000)
    assert capi.add_rmsnorm_quant_launch_shape(2252, 8192) == (512, 2)
    assert capi.add_rmsnorm_quant_launch_shape(2600, 8192) == (256, 4)
    assert capi.add_rmsnorm_quant_launch_shape(3000, 7168) == (256, 4)
    assert capi.add_rmsnorm_quant_launch_shape(4097, 7168) == (448, 2)
    # workgroups of five waves: a compute unit takes five of them, not six
    assert capi.add_rmsnorm_quant_launch_shape(1280, 5120) == (320, 2)
    assert capi.add_rmsnorm_quant_launch_shape(1281, 5120) == (192, 4)
    assert capi.add_rmsnorm_quant_launch_shape(1, 4096) == (256, 2)
    lanes, chunks = capi.add_rmsnorm_quant_launch_shape(4, 65600 * 2)    # rows that do not stay in registers
    assert chunks == 0 and lanes % 64 == 0
    # fp32 / fp64: chunks of 4 elements, kept in registers up to 4 x 1024 of them
    assert capi.add_rmsnorm_quant_launch_shape(128, 1024, torch.float32) == (128, 2)
    assert capi.add_rmsnorm_quant_launch_shape(128, 1024, torch.float64) == (256, 1)
    assert capi.add_rmsnorm_quant_launch_shape(128, 8192, torch.float64) == (1024, 2)
    assert capi.add_rmsnorm_quant_launch_shape(128, 12288, torch.float32) == (768, 4)
    assert capi.add_rmsnorm_quant_launch_shape(128, 16392, torch.float32) == (1024, 0)
    L = capi.lib()
    import ctypes as C
    a, b = C.c_int(0), C.c_int(0)
    assert L.gpuk_add_rmsnorm_quant_launch_shape(0, 1024, 0, C.byref(a), C.byref(b)) == 1
    assert L.gpuk_add_rmsnorm_quant_launch_shape(4, 1027, 0, C.byref(a), C.byref(b)) == 2
    assert L.gpuk_add_rmsnorm_quant_launch_shape(4, 1024, 0, None, C.byref(b)) == 1
    # the query refuses what the entry point refuses: rows that are no multiple of 8 elements (whatever the dtype),
    # and a dtype value that names no format
    assert L.gpuk_add_rmsnorm_quant_launch_shape(4, 16388, 2, C.byref(a), C.byref(b)) == 2
    assert L.gpuk_add_rmsnorm_quant_launch_shape(4, 1024, 7, C.byref(a), C.byref(b)) == 2


def test_rope_launch_shape_report():
    """gpuk_rope_rms_launch_shape computes on the host which rope kernel a batch gets, its grid and whether the rotated
    rows are stored past the L2; no GPU is needed."""
    from gpuk_amd import capi
    # 4096 tokens x (32, 8, 8) heads of 128 with a 16-bit cache: the batch fits the chip in one round, one wave per token
    assert capi.rope_rms_launch_shape(4096, 32, 8, 8, 128) == (1024, 256, True, 1)
    # 4200 tokens do not: one wave per group of 8 Q/K heads, four waves a workgroup, streamed stores
    assert capi.rope_rms_launch_shape(4200, 32, 8, 8, 128) == (5250, 256, True, False)
    assert capi.rope_rms_launch_shape(4096, 32, 8, 8, 128, set_kv=False) == (1024, 256, True, 1)   # in place too
    assert capi.rope_rms_launch_shape(2048, 32, 8, 8, 128, set_kv=False) == (2560, 256, True, 0)
    # 8192 tokens of 28+4+4 heads: two tokens per wave, the second through LDS, still one round
    assert capi.rope_rms_launch_shape(8192, 28, 4, 4, 128, n_axes=3) == (1024, 256, True, 2)
    assert capi.rope_rms_launch_shape(8192, 28, 4, 4, 128, n_axes=3, set_kv=False) == (1024, 256, True, 2)
    assert capi.rope_rms_launch_shape(4096, 32, 8, 8, 128, kv_fp8=True) == (1024, 256, True, 1)
    assert capi.rope_rms_launch_shape(2560, 32, 8, 8, 128, kv_fp8=True) == (3200, 256, True, 0)   # an fp8 cache: later
    # a decode batch: through the L2; single waves unless a workgroup of four holds whole tokens
    assert capi.rope_rms_launch_shape(16, 28, 4, 4, 128) == (16, 256, False, False)
    assert capi.rope_rms_launch_shape(16, 40, 8, 8, 128, kv_fp8=True) == (96, 64, False, False)
    # fp32 activations: a wave per 512/D Q/K heads, and per 512 elements of the V row when a cache is written
    assert capi.rope_rms_launch_shape(10, 4, 2, 2, 64, dtype=torch.float32) == (5, 256, True, False)
    assert capi.rope_rms_launch_shape(10, 4, 2, 2, 64, dtype=torch.float32, set_kv=False) == (3, 256, True, False)
    assert capi.rope_rms_launch_shape(4, 7, 2, 3, 256, dtype=torch.float64) == (7, 256, True, False)
    import ctypes as C
    L = capi.lib()
    o = [C.c_int(0) for _ in range(4)]
    refs = [C.byref(x) for x in o]
    assert L.gpuk_rope_rms_launch_shape(0, 32, 8, 8, 128, 1, 0, 1, 0, *refs) == 1
    assert L.gpuk_rope_rms_launch_shape(4, 32, 8, 8, 96, 1, 0, 1, 0, *refs) == 2
    assert L.gpuk_rope_rms_launch_shape(4, 32, 8, 8, 128, 2, 0, 1, 0, *refs) == 1
    assert L.gpuk_rope_rms_launch_shape(4, 32, 8, 8, 128, 1, 0, 1, 0, None, *refs[1:]) == 1
    assert L.gpuk_rope_rms_launch_shape(4, 32, 8, 8, 128, 1, 9, 1, 0, *refs) == 2   # no such dtype
