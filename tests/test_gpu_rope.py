"""GPU parity: fused QK-RMSNorm + RoPE / mRoPE (+ paged KV-cache write) against the CPU restatement of
the reference's torch oracle on the same seeded inputs, through the C ABI and through the torch ops.

The shape sweep follows the reference's own test scripts (test/test_fused_rope_rms.py:196-217,
test/test_fused_mrope_rms_set_kv.py:274-307): NeoX and GPT-J style, odd token counts, head sizes
64/128/256 with mRoPE sections [12,10,10] / [24,20,20] / [48,40,40], chunked and interleaved, a random
cos/sin table, fp8 cache with k_scale 1.5 and v_scale 2.0 -- but with distinct cache slots, so the result
is deterministic.
"""
import pytest
import torch

from gpuk_amd import workloads
from oracle import c_oracle, torch_oracle as O
from tests.util import assert_bits_equal, assert_codes_close, assert_heads_explained, assert_rotated_close

pytestmark = pytest.mark.gpu

SECTIONS = {64: [12, 10, 10], 128: [24, 20, 20], 256: [48, 40, 40]}


def to_dev(inp, device):
    return [t.to(device) for t in (inp.qkv, inp.qw, inp.kw, inp.cos_sin, inp.positions, inp.kv_loc)]


def oracle_inplace(inp, rstd_ulp_offset=0):
    q, k, v = O.rope_rms_ref(inp.qkv, inp.qw, inp.kw, inp.cos_sin, inp.positions, inp.num_tokens, inp.num_heads_q,
                             inp.num_heads_k, inp.num_heads_v, inp.head_size, inp.is_neox, inp.eps,
                             inp.mrope_section, inp.is_interleaved, rstd_ulp_offset)
    return torch.cat([q, k, v], dim=1)


def check_inplace(inp, got, tag):
    """Q and K heads of the in-place result: each bit-identical to the oracle at an rstd within one ULP; V untouched."""
    nqk = inp.num_heads_q + inp.num_heads_k
    got = got.cpu()
    cache = {}

    def want_at(off):
        if off not in cache:
            cache[off] = oracle_inplace(inp, off)
        return cache[off]

    assert_heads_explained(got[:, :nqk], lambda off: want_at(off)[:, :nqk], f"{tag} q,k", inp.head_size)
    assert_bits_equal(got[:, nqk:], want_at(0)[:, nqk:], f"{tag} v")


def run_inplace(inp, device):
    from gpuk_amd import capi

    qkv, qw, kw, cs, pos, _ = to_dev(inp, device)
    capi.rope_rms(qkv, qw, kw, cs, pos, inp.num_tokens, inp.num_heads_q, inp.num_heads_k, inp.num_heads_v,
                  inp.head_size, inp.is_neox, inp.eps, inp.mrope_section, inp.is_interleaved)
    torch.cuda.synchronize()
    return qkv


def run_set_kv(inp, device, via_op=False):
    qkv, qw, kw, cs, pos, loc = to_dev(inp, device)
    k0, v0 = inp.new_cache()
    kc, vc = k0.to(device), v0.to(device)
    q_out = torch.empty((inp.num_tokens, inp.num_heads_q, inp.head_size), dtype=qkv.dtype, device=device)
    args = (qkv, qw, kw, cs, pos, inp.num_tokens, inp.num_heads_q, inp.num_heads_k, inp.num_heads_v, inp.head_size,
            inp.is_neox)
    if via_op:
        import gpuk_amd as gpuk

        if inp.mrope_section is not None:
            gpuk.fused_mrope_3d_rms_set_kv(*args, inp.mrope_section, inp.is_interleaved, inp.eps, q_out, kc, vc, loc,
                                           inp.k_scale, inp.v_scale)
        else:
            gpuk.fused_rope_rms_set_kv(*args, inp.eps, q_out, kc, vc, loc, inp.k_scale, inp.v_scale)
    else:
        from gpuk_amd import capi

        capi.rope_rms_set_kv(*args, inp.eps, q_out, kc, vc, loc, inp.k_scale, inp.v_scale, inp.mrope_section,
                             inp.is_interleaved)
    torch.cuda.synchronize()
    assert torch.equal(qkv.cpu(), inp.qkv), "set_kv must not modify qkv"
    return q_out, kc, vc, (k0, v0)


def oracle_set_kv(inp, k0, v0, rstd_ulp_offset=0):
    q_ref = torch.empty((inp.num_tokens, inp.num_heads_q, inp.head_size), dtype=inp.qkv.dtype)
    k_ref, v_ref = k0.clone(), v0.clone()
    O.rope_rms_set_kv_ref(inp.qkv, inp.qw, inp.kw, inp.cos_sin, inp.positions, inp.num_tokens, inp.num_heads_q,
                          inp.num_heads_k, inp.num_heads_v, inp.head_size, inp.is_neox, inp.eps, q_ref, k_ref, v_ref,
                          inp.kv_loc, inp.k_scale, inp.v_scale, inp.mrope_section, inp.is_interleaved,
                          rstd_ulp_offset=rstd_ulp_offset)
    return q_ref, k_ref, v_ref


def check_set_kv(inp, got, tag):
    """q_out and the K rows of the named slots (16-bit values or fp8 codes): every head bit-identical to the oracle at
    an rstd within one ULP.  V rows bit-identical.  Every slot no token names byte-identical to what it held."""
    q_out, kc, vc, (k0, v0) = got
    cache = {}

    def want_at(off):
        if off not in cache:
            cache[off] = oracle_set_kv(inp, k0, v0, off)
        return cache[off]

    kc, vc = kc.cpu(), vc.cpu()
    loc = inp.kv_loc[inp.kv_loc >= 0]
    found = assert_heads_explained(q_out, lambda off: want_at(off)[0], f"{tag} q_out", inp.head_size)
    assert_heads_explained(kc[loc], lambda off: want_at(off)[1][loc], f"{tag} k_cache", inp.head_size)
    v_ref = want_at(0)[2]
    assert_bits_equal(vc[loc].view(torch.uint8), v_ref[loc].view(torch.uint8), f"{tag} v_cache")
    untouched = torch.ones(inp.num_slots, dtype=torch.bool)
    untouched[loc] = False
    assert_bits_equal(kc[untouched].view(torch.uint8), k0[untouched].view(torch.uint8), f"{tag} untouched k slots")
    assert_bits_equal(vc[untouched].view(torch.uint8), v0[untouched].view(torch.uint8), f"{tag} untouched v slots")
    return found


def make(tokens, heads, head_size, neox, seed, mrope=False, interleaved=False, fp8=False, hk=None, hv=None):
    inp = workloads.rope_inputs(tokens, heads, heads if hk is None else hk, heads if hv is None else hv, head_size,
                                seed=seed, max_pos=10000, num_slots=max(2 * tokens, 64), is_neox=neox,
                                random_table=True,
                                kv_dtype=torch.float8_e4m3fn if fp8 else torch.bfloat16,
                                k_scale=1.5 if fp8 else 1.0, v_scale=2.0 if fp8 else 1.0)
    if mrope:
        g = torch.Generator().manual_seed(seed + 1)
        inp.positions = torch.randint(0, 10000, (3, tokens), generator=g, dtype=torch.int64)
        inp.mrope_section = SECTIONS[head_size]
        inp.is_interleaved = interleaved
    return inp


@pytest.mark.parametrize("neox", [True, False])
@pytest.mark.parametrize("tokens", [513, 127, 3])
@pytest.mark.parametrize("head_size", [64, 128, 256])
def test_rope_inplace_sweep(device, neox, tokens, head_size):
    print(f"case inplace neox={neox} T={tokens} D={head_size}", flush=True)
    inp = make(tokens, 32, head_size, neox, seed=tokens + head_size)
    got = run_inplace(inp, device)
    check_inplace(inp, got, "in place")


@pytest.mark.parametrize("neox", [True, False])
@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("head_size", [64, 128, 256])
def test_mrope_inplace_sweep(device, neox, interleaved, head_size):
    print(f"case mrope inplace neox={neox} il={interleaved} D={head_size}", flush=True)
    inp = make(257, 32, head_size, neox, seed=7 + head_size, mrope=True, interleaved=interleaved)
    got = run_inplace(inp, device)
    check_inplace(inp, got, "in place")


@pytest.mark.parametrize("neox", [True, False])
@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("head_size", [64, 128, 256])
@pytest.mark.parametrize("fp8", [True, False])
def test_mrope_set_kv_sweep(device, neox, interleaved, head_size, fp8):
    print(f"case mrope set_kv neox={neox} il={interleaved} D={head_size} fp8={fp8}", flush=True)
    inp = make(131, 32, head_size, neox, seed=17 + head_size, mrope=True, interleaved=interleaved, fp8=fp8)
    check_set_kv(inp, run_set_kv(inp, device), "[mrope set_kv]")


@pytest.mark.parametrize("hq,hk,hv", [(32, 8, 8), (28, 4, 4), (64, 8, 8), (5, 3, 2), (1, 1, 1), (40, 40, 40),
                                      (36, 0, 8), (13, 0, 3), (0, 13, 5), (0, 5, 2), (0, 16, 16)])
@pytest.mark.parametrize("fp8", [True, False])
def test_rope_set_kv_head_mixes(device, hq, hk, hv, fp8):
    """GQA head mixes, including counts that do not fill a wave's group of heads and calls without K heads or without
    Q heads (then the cache or q_out is an empty tensor)."""
    print(f"case set_kv heads={hq},{hk},{hv} fp8={fp8}", flush=True)
    inp = make(67, hq, 128, True, seed=hq * 100 + hk, fp8=fp8, hk=hk, hv=hv)
    check_set_kv(inp, run_set_kv(inp, device), f"[set_kv {hq},{hk},{hv}]")


ALIGNED_SECTIONS = {64: [8, 16, 8], 128: [16, 24, 24], 256: [48, 40, 40]}


@pytest.mark.parametrize("neox", [True, False])
@pytest.mark.parametrize("head_size", [64, 128, 256])
def test_mrope_sections_on_multiples_of_8(device, neox, head_size):
    """Chunked sections whose boundaries are multiples of 8: the 8 frequencies a lane owns then share one axis."""
    print(f"case aligned sections neox={neox} D={head_size}", flush=True)
    for fp8 in (False, True):
        inp = make(131, 12, head_size, neox, seed=head_size + 7, mrope=True, interleaved=False, fp8=fp8, hk=4, hv=4)
        inp.mrope_section = ALIGNED_SECTIONS[head_size]
        check_set_kv(inp, run_set_kv(inp, device), f"[aligned D={head_size} fp8={fp8}]")
        got = run_inplace(inp, device)
        check_inplace(inp, got, "in place")


@pytest.mark.parametrize("threads", [64, 128, 512])
def test_launch_shape_variants(device, threads):
    """The workgroup size is a tuning choice only: every setting gives the same bits as the oracle."""
    from gpuk_amd import capi

    print(f"case variants threads={threads}", flush=True)
    capi.set_tuning("rope_block_threads", threads)
    try:
        for hs, neox, mrope, fp8, heads in ((128, True, False, False, (32, 8, 8)), (64, False, True, True, (20, 20, 20)),
                                            (256, True, True, False, (9, 3, 3)), (128, False, False, True, (64, 8, 8))):
            inp = make(45, heads[0], hs, neox, seed=hs + threads, mrope=mrope, interleaved=mrope, fp8=fp8,
                       hk=heads[1], hv=heads[2])
            check_set_kv(inp, run_set_kv(inp, device), f"[variant D={hs}]")
            got = run_inplace(inp, device)
            check_inplace(inp, got, "in place")
    finally:
        capi.set_tuning("rope_block_threads", 0)


HEAD_MIX_CASES = [
    # tokens, (hq, hk, hv), head size, neox, mrope, interleaved, fp8
    (45, (32, 8, 8), 128, True, False, False, False),     # whole units of Q heads, one of K heads
    (61, (28, 4, 4), 128, True, True, False, False),      # a unit that mixes Q and K heads; three position axes
    (37, (20, 20, 20), 64, False, True, True, True),      # 16 heads per unit, GPT-J pairs, fp8 cache
    (29, (9, 3, 3), 256, True, True, True, False),        # 4 heads per unit, a partly filled last unit
    (33, (64, 8, 8), 128, False, False, False, True),     # nine units per token, GPT-J pairs, fp8 cache
    (19, (3, 2, 1), 128, True, False, False, False),      # a single, partly filled unit per token
    (23, (7, 2, 0), 128, True, False, False, False),      # no V heads
    (41, (28, 4, 4), 128, True, "aligned", False, False),  # sections on multiples of 8: the lanes load from their axis's row
    (27, (6, 2, 2), 64, False, "aligned", False, True),   # the same with GPT-J pairs, head size 64, fp8 cache
    (31, (36, 0, 8), 128, True, False, False, False),     # no K heads: the last unit holds Q lanes and idle lanes only
    (31, (13, 0, 3), 128, False, False, False, True),     # the same with an fp8 cache, GPT-J pairs
    (35, (21, 0, 5), 64, True, True, False, False),       # no K heads, 16 heads per unit, three position axes
    (31, (0, 13, 5), 128, True, False, False, False),     # no Q heads
    (29, (0, 5, 2), 128, False, True, True, True),        # no Q heads, fp8 cache, interleaved sections
]


@pytest.mark.parametrize("case", range(len(HEAD_MIX_CASES)))
@pytest.mark.parametrize("threads", [0, 64, 512])
def test_head_mixes_under_both_store_policies(device, case, threads):
    """Mixes of Q, K and V heads (units of one kind, mixed units, partly filled units, a kind that is absent), padding
    tokens, text tokens among mRoPE tokens: the oracle's bits with the output rows stored through the L2 and past it,
    which must also agree with each other bit for bit, whatever the workgroup size."""
    from gpuk_amd import capi

    tokens, heads, hs, neox, mrope, interleaved, fp8 = HEAD_MIX_CASES[case]
    print(f"case head mix {HEAD_MIX_CASES[case]} threads={threads}", flush=True)
    inp = make(tokens, heads[0], hs, neox, seed=900 + case, mrope=bool(mrope), interleaved=interleaved, fp8=fp8, hk=heads[1],
               hv=heads[2])
    if mrope == "aligned":
        inp.mrope_section = ALIGNED_SECTIONS[hs]
        inp.positions[:, ::3] = inp.positions[0, ::3]   # every third token a text token: three equal positions
    if case == 0:   # two padding tokens
        inp.kv_loc[3], inp.kv_loc[tokens - 1] = -1, -5
    capi.set_tuning("rope_block_threads", threads)
    try:
        capi.set_tuning("rope_stream_rows", 1)
        base_set = run_set_kv(inp, device)
        base_inplace = run_inplace(inp, device)
        capi.set_tuning("rope_stream_rows", 2)
        got_set = run_set_kv(inp, device)
        got_inplace = run_inplace(inp, device)
    finally:
        capi.set_tuning("rope_block_threads", 0)
        capi.set_tuning("rope_stream_rows", 0)
    raw = lambda t: t.cpu().contiguous().view(torch.uint8)
    for name, a, b in zip(("q_out", "k_cache", "v_cache"), got_set[:3], base_set[:3]):
        assert torch.equal(raw(a), raw(b)), f"{name}: the two store policies differ"
    assert torch.equal(raw(got_inplace), raw(base_inplace)), "in place: the two store policies differ"
    check_set_kv(inp, got_set, f"[head mix {case}]")
    check_inplace(inp, got_inplace, "in place")


TOKEN_WAVE_CASES = [
    # tokens, (hq, hk, hv), neox, fp8, fp16
    (45, (32, 8, 8), True, False, False),     # five units: four of Q heads, one of K heads
    (61, (28, 4, 4), True, False, False),     # four units, the last one mixes Q and K heads
    (37, (25, 7, 8), False, True, False),     # a mixed unit in the middle, GPT-J pairs, fp8 cache
    (31, (36, 0, 8), True, False, False),     # no K heads: the last unit holds Q lanes and idle lanes
    (29, (0, 33, 5), False, False, False),    # no Q heads, a partly filled last unit, an odd count of V heads
    (33, (32, 8, 8), False, True, True),      # fp16 activations, fp8 cache
    (300, (30, 3, 1), True, False, False),    # two rows of waves' worth of workgroups, one V head
]


@pytest.mark.parametrize("case", range(len(TOKEN_WAVE_CASES)))
@pytest.mark.parametrize("gate", [-1, 0, 700])
def test_one_wave_per_token_kernel(device, case, gate):
    """Batches of up to 4096 tokens (25-40 Q and K heads, one position axis, a cache) that the other kernel cannot hold
    in one round run a kernel in which a wave takes a whole token, asks for everything it reads at once and holds its stores back
    until the launch's reads are through.  Forced onto small batches here, with the gate it would compute, none, and a
    long one (7 us): the oracle's bits, and the same bits as the kernel with one wave per group of heads."""
    from gpuk_amd import capi

    tokens, heads, neox, fp8, fp16 = TOKEN_WAVE_CASES[case]
    print(f"case token waves {TOKEN_WAVE_CASES[case]} gate={gate}", flush=True)
    inp = make(tokens, heads[0], 128, neox, seed=400 + case, fp8=fp8, hk=heads[1], hv=heads[2])
    if fp16:
        inp.qkv, inp.qw, inp.kw, inp.cos_sin = (t.to(torch.float16) for t in (inp.qkv, inp.qw, inp.kw, inp.cos_sin))
        if not fp8:
            inp.kv_dtype = torch.float16
    inp.kv_loc[2], inp.kv_loc[tokens - 1] = -1, -7        # two padding tokens
    try:
        capi.set_tuning("rope_token_waves", 1)
        base = run_set_kv(inp, device)
        capi.set_tuning("rope_token_waves", 2)
        capi.set_tuning("rope_token_gate", gate)
        n_axes = 1
        groups, lanes, _, token_waves = capi.rope_rms_launch_shape(tokens, *heads, 128, n_axes, inp.qkv.dtype, True, fp8)
        assert token_waves and (groups, lanes) == ((tokens + 3) // 4, 256), "the case must reach the kernel under test"
        got = run_set_kv(inp, device)
    finally:
        capi.set_tuning("rope_token_waves", 0)
        capi.set_tuning("rope_token_gate", -1)
    raw = lambda t: t.cpu().contiguous().view(torch.uint8)
    for name, a, b in zip(("q_out", "k_cache", "v_cache"), got[:3], base[:3]):
        assert torch.equal(raw(a), raw(b)), f"{name}: the two kernels differ"
    check_set_kv(inp, got, f"[token waves {case}]")


@pytest.mark.parametrize("gate", [0, 1, 400])
def test_unit_kernel_store_gate_changes_no_bits(device, gate):
    """The kernel with one wave per group of heads holds its stores back, where all of its waves are resident at
    once, until the launch's reads are through.  Forced onto small batches: no gate, the shortest, 4 us -- the oracle's
    bits every time, with one and three position axes, a 16-bit and an fp8 cache, and in place."""
    from gpuk_amd import capi

    print(f"case unit kernel gate {gate}", flush=True)
    capi.set_tuning("rope_unit_gate", gate)
    capi.set_tuning("rope_token_waves", 1)
    try:
        for heads, mrope, fp8 in (((32, 8, 8), False, False), ((64, 8, 8), False, True), ((28, 4, 4), True, False)):
            inp = make(77, heads[0], 128, True, seed=31 + gate, mrope=mrope, fp8=fp8, hk=heads[1], hv=heads[2])
            check_set_kv(inp, run_set_kv(inp, device), f"[unit gate {gate} {heads}]")
            check_inplace(inp, run_inplace(inp, device), f"[unit gate {gate} {heads} in place]")
    finally:
        capi.set_tuning("rope_unit_gate", -1)
        capi.set_tuning("rope_token_waves", 0)


TOKEN_WAVE_CASES_2 = [
    # tokens, (hq, hk, hv), neox, sections (None: one position axis), two tokens per wave, fp16
    (61, (28, 4, 4), True, [16, 24, 24], False, False),    # three axes, four units
    (61, (28, 4, 4), False, [16, 24, 24], False, False),   # ... GPT-J pairs: a lane's two pieces may sit on two axes
    (45, (32, 8, 8), True, [8, 24, 32], False, False),     # three axes, five units
    (61, (28, 4, 4), True, None, True, False),             # two tokens per wave, an odd count: the last wave has one
    (62, (28, 4, 4), True, [16, 24, 24], True, False),     # two tokens per wave and three axes
    (37, (25, 7, 4), False, [32, 16, 16], True, False),    # a unit that mixes Q and K heads, GPT-J
    (300, (30, 2, 1), True, [16, 24, 24], True, False),    # several workgroups, one V head
    (33, (28, 4, 4), True, [16, 24, 24], True, True),      # fp16 activations
    (1, (28, 4, 4), True, [16, 24, 24], True, False),      # a single token: one wave, no second token
]


@pytest.mark.parametrize("case", range(len(TOKEN_WAVE_CASES_2)))
@pytest.mark.parametrize("gate", [-1, 700])
def test_token_kernel_three_axes_and_two_tokens_per_wave(device, case, gate):
    """The one-wave-per-token kernel with three position axes (sections that split at multiples of 8 frequencies: each
    lane reads its cos/sin pieces from its axis's row) and with a second token per wave, which travels through LDS:
    forced onto small batches, the oracle's bits and the same bits as the kernel with one wave per group of heads.
    Tokens without a slot sit in the first and in the second half of the batch."""
    from gpuk_amd import capi

    tokens, heads, neox, sections, two, fp16 = TOKEN_WAVE_CASES_2[case]
    print(f"case token waves (2) {TOKEN_WAVE_CASES_2[case]} gate={gate}", flush=True)
    inp = make(tokens, heads[0], 128, neox, seed=500 + case, mrope=sections is not None, hk=heads[1], hv=heads[2])
    if sections is not None:
        inp.mrope_section = sections
    if fp16:
        inp.qkv, inp.qw, inp.kw, inp.cos_sin = (t.to(torch.float16) for t in (inp.qkv, inp.qw, inp.kw, inp.cos_sin))
        inp.kv_dtype = torch.float16
    if tokens > 2:
        inp.kv_loc[2], inp.kv_loc[tokens - 1] = -1, -7
    n_axes = 3 if sections is not None else 1
    try:
        capi.set_tuning("rope_token_waves", 1)
        base = run_set_kv(inp, device)
        capi.set_tuning("rope_token_waves", 3 if two else 2)
        capi.set_tuning("rope_token_gate", gate)
        groups, lanes, _, token_waves = capi.rope_rms_launch_shape(tokens, *heads, 128, n_axes, inp.qkv.dtype, True, False)
        waves = (tokens + 1) // 2 if two else tokens
        assert token_waves == (2 if two else 1) and (groups, lanes) == ((waves + 3) // 4, 256), "the case must reach the kernel under test"
        got = run_set_kv(inp, device)
        # the in-place ops run the same kernel without the V row and the scatter
        assert capi.rope_rms_launch_shape(tokens, *heads, 128, n_axes, inp.qkv.dtype, False, False)[3] == (2 if two else 1)
        got_inplace = run_inplace(inp, device)
        capi.set_tuning("rope_token_waves", 1)
        base_inplace = run_inplace(inp, device)
    finally:
        capi.set_tuning("rope_token_waves", 0)
        capi.set_tuning("rope_token_gate", -1)
    raw = lambda t: t.cpu().contiguous().view(torch.uint8)
    for name, a, b in zip(("q_out", "k_cache", "v_cache"), got[:3], base[:3]):
        assert torch.equal(raw(a), raw(b)), f"{name}: the two kernels differ"
    assert torch.equal(raw(got_inplace), raw(base_inplace)), "in place: the two kernels differ"
    check_set_kv(inp, got, f"[token waves (2) {case}]")
    check_inplace(inp, got_inplace, f"[token waves (2) {case}, in place]")


def test_token_kernel_leaves_other_sections_to_the_other_kernel(device):
    """Sections that do not split at multiples of 8 frequencies, or the interleaved map, cannot take their cos/sin
    pieces from one row per lane: even when the one-wave-per-token kernel is asked for, such calls run the other one
    (and meet the oracle)."""
    from gpuk_amd import capi

    capi.set_tuning("rope_token_waves", 3)
    try:
        for sections, interleaved in (([24, 20, 20], False), ([16, 24, 24], True)):
            inp = make(50, 28, 128, True, seed=77, mrope=True, interleaved=interleaved, hk=4, hv=4)
            inp.mrope_section = sections
            check_set_kv(inp, run_set_kv(inp, device), f"[sections {sections} interleaved={interleaved}]")
    finally:
        capi.set_tuning("rope_token_waves", 0)


@pytest.mark.parametrize("seed", range(24))
def test_token_kernel_random_shapes(device, seed):
    """Seeded random shapes for the one-wave-per-token kernel, forced onto small batches: 25-40 Q and K heads in any
    split (also none of one kind), 1-8 V heads, NeoX or GPT-J, one axis or three (random sections that split at
    multiples of 8 frequencies), a 16-bit or fp8 cache, one or two tokens per wave, with a cache write and in place;
    the same bits as the kernel with one wave per group of heads every time, and the oracle's bits."""
    from gpuk_amd import capi

    g = torch.Generator().manual_seed(9000 + seed)
    rnd = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    two = bool(rnd(0, 1))
    heads_qk = rnd(25, 32) if two else rnd(25, 40)
    hq = rnd(0, heads_qk)
    hk = heads_qk - hq
    hv = rnd(1, 4) if two else rnd(1, 8)
    tokens = rnd(1, 700)
    neox = bool(rnd(0, 1))
    mrope = bool(rnd(0, 1))
    fp8 = (not mrope) and (not two) and bool(rnd(0, 1))
    print(f"case token fuzz seed={seed} T={tokens} heads=({hq},{hk},{hv}) neox={neox} mrope={mrope} fp8={fp8} two={two}", flush=True)
    inp = make(tokens, hq, 128, neox, seed=9100 + seed, mrope=mrope, fp8=fp8, hk=hk, hv=hv)
    if mrope:
        a = 8 * rnd(0, 8)
        b = 8 * rnd(0, (64 - a) // 8)
        inp.mrope_section = [a, b, 64 - a - b]
    if tokens > 3:
        inp.kv_loc[rnd(0, tokens - 1)] = -1
    n_axes = 3 if mrope else 1
    try:
        capi.set_tuning("rope_token_waves", 1)
        base, base_inplace = run_set_kv(inp, device), run_inplace(inp, device)
        capi.set_tuning("rope_token_waves", 3 if two else 2)
        assert capi.rope_rms_launch_shape(tokens, hq, hk, hv, 128, n_axes, inp.qkv.dtype, True, fp8)[3] == (2 if two else 1)
        got, got_inplace = run_set_kv(inp, device), run_inplace(inp, device)
    finally:
        capi.set_tuning("rope_token_waves", 0)
    raw = lambda t: t.cpu().contiguous().view(torch.uint8)
    for name, x, y in zip(("q_out", "k_cache", "v_cache"), got[:3], base[:3]):
        assert torch.equal(raw(x), raw(y)), f"{name}: the two kernels differ"
    assert torch.equal(raw(got_inplace), raw(base_inplace)), "in place: the two kernels differ"
    check_set_kv(inp, got, f"[token fuzz {seed}]")
    check_inplace(inp, got_inplace, f"[token fuzz {seed}, in place]")


@pytest.mark.parametrize("tokens", [2047, 2048, 4096, 4097, 4351, 4352, 4608, 5121, 6143, 7424, 8191, 8192])
def test_second_tokens_are_dealt_out_over_every_wave(device, tokens):
    """Between 4097 and 8192 tokens the kernel runs 4096 waves; wave 4 (cu + 256 l) + i takes, beside token w, one of
    the tokens from 4096 on according to its place (l, i) among the waves of compute unit cu.  Every token must be
    taken exactly once: the same bits as the kernel with one wave per group of heads, q_out and both caches (tokens
    without a slot among them), with three axes and in place as well.  (Below 4608 tokens the arrangement is forced;
    up to 4096 tokens that is half as many waves, which deal in the same way where they come to a multiple of 1024.)"""
    from gpuk_amd import capi

    for mrope in (False, True):
        print(f"case second tokens T={tokens} mrope={mrope}", flush=True)
        inp = make(tokens, 24, 128, True, seed=tokens, mrope=mrope, hk=8, hv=3)
        if mrope:
            inp.mrope_section = [16, 24, 24]
        inp.kv_loc[5::11] = -1
        n_axes = 3 if mrope else 1
        try:
            capi.set_tuning("rope_token_waves", 0 if tokens >= 4608 else 3)
            waves = 4096 if tokens > 4096 else (tokens + 1) // 2
            assert capi.rope_rms_launch_shape(tokens, 24, 8, 3, 128, n_axes, inp.qkv.dtype, True, False) == ((waves + 3) // 4, 256, True, 2)
            got, got_inplace = run_set_kv(inp, device), run_inplace(inp, device)
            capi.set_tuning("rope_token_waves", 1)
            base, base_inplace = run_set_kv(inp, device), run_inplace(inp, device)
        finally:
            capi.set_tuning("rope_token_waves", 0)
        raw = lambda t: t.cpu().contiguous().view(torch.uint8)
        for name, x, y in zip(("q_out", "k_cache", "v_cache"), got[:3], base[:3]):
            assert torch.equal(raw(x), raw(y)), f"{name}: the two kernels differ"
        assert torch.equal(raw(got_inplace), raw(base_inplace)), "in place: the two kernels differ"
    check_set_kv(inp, got, f"[second tokens T={tokens}]")


def test_one_wave_per_token_kernel_by_rule(device):
    """The launcher's rule takes that kernel where the other one is clearly past what it holds at once (from 10240
    groups of heads: 2560 tokens of 28+4+4 heads, not 2559) up to the 4096 tokens it holds itself, and from there to
    8192 tokens, once an eighth of them have a second token, with 4096 waves that take one token each and share out
    the rest (4608, 5000, 7169, 8192 tokens here, not 4607 or 8193); with one or three position axes; with an fp8
    cache one token per wave only.  Every choice meets the oracle."""
    from gpuk_amd import capi

    for tokens, mrope, fp8, expect in ((2559, False, False, 0), (2560, False, False, 1), (3500, True, False, 1),
                                       (4096, False, False, 1), (4607, False, False, 0), (4608, False, False, 2), (5000, True, False, 2),
                                       (6144, True, False, 2), (7169, False, False, 2), (8192, True, False, 2),
                                       (8192, False, False, 2), (8193, False, False, 0), (2500, False, True, 0),
                                       (4000, False, True, 1), (6144, False, True, 0)):
        groups, lanes, _, token_waves = capi.rope_rms_launch_shape(tokens, 28, 4, 4, 128, 3 if mrope else 1, torch.bfloat16, True, fp8)
        waves = 4096 if expect == 2 else tokens
        assert token_waves == expect and (not expect or (groups, lanes) == ((waves + 3) // 4, 256)), (tokens, fp8, groups, lanes)
        inp = make(tokens, 28, 128, True, seed=tokens + 1, mrope=mrope, fp8=fp8, hk=4, hv=4)
        if mrope:
            inp.mrope_section = [16, 24, 24]
        if expect == 2:
            inp.kv_loc[::7] = -1   # tokens without a slot among the first and the second tokens of the waves
        check_set_kv(inp, run_set_kv(inp, device), f"[rule T={tokens} mrope={mrope} fp8={fp8}]")
    # 32+8+8 heads: five groups per token, one token per wave only
    assert capi.rope_rms_launch_shape(4097, 32, 8, 8, 128)[3] == 0
    # in place the other kernel holds out a little longer (to 11468 groups of heads)
    for tokens, mrope, expect in ((2800, False, 0), (3000, True, 1), (4500, False, 0), (4700, False, 2), (7800, True, 2), (8192, True, 2)):
        assert capi.rope_rms_launch_shape(tokens, 28, 4, 4, 128, 3 if mrope else 1, torch.bfloat16, False, False)[3] == expect
        inp = make(tokens, 28, 128, True, seed=tokens + 2, mrope=mrope, hk=4, hv=4)
        if mrope:
            inp.mrope_section = [16, 24, 24]
        check_inplace(inp, run_inplace(inp, device), f"[rule, in place, T={tokens} mrope={mrope}]")


def test_batch_sizes_around_the_streaming_rule(device):
    """Batches below and above the size from which the output rows are stored past the L2 (8 MB per call), with one
    and three position axes, an fp8 cache, and more V heads than the waves of a token cover in one stride: all of
    them meet the oracle."""
    cases = ((3000, (32, 8, 8), False, False), (6100, (12, 4, 4), False, True), (4000, (12, 4, 4), True, False),
             (4000, (12, 4, 4), True, True), (300, (32, 8, 8), False, False), (20100, (4, 4, 10), False, False))
    for tokens, heads, fp8, mrope in cases:
        inp = make(tokens, heads[0], 128, True, seed=tokens, mrope=mrope, fp8=fp8, hk=heads[1], hv=heads[2])
        check_set_kv(inp, run_set_kv(inp, device), f"[T={tokens} heads={heads} fp8={fp8} mrope={mrope}]")
        check_inplace(inp, run_inplace(inp, device), f"[in place T={tokens} heads={heads} mrope={mrope}]")


@pytest.mark.parametrize("hq,hk,hv,head_size", [(3, 1, 40, 64), (1, 1, 17, 256), (7, 2, 0, 128), (2, 9, 33, 128)])
def test_value_heads_outnumber_the_waves(device, hq, hk, hv, head_size):
    """The V row is shared out over the waves that rotate Q and K; with few Q/K heads and many V heads each wave
    walks several strides of it, with none the V part is empty."""
    for fp8 in (False, True):
        inp = make(29, hq, head_size, True, seed=hv + head_size, fp8=fp8, hk=hk, hv=hv)
        check_set_kv(inp, run_set_kv(inp, device), f"[V-heavy {hq},{hk},{hv} D={head_size} fp8={fp8}]")


def test_config3_qwen3_like(device):
    inp = workloads.config3()
    check_set_kv(inp, run_set_kv(inp, device), "[C3]")


@pytest.mark.parametrize("interleaved", [False, True])
def test_config4_qwen2vl_like(device, interleaved):
    inp = workloads.config4(is_interleaved=interleaved)
    check_set_kv(inp, run_set_kv(inp, device), f"[C4 il={interleaved}]")


@pytest.mark.parametrize("tokens", workloads.DECODE_TOKENS)
def test_config5_decode_fp8_cache(device, tokens):
    inp = workloads.config5_rope(tokens)
    check_set_kv(inp, run_set_kv(inp, device), f"[C5 T={tokens}]")


def test_torch_ops(device):
    """The drop-in path: torch.ops.gpuk.* with the reference's argument order."""
    import gpuk_amd as gpuk

    inp = make(97, 16, 128, True, seed=5)
    qkv, qw, kw, cs, pos, _ = to_dev(inp, device)
    gpuk.fused_rope_rms(qkv, qw, kw, cs, pos, inp.num_tokens, 16, 16, 16, 128, True, inp.eps)
    torch.cuda.synchronize()
    check_inplace(inp, qkv, "op fused_rope_rms")

    inp = make(97, 16, 128, False, seed=6, mrope=True, interleaved=True)
    qkv, qw, kw, cs, pos, _ = to_dev(inp, device)
    gpuk.fused_mrope_3d_rms(qkv, qw, kw, cs, pos, inp.num_tokens, 16, 16, 16, 128, False, inp.mrope_section, True,
                            inp.eps)
    torch.cuda.synchronize()
    check_inplace(inp, qkv, "op fused_mrope_3d_rms")

    inp = make(97, 16, 128, True, seed=8, mrope=True, fp8=True)
    check_set_kv(inp, run_set_kv(inp, device, via_op=True), "[op mrope set_kv fp8]")
    inp = make(97, 16, 128, True, seed=9)
    check_set_kv(inp, run_set_kv(inp, device, via_op=True), "[op rope set_kv bf16]")


def test_strided_positions(device):
    """positions is passed by stride (src/ops/fused_rope.cpp:104,121-122): a [T,3] buffer viewed as [3,T]."""
    import gpuk_amd as gpuk

    inp = make(65, 8, 128, True, seed=12, mrope=True)
    pos_t = inp.positions.t().contiguous()          # [T,3] storage
    inp.positions = pos_t.t()                        # [3,T] view with strides (1,3)
    assert not inp.positions.is_contiguous()
    qkv, qw, kw, cs, _, _ = to_dev(inp, device)
    pos = pos_t.to(device).t()
    gpuk.fused_mrope_3d_rms(qkv, qw, kw, cs, pos, 65, 8, 8, 8, 128, True, inp.mrope_section, False, inp.eps)
    torch.cuda.synchronize()
    check_inplace(inp, qkv, "strided positions")


def test_equal_axes_equal_plain_rope(device):
    """mRoPE with three identical position rows selects the same table row everywhere: plain RoPE."""
    inp = make(50, 8, 128, True, seed=13)
    plain = run_inplace(inp, device)
    inp.positions = inp.positions.unsqueeze(0).expand(3, -1).contiguous()
    inp.mrope_section = [24, 20, 20]
    for il in (False, True):
        inp.is_interleaved = il
        assert_bits_equal(run_inplace(inp, device), plain, f"mrope(equal axes, il={il}) vs rope")


def test_fp16_activations(device):
    inp = workloads.rope_inputs(33, 8, 4, 4, 128, seed=14, max_pos=4096, num_slots=128, dtype=torch.float16,
                                random_table=True)
    check_inplace(inp, run_inplace(inp, device), "fp16")


def test_matches_c_checker(device):
    inp = make(40, 8, 128, False, seed=15, mrope=True, interleaved=True, fp8=True)
    q_out, kc, vc, (k0, v0) = run_set_kv(inp, device)
    q_ref = torch.empty_like(q_out, device="cpu")
    k_ref, v_ref = k0.clone(), v0.clone()
    c_oracle.rope_rms(inp.qkv.clone(), inp.qw, inp.kw, inp.cos_sin, inp.positions, 40, 8, 8, 8, 128, False, inp.eps,
                      inp.mrope_section, True, q_ref, k_ref.view(torch.uint8), v_ref.view(torch.uint8), inp.kv_loc,
                      inp.k_scale, inp.v_scale)
    assert_rotated_close(q_out, q_ref, "q vs C")
    assert_codes_close(kc.cpu(), k_ref, "k codes vs C")
    assert_bits_equal(vc.cpu().view(torch.uint8), v_ref.view(torch.uint8), "v codes vs C")


def test_op_rejects_bad_arguments(device):
    import gpuk_amd as gpuk

    inp = make(8, 4, 128, True, seed=16)
    qkv, qw, kw, cs, pos, _ = to_dev(inp, device)
    with pytest.raises(RuntimeError):   # 2-D positions for the 1-axis op (reference: TORCH_CHECK fused_rope.cpp:26)
        gpuk.fused_rope_rms(qkv, qw, kw, cs, pos.unsqueeze(0), 8, 4, 4, 4, 128, True, 1e-6)
    with pytest.raises(RuntimeError):   # sections must sum to head_size/2 (reference: assert rope_rms_impl.h:513)
        gpuk.fused_mrope_3d_rms(qkv, qw, kw, cs, pos.unsqueeze(0).expand(3, -1).contiguous(), 8, 4, 4, 4, 128, True,
                                [16, 16, 16], False, 1e-6)
    with pytest.raises(RuntimeError):   # unsupported head size (reference: assert rope_rms_impl.h:473)
        gpuk.fused_rope_rms(qkv, qw, kw, cs, pos, 8, 4, 4, 4, 96, True, 1e-6)


def test_fp8_cache_saturates_out_of_range_values(device):
    """With scales far too small most quotients exceed 448.  The kernel clips them to +-448, as the reference kernel
    clips at its maximum (src/impl/rope_rms_impl.h:109-118 -> float8.h), where torch's cast would give NaN above 464:
    expected codes = e4m3fn(clamp(rT(o / scale), +-448)) from the oracle's rotated K and raw V."""
    print("case fp8 cache saturation", flush=True)
    inp = make(40, 8, 128, True, seed=91, fp8=True, hk=4, hv=4)
    inp.k_scale, inp.v_scale = 1.0 / 512.0, 1.0 / 300.0
    q_out, kc, vc, (k0, v0) = run_set_kv(inp, device)
    q, k, v = O.rope_rms_ref(inp.qkv, inp.qw, inp.kw, inp.cos_sin, inp.positions, 40, 8, 4, 4, 128, True, inp.eps)
    want_k = (k / inp.k_scale).clamp(-448, 448).to(torch.float8_e4m3fn)
    want_v = (v / inp.v_scale).clamp(-448, 448).to(torch.float8_e4m3fn)
    got_k, got_v = kc.cpu()[inp.kv_loc], vc.cpu()[inp.kv_loc]
    assert ((want_k.view(torch.uint8) & 0x7F) == 0x7E).float().mean() > 0.3      # the test does saturate
    assert not ((got_k.view(torch.uint8) & 0x7F) == 0x7F).any() and not ((got_v.view(torch.uint8) & 0x7F) == 0x7F).any()
    assert_codes_close(got_k, want_k, "saturated k codes")
    assert_bits_equal(got_v.view(torch.uint8), want_v.view(torch.uint8), "saturated v codes")


@pytest.mark.parametrize("fp8", [False, True])
def test_negative_slots_and_colliding_slots(device, fp8):
    """kv_loc edge cases.  A negative slot (padding token) keeps q_out and drops the token's K and V rows; tokens that
    name the same slot race: every 8-element piece of the slot's rows comes whole from one of them."""
    print(f"case kv_loc edge cases fp8={fp8}", flush=True)
    inp = make(64, 8, 128, True, seed=123, fp8=fp8, hk=2, hv=2)
    loc = inp.kv_loc.clone()
    loc[5], loc[17], loc[63] = -1, -1, -7
    inp.kv_loc = loc
    check_set_kv(inp, run_set_kv(inp, device), "[padded tokens]")   # slots of the kept tokens only; the rest untouched

    raw = (lambda t: t.view(torch.uint8)) if fp8 else (lambda t: t.view(torch.int16))

    # collisions: tokens 0..7 all name slot 3
    inp2 = make(64, 8, 128, True, seed=124, fp8=fp8, hk=2, hv=2)
    loc2 = inp2.kv_loc.clone()
    taken = set(loc2[8:].tolist())
    shared = next(s for s in range(inp2.num_slots) if s not in taken)
    loc2[:8] = shared
    inp2.kv_loc = loc2
    q_out, kc, vc, (k0, v0) = run_set_kv(inp2, device)
    candidates_k, candidates_v = [], []
    for t in range(8):   # the row each colliding token would write, from the oracle run with that token alone on the slot
        k_one, v_one = k0.clone(), v0.clone()
        only = loc2.clone()
        only[:8] = -1
        only[t] = shared
        O.rope_rms_set_kv_ref(inp2.qkv, inp2.qw, inp2.kw, inp2.cos_sin, inp2.positions, 64, 8, 2, 2, 128, True, inp2.eps,
                              torch.empty_like(q_out, device="cpu"), k_one, v_one, only, inp2.k_scale, inp2.v_scale)
        candidates_k.append(k_one[shared])
        candidates_v.append(v_one[shared])
    # What the kernel guarantees for a shared slot: every 8-element piece (one lane's store: 16 bytes of a 16-bit
    # cache, 8 bytes of an fp8 cache) comes whole from one of the colliding tokens.  Different pieces of the row are
    # written by different store instructions and waves, so the row as a whole may mix tokens.
    got_v = raw(vc.cpu()[shared]).reshape(-1, 8)
    cand_v = torch.stack([raw(c).reshape(-1, 8) for c in candidates_v])            # [8 tokens, pieces, 8]
    v_from_a_token = (cand_v == got_v[None]).all(dim=-1).any(dim=0)
    assert bool(v_from_a_token.all()), f"V pieces not from any colliding token: {(~v_from_a_token).nonzero().flatten().tolist()}"
    got_k = kc.cpu()[shared].float().reshape(-1, 8)
    cand_k = torch.stack([c.float().reshape(-1, 8) for c in candidates_k])
    rtol = 0.13 if fp8 else 1e-2
    k_close = ((cand_k - got_k[None]).abs() <= 5e-2 + rtol * cand_k.abs()).all(dim=-1).any(dim=0)
    assert bool(k_close.all()), f"K pieces not from any colliding token: {(~k_close).nonzero().flatten().tolist()}"


@pytest.mark.parametrize("token_waves", [0, 2, 3])
def test_rope_kernel_replayed_from_a_graph(device, token_waves):
    """The mRoPE + KV-write op recorded into a HIP graph: every replay, with fresh inputs copied into the captured
    buffers and eager work in between, equals the eager call on the same inputs -- with the kernel the rule picks,
    and with the one-wave-per-token kernel forced, one and two tokens per wave (the latter holds data in LDS and
    both time their stores by the wall clock)."""
    import gpuk_amd as gpuk
    from gpuk_amd import capi

    capi.set_tuning("rope_token_waves", token_waves)
    T, hq, hk, hv, D = 300, 28, 4, 4, 128
    inp = make(T, hq, D, True, seed=71, mrope=True, hk=hk, hv=hv)
    inp.mrope_section = ALIGNED_SECTIONS[D]
    qkv, qw, kw, cs, pos, loc = to_dev(inp, device)
    k0, v0 = inp.new_cache()
    static_qkv, static_pos = torch.zeros_like(qkv), pos.clone()
    q_out = torch.empty((T, hq, D), dtype=qkv.dtype, device=device)
    kc, vc = k0.to(device), v0.to(device)

    def call(src, positions, q, k, v):
        gpuk.fused_mrope_3d_rms_set_kv(src, qw, kw, cs, positions, T, hq, hk, hv, D, True, inp.mrope_section, False,
                                       inp.eps, q, k, v, loc, 1.0, 1.0)

    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            call(static_qkv, static_pos, q_out, kc, vc)    # warm-up outside the capture
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            call(static_qkv, static_pos, q_out, kc, vc)
        for rep in range(4):
            g = torch.Generator(device=device).manual_seed(200 + rep)
            x = torch.randn(qkv.shape, device=device, generator=g).to(qkv.dtype)
            p = torch.randint(0, 10000, (3, T), device=device, generator=g, dtype=torch.int64)
            p[:, ::4] = p[0, ::4]                           # every fourth token a text token
            static_qkv.copy_(x)
            static_pos.copy_(p)
            graph.replay()
            torch.cuda.synchronize()
            q2, k2, v2 = torch.empty_like(q_out), k0.to(device), v0.to(device)
            call(x, p, q2, k2, v2)
            torch.cuda.synchronize()
            raw = lambda t: t.view(torch.int16)
            assert torch.equal(raw(q_out), raw(q2)), f"replay {rep}: q_out"
            assert torch.equal(raw(kc[loc]), raw(k2[loc])) and torch.equal(raw(vc[loc]), raw(v2[loc])), f"replay {rep}: cache rows"
    finally:
        torch.cuda.synchronize()
        capi.set_tuning("rope_token_waves", 0)
