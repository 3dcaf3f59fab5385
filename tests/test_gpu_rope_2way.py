"""GPU parity of fused_rope_rms_2way against the CPU restatement of the reference's torch code
(test/test_fused_rope_rms_2way.py:37-81).  Shapes follow the reference's script (:223-246): two streams of 678 and
3608 tokens, 24 query and 25 key heads, head sizes 64 and 128, both rotation styles, batch 1 and 2."""
import pytest
import torch

from oracle import c_oracle, torch_oracle as O
from tests.util import assert_heads_explained, assert_rotated_close

pytestmark = pytest.mark.gpu


def make(B, T0, T1, Hq, Hk, D, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g).to(dtype)
    return dict(q0=mk(B, T0, Hq, D), k0=mk(B, T0, Hk, D), q1=mk(B, T1, Hq, D), k1=mk(B, T1, Hk, D),
                w=[mk(D) for _ in range(4)], cs0=mk(T0, D), cs1=mk(T1, D))


def run_op(c, B, T0, T1, Hq, Hk, D, il, device):
    import gpuk_amd as gpuk

    d = lambda t: t.to(device)
    q01, k01 = gpuk.fused_rope_rms_2way(d(c["q0"]), d(c["k0"]), d(c["q1"]), d(c["k1"]), *[d(w) for w in c["w"]],
                                        d(c["cs0"]), d(c["cs1"]), B, T0, T1, Hq, Hk, D, il, 1e-6)
    torch.cuda.synchronize()
    return q01, k01


@pytest.mark.parametrize("il", [True, False])
@pytest.mark.parametrize("B", [1, 2])
@pytest.mark.parametrize("D", [64, 128])
def test_reference_shapes(device, il, B, D):
    print(f"case 2way il={il} B={B} D={D}", flush=True)
    T0, T1, Hq, Hk = 678, 3608, 24, 25
    c = make(B, T0, T1, Hq, Hk, D, seed=D + B)
    q01, k01 = run_op(c, B, T0, T1, Hq, Hk, D, il, device)
    cache = {}

    def want_at(off):
        if off not in cache:
            cache[off] = O.rope_rms_2way_ref(c["q0"], c["k0"], c["q1"], c["k1"], *c["w"], c["cs0"], c["cs1"], B, T0, T1,
                                             Hq, Hk, D, il, 1e-6, off)
        return cache[off]

    assert q01.shape == (B, T0 + T1, Hq, D) and k01.shape == (B, T0 + T1, Hk, D)
    assert_heads_explained(q01, lambda off: want_at(off)[0], "out_q01", D)
    assert_heads_explained(k01, lambda off: want_at(off)[1], "out_k01", D)


@pytest.mark.parametrize("B,T0,T1,Hq,Hk,D", [(1, 1, 1, 1, 1, 256), (3, 5, 0, 7, 3, 128), (2, 0, 9, 2, 11, 64),
                                             (1, 33, 17, 9, 1, 256), (4, 3, 2, 16, 8, 128)])
def test_ragged_and_empty_streams(device, B, T0, T1, Hq, Hk, D):
    """Head counts that do not fill a wave, a stream with no tokens, head size 256, through the C ABI."""
    from gpuk_amd import capi

    for il in (False, True):
        c = make(B, T0, T1, Hq, Hk, D, seed=T0 * 10 + T1)
        d = lambda t: t.to(device)
        q01 = torch.full((B, T0 + T1, Hq, D), 7.0, dtype=torch.bfloat16, device=device)
        k01 = torch.full((B, T0 + T1, Hk, D), 7.0, dtype=torch.bfloat16, device=device)
        capi.rope_rms_2way(d(c["q0"]), d(c["k0"]), d(c["q1"]), d(c["k1"]), *[d(w) for w in c["w"]], d(c["cs0"]),
                           d(c["cs1"]), B, T0, T1, Hq, Hk, D, il, 1e-6, q01, k01)
        torch.cuda.synchronize()
        q_ref, k_ref = c_oracle.rope_rms_2way(c["q0"], c["k0"], c["q1"], c["k1"], *c["w"], c["cs0"], c["cs1"], B, T0, T1,
                                              Hq, Hk, D, il, 1e-6)
        assert_rotated_close(q01, q_ref, f"out_q01 il={il}")
        assert_rotated_close(k01, k_ref, f"out_k01 il={il}")


def test_fp16_and_rejections(device):
    import gpuk_amd as gpuk

    B, T0, T1, Hq, Hk, D = 2, 6, 4, 3, 2, 128
    c = make(B, T0, T1, Hq, Hk, D, seed=3, dtype=torch.float16)
    q01, k01 = run_op(c, B, T0, T1, Hq, Hk, D, False, device)
    want_at = lambda off: O.rope_rms_2way_ref(c["q0"], c["k0"], c["q1"], c["k1"], *c["w"], c["cs0"], c["cs1"], B, T0, T1, Hq,
                                              Hk, D, False, 1e-6, off)
    assert_heads_explained(q01, lambda off: want_at(off)[0], "fp16 q01", D)
    assert_heads_explained(k01, lambda off: want_at(off)[1], "fp16 k01", D)
    d = lambda t: t.to(device)
    with pytest.raises(RuntimeError):   # token count that does not match the tensors
        gpuk.fused_rope_rms_2way(d(c["q0"]), d(c["k0"]), d(c["q1"]), d(c["k1"]), *[d(w) for w in c["w"]], d(c["cs0"]),
                                 d(c["cs1"]), B, T0 + 1, T1, Hq, Hk, D, False, 1e-6)
    with pytest.raises(RuntimeError):   # non-contiguous input (reference: TORCH_CHECK fused_rope.cpp:175)
        gpuk.fused_rope_rms_2way(d(c["q0"]).transpose(1, 2), d(c["k0"]), d(c["q1"]), d(c["k1"]), *[d(w) for w in c["w"]],
                                 d(c["cs0"]), d(c["cs1"]), B, T0, T1, Hq, Hk, D, False, 1e-6)
