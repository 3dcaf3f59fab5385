"""Pins the scalar number formats of the CPU checkers against torch-CPU library routines and the
committed exhaustive table: bf16 / fp16 round-to-nearest-even, OCP e4m3fn encode and decode."""
import os

import numpy as np
import torch

from oracle import c_oracle

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def test_e4m3fn_table_is_exhaustive_and_matches_c_encoder():
    table = np.fromfile(os.path.join(GOLD, "e4m3fn_from_bf16.bin"), dtype=np.uint8)
    assert table.shape == (65536,)
    mine = c_oracle.e4m3fn_table_bf16().numpy()
    bad = np.nonzero(table != mine)[0]
    assert bad.size == 0, f"first mismatching bf16 patterns: {[hex(int(b)) for b in bad[:8]]}"


def test_e4m3fn_table_matches_live_torch():
    """The fixture is what this torch build produces (guards against a stale fixture)."""
    table = np.fromfile(os.path.join(GOLD, "e4m3fn_from_bf16.bin"), dtype=np.uint8)
    allbf = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    live = allbf.float().to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert (live == table).all()


def test_e4m3fn_known_answers():
    """Values the format definition fixes: max 448 = 0x7e, min normal 2^-6 = 0x08, min subnormal 2^-9 = 0x01,
    the tie 2^-10 rounds to even (0), 464 is the tie between 448 and the NaN slot and rounds to 448,
    anything past it is NaN under torch's cast; 240 (the reference's max_value) = 0x77."""
    L = c_oracle.lib()
    enc = L.gpuk_oracle_f32_to_e4m3fn
    assert enc(448.0) == 0x7E and enc(-448.0) == 0xFE
    assert enc(240.0) == 0x77
    assert enc(2.0 ** -6) == 0x08 and enc(2.0 ** -9) == 0x01
    assert enc(2.0 ** -10) == 0x00 and enc(1.5 * 2.0 ** -9) == 0x02   # ties to even
    assert enc(464.0) == 0x7E and enc(465.0) == 0x7F
    assert enc(1.0) == 0x38 and enc(1.0625) == 0x38 and enc(1.1875) == 0x3A  # ties at 1+1/16, 1+3/16
    assert enc(0.0) == 0x00 and enc(-0.0) == 0x80
    dec = L.gpuk_oracle_e4m3fn_to_f32
    for c in range(256):
        if (c & 0x7F) == 0x7F:
            continue
        v = dec(c)
        assert enc(v) == c, hex(c)
        assert v == torch.tensor([c], dtype=torch.uint8).view(torch.float8_e4m3fn).float().item()


def test_e4m3fn_encoder_on_random_fp32_matches_torch():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(200000, generator=g) * torch.exp(torch.randn(200000, generator=g) * 3)).float()
    x = x[x.abs() < 460]
    want = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    enc = c_oracle.lib().gpuk_oracle_f32_to_e4m3fn
    got = np.array([enc(float(v)) for v in x[:20000].tolist()], dtype=np.uint8)
    assert (got == want[:20000]).all()


def test_bf16_and_fp16_rounding_match_torch():
    z = np.load(os.path.join(GOLD, "bf16_round_cases.npz"))
    f = torch.from_numpy(z["fp32_bits"]).view(torch.float32)
    # the fixture agrees with the live casts
    assert (f.to(torch.bfloat16).view(torch.int16).numpy() == z["bf16_bits"]).all()
    assert (f.to(torch.float16).view(torch.int16).numpy() == z["fp16_bits"]).all()
    L = c_oracle.lib()
    vals = f.tolist()
    got_bf = np.array([L.gpuk_oracle_f32_to_bf16(v) for v in vals], dtype=np.uint16).view(np.int16)
    got_h = np.array([L.gpuk_oracle_f32_to_fp16(v) for v in vals], dtype=np.uint16).view(np.int16)
    assert (got_bf == z["bf16_bits"]).all()
    assert (got_h == z["fp16_bits"]).all()


def test_fp16_decode_all_patterns():
    L = c_oracle.lib()
    allh = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    want = allh.float()
    for i in list(range(0, 65536, 97)) + [0, 1, 0x3FF, 0x400, 0x7BFF, 0x8001, 0xFBFF]:
        w = want[i].item()
        if w != w:
            continue
        assert L.gpuk_oracle_fp16_to_f32(i) == w, hex(i)
