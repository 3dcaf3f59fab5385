"""Where the time goes inside a wave: reads the phase stamps of the profiling build (libgpuk_amd_stamps.so, built by
`python -m gpuk_amd.build --stamps`), in which every wave of the kernels records the shader clock at named points, the
100 MHz wall clock at its entry and exit, and its place on the chip.

    python -m gpuk_amd.stamps norm_quant [--tokens 1 128 512] [--hidden 7168]
    python -m gpuk_amd.stamps rope [--config c3|c4|c5] [--tokens N]

Prints, per phase, how long the waves of one launch spent in it (ns: median, 10th and 90th percentile over waves;
cycles are turned into ns with each launch's own ratio of wall-clock ticks to cycles), when waves start, first store
and end relative to the first wave's entry, and the launch's span.  The stamps cost each wave about a dozen scalar
clock reads and two full waits for its memory operations, so the span printed here is a little above the product
build's; the product build contains none of this.

The reference times whole calls only (test/cpp/test_small_kernel.cpp:98-178, aiter's perftest in test/*.py).
"""
from __future__ import annotations

import argparse
import ctypes as C
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from gpuk_amd import capi, workloads  # noqa: E402

SLOTS = 16   # kStampSlots of csrc/kernels/device_utils.h: 13 clock readings, wall clock at entry and exit, place
STAMPS_LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libgpuk_amd_stamps.so")

NORM_QUANT_PHASES = [
    (0, 1, "entry -> every load issued (addresses formed from the arguments the wave finds in its registers)"),
    (1, 2, "-> loads landed (memory latency)"),
    (2, 3, "-> phase 1: residual summed, rounded, stored; the lane's squares summed"),
    (3, 4, "-> sum of squares reduced over the workgroup (DPP, LDS, one barrier)"),
    (4, 5, "-> rstd (mean, square root and reciprocal, each correctly rounded)"),
    (5, 6, "-> phase 2: row normed (two roundings per element), the lane's maximum"),
    (6, 7, "-> row maximum reduced over the workgroup (DPP, LDS, one barrier)"),
    (7, 8, "-> scale and its reciprocal (two correctly rounded quotients)"),
    (8, 9, "-> phase 3: quotients, fp8 codes, stores issued"),
    (9, 10, "-> every store acknowledged"),
]
ROPE_UNIT_PHASES = [
    (0, 1, "entry -> activations and position requested, position and argument block arrived, weights and slot requested"),
    (1, 2, "-> cos/sin requested"),
    (2, 3, "-> everything landed"),
    (3, 4, "-> norm, rotation, rows stored (issued)"),
    (4, 5, "-> every store acknowledged"),
]

def bind():
    if not os.path.exists(STAMPS_LIB):
        raise SystemExit(f"{STAMPS_LIB} not built; run `python -m gpuk_amd.build --stamps`")
    capi.use_library(STAMPS_LIB)
    L = capi.lib()
    for name in ("gpuk_stamps_set_norm_quant", "gpuk_stamps_set_rope"):
        getattr(L, name).restype = C.c_int
        getattr(L, name).argtypes = [C.c_void_p, C.c_uint32]
    return L


def summarize(buf: torch.Tensor, phases, title: str):
    """buf: [waves, SLOTS] int64 on the host, rows of waves that ran."""
    d = buf[buf[:, SLOTS - 3] != 0]
    waves = d.shape[0]
    wall0, wall1 = d[:, SLOTS - 3], d[:, SLOTS - 2]
    t = d[:, :SLOTS - 3]
    last = torch.where(t != 0, torch.arange(SLOTS - 3).expand_as(t), torch.zeros_like(t)).max(dim=1).values
    t_last = t.gather(1, last[:, None]).squeeze(1)
    cyc = (t_last - t[:, 0]).double()
    ticks = (wall1 - wall0).double()      # 10 ns each
    # the shader clock in units of the stamps: one ratio for the launch, from the waves that ran longest
    long = ticks >= ticks.quantile(0.5)
    ns_per_cycle = float((ticks[long] * 10.0).sum() / cyc[long].sum())
    base = wall0.min()
    print(f"== {title}: {waves} waves; shader clock {1.0 / ns_per_cycle:.2f} counts per ns; "
          f"launch span {float(wall1.max() - base) * 0.01:.2f} us "
          f"(entry of the first wave to the last acknowledged store of the last)")
    q = lambda v, p: float(v.quantile(p))
    print(f"   wave entry after the first wave's   : median {q((wall0 - base).double(), .5) * .01:6.2f} us, "
          f"p90 {q((wall0 - base).double(), .9) * .01:6.2f}, last {float((wall0 - base).max()) * .01:6.2f}")
    print(f"   wave exit  after the first wave's entry: p10 {q((wall1 - base).double(), .1) * .01:6.2f} us, median "
          f"{q((wall1 - base).double(), .5) * .01:6.2f}, p90 {q((wall1 - base).double(), .9) * .01:6.2f}, "
          f"last {float((wall1 - base).max()) * .01:6.2f}")
    print(f"   wave lifetime                          : median {q(ticks, .5) * .01:6.2f} us, p10 {q(ticks, .1) * .01:6.2f}, "
          f"p90 {q(ticks, .9) * .01:6.2f}")
    total = 0.0
    for a, b, name in phases:
        ok = (t[:, a] != 0) & (t[:, b] != 0)
        dur = (t[ok, b] - t[ok, a]).double() * ns_per_cycle
        if dur.numel() == 0:
            continue
        total += q(dur, .5)
        print(f"   {q(dur, .5):8.0f} ns  (p10 {q(dur, .1):7.0f}, p90 {q(dur, .9):7.0f}; {dur.numel():6d} waves)  {name}")
    print(f"   {total:8.0f} ns  sum of the medians")
    # by XCD: do some parts of the chip finish later than others?
    place = d[:, SLOTS - 1]
    xcc = (place >> 32) & 0xF
    ends = (wall1 - base).double() * 0.01
    per = [f"{int(x)}: {float(ends[xcc == x].median()):.2f}/{float(ends[xcc == x].max()):.2f}" for x in xcc.unique().tolist()]
    print("   exit by XCD (median/last, us): " + "  ".join(per))
    return ns_per_cycle


def run_norm_quant(L, tokens_list, hidden, quant):
    dev = torch.device("cuda:0")
    for T in tokens_list:
        inp = workloads.norm_quant_inputs(T, hidden, seed=T, res_sigma=1.0)
        lanes, chunks = capi.add_rmsnorm_quant_launch_shape(T, hidden, torch.bfloat16)
        waves = T * (lanes // 64)
        buf = torch.zeros((waves, SLOTS), dtype=torch.int64, device=dev)
        assert L.gpuk_stamps_set_norm_quant(buf.data_ptr(), waves) == 0
        g = inp.gamma.to(dev)
        sets = [(inp.x.to(dev).clone(), inp.residual.to(dev).clone(), torch.empty((T, hidden), dtype=torch.bfloat16, device=dev),
                 torch.empty((T, hidden), dtype=torch.float8_e4m3fn if quant else torch.bfloat16, device=dev),
                 torch.empty((T, 1), dtype=torch.float32, device=dev)) for _ in range(8)]
        for rep in range(24):      # the last launch's stamps are the ones read; the others warm clocks and caches
            x, r, ro, no, sc = sets[rep % 8]
            if rep == 23:
                torch.cuda.synchronize()
                buf.zero_()
                torch.cuda.synchronize()
            capi.add_rmsnorm_quant(x, r, g, ro, no, sc, inp.eps, quant)
        torch.cuda.synchronize()
        summarize(buf.cpu(), NORM_QUANT_PHASES,
                  f"add_rmsnorm_quant_rows, {T} x {hidden} bf16, quant {quant}, {lanes} lanes x {chunks} chunks")
        assert L.gpuk_stamps_set_norm_quant(None, 0) == 0


def run_rope(L, config, tokens):
    dev = torch.device("cuda:0")
    if config == "c3":
        r = workloads.config3(num_tokens=tokens) if tokens else workloads.config3()
    elif config == "c4":
        r = workloads.config4(num_tokens=tokens) if tokens else workloads.config4()
    else:
        r = workloads.config5_rope(tokens or 128)
    T = r.num_tokens
    n_axes = 3 if r.mrope_section is not None else 1
    capi.set_tuning("rope_token_waves", 1)   # the stamps are in the kernel with one wave per group of heads
    groups, lanes, streamed, _ = capi.rope_rms_launch_shape(T, r.num_heads_q, r.num_heads_k, r.num_heads_v, r.head_size,
                                                                  n_axes, torch.bfloat16, True, r.kv_dtype == torch.float8_e4m3fn)
    waves = groups * (lanes // 64)
    buf = torch.zeros((waves, SLOTS), dtype=torch.int64, device=dev)
    assert L.gpuk_stamps_set_rope(buf.data_ptr(), waves) == 0
    k0, v0 = r.new_cache()
    qw, kw, cs, pos, loc = (t.to(dev) for t in (r.qw, r.kw, r.cos_sin, r.positions, r.kv_loc))
    sets = [(r.qkv.to(dev).clone(), torch.empty((T, r.num_heads_q, r.head_size), dtype=torch.bfloat16, device=dev),
             k0.to(dev), v0.to(dev)) for _ in range(4)]
    for rep in range(24):
        qkv, q_out, kc, vc = sets[rep % 4]
        if rep == 23:
            torch.cuda.synchronize()
            buf.zero_()
            torch.cuda.synchronize()
        capi.rope_rms_set_kv(qkv, qw, kw, cs, pos, T, r.num_heads_q, r.num_heads_k, r.num_heads_v, r.head_size, r.is_neox,
                             r.eps, q_out, kc, vc, loc, r.k_scale, r.v_scale, r.mrope_section, r.is_interleaved)
    torch.cuda.synchronize()
    title = (f"rope_rms_kernel, {config} T={T} heads {r.num_heads_q}/{r.num_heads_k}/{r.num_heads_v}, "
             f"{groups} workgroups x {lanes} lanes, rows stored {'past' if streamed else 'through'} the L2")
    summarize(buf.cpu(), ROPE_UNIT_PHASES, title)
    assert L.gpuk_stamps_set_rope(None, 0) == 0
    capi.set_tuning("rope_token_waves", 0)


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    sub = ap.add_subparsers(dest="what", required=True)
    nq = sub.add_parser("norm_quant")
    nq.add_argument("--tokens", type=int, nargs="+", default=[1, 128, 512])
    nq.add_argument("--hidden", type=int, default=7168)
    nq.add_argument("--quant", type=int, default=1, choices=[0, 1, 3])
    rp = sub.add_parser("rope")
    rp.add_argument("--config", choices=["c3", "c4", "c5"], default="c3")
    rp.add_argument("--tokens", type=int, default=0)
    args = ap.parse_args()
    assert torch.cuda.is_available(), "needs a GPU"
    L = bind()
    if args.what == "norm_quant":
        if args.quant == 3:
            raise SystemExit("static scale: pass a scale through the library's own entry point; not wired here")
        run_norm_quant(L, args.tokens, args.hidden, args.quant)
    else:
        run_rope(L, args.config, args.tokens)


if __name__ == "__main__":
    main()
