#!/usr/bin/env python3
"""Benchmark of the fused residual-add + RMSNorm + per-token FP8 quant path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

A step is one call of `torch.ops.gpuk.allreduce_rms` (quant_type 1, no all-reduce) over one 8192 x 8192
bf16 batch with 1 % +-50 outliers, inputs resident in HBM.  Buffers rotate over three distinct sets so no
cache can serve a repeat.  Prints ONE JSON line:

  value      achieved HBM GB/s over the K timed steps = algorithmic bytes (7*T*H + 4*T + 2*H) / wall time
  roofline   the same kernel timed per launch with HIP events on the launch stream, against 8 TB/s
  cpu_baseline  the restated torch reference on the host's cores on the same batch (at least 3 calls, about 10 s);
             where oracle/_ref was built, also the reference's own kernels timed on this GPU beside this repository's
  extras     secondary figures: copy-kernel ceiling, the fused kernel's traffic without its arithmetic, the RoPE +
             KV-write kernel on its two configurations with a plain copy of the same bytes beside each, decode-shape
             latencies (us/call)
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--prewarm-ms", type=float, default=40.0,
                    help="untimed run of the same step before the warmup steps, so that the GPU clocks have settled")
    ap.add_argument("--tokens", type=int, default=8192)
    ap.add_argument("--hidden", type=int, default=8192)
    ap.add_argument("--no-extras", action="store_true", help="skip the secondary measurements")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-rows", type=int, default=0, help="rows of the batch the CPU baseline runs on (0 = all of them)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU time budget of the baseline leg (at least 3 calls are made)")
    return ap.parse_args()


def settle_clocks(fn, ms=30.0):
    """Runs fn(i) untimed for `ms` milliseconds: after an idle spell (the CPU leg, buffer set-up) the GPU's clocks take
    some tens of milliseconds to come back up, which a short timed loop would otherwise measure."""
    import torch

    t0, n = time.perf_counter(), 0
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(10):
            fn(n)
            n += 1
        torch.cuda.synchronize()


def event_time_ms(fn, iters, warmup=3, settle_ms=30.0):
    """Average duration of fn() in ms from HIP events on the current stream (where fn launches)."""
    import torch

    if settle_ms > 0:
        settle_clocks(fn, settle_ms)
    for _ in range(warmup):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for i in range(iters):
        fn(i)
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def per_launch_ms(fn, iters):
    """Per-launch durations: one event pair around every launch, averaged."""
    import torch

    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(evs):
        a.record()
        fn(i)
        b.record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in evs)
    return sum(ts) / len(ts), ts[len(ts) // 2], ts[0]


def graph_time_us(call, n_in_graph=20, replays=30):
    """us per call with n_in_graph calls recorded into one HIP graph (call(i) must launch on the current stream and
    allocate nothing): the GPU-side cost of a call without the host's per-launch overhead."""
    import torch

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(n_in_graph):
            call(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(n_in_graph):
            call(i)
    settle_clocks(lambda i: g.replay(), 20.0)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(replays):
        g.replay()
    b.record()
    b.synchronize()
    return a.elapsed_time(b) * 1e3 / (replays * n_in_graph)


def traffic_from_profile(name):
    """HBM bytes per launch measured with rocprofv3 counters, if a summary for this workload is committed."""
    path = os.path.join(ROOT, "profiles", name)
    if not os.path.exists(path):
        return None
    m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", open(path).read(), re.M)
    return float(m.group(1)) if m else None


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this benchmark is a single-GPU kernel measurement; --gpus {args.gpus} is not supported "
              "(rows shard trivially across GPUs, no collective is involved)", file=sys.stderr)
        sys.exit(2)

    import torch

    import gpuk_amd as gpuk
    from gpuk_amd import capi, workloads

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    T, H = args.tokens, args.hidden

    # ------------------------------------------------------------------ primary: add + RMSNorm + per-token fp8
    inp = workloads.config2(T, H)
    NSETS = 3
    sets = []
    for s in range(NSETS):
        x = inp.x.to(dev) if s == 0 else torch.roll(sets[0][0], shifts=s, dims=0).contiguous()
        r = inp.residual.to(dev) if s == 0 else torch.roll(sets[0][1], shifts=s, dims=0).contiguous()
        sets.append((x, r, torch.empty_like(x), torch.empty((T, H), dtype=torch.float8_e4m3fn, device=dev),
                     torch.empty((T, 1), dtype=torch.float32, device=dev)))
    gamma = inp.gamma.to(dev)
    eps = inp.eps
    alg_bytes = workloads.norm_quant_bytes(T, H, quant=1)

    def step(i=0):
        x, r, ro, codes, sc = sets[i % NSETS]
        gpuk.allreduce_rms(0, x, r, gamma, ro, codes, sc, eps, gpuk.QUANT_FP8_DYNAMIC)

    # the clocks of an idle GPU take some tens of milliseconds to settle: run the step untimed first
    t_pre = time.perf_counter()
    n_pre = 0
    while (time.perf_counter() - t_pre) * 1e3 < args.prewarm_ms:
        for i in range(20):
            step(n_pre + i)
        n_pre += 20
        torch.cuda.synchronize()
    for i in range(args.warmup):
        step(i)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record()
    for i in range(args.steps):
        step(i)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    value = alg_bytes / (wall / args.steps) / 1e9

    # average launch duration of the kernel: HIP events on the launch stream around the same K back-to-back launches
    avg_ms = ev0.elapsed_time(ev1) / args.steps
    _, med_ms, min_ms = per_launch_ms(step, min(args.steps, 200))
    achieved = alg_bytes / (avg_ms * 1e-3) / 1e9
    lanes, chunks = capi.add_rmsnorm_quant_launch_shape(T, H, torch.bfloat16)
    profiled = (T, H) == (8192, 8192)   # the counter runs behind the committed traffic figure used this shape
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "traffic": traffic_from_profile("add_rmsnorm_quant_8192x8192.md") if profiled else None,
                "kernel": (f"add_rmsnorm_quant_rows<BF16, {chunks} chunks/lane, dynamic> ({T} workgroups x {lanes} lanes)"
                           if chunks else f"add_rmsnorm_quant_long_rows<BF16, dynamic> ({T} workgroups x {lanes} lanes)"),
                "avg_launch_us": round(avg_ms * 1e3, 2),
                "single_launch_median_us": round(med_ms * 1e3, 2), "single_launch_min_us": round(min_ms * 1e3, 2),
                "algorithmic_bytes": alg_bytes}

    # ------------------------------------------------------------------ CPU baseline (bounded sample)
    cpu_baseline = None
    if not args.no_cpu:
        from oracle import torch_oracle as O

        rows = min(args.cpu_rows, T) if args.cpu_rows > 0 else T
        ncores = os.cpu_count() or 1
        threads = int(os.environ.get("OMP_NUM_THREADS", ncores))
        torch.set_num_threads(threads)
        xs, rs = inp.x[:rows], inp.residual[:rows]
        O.add_rmsnorm_quant_ref(xs, rs, inp.gamma, eps, O.QUANT_DYNAMIC)
        times = []
        t_start = time.perf_counter()
        while len(times) < 3 or (time.perf_counter() - t_start < args.cpu_seconds and len(times) < 200):
            t0 = time.perf_counter()
            O.add_rmsnorm_quant_ref(xs, rs, inp.gamma, eps, O.QUANT_DYNAMIC)
            times.append(time.perf_counter() - t0)
        t_med = sorted(times)[len(times) // 2]
        cpu_baseline = {"value": round(workloads.norm_quant_bytes(rows, H, 1) / t_med / 1e9, 3), "unit": "GB/s",
                        "cores": torch.get_num_threads(), "kind": "port",
                        "sample": f"restated torch reference (oracle/torch_oracle.py) on CPU tensors, "
                                  f"{'all' if rows == T else 'first ' + str(rows) + ' of'} {T} "
                                  f"rows x {H}, median of {len(times)} calls over {time.perf_counter() - t_start:.1f} s "
                                  f"({t_med * 1e3:.0f} ms/call); host reports {ncores} cpus"}

        # Second baseline, same leg: the reference repository's own kernels (oracle/_ref, built from the reference's
        # headers where a checkout exists) timed on this GPU on the same inputs and buffer rotation.  For the norm-quant
        # path that is the reference's epilogue device code under a one-GPU caller (its kernels need 2+ GPUs), with the
        # reference's fp8 maximum of 240; for the rope path it is the reference's kernel as the reference launches it.
        from oracle import ref_kernels

        if ref_kernels.available():
            ref = {}

            def ref_norm_quant_us(tokens, hidden):
                d = workloads.config2(tokens, hidden)
                g_ = d.gamma.to(dev)
                bufs = [(d.x.to(dev), d.residual.to(dev), torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev),
                         torch.empty((tokens, hidden), dtype=torch.float8_e4m3fn, device=dev),
                         torch.empty((tokens, 1), dtype=torch.float32, device=dev)) for _ in range(3)]
                theirs = event_time_ms(lambda i=0: ref_kernels.epilogue_rows(*bufs[i % 3][:2], g_, *bufs[i % 3][2:], eps, 1), 50)
                ours = event_time_ms(lambda i=0: capi.add_rmsnorm_quant(*bufs[i % 3][:2], g_, *bufs[i % 3][2:], eps, 1, 240.0), 50)
                return round(theirs * 1e3, 2), round(ours * 1e3, 2)

            for tokens, hidden in ((8192, 8192), (8192, 4096)):
                theirs, ours = ref_norm_quant_us(tokens, hidden)
                ref[f"add_rmsnorm_quant_{tokens}x{hidden}_us"] = {"reference_epilogue": theirs, "this_repository": ours}

            def ref_rope_us(r):
                k0, v0 = r.new_cache()
                qw, kw, cs, pos, loc = (t.to(dev) for t in (r.qw, r.kw, r.cos_sin, r.positions, r.kv_loc))
                bufs = [(r.qkv.to(dev).clone(), torch.empty((r.num_tokens, r.num_heads_q, r.head_size), dtype=torch.bfloat16,
                                                            device=dev), k0.to(dev), v0.to(dev)) for _ in range(4)]
                shape = (r.num_tokens, r.num_heads_q, r.num_heads_k, r.num_heads_v, r.head_size, r.is_neox, r.eps)
                ref_kernels.mrope_rms_set_kv(bufs[0][0], qw, kw, cs, pos, *shape, *bufs[0][1:], loc, r.k_scale, r.v_scale,
                                             r.mrope_section, r.is_interleaved)   # once with the index range checks
                theirs = event_time_ms(lambda i=0: ref_kernels.mrope_rms_set_kv(
                    bufs[i % 4][0], qw, kw, cs, pos, *shape, *bufs[i % 4][1:], loc, r.k_scale, r.v_scale, r.mrope_section,
                    r.is_interleaved, check_values=False), 50)
                ours = event_time_ms(lambda i=0: capi.rope_rms_set_kv(
                    bufs[i % 4][0], qw, kw, cs, pos, *shape, *bufs[i % 4][1:], loc, r.k_scale, r.v_scale, r.mrope_section,
                    r.is_interleaved), 50)
                return round(theirs * 1e3, 2), round(ours * 1e3, 2)

            for name, r in (("rope_kv_qwen3_T4096_us", workloads.config3()), ("mrope_kv_qwen2vl_T8192_us", workloads.config4())):
                theirs, ours = ref_rope_us(r)
                ref[name] = {"reference_kernel": theirs, "this_repository": ours}
            # the two-stream op at the reference script's shape
            B2, T0, T1, Hq2, Hk2, D2 = 2, 678, 3608, 24, 25, 128
            g2 = torch.Generator(device=dev).manual_seed(7)
            mk = lambda *shape: torch.randn(shape, device=dev, generator=g2).to(torch.bfloat16)
            ins2 = [(mk(B2, T0, Hq2, D2), mk(B2, T0, Hk2, D2), mk(B2, T1, Hq2, D2), mk(B2, T1, Hk2, D2)) for _ in range(3)]
            rest = [mk(D2) for _ in range(4)] + [mk(T0, D2), mk(T1, D2)]
            outs2 = (torch.empty((B2, T0 + T1, Hq2, D2), dtype=torch.bfloat16, device=dev),
                     torch.empty((B2, T0 + T1, Hk2, D2), dtype=torch.bfloat16, device=dev))
            times = {}
            for who, fn in (("reference_kernel", ref_kernels.rope_rms_2way), ("this_repository", capi.rope_rms_2way)):
                times[who] = round(event_time_ms(lambda i=0: fn(*ins2[i % 3], *rest, B2, T0, T1, Hq2, Hk2, D2, False, 1e-6,
                                                                *outs2), 50) * 1e3, 2)
            ref["rope_2way_B2_678+3608_us"] = times
            del ins2, outs2
            cpu_baseline["reference_kernels_on_this_gpu"] = ref

    # ------------------------------------------------------------------ secondary figures
    extras = {}
    if not args.no_extras:
        # practical ceiling: plain copy, 512 MiB in + 512 MiB out
        nb = 512 << 20
        src = torch.empty(nb, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        cp_ms = event_time_ms(lambda i=0: capi.copy_bytes(dst, src, nb), 20)
        extras["copy_kernel_GBps"] = round(2 * nb / (cp_ms * 1e-3) / 1e9, 1)

        def windows(nbytes):
            """Offsets of windows of nbytes that tile the 512 MiB calibration buffers (at most 16, at least one): calls
            rotate over them, so that a window comes round again only after the rest of the buffer has passed through
            the 256 MB last-level cache.  None when not even one window fits."""
            if nbytes > nb:
                return None
            n = max(1, min(16, nb // nbytes))
            step = (nb - nbytes) // max(n - 1, 1) // 256 * 256 if n > 1 else 0
            return [k * step for k in range(n)]

        def copy_same_bytes_us(nbytes):
            """The plain copy kernel moving as many bytes as a call of a fused kernel moves (half in, half out)."""
            half = (nbytes // 2 + 15) // 16 * 16
            offs = windows(half)
            if offs is None:   # a shape given on the command line whose calls move more than the copy buffers hold
                return None
            n = len(offs)
            return round(event_time_ms(lambda i=0: capi.copy_bytes(dst[offs[i % n]:], src[offs[i % n]:], half), 100) * 1e3, 2)

        sink = torch.zeros(4, dtype=torch.int32, device=dev)

        def one_direction(read_bytes, write_bytes, workgroups, lanes):
            """What the memory system charges for a call's traffic one direction at a time: a kernel that only reads the
            call's read bytes, one that only writes its written bytes, and an empty grid of the call's launch shape (the
            cost of launching and draining it, which each of the two also contains once).  A fused kernel cannot be
            expected below read + write - launch: reads and writes do not overlap in the memory system."""
            rb, wb = read_bytes // 16 * 16, write_bytes // 16 * 16
            ro, wo = windows(rb), windows(wb)
            if ro is None or wo is None:
                return None
            rd = event_time_ms(lambda i=0: capi.read_bytes(src[ro[i % len(ro)]:], rb, sink), 100) * 1e3
            wr = event_time_ms(lambda i=0: capi.fill_bytes(dst[wo[i % len(wo)]:], wb, i), 100) * 1e3
            floor = graph_time_us(lambda i=0: capi.empty_grid(workgroups, lanes, 0), 20)
            return {"read_only_us": round(rd, 2), "read_GBps": round(rb / rd / 1e3, 1), "write_only_us": round(wr, 2),
                    "write_GBps": round(wb / wr / 1e3, 1), "empty_grid_us": round(floor, 2),
                    "read_plus_write_minus_launch_us": round(rd + wr - floor, 2)}

        # the fused kernel's own memory traffic without its arithmetic (same launch shape, mapping, streaming accesses
        # and barriers) on the benchmark's buffers: the ceiling of the access pattern, beside the kernel itself
        def skeleton_step(i=0):
            x, r, ro, codes, sc = sets[i % NSETS]
            capi.add_rmsnorm_quant_traffic_only(x, r, ro, codes, sc)

        sk_ms = event_time_ms(skeleton_step, 200)
        k_ms = event_time_ms(step, 200)
        extras["add_rmsnorm_quant_traffic_skeleton"] = {
            "traffic_skeleton_us": round(sk_ms * 1e3, 2), "kernel_us": round(k_ms * 1e3, 2),
            "kernel_over_skeleton": round(k_ms / sk_ms, 4),
            "skeleton_frac_of_8TBps": round(alg_bytes / (sk_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "copy_same_bytes_us": copy_same_bytes_us(alg_bytes),
            "one_direction_at_a_time": one_direction(4 * T * H + 2 * H, 3 * T * H + 4 * T, T, lanes)}

        def rope_case(r, n_sets):
            n_axes = 3 if r.mrope_section is not None else 1
            kv_elem = 1 if r.kv_dtype == torch.float8_e4m3fn else 2
            nbytes = workloads.rope_set_kv_bytes(r.num_tokens, r.num_heads_q, r.num_heads_k, r.num_heads_v,
                                                 r.head_size, n_axes, kv_elem)
            k0, v0 = r.new_cache()
            qw, kw, cs, pos, loc = (t.to(dev) for t in (r.qw, r.kw, r.cos_sin, r.positions, r.kv_loc))
            bufs = []
            for s in range(n_sets):
                bufs.append((r.qkv.to(dev).clone(), torch.empty((r.num_tokens, r.num_heads_q, r.head_size),
                                                                 dtype=torch.bfloat16, device=dev),
                             k0.to(dev), v0.to(dev)))

            def call(i=0):
                qkv, q_out, kc, vc = bufs[i % n_sets]
                capi.rope_rms_set_kv(qkv, qw, kw, cs, pos, r.num_tokens, r.num_heads_q, r.num_heads_k,
                                     r.num_heads_v, r.head_size, r.is_neox, r.eps, q_out, kc, vc, loc, r.k_scale,
                                     r.v_scale, r.mrope_section, r.is_interleaved)

            burst = event_time_ms(call, 200)
            avg, med, mn = per_launch_ms(call, 100)
            read_bytes = 2 * r.head_size * (r.num_heads_q + r.num_heads_k + r.num_heads_v) * r.num_tokens
            return nbytes, avg, med, mn, burst, read_bytes

        def rope_kernel_label(r):
            # what the launcher picks for this batch, asked of the library
            groups, lanes, streamed, token_waves = capi.rope_rms_launch_shape(
                r.num_tokens, r.num_heads_q, r.num_heads_k, r.num_heads_v, r.head_size,
                3 if r.mrope_section is not None else 1, torch.bfloat16, True, r.kv_dtype == torch.float8_e4m3fn)
            form = ("rope_rms_kernel (one wave per group of heads)", "rope_rms_token_kernel (one wave per token, stores gated "
                    "behind the launch's reads)", "rope_rms_token_kernel (one wave per two tokens, the second through LDS; "
                    "stores gated behind the launch's reads)")[token_waves]
            return f"{form}, {groups} workgroups x {lanes} lanes, rows stored {'past the L2' if streamed else 'through the L2'}"

        # (the third line: the second shape's kernel on text-only positions -- three equal rows, every token one table
        # row of its own -- at a token count of its own, so that a profiler's per-grid rows tell the two apart: its
        # fetched bytes beside the second line's show what the table rows of image tokens cost, which is nothing)
        for name, r in (("rope_kv_qwen3_T4096", workloads.config3()), ("mrope_kv_qwen2vl_T8192", workloads.config4()),
                        ("mrope_kv_text_only_T8184", workloads.config4(8184, text_only=True))):
            nbytes, avg, med, mn, burst, read_bytes = rope_case(r, 4)
            groups, lanes_b, _, _ = capi.rope_rms_launch_shape(r.num_tokens, r.num_heads_q, r.num_heads_k, r.num_heads_v,
                                                            r.head_size, 3 if r.mrope_section is not None else 1,
                                                            torch.bfloat16, True, False)
            extras[name] = {"us_per_call": round(burst * 1e3, 2), "avg_launch_us": round(avg * 1e3, 2),
                            "GBps": round(nbytes / (burst * 1e-3) / 1e9, 1),
                            "frac_of_8TBps": round(nbytes / (burst * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                            "algorithmic_bytes": nbytes, "copy_same_bytes_us": copy_same_bytes_us(nbytes),
                            "one_direction_at_a_time": one_direction(read_bytes, nbytes - read_bytes, groups, lanes_b),
                            "kernel": rope_kernel_label(r)}
        del src, dst

        # the two-stream op at the reference script's shape (test/test_fused_rope_rms_2way.py:223-246), and the no-KV
        # mRoPE op on the Qwen2-VL-like shape
        B2, T0, T1, Hq2, Hk2, D2 = 2, 678, 3608, 24, 25, 128
        g2 = torch.Generator(device=dev).manual_seed(7)
        mk = lambda *shape: torch.randn(shape, device=dev, generator=g2).to(torch.bfloat16)
        ins2 = [(mk(B2, T0, Hq2, D2), mk(B2, T0, Hk2, D2), mk(B2, T1, Hq2, D2), mk(B2, T1, Hk2, D2)) for _ in range(3)]
        w2 = [mk(D2) for _ in range(4)]
        cs0, cs1 = mk(T0, D2), mk(T1, D2)
        out2 = (torch.empty((B2, T0 + T1, Hq2, D2), dtype=torch.bfloat16, device=dev),
                torch.empty((B2, T0 + T1, Hk2, D2), dtype=torch.bfloat16, device=dev))

        def two_way_call(i=0):
            q0, k0_, q1, k1_ = ins2[i % 3]
            capi.rope_rms_2way(q0, k0_, q1, k1_, *w2, cs0, cs1, B2, T0, T1, Hq2, Hk2, D2, False, 1e-6, *out2)

        nb2 = 2 * (B2 * (T0 + T1) * (Hq2 + Hk2) * D2 * 2) + (T0 + T1) * D2 * 2 + 4 * D2 * 2
        ms2 = event_time_ms(two_way_call, 100)
        extras["rope_2way_B2_678+3608"] = {"us_per_call": round(ms2 * 1e3, 2), "GBps": round(nb2 / (ms2 * 1e-3) / 1e9, 1),
                                           "frac_of_8TBps": round(nb2 / (ms2 * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                                           "algorithmic_bytes": nb2}
        r4 = workloads.config4()
        qw4, kw4, cs4, pos4 = (t.to(dev) for t in (r4.qw, r4.kw, r4.cos_sin, r4.positions))
        qkv4 = [r4.qkv.to(dev).clone() for _ in range(4)]

        def mrope_inplace_call(i=0):
            capi.rope_rms(qkv4[i % 4], qw4, kw4, cs4, pos4, r4.num_tokens, r4.num_heads_q, r4.num_heads_k, r4.num_heads_v,
                          r4.head_size, r4.is_neox, r4.eps, r4.mrope_section, r4.is_interleaved)

        nb4 = workloads.rope_inplace_bytes(r4.num_tokens, r4.num_heads_q, r4.num_heads_k, r4.head_size, 3)
        ms4 = event_time_ms(mrope_inplace_call, 100)
        extras["mrope_inplace_qwen2vl_T8192"] = {"us_per_call": round(ms4 * 1e3, 2),
                                                 "GBps": round(nb4 / (ms4 * 1e-3) / 1e9, 1),
                                                 "frac_of_8TBps": round(nb4 / (ms4 * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                                                 "algorithmic_bytes": nb4}
        del ins2, out2, qkv4

        # decode shapes: per call, eager (host launch overhead included) and replayed from a HIP graph of 20 calls on
        # 20 distinct buffer sets (GPU-side cost)
        decode = {}
        NG = 20
        for t in workloads.DECODE_TOKENS_WIDE:
            d = workloads.config5_norm(t)
            g_ = d.gamma.to(dev)
            nq = [(d.x.to(dev).clone(), d.residual.to(dev).clone(), torch.empty((t, 7168), dtype=torch.bfloat16, device=dev),
                   torch.empty((t, 7168), dtype=torch.float8_e4m3fn, device=dev),
                   torch.empty((t, 1), dtype=torch.float32, device=dev)) for _ in range(NG)]

            def nq_call(i=0):
                x, r_, ro, codes, sc = nq[i % NG]
                capi.add_rmsnorm_quant(x, r_, g_, ro, codes, sc, d.eps, 1)

            r = workloads.config5_rope(t)
            k0, v0 = r.new_cache()
            qw, kw, cs, pos, loc = (z.to(dev) for z in (r.qw, r.kw, r.cos_sin, r.positions, r.kv_loc))
            kc, vc = k0.to(dev), v0.to(dev)
            rp = [(r.qkv.to(dev).clone(), torch.empty((t, r.num_heads_q, r.head_size), dtype=torch.bfloat16, device=dev))
                  for _ in range(NG)]

            def rope_call(i=0):
                qkv, q_out = rp[i % NG]
                capi.rope_rms_set_kv(qkv, qw, kw, cs, pos, t, r.num_heads_q, r.num_heads_k, r.num_heads_v, r.head_size,
                                     r.is_neox, r.eps, q_out, kc, vc, loc, r.k_scale, r.v_scale)

            def nq_skeleton_call(i=0):
                x, r_, ro, codes, sc = nq[i % NG]
                capi.add_rmsnorm_quant_traffic_only(x, r_, ro, codes, sc)

            decode[str(t)] = {"add_rmsnorm_quant_us": round(graph_time_us(nq_call, NG), 2),
                              "add_rmsnorm_quant_traffic_skeleton_us": round(graph_time_us(nq_skeleton_call, NG), 2),
                              "add_rmsnorm_quant_bytes": workloads.norm_quant_bytes(t, 7168, 1),
                              "rope_kv_fp8_us": round(graph_time_us(rope_call, NG), 2),
                              "add_rmsnorm_quant_eager_us": round(event_time_ms(nq_call, 200) * 1e3, 2),
                              "rope_kv_fp8_eager_us": round(event_time_ms(rope_call, 200) * 1e3, 2)}
        extras["decode_us_per_call"] = decode
        # static per-tensor quant at tokens=128, hidden=4096; scale = amax(normed)/448, taken once, outside the timing,
        # from the same kernel's unquantised output
        c1 = workloads.config1()
        c1_g = c1.gamma.to(dev)
        c1_normed = torch.empty((128, 4096), dtype=torch.bfloat16, device=dev)
        capi.add_rmsnorm_quant(c1.x.to(dev), c1.residual.to(dev), c1_g, torch.empty_like(c1_normed), c1_normed, None, c1.eps, 0)
        c1_scale = (c1_normed.float().abs().max() / 448.0).reshape(1)
        c1_bufs = [(c1.x.to(dev).clone(), c1.residual.to(dev).clone(), torch.empty((128, 4096), dtype=torch.bfloat16, device=dev),
                    torch.empty((128, 4096), dtype=torch.float8_e4m3fn, device=dev)) for _ in range(NG)]

        def c1_call(i=0):
            x, r_, ro, codes = c1_bufs[i % NG]
            capi.add_rmsnorm_quant(x, r_, c1_g, ro, codes, c1_scale, c1.eps, 3)

        extras["static_quant_T128_H4096_us_per_call"] = {"graph": round(graph_time_us(c1_call, NG), 2),
                                                         "eager": round(event_time_ms(c1_call, 200) * 1e3, 2),
                                                         "algorithmic_bytes": workloads.norm_quant_bytes(128, 4096, 3)}
        # the floor under those: a 1024-element increment kernel (one workgroup), same two ways of launching
        small = [torch.zeros(1024, dtype=torch.float32, device=dev) for _ in range(NG)]

        def small_call(i=0):
            capi.increment_floats(small[i % NG], 1024)

        extras["small_kernel_us_per_call"] = {"graph": round(graph_time_us(small_call, NG), 2),
                                              "eager": round(event_time_ms(small_call, 200) * 1e3, 2)}

        # a caller of both paths: one Qwen3-8B-sized decoder block, decode step of 32 sequences with 256 cached
        # positions each, replayed from a HIP graph; fused operators against the torch sequence on the same weights
        # (GEMMs and attention are torch's in both, so the difference is the memory-bound glue)
        with torch.no_grad():
            from gpuk_amd import consumer

            bargs = consumer.BlockArgs()
            torch.manual_seed(0)
            block = consumer.TransformerBlock(bargs, dev)
            nseq, ctx, bs = 32, 256, 16
            per_seq = ctx // bs + 1
            cache = consumer.PagedKVCache(nseq * per_seq, bs, bargs.n_kv_heads, bargs.head_dim, bargs.dtype, dev)
            table = torch.randperm(nseq * per_seq, device=dev).view(nseq, per_seq)
            idx = consumer.decode_batch(cache, table, torch.full((nseq,), ctx, device=dev))
            hid = torch.randn((nseq, bargs.dim), device=dev).to(bargs.dtype)
            res = torch.randn((nseq, bargs.dim), device=dev).to(bargs.dtype)
            fused_us = graph_time_us(lambda i=0: block(hid, res, *idx[:2], cache, *idx[2:]), 4, 20)
            unfused_us = graph_time_us(lambda i=0: block.forward_unfused(hid, res, *idx[:2], cache, *idx[2:]), 4, 20)
            extras["decoder_block_decode_us"] = {"fused_ops": round(fused_us, 1), "torch_sequence": round(unfused_us, 1),
                                                 "sequences": nseq, "context": ctx, "dim": bargs.dim,
                                                 "heads": [bargs.n_heads, bargs.n_kv_heads, bargs.n_kv_heads]}
            del block, cache

    out = {
        "metric": f"HBM GB/s add+RMSNorm+FP8 per-token quant @{T}x{H} bf16",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"residual-add + RMSNorm + dynamic per-token e4m3fn quant, tokens={T}, hidden={H}, "
                               "bf16, x~N(0,1), residual~N(0,sigma=2), gamma~N(1,0.1), 1% of x = +-50, eps=1e-6",
                   "entry": "torch.ops.gpuk.allreduce_rms(fptr=0, quant_type=1)", "buffer_sets": NSETS,
                   "prewarm_steps": n_pre},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "roofline": roofline, "cpu_baseline": cpu_baseline, "extras": extras,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
