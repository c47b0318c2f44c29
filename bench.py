#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extra] [--no-cpu]

One "step" is one fused quantized matmul (the kernel the recognizer emits) on
the small-batch decode shape: x bf16 [16,4096], W int4 affine g64
[14336,4096] (packed uint32 [14336,512], bf16 scale/bias tables), y bf16
[16,14336] -- seeded synthetic data, inputs resident in HBM.  Consecutive steps
rotate through enough distinct weight buffers (more than twice the 256 MB
last-level cache) that every launch streams its weights from HBM.  The K timed
steps are replayed from a HIP graph and bracketed by HIP events on the launch
stream.  Prints ONE JSON line.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "qmm GB/s (% HBM peak) decode GEMV; TFLOP/s (% MFMA peak) prefill GEMM"
HBM_PEAK_GBS = 8000.0            # MI355X HBM3E
PEAK_TFLOPS = {"bf16": 2500.0, "fp8": 5000.0, "fp4": 10100.0}
LLC_BYTES = 256 << 20


def _events_ms(fn_timed, stream):
    import torch
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record(stream)
    fn_timed()
    b.record(stream)
    torch.cuda.synchronize()
    return a.elapsed_time(b)


def run_rotating(make_call, n_sets, steps, warmup):
    """Time launches that cycle through `n_sets` bound calls.

    A HIP graph holding one launch per set is replayed a whole number of times:
    the `steps` asked for are rounded up to a multiple of `n_sets`, at least
    two replays, so that no launch inside the event bracket is an eager one
    (a kernel of a few microseconds launched call by call measures the host).
    Returns (milliseconds, launches timed)."""
    import torch
    calls = [make_call(i) for i in range(n_sets)]
    # The operands were produced on the default stream and the launches below run on a stream of their
    # own: everything queued so far (the weight sets' fills, the routing indices) has to be finished
    # first, or the first launches read buffers that are still being written.
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        for i in range(max(warmup, 1)):
            calls[i % n_sets].launch()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for c in calls:
                c.launch()
        graph.replay()                      # one untimed replay
        torch.cuda.synchronize()
        reps = max(2, -(-steps // n_sets))

        def timed():
            for _ in range(reps):
                graph.replay()
        ms = _events_ms(timed, torch.cuda.current_stream())
    return ms, reps * n_sets


def bench_decode(cfg, M, steps, warmup):
    import torch
    from metaljax_amd import kernels as K, synth
    wl = synth.make(cfg, M=M)
    x, w, s, b, _ = synth.to_device(wl)
    per_set = w.numel() * 4 + s.numel() * s.element_size() * (2 if b is not None else 1)
    n_sets = max(2, (2 * LLC_BYTES) // per_set + 1)
    sets = [(w, s, b)] + [(w.clone(), s.clone(), None if b is None else b.clone())
                          for _ in range(n_sets - 1)]
    ys = [torch.empty((wl.M, wl.N), dtype=torch.bfloat16, device="cuda") for _ in range(n_sets)]

    def make_call(i):
        wi, si, bi = sets[i]
        return K.BoundQmm(x, wi, si, bi, ys[i], group_size=wl.group_size, bits=wl.bits, mode=wl.mode)
    ms, launches = run_rotating(make_call, n_sets, steps, warmup)
    return wl, ms / launches * 1e3, launches, n_sets, ys[0]


def bench_decode_random(m, n, k, bits=4, mode="affine", tables="bf16", steps=200, warmup=20):
    """Per-launch time of a decode shape outside the named configurations, on
    random codes (timing only): graph replay over rotating weight sets."""
    import torch
    from metaljax_amd import kernels as K
    g = torch.Generator(device="cuda").manual_seed(n + k)
    words = k * bits // 32
    x = torch.randn((m, k), device="cuda", generator=g).bfloat16()
    if mode == "mxfp4":
        s = torch.randint(118, 132, (n, k // 32), dtype=torch.uint8, device="cuda", generator=g)
        b = None
        gs = 32
    else:
        dt = {"f16": torch.float16, "f32": torch.float32}.get(tables, torch.bfloat16)
        s = (torch.rand((n, k // 64), device="cuda", generator=g) * 0.01 + 0.005).to(dt)
        b = (-8 * s.float()).to(dt)
        gs = 64
    per_set = n * words * 4
    n_sets = max(2, (2 * LLC_BYTES) // per_set + 1)
    ws = [torch.randint(-2**31, 2**31 - 1, (n, words), dtype=torch.int32, device="cuda", generator=g)
          for _ in range(n_sets)]
    ys = [torch.empty((m, n), dtype=torch.bfloat16, device="cuda") for _ in range(n_sets)]
    ms, launches = run_rotating(lambda i: K.BoundQmm(x, ws[i], s, b, ys[i], group_size=gs, bits=bits, mode=mode),
                                n_sets, steps, warmup)
    us = ms * 1e3 / launches
    nbytes = n * words * 4 + s.numel() * s.element_size() * (1 if b is None else 2) + (m * k + m * n) * 2
    return {"us": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1),
            "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}


def _rel_l2(got, want):
    import numpy as np
    d = np.linalg.norm(got.astype(np.float64) - want.astype(np.float64))
    return float(d / max(np.linalg.norm(want.astype(np.float64)), 1e-30))


def oracle_check(wl, y, exact_weight):
    """rel-L2 of one output of a timed leg against the C oracle, outside the
    timed region.  `exact_weight`: against the exactly reconstructed weight,
    else against the weight tile rounded once to bf16 (what the prefill kernels
    stage)."""
    from oracle import c_oracle as C
    if wl.row_offsets is not None:
        want = C.grouped_qmm(wl.x, wl.w, wl.scales, wl.biases, wl.row_offsets, wl.group_size, wl.bits,
                             wl.mode, round_tile_bf16=not exact_weight)
    else:
        want = C.qmm(wl.x, wl.w, wl.scales, wl.biases, wl.group_size, wl.bits, wl.mode,
                     round_tile_bf16=not exact_weight)
    return _rel_l2(y.float().cpu().numpy(), want)


def bench_once(cfg, steps=40, warmup=4, check=True):
    """One of the other named shapes (C3 prefill, C4 MXFP4, C5 grouped): graph
    replay over rotating weight sets, like the decode legs, so that every
    launch streams its weights from HBM; the time includes the activation
    re-layout / split kernel that precedes the product.  One output is checked
    against the C oracle outside the timed region."""
    import torch
    from metaljax_amd import kernels as K, synth
    wl = synth.make(cfg)
    x, w, s, b, ro = synth.to_device(wl)
    per_set = w.numel() * 4 + s.numel() * s.element_size() * (2 if b is not None else 1)
    n_sets = max(2, (2 * LLC_BYTES) // per_set + 1)
    sets = [(w, s, b)] + [(w.clone(), s.clone(), None if b is None else b.clone()) for _ in range(n_sets - 1)]
    ys = [torch.empty((x.shape[0], wl.N), dtype=torch.bfloat16, device="cuda") for _ in range(n_sets)]

    def make_call(i):
        wi, si, bi = sets[i]
        if cfg == 5:        # every row of C5 belongs to an expert, so the output needs no zero fill
            return K.BoundGrouped(x, wi, si, bi, ro, ys[i], group_size=64, bits=4)
        return K.BoundQmm(x, wi, si, bi, ys[i], group_size=wl.group_size, bits=wl.bits, mode=wl.mode)
    ms, launches = run_rotating(make_call, n_sets, steps, warmup)
    us = ms * 1e3 / launches
    tf = wl.flops / us / 1e6
    out = {"workload": wl.name, "us": round(us, 2), "TFLOP/s": round(tf, 1),
           "GB/s": round(wl.algorithmic_bytes / us / 1e3, 1), "weight_sets": n_sets, "timed_launches": launches}
    if wl.mode == "mxfp4":
        # block-scaled matrix cores: each useful MFMA is issued twice (two FP6
        # activation terms), so both the useful and the issued rate are given
        # against the fp4 peak; the time includes the activation split kernel
        out["frac_of_fp4_mfma_peak"] = round(tf / PEAK_TFLOPS["fp4"], 4)
        out["issued_TFLOP/s"] = round(2 * tf, 1)
        out["issued_frac_of_fp4_mfma_peak"] = round(2 * tf / PEAK_TFLOPS["fp4"], 4)
    else:
        out["frac_of_bf16_mfma_peak"] = round(tf / PEAK_TFLOPS["bf16"], 4)
    if check:
        # bf16 outputs: distance from the exact-weight product (the 1e-2 bar),
        # and for the bf16-tile kernels from the rounded-tile product as well
        out["rel_l2_vs_exact_weight"] = float(f"{oracle_check(wl, ys[0], True):.3e}")
        if wl.mode == "affine":
            out["rel_l2_vs_bf16_tile"] = float(f"{oracle_check(wl, ys[0], False):.3e}")
        assert out["rel_l2_vs_exact_weight"] <= 1e-2, out
    return out


def bench_dense_bf16(m, n, k, steps=40, experts=1):
    """The same box's library matmul on bf16 operands of a named shape
    (x [M, K] x W [N, K]^T, `experts` of them one after another): the practical
    ceiling for a kernel that must also dequantize."""
    import torch
    n_sets = max(2, (2 * LLC_BYTES) // (experts * n * k * 2) + 1)
    ws = [torch.randn((experts, n, k), device="cuda", dtype=torch.bfloat16) for _ in range(n_sets)]
    x = torch.randn((experts, m, k), device="cuda", dtype=torch.bfloat16)
    ys = [torch.empty((experts, m, n), device="cuda", dtype=torch.bfloat16) for _ in range(n_sets)]

    def step(i):
        torch.bmm(x, ws[i].transpose(1, 2), out=ys[i])
    for i in range(n_sets):
        step(i)
    ms = _events_ms(lambda: [step(i % n_sets) for i in range(steps)], torch.cuda.current_stream())
    us = ms * 1e3 / steps
    tf = 2.0 * experts * m * n * k / us / 1e6
    return {"us": round(us, 2), "TFLOP/s": round(tf, 1), "frac_of_bf16_mfma_peak": round(tf / PEAK_TFLOPS["bf16"], 4)}


def bench_moe_decode(tokens, experts=8, topk=2, n=14336, k=4096, steps=60, warmup=6):
    """Expert-indexed decode (the call a recognized mixture-of-experts block
    makes per projection, reference src/metaljax/moe.py:1320): `tokens` tokens,
    each routed to `topk` of `experts` int4 g64 experts of [n, k], pairs in
    token order (unsorted, as the reference hands them over).  Graph replay
    over rotating weight sets; GB/s counts the weights and tables of the
    experts the routing touches, once each."""
    import torch
    from metaljax_amd import kernels as K
    g = torch.Generator(device="cuda").manual_seed(tokens * 131 + experts)
    words = k // 8
    per_set = experts * n * words * 4
    n_sets = max(2, (2 * LLC_BYTES) // per_set + 1)
    ws = [torch.randint(-2**31, 2**31 - 1, (experts, n, words), dtype=torch.int32, device="cuda", generator=g)
          for _ in range(n_sets)]
    s = (torch.rand((experts, n, k // 64), device="cuda", generator=g) * 0.015 + 0.005).bfloat16()
    b = (-8 * s.float()).bfloat16()
    x = torch.randn((tokens, k), device="cuda", generator=g).bfloat16()
    logits = torch.randn((tokens, experts), device="cuda", generator=g)
    rhs = torch.topk(logits, topk, dim=-1).indices.reshape(-1).to(torch.int32).contiguous()
    lhs = torch.arange(tokens, device="cuda", dtype=torch.int32).repeat_interleave(topk).contiguous()
    ys = [torch.empty((tokens * topk, n), dtype=torch.bfloat16, device="cuda") for _ in range(n_sets)]
    ms, launches = run_rotating(lambda i: K.BoundGather(x, ws[i], s, b, lhs, rhs, ys[i], group_size=64, bits=4),
                                n_sets, steps, warmup)
    us = ms * 1e3 / launches
    touched = int(torch.unique(rhs).numel())
    nbytes = touched * (n * words * 4 + 2 * n * (k // 64) * 2) + tokens * k * 2 + tokens * topk * n * 2
    return {"us": round(us, 2), "pairs": tokens * topk, "experts_touched": touched, "bytes": nbytes,
            "GB/s": round(nbytes / us / 1e3, 1), "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
            "timed_launches": launches}


def bench_engine_execute(cfg=2, m=16, calls=100):
    """Wall-clock time of `engine.execute` on the recognized program of a
    decode shape (a sub-channel int4 dot, the weight as i8 codes + scales +
    zero points, as a checkpoint holds it), buffers resident on the device:
    what the fused kernel costs behind the recognizer, the interpreter and the
    ctypes call, per call, after the first call has packed the weight.  Not a
    kernel figure: the host work of one call is most of it."""
    import numpy as np
    import torch
    from metaljax_amd import engine, qmm, synth
    sh = synth.SHAPES[cfg]
    n, k = sh["N"], sh["K"]
    rng = np.random.default_rng(7)
    q = rng.integers(-8, 8, size=(n, k)).astype(np.int8)
    scale = synth._bf16(rng.uniform(0.005, 0.02, size=(n, k // 64)))          # bf16 bit patterns
    zero = np.zeros((n, k // 64), np.int8)
    x = synth._bf16(rng.standard_normal((m, k)))
    ex = engine.compile_program(synth.affine_program_text(m, n, k), "mlir")
    bufs = [engine.buffer_from_host(q, engine._ENUM["S8"], q.shape),
            engine.buffer_from_host(scale, engine._ENUM["BF16"], scale.shape),
            engine.buffer_from_host(zero, engine._ENUM["S8"], zero.shape),
            engine.buffer_from_host(x, engine._ENUM["BF16"], x.shape)]
    qmm.reset_stats()
    out = engine.execute(ex, bufs)          # packs the weight
    torch.cuda.synchronize()
    stats = qmm.stats()
    for _ in range(5):
        out = engine.execute(ex, bufs)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(calls):
        out = engine.execute(ex, bufs)
    torch.cuda.synchronize()
    us = (time.perf_counter() - t0) * 1e6 / calls
    return {"us_per_call": round(us, 1), "calls": calls, "dots_recognized": stats.get("recognized", 0),
            "packs_built": stats.get("packs", 0), "fallbacks": stats.get("fallbacks", 0),
            "result_on_device": bool(getattr(out[0].data, "is_cuda", False)),
            "what": f"engine.execute of the recognized int4 g64 [{n},{k}] dot at M={m}, device-resident buffers, "
                    "wall clock including the interpreter and the ctypes call"}


def cpu_baseline(wl, budget_s=4.0):
    """The C restatement of the reference's unfused chain (oracle/qmm_oracle.c),
    timed on the host cores: the checker used as the reported CPU baseline."""
    from oracle import c_oracle as C
    reps, t_total = 0, 0.0
    C.qmm(wl.x, wl.w, wl.scales, wl.biases, wl.group_size, wl.bits, wl.mode, True)   # warm-up
    while reps < 2 or (t_total < budget_s and reps < 50):
        t0 = time.perf_counter()
        C.qmm(wl.x, wl.w, wl.scales, wl.biases, wl.group_size, wl.bits, wl.mode, True)
        t_total += time.perf_counter() - t0
        reps += 1
    sec = t_total / reps
    return {"value": round(wl.algorithmic_bytes / sec / 1e9, 3), "unit": "GB/s",
            "cores": C.num_threads(), "kind": "port",
            "sample": f"the full workload ({wl.M}x{wl.N}x{wl.K}), {reps} timed passes, "
                      f"{sec * 1e3:.1f} ms per pass, unpack + dequantize to a bf16 tile + f32-accumulate dot"}


def committed_traffic():
    """HBM bytes per launch of the decode kernel on C2, as measured by the
    FETCH_SIZE / WRITE_SIZE counter runs whose summary is committed under
    profiles/ (a counter run cannot happen inside this program); None when
    that summary is absent."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                        "decode_qmm_C2_int4_g64_hbm_traffic.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                return int(line.split(":")[1].split()[0])
    except OSError:
        pass
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-extra", action="store_true", help="skip the other named shapes")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--m16-only", action="store_true", help="run the headline decode leg only")
    ap.add_argument("--moe-decode", action="store_true",
                    help="time the expert-indexed decode legs only (for profiling those kernels)")
    ap.add_argument("--shape", choices=["C3", "C4", "C5"], default=None,
                    help="time one of the other named shapes only (for profiling that kernel)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run a 64 MiB read + 64 MiB write elementwise kernel five times, "
                         "for scaling FETCH_SIZE / WRITE_SIZE counter readings")
    ap.add_argument("--timeline", action="store_true",
                    help="print the decode kernel's clock-stamp timeline on C2 (needs a library built with "
                         "QMM_TIMELINE=1)")
    ap.add_argument("--probe", action="store_true",
                    help="time read-only and empty launches instead (what one launch over the "
                         "headline's bytes can reach on this GPU whatever its arithmetic)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU; --gpus {args.gpus} is not supported "
              "(rows of the weight are independent: more GPUs would each take a share of N)", file=sys.stderr)
        return 2
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible (the HIP path has no CPU fallback)", file=sys.stderr)
        return 3
    from metaljax_amd import kernels as K

    if args.calibration_copy:
        src = torch.arange(1 << 24, dtype=torch.int32, device="cuda")      # 64 MiB
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.bitwise_not(src, out=dst)
        torch.cuda.synchronize()
    if args.timeline:
        from metaljax_amd import profiling
        print(json.dumps({"decode_timeline_us": profiling.decode_timeline()}, indent=1))
        return 0
    if args.probe:
        from metaljax_amd import profiling
        print(json.dumps({"probe": profiling.stream_probe()}))
        return 0
    if args.shape:
        print(json.dumps({args.shape: bench_once(int(args.shape[1]), check=not args.no_cpu)}))
        return 0
    if args.moe_decode:
        print(json.dumps({"moe_decode": {f"{t} token(s)": bench_moe_decode(t) for t in (1, 16)}}))
        return 0
    wl, us, launches, n_sets, y = bench_decode(2, 16, args.steps, args.warmup)
    headline_rel_l2 = None if args.no_cpu else oracle_check(wl, y, True)     # outside the timed region
    assert headline_rel_l2 is None or headline_rel_l2 <= 1e-2, headline_rel_l2
    gbs = wl.algorithmic_bytes / us / 1e3
    kern, grid, block = K.plan(wl.M, wl.N, wl.K, wl.group_size, wl.bits, wl.mode)
    out = {
        "metric": METRIC, "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(us / 1e3, 6),
        "timed_launches": launches,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (seeded numpy draws, rng 1000+cfg; weights rotate through "
                f"{n_sets} distinct buffers so each launch streams from HBM)",
        "config": {"workload": "C2 small-batch decode qmm: x bf16 [16,4096] x W int4 affine g64 "
                               "[14336,4096] (u32 [14336,512], bf16 tables) -> y bf16 [16,14336]",
                   "M": wl.M, "N": wl.N, "K": wl.K, "bits": wl.bits, "group_size": wl.group_size,
                   "algorithmic_bytes": wl.algorithmic_bytes, "flops": wl.flops,
                   "kernel": "decode (M<=16)" if kern == 1 else "prefill", "grid": grid, "block": block},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": committed_traffic(),
                     "traffic_source": "profiles/decode_qmm_C2_int4_g64_hbm_traffic.txt (two rocprofv3 --pmc "
                                       "runs of this leg; a counter run cannot happen inside this program)"},
        "rel_l2_vs_oracle": None if headline_rel_l2 is None else float(f"{headline_rel_l2:.3e}"),
        "TFLOP/s": round(wl.flops / us / 1e6, 2),
    }
    if args.m16_only:
        print(json.dumps(out))
        return 0
    # second decode point: the same weight at M = 1
    def decode_leg(cfg, m):
        wlx, usx, nx, _, _ = bench_decode(cfg, m, max(args.steps // 4, 50), max(args.warmup // 4, 5))
        return {"workload": wlx.name, "us": round(usx, 2), "bytes": wlx.algorithmic_bytes,
                "GB/s": round(wlx.algorithmic_bytes / usx / 1e3, 1),
                "frac_of_hbm_peak": round(wlx.algorithmic_bytes / usx / 1e3 / HBM_PEAK_GBS, 4), "timed_launches": nx}
    out["decode_M1"] = decode_leg(2, 1)
    if not args.no_extra:
        # C1 is a decode shape: graph replay over rotating weight sets like the
        # headline leg (a 6-7 us kernel timed call by call would measure the host)
        out["other_shapes"] = {"C1": decode_leg(1, 1)}
        out["other_shapes"].update({f"C{c}": bench_once(c, check=not args.no_cpu) for c in (3, 4, 5)})
        # the library's bf16 matmul on the same shapes (no dequantization)
        out["dense_bf16"] = {"C3 [2048,4096]x[4096,4096]": bench_dense_bf16(2048, 4096, 4096),
                             "C4 [256,8192]x[8192,8192]": bench_dense_bf16(256, 8192, 8192),
                             "C5 8 x [128,4096]x[14336,4096]": bench_dense_bf16(128, 14336, 4096, experts=8)}
        # Legs outside the named configurations (random codes, timing only).  An exception in one of
        # them is reported in its place: it must not take the named configurations' line with it.
        def extra(fn, *a, **kw):
            try:
                return fn(*a, **kw)
            except Exception as why:                        # noqa: BLE001 -- reported, not hidden
                return {"error": f"{type(why).__name__}: {why}"}
        out["other_decode_shapes"] = {
            "int4 g64 [28672,4096] M=4": extra(bench_decode_random, 4, 28672, 4096),
            "int4 g64 [4096,14336] M=4": extra(bench_decode_random, 4, 4096, 14336),
            "int4 g64 f16 tables [14336,4096] M=4": extra(bench_decode_random, 4, 14336, 4096, tables="f16"),
            "int4 g64 f32 tables [14336,4096] M=4": extra(bench_decode_random, 4, 14336, 4096, tables="f32"),
            "int8 g64 [14336,4096] M=4": extra(bench_decode_random, 4, 14336, 4096, bits=8),
            "int4 g64 [37888,3584] M=4": extra(bench_decode_random, 4, 37888, 3584),
            "mxfp4 [8192,8192] M=1": extra(bench_decode_random, 1, 8192, 8192, mode="mxfp4"),
            "mxfp4 [5760,2880] M=1 (K no whole number of slices)": extra(bench_decode_random, 1, 5760, 2880, mode="mxfp4"),
            "mxfp4 [5760,2880] M=16": extra(bench_decode_random, 16, 5760, 2880, mode="mxfp4"),
        }
        out["moe_decode"] = {f"8 experts int4 g64 [14336,4096], top-2, {t} token(s)": extra(bench_moe_decode, t)
                             for t in (1, 16)}
        out["engine_execute_C2"] = extra(bench_engine_execute, 2, 16)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(wl)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
