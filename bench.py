#!/usr/bin/env python3
"""Benchmark of the GGUF quantized-matmul hot path on one MI355X.

Headline (BASELINE.json configs[1]): Q4_K decode GEMV, batch 1, over the seven projections of
one transformer layer (hidden 4096 / FFN 14336 / 32 q-heads / 8 kv-heads).  One step = one
layer = seven GEMVs, issued through the C ABI as one grouped launch
(TSHip_AddmmQuantGroupF32Device).  Several distinct layer copies are cycled so that the
256 MB Infinity Cache cannot serve the weights.  `value` is algorithmic GB/s
(weights + activations + outputs) over the timed region, inputs resident in HBM.

Prints ONE JSON line.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

Q8_0, Q4_K, Q5_K, Q6_K, MXFP4 = 8, 12, 13, 14, 39
HBM_PEAK_GBS = 8000.0
MFMA_FP16_PEAK_TFLOPS = 2516.6
MFMA_FP6_FP4_PEAK_TFLOPS = 10066.0   # dense fp6 / fp4 operands (two instructions per k-tile count 4 M N K operations)
# HBM bytes per launch of the grouped Q4_K GEMV come from rocprofv3 FETCH_SIZE + WRITE_SIZE runs, not from this script.
# The summary of those runs records the figure together with the SHA-256 of the kernel source it was measured on; the
# figure is reported only while the source still has that digest.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "gemv_q4k_layer_hbm_traffic.txt")
GEMV_SOURCE = os.path.join(ROOT, "tensorsharp_amd", "csrc", "gemv.hip")

LAYER = [  # name, N (out), K (in) — BASELINE.json configs[1]
    ("wq", 4096, 4096), ("wk", 1024, 4096), ("wv", 1024, 4096), ("wo", 4096, 4096),
    ("gate", 14336, 4096), ("up", 14336, 4096), ("down", 4096, 14336),
]


def row_bytes(t, k):
    return {2: 18 * (k // 32), 3: 20 * (k // 32), 6: 22 * (k // 32), 7: 24 * (k // 32), 20: 18 * (k // 32), Q8_0: 34 * (k // 32), Q4_K: 144 * (k // 256), Q5_K: 176 * (k // 256), Q6_K: 210 * (k // 256), MXFP4: 17 * (k // 32)}[t]


def algorithmic_bytes(t, n, k, m=1):
    return n * row_bytes(t, k) + m * k * 4 + m * n * 4


def cpu_baseline(layer_host, xs_host, n_threads):
    """Oracle port of the reference's managed loop nest (ModelBase.cs:924-991), all host threads,
    on the same seven matrices; best of 3 passes over one layer."""
    from oracle.oracle import Oracle
    try:
        orc = Oracle(fast=True)
        orc.lib.tso_max_threads()
    except OSError:
        orc = Oracle(fast=False)
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        for (name, n, k), w, x in zip(LAYER, layer_host, xs_host):
            orc.matmul_managed(Q4_K, w, n, k, x, vec_width=8, threads=n_threads)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    total = sum(algorithmic_bytes(Q4_K, n, k) for _, n, k in LAYER)
    return {"value": round(total / best / 1e9, 3), "unit": "GB/s", "cores": n_threads, "kind": "port",
            "sample": "one full layer (7 Q4_K GEMVs, 123.0 MB), best of 3 passes, OpenMP over output rows",
            "seconds_per_layer": round(best, 4)}


def cpu_reference_ggml(layer_host, xs_host, n_threads):
    """The reference's own ggml CPU matmul (activations quantized to Q8_K, integer dot products) on the same
    seven matrices, from the library built out of the reference's sources beside the oracle; None when that
    library is not there.  Best of 3 passes over one layer."""
    from oracle.oracle import Reference
    if not Reference.available():
        return None
    ref = Reference()
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        for (name, n, k), w, x in zip(LAYER, layer_host, xs_host):
            ref.mul_mat(Q4_K, w, n, k, x, threads=n_threads)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    total = sum(algorithmic_bytes(Q4_K, n, k) for _, n, k in LAYER)
    return {"value": round(total / best / 1e9, 3), "unit": "GB/s", "cores": n_threads, "kind": "reference",
            "sample": "one full layer (7 Q4_K GEMVs, 123.0 MB) through ggml's CPU backend as the reference builds it "
                      "(-O3, no -march), best of 3 passes",
            "seconds_per_layer": round(best, 4)}


def measured_traffic_bytes():
    """HBM bytes per launch from the committed counter summary, or None when the kernel source changed since."""
    import hashlib
    import re
    try:
        text = open(TRAFFIC_SUMMARY).read()
        digest = hashlib.sha256(open(GEMV_SOURCE, "rb").read()).hexdigest()
    except OSError:
        return None
    m_bytes = re.search(r"^traffic_bytes_per_launch:\s*(\d+)", text, re.M)
    m_sha = re.search(r"^gemv_source_sha256:\s*([0-9a-f]{64})", text, re.M)
    if not m_bytes or not m_sha or m_sha.group(1) != digest:
        return None
    return int(m_bytes.group(1))


def time_region(fn, steps, torch):
    """fn(i) launches step i on the current stream. Returns (event_ms, wall_ms)."""
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_time(e1), wall


def library_fp16_gemm_us(torch, dev, m, n, k, iters=20):
    """Reference point only, never part of `value` or of the product: the vendor library's GEMM (torch.matmul) on DENSE fp16
    operands of the same shape - no dequantization, half-precision inputs and output - timed like the calls beside it."""
    x = torch.randn((m, k), device=dev, dtype=torch.float16)
    w = (torch.randn((n, k), device=dev, dtype=torch.float32) * 0.02).to(torch.float16)

    def f(i):
        torch.matmul(x, w.t())
    for i in range(3):
        f(i)
    ev, wall = time_region(f, iters, torch)
    return ev * 1e3 / iters


def timeline(args, torch, dev, HipBasicOps, QuantizedWeight, synth):
    """Where the time of one decode launch goes: TSHip_SetGemvTimeline makes every wavefront of the GEMV kernel stamp the
    100 MHz constant clock at entry, after the activations are staged and at exit.  The launch is repeated (cycling weight
    copies larger than the memory-side cache) and every repetition is read back; times are relative to the launch's
    first entry, medians over the repetitions."""
    import ctypes as C
    import numpy as np
    from tensorsharp_amd import hip_native as N
    if args.timeline == "layer":
        shapes, t = [(n, k) for _, n, k in LAYER], Q4_K
    else:
        t, n, k = (int(v) for v in args.timeline.split(","))
        shapes = [(n, k)]
    wbytes = sum(n * row_bytes(t, k) for n, k in shapes)
    copies = max(2, min(48, int(700e6 // wbytes) + 1))
    xs = [torch.randn((1, k), device=dev, dtype=torch.float32) for _, k in shapes]
    ys = [torch.empty((1, n), device=dev, dtype=torch.float32) for n, _ in shapes]
    # (the packs hold raw addresses: the weights must stay alive beside them)
    keep = [[QuantizedWeight(synth.random_weight(t, n, k, dev, seed=77 * c + i), t, k, n) for i, (n, k) in enumerate(shapes)]
            for c in range(copies)]
    packs = [HipBasicOps.PrepareGroup(ys, xs, ws) for ws in keep]
    cap_waves = 1 << 13
    reps = max(8, min(args.steps, 64))
    buf = torch.zeros((reps, cap_waves * 8), dtype=torch.int64, device=dev)
    set_region = lambda r: N.check_result(N.lib().TSHip_SetGemvTimeline(C.c_void_p(buf[r].data_ptr()), cap_waves * 64), "timeline")
    # a decode stream: launches back to back, every one of the last `reps` stamping a region of its own
    set_region(0)
    for i in range(300):
        HipBasicOps.AddmmQuantGroupDevice(packs[i % copies])
    buf.zero_()
    for r in range(reps):
        set_region(r)
        HipBasicOps.AddmmQuantGroupDevice(packs[r % copies])
    torch.cuda.synchronize()
    # the same stream timed with HIP events, with the stamping build and with the normal one
    step = lambda i: HipBasicOps.AddmmQuantGroupDevice(packs[i % copies])
    set_region(0)
    ev_tl = time_region(step, 1000, torch)[0]
    N.lib().TSHip_SetGemvTimeline(None, 0)
    for i in range(200):
        step(i)
    ev_plain = time_region(step, 1000, torch)[0]
    runs = []
    for r in range(reps):
        a = buf[r].cpu().numpy().reshape(-1, 8)
        runs.append(a[a[:, 4] != 0].copy())
    first = np.array([r[:, 0].min() for r in runs], dtype=np.int64)
    last = np.array([r[:, 4].max() for r in runs], dtype=np.int64)
    stream = {"period_us_p50": round(float(np.median(np.diff(first))) * 0.01, 2),
              "span_us_p50": round(float(np.median(last - first)) * 0.01, 2),
              "gap_last_exit_to_next_entry_us_p50": round(float(np.median(first[1:] - last[:-1])) * 0.01, 2),
              "events_us_per_launch_stamping_build": round(ev_tl, 2), "events_us_per_launch_normal_build": round(ev_plain, 2)}  # ms over 1000 launches = us per launch
    waves = runs[0].shape[0]
    rel = lambda col: np.median(np.stack([(r[:, col] - r[:, 0].min()) * 0.01 for r in runs]), axis=0)       # us
    e, xa, s_, f1, x = rel(0), rel(1), rel(2), rel(3), rel(4)
    has_xa = bool(np.all(runs[0][:, 1] != 0))        # the eager build of the kernel leaves no "activations arrived" stamp
    xcc = (runs[0][:, 5] & 0xff).astype(int)
    prob = ((runs[0][:, 5] >> 8) & 0xff).astype(int)
    q = lambda v: [round(float(np.percentile(v, p)), 2) for p in (0, 10, 50, 90, 100)]
    per_xcc = {}
    for c in sorted(set(xcc.tolist())):
        m = xcc == c
        per_xcc[str(c)] = {"waves": int(m.sum()), "entry_min_p50_max": [round(float(f(e[m])), 2) for f in (np.min, np.median, np.max)],
                           "exit_p0_p10_p50_p90_p100": q(x[m]), "life_p50": round(float(np.median(x[m] - e[m])), 2)}
    per_prob = {str(pi): {"waves": int((prob == pi).sum()), "entry_p50": round(float(np.median(e[prob == pi])), 2),
                          "activations_arrived_p50": round(float(np.median(xa[prob == pi])), 2) if has_xa else None,
                          "staged_p50": round(float(np.median(s_[prob == pi])), 2),
                          "first_step_done_p50": round(float(np.median(f1[prob == pi])), 2),
                          "exit_p0_p10_p50_p90_p100": q(x[prob == pi])} for pi in sorted(set(prob.tolist()))}
    return {"timeline": args.timeline, "type": t, "shapes": shapes, "weight_bytes": wbytes, "weight_copies": copies, "repetitions": reps,
            "wavefronts": int(waves), "clock": "s_memrealtime, 10 ns", "stream": stream,
            "entry_p0_p10_p50_p90_p100": q(e), "activations_arrived_p0_p10_p50_p90_p100": q(xa) if has_xa else None,
            "staged_p0_p10_p50_p90_p100": q(s_), "first_step_done_p0_p10_p50_p90_p100": q(f1), "exit_p0_p10_p50_p90_p100": q(x),
            "stage_time_p50": round(float(np.median(s_ - e)), 2), "per_xcc": per_xcc, "per_problem": per_prob}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--copies", type=int, default=6, help="distinct layer copies cycled (6 x 123 MB > Infinity Cache)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a plain 1 GiB device-to-device copy (20 times): the known-size kernel against "
                         "which rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled")
    ap.add_argument("--aux", metavar="OP,TYPE,ROWS,K",
                    help="time only the dequantizer (OP = dequant: ROWS x K weights to fp32) or the embedding gather "
                         "(OP = get_rows: ROWS random rows of a 131072 x K table); for profiling a single kernel")
    ap.add_argument("--matmul", metavar="TYPE,M,N,K",
                    help="time only one matmul shape (GGUF type id, rows, out features, in features) through "
                         "TSHip_AddmmQuantF32Device, --steps calls after --warmup; for profiling a single kernel")
    ap.add_argument("--timeline", metavar="layer|TYPE,N,K",
                    help="per-wavefront entry / staged / exit times of one decode launch (the headline grouped launch, or a "
                         "single matrix) from the library's timeline build of the GEMV kernel; prints a JSON summary")
    ap.add_argument("--moe", metavar="T", type=int,
                    help="time only the configs[3] MoE expert stage (32 MXFP4 experts, top-4, 2880) at T tokens, --steps calls; "
                         "for profiling its kernels")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures the one-GPU kernel path only: this build has no multi-GPU code; run with --gpus 1.",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from tensorsharp_amd import HipBasicOps, QuantizedWeight, synth

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback exists for the HIP path).", file=sys.stderr)
        sys.exit(3)
    if not HipBasicOps.IsAvailable():
        from tensorsharp_amd import hip_native
        print("HIP backend unavailable: " + hip_native.get_last_error(), file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    HipBasicOps.UseCurrentStream()

    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)       # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(20):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes_read": src.numel() * 4, "calibrate_copy_bytes_written": src.numel() * 4,
                          "launches": 20}))
        return

    def aux_case(op, t, rows, k, iters, warm):
        """dequantizer / embedding gather through the device entry points; HBM bytes = blocks read + fp32 written"""
        table_rows = rows if op == "dequant" else 131072
        w = QuantizedWeight(synth.random_weight(t, table_rows, k, dev, seed=31), t, k, table_rows)
        out_t = torch.empty((rows, k), device=dev, dtype=torch.float32)
        gi = torch.Generator(device="cpu")
        gi.manual_seed(5)
        idx = [torch.randint(0, table_rows, (rows,), generator=gi, dtype=torch.int32).to(dev) for _ in range(8)]

        def f(i):
            if op == "dequant":
                HipBasicOps.DequantizeToFloat32Device(t, w.data, rows * k, out_t.view(-1))
            else:
                HipBasicOps.GetRowsQuantDevice(out_t, w, idx[i % 8])
        for i in range(warm):
            f(i)
        ev, wall = time_region(f, iters, torch)
        us = ev * 1e3 / iters
        b = rows * row_bytes(t, k) + rows * k * 4
        return {"us_per_call_events": round(us, 2), "bytes": b, "GBps": round(b / (us * 1e-6) / 1e9, 1),
                "pct_hbm_peak": round(100 * b / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 1)}

    # MoE expert stage (configs[3]): 32 MXFP4 experts, top-4, hidden 2880; T = 1 (decode, HBM-bound:
    # bytes of the 4 selected experts' gate_up + down blocks) and T = 256 (prefill, grouped GEMM)
    def moe(T, iters):
        E, H, F, k = 32, 2880, 2880, 4
        sets = [(synth.random_weight(MXFP4, E * 2 * F, H, dev, seed=500 + c),
                 synth.random_weight(MXFP4, E * H, F, dev, seed=600 + c)) for c in range(2)]
        hidden = torch.randn((T, H), device=dev, dtype=torch.float32)
        gi = torch.Generator(device="cpu")
        gi.manual_seed(11)
        idsets = [torch.stack([torch.randperm(E, generator=gi)[:k] for _ in range(T)]).to(torch.int32).to(dev)
                  for _ in range(8)]
        wts = torch.softmax(torch.randn((T, k), device=dev), dim=1).contiguous()

        def f(i):
            gu, dn = sets[i % 2]
            HipBasicOps.MoEExpertsGptOssForward(hidden, idsets[i % 8], wts, gu, None, dn, None, MXFP4, E, H, F)
        for i in range(5):
            f(i)
        ev, wall = time_region(f, iters, torch)
        us = ev * 1e3 / iters
        res = {"us_per_call_events": round(us, 1)}
        if T == 1:
            b = k * (2 * F + H) * row_bytes(MXFP4, H)
            res.update({"bytes": b, "GBps": round(b / (us * 1e-6) / 1e9, 1),
                        "pct_hbm_peak": round(100 * b / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 1)})
        else:
            # weight-streaming bound (about 120 FLOP per weight byte): bytes of all 32 experts are the figure
            # of merit, TFLOP/s beside it
            b = E * (2 * F + H) * row_bytes(MXFP4, H)
            fl = 2.0 * T * k * (2 * F * H + H * F)
            res.update({"bytes": b, "GBps": round(b / (us * 1e-6) / 1e9, 1),
                        "pct_hbm_peak": round(100 * b / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 1),
                        "TFLOPs": round(fl / (us * 1e-6) / 1e12, 1),
                        "pct_mfma_fp16_peak": round(100 * fl / (us * 1e-6) / 1e12 / MFMA_FP16_PEAK_TFLOPS, 1)})
        return res


    if args.timeline:
        print(json.dumps(timeline(args, torch, dev, HipBasicOps, QuantizedWeight, synth)))
        return

    if args.aux:
        op, t, rows, k = args.aux.split(",")
        r = aux_case(op, int(t), int(rows), int(k), args.steps, args.warmup)
        r["aux"] = {"op": op, "type": int(t), "rows": int(rows), "K": int(k)}
        print(json.dumps(r))
        return

    if args.moe:
        r = moe(args.moe, args.steps)
        r["moe"] = {"tokens": args.moe}
        print(json.dumps(r))
        return

    if args.matmul:
        t, m, n, k = (int(v) for v in args.matmul.split(","))
        # decode shapes cycle enough distinct weight copies to exceed the 256 MB memory-side cache
        wbytes = n * row_bytes(t, k)
        copies = 1 if m > 8 else max(2, min(64, int(600e6 // wbytes) + 1))
        ws = [QuantizedWeight(synth.random_weight(t, n, k, dev, seed=91 + c), t, k, n) for c in range(copies)]
        x = torch.randn((m, k), device=dev, dtype=torch.float32)
        y = torch.empty((m, n), device=dev, dtype=torch.float32)

        # a single row goes through TSHip_AddmmQuantGroupF32Device with one problem and the arguments marshalled once
        # (the same launch; building the views in Python on every call costs more than a short launch lasts)
        packs = [HipBasicOps.PrepareGroup([y], [x], [w]) for w in ws] if m == 1 else None

        def one(i):
            if packs:
                HipBasicOps.AddmmQuantGroupDevice(packs[i % copies])
                return
            w = ws[i % copies]
            HipBasicOps.AddmmQuantDevice(y, x, w.ptr, t, k, n, w.raw_bytes)
        for i in range(args.warmup):
            one(i)
        ev, wall = time_region(one, args.steps, torch)
        us = ev * 1e3 / args.steps
        b = algorithmic_bytes(t, n, k, m)
        res = {"matmul": {"type": t, "M": m, "N": n, "K": k, "weight_copies": copies}, "us_per_call_events": round(us, 2), "bytes": b,
               "GBps": round(b / (us * 1e-6) / 1e9, 1), "TFLOPs": round(2.0 * m * n * k / (us * 1e-6) / 1e12, 2)}
        if m >= 128:
            res["library_dense_fp16_gemm_us"] = round(library_fp16_gemm_us(torch, dev, m, n, k, min(args.steps, 20)), 1)
        print(json.dumps(res))
        return

    # ---- workload: `copies` layers of seven Q4_K matrices, device resident -------------------
    layers = []
    for c in range(args.copies):
        ws = [QuantizedWeight(synth.random_weight(Q4_K, n, k, dev, seed=1000 * c + i), Q4_K, k, n)
              for i, (_, n, k) in enumerate(LAYER)]
        layers.append(ws)
    g = torch.Generator(device=dev)
    g.manual_seed(7)
    xs = [torch.randn((1, k), generator=g, device=dev, dtype=torch.float32) for _, _, k in LAYER]
    ys = [torch.empty((1, n), device=dev, dtype=torch.float32) for _, n, _ in LAYER]
    packs = [HipBasicOps.PrepareGroup(ys, xs, ws) for ws in layers]
    step_bytes = sum(algorithmic_bytes(Q4_K, n, k) for _, n, k in LAYER)

    def step(i):
        HipBasicOps.AddmmQuantGroupDevice(packs[i % len(packs)])

    for i in range(args.warmup):
        step(i)
    # exactly --steps steps between two synchronisations ...
    k_ev_ms, k_wall_ms = time_region(step, args.steps, torch)
    # ... and, because a region of a few steps of 25 us each is mostly the cost of the two synchronisations and the first
    # ~10 ms of launches after an idle period run slower (500 steps average 24.9 us per launch where 2000 average 24.15),
    # a region of at least 1000 steps, entered after at least 800 launches, from which `value` is taken; both are reported
    timed_steps = max(args.steps, 1000)
    if timed_steps == args.steps:
        ev_ms, wall_ms = k_ev_ms, k_wall_ms
    else:
        for i in range(max(0, 800 - args.warmup - args.steps)):
            step(i)
        ev_ms, wall_ms = time_region(step, timed_steps, torch)
    assert all(bool(torch.isfinite(y).all()) for y in ys)
    ms_per_step = wall_ms / timed_steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    kern_us = ev_ms * 1e3 / timed_steps         # one launch per step: HIP-event time per launch
    achieved = step_bytes / (kern_us * 1e-6) / 1e9

    traffic = measured_traffic_bytes()

    out = {
        "metric": "Q4_K/Q8_0/MXFP4 matmul: decode GB/s (% HBM peak), prefill TFLOP/s (% MFMA)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "timed_steps": timed_steps,
        "exact_steps_region": {"steps": args.steps, "ms_per_step_wall": round(k_wall_ms / args.steps, 5),
                               "ms_per_step_events": round(k_ev_ms / args.steps, 5),
                               "GBps_wall": round(step_bytes / (k_wall_ms / args.steps * 1e-3) / 1e9, 1)}, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "q4_k weights x f32 activations (fp16 operands, f32 accumulate)",
        "data": "synthetic: W ~ N(0,0.02) in Q4_K blocks (min/max-fit quantizer), x ~ N(0,1) f32, "
                f"{args.copies} distinct layer copies cycled",
        "config": {"workload": "configs[1]: Q4_K decode GEMV batch 1, one layer's 7 projections "
                               "(4096/14336/32q/8kv), one grouped launch per layer",
                   "bytes_per_step": step_bytes, "launches_per_step": 1, "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 1)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "kernel": "tship::gemv_kernel<12, 0, false, 0, 1> (grouped Q4_K GEMV)", "avg_launch_us": round(kern_us, 3),
                     "bytes_per_launch": step_bytes},
    }

    # ---- the prefill half of the metric: configs[4] Q4_K, M = 2048, N = 21504, K = 5376 -------------------------
    # One call = the activation convert kernel + the MFMA GEMM; the HIP events bracket whole calls, so `achieved` prices
    # both launches against the fp16 matrix peak (the GEMM kernel alone is in the rocprofv3 summary).
    def prefill(t, m, n, k, iters=20):
        w = QuantizedWeight(synth.random_weight(t, n, k, dev, seed=91), t, k, n)
        x = torch.randn((m, k), device=dev, dtype=torch.float32)
        y = torch.empty((m, n), device=dev, dtype=torch.float32)

        def f(i):
            HipBasicOps.AddmmQuantDevice(y, x, w.ptr, t, k, n, w.raw_bytes)
        for i in range(3):
            f(i)
        ev, wall = time_region(f, iters, torch)
        us = ev * 1e3 / iters
        tf = 2.0 * m * n * k / (us * 1e-6) / 1e12
        res = {"us_per_call_events": round(us, 1), "TFLOPs": round(tf, 1), "pct_mfma_fp16_peak": round(100 * tf / MFMA_FP16_PEAK_TFLOPS, 1)}
        if m >= 512 and t in (Q4_K, Q8_0) and not args.no_extra:
            del w, y
            lib = library_fp16_gemm_us(torch, dev, m, n, k)
            res["library_dense_fp16_gemm"] = {"us_per_call_events": round(lib, 1),
                                              "pct_mfma_fp16_peak": round(100 * 2.0 * m * n * k / (lib * 1e-6) / 1e12 / MFMA_FP16_PEAK_TFLOPS, 1)}
        return res

    pm, pn, pk = 2048, 21504, 5376
    pre = prefill(Q4_K, pm, pn, pk, 20)
    out["roofline_prefill"] = {
        "bound": "mfma", "achieved": pre["TFLOPs"], "peak": MFMA_FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": round(pre["TFLOPs"] / MFMA_FP16_PEAK_TFLOPS, 4), "traffic": None,
        "workload": "configs[4]: Q4_K prefill GEMM M=2048 N=21504 K=5376, fp16 operands, f32 accumulate",
        "kernel": "tship::gemm_xw_kernel<tship::PQ4K, 256, 4> (+ tship::convert_x_kernel on the activations, inside the timed call)",
        "avg_call_us": pre["us_per_call_events"], "flops_per_call": 2 * pm * pn * pk, "calls_timed": 20}

    # The same shape with MXFP4 weights (the third format of the metric; BASELINE names MXFP4 for the MoE stage only, so
    # this is beside the metric's own prefill figure, not in place of it): the weight blocks go to the block-scaled
    # matrix instruction as they are and every activation is two MX fp6 terms, so a k-tile is two fp6 x fp4 instructions
    # where fp16 operands take four of half the rate.  The kernel's operand type is fp6 x fp4, so `frac` prices the
    # algorithmic flops against that instruction's peak; the figure against the fp16 peak of the other formats, and the
    # instruction rate (two terms per activation: twice the algorithmic flops), stand beside it.
    if not args.no_extra:
        mx = prefill(MXFP4, pm, pn, pk, 20)
        out["roofline_prefill_mxfp4"] = {
            "bound": "mfma", "achieved": mx["TFLOPs"], "peak": MFMA_FP6_FP4_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(mx["TFLOPs"] / MFMA_FP6_FP4_PEAK_TFLOPS, 4), "traffic": None,
            "frac_of_fp16_peak": round(mx["TFLOPs"] / MFMA_FP16_PEAK_TFLOPS, 4),
            "workload": "MXFP4 prefill GEMM M=2048 N=21504 K=5376: raw fp4 blocks x two MX fp6 (E2M3) activation terms, f32 accumulate",
            "kernel": "tship::gemm_mx_kernel<256, 3> (+ tship::convert_x_mx_kernel on the activations, inside the timed call)",
            "avg_call_us": mx["us_per_call_events"], "flops_per_call": 2 * pm * pn * pk, "calls_timed": 20,
            "instruction_ops_over_fp6_fp4_peak": round(2 * mx["TFLOPs"] / MFMA_FP6_FP4_PEAK_TFLOPS, 4)}

    # ---- secondary workloads (reported, not the headline) ---------------------------------------
    if not args.no_extra:
        extra = {}
        n_it = max(200, args.steps // 4)

        def one_matrix(t, n, k, copies):
            ws = [QuantizedWeight(synth.random_weight(t, n, k, dev, seed=77 + c), t, k, n) for c in range(copies)]
            x = torch.randn((1, k), device=dev, dtype=torch.float32)
            y = torch.empty((1, n), device=dev, dtype=torch.float32)

            # arguments marshalled once per weight copy (TSHip_AddmmQuantGroupF32Device with one problem, as a decode loop
            # would hold them): building the views of TSHip_AddmmQuantF32Device in Python on every call costs about
            # 6.5 us, more than the shortest launches last, and would be what the events measure
            packs = [HipBasicOps.PrepareGroup([y], [x], [w]) for w in ws]

            def f(i):
                HipBasicOps.AddmmQuantGroupDevice(packs[i % copies])
            for i in range(50):
                f(i)
            ev, wall = time_region(f, n_it, torch)
            b = algorithmic_bytes(t, n, k)
            return {"us_per_launch_events": round(ev * 1e3 / n_it, 3), "GBps": round(b / (ev * 1e-3 / n_it) / 1e9, 1),
                    "pct_hbm_peak": round(100 * b / (ev * 1e-3 / n_it) / 1e9 / HBM_PEAK_GBS, 1), "bytes": b}

        extra["cfg1_q8_0_gemv_9728x2560"] = one_matrix(Q8_0, 9728, 2560, 12)
        for name, n, k in (("gate", 14336, 4096), ("down", 4096, 14336), ("wq", 4096, 4096), ("wk", 1024, 4096)):
            extra[f"cfg2_q4_k_gemv_{name}_{n}x{k}"] = one_matrix(Q4_K, n, k, max(2, int(300e6 // (n * row_bytes(Q4_K, k))) + 1))
        extra["cfg4_mxfp4_gemv_gate_up_5760x2880"] = one_matrix(MXFP4, 5760, 2880, 32)
        extra["cfg4_mxfp4_gemv_down_2880x2880"] = one_matrix(MXFP4, 2880, 2880, 64)
        # output projection of a 128k-vocabulary model (the largest single GEMV of a decode step): Q8_0, and Q6_K (what
        # Q4_K_M files store it in)
        n_it_save, n_it = n_it, 50
        extra["lm_head_q8_0_gemv_128256x4096"] = one_matrix(Q8_0, 128256, 4096, 2)
        extra["lm_head_q6_k_gemv_128256x4096"] = one_matrix(Q6_K, 128256, 4096, 2)
        extra["q6_k_gemv_down_4096x14336"] = one_matrix(Q6_K, 4096, 14336, 8)
        n_it = n_it_save

        # prefill GEMMs (configs[2] and configs[4]): TFLOP/s = 2*M*N*K / time of the whole call
        # (activation convert kernel + MFMA GEMM), fp16 operands -> priced against 2516.6 TFLOP/s
        extra["cfg3_q4_k_gemm_512x14336x4096"] = prefill(Q4_K, 512, 14336, 4096)
        extra["cfg5_q4_k_gemm_2048x21504x5376"] = pre
        extra["cfg5_q8_0_gemm_2048x21504x5376"] = prefill(Q8_0, 2048, 21504, 5376, 10)
        extra["cfg5_q4_k_gemm_2048x5376x21504"] = prefill(Q4_K, 2048, 5376, 21504, 10)
        extra["cfg5_q8_0_gemm_2048x5376x21504"] = prefill(Q8_0, 2048, 5376, 21504, 10)
        extra["mxfp4_gemm_2048x21504x5376"] = mx
        extra["mxfp4_gemm_2048x5376x21504"] = prefill(MXFP4, 2048, 5376, 21504, 10)
        extra["mxfp4_gemm_1024x5760x2880"] = prefill(MXFP4, 1024, 5760, 2880)
        # small batches (speculative decoding / few concurrent sequences): weight streaming, GB/s is the figure of merit
        for m in (8, 32, 128):
            r = prefill(Q4_K, m, 14336, 4096)
            b = algorithmic_bytes(Q4_K, 14336, 4096, m)
            r.update({"bytes": b, "GBps": round(b / (r["us_per_call_events"] * 1e-6) / 1e9, 1)})
            extra[f"q4_k_gemm_{m}x14336x4096"] = r
        extra["q6_k_gemm_512x14336x4096"] = prefill(Q6_K, 512, 14336, 4096)
        extra["cfg4_mxfp4_moe_experts_T1"] = moe(1, n_it)
        extra["cfg4_mxfp4_moe_experts_T256"] = moe(256, 30)
        # whole-layer decode (TransformerLayerDecode) at configs[1] shapes: hidden 4096, 32 heads / 8 KV heads of 128,
        # intermediate 14336, Q4_K weights (fused QKV 6144 x 4096 and gate_up 28672 x 4096), fp32 KV cache; 8 distinct
        # layers cycled (984 MB of weights).  Bytes = weights + the KV rows read by the attention.
        def layer_decode(context, iters):
            hidden, heads, kvh, hd, inter, max_seq = 4096, 32, 8, 128, 14336, 4096
            q_dim, k_dim = heads * hd, kvh * hd
            mk = lambda n, k, sd: QuantizedWeight(synth.random_weight(Q4_K, n, k, dev, seed=sd), Q4_K, k, n)
            layers = []
            for c in range(8):
                layers.append({"qkv": mk(q_dim + 2 * k_dim, hidden, 3000 + 10 * c), "o": mk(hidden, q_dim, 3001 + 10 * c),
                               "gate_up": mk(2 * inter, hidden, 3002 + 10 * c), "down": mk(hidden, inter, 3003 + 10 * c),
                               "attn_norm": torch.ones(hidden, device=dev), "ffn_norm": torch.ones(hidden, device=dev),
                               "q_norm": torch.ones(hd, device=dev), "k_norm": torch.ones(hd, device=dev),
                               "k_cache": torch.randn((kvh, max_seq, hd), device=dev), "v_cache": torch.randn((kvh, max_seq, hd), device=dev)})
            h = torch.randn(hidden, device=dev)
            pos = context - 1

            def f(i):
                L = layers[i % 8]
                HipBasicOps.TransformerLayerDecode(h, L["attn_norm"], L["qkv"], L["q_norm"], L["k_norm"], L["o"], L["ffn_norm"],
                                                   L["gate_up"], L["down"], L["k_cache"], L["v_cache"], heads, kvh, hd, pos, 1e-6,
                                                   10000.0, 1.0, 2)
                if i % 8 == 7:
                    h.normal_()           # keep the running hidden state bounded
            for i in range(16):
                f(i)
            ev, wall = time_region(f, iters, torch)
            us = ev * 1e3 / iters
            wbytes = sum(layers[0][k].raw_bytes for k in ("qkv", "o", "gate_up", "down"))
            b = wbytes + 2 * kvh * context * hd * 4
            return {"us_per_layer_events": round(us, 1), "bytes": b, "GBps": round(b / (us * 1e-6) / 1e9, 1),
                    "pct_hbm_peak": round(100 * b / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 1), "context": context}

        extra["cfg2_q4_k_layer_decode_ctx512"] = layer_decode(512, 200)
        extra["cfg2_q4_k_layer_decode_ctx4096"] = layer_decode(4096, 200)
        # One decode step of a whole model of these layers (llama-3-8B shapes: 32 layers, 128256-entry vocabulary): the
        # 32 layer calls as one TSHip_TransformerModelDecodeDevice call, then the final RMSNorm + LM head (Q6_K, as Q4_K_M
        # files store it) as one TSHip_FusedRmsNormMatMulQuantF32Device call.  32 distinct layers (3.9 GB of weights).
        # Embedding lookup and sampling are not included.
        def model_decode(context, n_layers=32, iters=30):
            hidden, heads, kvh, hd, inter, max_seq, vocab = 4096, 32, 8, 128, 14336, 1024, 128256
            q_dim, k_dim = heads * hd, kvh * hd
            mk = lambda t, n, k, sd: QuantizedWeight(synth.random_weight(t, n, k, dev, seed=sd), t, k, n)
            layers = []
            for c in range(n_layers):
                layers.append({"qkv": mk(Q4_K, q_dim + 2 * k_dim, hidden, 5000 + 10 * c), "o": mk(Q4_K, hidden, q_dim, 5001 + 10 * c),
                               "gate_up": mk(Q4_K, 2 * inter, hidden, 5002 + 10 * c), "down": mk(Q4_K, hidden, inter, 5003 + 10 * c),
                               "attn_norm": torch.ones(hidden, device=dev), "ffn_norm": torch.ones(hidden, device=dev),
                               "q_norm": None, "k_norm": None,
                               "k_cache": torch.randn((kvh, max_seq, hd), device=dev), "v_cache": torch.randn((kvh, max_seq, hd), device=dev)})
            head = mk(Q6_K, vocab, hidden, 5999)
            out_norm = torch.ones(hidden, device=dev)
            logits = torch.empty((1, vocab), device=dev)
            h = torch.randn(hidden, device=dev)

            def f(i):
                HipBasicOps.TransformerModelDecode(h, layers, heads, kvh, hd, context - 1, 1e-6, 500000.0, 1.0, 2)
                HipBasicOps.FusedRmsNormMatMulQuant(logits, h.view(1, hidden), out_norm, 1e-6, head)
                h.normal_()
            for i in range(3):
                f(i)
            ev, wall = time_region(f, iters, torch)
            ms = ev / iters
            wbytes = n_layers * sum(layers[0][k].raw_bytes for k in ("qkv", "o", "gate_up", "down")) + head.raw_bytes
            b = wbytes + n_layers * 2 * kvh * context * hd * 4
            return {"ms_per_token_events": round(ms, 3), "tokens_per_s": round(1e3 / ms, 1), "bytes": b,
                    "GBps": round(b / (ms * 1e-3) / 1e9, 1), "pct_hbm_peak": round(100 * b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 1),
                    "layers": n_layers, "context": context, "launches_per_token": 6 * n_layers + 1}

        extra["llama8b_shape_q4_k_model_decode_ctx512"] = model_decode(512)
        # the same seven matrices as the headline, but as the dependent chain a decode step really runs (RMSNorm + QKV,
        # attention over 512 cached tokens, Wo + residual, RMSNorm + gate | up + SiLU, down + residual: six launches):
        # every launch pays its start, its tail and the gap to the next one, which the grouped launch pays once
        chain = extra["cfg2_q4_k_layer_decode_ctx512"]
        out["roofline_decode_chain"] = {
            "bound": "hbm", "achieved": chain["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(chain["GBps"] / HBM_PEAK_GBS, 4), "traffic": None,
            "workload": "configs[1] shapes as one dependent decode layer at context 512 (TSHip_TransformerLayerDecodeDevice)",
            "kernel": "six launches: tship::gemv_one_kernel<12, ...> x 4, tship::attn_decode_kernel, tship::attn_combine_kernel",
            "avg_call_us": chain["us_per_layer_events"], "bytes_per_call": chain["bytes"]}
        # fused SwiGLU FFN at decode (configs[1] shapes: hidden 4096, intermediate 14336, Q4_K, one token):
        # RMSNorm -> gate_up GEMV -> SiLU*up -> down GEMV + residual, one ABI call (4 launches)
        def fused_ffn(copies=3):
            Hd, Fd = 4096, 14336
            ws = [(QuantizedWeight(synth.random_weight(Q4_K, 2 * Fd, Hd, dev, seed=700 + c), Q4_K, Hd, 2 * Fd),
                   QuantizedWeight(synth.random_weight(Q4_K, Hd, Fd, dev, seed=800 + c), Q4_K, Fd, Hd)) for c in range(copies)]
            x = torch.randn((1, Hd), device=dev)
            nw = torch.ones(Hd, device=dev)
            res = torch.zeros((1, Hd), device=dev)

            def f(i):
                gu, dn = ws[i % copies]
                HipBasicOps.FusedFFNSwiGLUQuant(res, x, nw, 1e-6, gu, dn, Fd)
            for i in range(20):
                f(i)
            ev, wall = time_region(f, n_it, torch)
            us = ev * 1e3 / n_it
            b = (2 * Fd + Hd) * row_bytes(Q4_K, Hd) + 0  # gate_up rows of K=4096 ...
            b = 2 * Fd * row_bytes(Q4_K, Hd) + Hd * row_bytes(Q4_K, Fd)
            return {"us_per_call_events": round(us, 2), "bytes": b, "GBps": round(b / (us * 1e-6) / 1e9, 1),
                    "pct_hbm_peak": round(100 * b / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 1)}

        extra["cfg2_q4_k_fused_ffn_decode_4096x14336"] = fused_ffn()
        # dequantizer and embedding gather (HBM-bound: blocks read + fp32 written)
        extra["dequant_q4_k_14336x4096"] = aux_case("dequant", Q4_K, 14336, 4096, 50, 5)
        extra["dequant_q8_0_9728x2560"] = aux_case("dequant", Q8_0, 9728, 2560, 50, 5)
        extra["get_rows_q8_0_512_of_131072x4096"] = aux_case("get_rows", Q8_0, 512, 4096, 50, 5)
        out["extra"] = extra

    if not args.no_cpu:
        n_threads = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1)
        n_threads = min(n_threads, os.cpu_count() or 1)
        layer_host = [w.data.cpu().numpy() for w in layers[0]]
        xs_host = [x.cpu().numpy() for x in xs]
        out["cpu_baseline"] = cpu_baseline(layer_host, xs_host, n_threads)
        try:
            ggml = cpu_reference_ggml(layer_host, xs_host, n_threads)
        except (OSError, AssertionError, AttributeError) as e:      # reported beside the port, never required
            ggml = {"error": str(e)}
        if ggml is not None:
            out["cpu_baseline_ggml"] = ggml

    print(json.dumps(out))


if __name__ == "__main__":
    main()
