#!/usr/bin/env python3
"""Headline benchmark: 1-bit quantize + unquantize of a 2048 x 9304 fp32 gradient with in-place residual.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = QuantizeAsync (gradient + carried residual -> packed codes + new residual) followed by UnquantizeAsync
(packed codes -> fp32), through the C ABI, inputs resident in device memory. Buffer sets are rotated so that no step
finds its inputs in the 256 MB Infinity Cache. Prints ONE JSON line.

  value     algorithmic GB/s of the whole step: (16 + nbits/4) bytes per element + 16 bytes per column
            = 309,785,984 bytes for 2048 x 9304 at 1 bit, divided by the step time. The step time is the host clock
            around exactly K steps between two device synchronisations; nothing but the 2 K calls is issued in
            between, so with few steps the launch latency of the first kernel and the return of the closing wait
            are part of it (a 20-step run is about 1 ms long). gpu_timeline_ms_per_step, from a second pass of the
            same K steps, is first kernel start -> last kernel end by dispatch-attached events.
  roofline  the dominant kernel (quantize): algorithmic bytes per launch (12 + nbits/8 per element + 8 per column
            = 231,111,360) over its average duration measured with HIP events on the launch stream in a third,
            untimed pass of the same steps, against 8 TB/s of HBM
  cpu_baseline  the reference's own CPU quantizer (its headers, compiled under oracle/_ref) where that build is present,
            else the CPU oracle (a port of it), timed on this host, single thread like the reference, on the same
            matrix; the compiler flags of both CPU libraries are stated in the line
  configs   after the headline's timed region and event passes (so `value` is untouched), the other workloads of this
            path as whole steps through the gradient-set calls: speech DNN set (1 bit), ResNet-50 set (2, 4, 8 bits),
            the simulated 8-worker all-reduce of 2048 x 9304, the LSTM language-model set (1 bit, zero threshold); for
            each: step time, % of HBM peak, every call of a step timed between two stream events, and the roofline
            of the longest call (`--no-configs` leaves them out; `--config N` runs one of them alone)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

ROWS, COLS, NBITS = 2048, 9304, 1
# untimed set-up before the warm-up steps the caller asks for (handle, streams, clocks): at least this many steps and
# this much time
SETUP_STEPS = 50
SETUP_SECONDS = 0.5
HBM_PEAK_GBS = 8000.0


def algorithmic_bytes(rows, cols, nbits):
    elems = rows * cols
    quant = elems * 12 + elems * nbits // 8 + cols * 8
    unquant = elems * 4 + elems * nbits // 8 + cols * 8
    return quant, unquant


def cpu_baseline(budget_s=12.0):
    """Times the CPU oracle on the full 2048 x 9304 matrix (single thread, like the reference CPU quantizer)."""
    import numpy as np

    import datagen
    import oracle

    g = datagen.normal(datagen.case_seed(0), ROWS, COLS, 0.01)
    r = np.zeros_like(g, order="F")
    out = np.zeros_like(g, order="F")
    qb, ub = algorithmic_bytes(ROWS, COLS, NBITS)

    def run(threads, budget, use_ref=False):
        best = float("inf")
        passes = 0
        t_end = time.perf_counter() + budget
        while passes < 3 or (time.perf_counter() < t_end and passes < 40):
            t0 = time.perf_counter()
            q, _ = oracle.quantize(g, r, NBITS, False, r_out=r, threads=threads, use_ref=use_ref)
            oracle.unquantize(q, ROWS, COLS, NBITS, out=out, threads=threads, use_ref=use_ref)
            best = min(best, time.perf_counter() - t0)
            passes += 1
        return best, passes

    # the reference's own CPU quantizer (its headers, compiled under oracle/_ref) where that build is present; it is
    # single-threaded, like the reference's CPU path
    have_ref = oracle.ref_available()
    t1, p1 = run(1, budget_s if not have_ref else budget_s / 2)
    tr, pr = run(1, budget_s / 2, use_ref=True) if have_ref else (None, 0)
    cores = min(16, os.cpu_count() or 1)
    cpu_model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    cpu_model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    tn, pn = run(cores, budget_s / 3)
    tb = tr if have_ref else t1
    flags = oracle.build_flags()
    return {
        "value": round((qb + ub) / tb / 1e9, 4),
        "unit": "GB/s",
        "cores": 1,
        "kind": "reference" if have_ref else "port",
        "compiler_flags": {"reference": flags.get("CXXFLAGS"), "port": flags.get("CFLAGS"), "compilers": "g++ / gcc"},
        "port": {"cores": 1, "value": round((qb + ub) / t1 / 1e9, 4), "ms_per_step": round(t1 * 1e3, 2), "passes": p1},
        "cpu_model": cpu_model,
        "host_cpus": os.cpu_count(),
        "sample": "%d passes of quantize+unquantize over the full %dx%d fp32 matrix, 1 bit, best pass" % (pr if have_ref else p1, ROWS, COLS),
        "ms_per_step": round(tb * 1e3, 2),
        "elements_per_s": round(ROWS * COLS / tb, 1),
        "port_all_cores": {"cores": cores, "value": round((qb + ub) / tn / 1e9, 4), "ms_per_step": round(tn * 1e3, 2),
                      "passes": pn},
    }


TRAFFIC_PROFILE = os.path.join("profiles", "quantize_unquantize_2048x9304_1bit.md")


def profiled_traffic():
    """HBM bytes per launch of the quantize kernel from the committed counter summary (a line
    `traffic_bytes_per_launch quantize = N` in it), with the file it came from; (None, None) if there is none."""
    import re

    try:
        with open(os.path.join(ROOT, TRAFFIC_PROFILE)) as f:
            m = re.search(r"^\s*traffic_bytes_per_launch quantize = (\d+)", f.read(), re.M)
    except OSError:
        return None, None
    if not m:
        return None, None
    return int(m.group(1)), TRAFFIC_PROFILE + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a plain copy of known size)"


def rnd(x, n):
    return None if x is None else round(x, n)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)  # 53 ms of GPU time
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--zero-threshold", type=int, default=0, help="zeroThresholdFor1Bit (default off, as in config 1)")
    ap.add_argument("--sets", type=int, default=6, help="rotating buffer sets (each 231 MB)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-events", action="store_true",
                    help="skip the two untimed passes that carry HIP events (GPU timeline, kernel durations)")
    ap.add_argument("--event-every", type=int, default=2,
                    help="kernel-duration pass: attach timing events to the kernels of every n-th step")
    ap.add_argument("--config", type=int, default=0,
                    help="instead of the headline, one of the gradient-set workloads as whole steps: 2 speech DNN set (1 bit), "
                         "3 ResNet-50 set (2, 4, 8 bits: one line each), 4 simulated 8-worker all-reduce of 2048x9304, "
                         "5 LSTM language-model set (1 bit, zero threshold); one JSON line per workload with the time of "
                         "every call of a step and the roofline of the longest")
    ap.add_argument("--no-configs", action="store_true", help="headline only: skip the other four workloads that follow it")
    ap.add_argument("--config-steps", type=int, default=100, help="timed steps of each of the workloads that follow the headline")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="instead of the benchmark, run plain device copies of one 2048x9304 fp32 matrix "
                         "(76,218,368 bytes read and as many written per copy), for scaling hardware counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU only (K workers are simulated in one GPU's memory); "
                 "--gpus %d is not supported" % args.gpus)

    if args.config:
        from cntk_amd import config_bench

        # (the headline's defaults are 1000 steps of 52 us; a gradient-set step takes 0.1 - 0.7 ms)
        config_bench.run(args.config, steps=min(args.steps, 200), warmup=min(args.warmup, 20))
        return

    import torch

    import cntk_amd
    from cntk_amd import Matrix, MatrixQuantizerImpl, QuantizedMatrix

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = "cuda:0"
    if args.copy_calibration:
        src = [torch.randn(ROWS * COLS, device=dev, dtype=torch.float32) for _ in range(args.sets)]
        dst = [torch.empty(ROWS * COLS, device=dev, dtype=torch.float32) for _ in range(args.sets)]
        torch.cuda.synchronize()
        for i in range(args.steps):
            dst[i % args.sets].copy_(src[i % args.sets])
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": True, "copies": args.steps, "bytes_read_per_copy": ROWS * COLS * 4,
                          "bytes_written_per_copy": ROWS * COLS * 4}), flush=True)
        return
    zt = bool(args.zero_threshold)
    qz = MatrixQuantizerImpl.Create(0, False)  # issues on the main (null) stream = torch's current stream

    gen = torch.Generator(device=dev)
    gen.manual_seed(0x1B17)
    sets = []
    for _ in range(args.sets):
        G = Matrix(ROWS, COLS, 0, torch.randn(ROWS * COLS, generator=gen, device=dev, dtype=torch.float32) * 0.01)
        sets.append((G, Matrix(ROWS, COLS), QuantizedMatrix(ROWS, COLS, NBITS, 0), Matrix(ROWS, COLS)))
    torch.cuda.synchronize()

    # The timed loop calls the C ABI directly with pre-computed pointers: two calls per step, so that the host
    # stays well ahead of the GPU and the measured time is the GPU's.
    L, h = cntk_amd.lib(), qz._h
    qbytes = sets[0][2].GetSize()
    ptrs = [(G.Data(), R.Data(), Q.Buffer(), Out.Data()) for G, R, Q, Out in sets]
    izt = int(zt)

    # HIP events with timing, tied to the kernel dispatches themselves (start when the kernel begins, stop when it
    # has finished) on the stream the handle launches on: separate event records would idle the GPU for several
    # microseconds per kernel and show up in the very time they measure.
    import ctypes

    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
    hip.hipEventDestroy.argtypes = [ctypes.c_void_p]

    def new_event():
        e = ctypes.c_void_p()
        if hip.hipEventCreate(ctypes.byref(e)) != 0:
            raise RuntimeError("hipEventCreate failed")
        return e

    def elapsed_ms(a, b):
        ms = ctypes.c_float()
        if hip.hipEventElapsedTime(ctypes.byref(ms), a, b) != 0:
            raise RuntimeError("hipEventElapsedTime failed")
        return ms.value

    L.cntkq_debug_attach_events.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]

    def step(i, ev=None):
        g, r, q, o = ptrs[i % len(ptrs)]
        if ev is not None:
            L.cntkq_debug_attach_events(h, ev[0], ev[1])
        rc1 = L.cntkq_quantize_async(h, g, r, ROWS, COLS, q, qbytes, 0, NBITS, r, izt)
        if ev is not None:
            L.cntkq_debug_attach_events(h, ev[2], ev[3])
        rc2 = L.cntkq_unquantize_async(h, q, qbytes, 0, o, ROWS, COLS, NBITS, 0)
        if rc1 or rc2:
            raise RuntimeError(L.cntkq_last_error().decode())

    # set-up, outside warm-up and timing: first calls create streams and events, and the GPU needs some tenths of a
    # second of steady work before its clocks and memory system reach the state a training job runs in (measured: the
    # same kernels take 38.9 + 13.4 us in the first milliseconds after start-up and 37.7 + 12.6 us from then on)
    setup_steps = 0
    t_setup = time.perf_counter()
    while setup_steps < SETUP_STEPS or time.perf_counter() - t_setup < SETUP_SECONDS:
        for i in range(50):
            step(setup_steps + i)
        setup_steps += 50
        torch.cuda.synchronize()
    setup_s = time.perf_counter() - t_setup
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()

    # Timed region: exactly `steps` steps and nothing else, host clock around a device synchronisation on both sides.
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(args.warmup + i)
    t_enqueued = time.perf_counter()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    sec_per_step = (t1 - t0) / args.steps

    # Second pass, not part of `value`: the same steps again with a start event tied to the first dispatch and a stop
    # event to the last one, i.e. the GPU's own time for the K steps including the gaps between dependent launches but
    # without the launch latency of the first kernel and the return of the closing wait.
    # Third pass: start/stop events on the two kernels of every n-th step, for the kernel durations of `roofline`.
    # Creating a profiled dispatch costs the host about 25 us, which is why neither is done inside the timed region.
    timeline_ms = q_ms = u_ms = None
    n_timed = 0
    if not args.no_events:
        first, last = new_event(), new_event()
        none = ctypes.c_void_p()
        for i in range(args.steps):
            g, r, q, o = ptrs[(args.warmup + i) % len(ptrs)]
            if i == 0:
                L.cntkq_debug_attach_events(h, first, none)
            rc1 = L.cntkq_quantize_async(h, g, r, ROWS, COLS, q, qbytes, 0, NBITS, r, izt)
            if i == args.steps - 1:
                L.cntkq_debug_attach_events(h, none, last)
            rc2 = L.cntkq_unquantize_async(h, q, qbytes, 0, o, ROWS, COLS, NBITS, 0)
            if rc1 or rc2:
                raise RuntimeError(L.cntkq_last_error().decode())
        torch.cuda.synchronize()
        timeline_ms = elapsed_ms(first, last) / args.steps
        hip.hipEventDestroy(first)
        hip.hipEventDestroy(last)

        every = max(1, args.event_every)
        events = {i: [new_event() for _ in range(4)] for i in range(0, args.steps, every)}
        for i in range(args.steps):
            step(args.warmup + i, events.get(i))
        torch.cuda.synchronize()
        q_ms = sum(elapsed_ms(e[0], e[1]) for e in events.values()) / len(events)
        u_ms = sum(elapsed_ms(e[2], e[3]) for e in events.values()) / len(events)
        n_timed = len(events)
        for e in events.values():
            for x in e:
                hip.hipEventDestroy(x)
    qb, ub = algorithmic_bytes(ROWS, COLS, NBITS)
    total = qb + ub
    achieved = qb / (q_ms * 1e-3) / 1e9 if q_ms else None
    traffic, traffic_source = profiled_traffic()

    result = {
        "metric": "1-bit quantize+unquantize GB/s & % HBM peak, 2048x9304 fp32 gradient",
        "value": round(total / sec_per_step / 1e9, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "setup_steps": setup_steps,
        "setup_s": round(setup_s, 3),
        "ms_per_step": round(sec_per_step * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "quantize+unquantize 2048x9304 fp32, 1 bit, in-place residual carried across steps, "
                        "zeroThresholdFor1Bit %s" % ("on" if zt else "off"),
            "rows": ROWS, "cols": COLS, "nbits": NBITS, "zero_threshold_for_1bit": zt,
            "buffer_sets": len(sets), "algorithmic_bytes_per_step": total,
        },
        "pct_hbm_peak": round(100.0 * total / sec_per_step / 1e9 / HBM_PEAK_GBS, 2),
        "elements_per_s": round(ROWS * COLS / sec_per_step, 1),
        "gpu_timeline_ms_per_step": rnd(timeline_ms, 5),
        "kernel_ms": {"quantize": rnd(q_ms, 5), "unquantize": rnd(u_ms, 5), "launches_timed": n_timed},
        "host_enqueue_ms_per_step": round((t_enqueued - t0) / args.steps * 1e3, 5),
        "roofline": {
            "bound": "hbm",
            "kernel": "quantize (gradient + residual -> codes + residual)",
            "achieved": rnd(achieved, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": rnd(achieved / HBM_PEAK_GBS, 4) if achieved else None,
            "algorithmic_bytes_per_launch": qb,
            # not observed by this run: HBM bytes per launch of the quantize kernel as recorded in the committed
            # rocprofv3 counter summary (FETCH_SIZE + WRITE_SIZE, two runs, each scaled by what the same counter
            # reads for a plain device copy of known size); null when that file is absent
            "traffic": traffic,
            "traffic_source": traffic_source,
        },
    }
    if not args.no_configs:
        # the other workloads, after everything of the headline has been measured; the headline's buffers go first
        from cntk_amd import config_bench

        del sets, ptrs
        torch.cuda.empty_cache()
        configs = {}
        for cfg in (2, 3, 4, 5):
            for line in config_bench.run(cfg, steps=args.config_steps, warmup=10, emit=False):
                key = "%d_%dbit" % (cfg, line["workload"]["nbits"]) if cfg == 3 else str(cfg)
                configs[key] = {k: line[k] for k in ("value", "unit", "pct_hbm_peak", "steps", "warmup", "ms_per_step",
                                                     "gpu_timeline_ms_per_step", "workload", "calls", "calls_timed", "roofline")}
        result["configs"] = configs
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
