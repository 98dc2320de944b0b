"""The gradient-set workloads of this path measured as whole steps: `python bench.py --config {2,3,4,5}`.

    2  speech DNN (429-2048x7-9304: 16 matrices, 45.1 M parameters), 1 bit, mean threshold:
       quantize the set + unquantize the set, one gradient-set call each
    3  ResNet-50 (161 matrices, 25.6 M parameters), 2 / 4 / 8 bits (one JSON line per bit width): the same two calls
    4  1-bit all-reduce of 8 workers x 2048 x 9304 simulated in one GPU's memory: the 8 workers' quantizations (one
       call), the 8 owners' stripe reductions (one call, an owner per item), the packed aggregate unquantized into
       worker 0's gradient from the owners' stripes (one call)
    5  LSTM language model (100000x512, 4 x 1024x4096, 512x100000: 119 M parameters), 1 bit, zeroThresholdFor1Bit on:
       quantize the set + unquantize the set

Every line: algorithmic bytes per step (the per-element figures of the plain calls summed over the set), host-clock
time per step between two device synchronisations (`value` = bytes / that), the GPU's own time for the K steps between
two events on the stream, the duration of every call of a step (events recorded on the stream before and after the call,
in a separate pass: they include the gap of about 2 us before the call's first kernel), and `roofline` for the call that
takes most of the step. Residuals are carried (in place) from step to step; buffer sets are rotated so that no call finds
its inputs in the 256 MB last-level cache; every buffer set has its own quantizer handle, because a handle caches the
argument table of the last item list it saw.
"""
import ctypes
import json
import time

HBM_PEAK_GBS = 8000.0

SPEECH_DNN = [(429, 2048)] + [(2048, 2048)] * 6 + [(2048, 9304)] + [(2048, 1)] * 7 + [(9304, 1)]
LSTM_LM = [(100000, 512), (1024, 4096), (1024, 4096), (1024, 4096), (1024, 4096), (512, 100000)]


def resnet50_shapes():
    """53 convolutions as [kH*kW*Cin, Cout], the 2048x1000 classifier with its bias, batch-norm scale and bias per convolution."""
    convs = [(147, 64)]

    def stage(cin, mid, cout, blocks):
        out = [(cin, mid), (9 * mid, mid), (mid, cout), (cin, cout)]
        for _ in range(blocks - 1):
            out += [(cout, mid), (9 * mid, mid), (mid, cout)]
        return out

    convs += stage(64, 64, 256, 3) + stage(256, 128, 512, 4) + stage(512, 256, 1024, 6) + stage(1024, 512, 2048, 3)
    shapes = list(convs) + [(2048, 1000), (1000, 1)]
    for _, cout in convs:
        shapes += [(cout, 1), (cout, 1)]
    return shapes


def quantize_bytes(rows, cols, nbits):
    return rows * cols * 12 + packed_bytes(rows, cols, nbits)


def unquantize_bytes(rows, cols, nbits):
    return rows * cols * 4 + packed_bytes(rows, cols, nbits)


def packed_bytes(rows, cols, nbits):
    per = 32 // nbits
    return cols * (8 + 4 * ((rows + per - 1) // per))


class _Events:
    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]

    def new(self):
        e = ctypes.c_void_p()
        if self.hip.hipEventCreate(ctypes.byref(e)) != 0:
            raise RuntimeError("hipEventCreate failed")
        return e

    def record(self, e):
        # the null stream: where a handle without a dedicated stream issues, and torch's current stream here
        if self.hip.hipEventRecord(e, None) != 0:
            raise RuntimeError("hipEventRecord failed")

    def ms(self, a, b):
        out = ctypes.c_float()
        if self.hip.hipEventElapsedTime(ctypes.byref(out), a, b) != 0:
            raise RuntimeError("hipEventElapsedTime failed")
        return out.value


def _gradient(torch, gen, rows, cols, kind):
    n = rows * cols
    if kind == "student_t3":
        z = torch.randn(n, generator=gen, device="cuda:0", dtype=torch.float32)
        chi = torch.randn(3, n, generator=gen, device="cuda:0", dtype=torch.float32).square_().sum(0)
        return z / torch.sqrt(chi / 3.0) * 1e-3
    if kind == "outliers":
        a = torch.randn(n, generator=gen, device="cuda:0", dtype=torch.float32) * 0.01
        return torch.where(torch.rand(n, generator=gen, device="cuda:0") < 0.01, a * 50.0, a)
    g = torch.randn(n, generator=gen, device="cuda:0", dtype=torch.float32) * 0.01
    if kind == "sparse_columns" and rows >= 100000:
        keep = (torch.rand(cols, generator=gen, device="cuda:0") >= 0.9).to(torch.float32)
        g.view(cols, rows).mul_(keep[:, None])
    return g


def _gradient_set_steps(torch, shapes, nbits, zt, kind, sets_wanted):
    """Buffer sets for 'quantize the set, unquantize the set'. Returns (list of step closures, call names, bytes per call)."""
    from cntk_amd import Matrix, MatrixQuantizerImpl, QuantizedMatrix

    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(0x1B17 + nbits)
    steps = []
    keep = []
    for _ in range(sets_wanted):
        qz = MatrixQuantizerImpl.Create(0, False)
        G = [Matrix(r, c, 0, _gradient(torch, gen, r, c, kind)) for r, c in shapes]
        R = [Matrix(r, c) for r, c in shapes]
        Q = [QuantizedMatrix(r, c, nbits, 0) for r, c in shapes]
        Out = [Matrix(r, c) for r, c in shapes]
        pq = qz.PrepareQuantizeBatch([(G[i], R[i], Q[i], R[i]) for i in range(len(shapes))])
        pu = qz.PrepareUnquantizeBatch([(Q[i], Out[i]) for i in range(len(shapes))])
        keep.append((qz, G, R, Q, Out, pq, pu))
        steps.append([lambda qz=qz, pq=pq: qz.QuantizeBatchAsync(pq, zt), lambda qz=qz, pu=pu: qz.UnquantizeBatchAsync(pu, False)])
    names = ["quantize (gradient-set call)", "unquantize (gradient-set call)"]
    nbytes = [sum(quantize_bytes(r, c, nbits) for r, c in shapes), sum(unquantize_bytes(r, c, nbits) for r, c in shapes)]
    return steps, names, nbytes, keep


def _allreduce_steps(torch, rows, cols, k, nbits, zt, sets_wanted):
    """K workers in one GPU's memory: all workers' quantizations, all owners' stripe reductions, the aggregate decoded
    on worker 0 from the owners' stripes where they lie."""
    import cntk_amd
    from cntk_amd import Matrix, MatrixQuantizerImpl, QuantizedMatrix

    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(0x1B17 + 4000)
    steps, keep = [], []
    for _ in range(sets_wanted):
        qz = MatrixQuantizerImpl.Create(0, False)
        G = [Matrix(rows, cols, 0, _gradient(torch, gen, rows, cols, "normal")) for _ in range(k)]
        R = [Matrix(rows, cols) for _ in range(k)]
        Q = [QuantizedMatrix(rows, cols, nbits, 0) for _ in range(k)]
        ranges = [cntk_amd.stripe_range(cols, s, k) for s in range(k)]
        S = [Matrix(rows, n) for _, n in ranges]
        pq = qz.PrepareQuantizeBatch([(G[w], R[w], Q[w], R[w]) for w in range(k)])
        items, owners, views = [], [], []
        for s, (start, n) in enumerate(ranges):
            if n == 0:
                continue
            stripes = [Q[w].ColumnSlice(start, n) for w in range(k)]
            items.append((stripes, S[s], stripes[s], None))
            owners.append(s)
            views.append((stripes[s], G[0].ColumnSlice(start, n)))
        ps = qz.PrepareStripeReduceBatch(items)
        pu = qz.PrepareUnquantizeBatch(views)
        keep.append((qz, G, R, Q, S, pq, ps, pu, items, views))
        steps.append([lambda qz=qz, pq=pq: qz.QuantizeBatchAsync(pq, zt),
                      lambda qz=qz, ps=ps, owners=owners: qz.StripeReduceBatchAsync(ps, owners, zt),
                      lambda qz=qz, pu=pu: qz.UnquantizeBatchAsync(pu, False)])
    n = rows * cols
    qb = packed_bytes(rows, cols, nbits)
    names = ["quantize, all workers (one gradient-set call)", "stripe reduction, all owners (one call, an owner per item)",
             "unquantize of the packed aggregate (one gradient-set call over the owners' stripes)"]
    nbytes = [k * quantize_bytes(rows, cols, nbits), 8 * n + (k + 1) * qb, unquantize_bytes(rows, cols, nbits)]
    return steps, names, nbytes, keep


def run(config, steps=200, warmup=20, nbits_list=None, emit=True):
    """Measures workload `config`; returns its JSON lines (one per bit width for workload 3) and, with `emit`, prints them."""
    import torch

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    ev = _Events()
    lines = []
    if config == 3:
        variants = [(b, False) for b in (nbits_list or [2, 4, 8])]
    elif config == 5:
        variants = [(1, True)]
    else:
        variants = [(1, False)]
    for nbits, zt in variants:
        if config == 2:
            shapes, label = SPEECH_DNN, "speech DNN gradient set (16 matrices, 45,122,648 parameters), Student-t(3) x 1e-3"
            sets, names, nbytes, keep = _gradient_set_steps(torch, shapes, nbits, zt, "student_t3", 3)
        elif config == 3:
            shapes, label = resnet50_shapes(), "ResNet-50 gradient set (161 matrices, 25,557,032 parameters), N(0, 1e-4) with 1% outliers at 50x"
            sets, names, nbytes, keep = _gradient_set_steps(torch, shapes, nbits, zt, "outliers", 4)
        elif config == 4:
            label = "1-bit all-reduce, 8 workers x 2048 x 9304 in one GPU's memory (stripes of 2048 x 1163)"
            sets, names, nbytes, keep = _allreduce_steps(torch, 2048, 9304, 8, nbits, zt, 2)
        elif config == 5:
            shapes, label = LSTM_LM, "LSTM language-model gradient set (6 matrices, 119,177,216 parameters), embedding with 90% all-zero columns"
            sets, names, nbytes, keep = _gradient_set_steps(torch, shapes, nbits, zt, "sparse_columns", 2)
        else:
            raise SystemExit("bench.py --config takes 2, 3, 4 or 5 (config 1 is a parity case, the default run is the headline)")
        torch.cuda.synchronize()

        def step(i):
            for call in sets[i % len(sets)]:
                call()

        # the first call of a list builds and uploads its argument table; clocks settle over some tenths of a second
        t_setup = time.perf_counter()
        n_setup = 0
        while n_setup < 3 * len(sets) or time.perf_counter() - t_setup < 0.3:
            step(n_setup)
            n_setup += 1
            if n_setup % 8 == 0:
                torch.cuda.synchronize()
        for i in range(warmup):
            step(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            step(warmup + i)
        t_enq = time.perf_counter()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        sec = (t1 - t0) / steps

        # second pass: the GPU's own time for the same K steps
        a, b = ev.new(), ev.new()
        ev.record(a)
        for i in range(steps):
            step(warmup + i)
        ev.record(b)
        torch.cuda.synchronize()
        timeline_ms = ev.ms(a, b) / steps

        # third pass: every call between two events
        n_timed = min(steps, 40)
        marks = [[ev.new() for _ in range(len(names) + 1)] for _ in range(n_timed)]
        for i in range(n_timed):
            calls = sets[(warmup + i) % len(sets)]
            ev.record(marks[i][0])
            for c, call in enumerate(calls):
                call()
                ev.record(marks[i][c + 1])
            if i % 8 == 7:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        call_ms = [sum(ev.ms(m[c], m[c + 1]) for m in marks) / n_timed for c in range(len(names))]

        # fourth pass: the kernels of every call by events tied to the dispatches themselves (set when the call's first
        # launch starts and when its last one ends): no command between the launches, no launch floor in the figure
        from cntk_amd import lib
        L = lib()
        L.cntkq_debug_attach_events.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        spans = [[(ev.new(), ev.new()) for _ in names] for _ in range(n_timed)]
        for i in range(n_timed):
            j = (warmup + i) % len(sets)
            handle = keep[j][0]._h
            for c, call in enumerate(sets[j]):
                if L.cntkq_debug_attach_events(handle, spans[i][c][0], spans[i][c][1]) != 0:
                    raise RuntimeError("cntkq_debug_attach_events failed")
                call()
            if i % 8 == 7:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        kern_ms = [sum(ev.ms(sp[c][0], sp[c][1]) for sp in spans) / n_timed for c in range(len(names))]
        total = sum(nbytes)
        dom = max(range(len(names)), key=lambda c: kern_ms[c])
        achieved = nbytes[dom] / (kern_ms[dom] * 1e-3) / 1e9
        line = {
            "config": config,
            "metric": "gradient-set step GB/s (algorithmic bytes) & % HBM peak",
            "value": round(total / sec / 1e9, 2),
            "unit": "GB/s",
            "pct_hbm_peak": round(100.0 * total / sec / 1e9 / HBM_PEAK_GBS, 2),
            "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": round(sec * 1e3, 5),
            "gpu_timeline_ms_per_step": round(timeline_ms, 5),
            "host_enqueue_ms_per_step": round((t_enq - t0) / steps * 1e3, 5),
            "dtype": "f32", "data": "synthetic",
            "workload": {"workload": label, "nbits": nbits, "zero_threshold_for_1bit": zt, "buffer_sets": len(sets),
                         "algorithmic_bytes_per_step": total},
            # us: between two events recorded on the stream around the call (includes the launch floor of a few microseconds
            # and the records themselves); kernels_us: first launch start to last launch end by dispatch-attached events
            "calls": [{"call": names[c], "us": round(call_ms[c] * 1e3, 2), "kernels_us": round(kern_ms[c] * 1e3, 2),
                       "algorithmic_bytes": nbytes[c], "GBps": round(nbytes[c] / (call_ms[c] * 1e-3) / 1e9, 1),
                       "kernels_GBps": round(nbytes[c] / (kern_ms[c] * 1e-3) / 1e9, 1)} for c in range(len(names))],
            "calls_timed": n_timed,
            "roofline": {"bound": "hbm", "kernel": names[dom], "timed": "kernels_us", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "algorithmic_bytes_per_launch": nbytes[dom],
                         "traffic": None},
        }
        if emit:
            print(json.dumps(line), flush=True)
        lines.append(line)
        del sets, keep
        torch.cuda.empty_cache()
    return lines
