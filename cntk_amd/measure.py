"""Kernel timing for one matrix shape: quantize, unquantize and (optionally) the fused stripe reduction.

    python -m cntk_amd.measure --rows 2048 --cols 9304 --nbits 1 [--dtype f64] [--workers 8] [--zero-threshold 1]
                               [--steps 40] [--path 0..6]

Calls the C ABI directly. Every launch is timed with HIP events tied to the kernel dispatch (start when it begins,
stop when it has finished) on the stream the handle launches on; buffer sets are rotated so that no launch finds its
inputs in the 256 MB Infinity Cache. Prints one JSON line with the average kernel durations and the algorithmic
GB/s of each:
    quantize    elements * (3 * elem_bytes) + packed bytes
    unquantize  elements * elem_bytes + packed bytes
    stripe      workers * packed bytes in, packed bytes out, stripe residual read and written
"""
import argparse
import ctypes
import json
import sys

import torch

import cntk_amd
from cntk_amd import Matrix, MatrixQuantizerImpl, QuantizedMatrix


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--rows", type=int, required=True)
    ap.add_argument("--cols", type=int, required=True)
    ap.add_argument("--nbits", type=int, default=1)
    ap.add_argument("--dtype", choices=["f32", "f64"], default="f32")
    ap.add_argument("--zero-threshold", type=int, default=0)
    ap.add_argument("--workers", type=int, default=0, help="also time the stripe reduction over this many packed stripes")
    ap.add_argument("--steps", type=int, default=40)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--path", type=int, default=0, help="force a quantize kernel: 1 tile, 2 tall (re-reading), 3 column in LDS, 4 column in registers (16-byte accesses), "
                    "5 column in registers (one element per access), 6 several workgroups per column (strips)")
    ap.add_argument("--unq-mode", type=int, default=0, help="decoder choice: 0 automatic, 1 QWord-major with one store per value, 2 tile decoder, 3 automatic without the tile "
                    "decoder, 4 row-major decoder with the packed column in LDS, 5 row-major decoder that fetches its QWords itself, 6 the same over short columns")
    ap.add_argument("--tile-gs", type=int, default=0, help="threads per column of the tile kernels' statistics phase (0: the library's choice)")
    ap.add_argument("--budget-mb", type=int, default=1600, help="device memory for the rotating buffer sets")
    args = ap.parse_args()

    assert torch.cuda.is_available(), "needs the GPU"
    tdt = torch.float64 if args.dtype == "f64" else torch.float32
    eb = 8 if args.dtype == "f64" else 4
    rows, cols, nbits, zt = args.rows, args.cols, args.nbits, int(bool(args.zero_threshold))
    sfx = "_f64" if args.dtype == "f64" else ""
    L = cntk_amd.lib()
    qz = MatrixQuantizerImpl.Create(0, False)
    qz._set_tuning(quantize_path=args.path, unq_mode=args.unq_mode, tile_gs=args.tile_gs)
    h = qz._h

    # no fused stripe reduction above this height: the other two calls are still measured
    stripe_limit = getattr(L, "cntkq_stripe_reduce_max_rows" + sfx)(nbits)
    stripe_skipped = bool(args.workers) and not qz.StripeReduceTakes(rows, cols, nbits, zt, tdt)
    if stripe_skipped:
        args.workers = 0

    elems = rows * cols
    qbytes = QuantizedMatrix(rows, cols, nbits, 0, dtype=tdt).GetSize()
    per_set = elems * eb * 3 + qbytes * (1 + max(args.workers - 1, 0))
    nsets = max(2, min(12, (args.budget_mb << 20) // max(per_set, 1)))
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(7)
    sets = []
    for _ in range(nsets):
        G = Matrix(rows, cols, 0, (torch.randn(elems, generator=gen, device="cuda:0", dtype=torch.float32) * 0.01).to(tdt))
        R, Out = Matrix(rows, cols, dtype=tdt), Matrix(rows, cols, dtype=tdt)
        Q = QuantizedMatrix(rows, cols, nbits, 0, dtype=tdt)
        peers = [QuantizedMatrix(rows, cols, nbits, 0, dtype=tdt) for _ in range(max(args.workers - 1, 0))]
        sets.append((G, R, Q, Out, peers))
    torch.cuda.synchronize()

    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
    L.cntkq_debug_attach_events.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]

    def new_event():
        e = ctypes.c_void_p()
        if hip.hipEventCreate(ctypes.byref(e)) != 0:
            raise RuntimeError("hipEventCreate failed")
        return e

    def check(rc):
        if rc:
            raise RuntimeError(L.cntkq_last_error().decode())

    quantize = getattr(L, "cntkq_quantize_async" + sfx)
    unquantize = getattr(L, "cntkq_unquantize_async" + sfx)
    stripe = getattr(L, "cntkq_stripe_reduce_async" + sfx)

    # peers' packed stripes: quantize each set's gradient into them once (same bytes; only the traffic matters)
    for G, R, Q, Out, peers in sets:
        for P in peers:
            check(quantize(h, G.Data(), Out.Data(), rows, cols, P.Buffer(), qbytes, 0, nbits, Out.Data(), zt))
    torch.cuda.synchronize()

    total = args.warmup + args.steps
    evs = [[new_event() for _ in range(6)] for _ in range(args.steps)]
    for i in range(total):
        G, R, Q, Out, peers = sets[i % nsets]
        e = evs[i - args.warmup] if i >= args.warmup else None
        if e:
            L.cntkq_debug_attach_events(h, e[0], e[1])
        check(quantize(h, G.Data(), R.Data(), rows, cols, Q.Buffer(), qbytes, 0, nbits, R.Data(), zt))
        if args.workers:
            arr = (ctypes.c_void_p * args.workers)(Q.Buffer(), *[P.Buffer() for P in peers])
            if e:
                L.cntkq_debug_attach_events(h, e[4], e[5])
            check(stripe(h, arr, args.workers, 0, rows, cols, nbits, Out.Data(), Q.Buffer(), None, zt))
        if e:
            L.cntkq_debug_attach_events(h, e[2], e[3])
        check(unquantize(h, Q.Buffer(), qbytes, 0, Out.Data(), rows, cols, nbits, 0))
        if i % 8 == 7:
            torch.cuda.synchronize()  # keeps the host from running far ahead with profiled dispatches
    torch.cuda.synchronize()

    def avg_ms(a, b):
        tot = 0.0
        for e in evs:
            ms = ctypes.c_float()
            if hip.hipEventElapsedTime(ctypes.byref(ms), e[a], e[b]) != 0:
                raise RuntimeError("hipEventElapsedTime failed")
            tot += ms.value
        return tot / len(evs)

    q_ms, u_ms = avg_ms(0, 1), avg_ms(2, 3)
    q_bytes, u_bytes = elems * 3 * eb + qbytes, elems * eb + qbytes
    out = {
        "rows": rows, "cols": cols, "nbits": nbits, "dtype": args.dtype, "zero_threshold": bool(zt), "buffer_sets": nsets,
        "launches_timed": args.steps,
        "quantize": {"us": round(q_ms * 1e3, 2), "algorithmic_bytes": q_bytes, "GBps": round(q_bytes / q_ms / 1e6, 1)},
        "unquantize": {"us": round(u_ms * 1e3, 2), "algorithmic_bytes": u_bytes, "GBps": round(u_bytes / u_ms / 1e6, 1)},
    }
    if stripe_skipped:
        out["stripe_reduce"] = {"skipped": "columns of %d rows: the fused stripe reduction does not take them at %d bits (at most %d, and taller ones "
                                            "where the strip kernels do)" % (rows, nbits, stripe_limit)}
    if args.workers:
        s_ms = avg_ms(4, 5)
        s_bytes = (args.workers + 1) * qbytes + 2 * elems * eb
        out["stripe_reduce"] = {"workers": args.workers, "us": round(s_ms * 1e3, 2), "algorithmic_bytes": s_bytes,
                                "GBps": round(s_bytes / s_ms / 1e6, 1)}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    sys.exit(main())
