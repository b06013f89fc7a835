"""Benchmark sweeps of the two modules, the counterpart of the reference's notebook
(test_speed.ipynb cells 4-19: ``perf_report`` sweeps of T, E, B and I around the default shape
B64 T256 E32 K32 I128 J64, forward+backward time and peak memory of ``module(x, Ind).sum().backward()``).

    python -m expertscattergather_amd.sweep [--op gather|scatter|both] [--axis T|E|B|I|all]
                                            [--dtype bf16|f16|f32] [--ind-dtype int16|int32|int64]
                                            [--reps 50] [--csv out.csv]

Prints one line per point: median forward+backward time (HIP events around the autograd call, warm),
the same with the step replayed as a HIP graph where capture works, and ``torch.cuda.max_memory_allocated``
of one step.  Inputs follow the notebook: x ~ N(0,1), Ind uniform in [0, T) (with replacement), int16 by default.
"""
from __future__ import annotations

import argparse
import csv
import sys

import torch

DEFAULT = dict(B=64, T=256, E=32, K=32, I=128, J=64)
AXES = {
    "T": [32, 64, 128, 256, 384, 512, 640],          # test_speed.ipynb:225-244
    "E": [6, 12, 24, 32, 48, 60],                    # :363-372
    "B": [32, 64, 96, 128, 160],                     # :480-484
    "I": [128, 256, 512, 768],                       # :586-588
}
DTYPES = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}
IND_DTYPES = {"int16": torch.int16, "int32": torch.int32, "int64": torch.int64}


def _median_ms(fn, reps):
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        times.append(a.elapsed_time(b))
    times.sort()
    return times[len(times) // 2]


def measure(op, dims, dtype, ind_dtype, reps):
    from . import ExpertGather, ExpertScatter, hip_kernels
    B, T, E, K, I, J = (dims[k] for k in ("B", "T", "E", "K", "I", "J"))
    dev = torch.device("cuda:0")
    hip_kernels.release_workspaces()        # scratch of earlier points and of their capture streams
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    base_bytes = torch.cuda.memory_allocated()
    gen = torch.Generator(device="cpu").manual_seed(0)
    Ind = torch.randint(0, T, (B, E, K), generator=gen).to(ind_dtype).to(dev)
    if op == "gather":
        mod = ExpertGather(E, I, J).to(dev, dtype)
        x = torch.randn(B, T, I, generator=gen).to(dtype).to(dev).requires_grad_(True)
        step = lambda: mod(x, Ind).sum().backward()
    else:
        mod = ExpertScatter(E, J, I).to(dev, dtype)
        x = torch.randn(B, E, K, J, generator=gen).to(dtype).to(dev).requires_grad_(True)
        step = lambda: mod(x, Ind, T).sum().backward()
    step()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    step()
    torch.cuda.synchronize()
    peak_mb = (torch.cuda.max_memory_allocated() - base_bytes) / 2 ** 20       # parameters, inputs, gradients, scratch
    eager_ms = _median_ms(step, reps)
    graph_ms = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            step()
        graph_ms = _median_ms(g.replay, reps)
    except Exception:                       # capture is a bonus; the eager number stands
        torch.cuda.synchronize()
    return eager_ms, graph_ms, peak_mb


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--op", default="both", choices=["gather", "scatter", "both"])
    ap.add_argument("--axis", default="all", choices=["T", "E", "B", "I", "all"])
    ap.add_argument("--dtype", default="bf16", choices=list(DTYPES))
    ap.add_argument("--ind-dtype", default="int16", choices=list(IND_DTYPES))
    ap.add_argument("--reps", type=int, default=50)
    ap.add_argument("--csv", default=None)
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("sweep: needs a GPU (the kernels have no CPU fallback)", file=sys.stderr)
        return 2
    ops = ["gather", "scatter"] if args.op == "both" else [args.op]
    axes = list(AXES) if args.axis == "all" else [args.axis]
    rows = []
    print(f"{'op':8s} {'axis':4s} {'value':>6s} {'fwd+bwd ms':>11s} {'graph ms':>9s} {'peak MB':>9s}")
    for op in ops:
        for axis in axes:
            for v in AXES[axis]:
                dims = dict(DEFAULT)
                dims[axis] = v
                if dims["K"] > dims["T"]:
                    continue
                eager_ms, graph_ms, peak = measure(op, dims, DTYPES[args.dtype], IND_DTYPES[args.ind_dtype], args.reps)
                g = f"{graph_ms:9.4f}" if graph_ms is not None else f"{'-':>9s}"
                print(f"{op:8s} {axis:4s} {v:6d} {eager_ms:11.4f} {g} {peak:9.1f}", flush=True)
                rows.append({"op": op, "axis": axis, "value": v, "fwd_bwd_ms": eager_ms, "graph_ms": graph_ms, "peak_mb": peak,
                             "dtype": args.dtype, "ind_dtype": args.ind_dtype})
    if args.csv:
        with open(args.csv, "w", newline="") as fh:
            w = csv.DictWriter(fh, fieldnames=list(rows[0].keys()))
            w.writeheader()
            w.writerows(rows)
    return 0


if __name__ == "__main__":
    sys.exit(main())
