#!/usr/bin/env python3
"""Benchmark of the fused expert gather/scatter path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input at the default shape in
bf16 (B64 T256 E32 K32 I128 J64): gather forward -> scatter forward -> scatter backward (dY,
dW_scatter) -> gather backward (dX, dW_gather), i.e. the six kernel-equivalents of a full
autograd forward+backward.  Inputs are resident in HBM before the timed region starts.

Prints ONE JSON line.  `value` is microseconds per step (lower is better) of the step issued
through the drop-in modules and PyTorch's autograd (`ExpertScatter(ExpertGather(x, Ind), Ind,
T).backward(dOut)`), by the fastest of three ways of issuing it that `config.launch` names
(eager, a HIP graph of one step, a HIP graph of several steps); the same step through the four
launcher callables is reported beside it (`launcher_us_per_step`).  `roofline` describes the
dominant launch of the step, the one that takes the most time (algorithmic bytes or flops / its
average duration, measured with HIP events on the launch stream, warm and with the caches
flushed), `roofline_per_launch` every launch; `configs` holds the step and the per-launch times
of the other benchmark configurations; `cpu_baseline` is the torch port of the reference's
baselines timed on the host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0       # MI355X HBM3E, published
# MI355X dense matrix peaks (TFLOP/s) of the arithmetic each configuration multiplies in
MFMA_PEAK_TFLOPS = {"f32": 157.3, "bf16": 2500.0, "f16": 2500.0, "fp8": 5000.0}

PROFILES = os.path.join(ROOT, "profiles")


def kernel_list(kernels):
    """'a + b + a + b + c' -> '2 x (a + b) + c'; a call that works through batch groups launches the same kernels once per group"""
    out, i, n = [], 0, len(kernels)
    while i < n:
        best = (1, 1)                       # (period, repeats) of the longest repeated run that starts at i
        for period in range(1, (n - i) // 2 + 1):
            reps = 1
            while kernels[i + reps * period:i + (reps + 1) * period] == kernels[i:i + period]:
                reps += 1
            if reps > 1 and reps * period > best[0] * best[1]:
                best = (period, reps)
        period, reps = best
        unit = " + ".join(kernels[i:i + period])
        out.append(f"{reps} x ({unit})" if reps > 1 else unit)
        i += period * reps
    return " + ".join(out)


def recorded_traffic():
    """HBM-side bytes per launch from the rocprofv3 --pmc summaries under profiles/ (FETCH_SIZE + WRITE_SIZE of
    `bench.py --pmc-probe` runs, each scaled by what the same counter reads for a 64 MiB copy).  Counters cannot be read
    from inside this process, so the figures are the recorded ones: lines
    `traffic <workload> <launch> <bytes> <kernel>+<kernel>...`; the last field names the kernels the launch ran when the
    counters were read (a launch has one line per set of kernels it can select, e.g. per scatter mode), and a figure is
    reported only for the set of kernels selected now."""
    import glob
    import re
    found = {}
    for path in sorted(glob.glob(os.path.join(PROFILES, "*.md")) + glob.glob(os.path.join(PROFILES, "*.txt"))):
        for m in re.finditer(r"^\s*traffic (\S+) (\S+) (\d+)[ \t]+(\S+)\s*$", open(path).read(), flags=re.M):
            found[(m.group(1), m.group(2), tuple(sorted(set(m.group(4).split("+")))))] = {
                "bytes": int(m.group(3)), "source": os.path.relpath(path, ROOT)}
    return found


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="C2", help="workload (C2 = the metric's configuration)")
    ap.add_argument("--mode", default=None, choices=["deterministic", "atomic", "compact"], help="scatter mode (default: env / deterministic)")
    ap.add_argument("--fp8-act", action="store_true",
                    help="C5 only: quantise the activations per row to e4m3 and multiply on the fp8 matrix instruction")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only, no HIP graph replays")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="C2 only: skip the other configurations (the `configs` key)")
    ap.add_argument("--kernel-reps", type=int, default=200, help="launches per kernel for the per-kernel timing")
    ap.add_argument("--no-cold", action="store_true", help="skip the timing of each launch with the caches flushed in between")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="only launch a 64 MiB device copy (3x) and one entry point of the path (5x), for rocprofv3 --pmc runs")
    ap.add_argument("--probe-kernel", default="gather", choices=["gather", "scatter", "dw", "scatter_bwd", "gather_bwd", "mlp", "mlp_separate"],
                    help="which entry point --pmc-probe launches: gather forward, scatter forward, the stand-alone weight "
                         "gradient, one of the two backward calls (each shares its launch with a weight gradient), the "
                         "inference block gather -> relu -> scatter as one kernel (mlp; 16-bit small-expert shapes) or the "
                         "same as three launches (mlp_separate)")
    return ap.parse_args()


def time_loop(fn, n):
    import torch
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / n


def graph_of(fn, steps_per_graph):
    """`steps_per_graph` calls of fn captured into one HIP graph (on a side stream, after three eager calls there)."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        keep = [fn() for _ in range(steps_per_graph)]
    return graph, keep


def steps_per_graph_for(steps, most=20):
    """the largest divisor of `steps` up to `most`: K timed steps are then a whole number of replays"""
    return max(d for d in range(1, most + 1) if steps % d == 0)


def time_routes(fn, steps, warmup, no_graph, many):
    """us per call of `fn` issued eagerly, as a HIP graph of one call, and (`many`) as a HIP graph of several calls
    replayed back to back (a replay costs a fixed few microseconds on top of its kernels, whatever it holds)."""
    import torch
    for _ in range(max(warmup, 3)):
        fn()
    out = {"eager": time_loop(fn, steps) * 1e6, "graph": None, "graph_many": None, "steps_per_graph": None}
    if no_graph:
        return out
    try:
        graph, keep = graph_of(fn, 1)
        for _ in range(max(warmup, 3)):
            graph.replay()
        out["graph"] = time_loop(graph.replay, steps) * 1e6
        del graph, keep
        if many:
            spg = steps_per_graph_for(steps)
            graph, keep = graph_of(fn, spg)
            for _ in range(3):
                graph.replay()
            out["graph_many"] = time_loop(graph.replay, steps // spg) * 1e6 / spg
            out["steps_per_graph"] = spg
            del graph, keep
    except Exception as exc:        # report, fall back to the eager number
        print(f"bench.py: graph capture failed ({exc}); reporting eager timing", file=sys.stderr)
    torch.cuda.synchronize()
    return out


def best_route(routes):
    labels = {"eager": "eager launches", "graph": "hip graph replay, one step per replay",
              "graph_many": f"hip graph replay, {routes['steps_per_graph']} steps per replay"}
    name = min((k for k in labels if routes.get(k) is not None), key=lambda k: routes[k])
    return routes[name], labels[name]


class Workload:
    """One benchmark configuration resident on the GPU: the step through the Python ops and every launch of the step
    through the C ABI on preallocated outputs."""

    def __init__(self, name, mode, fp8_act=False):
        import torch
        from expertscattergather_amd import _abi, hip_kernels as hk, workloads as wl
        self.torch, self.hk, self.abi, self.wl = torch, hk, _abi, wl
        self.name, self.mode = name, mode
        self.cfg = cfg = wl.CONFIGS[name]
        self.dims = B, T, E, K, I, J = cfg.dims
        self.dev = dev = torch.device("cuda:0")
        self.inp = inp = wl.make_inputs(cfg)
        self.X, self.Wg, self.Ws, self.dOut, self.Ind = (inp[k].to(dev) for k in ("X", "Wg", "Ws", "dOut", "Ind"))
        self.fwd_only = name in ("C1", "C5")
        self.fp8 = name == "C5"
        self.fp8_act = self.fp8 and fp8_act
        if self.fp8:        # the configuration's weights: e4m3 bytes and a per-expert, per-column fp32 scale
            self.Wq_c, self.scale_c = wl.quantize_fp8_weights(inp["Wg"].float())
            self.Wq, self.Wscale = self.Wq_c.to(dev), self.scale_c.to(dev)
        self.dtype_name = "bf16" if cfg.dtype == torch.bfloat16 else ("f16" if cfg.dtype == torch.float16 else "f32")
        self.mfma_peak = MFMA_PEAK_TFLOPS["fp8" if self.fp8_act else self.dtype_name]
        self._launch_fns = None

    # ---- the step through the four launcher callables
    def step(self):
        torch, hk = self.torch, self.hk
        X, Wg, Ws, dOut, Ind, T = self.X, self.Wg, self.Ws, self.dOut, self.Ind, self.dims[1]
        # a training step routes anew: the table that the gather forward leaves with Ind for the scatter forward and the
        # gather's backward is rebuilt in every step, never carried over from the step before
        hk.invalidate_routing_table(Ind)
        with hk.scatter_mode_scope(self.mode):
            if self.fp8_act:
                Y = hk.expert_gather_fp8_forward(X, self.Wq, self.Wscale, Ind)
            elif self.fp8:
                Y = hk.expert_gather_fp8w_forward(X, self.Wq, self.Wscale, Ind)
            else:
                Y = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)
            out = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
            if self.fwd_only:
                return Y, out
            dY, dWs = hk.expert_scatter_backward_call(Y, Ws, Ind, dOut, torch.float32)
            dX, dWg = hk.expert_gather_backward_call(X, Wg, Ind, dY, torch.float32)
        return Y, out, dX, dWg, dWs

    # ---- the same step through the modules and autograd
    def autograd_step_fn(self):
        torch, hk = self.torch, self.hk
        import expertscattergather_amd as egs
        B, T, E, K, I, J = self.dims
        gmod = egs.ExpertGather(E, I, J).to(self.dev, self.cfg.dtype)
        smod = egs.ExpertScatter(E, J, I).to(self.dev, self.cfg.dtype)
        gmod.scatter_mode = smod.scatter_mode = self.mode
        with torch.no_grad():
            gmod.W.copy_(self.Wg); smod.W.copy_(self.Ws)
        xg = self.X.clone().requires_grad_(True)
        Ind, dOut = self.Ind, self.dOut

        def autograd_step():
            hk.invalidate_routing_table(Ind)
            xg.grad = None; gmod.W.grad = None; smod.W.grad = None
            smod(gmod(xg, Ind), Ind, T).backward(dOut)
            return xg.grad, gmod.W.grad, smod.W.grad

        return autograd_step

    # ---- every launch of the step through the C ABI, on preallocated outputs
    def launch_fns(self):
        if self._launch_fns is not None:
            return self._launch_fns
        torch, hk, _abi, wl = self.torch, self.hk, self.abi, self.wl
        cfg, dev = self.cfg, self.dev
        B, T, E, K, I, J = self.dims
        X, Wg, Ws, dOut, Ind = self.X, self.Wg, self.Ws, self.dOut, self.Ind
        fp8, fp8_act = self.fp8, self.fp8_act
        lib = _abi.lib()
        d = _abi.Dims(B, T, E, K, I, J)
        dt = hk.dtype_to_type_id(cfg.dtype)
        stream = torch.cuda.current_stream().cuda_stream
        Y = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32) if not fp8 else hk.expert_gather_fp8w_forward(X, self.Wq, self.Wscale, Ind)
        out = torch.empty(B, T, I, device=dev, dtype=cfg.dtype)
        dYb, dXb = torch.empty_like(Y), torch.empty(B, T, I, device=dev, dtype=cfg.dtype)
        dWg_b, dWs_b = torch.empty(E, I, J, device=dev, dtype=cfg.dtype), torch.empty(E, J, I, device=dev, dtype=cfg.dtype)
        mode = hk._MODES[self.mode]
        ws_bytes = max(lib.egs_workspace_bytes(_abi.OP_GATHER_BACKWARD, mode, d, dt), lib.egs_workspace_bytes(_abi.OP_DW, mode, d, dt), 256)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        f8ws_bytes = lib.egs_gather_gemm_fp8act_workspace_bytes(d) if fp8_act else 0
        f8ws = torch.empty(max(f8ws_bytes, 256), dtype=torch.uint8, device=dev)
        I64 = _abi.IND_I64
        # the launches as a step issues them: where the sizes have a routing table, the gather forward builds it and the
        # scatter forward and the gather's backward read it
        tab_bytes = 0 if fp8 else lib.egs_routing_table_bytes(d, dt)
        tab = torch.empty(max(tab_bytes, 256), dtype=torch.uint8, device=dev)
        self.tab_bytes = int(tab_bytes)
        self.keep = (Y, out, dYb, dXb, dWg_b, dWs_b, ws, f8ws, tab)

        def k_gather():
            if fp8_act:     # row quantiser + fp8 x fp8 product: both launches are part of the call
                return lib.egs_gather_gemm_fp8act(X.data_ptr(), self.Wq.data_ptr(), self.Wscale.data_ptr(), Ind.data_ptr(), Y.data_ptr(),
                                                  f8ws.data_ptr(), f8ws_bytes, d, T * I, I, I64, stream)
            if fp8:
                return lib.egs_gather_gemm(X.data_ptr(), self.Wq.data_ptr(), Ind.data_ptr(), Y.data_ptr(), self.Wscale.data_ptr(), d, T * I, I,
                                           dt, _abi.FP8_E4M3, I64, _abi.W_EIJ, stream)
            if tab_bytes:
                return lib.egs_expert_gather_forward_table(X.data_ptr(), Wg.data_ptr(), Ind.data_ptr(), Y.data_ptr(), tab.data_ptr(),
                                                           tab_bytes, d, T * I, I, dt, I64, stream)
            return lib.egs_expert_gather_forward(X.data_ptr(), Wg.data_ptr(), Ind.data_ptr(), Y.data_ptr(), d, T * I, I, dt, I64, stream)

        def k_scatter():
            if tab_bytes:
                return lib.egs_expert_scatter_forward_table(Y.data_ptr(), Ws.data_ptr(), Ind.data_ptr(), tab.data_ptr(), tab_bytes,
                                                            out.data_ptr(), ws.data_ptr(), ws_bytes, d, dt, I64, mode, stream)
            return lib.egs_expert_scatter_forward(Y.data_ptr(), Ws.data_ptr(), Ind.data_ptr(), out.data_ptr(), ws.data_ptr(), ws_bytes, d,
                                                  dt, I64, mode, stream)

        def k_scatter_bwd():
            return lib.egs_expert_scatter_backward(Y.data_ptr(), Ws.data_ptr(), Ind.data_ptr(), dOut.data_ptr(), dYb.data_ptr(),
                                                   dWs_b.data_ptr(), ws.data_ptr(), ws_bytes, d, T * I, I, dt, I64, stream)

        def k_gather_bwd():
            if tab_bytes:
                return lib.egs_expert_gather_backward_table(X.data_ptr(), Wg.data_ptr(), Ind.data_ptr(), tab.data_ptr(), tab_bytes,
                                                            dYb.data_ptr(), dXb.data_ptr(), dWg_b.data_ptr(), ws.data_ptr(), ws_bytes,
                                                            d, T * I, I, dt, I64, mode, stream)
            return lib.egs_expert_gather_backward(X.data_ptr(), Wg.data_ptr(), Ind.data_ptr(), dYb.data_ptr(), dXb.data_ptr(),
                                                  dWg_b.data_ptr(), ws.data_ptr(), ws_bytes, d, T * I, I, dt, I64, mode, stream)

        def k_dw():
            return lib.egs_dw(X.data_ptr(), Y.data_ptr(), Ind.data_ptr(), dWg_b.data_ptr(), ws.data_ptr(), ws_bytes, d, T * I, I, dt, dt,
                              I64, _abi.W_EIJ, stream)

        act = 2 if cfg.dtype != torch.float32 else 4
        gemm_bytes = wl.algorithmic_bytes(self.dims, act)
        gather_bytes = wl.algorithmic_bytes(self.dims, act, w_bytes=1, fp8_scales=True) if fp8 else gemm_bytes
        dw_bytes = wl.algorithmic_bytes(self.dims, act, dw=True)
        kflops = wl.flops(self.dims)
        # launch -> (function, algorithmic bytes, flops): the backward calls compute two kernel-equivalents each
        launches = {"expert_gather_forward": (k_gather, gather_bytes, kflops), "expert_scatter_forward": (k_scatter, gemm_bytes, kflops)}
        if not self.fwd_only:
            launches["expert_scatter_backward"] = (k_scatter_bwd, gemm_bytes + dw_bytes, 2 * kflops)
            launches["expert_gather_backward"] = (k_gather_bwd, gemm_bytes + dw_bytes, 2 * kflops)
        self.k_dw = k_dw
        self.chain_bytes = (gather_bytes + gemm_bytes) if self.fwd_only else 4 * gemm_bytes + 2 * dw_bytes
        self.chain_flops = (2 if self.fwd_only else 6) * kflops
        assert k_gather() == 0      # the table is in place before the launches that read it are timed
        # the kernels each launch selects for these operands, as the library reports them
        self.kernels = {}
        for lname, (fn, _, _) in launches.items():
            with _abi.launch_log() as log:
                assert fn() == 0
            self.kernels[lname] = log.kernels
        torch.cuda.synchronize()
        self._launch_fns = launches
        return launches

    def time_kernel(self, fn, reps):
        torch = self.torch
        for _ in range(5):
            assert fn() == 0
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(reps):
            fn()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) * 1e-3 / reps

    def time_kernel_cold(self, fn, reps, flush):
        torch = self.torch
        total = 0.0
        for _ in range(reps):
            flush.add_(1)
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            fn()
            stop.record()
            torch.cuda.synchronize()
            total += start.elapsed_time(stop) * 1e-3
        return total / reps

    def roofline_of(self, lname, t, t_cold, traffic):
        # the roof that binds a launch is the slower of "move its algorithmic bytes at 8 TB/s" and "do its flops at the
        # dense matrix peak of the arithmetic type"
        _, nbytes, nflops = self.launch_fns()[lname]
        t_hbm, t_mfma = nbytes / (HBM_PEAK_GBPS * 1e9), nflops / (self.mfma_peak * 1e12)
        kernels = self.kernels[lname]
        # counters read for other kernels than the ones selected now say nothing about this launch
        # (nor do counters read in the ordered modes about the "atomic" mode, whose kernels carry the same names)
        tr = None if self.fp8_act or self.mode == "atomic" else traffic.get((self.name, lname, tuple(sorted(set(kernels)))))
        common = {"launch": lname, "kernel": kernel_list(kernels), "avg_launch_us": round(t * 1e6, 3),
                  "avg_launch_us_cold": None if t_cold is None else round(t_cold * 1e6, 3),
                  "algorithmic_bytes": nbytes, "algorithmic_flops": nflops,
                  "hbm_frac": round(nbytes / t * 1e-9 / HBM_PEAK_GBPS, 4), "mfma_frac": round(nflops / t * 1e-12 / self.mfma_peak, 4),
                  "traffic": None if tr is None else tr["bytes"], "traffic_source": None if tr is None else tr["source"]}
        if t_hbm >= t_mfma:
            return {"bound": "hbm", "achieved": round(nbytes / t * 1e-9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": round(nbytes / t * 1e-9 / HBM_PEAK_GBPS, 4), **common}
        return {"bound": "mfma", "achieved": round(nflops / t * 1e-12, 2), "peak": self.mfma_peak, "unit": "TFLOP/s",
                "frac": round(nflops / t * 1e-12 / self.mfma_peak, 4), **common}


def side_config(name, mode, traffic, fp8_act=False):
    """Step and per-launch times of one of the other configurations, in brief (no CPU baseline, no cold launches)."""
    import torch
    w = Workload(name, mode, fp8_act)
    B, T, E, K, I, J = w.dims
    routes = time_routes(w.step, 10, 3, False, many=False)
    step_us, how = best_route(routes)
    launches = w.launch_fns()
    warm = {lname: w.time_kernel(fn, 10) for lname, (fn, _, _) in launches.items()}
    dom = max(warm, key=warm.get)
    roofs = {lname: w.roofline_of(lname, warm[lname], None, traffic) for lname in launches}
    res = {"workload": f"{w.cfg.name}: B{B} T{T} E{E} K{K} I{I} J{J} {w.cfg.what}", "scatter_mode": mode,
           "scatter_workspace_bytes": int(w.abi.lib().egs_workspace_bytes(w.abi.OP_GEMM_SCATTER, w.hk._MODES[mode], w.abi.Dims(*w.dims),
                                                                             w.hk.dtype_to_type_id(w.cfg.dtype))),
           "dtype": ("fp8 x fp8" if fp8_act else w.dtype_name + (" (fp8 e4m3 weights)" if w.fp8 else "")),
           "step_us": round(step_us, 1), "launch": how,
           "step_hbm_frac": round(w.chain_bytes / (step_us * 1e-6) * 1e-9 / HBM_PEAK_GBPS, 4),
           "step_mfma_frac": round(w.chain_flops / (step_us * 1e-6) * 1e-12 / w.mfma_peak, 4),
           "launch_us": {k: round(v * 1e6, 1) for k, v in warm.items()},
           "kernels": {k: kernel_list(v) for k, v in w.kernels.items()},
           "dominant": {k: roofs[dom][k] for k in ("launch", "kernel", "bound", "frac", "achieved", "unit", "hbm_frac", "mfma_frac", "traffic")},
           "frac_per_launch": {k: {"bound": r["bound"], "frac": r["frac"]} for k, r in roofs.items()}}
    del w
    torch.cuda.empty_cache()
    return res


def pmc_probe(args):
    import torch
    from expertscattergather_amd import _abi, hip_kernels as hk, workloads as wl
    dev = torch.device("cuda:0")
    cfg = wl.CONFIGS[args.config]
    B, T, E, K, I, J = cfg.dims
    inp = wl.make_inputs(cfg)
    X, Wg, Ws, dOut, Ind = (inp[k].to(dev) for k in ("X", "Wg", "Ws", "dOut", "Ind"))
    # FETCH_SIZE / WRITE_SIZE calibration: a copy kernel of known size next to the dominant kernel
    src = torch.empty(64 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    if args.config == "C5":     # the configuration's own weights: e4m3 bytes and fp32 scales
        Wq_p, scale_p = (t.to(dev) for t in wl.quantize_fp8_weights(inp["Wg"].float()))
    Yp = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32) if args.config != "C5" else None
    if args.probe_kernel == "dw":
        dWp = torch.empty_like(Wg)
        dp = _abi.Dims(B, T, E, K, I, J)
        dtp = hk.dtype_to_type_id(cfg.dtype)
        wsb = max(_abi.lib().egs_workspace_bytes(_abi.OP_DW, 0, dp, dtp), 256)
        wsp = torch.empty(wsb, dtype=torch.uint8, device=dev)
    for _ in range(5):
        if args.config == "C5":
            hk.expert_gather_fp8w_forward(X, Wq_p, scale_p, Ind)
        elif args.probe_kernel == "gather":
            hk.invalidate_routing_table(Ind)        # every dispatch builds the routing table, as the first of a step does
            hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)
        elif args.probe_kernel == "scatter":
            hk.expert_scatter_forward_call(Yp, Ws, Ind, T, torch.float32)
        elif args.probe_kernel == "scatter_bwd":
            hk.expert_scatter_backward_call(Yp, Ws, Ind, dOut, torch.float32)
        elif args.probe_kernel == "gather_bwd":
            hk.expert_gather_backward_call(X, Wg, Ind, Yp, torch.float32)
        elif args.probe_kernel == "mlp":
            hk.expert_mlp_forward(X, Wg, Ws, Ind, "relu", force_block=True)
        elif args.probe_kernel == "mlp_separate":
            hk.expert_scatter_forward_call(torch.relu(hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)), Ws, Ind, T,
                                           torch.float32)
        else:
            rc = _abi.lib().egs_dw(X.data_ptr(), Yp.data_ptr(), Ind.data_ptr(), dWp.data_ptr(), wsp.data_ptr(), wsb, dp,
                                   T * I, I, dtp, dtp, _abi.IND_I64, _abi.W_EIJ, torch.cuda.current_stream().cuda_stream)
            assert rc == 0
    torch.cuda.synchronize()
    print(json.dumps({"pmc_probe": True, "copy_bytes_read": 64 << 20, "copy_bytes_written": 64 << 20}))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no sharding, no collectives); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from expertscattergather_amd import hip_kernels as hk

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(torch.device("cuda:0"))
    hk.create_kernels()
    if args.mode:
        hk.set_scatter_mode(args.mode)
    mode = hk.get_scatter_mode()
    if args.pmc_probe:
        pmc_probe(args)
        return
    if args.fp8_act and args.config != "C5":
        print("bench.py: --fp8-act applies to the fp8-weight configuration C5 only", file=sys.stderr)
        sys.exit(2)

    w = Workload(args.config, mode, args.fp8_act)
    cfg = w.cfg
    B, T, E, K, I, J = w.dims
    headline = args.config == "C2"

    # ------------------------------------------------------------------ whole-step timing
    # through the four launcher callables ...
    launcher = time_routes(w.step, args.steps, args.warmup, args.no_graph, many=headline)
    # ... and through the modules and PyTorch's autograd: the same four launches (forward + backward configurations)
    autograd = None
    if not w.fwd_only and not w.fp8:
        autograd = time_routes(w.autograd_step_fn(), args.steps, min(args.warmup, 10), args.no_graph, many=headline)
    if autograd is not None:
        step_us, how = best_route(autograd)
        how = "modules + autograd, " + how
    else:
        step_us, how = best_route(launcher)
        how = "launcher callables, " + how
    step_s = step_us * 1e-6

    # ------------------------------------------------------------------ per-launch timing (HIP events)
    # Every launch of the step through the C ABI, back to back on torch's current stream (the stream the launches are
    # enqueued on), bracketed by HIP events; and once more with the caches flushed before every launch.
    launches = w.launch_fns()
    reps = args.kernel_reps if args.config in ("C1", "C2") else max(5, args.kernel_reps // 10)
    warm = {name: w.time_kernel(fn, reps) for name, (fn, _, _) in launches.items()}
    # a buffer larger than the 256 MB Infinity Cache, rewritten between launches for the cold numbers
    flush = None if args.no_cold else torch.empty(640 << 20, dtype=torch.uint8, device=w.dev)
    cold = None if flush is None else {name: w.time_kernel_cold(fn, 10, flush) for name, (fn, _, _) in launches.items()}
    dw_alone_s = None if w.fwd_only else w.time_kernel(w.k_dw, reps)
    del flush
    traffic = recorded_traffic()
    # the dominant launch is the one that takes most of a step (every launch runs once per step)
    dom = max(warm, key=warm.get)
    rooflines = {name: w.roofline_of(name, warm[name], None if cold is None else cold[name], traffic) for name in launches}

    # ------------------------------------------------------------------ CPU baseline (bounded sample)
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import torch_port as P
        inp = w.inp
        cores = torch.get_num_threads()
        # bounded sample: the first nb batch elements (batch elements are independent), scaled to the full batch
        nb = {"C1": B, "C2": B, "C3": 1, "C4": 4, "C5": 1}.get(args.config, B)
        Xc, dOc = (inp[k][:nb].float() for k in ("X", "dOut"))
        Wgc, Wsc = (inp[k].float() for k in ("Wg", "Ws"))
        if w.fp8:
            Wgc = w.Wq_c.float() * w.scale_c[:, None, :]        # dequantise-then-einsum, as the configuration's reference does
        Ic = inp["Ind"][:nb]

        def cpu_step():
            if w.fwd_only:
                with torch.no_grad():
                    return P.scatter(P.gather(Xc, Wgc, Ic), Wsc, Ic, T)
            return P.chain_fwd_bwd(Xc, Wgc, Wsc, Ic, dOc)

        cpu_step()
        times = []
        t_begin = time.perf_counter()
        while len(times) < 5 and (time.perf_counter() - t_begin < 20.0 or len(times) < 2):
            t0 = time.perf_counter()
            cpu_step()
            times.append(time.perf_counter() - t0)
        times.sort()
        scale_to_full = B / nb
        cpu = {"value": round(times[len(times) // 2] * 1e6 * scale_to_full, 1), "unit": "us", "cores": cores, "kind": "port",
               "sample": f"median of {len(times)} {cfg.name} steps of oracle/torch_port.py over {nb} of {B} batch elements"
                         f"{'' if nb == B else f' (time scaled by {scale_to_full:g})'} (torch CPU, fp32 arithmetic "
                         f"on the {str(cfg.dtype).split('.')[-1]}-rounded inputs)"}

    # ------------------------------------------------------------------ the other configurations, in brief
    configs = None
    if headline and not args.no_configs:
        configs = {}
        for name, m in (("C1", "deterministic"), ("C3", "deterministic"), ("C4", "deterministic"), ("C4", "atomic"), ("C4", "compact"),
                        ("C5", "deterministic")):
            t0 = time.perf_counter()
            try:
                configs[name if name != "C4" else f"C4-{m}"] = dict(side_config(name, m, traffic), bench_s=round(time.perf_counter() - t0, 1))
            except Exception as exc:
                configs[name if name != "C4" else f"C4-{m}"] = {"error": f"{type(exc).__name__}: {exc}"}
                print(f"bench.py: configuration {name} ({m}) failed: {exc}", file=sys.stderr)

    r3 = lambda v: None if v is None else round(v, 2)
    sum_launch = sum(warm.values()) * 1e6
    result = {
        "metric": "fused gather+scatter fwd+bwd time per call at B64 T256 E32 K32 I128 J64" if args.config in ("C1", "C2")
                  else f"fused gather+scatter time per call at {cfg.name}",
        "value": round(step_us, 2),
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("fp8 (e4m3 weights, activations quantised per row to e4m3, fp32 accumulation)" if w.fp8_act
                  else w.dtype_name + (" (fp8 e4m3 weights)" if w.fp8 else "")),
        "data": "synthetic",
        "config": {"workload": f"{cfg.name}: B{B} T{T} E{E} K{K} I{I} J{J} {cfg.what}", "scatter_mode": mode, "launch": how},
        "step_hbm_gbps": round(w.chain_bytes / step_s * 1e-9, 1),
        "step_hbm_frac": round(w.chain_bytes / step_s * 1e-9 / HBM_PEAK_GBPS, 4),
        "step_tflops": round(w.chain_flops / step_s * 1e-12, 2),
        "autograd_us_per_step": None if autograd is None else {k: (v if k == "steps_per_graph" else r3(v)) for k, v in autograd.items()},
        "launcher_us_per_step": {k: (v if k == "steps_per_graph" else r3(v)) for k, v in launcher.items()},
        "sum_launch_us": round(sum_launch, 2),
        "value_minus_sum_launch_us": round(step_us - sum_launch, 2),
        "routing_table_bytes": int(w.tab_bytes),
        "launch_us": {k: round(v * 1e6, 2) for k, v in warm.items()},
        "launch_us_cold": None if cold is None else {k: round(v * 1e6, 2) for k, v in cold.items()},
        "dw_alone_us": None if dw_alone_s is None else round(dw_alone_s * 1e6, 2),
        "roofline": rooflines[dom],
        "roofline_per_launch": rooflines,
        "cpu_baseline": cpu,
        "configs": configs,
    }
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
