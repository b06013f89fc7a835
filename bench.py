#!/usr/bin/env python3
"""Benchmark of the fused expert gather/scatter path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input at the default shape in
bf16 (B64 T256 E32 K32 I128 J64): gather forward -> scatter forward -> scatter backward (dY,
dW_scatter) -> gather backward (dX, dW_gather), i.e. the six kernel-equivalents of a full
autograd forward+backward.  Inputs are resident in HBM before the timed region starts.

Prints ONE JSON line.  `value` is microseconds per step (lower is better); `roofline`
describes the dominant launch of the step, the one that takes the most time (algorithmic bytes
or flops / its average duration, measured with HIP events on the launch stream, warm and with
the caches flushed), `roofline_per_launch` every launch; `cpu_baseline` is the torch port of
the reference's baselines timed on the host cores.
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

# kernel (as rocprofv3 names it) behind each launch of the path, per workload; where a call runs several kernels
# the one that takes most of its time is named and the others are listed in the profile summaries
LAUNCH_KERNELS = {
    "C2": {"expert_gather_forward": "rows_small_kernel", "expert_scatter_forward": "scatter_fused_table_kernel",
           "expert_scatter_backward": "rows_dw_tile_kernel", "expert_gather_backward": "scatter_fused_dwtile_table_kernel"},
    "C1": {"expert_gather_forward": "rows_small_f32_kernel", "expert_scatter_forward": "scatter_fused_table_kernel"},
    "C3": {"expert_gather_forward": "rows_gemm_dl_kernel", "expert_scatter_forward": "rows_gemm_dl_kernel + segment_sum_kernel",
           "expert_scatter_backward": "rows_gemm_dl_kernel + dw_dl_kernel", "expert_gather_backward": "rows_gemm_dl_kernel + segment_sum_kernel + dw_dl_kernel"},
    "C4": {"expert_gather_forward": "rows_gemm_dl_kernel", "expert_scatter_forward": "rows_gemm_dl_kernel + segment_sum_kernel",
           "expert_scatter_backward": "rows_gemm_dl_kernel + dw_dl_kernel", "expert_gather_backward": "rows_gemm_dl_kernel + segment_sum_kernel + dw_dl_kernel"},
    "C5": {"expert_gather_forward": "rows_gemm_dl_kernel", "expert_scatter_forward": "rows_gemm_dl_kernel + segment_sum_kernel"},
}


def recorded_traffic():
    """HBM-side bytes per launch from the rocprofv3 --pmc summaries under profiles/ (FETCH_SIZE + WRITE_SIZE of
    `bench.py --pmc-probe` runs, each scaled by what the same counter reads for a 64 MiB copy).  Counters cannot be read
    from inside this process, so the figures are the recorded ones: lines `traffic <workload> <launch> <bytes>`."""
    import glob
    import re
    found = {}
    for path in sorted(glob.glob(os.path.join(PROFILES, "*.md")) + glob.glob(os.path.join(PROFILES, "*.txt"))):
        for m in re.finditer(r"^\s*traffic (\S+) (\S+) (\d+)\s*$", open(path).read(), flags=re.M):
            found[(m.group(1), m.group(2))] = {"bytes": int(m.group(3)), "source": os.path.relpath(path, ROOT)}
    return found


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="C2", help="workload (C2 = the metric's configuration)")
    ap.add_argument("--mode", default=None, choices=["deterministic", "atomic"], help="scatter mode (default: env / deterministic)")
    ap.add_argument("--fp8-act", action="store_true",
                    help="C5 only: quantise the activations per row to e4m3 and multiply on the fp8 matrix instruction")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of a HIP graph replay")
    ap.add_argument("--no-cpu-baseline", action="store_true")
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


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no sharding, no collectives); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from expertscattergather_amd import _abi, hip_kernels as hk, workloads as wl

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    hk.create_kernels()
    if args.mode:
        hk.set_scatter_mode(args.mode)
    cfg = wl.CONFIGS[args.config]
    B, T, E, K, I, J = cfg.dims
    inp = wl.make_inputs(cfg)
    X, Wg, Ws, dOut, Ind = (inp[k].to(dev) for k in ("X", "Wg", "Ws", "dOut", "Ind"))
    fwd_only = args.config in ("C1", "C5")

    if args.pmc_probe:
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
        return

    fp8 = args.config == "C5"
    if args.fp8_act and not fp8:
        print("bench.py: --fp8-act applies to the fp8-weight configuration C5 only", file=sys.stderr)
        sys.exit(2)
    fp8_act = fp8 and args.fp8_act
    if fp8:     # the configuration's weights: e4m3 bytes and a per-expert, per-column fp32 scale
        Wq_c, scale_c = wl.quantize_fp8_weights(inp["Wg"].float())
        Wq, Wscale = Wq_c.to(dev), scale_c.to(dev)

    def step():
        # a training step routes anew: the table that the gather forward leaves with Ind for the scatter forward and the
        # gather's backward is rebuilt in every step, never carried over from the step before
        hk.invalidate_routing_table(Ind)
        if fp8_act:
            Y = hk.expert_gather_fp8_forward(X, Wq, Wscale, Ind)
        elif fp8:
            Y = hk.expert_gather_fp8w_forward(X, Wq, Wscale, Ind)
        else:
            Y = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)
        out = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
        if fwd_only:
            return Y, out
        dY, dWs = hk.expert_scatter_backward_call(Y, Ws, Ind, dOut, torch.float32)
        dX, dWg = hk.expert_gather_backward_call(X, Wg, Ind, dY, torch.float32)
        return Y, out, dX, dWg, dWs

    # ------------------------------------------------------------------ whole-step timing
    for _ in range(max(args.warmup, 3)):
        step()
    torch.cuda.synchronize()

    def time_loop(fn, n):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n

    eager_s = time_loop(step, args.steps)
    graph_s = None
    if not args.no_graph:
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    step()          # workspace for the capture stream exists before capture
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                keep = step()
            for _ in range(max(args.warmup, 3)):
                graph.replay()
            graph_s = time_loop(graph.replay, args.steps)
            del keep
        except Exception as exc:        # report, fall back to the eager number
            print(f"bench.py: graph capture failed ({exc}); reporting eager timing", file=sys.stderr)
            graph_s = None
    # the step time reported is the faster of the two ways of issuing the same launches
    use_graph = graph_s is not None and graph_s <= eager_s
    step_s = graph_s if use_graph else eager_s

    # ------------------------------------------------------------------ the same step through the modules and autograd
    # ExpertScatter(ExpertGather(x, Ind), Ind, T).backward(dOut): the same four launches, issued by PyTorch's autograd
    # engine (reported beside the step, not as the step: at these sizes it times the engine, not the kernels)
    autograd_us = None
    if not fwd_only and not fp8:
        import expertscattergather_amd as egs
        gmod = egs.ExpertGather(E, I, J).to(dev, cfg.dtype)
        smod = egs.ExpertScatter(E, J, I).to(dev, cfg.dtype)
        with torch.no_grad():
            gmod.W.copy_(Wg); smod.W.copy_(Ws)
        xg = X.clone().requires_grad_(True)

        def autograd_step():
            xg.grad = None; gmod.W.grad = None; smod.W.grad = None
            smod(gmod(xg, Ind), Ind, T).backward(dOut)

        for _ in range(5):
            autograd_step()
        n_auto = max(10, min(args.steps, 100))
        autograd_us = {"eager": round(time_loop(autograd_step, n_auto) * 1e6, 2), "graph": None}
        if not args.no_graph:
            try:
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    for _ in range(3):
                        autograd_step()
                torch.cuda.current_stream().wait_stream(side)
                torch.cuda.synchronize()
                agraph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(agraph, stream=side):
                    autograd_step()
                for _ in range(5):
                    agraph.replay()
                autograd_us["graph"] = round(time_loop(agraph.replay, n_auto) * 1e6, 2)
            except Exception as exc:
                print(f"bench.py: graph capture of the autograd step failed ({exc})", file=sys.stderr)

    # ------------------------------------------------------------------ per-launch timing (HIP events)
    # Every launch of the step through the C ABI, back to back on torch's current stream (the stream the launches are
    # enqueued on), bracketed by HIP events; and once more with the caches flushed before every launch.
    act = 2 if cfg.dtype != torch.float32 else 4
    lib = _abi.lib()
    d = _abi.Dims(B, T, E, K, I, J)
    dt = hk.dtype_to_type_id(cfg.dtype)
    stream = torch.cuda.current_stream().cuda_stream
    Y = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32) if not fp8 else hk.expert_gather_fp8w_forward(X, Wq, Wscale, Ind)
    out = torch.empty(B, T, I, device=dev, dtype=cfg.dtype)
    dYb, dXb = torch.empty_like(Y), torch.empty(B, T, I, device=dev, dtype=cfg.dtype)
    dWg_b, dWs_b = torch.empty(E, I, J, device=dev, dtype=cfg.dtype), torch.empty(E, J, I, device=dev, dtype=cfg.dtype)
    mode = 0 if hk.get_scatter_mode() == "deterministic" else 1
    ws_bytes = max(lib.egs_workspace_bytes(_abi.OP_GATHER_BACKWARD, mode, d, dt), lib.egs_workspace_bytes(_abi.OP_DW, mode, d, dt), 256)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    f8ws_bytes = lib.egs_gather_gemm_fp8act_workspace_bytes(d) if fp8_act else 0
    f8ws = torch.empty(max(f8ws_bytes, 256), dtype=torch.uint8, device=dev)
    I64 = _abi.IND_I64
    # the launches as a step issues them: where the sizes have a routing table, the gather forward builds it and the
    # scatter forward and the gather's backward read it
    tab_bytes = 0 if fp8 else lib.egs_routing_table_bytes(d, dt)
    tab = torch.empty(max(tab_bytes, 256), dtype=torch.uint8, device=dev)

    def k_gather():
        if fp8_act:     # row quantiser + fp8 x fp8 product: both launches are part of the call
            return lib.egs_gather_gemm_fp8act(X.data_ptr(), Wq.data_ptr(), Wscale.data_ptr(), Ind.data_ptr(), Y.data_ptr(),
                                              f8ws.data_ptr(), f8ws_bytes, d, T * I, I, I64, stream)
        if fp8:
            return lib.egs_gather_gemm(X.data_ptr(), Wq.data_ptr(), Ind.data_ptr(), Y.data_ptr(), Wscale.data_ptr(), d, T * I, I, dt,
                                       _abi.FP8_E4M3, I64, _abi.W_EIJ, stream)
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

    # a buffer larger than the 256 MB Infinity Cache, rewritten between launches for the cold numbers
    flush = None if args.no_cold else torch.empty(640 << 20, dtype=torch.uint8, device=dev)

    def time_kernel(fn, reps):
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

    def time_kernel_cold(fn, reps):
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

    dims = cfg.dims
    gemm_bytes = wl.algorithmic_bytes(dims, act)
    gather_bytes = wl.algorithmic_bytes(dims, act, w_bytes=1, fp8_scales=True) if fp8 else gemm_bytes
    dw_bytes = wl.algorithmic_bytes(dims, act, dw=True)
    kflops = wl.flops(dims)
    reps = args.kernel_reps if args.config in ("C1", "C2") else max(5, args.kernel_reps // 10)
    # launch -> (function, algorithmic bytes, flops): the backward calls compute two kernel-equivalents each
    launches = {"expert_gather_forward": (k_gather, gather_bytes, kflops), "expert_scatter_forward": (k_scatter, gemm_bytes, kflops)}
    if not fwd_only:
        launches["expert_scatter_backward"] = (k_scatter_bwd, gemm_bytes + dw_bytes, 2 * kflops)
        launches["expert_gather_backward"] = (k_gather_bwd, gemm_bytes + dw_bytes, 2 * kflops)
    assert k_gather() == 0      # the table is in place before the launches that read it are timed
    warm = {name: time_kernel(fn, reps) for name, (fn, _, _) in launches.items()}
    cold = None if flush is None else {name: time_kernel_cold(fn, 10) for name, (fn, _, _) in launches.items()}
    dw_alone_s = None if fwd_only else time_kernel(k_dw, reps)
    del flush
    n_equiv = 2 if fwd_only else 6
    chain_bytes = (gather_bytes + gemm_bytes) if fwd_only else 4 * gemm_bytes + 2 * dw_bytes
    chain_flops = n_equiv * kflops
    dtype_name = "bf16" if cfg.dtype == torch.bfloat16 else ("f16" if cfg.dtype == torch.float16 else "f32")
    mfma_peak = MFMA_PEAK_TFLOPS["fp8" if fp8_act else dtype_name]
    traffic = recorded_traffic()

    def roofline_of(name):
        # the roof that binds a launch is the slower of "move its algorithmic bytes at 8 TB/s" and "do its flops at the
        # dense matrix peak of the arithmetic type"
        _, nbytes, nflops = launches[name]
        t = warm[name]
        t_hbm, t_mfma = nbytes / (HBM_PEAK_GBPS * 1e9), nflops / (mfma_peak * 1e12)
        tr = traffic.get((args.config, name))
        common = {"launch": name, "kernel": LAUNCH_KERNELS.get(args.config, {}).get(name), "avg_launch_us": round(t * 1e6, 3),
                  "avg_launch_us_cold": None if cold is None else round(cold[name] * 1e6, 3),
                  "algorithmic_bytes": nbytes, "algorithmic_flops": nflops,
                  "hbm_frac": round(nbytes / t * 1e-9 / HBM_PEAK_GBPS, 4), "mfma_frac": round(nflops / t * 1e-12 / mfma_peak, 4),
                  "traffic": None if tr is None or fp8_act else tr["bytes"], "traffic_source": None if tr is None or fp8_act else tr["source"]}
        if t_hbm >= t_mfma:
            return {"bound": "hbm", "achieved": round(nbytes / t * 1e-9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": round(nbytes / t * 1e-9 / HBM_PEAK_GBPS, 4), **common}
        return {"bound": "mfma", "achieved": round(nflops / t * 1e-12, 2), "peak": mfma_peak, "unit": "TFLOP/s",
                "frac": round(nflops / t * 1e-12 / mfma_peak, 4), **common}

    # the dominant launch is the one that takes most of a step (every launch runs once per step)
    dom = max(warm, key=warm.get)
    rooflines = {name: roofline_of(name) for name in launches}

    # ------------------------------------------------------------------ CPU baseline (bounded sample)
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import torch_port as P
        cores = torch.get_num_threads()
        # bounded sample: the first nb batch elements (batch elements are independent), scaled to the full batch
        nb = {"C1": B, "C2": B, "C3": 1, "C4": 4, "C5": 1}.get(args.config, B)
        Xc, dOc = (inp[k][:nb].float() for k in ("X", "dOut"))
        Wgc, Wsc = (inp[k].float() for k in ("Wg", "Ws"))
        if fp8:
            Wgc = Wq_c.float() * scale_c[:, None, :]        # dequantise-then-einsum, as the configuration's reference does
        Ic = inp["Ind"][:nb]

        def cpu_step():
            if fwd_only:
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

    result = {
        "metric": "fused gather+scatter fwd+bwd time per call at B64 T256 E32 K32 I128 J64" if args.config in ("C1", "C2")
                  else f"fused gather+scatter time per call at {cfg.name}",
        "value": round(step_s * 1e6, 2),
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("fp8 (e4m3 weights, activations quantised per row to e4m3, fp32 accumulation)" if fp8_act
                  else dtype_name + (" (fp8 e4m3 weights)" if fp8 else "")),
        "data": "synthetic",
        "config": {"workload": f"{cfg.name}: B{B} T{T} E{E} K{K} I{I} J{J} {cfg.what}", "scatter_mode": hk.get_scatter_mode(),
                   "launch": "hip graph replay" if use_graph else "eager launches through the Python ops"},
        "step_hbm_gbps": round(chain_bytes / step_s * 1e-9, 1),
        "step_hbm_frac": round(chain_bytes / step_s * 1e-9 / HBM_PEAK_GBPS, 4),
        "step_tflops": round(chain_flops / step_s * 1e-12, 2),
        "eager_us_per_step": round(eager_s * 1e6, 2),
        "graph_us_per_step": None if graph_s is None else round(graph_s * 1e6, 2),
        "autograd_us_per_step": autograd_us,
        "routing_table_bytes": int(tab_bytes),
        "launch_us": {k: round(v * 1e6, 2) for k, v in warm.items()},
        "launch_us_cold": None if cold is None else {k: round(v * 1e6, 2) for k, v in cold.items()},
        "dw_alone_us": None if dw_alone_s is None else round(dw_alone_s * 1e6, 2),
        "roofline": rooflines[dom],
        "roofline_per_launch": rooflines,
        "cpu_baseline": cpu,
    }
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
