"""Host-side behaviour that needs no GPU: module construction and parameters, op registration
with fake implementations, error paths, scatter-mode switch, synthetic workloads."""
import math

import pytest
import torch

import expertscattergather_amd as egs
from expertscattergather_amd import hip_kernels as hk, workloads as wl


def test_modules_construct_on_cpu_with_reference_parameter_shapes():
    g = egs.ExpertGather(5, 12, 7)
    s = egs.ExpertScatter(5, 7, 12, bias=True)
    assert g.W.shape == (5, 12, 7) and g.bias is None           # reference egs/torch_interface.py:15-19
    assert s.W.shape == (5, 7, 12) and s.bias.shape == (5, 1, 12)
    assert g.W.abs().max() <= 1 / math.sqrt(12) and s.W.abs().max() <= 1 / math.sqrt(12)
    assert set(g.state_dict()) == {"W"} and set(s.state_dict()) == {"W", "bias"}
    g2 = egs.ExpertGather(5, 12, 7); g2.load_state_dict(g.state_dict())
    assert torch.equal(g2.W, g.W)
    before = g.W
    assert g.to(torch.bfloat16) is g and g.W.dtype == torch.bfloat16 and g.W is before   # optimizer references survive


def test_no_cpu_fallback():
    g = egs.ExpertGather(2, 8, 4)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        g(torch.randn(1, 3, 8), torch.zeros(1, 2, 2, dtype=torch.int64))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        egs.ExpertScatter(2, 4, 8)(torch.randn(1, 2, 2, 4), torch.zeros(1, 2, 2, dtype=torch.int64), 3)


def test_ops_are_registered_with_fake_implementations():
    hk.create_kernels(); hk.create_kernels()                     # idempotent
    ops = torch.ops.egs_amd
    X = torch.empty(2, 5, 8, device="meta"); Wg = torch.empty(4, 8, 6, device="meta")
    Ws = torch.empty(4, 6, 8, device="meta"); Ind = torch.empty(2, 4, 3, dtype=torch.int64, device="meta")
    Y = ops.expert_gather_forward_call_fn(X, Wg, Ind, torch.float32)
    assert Y.shape == (2, 4, 3, 6) and Y.dtype == X.dtype
    dX, dW = ops.expert_gather_backward_call_fn(X, Wg, Ind, Y, torch.float32)
    assert dX.shape == X.shape and dW.shape == Wg.shape and dX is not X and dW is not Wg
    out = ops.expert_scatter_forward_call_fn(Y, Ws, Ind, 5, torch.float32)
    assert out.shape == (2, 5, 8)
    dY, dWs = ops.expert_scatter_backward_call_fn(Y, Ws, Ind, out, torch.float32)
    assert dY.shape == Y.shape and dWs.shape == Ws.shape
    # the module-level callables send meta tensors through the ops (and so through the fake implementations)
    assert hk.expert_gather_forward_call(X, Wg, Ind, torch.float32).shape == (2, 4, 3, 6)
    assert hk.expert_scatter_forward_call(Y, Ws, Ind, 5, torch.float32).shape == (2, 5, 8)


def test_autograd_functions_trace_on_meta_tensors():
    X = torch.empty(2, 5, 8, device="meta", requires_grad=True)
    W = torch.empty(4, 8, 6, device="meta", requires_grad=True)
    Ind = torch.empty(2, 4, 3, dtype=torch.int64, device="meta")
    Y = hk.ExpertGatherFunction.apply(X, W, Ind)
    Y.sum().backward()
    assert X.grad.shape == X.shape and W.grad.shape == W.shape
    Ws = torch.empty(4, 6, 8, device="meta", requires_grad=True)
    out = hk.ExpertScatterFunction.apply(Y.detach().requires_grad_(True), Ws, Ind, 5)
    out.sum().backward()
    assert Ws.grad.shape == Ws.shape


def test_dtype_ids_and_errors():
    assert [hk.dtype_to_type_id(d) for d in (torch.float32, torch.float16, torch.bfloat16)] == [0, 1, 2]
    with pytest.raises(ValueError, match="Unknown dtype"):
        hk.dtype_to_type_id(torch.float64)


def test_scatter_mode_switch():
    assert hk.get_scatter_mode() in ("deterministic", "atomic")
    keep = hk.get_scatter_mode()
    hk.set_scatter_mode("ATOMIC"); assert hk.get_scatter_mode() == "atomic"
    with pytest.raises(ValueError):
        hk.set_scatter_mode("fastest")
    hk.set_scatter_mode(keep)


def test_scatter_mode_scope_and_module_attribute():
    """The mode in force is: innermost scope of the thread, else the process-wide setting; a module's
    `scatter_mode` attribute is such a scope around its call, and other threads do not see it."""
    import threading
    import expertscattergather_amd as egs
    keep = hk.get_scatter_mode()
    try:
        hk.set_scatter_mode("deterministic")
        with hk.scatter_mode_scope("atomic"):
            assert hk.get_scatter_mode() == "atomic"
            with hk.scatter_mode_scope(None):
                assert hk.get_scatter_mode() == "atomic"
            with hk.scatter_mode_scope("Deterministic"):
                assert hk.get_scatter_mode() == "deterministic"
            assert hk.get_scatter_mode() == "atomic"
            seen = []
            th = threading.Thread(target=lambda: seen.append(hk.get_scatter_mode()))
            th.start(); th.join()
            assert seen == ["deterministic"]
        assert hk.get_scatter_mode() == "deterministic"
        with pytest.raises(ValueError):
            hk.scatter_mode_scope("fastest")
        g, s = egs.ExpertGather(2, 8, 4), egs.ExpertScatter(2, 4, 8)
        assert g.scatter_mode is None and s.scatter_mode is None
        # the modules hand the mode in force to their Functions: record it instead of launching
        seen = []
        orig_g, orig_s = hk.expert_gather_forward_call, hk.expert_scatter_forward_call
        hk.expert_gather_forward_call = lambda X, W, Ind, dt: (seen.append(hk.get_scatter_mode()), torch.zeros(1, 2, 3, 4))[1]
        hk.expert_scatter_forward_call = lambda Y, W, Ind, T, dt: (seen.append(hk.get_scatter_mode()), torch.zeros(1, T, 8))[1]
        try:
            Ind = torch.zeros(1, 2, 3, dtype=torch.int64)
            g.scatter_mode = "atomic"
            g(torch.zeros(1, 5, 8), Ind)
            s(torch.zeros(1, 2, 3, 4), Ind, 5)
            s.scatter_mode = "atomic"
            s(torch.zeros(1, 2, 3, 4), Ind, 5)
        finally:
            hk.expert_gather_forward_call, hk.expert_scatter_forward_call = orig_g, orig_s
        assert seen == ["atomic", "deterministic", "atomic"] and hk.get_scatter_mode() == "deterministic"
    finally:
        hk.set_scatter_mode(keep)


def test_workloads_follow_the_benchmark_configurations():
    assert wl.CONFIGS["C2"].dims == (64, 256, 32, 32, 128, 64)
    assert wl.algorithmic_bytes(wl.CONFIGS["C2"].dims, 2) == 13631488
    assert wl.algorithmic_bytes(wl.CONFIGS["C1"].dims, 4) == 26738688
    assert wl.algorithmic_bytes(wl.CONFIGS["C3"].dims, 2) == 270532608
    assert wl.algorithmic_bytes(wl.CONFIGS["C4"].dims, 2) == 59768832
    assert wl.algorithmic_bytes(wl.CONFIGS["C5"].dims, 2, 1, fp8_scales=True) == 1078460416
    assert wl.flops(wl.CONFIGS["C2"].dims) == 2 * 64 * 32 * 32 * 128 * 64
    inp = wl.make_inputs(wl.CONFIGS["C2"], dims=(3, 40, 4, 8, 16, 8))
    Ind = inp["Ind"]
    assert Ind.shape == (3, 4, 8) and Ind.min() >= 0 and Ind.max() < 40
    for b in range(3):
        for e in range(4):
            assert Ind[b, e].unique().numel() == 8             # without replacement per (b, e)
    again = wl.make_inputs(wl.CONFIGS["C2"], dims=(3, 40, 4, 8, 16, 8))
    assert all(torch.equal(inp[k], again[k]) for k in inp)       # seeded
    z = wl.make_inputs(wl.CONFIGS["C4"], dims=(2, 64, 4, 32, 16, 8))["Ind"]
    assert z.min() >= 0 and z.max() < 64
    assert max(z[b, e].unique().numel() for b in range(2) for e in range(4)) < 32   # Zipf repeats tokens
    Wq, scale = wl.quantize_fp8_weights(torch.randn(3, 16, 8))
    assert Wq.dtype == torch.float8_e4m3fn and scale.shape == (3, 8)
    assert (Wq.float().abs().amax(dim=1) <= 448).all()


def test_expert_choice_router_picks_top_k_tokens_per_expert():
    import torch
    from expertscattergather_amd.router import expert_choice_router
    gen = torch.Generator().manual_seed(3)
    B, T, E, K = 3, 17, 5, 4
    logits = torch.randn(B, T, E, generator=gen)
    Ind, scores = expert_choice_router(logits, K, torch.int16)
    assert Ind.shape == (B, E, K) and Ind.dtype == torch.int16 and scores.shape == (B, E, K)
    aff = torch.softmax(logits, -1)
    for b in range(B):
        for e in range(E):
            order = sorted(range(T), key=lambda t: -float(aff[b, t, e]))[:K]
            assert Ind[b, e].tolist() == order
            assert len(set(Ind[b, e].tolist())) == K
            assert torch.allclose(scores[b, e], aff[b, Ind[b, e].long(), e])
    import pytest
    with pytest.raises(ValueError):
        expert_choice_router(torch.randn(1, 300, 2), 2, torch.uint8)      # ids up to 299 do not fit
    with pytest.raises(ValueError):
        expert_choice_router(logits, T + 1)


def test_bench_refuses_more_than_one_gpu():
    """`bench.py --gpus N` with N above 1 exits with a message instead of measuring anything."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)
    assert res.returncode != 0
    assert "one GPU" in res.stderr and res.stdout.strip() == ""


def test_bench_names_repeated_kernel_groups_and_reads_recorded_traffic_by_kernels():
    """bench.py reports, per launch, the kernels the library's launch log named; a call that works through batch groups
    repeats a group of kernels, which the name collapses.  The HBM-side traffic of a launch is a recorded figure
    (rocprofv3 cannot run inside the benchmark): a line per (workload, launch, set of kernels) under profiles/, used only
    when the kernels are the ones selected now."""
    import importlib.util
    import os
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("egs_bench", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    assert bench.kernel_list(["a"]) == "a" and bench.kernel_list([]) == ""
    assert bench.kernel_list(["a", "b", "a", "b"]) == "2 x (a + b)"
    assert bench.kernel_list(["a", "b"] * 8 + ["c"]) == "8 x (a + b) + c"
    assert bench.kernel_list(["t", "a", "b", "a", "b", "c", "c"]) == "t + 2 x (a + b) + 2 x (c)"
    found = bench.recorded_traffic()
    assert ("C2", "expert_gather_backward", ("scatter_fused_dwtile_table_kernel",)) in found
    # one launch, two sets of kernels (deterministic and compact mode), two figures
    c4 = {k[2]: v["bytes"] for k, v in found.items() if k[:2] == ("C4", "expert_scatter_forward")}
    assert c4[("scatter_pass_kernel",)] < c4[("rows_gemm_dl_kernel", "segment_sum_kernel")] // 4
    # every recorded line names its kernels, and its source file is where the line is
    for path in sorted(os.listdir(os.path.join(root, "profiles"))):
        text = open(os.path.join(root, "profiles", path)).read()
        for line in re.findall(r"^\s*traffic .*$", text, flags=re.M):
            assert re.match(r"^\s*traffic C[1-5] expert_\w+ \d+ [\w+]+\s*$", line), (path, line)
    for key, rec in found.items():
        assert os.path.exists(os.path.join(root, rec["source"])), key


def test_compute_dtype_follows_the_reference_kernels():
    # out_type float16 / bfloat16: both operands are cast to it (reference egs/triton_kernels.py:122-127);
    # float32: operands stay as they are - a shared 16-bit type is multiplied in that type, mixed types meet in float32
    f32, f16, bf16 = torch.float32, torch.float16, torch.bfloat16
    t = lambda dt: torch.empty(1, dtype=dt)
    assert hk._compute_dtype(bf16, t(f32), t(f32)) == bf16
    assert hk._compute_dtype(bf16, t(bf16), t(f32)) == bf16
    assert hk._compute_dtype(f16, t(bf16), t(f32)) == f16
    assert hk._compute_dtype(f32, t(bf16), t(bf16)) == bf16
    assert hk._compute_dtype(f32, t(bf16), t(f32)) == f32
    assert hk._compute_dtype(f32, t(f16), t(bf16), t(f32)) == f32
    assert hk._compute_dtype(f32, t(f32), t(f32)) == f32
    with pytest.raises(ValueError, match="Unknown dtype"):
        hk._compute_dtype(torch.int32, t(f32), t(f32))
    with pytest.raises(ValueError, match="Unknown dtype"):
        hk._compute_dtype(f32, t(torch.float64), t(f32))


def test_mixed_precision_shapes_and_dtypes_on_meta_tensors():
    # bf16 activations with an fp32 parameter, as under autocast-style use of the reference: results in the activation's
    # dtype, weight gradient in the parameter's dtype (reference egs/triton_kernels.py:375, :408-409)
    X = torch.empty(2, 5, 8, device="meta", dtype=torch.bfloat16, requires_grad=True)
    W = torch.empty(4, 8, 6, device="meta", dtype=torch.float32, requires_grad=True)
    Ind = torch.empty(2, 4, 3, dtype=torch.int16, device="meta")
    Y = hk.ExpertGatherFunction.apply(X, W, Ind, torch.bfloat16)
    assert Y.dtype == torch.bfloat16
    Y.sum().backward()
    assert X.grad.dtype == torch.bfloat16 and W.grad.dtype == torch.float32


def test_ops_are_differentiable_when_called_directly():
    hk.create_kernels()
    X = torch.empty(2, 5, 8, device="meta", requires_grad=True)
    W = torch.empty(4, 8, 6, device="meta", requires_grad=True)
    Ind = torch.empty(2, 4, 3, dtype=torch.int64, device="meta")
    Y = torch.ops.egs_amd.expert_gather_forward_call_fn(X, W, Ind, torch.float32)
    assert Y.requires_grad
    Y.sum().backward()
    assert X.grad.shape == X.shape and W.grad.shape == W.shape


def test_reference_namespace_alias():
    # the reference registers its ops as mylib::* (egs/triton_kernels.py:362); the alias is opt-in
    hk.register_reference_namespace("mylib_alias_for_test")
    hk.register_reference_namespace("mylib_alias_for_test")          # idempotent
    ops = torch.ops.mylib_alias_for_test
    X = torch.empty(2, 5, 8, device="meta"); W = torch.empty(4, 8, 6, device="meta")
    Ind = torch.empty(2, 4, 3, dtype=torch.int64, device="meta")
    assert ops.expert_gather_forward_call_fn(X, W, Ind, torch.float32).shape == (2, 4, 3, 6)
    assert ops.expert_scatter_forward_call_fn(torch.empty(2, 4, 3, 6, device="meta"), torch.empty(4, 6, 8, device="meta"), Ind, 5,
                                              torch.float32).shape == (2, 5, 8)


def test_scratch_is_allocated_per_call():
    # no buffer survives a call: nothing whose address a captured graph could keep after it has been freed or regrown
    keep, ptr, n = hk._workspace(torch.device("cpu"), 0)
    assert keep is None and ptr is None and n == 0
    keep, ptr, n = hk._workspace(torch.device("cpu"), 1000)
    assert keep.numel() == 1000 and ptr == keep.data_ptr() and n == 1000
    assert not hasattr(hk, "_workspaces")
    hk.release_workspaces()                                           # harmless no-op


def test_inference_block_traces_on_meta_tensors():
    X = torch.empty(2, 5, 64, device="meta", dtype=torch.bfloat16); Wg = torch.empty(4, 64, 32, device="meta", dtype=torch.bfloat16)
    Ws = torch.empty(4, 32, 64, device="meta", dtype=torch.bfloat16); Ind = torch.empty(2, 4, 3, dtype=torch.int16, device="meta")
    out = hk.expert_mlp_forward(X, Wg, Ws, Ind, "gelu")
    assert out.device.type == "meta" and tuple(out.shape) == (2, 5, 64) and out.dtype == torch.bfloat16
    # the heuristic that chooses between the one kernel and the separate launches
    assert hk._mlp_block_pays(64, 32, 32, 128, 64, 1) and not hk._mlp_block_pays(64, 32, 32, 128, 64, 2)
    assert hk._mlp_block_pays(64, 16, 32, 128, 64, 2) and not hk._mlp_block_pays(128, 32, 32, 128, 64, 1)
