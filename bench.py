#!/usr/bin/env python3
"""Benchmark of the MI355X hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the add + RMSNorm graph (bf16, h and r [8192, 4096]) --
the second configuration of the benchmark definition, the one its HBM metric
is quoted on -- through the hand-written HIP kernel, launched via the C-ABI
launcher on torch's current stream with all inputs already resident in HBM.
One JSON line is printed.  `value` is algorithmic bytes per second for the
timed steps; `roofline` prices the kernel against the 8 TB/s HBM peak;
`all_configs` carries the same measurement for every graph of the benchmark
definition (HIP-graph replays, so that launch overhead does not hide kernels
of a few microseconds); `cpu_baseline` is the same graph on the host cores.

Only one GPU is used; --gpus above 1 is refused.
"""
from __future__ import annotations

import argparse
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 matrix rate

# HBM-side bytes per call, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of
# `bench.py --pmc-config <n>`, each scaled by what the same counter reads for a plain
# copy kernel of known size in the same run.  Keyed by (configuration, path); an entry
# applies only while the call still launches exactly the symbols that were profiled.
MEASURED_TRAFFIC: dict = {
    ('1', 'kernel'): {"symbols": ["fused_relu_sigmoid_rowsum_f32_b256_t256"], "fetch_bytes": 16_817_825, "write_bytes": 32_732,
        "profile": "profiles/rowsum_f32_1024x4096_warm_pmc.txt"},
    ('1', 'torch.compile'): {"symbols": ["hip_row_0"], "fetch_bytes": 16_805_538, "write_bytes": 32_732,
        "profile": "profiles/rowsum_f32_1024x4096_warm_pmc.txt"},
    ('1cold', 'kernel'): {"symbols": ["fused_relu_sigmoid_rowsum_f32_b256_t256"], "fetch_bytes": 16_819_020, "write_bytes": 32_741,
        "profile": "profiles/rowsum_f32_1024x4096_cold_pmc.txt"},
    ('2', 'kernel'): {"symbols": ["add_rmsnorm_bf16_b512_t512_i1"], "fetch_bytes": 134_289_613, "write_bytes": 134_203_759,
        "profile": "profiles/add_rmsnorm_bf16_8192x4096_pmc.txt"},
    ('2', 'torch.compile'): {"symbols": ["hip_row_0"], "fetch_bytes": 134_297_805, "write_bytes": 134_282_709,
        "profile": "profiles/add_rmsnorm_bf16_8192x4096_pmc.txt"},
    ('3', 'kernel'): {"symbols": ["col_mean_var_argmax_partial_f32_c32_r8_u8", "col_mean_var_argmax_final_f32_c4_s16"], "fetch_bytes": 138_623_472, "write_bytes": 536_020,
        "profile": "profiles/col_mean_var_argmax_f32_65536x512_pmc.txt"},
    ('3', 'torch.compile'): {"symbols": ["hip_col_0_partial", "hip_col_0_final"], "fetch_bytes": 144_903_176, "write_bytes": 1_321_636,
        "profile": "profiles/col_mean_var_argmax_f32_65536x512_pmc.txt"},
    ('4a', 'kernel'): {"symbols": ["gather_rows_b16_b256_t128_r2"], "fetch_bytes": 66_422_229, "write_bytes": 67_173_304,
        "profile": "profiles/gather_rows_bf16_50304x1024_32768_pmc.txt"},
    ('4a', 'torch.compile'): {"symbols": ["hip_pointwise_0"], "fetch_bytes": 65_564_107, "write_bytes": 67_078_688,
        "profile": "profiles/gather_rows_bf16_50304x1024_32768_pmc.txt"},
    ('4b', 'kernel'): {"symbols": ["permute_copy_b16_b256_p16_t8x2"], "fetch_bytes": 268_432_000, "write_bytes": 268_533_552,
        "profile": "profiles/permute_0213_bf16_16x2048x32x128_pmc.txt"},
    ('4b', 'torch.compile'): {"symbols": ["hip_pointwise_0"], "fetch_bytes": 268_441_216, "write_bytes": 268_522_739,
        "profile": "profiles/permute_0213_bf16_16x2048x32x128_pmc.txt"},
    ('f1a', 'kernel'): {"symbols": ["ring_forward_update_bf16_d128_s8"], "fetch_bytes": 251_735_288, "write_bytes": 126_523_105,
        "profile": "profiles/ring_forward_update_bf16_8192x1x6144_n48_pmc.txt"},
    ('f1a', 'torch.compile'): {"symbols": ["hip_pointwise_0", "hip_pointwise_1"], "fetch_bytes": 327_170_359, "write_bytes": 125_696_749,
        "profile": "profiles/ring_forward_update_bf16_8192x1x6144_n48_pmc.txt"},
    ('f1b', 'torch.compile'): {"symbols": ["hip_pointwise_0", "hip_pointwise_1"], "fetch_bytes": 410_535_752, "write_bytes": 202_736_322,
        "profile": "profiles/ring_forward_update_lse_f32_1x48x8192x128_pmc.txt"},
    ('f1c', 'torch.compile'): {"symbols": ["hip_pointwise_0", "hip_pointwise_0", "hip_pointwise_0"], "fetch_bytes": 604_001_787, "write_bytes": 301_749_079,
        "profile": "profiles/ring_backward_update_bf16_3x2x16384x1x1536_pmc.txt"},
}

# Kernel durations (microseconds, average over the dispatches of a warm run) from the committed
# rocprofv3 kernel traces of `bench.py --pmc-config <n>`: the benchmark definition's "GPU time" of a
# graph is the sum over its kernels.  Keyed like MEASURED_TRAFFIC and used under the same rule.
KERNEL_TRACE_US: dict = {
    ('1', 'kernel'): {"symbols": ["fused_relu_sigmoid_rowsum_f32_b256_t256"], "us": [4.1], "profile": "profiles/rowsum_f32_1024x4096_warm_pmc.txt"},
    ('1', 'torch.compile'): {"symbols": ["hip_row_0"], "us": [4.04], "profile": "profiles/rowsum_f32_1024x4096_warm_pmc.txt"},
    ('1cold', 'kernel'): {"symbols": ["fused_relu_sigmoid_rowsum_f32_b256_t256"], "us": [6.17], "profile": "profiles/rowsum_f32_1024x4096_cold_pmc.txt"},
    ('2', 'kernel'): {"symbols": ["add_rmsnorm_bf16_b512_t512_i1"], "us": [37.99], "profile": "profiles/add_rmsnorm_bf16_8192x4096_pmc.txt"},
    ('2', 'torch.compile'): {"symbols": ["hip_row_0"], "us": [37.56], "profile": "profiles/add_rmsnorm_bf16_8192x4096_pmc.txt"},
    ('3', 'kernel'): {"symbols": ["col_mean_var_argmax_partial_f32_c32_r8_u8", "col_mean_var_argmax_final_f32_c4_s16"], "us": [23.65, 4.12], "profile": "profiles/col_mean_var_argmax_f32_65536x512_pmc.txt"},
    ('3', 'torch.compile'): {"symbols": ["hip_col_0_partial", "hip_col_0_final"], "us": [24.02, 4.78], "profile": "profiles/col_mean_var_argmax_f32_65536x512_pmc.txt"},
    ('4a', 'kernel'): {"symbols": ["gather_rows_b16_b256_t128_r2"], "us": [20.61], "profile": "profiles/gather_rows_bf16_50304x1024_32768_pmc.txt"},
    ('4a', 'torch.compile'): {"symbols": ["hip_pointwise_0"], "us": [20.31], "profile": "profiles/gather_rows_bf16_50304x1024_32768_pmc.txt"},
    ('4b', 'kernel'): {"symbols": ["permute_copy_b16_b256_p16_t8x2"], "us": [76.29], "profile": "profiles/permute_0213_bf16_16x2048x32x128_pmc.txt"},
    ('4b', 'torch.compile'): {"symbols": ["hip_pointwise_0"], "us": [76.01], "profile": "profiles/permute_0213_bf16_16x2048x32x128_pmc.txt"},
    ('f1a', 'kernel'): {"symbols": ["ring_forward_update_bf16_d128_s8"], "us": [59.16], "profile": "profiles/ring_forward_update_bf16_8192x1x6144_n48_pmc.txt"},
    ('f1a', 'torch.compile'): {"symbols": ["hip_pointwise_0", "hip_pointwise_1"], "us": [11.9, 58.43], "profile": "profiles/ring_forward_update_bf16_8192x1x6144_n48_pmc.txt"},
    ('f1b', 'torch.compile'): {"symbols": ["hip_pointwise_0", "hip_pointwise_1"], "us": [5.0, 92.55], "profile": "profiles/ring_forward_update_lse_f32_1x48x8192x128_pmc.txt"},
    ('f1c', 'torch.compile'): {"symbols": ["hip_pointwise_0", "hip_pointwise_0", "hip_pointwise_0"], "us": [47.96, 47.96, 47.96], "profile": "profiles/ring_backward_update_bf16_3x2x16384x1x1536_pmc.txt"},
    ('2cold', 'kernel'): {"symbols": ["add_rmsnorm_bf16_b512_t512_i1"], "us": [45.47], "profile": "profiles/kernel_traces_per_config.txt"},
    ('2cold', 'torch.compile'): {"symbols": ["hip_row_0"], "us": [45.06], "profile": "profiles/kernel_traces_per_config.txt"},
    ('3cold', 'kernel'): {"symbols": ["col_mean_var_argmax_partial_f32_c32_r8_u8", "col_mean_var_argmax_final_f32_c4_s16"], "us": [26.39, 4.01], "profile": "profiles/kernel_traces_per_config.txt"},
    ('3cold', 'torch.compile'): {"symbols": ["hip_col_0_partial", "hip_col_0_final"], "us": [25.89, 4.74], "profile": "profiles/kernel_traces_per_config.txt"},
    ('4acold', 'kernel'): {"symbols": ["gather_rows_b16_b256_t128_r2"], "us": [23.89], "profile": "profiles/kernel_traces_per_config.txt"},
    ('4acold', 'torch.compile'): {"symbols": ["hip_pointwise_0"], "us": [24.02], "profile": "profiles/kernel_traces_per_config.txt"},
    ('4bcold', 'kernel'): {"symbols": ["permute_copy_b16_b256_p16_t8x2"], "us": [84.4], "profile": "profiles/kernel_traces_per_config.txt"},
    ('4bcold', 'torch.compile'): {"symbols": ["hip_pointwise_0"], "us": [86.53], "profile": "profiles/kernel_traces_per_config.txt"},
    ('5', 'kernel'): {"symbols": ["fused_attention_fwd_bf16_d128_causal_v5"], "us": [575.06], "profile": "profiles/kernel_traces_per_config.txt"},
    ('5', 'torch.compile'): {"symbols": ["fused_attention_fwd_bf16_d128_causal_v5"], "us": [575.06], "profile": "profiles/kernel_traces_per_config.txt"},
    ('5b', 'kernel'): {"symbols": ["attention_bwd_stats_bf16_d128", "attention_bwd8_dk_bf16_d128_causal", "attention_bwd8_dv_bf16_d128_causal", "attention_bwd8_dq_bf16_d128_causal"], "us": [53.94, 796.63, 587.58, 759.39], "profile": "profiles/kernel_traces_per_config.txt"},
}

ALGO_BYTES = {
    "rowsum": 16_781_312,
    "add_rmsnorm": 268_443_648,
    "col_mean_var_argmax": 134_225_920,
    "gather": 134_479_872,
    "permute": 536_870_912,
}
ATTN_FLOPS_CAUSAL = 549_755_813_888


def _event_time_ms(fn, reps: int) -> float:
    import torch

    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / reps


# input sets visited in turn by the cold rows of all_configs (reads of about 1 GiB per pass)
COLD_COPIES = {"2": 8, "3": 8, "4a": 8, "4b": 4}


def _cold_sets(torch, args, copies: int) -> list:
    """`copies` input sets for one configuration: the given one plus fresh random copies of its
    large floating-point operands (small operands and index tensors are shared)."""
    dev = "cuda:0"
    return [args] + [tuple(torch.randn(a.shape, device=dev).to(a.dtype) if a.is_floating_point() and a.numel() > (1 << 20)
                           else a for a in args) for _ in range(copies - 1)]


def _graph_time_ms(fn, launches_per_graph: int = 20, replays: int = 5) -> float:
    """Per-launch time with the launches recorded in a HIP graph, so the host's
    per-launch cost does not bound kernels that run for a few microseconds."""
    import torch

    fn()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(launches_per_graph):
            fn()
    g.replay()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(replays):
        g.replay()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / (replays * launches_per_graph)


def _config_table(K, torch, only=None):
    """name -> builder of (direct call, graph function, arguments, algorithmic work, bound) for every graph
    of the benchmark definition.  Builders allocate their seeded inputs when called and not before."""
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    dev = "cuda:0"

    def c1():
        torch.manual_seed(0)
        x = torch.randn(1024, 4096).to(dev)
        return (K.fused_relu_sigmoid_rowsum, lambda x: (torch.relu(2 * x + 1) * torch.sigmoid(x)).sum(-1), (x,),
                ALGO_BYTES["rowsum"], "hbm")

    def c2():
        torch.manual_seed(0)
        h = torch.randn(8192, 4096).bfloat16().to(dev)
        r = torch.randn(8192, 4096).bfloat16().to(dev)
        w = (1 + 0.02 * torch.randn(4096)).bfloat16().to(dev)

        def rms(h, r, w):
            s = h + r
            sf = s.float()
            return (sf * torch.rsqrt(sf.pow(2).mean(-1, keepdim=True) + 1e-6) * w.float()).to(torch.bfloat16), s

        return (lambda h, r, w: K.add_rmsnorm(h, r, w, 1e-6), rms, (h, r, w), ALGO_BYTES["add_rmsnorm"], "hbm")

    def c3():
        torch.manual_seed(0)
        x = torch.randn(65536, 512).to(dev)
        return (K.col_mean_var_argmax, lambda x: (x.mean(0), x.var(0, unbiased=False), x.argmax(0)), (x,),
                ALGO_BYTES["col_mean_var_argmax"], "hbm")

    def c4a():
        torch.manual_seed(0)
        table = (0.02 * torch.randn(50304, 1024)).bfloat16().to(dev)
        idx = torch.randint(0, 50304, (32768,), dtype=torch.int64).to(dev)
        return (K.gather_rows, lambda t, i: t[i], (table, idx), ALGO_BYTES["gather"], "hbm")

    def c4b():
        torch.manual_seed(0)
        t = torch.randn(16, 2048, 32, 128).bfloat16().to(dev)
        return (K.permute_0213_contiguous, lambda t: t.permute(0, 2, 1, 3).contiguous(), (t,), ALGO_BYTES["permute"], "hbm")

    def c5():
        torch.manual_seed(0)
        q = torch.randn(4, 32, 4096, 128).bfloat16().to(dev)
        k = torch.randn(4, 32, 4096, 128).bfloat16().to(dev)
        v = torch.randn(4, 32, 4096, 128).bfloat16().to(dev)
        return (lambda q, k, v: K.fused_attention(q, k, v, 128 ** -0.5, True),
                lambda q, k, v: npu_fusion_attention_graph(q, k, v, 32, "BNSD", scale=128 ** 0.5, sparse_mode=3)[0],
                (q, k, v), ATTN_FLOPS_CAUSAL, "mfma")

    table = {
        "1 pointwise+rowsum fp32 [1024,4096] (cache-warm)": c1,
        "2 add+rmsnorm bf16 [8192,4096]": c2,
        "3 col mean/var/argmax fp32 [65536,512]": c3,
        "4a gather bf16 [50304,1024][32768]": c4a,
        "4b permute(0,2,1,3) bf16 [16,2048,32,128]": c4b,
        "5 causal attention bf16 [4,32,4096,128]": c5,
    }
    table.update(_ring_merge_table(K, torch))
    if only is not None:
        table = {k: v for k, v in table.items() if k.split()[0] == only}
    return table


def _launched_symbols(fn) -> list:
    """Kernel symbols one call of fn enqueues through the C-ABI launcher, in order."""
    from inductor_x_amd import launcher

    launcher.launch_log = []
    try:
        fn()
    finally:
        log, launcher.launch_log = launcher.launch_log, None
    return log


def _traffic_for(config: str, path: str, symbols: list, work):
    """HBM-side bytes per call from the committed counter profiles, or None when a launched symbol
    is not the one that was profiled (the table then no longer describes what ran)."""
    rec = MEASURED_TRAFFIC.get((config.split()[0], path))
    if rec is None or list(rec["symbols"]) != list(symbols):
        return None
    total = rec["fetch_bytes"] + rec["write_bytes"]
    return {"bytes": total, "fetch_bytes": rec["fetch_bytes"], "write_bytes": rec["write_bytes"],
            "over_algorithmic": round(total / work, 4), "profile": rec["profile"]}


def _kernel_us_for(config: str, path: str, symbols: list):
    """Sum of the committed kernel-trace durations of a call's kernels, or None when the call no
    longer launches the symbols that were traced."""
    rec = KERNEL_TRACE_US.get((config.split()[0], path))
    if rec is None or list(rec["symbols"]) != list(symbols):
        return None
    return round(sum(rec["us"]), 2)


def _per_config_summary(rows: list) -> dict:
    """Compact table of all_configs for the roofline object: configuration -> fraction of the roofline
    per path (and the traced kernel time where the committed trace covers the launched symbols)."""
    per: dict = {}
    for rec in rows:
        if "frac" not in rec:
            continue
        key = rec["config"].split()[0]
        path = "kernel" if rec["path"] == "kernel" else "compile"
        e = per.setdefault(key, {})
        e[path] = rec["frac"]
        kus = _kernel_us_for(rec["config"], rec["path"], rec.get("kernels", []))
        if kus is not None:
            e[path + "_kernel_us"] = kus
    return per


def _all_configs(K, torch) -> list:
    """Every graph of the benchmark definition, two ways: the hand-written kernel
    family called directly through the launcher ("kernel"), and the same graph
    written in PyTorch and compiled through the backend's import hook
    ("torch.compile": generated HIP kernels; the attention graph reaches the
    MFMA kernel through the custom op)."""
    import inductor_x_amd  # noqa: F401  registers the Inductor backend

    dev = "cuda:0"
    out = []

    def add(name, path, fn, work, bound, error=None):
        if error is not None:
            out.append({"config": name, "path": path, "error": error})
            return
        try:
            symbols = _launched_symbols(fn)
        except Exception as e:
            out.append({"config": name, "path": path, "error": f"{type(e).__name__}: {e}"[:200]})
            return
        try:
            ms = _graph_time_ms(fn)
            how = "hip-graph replay"
        except Exception as e:  # capture unsupported: time the plain loop instead
            try:
                ms = _event_time_ms(fn, 20)
                how = f"event loop ({type(e).__name__})"
            except Exception as e2:
                out.append({"config": name, "path": path, "error": f"{type(e2).__name__}: {e2}"[:200]})
                return
        rec = {"config": name, "path": path, "ms": round(ms, 5), "bound": bound, "kernels": symbols, "timing": how}
        if bound == "hbm":
            ach = work / ms / 1e6
            rec.update({"achieved": round(ach, 1), "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
                        "traffic": _traffic_for(name, path, symbols, work)})
        else:
            ach = work / ms / 1e9
            rec.update({"achieved": round(ach, 1), "unit": "TFLOP/s", "frac": round(ach / MFMA_BF16_PEAK_TFLOPS, 4)})
        out.append(rec)

    def both(name, direct, graph_fn, args, work, bound):
        if direct is not None:
            add(name, "kernel", lambda: direct(*args), work, bound)
        try:
            torch._dynamo.reset()
            cf = torch.compile(graph_fn)
            cf(*args)
            add(name, "torch.compile", lambda: cf(*args), work, bound)
        except Exception as e:
            out.append({"config": name, "path": "torch.compile", "error": f"{type(e).__name__}: {e}"[:200]})

    for name, build in _config_table(K, torch).items():
        direct, graph_fn, args, work, bound = build()
        both(name, direct, graph_fn, args, work, bound)
        if name.startswith("1 "):
            # The same kernel on inputs that cannot be cache-resident: 72 distinct 16 MiB
            # inputs (1.1 GiB, several times the 256 MB memory-side cache) visited in
            # turn, one pass over all of them per graph replay.
            xs = [args[0]] + [torch.randn(1024, 4096, device=dev) for _ in range(71)]
            turn = [0]

            def cold():
                turn[0] = (turn[0] + 1) % len(xs)
                return K.fused_relu_sigmoid_rowsum(xs[turn[0]])

            cname = "1cold pointwise+rowsum fp32 [1024,4096] (cold: 72 inputs in turn)"
            try:
                ms = _graph_time_ms(cold, launches_per_graph=len(xs))
                ach = ALGO_BYTES["rowsum"] / ms / 1e6
                syms = _launched_symbols(cold)
                out.append({"config": cname, "path": "kernel", "ms": round(ms, 5), "bound": "hbm", "kernels": syms,
                            "achieved": round(ach, 1), "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
                            "timing": "hip-graph replay",
                            "traffic": _traffic_for(cname, "kernel", syms, ALGO_BYTES["rowsum"])})
            except Exception as e:
                out.append({"config": cname, "path": "kernel", "error": f"{type(e).__name__}: {e}"[:200]})
            del xs
        if name.split()[0] in COLD_COPIES:
            # The same graph on inputs that cannot be cache-resident: several distinct sets of the
            # large operands (about 1 GiB of reads together, four times the memory-side cache)
            # visited in turn, one pass over all of them per graph replay.  The rows above replay
            # one input set, whose reads the 256 MiB cache can partly serve again.
            copies = COLD_COPIES[name.split()[0]]
            sets = _cold_sets(torch, args, copies)
            cname = name.split()[0] + "cold " + name.split(" ", 1)[1] + f" (cold: {copies} input sets in turn)"
            for path, call in (("kernel", direct), ("torch.compile", None)):
                turn = [0]
                if call is None:
                    try:
                        torch._dynamo.reset()
                        call = torch.compile(graph_fn)
                        call(*args)
                    except Exception as e:
                        out.append({"config": cname, "path": path, "error": f"{type(e).__name__}: {e}"[:200]})
                        continue

                def cold(call=call, turn=turn):
                    turn[0] = (turn[0] + 1) % len(sets)
                    return call(*sets[turn[0]])

                try:
                    ms = _graph_time_ms(cold, launches_per_graph=len(sets))
                    ach = work / ms / 1e6
                    out.append({"config": cname, "path": path, "ms": round(ms, 5), "bound": bound,
                                "kernels": _launched_symbols(cold), "achieved": round(ach, 1), "unit": "GB/s",
                                "frac": round(ach / HBM_PEAK_GBS, 4), "timing": "hip-graph replay", "traffic": None})
                except Exception as e:
                    out.append({"config": cname, "path": path, "error": f"{type(e).__name__}: {e}"[:200]})
            del sets
        if name.startswith("5 "):
            # Backward of the same graph (the caller next to the forward on the
            # training path): five matrix products plus two recomputed ones, counted
            # by the usual convention as 2.5 x the forward's algorithmic FLOPs.
            q, k, v = args
            o, m, l = K.fused_attention(q, k, v, 128 ** -0.5, True)[:3]
            do = torch.randn_like(o)
            add("5b causal attention backward bf16 [4,32,4096,128]", "kernel",
                lambda: K.fused_attention_backward(q, k, v, o, do, m, l, 128 ** -0.5, True), 2.5 * ATTN_FLOPS_CAUSAL, "mfma")
            del o, m, l, do
        del direct, graph_fn, args
    return out


def _ring_merge_table(K, torch) -> dict:
    """The merge steps of ring attention at the reference's shapes (the callers next to the fused
    attention op on a sequence-parallel path); HBM-bound.  Algorithmic bytes: every operand read
    once, every result written once.  name -> builder of (direct call or None, graph function,
    arguments, algorithmic bytes, bound), as _config_table."""
    dev = "cuda:0"

    def trans(x):
        b, n, s, d = x.shape
        return x.permute(2, 0, 1, 3).reshape(s, b, n * d)

    def bcast(x, h):
        n = x.shape[1]
        return trans(x[..., 0].unsqueeze(3).repeat(1, 1, 1, h // n))

    def forward_update(po, pm, ps, co, cm, cs):
        m = torch.maximum(pm, cm)
        a, b = ps * torch.exp(pm - m), cs * torch.exp(cm - m)
        tot = a + b
        return (po * bcast(a / tot, po.shape[-1]) + co * bcast(b / tot, po.shape[-1])).to(po.dtype), m, tot

    def forward_update_la(po, pl, co, cl):
        lse = torch.log(torch.exp(cl) + torch.exp(pl))
        return torch.exp(pl - lse) * po + torch.exp(cl - lse) * co, lse

    def backward_update(dq, dk, dv, cdq, cdk, cdv):
        dq.add_(cdq.view(dq.shape))
        dk.add_(cdk.view(dk.shape))
        dv.add_(cdv.view(dv.shape))

    def f1a():
        torch.manual_seed(0)
        DS, B, H, N = 8192, 1, 6144, 48
        st = lambda off: (torch.rand(B, N, DS, device=dev) + off).unsqueeze(3).repeat(1, 1, 1, 8).contiguous()  # noqa: E731
        args = (torch.randn(DS, B, H, device=dev).bfloat16(), st(0.0), st(0.5), torch.randn(DS, B, H, device=dev).bfloat16(),
                st(0.0), st(0.5))
        return K.ring_forward_update, forward_update, args, 3 * DS * B * H * 2 + 6 * B * N * DS * 8 * 4, "hbm"

    def f1b():
        torch.manual_seed(0)
        B, N, DS, D = 1, 48, 8192, 128
        args = (torch.randn(B, N, DS, D, device=dev), torch.rand(B, N, DS, 1, device=dev), torch.randn(B, N, DS, D, device=dev),
                torch.rand(B, N, DS, 1, device=dev))
        return None, forward_update_la, args, 3 * B * N * DS * D * 4 + 3 * B * N * DS * 4, "hbm"

    def f1c():
        torch.manual_seed(0)
        S, B, H = 16384, 1, 1536
        args = tuple(torch.randn(2, S, B, H, device=dev).bfloat16() for _ in range(3)) + tuple(
            torch.randn(2 * S, B, H, device=dev).bfloat16() for _ in range(3))
        return None, backward_update, args, 3 * 3 * 2 * S * B * H * 2, "hbm"

    return {
        "f1a ring forward_update bf16 [8192,1,6144] N=48": f1a,
        "f1b ring forward_update (log-sum-exp) fp32 [1,48,8192,128]": f1b,
        "f1c ring backward_update bf16 3 x [2,16384,1,1536]": f1c,
    }


def _pmc_run(K, torch, which: str, steps: int, warmup: int) -> dict:
    """Plain (ungraphed) launches of one configuration, both paths, plus the copy probe: the
    program a counter collection run (rocprofv3 --pmc) wraps.  Counters come back per dispatch
    and per kernel name, so the two paths and the probe separate in the output."""
    import inductor_x_amd  # noqa: F401

    dev = "cuda:0"
    res = {"pmc_config": which, "steps": steps}
    cold = which.endswith("cold")
    base = which[:-4] if cold else which
    table = _config_table(K, torch, only=base)
    if not table or (cold and base != "1" and base not in COLD_COPIES):
        raise SystemExit(f"bench.py: no configuration {which!r} (1, 1cold, 2, 2cold, 3, 3cold, 4a, 4acold, 4b, 4bcold, 5, f1a, f1b, f1c)")
    (name, build), = table.items()
    direct, graph_fn, args, work, bound = build()
    if cold and base == "1":
        sets = [args] + [(torch.randn(1024, 4096, device=dev),) for _ in range(71)]
    elif cold:
        sets = _cold_sets(torch, args, COLD_COPIES[base])
    else:
        sets = [args]
    if direct is not None:
        for i in range(warmup + steps):
            direct(*sets[i % len(sets)])
        res["kernels"] = _launched_symbols(lambda: direct(*args))
    if not (cold and base == "1"):
        torch._dynamo.reset()
        cf = torch.compile(graph_fn)
        for i in range(warmup + steps):
            cf(*sets[i % len(sets)])
        res["compiled_kernels"] = _launched_symbols(lambda: cf(*args))
    torch.cuda.synchronize()
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    for _ in range(10):
        K.copy_bytes(dst, src)
    torch.cuda.synchronize()
    res["copy_probe"] = {"kernel": "copy_b128", "bytes_read": 256 << 20, "bytes_written": 256 << 20, "launches": 10}
    return res


# --------------------------------------------------------------------------
# CPU baseline leg (own process: it must not see the backend's import hook)
# --------------------------------------------------------------------------
def _cpu_baseline_child() -> None:
    """Times the add + RMSNorm graph on the host: Inductor's C++/OpenMP code
    generation (torch.compile on CPU tensors) at the full [8192, 4096] shape,
    and the C oracle (the checker's port) on a 1024-row sample."""
    import numpy as np
    import torch

    res = {"cores": torch.get_num_threads(), "cpu_count": os.cpu_count()}
    torch.manual_seed(0)
    rows, cols = 8192, 4096
    h = torch.randn(rows, cols).bfloat16()
    r = torch.randn(rows, cols).bfloat16()
    w = (1 + 0.02 * torch.randn(cols)).bfloat16()

    def f(h, r, w):
        s = h + r
        sf = s.float()
        out = (sf * torch.rsqrt(sf.pow(2).mean(-1, keepdim=True) + 1e-6) * w.float()).to(torch.bfloat16)
        return out, s

    try:
        cf = torch.compile(f)
        t0 = time.perf_counter()
        cf(h, r, w)
        res["inductor_compile_s"] = round(time.perf_counter() - t0, 1)
        for _ in range(3):
            cf(h, r, w)
        ts = []
        for _ in range(15):
            t0 = time.perf_counter()
            cf(h, r, w)
            ts.append(time.perf_counter() - t0)
        ms = sorted(ts)[len(ts) // 2] * 1e3
        res["inductor_ms"] = round(ms, 3)
        res["inductor_gbs"] = round(ALGO_BYTES["add_rmsnorm"] / ms / 1e6, 2)
    except Exception as e:  # no host compiler etc.
        res["inductor_error"] = f"{type(e).__name__}: {e}"[:200]
    try:
        from oracle import oracle as O

        bits = lambda t: t.view(torch.int16).numpy().view(np.uint16)  # noqa: E731
        n = 1024
        hb, rb, wb = bits(h[:n]), bits(r[:n]), bits(w)
        O.add_rmsnorm_bf16(hb, rb, wb)
        ts = []
        for _ in range(5):
            t0 = time.perf_counter()
            O.add_rmsnorm_bf16(hb, rb, wb)
            ts.append(time.perf_counter() - t0)
        ms = sorted(ts)[len(ts) // 2] * 1e3
        res["oracle_ms_1024_rows"] = round(ms, 3)
        res["oracle_gbs"] = round(ALGO_BYTES["add_rmsnorm"] * n / rows / ms / 1e6, 2)
        res["oracle_threads"] = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    except Exception as e:
        res["oracle_error"] = f"{type(e).__name__}: {e}"[:200]
    res["all_configs"] = _cpu_all_configs(torch)
    print("CPU_BASELINE " + json.dumps(res))


def _cpu_all_configs(torch) -> list:
    """The other graphs of the benchmark definition on the host, same seeded
    inputs, torch.compile on CPU tensors (attention: the library's fused CPU
    kernel inside the compiled function, as the unfused graph would hold an
    8 GiB score tensor).  A few calls each: a baseline, not a target."""
    import torch.nn.functional as F

    out = []

    def run(name, fn, args, work, unit, warm, reps):
        try:
            cf = torch.compile(fn)
            for _ in range(warm):
                cf(*args)
            ts = []
            for _ in range(reps):
                t0 = time.perf_counter()
                cf(*args)
                ts.append(time.perf_counter() - t0)
            ms = sorted(ts)[len(ts) // 2] * 1e3
            scale = 1e6 if unit == "GB/s" else 1e9
            out.append({"config": name, "ms": round(ms, 3), "achieved": round(work / ms / scale, 3), "unit": unit,
                        "calls": reps})
        except Exception as e:
            out.append({"config": name, "error": f"{type(e).__name__}: {e}"[:200]})

    torch.manual_seed(0)
    x = torch.randn(1024, 4096)
    run("1 pointwise+rowsum fp32 [1024,4096]", lambda x: (torch.relu(2 * x + 1) * torch.sigmoid(x)).sum(-1), (x,),
        ALGO_BYTES["rowsum"], "GB/s", 3, 15)
    torch.manual_seed(0)
    x = torch.randn(65536, 512)
    run("3 col mean/var/argmax fp32 [65536,512]", lambda x: (x.mean(0), x.var(0, unbiased=False), x.argmax(0)), (x,),
        ALGO_BYTES["col_mean_var_argmax"], "GB/s", 2, 7)
    torch.manual_seed(0)
    table = (0.02 * torch.randn(50304, 1024)).bfloat16()
    idx = torch.randint(0, 50304, (32768,), dtype=torch.int64)
    run("4a gather bf16 [50304,1024][32768]", lambda t, i: t[i], (table, idx), ALGO_BYTES["gather"], "GB/s", 2, 7)
    del table, idx
    torch.manual_seed(0)
    t = torch.randn(16, 2048, 32, 128).bfloat16()
    run("4b permute(0,2,1,3) bf16 [16,2048,32,128]", lambda t: t.permute(0, 2, 1, 3).contiguous(), (t,),
        ALGO_BYTES["permute"], "GB/s", 2, 5)
    del t
    torch.manual_seed(0)
    q = torch.randn(4, 32, 4096, 128).bfloat16()
    k = torch.randn(4, 32, 4096, 128).bfloat16()
    v = torch.randn(4, 32, 4096, 128).bfloat16()
    run("5 causal attention bf16 [4,32,4096,128]",
        lambda q, k, v: F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=128 ** -0.5), (q, k, v),
        ATTN_FLOPS_CAUSAL, "TFLOP/s", 1, 3)
    return out


def _cpu_baseline() -> dict:
    try:
        proc = subprocess.run(
            [sys.executable, os.path.abspath(__file__), "--cpu-baseline-child"],
            capture_output=True, text=True, timeout=420, cwd=ROOT,
        )
        line = [l for l in proc.stdout.splitlines() if l.startswith("CPU_BASELINE ")]
        if not line:
            return {"value": None, "unit": "GB/s", "cores": None, "kind": "port",
                    "sample": "cpu baseline leg produced no result: " + proc.stderr[-200:]}
        res = json.loads(line[-1][len("CPU_BASELINE "):])
    except Exception as e:
        return {"value": None, "unit": "GB/s", "cores": None, "kind": "port", "sample": f"failed: {e}"[:200]}
    if "inductor_gbs" in res:
        return {
            "value": res["inductor_gbs"], "unit": "GB/s", "cores": res["cores"], "kind": "port",
            "sample": "same add+rmsnorm graph, full [8192,4096] bf16, torch.compile on CPU tensors "
                      "(Inductor C++/OpenMP codegen), median of 15 calls after 4 warm-ups",
            "ms": res["inductor_ms"], "compile_s": res.get("inductor_compile_s"), "host_cpus": res["cpu_count"],
            "oracle_port": {"value": res.get("oracle_gbs"), "unit": "GB/s", "threads": res.get("oracle_threads"),
                            "sample": "C oracle (oracle/oracle.c, OpenMP) on the first 1024 rows, median of 5"},
            "all_configs": res.get("all_configs"),
        }
    return {
        "value": res.get("oracle_gbs"), "unit": "GB/s", "cores": res.get("oracle_threads"), "kind": "port",
        "sample": "C oracle (oracle/oracle.c, OpenMP) on the first 1024 of 8192 rows, median of 5; "
                  "Inductor CPU leg failed: " + res.get("inductor_error", "?"),
    }


def _launch_floor(K, torch) -> dict:
    """Per-launch time of a kernel that moves next to nothing (a 4 KiB copy by one workgroup) and
    of the cfg 1 row sum, both as 20 dependent launches per HIP graph: the first is what this
    machine charges for a launch in a chain, whatever the kernel does."""
    dev = "cuda:0"
    torch.manual_seed(0)
    a = torch.zeros(4096, dtype=torch.uint8, device=dev)
    b = torch.empty_like(a)
    x = torch.randn(1024, 4096, device=dev)
    for _ in range(30):
        K.copy_bytes(b, a)
        K.fused_relu_sigmoid_rowsum(x)
    tiny = min(_graph_time_ms(lambda: K.copy_bytes(b, a)) for _ in range(3))
    rows = min(_graph_time_ms(lambda: K.fused_relu_sigmoid_rowsum(x)) for _ in range(3))
    return {"launch_floor_us": round(tiny * 1e3, 3), "kernel": "copy_b128 (4 KiB, one workgroup)",
            "cfg1_us": round(rows * 1e3, 3), "cfg1_kernel": _launched_symbols(lambda: K.fused_relu_sigmoid_rowsum(x)),
            "cfg1_at_peak_us": round(ALGO_BYTES["rowsum"] / HBM_PEAK_GBS / 1e3, 3),
            "timing": "hip-graph replay, 20 dependent launches per graph, best of 3 x 5 replays"}


def _attention_ceiling(torch) -> dict:
    """Rates of the probe kernels (one workgroup of eight wavefronts per CU, 256 workgroups): nanoseconds per
    step -- one MFMA 32x32x16 bf16 and / or one 1 KiB LDS fragment -- and what follows from them."""
    from inductor_x_amd import codecache, launcher

    path = codecache.compile_source(codecache.probe_source("probe_kernels.hip"), label="probe_kernels", prefer_intree=True)
    with open(path, "rb") as f:
        mod = launcher.Module(f.read(), label="probe_kernels")
    out = torch.zeros(512, device="cuda:0")
    stream = torch._C._cuda_getCurrentRawStream(0)
    iters = 20000
    names = ["mfma_only", "ds_read_b128_only", "ds_read_b64_x2_only", "ds_read_b64_tr_b16_x2_only",
             "fragment_per_mfma", "mfma_with_vector_work", "fragment_per_mfma_with_vector_work"]
    ns = {}
    for mode, name in enumerate(names):
        fn = mod.function(f"attention_resource_probe_m{mode}")
        launch = lambda: fn.launch("Pi", (out.data_ptr(), iters), (256, 1, 1), (512,), stream, 65536)  # noqa: E731
        for _ in range(3):
            launch()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):
            t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0.record()
            launch()
            t1.record()
            t1.synchronize()
            best = min(best, t0.elapsed_time(t1))
        ns[name] = best * 1e6 / (iters * 16) / 2  # per step per SIMD (two wavefronts share one)
    # the 64-queries-per-wavefront design: four wavefronts (one per SIMD), two MFMAs per step
    fn = mod.function("attention_resource_probe_m7")
    for _ in range(3):
        fn.launch("Pi", (out.data_ptr(), iters), (256, 1, 1), (256,), stream, 65536)
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(3):
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        fn.launch("Pi", (out.data_ptr(), iters), (256, 1, 1), (256,), stream, 65536)
        t1.record()
        t1.synchronize()
        best = min(best, t0.elapsed_time(t1))
    ns_wide = best * 1e6 / (iters * 16) / 2  # per MFMA per SIMD
    mfma = ns["mfma_only"]  # 32 cycles
    clock_ghz = 32 / mfma
    lds = lambda n: round(4 * 1024 / (ns[n] / mfma * 32), 1)  # noqa: E731  bytes per clock per CU
    frac = lambda n: round(mfma / ns[n], 3)  # noqa: E731
    return {
        "ns_per_step_per_simd": {k: round(v, 2) for k, v in ns.items()},
        "clock_ghz_under_mfma_load": round(clock_ghz, 3),
        "lds_bytes_per_clock_per_cu": {n: lds(n) for n in names[1:4]},
        "lds_bytes_per_clock_needed_at_full_mfma_rate": 128.0,
        "mfma_rate_vs_alone": {n: frac(n) for n in names[4:]},
        "ceiling_of_datasheet_peak": round(frac(names[6]) * clock_ghz / 2.4, 3),
        "one_wavefront_per_simd_64_queries": {"ns_per_mfma_per_simd": round(ns_wide, 2), "mfma_rate_vs_alone": round(mfma / ns_wide, 3),
                                              "ceiling_of_datasheet_peak": round(mfma / ns_wide * clock_ghz / 2.4, 3)},
        "note": "fragment_per_mfma_with_vector_work is the instruction mix of the attention loop (one fragment, four "
                "fma, one exp2, one add per MFMA, two wavefronts per SIMD) with no dependence between the three streams",
    }


def _attention_timeline(torch) -> dict:
    """Where a workgroup of the fused attention forward spends its time at q, k, v [4,32,4096,128] bf16: the
    measurement build of the shipped kernel template (csrc/probes/attention_timeline.hip) records the 100 MHz
    clock at seven points of every query block; ten launches back to back, the last one is read."""
    import numpy as np

    from inductor_x_amd import codecache, kernels as K, launcher

    path = codecache.compile_source(codecache.probe_source("attention_timeline.hip"), label="attention_timeline", prefer_intree=True)
    with open(path, "rb") as f:
        mod = launcher.Module(f.read(), label="attention_timeline")
    dev = "cuda:0"
    torch.manual_seed(0)
    B, N, S, D = 4, 32, 4096, 128
    q, k, v = (torch.randn(B, N, S, D, device=dev).bfloat16() for _ in range(3))
    scale = D ** -0.5
    n_qb = S // 256
    n_blocks = B * N * n_qb
    out = torch.empty_like(q)
    smax = torch.empty(B, N, S, 8, device=dev)
    ssum = torch.empty_like(smax)
    times = torch.zeros(n_blocks * 2 * 8, dtype=torch.int64, device=dev)
    stream = torch._C._cuda_getCurrentRawStream(0)
    cus = launcher.device_props(0).cu_count
    res = {"shape": [B, N, S, D], "clock": "s_memrealtime, 100 MHz", "launches": "10 back to back after 10 warm-ups, last one read"}
    for causal, name in ((True, "causal"), (False, "full")):
        fn = mod.function(f"attention_timeline_bf16_d128_{name}")
        per_head = (n_qb + 1) // 2 if causal else n_qb
        grid = (min(8 * ((B * N + 7) // 8) * per_head, 8 * (cus // 8)), 1, 1)
        launch = lambda: fn.launch("PPPPPPiiifP", (q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), smax.data_ptr(),  # noqa: E731
                                                   ssum.data_ptr(), B * N, S, S, scale * 1.4426950408889634, times.data_ptr()),
                                   grid, (512,), stream, 65536)
        ref = K.fused_attention(q, k, v, scale, causal)
        for _ in range(10):
            launch()
        torch.cuda.synchronize()
        same = bool(torch.equal(out, ref[0]) and torch.equal(smax, ref[1]) and torch.equal(ssum, ref[2]))
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        for _ in range(10):
            launch()
        t1.record()
        t1.synchronize()
        tr = times.cpu().numpy().reshape(n_blocks, 2, 8).astype(np.float64)
        us = tr[:, :, :7] * 0.01
        w0 = us[:, 0, :]
        qb = np.arange(n_blocks) % n_qb
        tiles = (4 * qb + 4) if causal else np.full(n_blocks, S // 64)
        seg = lambda a, b, m=slice(None): float(np.mean(w0[m, b] - w0[m, a]))  # noqa: E731
        unguarded_tiles = np.maximum(tiles - (6 if causal else 2), 0)  # first step and last step lie outside, causal: the diagonal too
        long_blocks = unguarded_tiles >= 8
        per_tile = float(np.sum((w0[:, 3] - w0[:, 2])[long_blocks]) / np.sum(unguarded_tiles[long_blocks]))
        start = w0[:, 0].min()
        wg = tr[:, 0, 7].astype(np.int64)
        ends, gaps = {}, []
        for g in np.unique(wg):
            m = np.where(wg == g)[0]
            o = m[np.argsort(w0[m, 0])]
            block_end = us[o, :, 6].max(axis=1)
            ends[int(g)] = block_end[-1] - start
            gaps += list(w0[o[1:], 0] - block_end[:-1])
        end = np.array([ends[g] for g in sorted(ends)])
        die = np.array(sorted(ends)) % 8
        row = {
            "matches_shipped_kernel": same,
            "launch_us_mean_of_10": round(t0.elapsed_time(t1) * 100, 1),
            "traced_launch_span_us": round(float(us[:, :, 6].max() - start), 1),
            "mean_us_per_query_block": {
                "queries_and_first_two_k_tiles_land": round(seg(0, 1), 2),
                "first_score_product_and_first_step": round(seg(1, 2), 2),
                "unguarded_steps": round(seg(2, 3), 2),
                "guarded_steps_and_last_step": round(seg(3, 4), 2),
                "normalise_stage_issue_stores": round(seg(4, 5), 2),
                "statistics_and_barrier": round(seg(5, 6), 2),
                "whole_block": round(seg(0, 6), 2),
                "idle_before_next_block": round(float(np.mean(gaps)), 2),
            },
            "us_per_unguarded_tile_step": round(per_tile, 3),
            "mean_tiles_per_block": float(np.mean(tiles)),
            "us_per_block_beyond_tiles_times_step": round(seg(0, 6) + float(np.mean(gaps)) - float(np.mean(tiles)) * per_tile, 2),
            "workgroup_end_us": {"mean": round(float(end.mean()), 1), "max": round(float(end.max()), 1),
                                 "per_die_mean": [round(float(end[die == x].mean()), 1) for x in range(8)],
                                 "spread_within_a_die_max": round(float(max(end[die == x].max() - end[die == x].min() for x in range(8))), 1)},
        }
        if causal:
            row["by_query_block"] = {
                str(b): {"tiles": 4 * b + 4, "land": round(seg(0, 1, qb == b), 2), "first": round(seg(1, 2, qb == b), 2),
                         "unguarded": round(seg(2, 3, qb == b), 2), "guarded_and_last": round(seg(3, 4, qb == b), 2),
                         "epilogue": round(seg(4, 6, qb == b), 2), "block": round(seg(0, 6, qb == b), 2)}
                for b in (0, 1, 7, 8, 15)}
        res[name] = row
    return res


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=int(os.environ.get("WORLD_SIZE", "1")))
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-all-configs", action="store_true")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 256 MiB copy kernel 10 times (calibrates HBM byte counters under rocprofv3 --pmc)")
    ap.add_argument("--pmc-config", default=None,
                    help="run only plain launches of one configuration (1, 2, 3, 4a, 4b, 5, f1a, f1b, f1c; 1cold, 2cold, 3cold, "
                         "4acold, 4bcold visit several input sets in turn), both paths, and the "
                         "copy probe: the program for a rocprofv3 --pmc counter run")
    ap.add_argument("--launch-floor", action="store_true",
                    help="time a 4 KiB copy (one workgroup) and the cfg 1 row sum the same way, 20 dependent launches per "
                         "HIP graph: what a launch costs on this machine before any data moves")
    ap.add_argument("--attention-timeline", action="store_true",
                    help="run the measurement build of the fused attention forward (csrc/probes/attention_timeline.hip) "
                         "and print where a workgroup's time goes per query block")
    ap.add_argument("--attention-ceiling", action="store_true",
                    help="run the resource probes of csrc/probes/probe_kernels.hip: what one CU sustains of MFMA, LDS operand "
                         "reads and softmax-like vector work, alone and together (the ceiling of the attention design)")
    ap.add_argument("--cpu-baseline-child", action="store_true", help=argparse.SUPPRESS)
    args = ap.parse_args()

    if args.cpu_baseline_child:
        _cpu_baseline_child()
        return
    if args.gpus != 1:
        print("bench.py: this build uses exactly one GPU (no collectives, no sharding); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from inductor_x_amd import kernels as K

    if args.pmc_config is not None:
        print(json.dumps(_pmc_run(K, torch, args.pmc_config, args.steps, args.warmup)))
        return
    if args.launch_floor:
        print(json.dumps(_launch_floor(K, torch)))
        return
    if args.attention_timeline:
        print(json.dumps(_attention_timeline(torch)))
        return
    if args.attention_ceiling:
        print(json.dumps(_attention_ceiling(torch)))
        return
    dev = "cuda:0"
    torch.manual_seed(0)
    rows, cols = 8192, 4096
    h = torch.randn(rows, cols).bfloat16().to(dev)
    r = torch.randn(rows, cols).bfloat16().to(dev)
    w = (1 + 0.02 * torch.randn(cols)).bfloat16().to(dev)

    def step():
        return K.add_rmsnorm(h, r, w, 1e-6)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        step()
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ev_ms = start.elapsed_time(end)
    ms_per_step = wall_ms / args.steps
    kernel_ms = ev_ms / args.steps  # one kernel per step: event time per launch
    value = ALGO_BYTES["add_rmsnorm"] / ms_per_step / 1e6
    achieved = ALGO_BYTES["add_rmsnorm"] / kernel_ms / 1e6

    line = {
        "metric": "fused-kernel HBM GB/s (add+rmsnorm bf16); all_configs carries every graph incl. fused-attn TFLOP/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic (seed 0, N(0,1) h and r, N(1,0.02) weight), resident in HBM before timing",
        "config": {"workload": "residual-add + RMSNorm, bf16, h,r [8192,4096], w [4096], eps 1e-6, returns (norm, h+r)",
                   "algorithmic_bytes_per_step": ALGO_BYTES["add_rmsnorm"]},
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": None,
        },
    }
    step_symbols = _launched_symbols(step)
    line["config"]["kernel"] = step_symbols
    tr = _traffic_for("2 add+rmsnorm", "kernel", step_symbols, ALGO_BYTES["add_rmsnorm"])
    if tr is not None:
        line["roofline"]["traffic"] = tr["bytes"]
        line["roofline"]["traffic_profile"] = tr["profile"]
    del h, r, w
    if args.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(10):
            K.copy_bytes(dst, src)
        torch.cuda.synchronize()
        line["copy_probe"] = {"kernel": "copy_b128", "bytes_read": 256 << 20, "bytes_written": 256 << 20, "launches": 10}
        del src, dst
    if not args.no_all_configs:
        line["all_configs"] = _all_configs(K, torch)
        per = _per_config_summary(line["all_configs"])
        # `frac` replays one input set, whose reads the 256 MiB memory-side cache partly serves again;
        # `frac_cold` visits eight input sets in turn (1 GiB of reads per pass): the figure for HBM itself
        line["roofline"]["frac_cold"] = per.get("2cold", {}).get("kernel")
        line["roofline"]["per_config"] = per
        line["roofline"]["per_config_note"] = ("fraction of 8 TB/s (configs 1-4, f1*) or of 2.5 PFLOP/s bf16 (5, 5b); 'kernel' = "
                                               "hand-written family, 'compile' = through torch.compile; '*cold' rows visit several "
                                               "input sets in turn so nothing is cache-resident; '*_kernel_us' = committed rocprofv3 "
                                               "kernel-trace duration of the launched symbols")
    line["cpu_baseline"] = (
        {"value": None, "unit": "GB/s", "cores": None, "kind": "port", "sample": "skipped (--no-cpu-baseline)"}
        if args.no_cpu_baseline else _cpu_baseline()
    )
    print(json.dumps(line))


if __name__ == "__main__":
    main()
