#!/usr/bin/env python3
"""Benchmark of the sparse-plus-dense GEMM path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

A *step* is one pass of the hot path over the configuration the metric is quoted on:
the fp32 CSR SpMM sweep of config 2 (4096x4096 sparse A at 70/80/90/95/98 % sparsity with
geometric row lengths, times a dense 4096 x {64,128,256} B) = 15 SpMM launches, captured
once into a hipGraph through the graph builder and replayed.  All operands are resident
in HBM before the timed region; CSR construction is set-up work and is not timed.

One JSON line is printed.  ``value`` = algorithmic GB of one sweep / seconds per sweep.
``roofline`` describes the SpMM kernel instantiation that takes the most time in the
sweep; ``cpu_baseline`` is the single-core C port of the same sweep timed on this host;
``extras`` holds the per-cell table, the fp16 sweep, SDDMM (configs 1 and 3), the bf16
MFMA GEMM and the sparse+dense co-run of config 4 (serialized / two-branch graph / fused).
"""
from __future__ import annotations

import argparse
import contextlib
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0           # MI355X HBM3E
MFMA_PEAK_TFLOPS_16BIT = 2500.0  # dense bf16 / fp16
VALU_PEAK_TFLOPS_FP32 = 78.6     # vector fp32 FMA without packed math (the build disables v_pk_*_f32)
CELL_REPEATS = 20                # launches of one cell inside its timing graph
# HBM-side bytes per launch (L2 misses + write-backs), mean over the five sparsities a kernel serves in
# the sweep, from two `rocprofv3 --pmc` runs (FETCH_SIZE, WRITE_SIZE) of `bench.py --pmc-probe`, each
# scaled by the counter's reading for a plain 256 MiB copy (x2.000 and x1.000): see
# profiles/spmm_fp32_config2_hbm_traffic_pmc.txt.  Counters cannot be read inside a timing run.
MEASURED_TRAFFIC_MB = {   # (sparsity, n) -> MB per launch of the row kernel
    (0.7, 64): 51.30, (0.7, 128): 61.56, (0.7, 256): 174.86, (0.8, 64): 37.78, (0.8, 128): 47.37, (0.8, 256): 134.22,
    (0.9, 64): 24.31, (0.9, 128): 33.78, (0.9, 256): 83.51, (0.95, 64): 17.59, (0.95, 128): 27.04, (0.95, 256): 61.88,
    (0.98, 64): 13.56, (0.98, 128): 23.01, (0.98, 256): 49.03,
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-extras", action="store_true", help="skip fp16 / SDDMM / GEMM / co-run sections")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="for `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE`: 3 plain copies of 256 MiB (iex_copy_bytes), then "
                         "3 launches of each cell of the dominant SpMM kernel, and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py measures one GPU: every box of this build has a single MI355X and the path has no "
            "cross-GPU step (rows of A shard with no exchange). Run with --gpus 1.")
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        log("bench.py needs a GPU (the product path has no CPU fallback).")
        sys.exit(2)
    import intrasm_engine_amd  # noqa: F401
    from intrasm_engine_amd import workloads as W
    from intrasm_engine_amd import interleaving as IL
    from intrasm_engine_amd.pytorch.cpp_extensions.cuda_graph_constructor import TorchCUDAGraphConstructor

    ops = torch.ops.iex_ops
    dev = torch.device("cuda:0")
    t_setup = time.time()

    # ------------------------------------------------------------- inputs (config 2)
    mats = {s: W.config2_matrix(s) for s in W.C2_SPARSITIES}
    dens = {n: W.config2_dense(n) for n in W.C2_NS}

    def csr_dev(csr, vdtype=torch.float32, idtype=torch.int32):
        return (torch.from_numpy(csr.row_indices).to(dev), torch.from_numpy(csr.values).to(dev).to(vdtype),
                torch.from_numpy(csr.row_offsets).to(dev), torch.from_numpy(csr.column_indices).to(dev).to(idtype))

    mats32 = {s: csr_dev(m) for s, m in mats.items()}
    dens32 = {n: torch.from_numpy(b).to(dev) for n, b in dens.items()}
    cells = [(s, n) for s in W.C2_SPARSITIES for n in W.C2_NS]

    def spmm32(s, n):
        ri, v, ro, ci = mats32[s]
        return lambda: ops.spmm_sputnik_reuse_weight(dens32[n], ri, v, ro, ci, mats[s].m)

    def cell_bytes(s, n, sv=4, si=4):
        c = mats[s]
        return W.spmm_bytes(c.m, c.k, n, c.nnz, 1, sv, si)

    if args.pmc_probe:
        from intrasm_engine_amd import _lib
        nbytes = 256 << 20
        src = torch.zeros(nbytes // 4, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            _lib.check(_lib.load().iex_copy_bytes(dst.data_ptr(), src.data_ptr(), nbytes,
                                                  torch.cuda.current_stream().cuda_stream), "copy")
        torch.cuda.synchronize()
        for s_, n_ in cells:       # dispatch order = cell order, 3 launches each
            fn = spmm32(s_, n_)
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
        log(f"[bench] pmc probe done: copy of {nbytes} bytes x3 (copy_kernel), then every fp32 cell x3 in the order "
            + " ".join(f"({s_},{n_}):{cell_bytes(s_, n_)}B" for s_, n_ in cells))
        return

    sweep_bytes = sum(cell_bytes(s, n) for s, n in cells)
    sweep_flops = sum(W.spmm_flops(mats[s].nnz, n) for s, n in cells)
    log(f"[bench] set-up {time.time() - t_setup:.1f}s; sweep = {len(cells)} launches, "
        f"{sweep_bytes / 1e6:.1f} MB algorithmic, {sweep_flops / 1e9:.2f} GFLOP")

    # --------------------------------------------------------------- the timed step
    constructor, keep = IL.capture_serialized([spmm32(s, n) for s, n in cells])
    constructor.instantiate_graph_exec()
    for _ in range(args.warmup):
        constructor.execute_graph()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        constructor.execute_graph()
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = start.elapsed_time(end) / args.steps
    constructor.destroy_graph_exec()
    del keep
    value = sweep_bytes / 1e9 / (ms_per_step * 1e-3)
    log(f"[bench] {ms_per_step * 1e3:.1f} us per sweep (host wall {wall_ms / args.steps * 1e3:.1f} us) -> {value:.1f} GB/s")

    # ------------------------------------------- per-cell launch durations (HIP events)
    def time_cell(fn, repeats=CELL_REPEATS, samples=5):
        """Average duration of one launch: `repeats` launches in one graph on the current
        stream, events around the graph launch, median of `samples`."""
        ms = IL.time_execs([fn] * repeats, repeats=samples, warmup=1)
        return ms / repeats * 1e3  # us

    def variant_of(csr, n, sv):
        """(VEC, LPG, WPR) of the row kernel for an aligned operand (spmm_pick_shape / pick_wpr)."""
        mean = csr.nnz / csr.m
        wpr = 4 if mean >= 24 else 1
        kmax = 16 // sv
        vec, lpg = kmax, 64
        while vec > 1 and n % vec:
            vec //= 2
        if vec == kmax:
            while lpg > 8 and (lpg // 2) * vec >= n:
                lpg //= 2
        else:
            while vec > 1 and 64 * vec // 2 >= n:
                vec //= 2
        return vec, lpg, wpr

    table = []
    for s, n in cells:
        us = time_cell(spmm32(s, n))
        by, fl = cell_bytes(s, n), W.spmm_flops(mats[s].nnz, n)
        vec, lpg, wpr = variant_of(mats[s], n, 4)
        kernel = f"spmm_kernel<float, int, {vec}, {lpg}, {wpr}>"
        c = mats[s]
        # the dispatcher's rule for the fp32 matrix-core kernel (spmm.hip, mfma_f32_variant)
        if c.nnz / (c.m * c.k) >= 0.27 and n % 4 == 0 and -(-c.m // 32) * -(-n // 128) >= 200 and n / (-(-n // 128) * 128) >= 0.75:
            kernel = "spmm_mfma_f32_kernel<32, 4, 1, 16, true>"
        table.append({"sparsity": s, "n": n, "nnz": mats[s].nnz, "us": round(us, 2), "GBps": round(by / us / 1e3, 1),
                      "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4), "GFLOPs": round(fl / us / 1e3, 1),
                      "valu_frac": round(fl / us / 1e6 / VALU_PEAK_TFLOPS_FP32, 4),
                      "kernel": kernel, "bytes": by})
        log(f"[bench] fp32 s={s} n={n}: {us:.2f} us  {by / us / 1e3:.0f} GB/s  {fl / us / 1e3:.0f} GFLOP/s")

    by_kernel = {}
    for row in table:
        by_kernel.setdefault(row["kernel"], []).append(row)
    dom_name, dom_rows = max(by_kernel.items(), key=lambda kv: sum(r["us"] for r in kv[1]))
    dom_bytes = statistics.mean(r["bytes"] for r in dom_rows)
    dom_us = statistics.mean(r["us"] for r in dom_rows)
    roofline = {"bound": "hbm", "achieved": round(dom_bytes / dom_us / 1e3, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(dom_bytes / dom_us / 1e3 / HBM_PEAK_GBPS, 4),
                "traffic": (round(statistics.mean(MEASURED_TRAFFIC_MB[(r["sparsity"], r["n"])] for r in dom_rows) * 1e6)
                            if dom_name.startswith("spmm_kernel<float") and all((r["sparsity"], r["n"]) in MEASURED_TRAFFIC_MB for r in dom_rows)
                            else None),
                "kernel": dom_name, "avg_launch_us": round(dom_us, 2),
                "algorithmic_bytes_per_launch": int(dom_bytes),
                "cells": [[r["sparsity"], r["n"]] for r in dom_rows],
                "gather_bytes_per_launch": int(statistics.mean(r["nnz"] * r["n"] * 4 for r in dom_rows)),
                "gather_TBps": round(statistics.mean(r["nnz"] * r["n"] * 4 for r in dom_rows) / dom_us / 1e6, 2),
                "note": "every nonzero gathers n*4 bytes of the dense operand from L2 (gather_bytes_per_launch); the "
                        "kernel is bound by that L2->CU bandwidth (gather_TBps), not by HBM, so frac stays small; "
                        "traffic = HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE"}

    result = {
        "metric": "SpMM/SDDMM GB/s and % HBM peak; co-run makespan vs serialized (%) on 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config 2: fp32 CSR SpMM sweep, A 4096x4096 at {70,80,90,95,98}% sparsity (geometric "
                               "row lengths), B 4096x{64,128,256}; one step = the 15 launches in one hipGraph",
                   "value_is": "algorithmic bytes of the sweep / time per sweep",
                   "pct_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2), "cache": "warm (operands stay in L2 / MALL between steps)"},
        "roofline": roofline,
    }
    extras = {"cells_fp32": [{k: v for k, v in r.items() if k != "bytes"} for r in table],
              "sweep_GFLOPs": round(sweep_flops / (ms_per_step * 1e-3) / 1e9, 1)}

    # ------------------------------------------------------------------ CPU baseline
    if not args.no_cpu:
        import oracle  # test infrastructure, used here only as the measured CPU port
        oracle.build()
        t0 = time.perf_counter()
        passes = 0
        while passes < 3 or time.perf_counter() - t0 < 12.0:   # about 12 s of CPU work
            for s, n in cells:
                c = mats[s]
                oracle.spmm_f32(dens[n], c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
            passes += 1
        cpu_s = (time.perf_counter() - t0) / passes
        result["cpu_baseline"] = {"value": round(sweep_bytes / 1e9 / cpu_s, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                                  "sample": f"{passes} full passes over the same 15 fp32 cells (single-threaded C port "
                                            f"of the oracle, gcc -O3), {cpu_s:.2f} s per pass",
                                  "host_cpu_count": os.cpu_count()}
        log(f"[bench] CPU port: {cpu_s:.2f} s per sweep ({passes} passes) -> {sweep_bytes / 1e9 / cpu_s:.2f} GB/s on 1 core")
        # the library baselines the task names: torch.sparse CSR and scipy CSR on the host cores
        try:
            tcpu = {}
            sample = [(s, 128) for s in W.C2_SPARSITIES]
            nthreads = torch.get_num_threads()
            t0 = time.perf_counter()
            for s, n in sample:
                c = mats[s]
                a_t = torch.sparse_csr_tensor(torch.from_numpy(c.row_offsets), torch.from_numpy(c.column_indices),
                                              torch.from_numpy(c.values), size=(c.m, c.k))
                _ = a_t @ torch.from_numpy(dens[n][0])
            tcpu["torch_sparse_csr_s"] = round(time.perf_counter() - t0, 3)
            tcpu["torch_threads"] = nthreads
            import scipy.sparse as sp
            t0 = time.perf_counter()
            for s, n in sample:
                c = mats[s]
                _ = sp.csr_matrix((c.values, c.column_indices, c.row_offsets), shape=(c.m, c.k)) @ dens[n][0]
            tcpu["scipy_csr_s"] = round(time.perf_counter() - t0, 3)
            sample_bytes = sum(cell_bytes(s, n) for s, n in sample)
            tcpu["sample"] = "the five n=128 cells"
            tcpu["torch_sparse_csr_GBps"] = round(sample_bytes / 1e9 / tcpu["torch_sparse_csr_s"], 3)
            tcpu["scipy_csr_GBps"] = round(sample_bytes / 1e9 / tcpu["scipy_csr_s"], 3)
            gpu_sample_us = sum(r["us"] for r in table if r["n"] == 128)
            tcpu["gpu_same_sample_GBps"] = round(sample_bytes / gpu_sample_us / 1e3, 1)
            extras["cpu_libraries"] = tcpu
        except Exception as e:  # a library baseline must not take the bench down
            extras["cpu_libraries"] = {"error": repr(e)}

    # ------------------------------------------------------------------------ extras
    if not args.no_extras:
        try:
            extras.update(run_extras(torch, ops, dev, W, IL, mats, dens, csr_dev, time_cell, variant_of, log))
        except Exception as e:
            import traceback
            traceback.print_exc(file=sys.stderr)
            extras["error"] = repr(e)
    result["extras"] = extras
    print(json.dumps(result), flush=True)


def run_extras(torch, ops, dev, W, IL, mats, dens, csr_dev, time_cell, variant_of, log):
    out = {}
    # ---- fp16 sweep (int16 column indices, the reference's half layout)
    rows = []
    for s in W.C2_SPARSITIES:
        c = mats[s]
        ri, v, ro, ci = csr_dev(c, torch.float16, torch.int16)
        for n in W.C2_NS:
            b = torch.from_numpy(dens[n]).to(dev).half()
            us = time_cell(lambda: ops.spmm_sputnik_reuse_weight_half(b, ri, v, ro, ci, c.m))
            by = W.spmm_bytes(c.m, c.k, n, c.nnz, 1, 2, 2)
            fl = W.spmm_flops(c.nnz, n)
            rows.append({"sparsity": s, "n": n, "us": round(us, 2), "GBps": round(by / us / 1e3, 1),
                         "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4), "GFLOPs": round(fl / us / 1e3, 1)})
    out["cells_fp16_i16"] = rows
    log("[bench] fp16 sweep done")

    # ---- SDDMM: config 1 (fp32, batch-summed) and config 3 (fp16, 16 heads, per-head output)
    a1, _, lhs1, rhs1 = W.config1()
    ri, _, ro, ci = csr_dev(a1)
    l1, r1 = torch.from_numpy(lhs1).to(dev), torch.from_numpy(rhs1).to(dev)
    us = time_cell(lambda: ops.sddmm_sputnik_atomic_upd_weight(l1, r1, ri, ro, ci))
    by = W.sddmm_bytes(a1.m, 64, a1.k, a1.nnz, 1, 4, True)
    out["sddmm_c1_fp32"] = {"us": round(us, 2), "GBps": round(by / us / 1e3, 1), "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4),
                            "GFLOPs": round(W.sddmm_flops(a1.nnz, 64) / us / 1e3, 1)}
    pat, q, k, v = W.config3()
    ri3, _, ro3, ci3 = csr_dev(pat)
    qt, kt, vt = (torch.from_numpy(x).to(dev).half() for x in (q, k, v))
    us = time_cell(lambda: ops.sddmm_sputnik_half(qt, kt, ri3, ro3, ci3), repeats=10)
    by = W.sddmm_bytes(pat.m, 64, pat.k, pat.nnz, 16, 2, False)
    out["sddmm_c3_fp16_16heads"] = {"nnz": pat.nnz, "sparsity": round(pat.sparsity, 4), "us": round(us, 2),
                                    "GBps": round(by / us / 1e3, 1), "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4),
                                    "GFLOPs": round(W.sddmm_flops(pat.nnz, 64, 16) / us / 1e3, 1)}
    scores = ops.sddmm_sputnik_half(qt, kt, ri3, ro3, ci3)
    us = time_cell(lambda: ops.spmm_sputnik_batched_values(vt, ri3, scores, ro3, ci3, pat.m), repeats=10)
    by = W.spmm_bytes(pat.m, pat.k, 64, pat.nnz, 16, 2, 4, True)
    out["spmm_c3_fp16_16heads"] = {"us": round(us, 2), "GBps": round(by / us / 1e3, 1),
                                   "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4),
                                   "GFLOPs": round(W.spmm_flops(pat.nnz, 64, 16) / us / 1e3, 1)}
    from intrasm_engine_amd.pytorch.sparse_attention import sparse_attention
    us_block = time_cell(lambda: sparse_attention(qt, kt, vt, ri3, ro3, ci3), repeats=10)
    us_softmax = time_cell(lambda: ops.csr_softmax_(scores, ri3, ro3, 0.125), repeats=10)
    out["attention_block_c3_fp16_16heads"] = {
        "us": round(us_block, 2), "softmax_us": round(us_softmax, 2),
        "what": "SDDMM -> softmax over CSR rows -> SpMM, three launches; 16 heads x 4096 tokens x 64",
        "GFLOPs": round((W.sddmm_flops(pat.nnz, 64, 16) + W.spmm_flops(pat.nnz, 64, 16)) / us_block / 1e3, 1)}
    # the weight gradient of a sparse linear layer is an SDDMM with k = tokens: config 4's weight (11008 x 4096 at
    # 90 %) against 2048 tokens, fp16; the operator computes the dense product on the matrix cores and samples it
    from intrasm_engine_amd.pytorch import ops as pyops_
    w4g = W.config4()[0]
    riw_, _, row_, ciw_ = csr_dev(w4g)
    gy = (torch.randn(1, w4g.m, 2048, device=dev, generator=torch.Generator(dev).manual_seed(2)) * 0.1).half()
    xx = torch.randn(1, w4g.k, 2048, device=dev, generator=torch.Generator(dev).manual_seed(3)).half()
    kw_ = dict(sum_over_batch=False, dtypes=(torch.float16,))
    us_g = time_cell(lambda: pyops_._sddmm(gy, xx, riw_, row_, ciw_, force_variant=1, **kw_), repeats=3, samples=3)
    us_d = time_cell(lambda: ops.sddmm_sputnik_half(gy, xx, riw_, row_, ciw_), repeats=5)
    out["sddmm_weight_gradient_c4_fp16"] = {
        "what": "SDDMM on config 4's mask (11008 x 4096, 90 % sparse) with k = 2048 tokens",
        "gather_kernel_us": round(us_g, 1), "operator_us": round(us_d, 1),
        "operator_path": "dense product by the GEMM into a workspace, then sampling",
        "operator_dense_equivalent_TFLOPs": round(2.0 * w4g.m * w4g.k * 2048 / us_d / 1e6, 1)}
    # the same layer as an autograd function: forward SpMM, backward SpMM with the transposed weight (gradient of
    # the activation) + that SDDMM (gradient of the values); one training step of a sparse linear layer, eager
    from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.sputnik import spmm as spmm_fn
    from intrasm_engine_amd.pytorch import utils as U_
    vals_ = torch.from_numpy(w4g.values).to(dev).half().requires_grad_(True)
    info_ = U_.transpose_info(w4g.m, w4g.k, row_, ciw_)
    x2 = xx[0].detach().clone().requires_grad_(True)          # (k, tokens)
    g2 = gy[0].detach().clone()                               # (m, tokens)

    def train_step():
        vals_.grad = None
        x2.grad = None
        spmm_fn(x2, riw_, vals_, row_, ciw_, w4g.m, info_).backward(g2)

    us_step = time_cell(train_step, repeats=3, samples=3)
    out["sparse_linear_training_step_c4_fp16"] = {
        "what": "MySpMM forward + backward on config 4's weight, 2048 tokens, fp16, int32 indices, eager",
        "us": round(us_step, 1), "nonzero_GFLOP": round(3 * 2.0 * w4g.nnz * 2048 / 1e9, 2),
        "dense_equivalent_TFLOPs": round(3 * 2.0 * w4g.m * w4g.k * 2048 / us_step / 1e6, 1)}
    del gy, xx, riw_, row_, ciw_, w4g, vals_, info_, x2, g2
    log("[bench] SDDMM done")

    # ---- where the HBM roof binds: two points of the reference's xformers-style SpMM sweep (fp32, per-batch values;
    # a sparse M x K pattern with a small K times a dense K x M operand: the M x M output per batch entry is the traffic)
    from intrasm_engine_amd.benchmarks import benchmark_spmm as xf
    pts = {}
    for label, cfg in (("swin_t_stage1_B96_M3136_K32_s0.9844", ((96, 3136, 32), 0.9844)),
                       ("basic_B8_M4096_K32_s0.90", ((8, 4096, 32), 0.90))):
        with contextlib.redirect_stdout(sys.stderr):     # (the sweep prints its own line; stdout carries only the JSON line)
            r = xf.bench_spmm([cfg], repeats=4, check=False)[0]
        pts[label] = {"us": round(r["us"], 1), "GBps": round(r["GBps"], 1), "hbm_frac": round(r["GBps"] / HBM_PEAK_GBPS, 4),
                      "output_GB": round(cfg[0][0] * cfg[0][1] * cfg[0][1] * 4 / 1e9, 2)}
    out["output_bound_sweep_points_fp32"] = pts

    # ---- config 4: fp16 SpMM 11008x4096 @90% x 4096x2048  ||  bf16 GEMM 4096x4096x2048
    w, x, ga, gb = W.config4()
    riw, vw, row, ciw = csr_dev(w, torch.float16, torch.int16)
    xt = torch.from_numpy(x).to(dev).half()
    gat, gbt = torch.from_numpy(ga).to(dev).bfloat16(), torch.from_numpy(gb).to(dev).bfloat16()
    reps = 4
    spmm_execs = [lambda: ops.spmm_sputnik_reuse_weight_half(xt, riw, vw, row, ciw, w.m)] * reps
    gemm_execs = [lambda: ops.gemm_mfma(gat, gbt, False)] * reps
    fused_execs = [lambda: ops.fused_spmm_gemm(xt, riw, vw, row, ciw, w.m, gat, gbt, False, 0)] * reps
    fused_g_execs = [lambda: ops.fused_spmm_gemm(xt, riw, vw, row, ciw, w.m, gat, gbt, False, 64)] * reps
    t_spmm = IL.run_non_interleaving(spmm_execs) / reps
    t_gemm = IL.run_non_interleaving(gemm_execs) / reps
    t_serial = IL.run_non_interleaving(spmm_execs, gemm_execs) / reps
    t_graph = IL.run_interleaving(spmm_execs, gemm_execs) / reps
    t_fused = IL.run_non_interleaving(fused_execs) / reps
    t_fused_g = IL.run_non_interleaving(fused_g_execs) / reps
    # the same pair with the SpMM forced onto the gather (row) kernel: vector ALU + L2 beside the matrix cores,
    # the resource split the reference's co-run experiment is about
    from intrasm_engine_amd.pytorch import ops as pyops
    gather_execs = [lambda: pyops._spmm(xt, riw, vw, row, ciw, w.m, per_batch_values=False, accumulate=False,
                                        dtypes=(torch.float16,), allow_i16=True, force_variant=1)] * reps
    t_gather = IL.run_non_interleaving(gather_execs) / reps
    t_graph_gather = IL.run_interleaving(gather_execs, gemm_execs) / reps
    # the library's choice above has a workspace to use (the operator allocates one) and takes the dense-form
    # path; without one the 8-wave matrix-core SpMM kernel runs, the kernel the fused launch shares its SpMM role with
    mc_execs = [lambda: pyops._spmm(xt, riw, vw, row, ciw, w.m, per_batch_values=False, accumulate=False,
                                    dtypes=(torch.float16,), allow_i16=True, no_workspace=True)] * reps
    t_mc = IL.run_non_interleaving(mc_execs) / reps
    t_graph_mc = IL.run_interleaving(mc_execs, gemm_execs) / reps
    fl_s, fl_g = W.spmm_flops(w.nnz, 2048), W.gemm_flops(4096, 2048, 4096)
    by_s = W.spmm_bytes(w.m, w.k, 2048, w.nnz, 1, 2, 2)
    out["config4"] = {
        "spmm_ms": round(t_spmm, 4), "spmm_GBps": round(by_s / t_spmm / 1e6, 1), "spmm_GFLOPs": round(fl_s / t_spmm / 1e6, 1),
        "spmm_hbm_frac": round(by_s / t_spmm / 1e6 / HBM_PEAK_GBPS, 4),
        "spmm_valu_frac": round(fl_s / t_spmm / 1e9 / VALU_PEAK_TFLOPS_FP32, 4),
        "gemm_ms": round(t_gemm, 4), "gemm_TFLOPs": round(IL.gemm_tflops(4096, 2048, 4096, t_gemm), 1),
        "gemm_mfma_frac": round(IL.gemm_tflops(4096, 2048, 4096, t_gemm) / MFMA_PEAK_TFLOPS_16BIT, 4),
        "serialized_sum_ms": round(t_spmm + t_gemm, 4), "serialized_one_stream_ms": round(t_serial, 4),
        "two_branch_graph_ms": round(t_graph, 4), "fused_launch_ms": round(t_fused, 4),
        "fused_launch_gemm_in_groups_of_64_ms": round(t_fused_g, 4),
        "graph_makespan_pct_of_serialized": round(100 * t_graph / (t_spmm + t_gemm), 1),
        "fused_makespan_pct_of_serialized": round(100 * t_fused / (t_spmm + t_gemm), 1),
        "spmm_matrix_core_kernel_ms": round(t_mc, 4), "two_branch_graph_matrix_core_kernel_ms": round(t_graph_mc, 4),
        "matrix_core_kernel_graph_makespan_pct_of_serialized": round(100 * t_graph_mc / (t_mc + t_gemm), 1),
        "fused_makespan_pct_of_serialized_matrix_core_kernel": round(100 * t_fused / (t_mc + t_gemm), 1),
        "spmm_row_kernel_ms": round(t_gather, 4), "two_branch_graph_row_kernel_ms": round(t_graph_gather, 4),
        "row_kernel_graph_makespan_pct_of_serialized": round(100 * t_graph_gather / (t_gather + t_gemm), 1),
        "spmm_dense_equivalent_TFLOPs": round(2.0 * w.m * w.k * 2048 / t_spmm / 1e9, 1),
        "repeats_per_graph": reps,
    }
    log(f"[bench] config 4: spmm {t_spmm:.3f} ms, gemm {t_gemm:.3f} ms, graph {t_graph:.3f} ms, fused {t_fused:.3f} ms")
    del w, x, ga, gb, riw, vw, row, ciw, xt, gat, gbt, spmm_execs, gemm_execs, fused_execs, fused_g_execs, gather_execs, mc_execs

    # ---- the dense GEMM alone on larger shapes (bf16, B as (K, N)): how far the matrix cores are used
    rows_gemm = []
    for (gm, gn, gk) in ((8192, 8192, 8192), (4096, 8192, 4096), (11008, 8192, 4096)):
        ga2 = torch.randn(gm, gk, device=dev).bfloat16()
        gb2 = torch.randn(gk, gn, device=dev).bfloat16()
        t = IL.run_non_interleaving([lambda: ops.gemm_mfma(ga2, gb2, False)] * reps) / reps
        tf = IL.gemm_tflops(gm, gn, gk, t)
        rows_gemm.append({"m": gm, "n": gn, "k": gk, "ms": round(t, 4), "TFLOPs": round(tf, 1),
                          "mfma_frac": round(tf / MFMA_PEAK_TFLOPS_16BIT, 4)})
        del ga2, gb2
    out["gemm_bf16"] = rows_gemm

    # ---- config 5: LLaMA-7B-shaped sparse decoder layer, 16 sequences x 512 tokens, three variants
    from intrasm_engine_amd.decoder_layer import SparseDecoderLayer
    hidden, heads, mlp, seqs, L = 4096, 32, 11008, 16, 512
    weights = W.config5_weights()
    layer = SparseDecoderLayer(weights, hidden, heads, mlp, dev)
    x5 = torch.from_numpy(W.config5_activation(hidden=hidden, tokens=seqs * L)[0]).to(dev).half()
    half = seqs * L // 2
    xa, xb = x5[:, :half].contiguous(), x5[:, half:].contiguous()

    def time_capture(make, samples=3):
        constructor, keep = make()
        ms = statistics.median(IL._time_graph(constructor, samples, 1))
        del keep
        return ms

    t_ser = time_capture(lambda: layer.capture_serialized(x5, seqs))
    t_ser_halves = time_capture(lambda: IL.capture_serialized([lambda: (layer.forward(xa, seqs // 2), layer.forward(xb, seqs // 2))]))
    t_ms = time_capture(lambda: layer.capture_multistream(xa, xb, seqs // 2))
    t_fu = time_capture(lambda: layer.capture_fused(xa, xb, seqs // 2, 0))
    spmm_flops5 = sum(2 * weights[n_].nnz * seqs * L for n_ in weights)
    attn_flops5 = 2 * 2 * seqs * heads * L * L * (hidden // heads)
    out["config5"] = {
        "shape": "hidden 4096, 32 heads, MLP 11008, 16 x 512 tokens, fp16; q/k/v/o 2:4, gate/up/down 80% unstructured",
        "elementwise_ops_included": "softmax(QK^T/sqrt(d)), SiLU(gate)*up, two residual adds (PyTorch kernels); no RoPE / norm / mask",
        "serialized_ms": round(t_ser, 3), "serialized_two_halves_ms": round(t_ser_halves, 3),
        "multistream_graph_ms": round(t_ms, 3), "fused_ms": round(t_fu, 3),
        "multistream_pct_of_serialized": round(100 * t_ms / t_ser, 1), "fused_pct_of_serialized": round(100 * t_fu / t_ser, 1),
        "spmm_GFLOP": round(spmm_flops5 / 1e9, 1), "attention_GFLOP": round(attn_flops5 / 1e9, 1),
        "layer_TFLOPs_serialized": round((spmm_flops5 + attn_flops5) / t_ser / 1e9, 1),
    }
    log(f"[bench] config 5: serialized {t_ser:.2f} ms, two-stream graph {t_ms:.2f} ms, fused {t_fu:.2f} ms")
    del layer

    # ---- the SpMM kernel families side by side on three projections of that layer (n = 8192 tokens, fp16,
    # int16 indices) and on the config-4 operand: row kernel (gathers from L2), LDS-staged gather, matrix cores
    from intrasm_engine_amd.pytorch import ops as pyops
    fam = {}
    w4 = W.config4()[0]
    for name, c, n_ in (("q_2to4_4096x4096_n8192", weights["q"], seqs * L), ("gate_80pct_11008x4096_n8192", weights["gate"], seqs * L),
                        ("down_80pct_4096x11008_n8192", weights["down"], seqs * L), ("config4_90pct_11008x4096_n2048", w4, 2048)):
        ri, v, ro, ci = csr_dev(c, torch.float16, torch.int16)
        xin = torch.randn(1, c.k, n_, device=dev, generator=torch.Generator(dev).manual_seed(1)).half()
        kw = dict(per_batch_values=False, accumulate=False, dtypes=(torch.float16,), allow_i16=True)
        row = {}
        for label, force in (("row_kernel_ms", dict(force_variant=1)), ("lds_staged_ms", dict(force_variant=2)),
                             ("matrix_core_4waves_ms", dict(force_variant=3)), ("matrix_core_8waves_ms", dict(force_variant=4)),
                             ("no_workspace_choice_ms", dict(no_workspace=True)), ("dense_form_then_gemm_ms", dict(force_variant=7)),
                             ("library_choice_ms", {})):
            row[label] = round(IL.time_execs([lambda: pyops._spmm(xin, ri, v, ro, ci, c.m, **force, **kw)] * 2, repeats=3) / 2, 4)
        dense_flops = 2.0 * c.m * c.k * n_
        row["density"] = round(c.nnz / (c.m * c.k), 4)
        row["library_choice_dense_equivalent_TFLOPs"] = round(dense_flops / row["library_choice_ms"] / 1e9, 1)
        row["library_choice_nonzero_TFLOPs"] = round(2.0 * c.nnz * n_ / row["library_choice_ms"] / 1e9, 1)
        row["library_choice_mfma_frac_dense_equivalent"] = round(dense_flops / row["library_choice_ms"] / 1e9 / MFMA_PEAK_TFLOPS_16BIT, 4)
        fam[name] = row
        del ri, v, ro, ci, xin
    out["spmm_kernel_families_fp16"] = fam
    log("[bench] kernel families: " + ", ".join(f"{k_}: row {r_['row_kernel_ms']} / lds {r_['lds_staged_ms']} / mfma {r_['matrix_core_8waves_ms']} ms"
                                               for k_, r_ in fam.items()))
    return out


if __name__ == "__main__":
    main()
