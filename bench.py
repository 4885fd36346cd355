#!/usr/bin/env python3
"""Benchmark of the sparse-plus-dense GEMM path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

A *step* is one pass of the hot path over the configuration the metric is quoted on:
the fp32 CSR SpMM sweep of config 2 (4096x4096 sparse A at 70/80/90/95/98 % sparsity with
geometric row lengths, times a dense 4096 x {64,128,256} B) = 15 SpMM launches, captured
once into a hipGraph through the graph builder and replayed.  The launches are independent
of each other and the graph holds them on two parallel branches: each launch is told that
it has a neighbour, the cells that then run on the fp32 matrix cores form one branch and the
gather-bound cells the other.  The same launches on one branch, and on two branches with
every kernel as the library chooses it alone, are timed beside the step and reported in
``config``.  All operands are resident in HBM before the timed region; CSR construction is
set-up work and is not timed.

One JSON line is printed.  ``value`` = algorithmic GB of one sweep / seconds per sweep.
``roofline`` describes the SpMM kernel instantiation that takes the most time in the
sweep (its name is read from the library, its HBM traffic from the committed counter
summary taken on that same kernel); ``cpu_baseline`` is torch.sparse CSR on the host cores
over the same 15 cells (median of 5 per cell);
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
MFMA_PEAK_TFLOPS_FP32 = 157.3    # dense fp32 MFMA
CELL_REPEATS = 20                # launches of one cell inside its timing graph
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "spmm_fp32_config2_hbm_traffic_pmc.txt")
COLD_SCRATCH_BYTES = 512 << 20   # written between cold-cache samples (> the 256 MB last-level cache)


def read_traffic_profile():
    """HBM-side bytes per launch (L2 misses + write-backs) of every fp32 cell, from the committed summary of two
    `rocprofv3 --pmc` runs (FETCH_SIZE, WRITE_SIZE) of `bench.py --pmc-probe`, each scaled by the counter's reading for
    a plain 256 MiB copy.  Counters cannot be read inside a timing run, so the figure is tied to the kernel it was
    measured on: each line carries the kernel name the library reported for that cell, and a cell whose kernel has
    changed since is not used.  Returns ({(sparsity, n): (kernel, bytes)}, commit)."""
    cells, commit = {}, None
    try:
        for line in open(TRAFFIC_PROFILE):
            if line.startswith("measured_at_commit"):
                commit = line.split()[1]
            if line.startswith("cell "):
                f = {k.strip(): v.strip() for k, v in (kv.split("=", 1) for kv in line.split("|")[1:])}
                cells[(float(f["sparsity"]), int(f["n"]))] = (f["kernel"], float(f["traffic_bytes"]))
    except (OSError, KeyError, ValueError):
        pass
    return cells, commit


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def fused_timeline(dev, csr_dev, log):
    """Per-workgroup timeline of config 4's fused launch (matrix-core kernel) for the three orders of its two kinds of
    workgroup: which CU ran what, when each CU went idle, and how much CU time the tail leaves unused."""
    import collections
    import torch
    from intrasm_engine_amd import _lib, workloads as W
    lib = _lib.load()
    ops = torch.ops.iex_ops
    w, x, ga, gb = W.config4()
    riw, vw, row, ciw = csr_dev(w, torch.float16, torch.int16)
    xt = torch.from_numpy(x).to(dev).half()
    gat, gbt = torch.from_numpy(ga).to(dev).bfloat16(), torch.from_numpy(gb).to(dev).bfloat16()
    buf = torch.zeros(4 * 4096, dtype=torch.int64, device=dev)
    for label, order in (("GEMM tiles first (interleave 0)", 0), ("in groups of 64", 64), ("SpMM tiles first (interleave -1)", -1)):
        for _ in range(3):
            ops.fused_spmm_gemm(xt, riw, vw, row, ciw, w.m, gat, gbt, False, order)
        torch.cuda.synchronize()
        _lib.check(lib.iex_fused_timeline(buf.data_ptr()), "fused_timeline")
        try:
            buf.zero_()
            ops.fused_spmm_gemm(xt, riw, vw, row, ciw, w.m, gat, gbt, False, order)
            torch.cuda.synchronize()
        finally:
            lib.iex_fused_timeline(None)
        trail = _lib.last_kernels()
        t = buf.cpu().numpy().reshape(-1, 4)
        t = t[t[:, 1] != 0]
        t0 = t[:, 0].min()
        began, ended = (t[:, 0] - t0) / 100.0, (t[:, 1] - t0) / 100.0       # microseconds (100 MHz clock)
        is_gemm = (t[:, 3] >> 32) != 0
        place = ((t[:, 2] >> 16) << 8) | ((t[:, 2] >> 8) & 0xff)             # (XCD, shader engine / array / CU)
        per_cu = collections.defaultdict(list)
        for i in np.argsort(began):
            per_cu[int(place[i])].append((float(began[i]), float(ended[i]), bool(is_gemm[i])))
        makespan = float(ended.max())
        busy = float((ended - began).sum())
        shapes = collections.Counter("".join("G" if g else "S" for _, _, g in v) for v in per_cu.values())
        idle_at = np.array(sorted(v[-1][1] for v in per_cu.values()))
        overlap = sum(1 for v in per_cu.values() for a, b in zip(v, v[1:]) if b[0] < a[1] - 0.5)
        log(f"== {label}: {trail}")
        log(f"   {len(t)} workgroups on {len(per_cu)} CUs; SpMM tile {np.median((ended - began)[~is_gemm]):.1f} us (median; "
            f"{(ended - began)[~is_gemm].min():.1f}-{(ended - began)[~is_gemm].max():.1f}), GEMM tile {np.median((ended - began)[is_gemm]):.1f} us "
            f"({(ended - began)[is_gemm].min():.1f}-{(ended - began)[is_gemm].max():.1f}); two workgroups on one CU at a time: {overlap} cases")
        log(f"   makespan {makespan:.1f} us; CU time used {busy:.0f} of {makespan * len(per_cu):.0f} CU-us = {100 * busy / (makespan * len(per_cu)):.1f} %; "
            f"bound by the work {busy / len(per_cu):.1f} us")
        log("   what a CU ran, in order (S = SpMM tile, G = GEMM tile): " + ", ".join(f"{k} x {v}" for k, v in sorted(shapes.items(), key=lambda kv: -kv[1])))
        log("   CUs idle from (us): " + ", ".join(f"{q} %: {idle_at[min(len(idle_at) - 1, int(q / 100 * len(idle_at)))]:.0f}" for q in (0, 10, 25, 50, 75, 90)) +
            f", last {idle_at[-1]:.0f}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-extras", action="store_true", help="skip fp16 / SDDMM / GEMM / co-run sections")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="for `rocprofv3 --pmc ...`: 3 plain copies of 256 MiB (iex_copy_bytes), then 3 launches of each "
                         "fp32 cell, and exit")
    ap.add_argument("--gemm-probe", action="store_true",
                    help="bf16 GEMM (B as (K, N)): every tile shape on a few products, one line per product on stdout; with "
                         "--gemm-probe-tile T only that shape on config 4's product, 3 launches (for rocprofv3 --pmc)")
    ap.add_argument("--gemm-probe-tile", type=int, default=-1)
    ap.add_argument("--spmm-probe", action="store_true",
                    help="config 3's SpMM against V (fp16, 16 heads), 3 launches of what the operator picks and 3 of the row kernel "
                         "(for rocprofv3; no JSON line)")
    ap.add_argument("--sddmm-probe", action="store_true",
                    help="config 3's SDDMM (fp16, 16 heads), 3 launches of what the operator picks and 3 of the gather kernel "
                         "(for rocprofv3 --kernel-trace / --pmc)")
    ap.add_argument("--softmax-probe", action="store_true",
                    help="config 3's softmax over CSR rows (fp16, 16 heads): 5 launches with a positive scale (four rows per "
                         "wavefront) and 5 with a negative one (the kernel with a wavefront per row), for rocprofv3")
    ap.add_argument("--fused-timeline", action="store_true",
                    help="config 4's fused launch in its three workgroup orders with the per-workgroup timeline switched on "
                         "(iex_fused_timeline): prints, per order, what each CU ran and when it went idle")
    ap.add_argument("--overlap-probe", action="store_true",
                    help="for `rocprofv3 --kernel-trace`: 3 replays of config 4's two-branch graph, and exit")
    ap.add_argument("--summarize-pmc", nargs=3, metavar=("FETCH_CSV", "WRITE_CSV", "CELLS_JSON"),
                    help="turn the counter_collection.csv of the FETCH_SIZE and of the WRITE_SIZE run of --pmc-probe and its "
                         "pmc_probe_cells.json into profiles/spmm_fp32_config2_hbm_traffic_pmc.txt (no GPU needed)")
    args = ap.parse_args()
    if args.summarize_pmc:
        summarize_pmc(*args.summarize_pmc)
        return
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
    from intrasm_engine_amd.pytorch import ops as pyops
    from intrasm_engine_amd.pytorch.cpp_extensions.cuda_graph_constructor import TorchCUDAGraphConstructor

    ops = torch.ops.iex_ops
    dev = torch.device("cuda:0")
    t_setup = time.time()

    # ------------------------------------------------------------- inputs (config 2)
    mats = {s: W.config2_matrix(s) for s in W.C2_SPARSITIES}
    dens = {n: W.config2_dense(n) for n in W.C2_NS}

    def csr_dev(csr, vdtype=torch.float32, idtype=torch.int32, tables=False):
        t = (torch.from_numpy(csr.row_indices).to(dev), torch.from_numpy(csr.values).to(dev).to(vdtype),
             torch.from_numpy(csr.row_offsets).to(dev), torch.from_numpy(csr.column_indices).to(dev).to(idtype))
        # looked at once, outside any capture (the timing loops capture their launches): canonical CSR gets every kernel
        # family; an attention mask with structure also gets the tables of its kernels made here (tables=True), a weight not
        pyops.prepare_pattern(t[2], t[3], csr.k, tables=tables)
        return t

    mats32 = {s: csr_dev(m) for s, m in mats.items()}
    dens32 = {n: torch.from_numpy(b).to(dev) for n, b in dens.items()}
    cells = [(s, n) for s in W.C2_SPARSITIES for n in W.C2_NS]

    def spmm32_alone(s, n):
        """The launch of a cell as the library chooses it when it knows of no neighbour."""
        ri, v, ro, ci = mats32[s]
        return lambda: ops.spmm_sputnik_reuse_weight(dens32[n], ri, v, ro, ci, mats[s].m)

    def spmm32(s, n):
        """The launch of a cell as it runs in the timed step: told that it shares the chip with a gather-bound launch
        (IEX_SPMM_BESIDE_GATHER_KERNEL; the timed graph has two parallel branches)."""
        alone = spmm32_alone(s, n)

        def call():
            with pyops.kernel_params(spmm={"beside_gather_kernel": True}):
                return alone()
        return call

    def cell_bytes(s, n, sv=4, si=4):
        c = mats[s]
        return W.spmm_bytes(c.m, c.k, n, c.nnz, 1, sv, si)

    from intrasm_engine_amd import _lib

    def kernel_of(fn):
        """Kernel name(s) the library launches for this call: asked of the library after one eager call."""
        fn()
        torch.cuda.synchronize()
        return _lib.last_kernels()

    if args.pmc_probe:
        # for `rocprofv3 --pmc ...`: 3 plain copies of 256 MiB (the calibration of FETCH_SIZE / WRITE_SIZE), then every
        # fp32 cell 3 times in cell order; the kernel names go to stderr and to pmc_probe_cells.json in the output folder
        nbytes = 256 << 20
        src = torch.zeros(nbytes // 4, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            _lib.check(_lib.load().iex_copy_bytes(dst.data_ptr(), src.data_ptr(), nbytes,
                                                  torch.cuda.current_stream().cuda_stream), "copy")
        torch.cuda.synchronize()
        names = []
        for s_, n_ in cells:       # dispatch order = cell order, 3 launches each
            fn = spmm32(s_, n_)
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            names.append({"sparsity": s_, "n": n_, "kernel": _lib.last_kernels(), "algorithmic_bytes": cell_bytes(s_, n_)})
        os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
        json.dump({"copy_bytes": nbytes, "cells": names}, open(os.path.join(ROOT, "gpurun_out", "pmc_probe_cells.json"), "w"))
        log("[bench] pmc probe done: copy of %d bytes x3 (copy_kernel), then every fp32 cell x3" % nbytes)
        return

    if args.gemm_probe:
        from intrasm_engine_amd.pytorch import ops as pyops_g
        if args.gemm_probe_tile >= 0:
            a_ = torch.randn(4096, 4096, device=dev).bfloat16()
            b_ = torch.randn(4096, 2048, device=dev).bfloat16()
            with pyops_g.kernel_params(gemm={"tile": args.gemm_probe_tile} if args.gemm_probe_tile else None):
                for _ in range(3):
                    ops.gemm_mfma(a_, b_, False)
            torch.cuda.synchronize()
            return
        names = {0: "chosen", 5: "128x128", 6: "128x256/4 waves", 10: "128x256/8 waves", 11: "128x256/8 waves, K steps of 64", 7: "256x256",
                 12: "256x256, K split over 2 workgroups"}
        for (gm, gn, gk) in ((4096, 2048, 4096), (4096, 4096, 4096), (11008, 4096, 4096), (4096, 8192, 4096), (8192, 8192, 8192), (2048, 2048, 2048)):
            a_ = torch.randn(gm, gk, device=dev).bfloat16()
            b_ = torch.randn(gk, gn, device=dev).bfloat16()
            cells_ = []
            for tile_ in (0, 0, 5, 6, 10, 11, 7, 12):       # (the first pass warms the clocks up and is dropped)
                with pyops_g.kernel_params(gemm={"tile": tile_} if tile_ else None):
                    f_ = lambda: ops.gemm_mfma(a_, b_, False)
                    f_()
                    ms_ = IL.time_execs([f_] * 10, repeats=3) / 10
                cells_.append(f"{names[tile_]} {IL.gemm_tflops(gm, gn, gk, ms_):.0f}")
            print(f"{gm} x {gn} x {gk} (TFLOP/s): " + " | ".join(cells_[1:]), flush=True)
            del a_, b_
        return

    if args.sddmm_probe:
        from intrasm_engine_amd.pytorch import ops as pyops_s
        pat_, q_, k_, _ = W.config3()
        ri_, _, ro_, ci_ = csr_dev(pat_)
        qt_, kt_ = (torch.from_numpy(x).to(dev).half() for x in (q_, k_))
        for _ in range(3):
            ops.sddmm_sputnik_half(qt_, kt_, ri_, ro_, ci_)
        log("[sddmm-probe] operator:", _lib.last_kernels())
        with pyops_s.kernel_params(sddmm={"force_variant": 1}):
            for _ in range(3):
                ops.sddmm_sputnik_half(qt_, kt_, ri_, ro_, ci_)
        log("[sddmm-probe] gather kernel:", _lib.last_kernels())
        torch.cuda.synchronize()
        return

    if args.softmax_probe:
        pat_, _, _, _ = W.config3()
        ri_, _, ro_, _ = csr_dev(pat_)
        base_ = torch.randn(16, pat_.nnz, device=dev, generator=torch.Generator(dev).manual_seed(5)).half()
        for scale_ in (0.125, -0.125):
            for _ in range(5):
                ops.csr_softmax_(base_.clone(), ri_, ro_, scale_)
        torch.cuda.synchronize()
        return

    if args.spmm_probe:
        from intrasm_engine_amd.pytorch import ops as pyops_s
        pat_, _, _, v_ = W.config3()
        ri_, _, ro_, ci_ = csr_dev(pat_)
        vt_ = torch.from_numpy(v_).to(dev).half()
        probs_ = (torch.rand(16, pat_.nnz, device=dev, generator=torch.Generator(dev).manual_seed(4)) / 280).half()
        for _ in range(3):
            ops.spmm_sputnik_batched_values(vt_, ri_, probs_, ro_, ci_, pat_.m)
        log("[spmm-probe] operator:", _lib.last_kernels())
        with pyops_s.kernel_params(spmm={"force_variant": 1}):
            for _ in range(3):
                ops.spmm_sputnik_batched_values(vt_, ri_, probs_, ro_, ci_, pat_.m)
        log("[spmm-probe] row kernel:", _lib.last_kernels())
        torch.cuda.synchronize()
        return

    if args.fused_timeline:
        fused_timeline(dev, csr_dev, log)
        return

    if args.overlap_probe:
        # for `rocprofv3 --kernel-trace`: config 4's two-branch graph (SpMM kernel || GEMM), 3 replays
        from intrasm_engine_amd.pytorch import ops as pyops
        w, x, ga, gb = W.config4()
        riw, vw, row, ciw = csr_dev(w, torch.float16, torch.int16)
        xt = torch.from_numpy(x).to(dev).half()
        gat, gbt = torch.from_numpy(ga).to(dev).bfloat16(), torch.from_numpy(gb).to(dev).bfloat16()
        kw = dict(per_batch_values=False, accumulate=False, dtypes=(torch.float16,), allow_i16=True)
        for label, extra in (("matrix-core SpMM kernel || GEMM", dict(no_workspace=True)), ("row-kernel SpMM || GEMM", dict(force_variant=1))):
            constructor, keep = IL.capture_interleaved([lambda: pyops._spmm(xt, riw, vw, row, ciw, w.m, **extra, **kw)] * 2,
                                                       [lambda: ops.gemm_mfma(gat, gbt, False)] * 2)
            constructor.instantiate_graph_exec()
            for _ in range(3):
                constructor.execute_graph()
                constructor.synchronize()
            constructor.destroy_graph_exec()
            log(f"[bench] overlap probe: {label}, 3 replays of a graph with 2 + 2 kernels on two branches")
            del keep
        return

    sweep_bytes = sum(cell_bytes(s, n) for s, n in cells)
    sweep_flops = sum(W.spmm_flops(mats[s].nnz, n) for s, n in cells)
    log(f"[bench] set-up {time.time() - t_setup:.1f}s; sweep = {len(cells)} launches, "
        f"{sweep_bytes / 1e6:.1f} MB algorithmic, {sweep_flops / 1e9:.2f} GFLOP")

    # --------------------------------------------------------------- the timed step
    # One step = the 15 launches of the sweep in one hipGraph.  The launches are independent, so the graph holds them on
    # two parallel branches: the gap between two kernels of one branch (2-4 us) and the tails of the short launches are
    # covered by the other branch, and kernels bound by different units overlap.  Three and four branches measured slower
    # than two (710 / 735 against 653-672 us where one branch takes 716).  The same launches on one branch, and on two
    # branches without the neighbour hint, are timed beside it (config.one_branch_sweep_us, config.two_branches_...).
    def time_sweep(lists):
        constructor, keep = IL.capture_serialized(lists[0]) if len(lists) == 1 else IL.capture_interleaved(*lists)
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
        wall = (time.perf_counter() - t0) * 1e3
        ms = start.elapsed_time(end) / args.steps
        constructor.destroy_graph_exec()
        del keep
        return ms, wall

    by_cost = sorted(cells, key=lambda c: -mats[c[0]].nnz * c[1])
    ms_one_branch, _ = time_sweep([[spmm32_alone(s, n) for s, n in cells]])
    # two branches, every launch as the library would choose it alone: neighbours in cost side by side
    plain_branches = [by_cost[0::2], by_cost[1::2]]
    ms_two_plain, _ = time_sweep([[spmm32_alone(s, n) for s, n in b] for b in plain_branches])
    # two branches, and the launches are told that they have a neighbour (IEX_SPMM_BESIDE_GATHER_KERNEL): where the
    # fp32 matrix-core kernel and the row kernel are close the library then takes the matrix cores, which leaves the
    # L2 -> CU path to the other branch.  The cells that run on the matrix cores go to one branch, the gather-bound
    # ones to the other, both longest first: kernels of different units side by side, the reference's co-run premise.
    hinted_kernel = {c: kernel_of(spmm32(*c)) for c in cells}
    on_matrix_cores = [c for c in by_cost if "mfma" in hinted_kernel[c]]
    branches = [on_matrix_cores, [c for c in by_cost if c not in on_matrix_cores]]
    if not branches[0] or not branches[1]:
        branches = plain_branches
    ms_same_serialized, _ = time_sweep([[spmm32(s, n) for s, n in cells]])     # the timed graph's kernels, one after the other
    ms_per_step, wall_ms = time_sweep([[spmm32(s, n) for s, n in b] for b in branches])
    value = sweep_bytes / 1e9 / (ms_per_step * 1e-3)
    log(f"[bench] {ms_per_step * 1e3:.1f} us per sweep on two branches ({len(branches[0])} cells on the matrix cores beside {len(branches[1])} "
        f"gather-bound ones), {ms_two_plain * 1e3:.1f} us on two branches with every kernel as chosen alone, {ms_one_branch * 1e3:.1f} us on one "
        f"(host wall {wall_ms / args.steps * 1e3:.1f} us) -> {value:.1f} GB/s")

    # ------------------------------------------- per-cell launch durations (HIP events)
    def time_cell(fn, repeats=CELL_REPEATS, samples=5):
        """Average duration of one launch, caches warm: `repeats` launches in one graph on the current
        stream, events around the graph launch, median of `samples`."""
        ms = IL.time_execs([fn] * repeats, repeats=samples, warmup=1)
        return ms / repeats * 1e3  # us

    cold_scratch = torch.empty(COLD_SCRATCH_BYTES // 4, dtype=torch.float32, device=dev)

    def time_cold(fn, samples=7):
        """Duration of one launch with cold caches: 512 MB are written between samples (more than the 256 MB
        last-level cache, the reference's protocol: benchmark/utils_bench_transformer.py:60,73-75), one eager launch
        between two events on the current stream, median of `samples`.  Includes the few us of an eager launch."""
        fn()
        times = []
        for i in range(samples):
            cold_scratch.fill_(float(i))
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b))
        return statistics.median(times) * 1e3  # us

    table = []
    for s, n in cells:
        kernel = kernel_of(spmm32(s, n))
        us = time_cell(spmm32(s, n))
        cold = time_cold(spmm32(s, n))
        by, fl = cell_bytes(s, n), W.spmm_flops(mats[s].nnz, n)
        table.append({"sparsity": s, "n": n, "nnz": mats[s].nnz, "us": round(us, 2), "cold_us": round(cold, 2),
                      "GBps": round(by / us / 1e3, 1), "cold_GBps": round(by / cold / 1e3, 1),
                      "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4), "GFLOPs": round(fl / us / 1e3, 1),
                      "valu_frac": round(fl / us / 1e6 / VALU_PEAK_TFLOPS_FP32, 4),
                      "gather_TBps": round(mats[s].nnz * n * 4 / us / 1e6, 2),
                      "bound": ("vector ALU (fp32 MFMAs run on it, and so does the expansion of the sparse operand)" if "mfma_f32" in kernel else
                                "L2 -> CU path (every nonzero gathers n * 4 bytes of the dense operand out of L2: gather_TBps, against about 26 TB/s that this path has delivered at best)"
                                if mats[s].nnz * n * 4 / us / 1e6 >= 15.0 else "launch and ramp-up (the kernel is a few microseconds long)"),
                      "kernel": kernel, "bytes": by})
        alone_kernel = kernel_of(spmm32_alone(s, n))
        if alone_kernel != kernel:      # (the library's choice for this cell without a neighbour, and how long that takes alone)
            table[-1]["kernel_chosen_without_neighbour"] = alone_kernel
            table[-1]["us_of_that_kernel_alone"] = round(time_cell(spmm32_alone(s, n)), 2)
        log(f"[bench] fp32 s={s} n={n}: {us:.2f} us warm, {cold:.2f} us cold  {by / us / 1e3:.0f} GB/s  {fl / us / 1e3:.0f} GFLOP/s  {kernel}")

    by_kernel = {}
    for row in table:
        by_kernel.setdefault(row["kernel"], []).append(row)
    dom_name, dom_rows = max(by_kernel.items(), key=lambda kv: sum(r["us"] for r in kv[1]))
    dom_bytes = statistics.mean(r["bytes"] for r in dom_rows)
    dom_us = statistics.mean(r["us"] for r in dom_rows)
    measured, measured_commit = read_traffic_profile()
    usable = [measured.get((r["sparsity"], r["n"])) for r in dom_rows]
    traffic_ok = all(u is not None and u[0] == dom_name for u in usable)
    traffic = round(statistics.mean(u[1] for u in usable)) if traffic_ok else None
    traffic_source = (f"profiles/{os.path.basename(TRAFFIC_PROFILE)}, measured at commit {measured_commit} on the same "
                      "kernel instantiation (name compared with what the library reports now)") if traffic_ok else \
        "none: the committed counter summary was taken on another kernel than the one the library launches now"
    common = {"traffic": traffic, "traffic_source": traffic_source, "kernel": dom_name,
              "kernel_name_from": "iex_last_kernels() after an eager call of each cell, as it runs in the timed graph",
              "avg_launch_us": round(dom_us, 2), "algorithmic_bytes_per_launch": int(dom_bytes),
              "cells": [[r["sparsity"], r["n"]] for r in dom_rows],
              "share_of_the_sweeps_kernel_time": round(sum(r["us"] for r in dom_rows) / sum(r["us"] for r in table), 3)}
    if "mfma_f32" in dom_name:
        # the fp32 matrix-core kernel: bound by the matrix / vector ALUs (fp32 MFMAs execute on the vector ALUs), counted
        # on algorithmic flops (2 * nnz * n); it also multiplies the zeros of the tiles it expands
        dom_flops = statistics.mean(W.spmm_flops(r["nnz"], r["n"]) for r in dom_rows)
        dense_flops = statistics.mean(2.0 * mats[r["sparsity"]].m * mats[r["sparsity"]].k * r["n"] for r in dom_rows)
        roofline = {"bound": "mfma", "achieved": round(dom_flops / dom_us / 1e6, 2), "peak": MFMA_PEAK_TFLOPS_FP32, "unit": "TFLOP/s",
                    "frac": round(dom_flops / dom_us / 1e6 / MFMA_PEAK_TFLOPS_FP32, 4), **common,
                    "algorithmic_flops_per_launch": int(dom_flops),
                    "dense_equivalent_TFLOPs": round(dense_flops / dom_us / 1e6, 1),
                    "dense_equivalent_frac": round(dense_flops / dom_us / 1e6 / MFMA_PEAK_TFLOPS_FP32, 4),
                    "hbm_frac": round(dom_bytes / dom_us / 1e3 / HBM_PEAK_GBPS, 4),
                    "note": "fp32 matrix-core SpMM (v_mfma_f32_32x32x2_f32): achieved = 2 * nnz * n per launch / launch duration "
                            "against the fp32 MFMA peak; the kernel multiplies whole 32 x 128 tiles of the expanded sparse operand "
                            "(dense_equivalent_*), and fp32 MFMAs share the vector ALUs with that expansion; traffic = HBM-side bytes "
                            "per launch from rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE"}
    else:
        roofline = {"bound": "hbm", "achieved": round(dom_bytes / dom_us / 1e3, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": round(dom_bytes / dom_us / 1e3 / HBM_PEAK_GBPS, 4), **common,
                    "gather_bytes_per_launch": int(statistics.mean(r["nnz"] * r["n"] * 4 for r in dom_rows)),
                    "gather_TBps": round(statistics.mean(r["nnz"] * r["n"] * 4 for r in dom_rows) / dom_us / 1e6, 2),
                    "note": "every nonzero gathers n*4 bytes of the dense operand from L2 (gather_bytes_per_launch); the "
                            "kernel is bound by that L2->CU bandwidth (gather_TBps), not by HBM, so frac stays small; "
                            "traffic = HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE"}
    # the gather-bound kernel with the largest share, for the record, when the dominant one is the matrix-core kernel
    gather_rows = max(((k, v) for k, v in by_kernel.items() if "mfma" not in k), key=lambda kv: sum(r["us"] for r in kv[1]), default=None)
    if gather_rows is not None and gather_rows[0] != dom_name:
        g_us = statistics.mean(r["us"] for r in gather_rows[1])
        g_by = statistics.mean(r["bytes"] for r in gather_rows[1])
        roofline["largest_gather_kernel"] = {"kernel": gather_rows[0], "cells": [[r["sparsity"], r["n"]] for r in gather_rows[1]],
                                             "avg_launch_us": round(g_us, 2), "hbm_frac": round(g_by / g_us / 1e3 / HBM_PEAK_GBPS, 4),
                                             "gather_TBps": round(statistics.mean(r["nnz"] * r["n"] * 4 for r in gather_rows[1]) / g_us / 1e6, 2)}

    cold_sweep_us = sum(r["cold_us"] for r in table)
    result = {
        "metric": "SpMM/SDDMM GB/s and % HBM peak; co-run makespan vs serialized (%) on 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config 2: fp32 CSR SpMM sweep, A 4096x4096 at {70,80,90,95,98}% sparsity (geometric "
                               "row lengths), B 4096x{64,128,256}; one step = the 15 launches in one hipGraph on two parallel branches (matrix-core cells beside gather-bound cells)",
                   "value_is": "algorithmic bytes of the sweep / time per sweep",
                   "pct_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2), "cache": "warm (operands stay in L2 / MALL between steps)",
                   "graph": "two parallel branches: " + " | ".join(", ".join(f"{s}/{n}" for s, n in b) for b in branches),
                   "one_branch_sweep_us": round(ms_one_branch * 1e3, 1),
                   "two_branches_every_kernel_as_chosen_alone_us": round(ms_two_plain * 1e3, 1),
                   "same_kernels_on_one_branch_us": round(ms_same_serialized * 1e3, 1),
                   "corun_makespan_pct_of_the_same_kernels_serialized": round(100 * ms_per_step / ms_same_serialized, 1),
                   "corun_makespan_pct_of_the_sweep_as_chosen_alone_serialized": round(100 * ms_per_step / ms_one_branch, 1),
                   "kernels_in_the_timed_graph": {f"{s}/{n}": hinted_kernel[(s, n)].split(" (")[0] for s, n in cells},
                   "cold_cache_sweep_us": round(cold_sweep_us, 1),
                   "cold_cache_GBps": round(sweep_bytes / cold_sweep_us / 1e3, 1),
                   "cold_cache_protocol": "per cell: 512 MB written, then one eager launch between two events; sum of the 15 medians of 7"},
        "roofline": roofline,
    }
    extras = {"cells_fp32": [{k: v for k, v in r.items() if k != "bytes"} for r in table],
              "sweep_GFLOPs": round(sweep_flops / (ms_per_step * 1e-3) / 1e9, 1)}

    # ------------------------------------------------------------------ CPU baselines
    if not args.no_cpu:
        # the reference's CPU path for this metric: torch.sparse CSR @ dense on the host cores, every one of the
        # 15 cells, median of 5 runs per cell after one untimed run
        nthreads = torch.get_num_threads()
        cpu_cells = []
        for s, n in cells:
            c = mats[s]
            a_t = torch.sparse_csr_tensor(torch.from_numpy(c.row_offsets), torch.from_numpy(c.column_indices),
                                          torch.from_numpy(c.values), size=(c.m, c.k))
            b_t = torch.from_numpy(dens[n][0])
            _ = a_t @ b_t
            ts = []
            for _ in range(5):
                t0 = time.perf_counter()
                _ = a_t @ b_t
                ts.append(time.perf_counter() - t0)
            cpu_cells.append(statistics.median(ts))
        cpu_s = sum(cpu_cells)
        result["cpu_baseline"] = {"value": round(sweep_bytes / 1e9 / cpu_s, 3), "unit": "GB/s", "cores": nthreads, "kind": "reference",
                                  "library": "torch.sparse_csr_tensor @ dense (fp32), the CPU path the metric names; the reference's own "
                                             "native path is CUDA-only and cannot be built here",
                                  "sample": f"all 15 fp32 cells of the same sweep, median of 5 runs per cell, {cpu_s * 1e3:.1f} ms per sweep",
                                  "torch_num_threads": nthreads, "host_cpu_count": os.cpu_count()}
        log(f"[bench] torch.sparse CSR on {nthreads} threads: {cpu_s * 1e3:.1f} ms per sweep -> {sweep_bytes / 1e9 / cpu_s:.2f} GB/s")
        extras["cpu"] = cpu_extras(torch, W, mats, dens, cells, cell_bytes, sweep_bytes, nthreads, log)

    # ------------------------------------------------------------------------ extras
    if not args.no_extras:
        try:
            extras.update(run_extras(torch, ops, dev, W, IL, mats, dens, csr_dev, time_cell, time_cold, kernel_of, log))
        except Exception as e:
            import traceback
            traceback.print_exc(file=sys.stderr)
            extras["error"] = repr(e)
    result["extras"] = extras
    print(json.dumps(result), flush=True)


def summarize_pmc(fetch_csv, write_csv, cells_json):
    """Writes profiles/spmm_fp32_config2_hbm_traffic_pmc.txt from the two counter runs of `--pmc-probe`."""
    import csv
    import subprocess

    def per_dispatch(path, counter):
        out = {}
        for r in csv.DictReader(open(path)):
            if r["Counter_Name"] == counter:
                out[int(r["Dispatch_Id"])] = (r["Kernel_Name"], float(r["Counter_Value"]))
        return [out[k] for k in sorted(out)]

    probe = json.load(open(cells_json))
    cells, nbytes = probe["cells"], probe["copy_bytes"]
    readings = {}
    for counter, path in (("FETCH_SIZE", fetch_csv), ("WRITE_SIZE", write_csv)):
        d = per_dispatch(path, counter)
        copies = [v for name, v in d if "copy_kernel" in name]
        last_copy = max(i for i, (name, _) in enumerate(d) if "copy_kernel" in name)
        spmm = [(name, v) for name, v in d[last_copy + 1:] if "spmm" in name]
        assert len(copies) == 3 and len(spmm) == 3 * len(cells), (counter, len(copies), len(spmm))
        readings[counter] = (statistics.median(copies), [statistics.median(v for _, v in spmm[3 * i: 3 * i + 3]) for i in range(len(cells))],
                             [spmm[3 * i][0] for i in range(len(cells))])
    f_copy, f_cells, f_names = readings["FETCH_SIZE"]
    w_copy, w_cells, _ = readings["WRITE_SIZE"]
    f_scale, w_scale = nbytes / (f_copy * 1024.0), nbytes / (w_copy * 1024.0)
    commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], stdout=subprocess.PIPE, text=True).stdout.strip() or "unknown"
    lines = [
        "HBM-side traffic (L2 misses + write-backs) of the 15 fp32 cells of config 2, one MI355X, per launch.",
        "Two counter runs of the same committed command (rocprofv3 does not split counters over passes), then this summary:",
        "  rocprofv3 --pmc FETCH_SIZE -d gpurun_out/pmc_fetch -o p --output-format csv -- python3 bench.py --pmc-probe",
        "  rocprofv3 --pmc WRITE_SIZE -d gpurun_out/pmc_write -o p --output-format csv -- python3 bench.py --pmc-probe",
        "  python3 bench.py --summarize-pmc gpurun_out/pmc_fetch/p_counter_collection.csv gpurun_out/pmc_write/p_counter_collection.csv gpurun_out/pmc_probe_cells.json",
        "Both counters read KiB per dispatch; each is scaled by what it reads for a plain copy of known size (iex_copy_bytes,",
        "256 MiB read and 256 MiB written, three dispatches, median).  Every cell: three dispatches, median.  `kernel` is what",
        "the library reported for the cell in the probe run (iex_last_kernels); bench.py uses a line only while that still",
        "holds.  traffic_bytes = fetch_kib * 1024 * fetch_scale + write_kib * 1024 * write_scale.",
        f"measured_at_commit {commit}",
        f"calibration | copy_bytes={nbytes} | fetch_kib={f_copy:.0f} | fetch_scale={f_scale:.3f} | write_kib={w_copy:.0f} | write_scale={w_scale:.3f}",
    ]
    for i, c in enumerate(cells):
        traffic = f_cells[i] * 1024 * f_scale + w_cells[i] * 1024 * w_scale
        assert c["kernel"].split("<")[0] in f_names[i], (c["kernel"], f_names[i])
        lines.append(f"cell | sparsity={c['sparsity']} | n={c['n']} | kernel={c['kernel']} | fetch_kib={f_cells[i]:.0f} | write_kib={w_cells[i]:.0f} | "
                     f"traffic_bytes={traffic:.0f} | algorithmic_bytes={c['algorithmic_bytes']} | ratio={traffic / c['algorithmic_bytes']:.2f}")
    open(TRAFFIC_PROFILE, "w").write("\n".join(lines) + "\n")
    print("\n".join(lines))


def cpu_extras(torch, W, mats, dens, cells, cell_bytes, sweep_bytes, nthreads, log):
    """The other CPU legs: the single-core C port of the oracle and scipy CSR on the same sweep, the SDDMM of config 1
    (gather form in numpy, torch.sparse.sampled_addmm) and the GEMM of config 4 (torch.matmul, fp32)."""
    out = {}
    import oracle  # test infrastructure, used here only as a measured CPU port
    oracle.build()
    t0, passes = time.perf_counter(), 0
    while passes < 2 or time.perf_counter() - t0 < 6.0:
        for s, n in cells:
            c = mats[s]
            oracle.spmm_f32(dens[n], c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
        passes += 1
    port_s = (time.perf_counter() - t0) / passes
    out["c_port_single_core"] = {"GBps": round(sweep_bytes / 1e9 / port_s, 3), "s_per_sweep": round(port_s, 3), "passes": passes,
                                 "what": "oracle.c compiled with gcc -O3, one thread, all 15 cells"}
    try:
        import scipy.sparse as sp
        ts = []
        for s, n in cells:
            c = mats[s]
            a_s = sp.csr_matrix((c.values, c.column_indices, c.row_offsets), shape=(c.m, c.k))
            reps = []
            for _ in range(3):
                t0 = time.perf_counter()
                _ = a_s @ dens[n][0]
                reps.append(time.perf_counter() - t0)
            ts.append(statistics.median(reps))
        out["scipy_csr"] = {"GBps": round(sweep_bytes / 1e9 / sum(ts), 3), "s_per_sweep": round(sum(ts), 3),
                            "what": "scipy.sparse.csr_matrix @ dense, all 15 cells, median of 3 per cell (single-threaded)"}
    except Exception as e:  # a library baseline must not take the bench down
        out["scipy_csr"] = {"error": repr(e)}
    # SDDMM, config 1: mask 1024 x 1024 at 90 %, k = 64, fp32
    try:
        a1, _, lhs1, rhs1 = W.config1()
        rows = np.repeat(np.arange(a1.m), np.diff(a1.row_offsets))
        reps = []
        for _ in range(5):
            t0 = time.perf_counter()
            _ = np.einsum("ij,ij->i", lhs1[0][rows], rhs1[0][a1.column_indices])
            reps.append(time.perf_counter() - t0)
        by = W.sddmm_bytes(a1.m, 64, a1.k, a1.nnz, 1, 4, True)
        out["sddmm_c1_numpy_gather"] = {"ms": round(statistics.median(reps) * 1e3, 3), "GBps": round(by / statistics.median(reps) / 1e9, 3)}
        mask = torch.sparse_csr_tensor(torch.from_numpy(a1.row_offsets), torch.from_numpy(a1.column_indices),
                                       torch.zeros(a1.nnz), size=(a1.m, a1.k))
        lt, rt = torch.from_numpy(lhs1[0]), torch.from_numpy(rhs1[0]).t().contiguous()
        _ = torch.sparse.sampled_addmm(mask, lt, rt, beta=0.0)
        reps = []
        for _ in range(5):
            t0 = time.perf_counter()
            _ = torch.sparse.sampled_addmm(mask, lt, rt, beta=0.0)
            reps.append(time.perf_counter() - t0)
        out["sddmm_c1_torch_sampled_addmm"] = {"ms": round(statistics.median(reps) * 1e3, 3), "threads": nthreads,
                                               "GBps": round(by / statistics.median(reps) / 1e9, 3)}
    except Exception as e:
        out["sddmm_c1_cpu"] = {"error": repr(e)}
    # GEMM, config 4's shape (4096 x 4096 x 2048), torch.matmul in fp32 on the host
    try:
        ga, gb = torch.randn(4096, 4096), torch.randn(4096, 2048)
        _ = ga @ gb
        reps = []
        for _ in range(3):
            t0 = time.perf_counter()
            _ = ga @ gb
            reps.append(time.perf_counter() - t0)
        out["gemm_c4_torch_matmul_fp32"] = {"ms": round(statistics.median(reps) * 1e3, 1), "threads": nthreads,
                                            "TFLOPs": round(2.0 * 4096 * 4096 * 2048 / statistics.median(reps) / 1e12, 3)}
    except Exception as e:
        out["gemm_c4_cpu"] = {"error": repr(e)}
    log(f"[bench] CPU legs: {json.dumps(out)}")
    return out


def run_extras(torch, ops, dev, W, IL, mats, dens, csr_dev, time_cell, time_cold, kernel_of, log):
    out = {}
    # ---- fp16 sweep (int16 column indices, the reference's half layout)
    rows = []
    calls16 = {}
    for s in W.C2_SPARSITIES:
        c = mats[s]
        ri, v, ro, ci = csr_dev(c, torch.float16, torch.int16)
        for n in W.C2_NS:
            b = torch.from_numpy(dens[n]).to(dev).half()
            calls16[(s, n)] = (lambda b=b, ri=ri, v=v, ro=ro, ci=ci, m=c.m: ops.spmm_sputnik_reuse_weight_half(b, ri, v, ro, ci, m))
            us = time_cell(lambda: ops.spmm_sputnik_reuse_weight_half(b, ri, v, ro, ci, c.m))
            by = W.spmm_bytes(c.m, c.k, n, c.nnz, 1, 2, 2)
            fl = W.spmm_flops(c.nnz, n)
            rows.append({"sparsity": s, "n": n, "us": round(us, 2), "GBps": round(by / us / 1e3, 1),
                         "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4), "GFLOPs": round(fl / us / 1e3, 1),
                         "kernel": kernel_of(calls16[(s, n)])})
    out["cells_fp16_i16"] = rows
    # the same 15 launches as one graph: on one branch, and on two -- the cells that run on the matrix cores (dense form
    # + GEMM) on one, the gather-bound ones on the other, as in the timed fp32 step; and dealt alternately by nnz * n
    order16 = sorted(calls16, key=lambda c: -mats[c[0]].nnz * c[1])
    on_mc = [c for c in order16 if "gemm" in next(r["kernel"] for r in rows if (r["sparsity"], r["n"]) == c)]
    rest = [c for c in order16 if c not in on_mc]
    out["sweep_fp16_i16"] = {
        "one_branch_us": round(IL.run_non_interleaving([calls16[c] for c in calls16]) * 1e3, 1),
        "two_branches_us": round(IL.run_interleaving([calls16[c] for c in on_mc], [calls16[c] for c in rest]) * 1e3, 1) if on_mc and rest else None,
        "two_branches_are": f"{len(on_mc)} cells on the matrix cores (dense form + GEMM) | {len(rest)} gather-bound cells",
        "two_branches_dealt_alternately_us": round(IL.run_interleaving([calls16[c] for c in order16[0::2]], [calls16[c] for c in order16[1::2]]) * 1e3, 1),
        "sum_of_cells_us": round(sum(r["us"] for r in rows), 1)}
    log("[bench] fp16 sweep done")

    # ---- SDDMM: config 1 (fp32, batch-summed) and config 3 (fp16, 16 heads, per-head output)
    a1, _, lhs1, rhs1 = W.config1()
    ri, _, ro, ci = csr_dev(a1)
    l1, r1 = torch.from_numpy(lhs1).to(dev), torch.from_numpy(rhs1).to(dev)
    us = time_cell(lambda: ops.sddmm_sputnik_atomic_upd_weight(l1, r1, ri, ro, ci))
    by = W.sddmm_bytes(a1.m, 64, a1.k, a1.nnz, 1, 4, True)
    out["sddmm_c1_fp32"] = {"us": round(us, 2), "GBps": round(by / us / 1e3, 1), "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4),
                            "GFLOPs": round(W.sddmm_flops(a1.nnz, 64) / us / 1e3, 1),
                            "kernel": kernel_of(lambda: ops.sddmm_sputnik_atomic_upd_weight(l1, r1, ri, ro, ci)),
                            "bound": "launch (1.4 MB of operands: the kernel is a few microseconds of ramp-up and drain)"}
    # config 1's SpMM: A 1024 x 1024 at 90 %, B 1024 x 256, fp32
    v1 = torch.from_numpy(a1.values).to(dev)
    b1 = torch.from_numpy(W.config1()[1]).to(dev)
    us = time_cell(lambda: ops.spmm_sputnik_reuse_weight(b1, ri, v1, ro, ci, a1.m))
    by = W.spmm_bytes(a1.m, a1.k, b1.shape[2], a1.nnz, 1, 4, 4)
    fl = W.spmm_flops(a1.nnz, b1.shape[2])
    out["spmm_c1_fp32"] = {"us": round(us, 2), "cold_us": round(time_cold(lambda: ops.spmm_sputnik_reuse_weight(b1, ri, v1, ro, ci, a1.m)), 2),
                           "GBps": round(by / us / 1e3, 1), "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4),
                           "GFLOPs": round(fl / us / 1e3, 1), "valu_frac": round(fl / us / 1e6 / VALU_PEAK_TFLOPS_FP32, 4),
                           "kernel": kernel_of(lambda: ops.spmm_sputnik_reuse_weight(b1, ri, v1, ro, ci, a1.m)),
                           "bound": "launch (2.9 MB of operands, 0.4 us at either roof)"}
    pat, q, k, v = W.config3()
    ri3, _, ro3, ci3 = csr_dev(pat, tables=True)
    qt, kt, vt = (torch.from_numpy(x).to(dev).half() for x in (q, k, v))
    us = time_cell(lambda: ops.sddmm_sputnik_half(qt, kt, ri3, ro3, ci3), repeats=10)
    by = W.sddmm_bytes(pat.m, 64, pat.k, pat.nnz, 16, 2, False)
    out["sddmm_c3_fp16_16heads"] = {"nnz": pat.nnz, "sparsity": round(pat.sparsity, 4), "us": round(us, 2),
                                    "cold_us": round(time_cold(lambda: ops.sddmm_sputnik_half(qt, kt, ri3, ro3, ci3)), 2),
                                    "kernel": kernel_of(lambda: ops.sddmm_sputnik_half(qt, kt, ri3, ro3, ci3)),
                                    "GBps": round(by / us / 1e3, 1), "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4),
                                    "GFLOPs": round(W.sddmm_flops(pat.nnz, 64, 16) / us / 1e3, 1)}
    from intrasm_engine_amd.pytorch import ops as pyops_k
    plan_ = pyops_k.SddmmPlan()       # a caller with a fixed mask keeps the tables: the setup kernel runs once
    pyops_k.sddmm_half_planned(qt, kt, ri3, ro3, ci3, plan_)
    out["sddmm_c3_fp16_16heads"]["tables_kept_us"] = round(time_cell(lambda: pyops_k.sddmm_half_planned(qt, kt, ri3, ro3, ci3, plan_), repeats=10), 2)
    out["sddmm_c3_fp16_16heads"]["tables_kept_kernel"] = kernel_of(lambda: pyops_k.sddmm_half_planned(qt, kt, ri3, ro3, ci3, plan_))
    with pyops_k.kernel_params(sddmm={"force_variant": 1}):
        out["sddmm_c3_fp16_16heads"]["gather_kernel_us"] = round(time_cell(lambda: ops.sddmm_sputnik_half(qt, kt, ri3, ro3, ci3), repeats=10), 2)
    # the same operator on other masks (16 heads x 4096 x 4096, k = 64): what it picks by itself against the gather kernel
    import numpy as np_
    rng_ = np_.random.default_rng(0)
    idx_ = np_.arange(4096)
    masks_ = {"band_512_plus_32_scattered": W.config3(band=512, extra=32)[0],
              "band_128_plus_16_scattered": W.config3(band=128, extra=16)[0]}
    for label_, m_ in (("block_diagonal_256", (idx_[:, None] // 256) == (idx_[None, :] // 256)),
                       ("causal_window_512", (idx_[:, None] >= idx_[None, :]) & (idx_[:, None] - idx_[None, :] < 512))):
        ro_, ci_, _ = W.csr_from_mask(m_)
        masks_[label_] = W.CSR(4096, 4096, np_.ones(ci_.shape[0], np_.float32), W.swizzle_from_offsets(ro_), ro_, ci_)
    for d_ in (0.01, 0.05, 0.10, 0.20):
        ro_, ci_ = W.csr_from_row_lengths(rng_, 4096, 4096, np_.full(4096, int(4096 * d_)))
        masks_[f"equal_rows_random_columns_{d_:.2f}"] = W.CSR(4096, 4096, np_.ones(ci_.shape[0], np_.float32), W.swizzle_from_offsets(ro_), ro_, ci_)
    rows_m = []
    for label_, c_ in masks_.items():
        rim, _, rom, cim = csr_dev(c_, tables=True)
        f_ = lambda: ops.sddmm_sputnik_half(qt, kt, rim, rom, cim)
        us_op = time_cell(f_, repeats=5, samples=3)
        with pyops_k.kernel_params(sddmm={"force_variant": 1}):
            us_ga = time_cell(f_, repeats=5, samples=3)
        rows_m.append({"mask": label_, "density": round(c_.nnz / 4096 / 4096, 4), "operator_us": round(us_op, 1), "gather_kernel_us": round(us_ga, 1),
                       "operator_kernel": kernel_of(f_)})
        del rim, rom, cim
    out["sddmm_fp16_16heads_by_mask"] = rows_m
    # the second product of attention on the same masks (values per head, n = 64): what the operator picks by itself, the same
    # with tables and lists kept in a plan, and the row kernel
    rows_p = []
    v16_ = torch.randn(16, 4096, 64, device=dev, generator=torch.Generator(dev).manual_seed(5)).half()
    for label_, c_ in masks_.items():
        rim, _, rom, cim = csr_dev(c_, tables=True)
        pr_ = (torch.rand(16, c_.nnz, device=dev, generator=torch.Generator(dev).manual_seed(6)) / 280).half()
        f_ = lambda: ops.spmm_sputnik_batched_values(v16_, rim, pr_, rom, cim, 4096)
        us_op = time_cell(f_, repeats=5, samples=3)
        name_ = kernel_of(f_)
        row_ = {"mask": label_, "density": round(c_.nnz / 4096 / 4096, 4), "operator_us": round(us_op, 1), "operator_kernel": name_}
        if "spmm_blocks_kernel" in name_:
            pl_ = pyops_k.SddmmPlan()
            g_ = lambda: pyops_k.spmm_batched_values_planned(v16_, rim, pr_, rom, cim, 4096, pl_)
            g_()
            row_["tables_kept_us"] = round(time_cell(g_, repeats=5, samples=3), 1)
        with pyops_k.kernel_params(spmm={"force_variant": 1}):
            row_["row_kernel_us"] = round(time_cell(f_, repeats=5, samples=3), 1)
        rows_p.append(row_)
        del rim, rom, cim, pr_
    out["spmm_fp16_16heads_by_mask"] = rows_p
    scores = ops.sddmm_sputnik_half(qt, kt, ri3, ro3, ci3)
    us = time_cell(lambda: ops.spmm_sputnik_batched_values(vt, ri3, scores, ro3, ci3, pat.m), repeats=10)
    by = W.spmm_bytes(pat.m, pat.k, 64, pat.nnz, 16, 2, 4, True)
    out["spmm_c3_fp16_16heads"] = {"us": round(us, 2), "GBps": round(by / us / 1e3, 1),
                                   "cold_us": round(time_cold(lambda: ops.spmm_sputnik_batched_values(vt, ri3, scores, ro3, ci3, pat.m)), 2),
                                   "kernel": kernel_of(lambda: ops.spmm_sputnik_batched_values(vt, ri3, scores, ro3, ci3, pat.m)),
                                   "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4),
                                   "GFLOPs": round(W.spmm_flops(pat.nnz, 64, 16) / us / 1e3, 1)}
    # the same plan as the SDDMM's: the tables are shared, the SpMM keeps two lists of its own behind them
    f_planned = lambda: pyops_k.spmm_batched_values_planned(vt, ri3, scores, ro3, ci3, pat.m, plan_)
    f_planned()
    out["spmm_c3_fp16_16heads"]["tables_kept_us"] = round(time_cell(f_planned, repeats=10), 2)
    out["spmm_c3_fp16_16heads"]["tables_kept_kernel"] = kernel_of(f_planned)
    with pyops_k.kernel_params(spmm={"force_variant": 1}):
        out["spmm_c3_fp16_16heads"]["row_kernel_us"] = round(time_cell(lambda: ops.spmm_sputnik_batched_values(vt, ri3, scores, ro3, ci3, pat.m), repeats=10), 2)
    from intrasm_engine_amd.pytorch.sparse_attention import sparse_attention
    us_block = time_cell(lambda: sparse_attention(qt, kt, vt, ri3, ro3, ci3), repeats=10)
    us_block_planned = time_cell(lambda: sparse_attention(qt, kt, vt, ri3, ro3, ci3, plan=plan_), repeats=10)
    us_softmax = time_cell(lambda: ops.csr_softmax_(scores, ri3, ro3, 0.125), repeats=10)
    out["attention_block_c3_fp16_16heads"] = {
        "us": round(us_block, 2), "with_tables_kept_us": round(us_block_planned, 2), "softmax_us": round(us_softmax, 2),
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
    # Eight distinct operand sets per branch, as the reference's harness runs them (tests/test_interleaving.py:544,617):
    # every repetition reads its own copy of the weight (same pattern, values of its own), activation and GEMM
    # operands, so no repetition finds the previous one's operands in the caches.
    from intrasm_engine_amd.pytorch import ops as pyops
    w, x, ga, gb = W.config4()
    reps = 8
    riw, vw, row, ciw = csr_dev(w, torch.float16, torch.int16)
    gen = torch.Generator(dev).manual_seed(4)
    sets = []
    for i in range(reps):
        sign = (torch.randint(0, 2, vw.shape, device=dev, generator=gen) * 2 - 1).to(vw.dtype)
        sets.append((riw.clone(), vw * sign if i else vw, row.clone(), ciw.clone(),   # (patterns of the copies: looked at below)
                     torch.randn(1, w.k, 2048, device=dev, generator=gen).half() if i else torch.from_numpy(x).to(dev).half(),
                     torch.randn(4096, 4096, device=dev, generator=gen).bfloat16() if i else torch.from_numpy(ga).to(dev).bfloat16(),
                     torch.randn(4096, 2048, device=dev, generator=gen).bfloat16() if i else torch.from_numpy(gb).to(dev).bfloat16()))
    for t in sets:
        pyops.prepare_pattern(t[2], t[3], w.k, tables=False)
    kw4 = dict(per_batch_values=False, accumulate=False, dtypes=(torch.float16,), allow_i16=True)

    def spmm_list(**extra):
        return [(lambda t=t: pyops._spmm(t[4], t[0], t[1], t[2], t[3], w.m, **extra, **kw4)) for t in sets]

    spmm_execs = [(lambda t=t: ops.spmm_sputnik_reuse_weight_half(t[4], t[0], t[1], t[2], t[3], w.m)) for t in sets]
    gemm_execs = [(lambda t=t: ops.gemm_mfma(t[5], t[6], False)) for t in sets]
    fused_execs = [(lambda t=t: ops.fused_spmm_gemm(t[4], t[0], t[1], t[2], t[3], w.m, t[5], t[6], False, 0)) for t in sets]
    fused_g_execs = [(lambda t=t: ops.fused_spmm_gemm(t[4], t[0], t[1], t[2], t[3], w.m, t[5], t[6], False, 64)) for t in sets]
    fused_s_execs = [(lambda t=t: ops.fused_spmm_gemm(t[4], t[0], t[1], t[2], t[3], w.m, t[5], t[6], False, -1)) for t in sets]
    t_spmm = IL.run_non_interleaving(spmm_execs) / reps
    t_gemm = IL.run_non_interleaving(gemm_execs) / reps
    t_serial = IL.run_non_interleaving(spmm_execs, gemm_execs) / reps
    t_graph = IL.run_interleaving(spmm_execs, gemm_execs) / reps
    t_fused = IL.run_non_interleaving(fused_execs) / reps
    t_fused_g = IL.run_non_interleaving(fused_g_execs) / reps
    t_fused_s = IL.run_non_interleaving(fused_s_execs) / reps
    # the same pair with the SpMM forced onto the gather (row) kernel: vector ALU + L2 beside the matrix cores,
    # the resource split the reference's co-run experiment is about
    gather_execs = spmm_list(force_variant=1)
    t_gather = IL.run_non_interleaving(gather_execs) / reps
    t_graph_gather = IL.run_interleaving(gather_execs, gemm_execs) / reps
    # the library's choice above has a workspace to use (the operator allocates one) and takes the dense-form
    # path; without one the 8-wave matrix-core SpMM kernel runs, the kernel the fused launch shares its SpMM role with
    mc_execs = spmm_list(no_workspace=True)
    t_mc = IL.run_non_interleaving(mc_execs) / reps
    t_graph_mc = IL.run_interleaving(mc_execs, gemm_execs) / reps
    k_spmm, k_gemm, k_fused = kernel_of(spmm_execs[0]), kernel_of(gemm_execs[0]), kernel_of(fused_execs[0])
    cold_spmm, cold_gemm = time_cold(spmm_execs[0]) / 1e3, time_cold(gemm_execs[0]) / 1e3
    fl_s, fl_g = W.spmm_flops(w.nnz, 2048), W.gemm_flops(4096, 2048, 4096)
    by_s = W.spmm_bytes(w.m, w.k, 2048, w.nnz, 1, 2, 2)
    out["config4"] = {
        "spmm_ms": round(t_spmm, 4), "spmm_GBps": round(by_s / t_spmm / 1e6, 1), "spmm_GFLOPs": round(fl_s / t_spmm / 1e6, 1),
        "spmm_hbm_frac": round(by_s / t_spmm / 1e6 / HBM_PEAK_GBPS, 4),
        "spmm_bound": "MFMA (the operator's path multiplies the dense form of the sparse operand on the matrix cores)",
        "spmm_mfma_frac_dense_equivalent": round(2.0 * w.m * w.k * 2048 / t_spmm / 1e9 / MFMA_PEAK_TFLOPS_16BIT, 4),
        "spmm_kernels": k_spmm, "gemm_kernels": k_gemm, "fused_kernels": k_fused,
        "spmm_cold_ms": round(cold_spmm, 4), "gemm_cold_ms": round(cold_gemm, 4),
        "gemm_ms": round(t_gemm, 4), "gemm_TFLOPs": round(IL.gemm_tflops(4096, 2048, 4096, t_gemm), 1),
        "gemm_mfma_frac": round(IL.gemm_tflops(4096, 2048, 4096, t_gemm) / MFMA_PEAK_TFLOPS_16BIT, 4),
        "serialized_sum_ms": round(t_spmm + t_gemm, 4), "serialized_one_stream_ms": round(t_serial, 4),
        "two_branch_graph_ms": round(t_graph, 4), "fused_launch_ms": round(t_fused, 4),
        "fused_launch_gemm_in_groups_of_64_ms": round(t_fused_g, 4),
        "fused_launch_spmm_tiles_first_ms": round(t_fused_s, 4),
        "fused_spmm_tiles_first_pct_of_serialized_matrix_core_kernel": round(100 * t_fused_s / (t_mc + t_gemm), 1),
        "gemm_bound": "MFMA",
        "graph_makespan_pct_of_serialized": round(100 * t_graph / (t_spmm + t_gemm), 1),
        "fused_makespan_pct_of_serialized": round(100 * t_fused / (t_spmm + t_gemm), 1),
        "spmm_matrix_core_kernel_ms": round(t_mc, 4), "two_branch_graph_matrix_core_kernel_ms": round(t_graph_mc, 4),
        "matrix_core_kernel_graph_makespan_pct_of_serialized": round(100 * t_graph_mc / (t_mc + t_gemm), 1),
        "fused_makespan_pct_of_serialized_matrix_core_kernel": round(100 * t_fused / (t_mc + t_gemm), 1),
        "spmm_row_kernel_ms": round(t_gather, 4), "two_branch_graph_row_kernel_ms": round(t_graph_gather, 4),
        "row_kernel_graph_makespan_pct_of_serialized": round(100 * t_graph_gather / (t_gather + t_gemm), 1),
        "spmm_dense_equivalent_TFLOPs": round(2.0 * w.m * w.k * 2048 / t_spmm / 1e9, 1),
        "repeats_per_graph": reps, "operand_sets": f"{reps} distinct (own copies of the CSR arrays, values, activation and GEMM operands per repetition)",
    }
    log(f"[bench] config 4: spmm {t_spmm:.3f} ms, gemm {t_gemm:.3f} ms, graph {t_graph:.3f} ms, fused {t_fused:.3f} ms")
    del w, x, ga, gb, riw, vw, row, ciw, sets, spmm_execs, gemm_execs, fused_execs, fused_g_execs, fused_s_execs, gather_execs, mc_execs
    reps = 4

    # ---- the dense GEMM alone on larger shapes (bf16, B as (K, N)): how far the matrix cores are used
    rows_gemm = []
    for (gm, gn, gk) in ((8192, 8192, 8192), (4096, 8192, 4096), (11008, 8192, 4096), (4096, 2048, 4096)):
        ga2 = torch.randn(gm, gk, device=dev).bfloat16()
        gb2 = torch.randn(gk, gn, device=dev).bfloat16()
        # one protocol for both: 3 launches to warm up, then 16 back to back between two events on the current stream
        # (eager: the vendor library refuses to run under stream capture; a graph of a few launches started from an idle
        # GPU, the protocol of the co-run legs, reads 8-10 % lower for either kernel while the clock ramps up)
        def back_to_back(fn, warm=3, n=16):
            for _ in range(warm):
                fn()
            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            ev0.record()
            for _ in range(n):
                fn()
            ev1.record()
            torch.cuda.synchronize()
            return ev0.elapsed_time(ev1) / n
        t = min(back_to_back(lambda: ops.gemm_mfma(ga2, gb2, False)) for _ in range(2))
        tf = IL.gemm_tflops(gm, gn, gk, t)
        t_graph4 = IL.run_non_interleaving([lambda: ops.gemm_mfma(ga2, gb2, False)] * reps) / reps
        # the vendor library on the same operands in the same run, as a comparator (never on the product path)
        t_lib = min(back_to_back(lambda: torch.matmul(ga2, gb2)) for _ in range(2))
        rows_gemm.append({"m": gm, "n": gn, "k": gk, "ms": round(t, 4), "TFLOPs": round(tf, 1),
                          "mfma_frac": round(tf / MFMA_PEAK_TFLOPS_16BIT, 4), "kernel": kernel_of(lambda: ops.gemm_mfma(ga2, gb2, False)),
                          "protocol": "3 warm-up launches, then 16 back to back between two events, best of 2; the same for torch.matmul",
                          "graph_of_4_from_idle_ms": round(t_graph4, 4), "graph_of_4_from_idle_TFLOPs": round(IL.gemm_tflops(gm, gn, gk, t_graph4), 1),
                          "torch_matmul_is": "torch.matmul (hipBLASLt) on the same operands, eager, a comparator only",
                          "torch_matmul_ms": round(t_lib, 4), "torch_matmul_TFLOPs": round(IL.gemm_tflops(gm, gn, gk, t_lib), 1)})
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
    t_fu_lpt = time_capture(lambda: layer.capture_fused(xa, xb, seqs // 2, None))
    spmm_flops5 = sum(2 * weights[n_].nnz * seqs * L for n_ in weights)
    attn_flops5 = 2 * 2 * seqs * heads * L * L * (hidden // heads)
    out["config5"] = {
        "shape": "hidden 4096, 32 heads, MLP 11008, 16 x 512 tokens, fp16; q/k/v/o 2:4, gate/up/down 80% unstructured",
        "elementwise_ops_included": "softmax(QK^T/sqrt(d)), SiLU(gate)*up, two residual adds (PyTorch kernels); no RoPE / norm / mask",
        "serialized_ms": round(t_ser, 3), "serialized_two_halves_ms": round(t_ser_halves, 3),
        "multistream_graph_ms": round(t_ms, 3), "fused_ms": round(t_fu, 3), "fused_longer_tiles_first_ms": round(t_fu_lpt, 3),
        "multistream_pct_of_serialized": round(100 * t_ms / t_ser, 1), "fused_pct_of_serialized": round(100 * t_fu / t_ser, 1),
        "fused_longer_tiles_first_pct_of_serialized": round(100 * t_fu_lpt / t_ser, 1),
        "spmm_GFLOP": round(spmm_flops5 / 1e9, 1), "attention_GFLOP": round(attn_flops5 / 1e9, 1),
        "layer_TFLOPs_serialized": round((spmm_flops5 + attn_flops5) / t_ser / 1e9, 1),
    }
    log(f"[bench] config 5: serialized {t_ser:.2f} ms, two-stream graph {t_ms:.2f} ms, fused {t_fu:.2f} ms (GEMM tiles first), {t_fu_lpt:.2f} ms (longer tiles first)")
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
