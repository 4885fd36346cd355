"""SpMM over the shapes of the reference's xformers-style sweep
(3rdparty/MyXformers/benchmarks/benchmark_spmm.py:38-103): for every ((B, M, K), sparsity) a random
M x K pattern (row lengths rounded to the reference's ``divisible_by=16`` granularity is not needed
here: the kernels have no alignment rule), values per batch entry, dense operand (B, K, M), the
product timed as one graph of repeated launches.

    python3 -m intrasm_engine_amd.benchmarks.benchmark_spmm [--quick] [--dtype fp32|fp16]

Shapes: Swin-T stages, the "basic" sizes and the ViT/DeiT sizes of the reference, same sparsities.
Each result is first checked against a dense batched product on the device (the reference's sweep
has no such check; it is cheap and catches a mis-built pattern).  Prints one line per configuration:
microseconds per launch, GFLOP/s on nonzero flops, algorithmic GB/s.
"""
from __future__ import annotations

import argparse
import itertools

import numpy as np
import torch

import intrasm_engine_amd  # noqa: F401  (registers the operators, makes a capture stream current)
from intrasm_engine_amd import workloads as W
from intrasm_engine_amd.interleaving import time_execs

SWIN_T = list(zip([(96, 3136, 32), (192, 784, 32), (384, 196, 32), (768, 49, 32)], (0.9844, 0.9375, 0.75, 0.0)))
BASIC = list(itertools.product([(32, 1024, 32), (32, 1024, 128), (8, 4096, 32), (8, 4096, 128)],
                               [0.90, 0.93, 0.95, 0.97, 0.98, 0.99, 0.995, 0.999]))
VIT = list(itertools.product([(192, 785, 64), (192, 197, 64), (384, 785, 64), (384, 197, 64)],
                             [0.70, 0.80, 0.85, 0.90, 0.93, 0.95, 0.97]))
QUICK = [((4, 196, 32), 0.75), ((2, 1024, 128), 0.95), ((3, 49, 32), 0.0)]


def random_pattern(rng: np.random.Generator, m: int, k: int, sparsity: float):
    """Each entry kept with probability 1 - sparsity (the reference's _create_random_sparsity)."""
    mask = rng.random((m, k)) >= sparsity
    ro, ci, _ = W.csr_from_mask(mask)
    return ro, ci, W.swizzle_from_offsets(ro)


def bench_spmm(configs, dtype=torch.float32, repeats=8, seed=0, check=True):
    ops = torch.ops.iex_ops
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    sv = torch.empty((), dtype=dtype).element_size()
    results = []
    for (batch, m, k), sparsity in configs:
        ro, ci, ri = random_pattern(rng, m, k, sparsity)
        nnz = int(ci.shape[0])
        ro_t, ci_t, ri_t = (torch.from_numpy(x).to(dev) for x in (ro, ci, ri))
        values = torch.rand(batch, nnz, generator=g).to(dev).to(dtype)
        b = torch.rand(batch, k, m, generator=g).to(dev).to(dtype)
        run = lambda: ops.spmm_sputnik_batched_values(b, ri_t, values, ro_t, ci_t, m)  # noqa: E731
        out = run()
        if check:
            rows = torch.repeat_interleave(torch.arange(m, device=dev), torch.diff(ro_t.long()))
            dense = torch.zeros(batch, m, k, device=dev, dtype=torch.float32)
            dense[:, rows, ci_t.long()] = values.float()
            want = torch.bmm(dense, b.float())
            tol = 1e-5 if dtype == torch.float32 else 1e-2
            err = (out.float() - want).abs().max().item()
            bound = tol * max(1.0, float(torch.bmm(dense.abs(), b.float().abs()).max()))
            if not err <= bound:
                raise RuntimeError(f"B={batch} M={m} K={k} sparsity={sparsity}: max error {err:.3g} > {bound:.3g}")
        us = time_execs([run] * repeats, repeats=5) / repeats * 1e3
        flops = W.spmm_flops(nnz, m, batch)
        nbytes = W.spmm_bytes(m, k, m, nnz, batch, sv, 4, True)
        results.append({"B": batch, "M": m, "K": k, "sparsity": sparsity, "nnz": nnz, "us": us,
                        "GFLOPs": flops / us / 1e3 if us > 0 else 0.0, "GBps": nbytes / us / 1e3 if us > 0 else 0.0})
        print(f"spmm B={batch:4d}, M=N={m:4d}, K={k:3d}, prob={sparsity:0.4f}  nnz={nnz:8d}  {us:9.2f} us  "
              f"{results[-1]['GFLOPs']:9.1f} GFLOP/s  {results[-1]['GBps']:8.1f} GB/s", flush=True)
    return results


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--quick", action="store_true", help="three small configurations")
    ap.add_argument("--dtype", choices=("fp32", "fp16"), default="fp32")
    args = ap.parse_args(argv)
    dtype = torch.float32 if args.dtype == "fp32" else torch.float16
    if args.quick:
        bench_spmm(QUICK, dtype)
        return 0
    for name, configs in (("Swin Transformer", SWIN_T), ("ViT", VIT), ("basic", BASIC)):
        print(name, flush=True)
        bench_spmm(configs, dtype)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
