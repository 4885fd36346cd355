"""Time every kernel of the dense companion GEMM on one problem size, the counterpart of the
reference's CUTLASS tile sweep (tests/profile_cutlass.py:32-70: for each tile description build the
matmul, time it with ``run_non_interleaving``, print ``gemm_tflops``).

    python3 -m intrasm_engine_amd.tuning.profile_gemm -m 8192 -n 8192 -k 8192 [--dtype bf16] [--trans-b]

Prints one line per kernel of :data:`GEMM_TILES`; every result is first compared with the library's
own choice (all kernels accumulate in the same order, so the outputs must be equal).
"""
from __future__ import annotations

import argparse

import torch

import intrasm_engine_amd  # noqa: F401  (registers the operators, makes a capture stream current)
from intrasm_engine_amd.interleaving import gemm_tflops, run_non_interleaving
from intrasm_engine_amd.pytorch import ops as pyops
from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.torch import GEMM_TILES


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("-m", type=int, default=1024)
    ap.add_argument("-n", type=int, default=1024)
    ap.add_argument("-k", type=int, default=1024)
    ap.add_argument("--dtype", choices=("bf16", "fp16"), default="bf16")
    ap.add_argument("--trans-b", action="store_true", help="B given as (n, k)")
    ap.add_argument("--repeats", type=int, default=4, help="launches per timed graph")
    args = ap.parse_args(argv)
    dev = torch.device("cuda:0")
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float16
    g = torch.Generator().manual_seed(0)
    a = torch.randn(args.m, args.k, generator=g).to(dev).to(dtype)
    b = torch.randn((args.n, args.k) if args.trans_b else (args.k, args.n), generator=g).to(dev).to(dtype)
    ops = torch.ops.iex_ops
    want = ops.gemm_mfma(a, b, args.trans_b)
    for name, code in GEMM_TILES.items():
        try:
            with pyops.kernel_params(gemm={"tile": code}):
                got = ops.gemm_mfma(a, b, args.trans_b)
                same = torch.equal(got, want)
                ms = run_non_interleaving([lambda: ops.gemm_mfma(a, b, args.trans_b)] * args.repeats) / args.repeats
            print(f"gemm {args.dtype} {'NT' if args.trans_b else 'NN'} {args.m}x{args.n}x{args.k} {name:20s} "
                  f"{ms * 1e3:9.1f} us {gemm_tflops(args.m, args.n, args.k, ms):8.1f} TFLOP/s"
                  f"{'' if same else '   DIFFERS from the default kernel'}", flush=True)
        except Exception as e:  # the reference prints and goes on (tests/profile_cutlass.py:49-53)
            print(f"[skipped] {name}: {e}", flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
