"""Row kernel against the row-length schedule (SpMM family 11) on the 15 cells of the fp32 headline sweep
(A 4096 x 4096 at 70 ... 98 % sparsity, B 4096 x {64, 128, 256}).

Per cell: what the library picks without the row-length histogram (the row kernel with wavefronts per row from the mean
row length, family 1; the fp32 matrix-core kernel on the densest cell), the
row-length schedule with the chunk budget the library would choose, and the same with the budget forced to 1, 2, 4, 8
and 16 chunks of 64 nonzeros per wavefront; then what the operator picks by itself.  Times are microseconds per launch:
200 launches in one graph, median of 5 replays.

    python3 -m intrasm_engine_amd.benchmarks.spmm_rows_by_length [f32|f16]
"""
import sys

import numpy as np
import torch

from intrasm_engine_amd import _lib, workloads as W
from intrasm_engine_amd.pytorch import ops as pyops

ops = torch.ops.iex_ops


def time_us(fn, iters=200):
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(iters):
            fn()
    g.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ts = []
    for _ in range(5):
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b) / iters * 1e3)
    return float(np.median(ts))


def main():
    dev = torch.device("cuda:0")
    dtype = torch.float16 if len(sys.argv) > 1 and sys.argv[1] == "f16" else torch.float32
    f = ops.spmm_sputnik_reuse_weight if dtype == torch.float32 else ops.spmm_sputnik_reuse_weight_half
    print(f"{'cell':>12} {'family 1':>9} {'family 11':>10} {'ratio':>6}   chunks per wavefront forced to 1 / 2 / 4 / 8 / 16      operator", flush=True)
    total = {"row": 0.0, "rows_by_length": 0.0, "operator": 0.0}
    for s in W.C2_SPARSITIES:
        c = W.config2_matrix(s)
        ri = torch.from_numpy(c.row_indices).to(dev)
        v = torch.from_numpy(c.values).to(dev).to(dtype)
        ro = torch.from_numpy(c.row_offsets).to(dev)
        ci = torch.from_numpy(c.column_indices).to(dev)
        if dtype == torch.float16:
            ci = ci.to(torch.int16)
        pyops.prepare_pattern(ro, ci, c.k, tables=False)
        ci_plain = ci.clone()                           # the same pattern, known to be canonical, row lengths unknown:
        pyops._set_note(ro, ci_plain, c.k, 0, None)     # calls on it cannot take the row-length schedule
        for n in W.C2_NS:
            b = torch.from_numpy(W.config2_dense(n)).to(dev).to(dtype)
            call = lambda: f(b, ri, v, ro, ci, c.m)
            t_row = time_us(lambda: f(b, ri, v, ro, ci_plain, c.m))
            with pyops.kernel_params(spmm={"force_variant": 11}):
                call()
                trail = _lib.last_kernels()
                t_new = time_us(call)
            forced = []
            for code in (1, 2, 3, 4, 5):
                with pyops.kernel_params(spmm={"force_variant": 11, "force_rpw": code}):
                    forced.append(time_us(call))
            call()
            picked = _lib.last_kernels().split("<")[0]
            t_op = time_us(call)
            total["row"] += t_row
            total["rows_by_length"] += t_new
            total["operator"] += t_op
            print(f"{s:>6}, {n:>4} {t_row:9.2f} {t_new:10.2f} {t_new / t_row:6.2f}   " + " / ".join(f"{t:6.1f}" for t in forced) +
                  f"   {t_op:7.2f} {picked}   [{trail[trail.find('('):]}]", flush=True)
    print("sweep: " + ", ".join(f"{k} {t:.1f} us" for k, t in total.items()), flush=True)


if __name__ == "__main__":
    main()
