"""The xformers-style SpMM sweep harness (reference 3rdparty/MyXformers/benchmarks/benchmark_spmm.py):
the shape lists are the reference's, and a quick run checks every product against a dense batched
product before timing it."""
import pytest

pytestmark = pytest.mark.gpu


def test_shape_lists_are_the_references():
    from intrasm_engine_amd.benchmarks import benchmark_spmm as bs
    assert bs.SWIN_T == [((96, 3136, 32), 0.9844), ((192, 784, 32), 0.9375), ((384, 196, 32), 0.75), ((768, 49, 32), 0.0)]
    assert len(bs.BASIC) == 4 * 8 and bs.BASIC[0] == ((32, 1024, 32), 0.90) and bs.BASIC[-1] == ((8, 4096, 128), 0.999)
    assert len(bs.VIT) == 4 * 7 and bs.VIT[0] == ((192, 785, 64), 0.70) and bs.VIT[-1] == ((384, 197, 64), 0.97)


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
def test_quick_sweep_runs_and_checks(dev, capsys, dtype):
    from intrasm_engine_amd.benchmarks import benchmark_spmm as bs
    assert bs.main(["--quick", "--dtype", dtype]) == 0
    lines = [ln for ln in capsys.readouterr().out.splitlines() if ln.startswith("spmm B=")]
    assert len(lines) == len(bs.QUICK)
    assert all("GFLOP/s" in ln and "GB/s" in ln for ln in lines)
    # an all-kept pattern (sparsity 0) has m * k nonzeros
    assert f"nnz={49 * 32:8d}" in lines[-1]
