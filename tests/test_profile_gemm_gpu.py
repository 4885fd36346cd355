"""The GEMM tile sweep tool (counterpart of the reference's tests/profile_cutlass.py): one line per
kernel, none skipped, none differing from the library's own choice."""
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("extra", [[], ["--trans-b", "--dtype", "fp16"]])
def test_profile_gemm_lists_every_kernel(dev, capsys, extra):
    from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.torch import GEMM_TILES
    from intrasm_engine_amd.tuning.profile_gemm import main
    assert main(["-m", "384", "-n", "264", "-k", "200", "--repeats", "2", *extra]) == 0
    lines = [ln for ln in capsys.readouterr().out.splitlines() if ln.startswith("gemm ")]
    assert len(lines) == len(GEMM_TILES)
    for name, line in zip(GEMM_TILES, lines):
        assert f" {name} " in line and "TFLOP/s" in line and "DIFFERS" not in line
