"""Compile ``libiex_hip.so`` for gfx950:  ``python intrasm_engine_amd/csrc/build.py``
(run it as a script: importing the package needs the library to exist already)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def build(force: bool = True, jobs: int = 8) -> str:
    cmd = ["make", "-C", HERE, f"-j{jobs}"]
    if force:
        cmd.append("-B")
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 target feature and says so: harmless
    lines = [ln for ln in proc.stdout.splitlines() if "packed-fp32-ops" not in ln]
    if proc.returncode != 0:
        sys.stderr.write("\n".join(lines) + "\n")
        raise RuntimeError("building libiex_hip.so failed")
    out = os.path.normpath(os.path.join(HERE, "..", "libiex_hip.so"))
    assert os.path.exists(out)
    return out


if __name__ == "__main__":
    print(build())
