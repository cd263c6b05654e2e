"""Compile libhcomm_gfx.so for gfx950 (hipcc cross-compiles without a GPU)."""
import os
import subprocess

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB = os.path.join(CSRC, "libhcomm_gfx.so")


def build(force: bool = True, jobs: int = 8) -> str:
    """Run make in csrc/.  With force, every object is rebuilt."""
    cmd = ["make", "-C", CSRC, "-j%d" % jobs]
    if force:
        cmd.insert(1, "-B")
    subprocess.run(cmd, check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if not os.path.exists(LIB):
        raise RuntimeError("build finished but %s is missing" % LIB)
    return LIB


if __name__ == "__main__":
    print(build())
