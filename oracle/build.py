"""Compile the C oracle (oracle/gs_oracle.c, oracle/gs_oracle_backward.c) into oracle/libgs_oracle.so with gcc.

Test infrastructure only: the shipped library never links or loads this.
There is no buildable reference source for this path (the rasterizer is an
empty third-party submodule in the reference tree), so no oracle/_ref exists.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRCS = [os.path.join(HERE, "gs_oracle.c"), os.path.join(HERE, "gs_oracle_backward.c")]
OUT = os.path.join(HERE, "libgs_oracle.so")

# -ffp-contract=off: the integer pipeline (depth bits, radius, tile rectangle)
# is defined by unfused IEEE fp32 operations in the written order.
FLAGS = ["-O2", "-ffp-contract=off", "-fno-fast-math", "-fopenmp", "-shared", "-fPIC", "-Wall", "-Wextra"]


def build(force: bool = True) -> str:
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= max(os.path.getmtime(s) for s in SRCS):
        return OUT
    cmd = ["gcc", *FLAGS, "-o", OUT, *SRCS, "-lm"]
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
