"""Build oracle/brute.c into oracle/libbrute.so with gcc (test infrastructure only).

The reference's own implementation of this path is AscendC device code whose build needs
the CANN toolkit (xlite/CMakeLists.txt:126-133), so there is no `oracle/_ref` build: the
brute-force restatement below is what pins the PyTorch oracle.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "brute.c")
OUT = os.path.join(HERE, "libbrute.so")


def build(force: bool = True) -> str:
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= os.path.getmtime(SRC):
        return OUT
    cmd = ["gcc", "-O2", "-std=c11", "-ffp-contract=off", "-fPIC", "-shared", SRC, "-o", OUT, "-lm"]
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
