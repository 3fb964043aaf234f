"""Compile the gfx950 attention library (gvirt_amd/csrc/*.hip) into gvirt_amd/libxlite_hip.so.

Usage: python -m gvirt_amd.build [--if-stale] [--verbose]
hipcc cross-compiles for gfx950 without a GPU; the .so is built in-tree and loaded with ctypes.
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libxlite_hip.so")
OBJ_DIR = os.path.join(CSRC, "build")

# packed fp32 ops are switched off on purpose (device code only); the host pass of hipcc does
# not know the feature and says so, which is harmless
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-inline-asm", "-ffp-contract=off"]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _stale() -> bool:
    if not os.path.exists(OUT):
        return True
    newest = max(os.path.getmtime(p) for p in sources() + glob.glob(os.path.join(CSRC, "*.h")) +
                 [os.path.join(HERE, "..", "include", "xlite_hip.h")])
    return newest > os.path.getmtime(OUT)


def build(force: bool = True, verbose: bool = False) -> str:
    if not force and not _stale():
        return OUT
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
        cmd = [hipcc] + FLAGS + ["-c", src, "-o", obj]
        if verbose:
            cmd.insert(1, "-Rpass-analysis=kernel-resource-usage")
        r = subprocess.run(cmd, capture_output=True, text=True)
        out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                        if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
        return obj, out

    with ThreadPoolExecutor(max_workers=min(8, len(sources()))) as ex:
        results = list(ex.map(compile_one, sources()))
    if verbose:
        for _, out in results:
            print(out)
    objs = [o for o, _ in results]
    tmp = OUT + ".tmp"
    subprocess.check_call([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs)
    os.replace(tmp, OUT)
    return OUT


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv, verbose="--verbose" in sys.argv))
