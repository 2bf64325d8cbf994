"""Build libgs355.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m landmarksystem_amd.csrc.build

hipcc cross-compiles without a GPU.  Flags:
  --offload-arch=gfx950           the only target; no other code objects
  -packed-fp32-ops disabled       packed FP32 VALU forms are not generated
  -ffp-contract=off (preprocess)  the arithmetic that feeds the integer
                                  pipeline (depth bits, radius, tile rectangle)
                                  is defined as unfused IEEE fp32 operations
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
INCLUDE = os.path.join(REPO, "include")
OUT = os.path.join(os.path.dirname(HERE), "libgs355.so")
OBJ_DIR = os.path.join(HERE, "build")

COMMON = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", INCLUDE, "-I", HERE, "-Wall", "-Wno-unused-command-line-argument",
]

# (source, extra flags)
SOURCES = [
    ("gs355_abi.hip", []),
    ("gs355_preprocess.hip", ["-ffp-contract=off"]),
    ("gs355_scan.hip", []),
    ("gs355_sort.hip", []),
    ("gs355_bin.hip", []),
    ("gs355_gather.hip", []),
    ("gs355_decode.hip", []),
    ("gs355_blend.hip", []),
    ("gs355_backward.hip", []),
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(job):
    src, extra = job
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *COMMON, *extra, "-c", os.path.join(HERE, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, " ".join(cmd), res.stderr))
    warn = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    return obj, warn


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        results = list(pool.map(_compile, SOURCES))
    objs = [o for o, _ in results]
    if verbose:
        for _, w in results:
            if w:
                print(w, file=sys.stderr)
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (" ".join(cmd), res.stderr))
    return OUT


if __name__ == "__main__":
    print(build())
