"""Builds rocwmma_amd/librocwmma_amd.so (gfx950 only) from rocwmma_amd/csrc/*.hip with hipcc.

The library is built in-tree; tests, the smoke check and the benchmark load what is there and
only build when nothing is."""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "librocwmma_amd.so")

SOURCES = ["api.hip", "gemm_wave_tile.hip", "gemm_blocked.hip", "gemm_skinny.hip", "gemv.hip", "dlrm.hip", "selftest.hip"]

# -packed-fp32-ops off: packed FP32 instructions are not generated for this target build.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-DNDEBUG",
    "-I" + os.path.join(ROOT, "include"),
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-pass-failed",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc()] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout[-4000:]}")
    return obj


def build_library(force=True, jobs=None):
    """Compile every translation unit and link the shared library.  Returns its path."""
    if not force and os.path.exists(LIB_PATH):
        return LIB_PATH
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = jobs or min(len(SOURCES), int(os.environ.get("MAX_JOBS", "8")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout[-4000:]}")
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force=True))
    sys.exit(0)
