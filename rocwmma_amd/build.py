"""Builds rocwmma_amd/librocwmma_amd.so, the product library, and rocwmma_amd/librocwmma_amd_aux.so,
the test and benchmark support library (gfx950 only) from rocwmma_amd/csrc/*.hip with hipcc.

The libraries are built in-tree; tests, the smoke check and the benchmark load what is there and
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
AUX_LIB_PATH = os.path.join(HERE, "librocwmma_amd_aux.so")

SOURCES = ["api.hip", "gemm_wave_tile.hip", "gemm_blocked.hip", "gemm_streamk.hip", "gemm_skinny.hip", "gemm_mx.hip", "gemm_fused.hip", "gemv.hip", "dlrm.hip", "dlrm_f32.hip", "dlrm_general.hip"]
# test and benchmark support: fragment-API self-test kernels and measurement probes
AUX_SOURCES = ["aux_api.hip", "selftest.hip", "mfma_ceiling.hip", "mfma_streams.hip", "stream_ceiling.hip"]

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


def _link(path, objs):
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", path] + objs
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout[-4000:]}")


def build_library(force=True, jobs=None, only=None):
    """Compile every translation unit and link both shared libraries.  Returns the product
    library's path.  `only`: a list of source names to recompile (the other objects are reused)."""
    if not force and os.path.exists(LIB_PATH) and os.path.exists(AUX_LIB_PATH):
        return LIB_PATH
    os.makedirs(OBJ_DIR, exist_ok=True)
    todo = [s for s in SOURCES + AUX_SOURCES if only is None or s in only]
    jobs = jobs or min(len(todo), int(os.environ.get("MAX_JOBS", "8")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=max(jobs, 1)) as pool:
        list(pool.map(_compile, todo))
    obj = lambda s: os.path.join(OBJ_DIR, os.path.splitext(s)[0] + ".o")
    _link(LIB_PATH, [obj(s) for s in SOURCES])
    _link(AUX_LIB_PATH, [obj(s) for s in AUX_SOURCES])
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force=True, only=sys.argv[1:] or None))
    sys.exit(0)
