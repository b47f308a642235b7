"""Builds the reference's sample programs against this repository's headers (drop-in check).

The sample sources are compiled where they lie in the reference checkout (nothing is copied);
the executables go to tests/dropin/_bin/, which is git-ignored and travels to the GPU box with
the rest of the tree.  tests/test_gpu_reference_samples.py runs them there: each sample
validates its own GPU result against its own CPU code and prints PASSED or FAILED.

  simple_hgemm, simple_dlrm : compiled as they are, with their own main().
  simple_sgemv, perf_hgemm  : their host code asks the helper header which device it runs on,
                              and that helper (samples/common.hpp:65-80, 113-130) only knows
                              gfx908..gfx942.  The sample is included from a two-line driver that
                              answers "yes" for it and calls the sample's test function (for
                              perf_hgemm at 1024^3 instead of 7168^3, whose CPU check takes minutes).

Validation needs the samples' debug path (no -DNDEBUG).
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REFERENCE_SAMPLES = "/root/reference/samples"
BIN = os.path.join(HERE, "_bin")

DRIVERS = {
    "simple_hgemm": None,
    "simple_dlrm": None,
    "simple_sgemv": """
#include <rocwmma/rocwmma.hpp>
#include "common.hpp"
#define isF32Supported() true
#define main reference_sample_main
#include "simple_sgemv.cpp"
#undef main
int main()
{
    sgemv_test(256, T_BLOCK_Y * ROCWMMA_N, 256, 2.1f, 2.1f);
    return 0;
}
""",
    "perf_hgemm": """
#include <rocwmma/rocwmma.hpp>
#include "common.hpp"
#define isGfx9() true
#define main reference_sample_main
#include "perf_hgemm.cpp"
#undef main
int main()
{
    gemm_test(1024, 1024, 1024, 2, 2);
    return 0;
}
""",
}


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.exists(cand):
            return cand
    return None


def available():
    return os.path.isdir(REFERENCE_SAMPLES) and _hipcc() is not None


def build(verbose=False):
    """Compiles every sample; returns the list of executables.  Raises on a compile error."""
    if not available():
        return []
    os.makedirs(BIN, exist_ok=True)
    out = []
    for name, driver in DRIVERS.items():
        if driver is None:
            src = os.path.join(REFERENCE_SAMPLES, name + ".cpp")
        else:
            src = os.path.join(BIN, name + "_driver.cpp")
            with open(src, "w") as f:
                f.write(driver)
        exe = os.path.join(BIN, name)
        cmd = [_hipcc(), "--offload-arch=gfx950", "-std=c++17", "-O2", "-fopenmp",
               "-I" + os.path.join(ROOT, "include"), "-I" + REFERENCE_SAMPLES,
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
               src, "-o", exe]
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"{name}: hipcc failed\n{res.stdout[-3000:]}")
        if driver is not None:
            os.remove(src)
        if verbose:
            print(exe)
        out.append(exe)
    return out


if __name__ == "__main__":
    if not available():
        print("reference checkout or hipcc not present: nothing built")
        sys.exit(0)
    build(verbose=True)
