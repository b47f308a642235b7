"""Drop-in proof for the header API: the reference's own sample kernels compile unchanged.

The four samples the hot path is made of (samples/simple_hgemm.cpp, perf_hgemm.cpp,
simple_dlrm.cpp, simple_sgemv.cpp in the reference tree) are compiled for gfx950, device and
host pass, with this repository's include/ in front of the include path.  The dependency list of
each compilation must contain this repository's rocwmma headers and none from the reference's
library/ directory or from the rocWMMA that ships with the toolchain.

Needs the reference checkout (present only on the development container) and hipcc; skipped
where either is missing.  Nothing is run, so no GPU is needed.
"""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE = "/root/reference"
SAMPLES = ["simple_hgemm", "perf_hgemm", "simple_dlrm", "simple_sgemv"]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.exists(cand):
            return cand
    return None


@pytest.mark.parametrize("sample", SAMPLES)
def test_reference_sample_compiles_against_these_headers(sample, tmp_path):
    src = os.path.join(REFERENCE, "samples", sample + ".cpp")
    hipcc = _hipcc()
    if not os.path.exists(src):
        pytest.skip("reference checkout not present")
    if hipcc is None:
        pytest.skip("hipcc not present")
    obj = tmp_path / (sample + ".o")
    dep = tmp_path / (sample + ".d")
    cmd = [hipcc, "--offload-arch=gfx950", "-std=c++17", "-O1",
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(REFERENCE, "samples"),
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-Wno-unused-command-line-argument",
           "-MD", "-MF", str(dep), "-c", src, "-o", str(obj)]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert res.returncode == 0, res.stdout[-3000:]
    assert obj.exists() and obj.stat().st_size > 0
    deps = " ".join(p.read_text() for p in tmp_path.glob("*.d"))
    ours = os.path.join(ROOT, "include", "rocwmma", "rocwmma.hpp")
    assert ours in deps, "the sample did not pick up this repository's rocwmma.hpp"
    assert os.path.join(REFERENCE, "library") not in deps
    assert "/opt/rocm/include/rocwmma" not in deps
