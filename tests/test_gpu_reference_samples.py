"""Drop-in check on the GPU: the reference's sample programs, built against this repository's
headers by tests/dropin/build_samples.py, run and validate themselves (each sample compares its
GPU result with its own CPU code and prints PASSED or FAILED).

The executables are built on the development machine (where the reference checkout is) and
travel with the tree; where they are absent the tests fail (ROCWMMA_AMD_REQUIRE_DROPIN=0 skips them instead)."""
import os
import subprocess

import pytest

from util import dropin_missing

pytestmark = pytest.mark.gpu

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dropin", "_bin")
# sample -> number of self-checks it prints
# (the f32 and f64 samples are not among the workloads the library is built for; they compile and
# pass as they are and are kept as further evidence for the header API)
SAMPLES = {"simple_hgemm": 1, "perf_hgemm": 1, "simple_sgemv": 1, "simple_dlrm": 3, "simple_sgemm": 1, "perf_sgemm": 1,
           "simple_dgemm": 1, "perf_dgemm": 1, "simple_dgemv": 1}


@pytest.mark.parametrize("sample", sorted(SAMPLES))
def test_reference_sample_runs_and_validates_itself(sample):
    exe = os.path.join(BIN, sample)
    if not os.path.exists(exe):
        dropin_missing("sample executables")
    res = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
    tail = res.stdout[-1500:]
    assert res.returncode == 0, tail
    assert "FAILED" not in res.stdout, tail
    assert res.stdout.count("PASSED") == SAMPLES[sample], tail
