"""Drop-in checks on the GPU, part 1: the reference's cooperative, LDS double-buffered multi-block GEMM test
kernel (test/gemm/gemm_PGR1_LB2_MP0_MB_CP/device/kernel_device_func.hpp in the reference tree) and its
two GEMM test kernels without LDS (test/gemm/gemm_PGR0_LB0_MP0_{MB,SB}_NC/device/kernel_device_func.hpp),
compiled unchanged against this repository's headers, over a matrix of element types, block sizes,
A/B/C layouts, LDS layouts, cooperation levels (block / wave / workgroup), LDS mappings
(NT / TN / register file), blocks per wave and thread-block shapes.

Operands are small integers, so every case must match a plain CPU loop bit for bit whatever the
accumulation order.

Part 2: the device kernels of the reference's unit tests that use only the public API
(test/unit/*/device/*.hpp: load / store, cooperative load / store, fill, load and store contamination,
MappingUtil coordinate maps and their overrides), over the reference's block sizes
(16..256 x 8..256, test/unit/unit_test_params.hpp:89-141), both layouts, nine element types and six
thread-block shapes; each must move exactly the elements its contract says (tests/dropin/unit_kernels.cpp).

Part 3: the reference's DLRM dot-interaction test kernels (test/dlrm/device/dlrm_dot_{fwd,bwd}.hpp and the
LDS variants dlrm_dot_{fwd,bwd}_lds.hpp, which keep fragments in LDS as a register file and, in the backward
pass, reinterpret cooperatively loaded fragments as register-file fragments), for f16 and f32, tiles of 16
and 32 and the reference's problem sizes; inputs are -1, 0, 1 so results must equal a CPU loop exactly
(tests/dropin/dlrm_kernels.cpp).

tests/dropin/build_samples.py enumerates the cases and builds the executables
on the development machine (where the reference checkout is); they travel with the tree.  Where
they are absent the tests fail (ROCWMMA_AMD_REQUIRE_DROPIN=0 skips them instead)."""
import os
import re
import subprocess
import sys

import pytest

from util import dropin_missing

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "dropin"))
import build_samples  # noqa: E402

BIN = os.path.join(HERE, "dropin", "_bin")
# Cases the reference kernels' own guards reject, per executable (build_samples.py deals the case lists over
# MATRIX_UNITS executables; the counts change only with those lists)
COOP_GEMM_REJECTED = [13, 16, 12, 16, 10, 12, 0, 0]
UNIT_KERNELS_REJECTED = [11, 11, 11, 15, 12, 15, 11, 14]


@pytest.mark.parametrize("unit", range(build_samples.MATRIX_UNITS))
def test_reference_cooperative_gemm_kernel_matrix(unit):
    exe = os.path.join(BIN, f"coop_gemm_matrix_{unit}")
    if not os.path.exists(exe):
        dropin_missing("kernel-matrix executables")
    expected = len(build_samples.coop_gemm_units()[unit][1])
    res = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
    tail = res.stdout[-2000:]
    failed = [line for line in res.stdout.splitlines() if line.startswith("FAILED")]
    assert not failed, "\n".join(failed[:10])
    assert res.returncode == 0, tail
    summary = re.search(r"SUMMARY: (\d+) passed, (\d+) failed, (\d+) skipped", res.stdout)
    assert summary, tail
    passed, nfailed, skipped = map(int, summary.groups())
    assert nfailed == 0 and passed + skipped == expected, tail
    # the kernel's own guard rejects some cases (register budget; the register-file LDS mapping
    # needs a single wave): exactly these many per executable, so that a case that stops running shows
    assert skipped == COOP_GEMM_REJECTED[unit], (skipped, COOP_GEMM_REJECTED[unit], tail)


@pytest.mark.parametrize("unit", range(build_samples.MATRIX_UNITS))
def test_reference_unit_test_kernels(unit):
    exe = os.path.join(BIN, f"unit_kernels_{unit}")
    if not os.path.exists(exe):
        dropin_missing("unit-kernel executables")
    expected = len(build_samples.unit_kernel_units()[unit][1])
    res = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
    tail = res.stdout[-2000:]
    failed = [line for line in res.stdout.splitlines() if line.startswith("FAILED")]
    assert not failed, "\n".join(failed[:10])
    assert res.returncode == 0, tail
    summary = re.search(r"SUMMARY: (\d+) passed, (\d+) failed, (\d+) skipped", res.stdout)
    assert summary, tail
    passed, nfailed, skipped = map(int, summary.groups())
    assert nfailed == 0 and passed + skipped == expected, tail
    # the kernels' own guard rejects blocks that exceed a wave's register budget (e.g. 256 x 256 f64):
    # exactly these many per executable
    assert skipped == UNIT_KERNELS_REJECTED[unit], (skipped, UNIT_KERNELS_REJECTED[unit], tail)


def test_reference_dlrm_test_kernels():
    exe = os.path.join(BIN, "dlrm_kernels")
    if not os.path.exists(exe):
        dropin_missing("DLRM kernel executable")
    res = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
    tail = res.stdout[-2000:]
    failed = [line for line in res.stdout.splitlines() if line.startswith("FAILED")]
    assert not failed, "\n".join(failed[:10])
    assert res.returncode == 0, tail
    summary = re.search(r"SUMMARY: (\d+) passed, (\d+) failed, (\d+) skipped", res.stdout)
    assert summary, tail
    # 2 element types x 2 tile sizes x 4 problem sizes x {forward, backward} x {plain, LDS}
    assert tuple(map(int, summary.groups())) == (64, 0, 0), tail
