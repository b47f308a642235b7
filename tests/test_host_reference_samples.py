"""Drop-in proof for the header API: the reference's own sample kernels compile unchanged.

The four samples the hot path is made of (samples/simple_hgemm.cpp, perf_hgemm.cpp,
simple_dlrm.cpp, simple_sgemv.cpp in the reference tree) and its f32 / f64 samples
(simple_sgemm.cpp, perf_sgemm.cpp, simple_dgemm.cpp, perf_dgemm.cpp, simple_dgemv.cpp) are compiled for gfx950, device and
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
SAMPLES = ["simple_hgemm", "perf_hgemm", "simple_dlrm", "simple_sgemv", "simple_sgemm", "perf_sgemm",
           "simple_dgemm", "perf_dgemm", "simple_dgemv"]


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


# The reference's own test kernels (device side only; their GTest hosts are not involved).  They
# gate their bodies on the architecture identifiers they know, so the device pass is told to report
# gfx942's identifier (ROCWMMA_AMD_REPORT_ARCH_ID); nothing else is changed.
TEST_KERNEL_UNITS = {
    "unit_load_store_fill_contamination_coop": """
#include <hip/hip_runtime.h>
#include "load_store_matrix_sync_test/device/load_store_matrix_sync.hpp"
#include "fill_fragment_test/device/fill_fragment.hpp"
#include "contamination_test/device/load_contamination.hpp"
#include "contamination_test/device/store_contamination.hpp"
#include "load_store_matrix_coop_sync_test/device/load_store_matrix_coop_sync.hpp"
namespace rocwmma {
template __global__ void LoadStoreMatrixSyncA<32, 16, float16_t, row_major>(uint32_t, uint32_t, float16_t const*, float16_t*, uint32_t, float16_t, float16_t);
template __global__ void LoadStoreMatrixSyncA<256, 8, float32_t, col_major>(uint32_t, uint32_t, float32_t const*, float32_t*, uint32_t, float32_t, float32_t);
template __global__ void LoadStoreMatrixSyncB<64, 32, int8_t, col_major>(uint32_t, uint32_t, int8_t const*, int8_t*, uint32_t, int8_t, int8_t);
template __global__ void LoadStoreMatrixSyncAcc<32, 32, float32_t, row_major>(uint32_t, uint32_t, float32_t const*, float32_t*, uint32_t, float32_t, float32_t);
}
""",
    "dlrm_test_kernels": """
#include <hip/hip_runtime.h>
#include <rocwmma/rocwmma.hpp>
#include "dlrm/device/dlrm_dot_fwd.hpp"
#include "dlrm/device/dlrm_dot_bwd.hpp"
namespace rocwmma {
template __global__ void dlrmDotFwd<float16_t, 16>(const float16_t* __restrict, float16_t* __restrict, float*, uint, uint, uint, uint, uint, uint);
template __global__ void trilReconstruct<float16_t>(const float16_t* __restrict, float16_t* __restrict, uint, uint, uint, uint, uint);
template __global__ void dlrmDotBwd<float16_t, 16>(const float16_t* __restrict, const float16_t* __restrict, float16_t* __restrict, float16_t* __restrict, float16_t* __restrict, uint, uint, uint, uint, uint, uint);
}
""",
    "gemm_single_block_test_kernel": """
#include <hip/hip_runtime.h>
#include <iostream>
#include <rocwmma/rocwmma.hpp>
#include "gemm/gemm_PGR0_LB0_MP0_SB_NC/device/kernel_device_func.hpp"
namespace rocwmma {
template __global__ void gemm_PGR0_LB0_MP0_SB_NC<32, 32, 16, float16_t, float32_t, float32_t, row_major, col_major, row_major, row_major, 128, 2, 64, 0x942>(uint32_t, uint32_t, uint32_t, float16_t const*, float16_t const*, float32_t const*, float32_t*, uint32_t, uint32_t, uint32_t, uint32_t, float32_t, float32_t);
template __global__ void gemm_PGR0_LB0_MP0_SB_NC<16, 16, 64, int8_t, int32_t, int32_t, col_major, row_major, row_major, row_major, 64, 4, 64, 0x942>(uint32_t, uint32_t, uint32_t, int8_t const*, int8_t const*, int32_t const*, int32_t*, uint32_t, uint32_t, uint32_t, uint32_t, int32_t, int32_t);
}
""",
    "gemm_cooperative_lds_test_kernel": """
#include <hip/hip_runtime.h>
#include <iostream>
#include <rocwmma/rocwmma.hpp>
#include <rocwmma/rocwmma_coop.hpp>
#include <rocwmma/rocwmma_transforms.hpp>
#include "gemm_PGR1_LB2_MP0_MB_CP/device/kernel_device_func.hpp"
namespace rocwmma {
template __global__ void gemm_PGR1_LB2_MP0_MB_CP<32, 32, 16, float16_t, float32_t, float32_t, row_major, col_major, row_major, row_major, col_major, CooperativeGemm::WorkgroupLevel::LdsNT, 2, 2, 128, 2, 64, 0x942>(uint32_t, uint32_t, uint32_t, float16_t const*, float16_t const*, float32_t const*, float32_t*, uint32_t, uint32_t, uint32_t, uint32_t, float32_t, float32_t);
template __global__ void gemm_PGR1_LB2_MP0_MB_CP<16, 16, 64, int8_t, int32_t, int32_t, col_major, row_major, col_major, col_major, row_major, CooperativeGemm::BlockLevel::LdsTN, 2, 4, 64, 4, 64, 0x942>(uint32_t, uint32_t, uint32_t, int8_t const*, int8_t const*, int32_t const*, int32_t*, uint32_t, uint32_t, uint32_t, uint32_t, int32_t, int32_t);
template __global__ void gemm_PGR1_LB2_MP0_MB_CP<16, 16, 128, float8_t, float32_t, float32_t, row_major, col_major, row_major, row_major, row_major, CooperativeGemm::WaveLevel::LdsNT, 2, 2, 128, 2, 64, 0x942>(uint32_t, uint32_t, uint32_t, float8_t const*, float8_t const*, float32_t const*, float32_t*, uint32_t, uint32_t, uint32_t, uint32_t, float32_t, float32_t);
// pieces of the library surface that kernel's helpers lean on
static_assert(Waitcnt<3, 2>::encoded == (3 | (2 << 8) | (7 << 4)), "s_waitcnt encoding");
static_assert(std::is_same<WaitVmcnt<5>, Waitcnt<5, 0>>::value && std::is_same<WaitLgkmcnt<1>, Waitcnt<0, 1>>::value, "");
static_assert(std::is_same<DataLayout::Array1d<col_major>, GetDataLayout_t<fragment<matrix_b, 16, 16, 16, float16_t, col_major>>>::value, "");
static_assert(DataLayout::RowMajor::fromMatrixCoord(make_coord2d(3u, 5u), 100u) == 305u && DataLayout::ColMajor::fromMatrixCoord(make_coord2d(3u, 5u), 100u) == 503u, "");
static_assert(GetCoopIOConfig_t<fragment<matrix_a, 128, 16, 16, float16_t, row_major>, 4>::IOTraits::IOCount * 4u == GetCoopIOConfig_t<fragment<matrix_a, 128, 16, 16, float16_t, row_major>>::IOTraits::IOCount, "");
static_assert(detail::WaveSpace<128, 2>::workgroupDim() == make_coord2d(2u, 2u), "compile-time workgroup shape");
constexpr bool sameText(const char* a, const char* b) { return *a == *b && (*a == 0 || sameText(a + 1, b + 1)); }
static_assert(sameText(dataTypeToString<float16_t>(), "f16") && sameText(dataTypeToString<bfloat8_t>(), "bf8") && sameText(dataTypeToString<row_major>(), "T") && sameText(dataTypeToString<col_major>(), "N"), "");
}
""",
}


@pytest.mark.parametrize("unit", sorted(TEST_KERNEL_UNITS))
def test_reference_test_kernels_compile_against_these_headers(unit, tmp_path):
    tests_dir = os.path.join(REFERENCE, "test")
    hipcc = _hipcc()
    if not os.path.isdir(tests_dir):
        pytest.skip("reference checkout not present")
    if hipcc is None:
        pytest.skip("hipcc not present")
    src = tmp_path / (unit + ".cpp")
    src.write_text(TEST_KERNEL_UNITS[unit])
    obj = tmp_path / (unit + ".o")
    dep = tmp_path / (unit + ".d")
    cmd = [hipcc, "--offload-arch=gfx950", "-std=c++17", "-O1", "-DROCWMMA_AMD_REPORT_ARCH_ID=0x942",
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(tests_dir, "unit"), "-I" + tests_dir,
           "-I" + os.path.join(tests_dir, "gemm"),
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
           "-MD", "-MF", str(dep), "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert res.returncode == 0, res.stdout[-3000:]
    deps = " ".join(p.read_text() for p in tmp_path.glob("*.d"))
    assert os.path.join(ROOT, "include", "rocwmma", "rocwmma.hpp") in deps
    assert os.path.join(REFERENCE, "library") not in deps
    assert "/opt/rocm/include/rocwmma" not in deps
