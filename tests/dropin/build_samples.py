"""Builds the reference's sample programs and its cooperative GEMM test kernel against this
repository's headers (drop-in check).

The sample sources are compiled where they lie in the reference checkout (nothing is copied);
the executables go to tests/dropin/_bin/, which is git-ignored and travels to the GPU box with
the rest of the tree.  tests/test_gpu_reference_samples.py runs them there: each sample
validates its own GPU result against its own CPU code and prints PASSED or FAILED.

  simple_hgemm, simple_dlrm : compiled as they are, with their own main().
  simple_sgemv, perf_hgemm, simple_sgemm, perf_sgemm, simple_dgemm, perf_dgemm, simple_dgemv (the f32
                              and f64 samples are outside the workloads this library is built for
                              and come along with the header API)
                            : their host code asks the helper header which device it runs on,
                              and that helper (samples/common.hpp:65-80, 113-130) only knows
                              gfx908..gfx942.  The sample is included from a two-line driver that
                              answers "yes" for it and calls the sample's test function (for
                              perf_hgemm at 1024^3 instead of 7168^3, whose CPU check takes minutes).

Validation needs the samples' debug path (no -DNDEBUG).

Kernel matrix: the reference's cooperative LDS double-buffered GEMM test kernel
(test/gemm/gemm_PGR1_LB2_MP0_MB_CP/device/kernel_device_func.hpp) and its two GEMM test kernels
without LDS (test/gemm/gemm_PGR0_LB0_MP0_{MB,SB}_NC/device/kernel_device_func.hpp) are instantiated by
tests/dropin/coop_gemm_matrix.cpp (host side only, written here) over the case list that
coop_gemm_cases() enumerates: the axes of the reference's own test matrix
(test/gemm/gemm_common_test_params.hpp:44-330, test/gemm/gemm_PGR1_LB2_MP0_MB_CP/test/*):
element types, block sizes, A/B/C layouts, LDS layout, cooperation level and LDS mapping, blocks
per wave, thread-block shape.  tests/test_gpu_reference_kernel_matrix.py runs the executables.

Unit-test kernels and DLRM kernels: tests/dropin/unit_kernels.cpp and tests/dropin/dlrm_kernels.cpp are
the host sides for the device kernels under test/unit/*/device and test/dlrm/device.
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
    "simple_sgemm": """
#include <rocwmma/rocwmma.hpp>
#include "common.hpp"
#define isF32Supported() true
#define main reference_sample_main
#include "simple_sgemm.cpp"
#undef main
int main()
{
    gemm_test(256, 256, 256, 2.1f, 2.1f);
    return 0;
}
""",
    "perf_sgemm": """
#include <rocwmma/rocwmma.hpp>
#include "common.hpp"
#define isF32Supported() true
#define isGfx9() true
#define main reference_sample_main
#include "perf_sgemm.cpp"
#undef main
int main()
{
    gemm_test(1024, 1024, 1024, 2, 2);
    return 0;
}
""",
    "simple_dgemm": """
#include <rocwmma/rocwmma.hpp>
#include "common.hpp"
#define isF64Supported() true
#define main reference_sample_main
#include "simple_dgemm.cpp"
#undef main
int main()
{
    gemm_test(256, 256, 256, 2.1, 2.1);
    return 0;
}
""",
    "perf_dgemm": """
#include <rocwmma/rocwmma.hpp>
#include "common.hpp"
#define isF64Supported() true
#define isGfx9() true
#define main reference_sample_main
#include "perf_dgemm.cpp"
#undef main
int main()
{
    gemm_test(1024, 1024, 1024, 2, 2);
    return 0;
}
""",
    "simple_dgemv": """
#include <rocwmma/rocwmma.hpp>
#include "common.hpp"
#define isF64Supported() true
#define main reference_sample_main
#include "simple_dgemv.cpp"
#undef main
int main()
{
    dgemv_test(256, T_BLOCK_Y * ROCWMMA_N, 256, 2.1, 2.1);
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


REFERENCE_TESTS = "/root/reference/test"
MATRIX_UNITS = 8  # translation units (and executables) the case list is dealt over

# (input, output, compute) -> block sizes (BlockM = BlockN, BlockK) a matrix instruction exists for
_MATRIX_TYPES = [
    (("f16", "f32", "f32"), [(16, 16), (16, 32), (16, 64), (32, 8), (32, 16), (32, 32)]),
    (("f16", "f16", "f32"), [(16, 32), (32, 16)]),
    (("bf16", "f32", "f32"), [(16, 16), (16, 32), (32, 8), (32, 16)]),
    (("bf16", "bf16", "f32"), [(16, 32), (32, 16)]),
    (("f32", "f32", "f32"), [(16, 4), (16, 8), (32, 2), (32, 4)]),
    (("i8", "i32", "i32"), [(16, 32), (16, 64), (32, 16), (32, 32)]),
    (("f8", "f32", "f32"), [(16, 32), (16, 64), (16, 128), (32, 16), (32, 64)]),
    (("bf8", "f32", "f32"), [(16, 32), (16, 128), (32, 16), (32, 64)]),
    (("f64", "f64", "f64"), [(16, 4), (16, 8), (16, 16)]),
    (("h16", "f32", "f32"), [(16, 32), (32, 16)]),
    (("h16", "h16", "f32"), [(16, 16), (32, 8)]),
    # narrow outputs and 16-bit compute types (test/gemm/gemm_common_test_params.hpp:51-56,88-113)
    (("i8", "i8", "i32"), [(16, 64), (32, 32)]),
    (("f16", "f16", "f16"), [(16, 32), (32, 16)]),
    (("bf16", "bf16", "bf16"), [(16, 32), (32, 8)]),
    (("h16", "h16", "h16"), [(16, 16), (32, 16)]),
]
_CONFIGS = ["Block::LdsNT", "Block::LdsTN", "Block::LdsRF", "Wave::LdsNT", "Wave::LdsTN", "Wg::LdsNT", "Wg::LdsTN"]
_BLOCKS = [(1, 1), (2, 2), (1, 2), (2, 1), (4, 2), (2, 4), (4, 4), (1, 4)]
_TBLOCKS = [(128, 2), (64, 1), (64, 4), (256, 1), (128, 1), (64, 2)]


def coop_gemm_cases():
    """The CASE(...) lines, deterministic.  f16 -> f32 gets the full product of block sizes x A/B
    layouts x LDS layouts x configs; the other types walk the same axes diagonally.  Blocks per wave,
    thread-block shape and the C/D layout rotate with the case index.  Cases the kernel's own guard
    rejects (register budget, LdsRF with more than one wave) are reported as skipped at run time."""
    cases = []

    def add(types, size, la, lb, lds, cfg):
        i = len(cases)
        # (32-wide blocks: at most 2 x 2 per wave, more exceeds the kernel's register budget; the
        # index is skewed so that the cases dealt to one translation unit differ in blocks per wave)
        nblocks = 4 if size[0] == 32 else len(_BLOCKS)
        bx, by = _BLOCKS[(i + i // MATRIX_UNITS) % nblocks]
        tx, ty = (64, 1) if cfg.endswith("LdsRF") and i % 2 == 0 else _TBLOCKS[(i // 3) % len(_TBLOCKS)]
        lc = "RC"[(i // 2) % 2]
        cases.append(f"CASE({size[0]}, {size[0]}, {size[1]}, {types[0]}, {types[1]}, {types[2]}, "
                     f"{la}, {lb}, {lc}, {lds}, {cfg}, {bx}, {by}, {tx}, {ty});")

    for types, sizes in _MATRIX_TYPES:
        full = types == ("f16", "f32", "f32")
        n = 0
        for size in sizes:
            for cfg in _CONFIGS:
                for la, lb in (("R", "C"), ("C", "R"), ("R", "R"), ("C", "C")):
                    for lds in ("R", "C"):
                        n += 1
                        if full or n % 8 == (len(cases) // 5) % 8:
                            add(types, size, la, lb, lds, cfg)

    # the two kernels without LDS (test/gemm/gemm_PGR0_LB0_MP0_{MB,SB}_NC): every type, block size
    # and A/B layout pair
    for types, sizes in _MATRIX_TYPES:
        for size in sizes:
            for la, lb in (("R", "C"), ("C", "R"), ("R", "R"), ("C", "C")):
                i = len(cases)
                nblocks = 4 if size[0] == 32 else len(_BLOCKS)
                bx, by = _BLOCKS[1 + (i + i // MATRIX_UNITS) % (nblocks - 1)]  # more than one block
                tx, ty = _TBLOCKS[(i // 3) % len(_TBLOCKS)]
                lc = "RC"[(i // 2) % 2]
                head = f"{size[0]}, {size[0]}, {size[1]}, {types[0]}, {types[1]}, {types[2]}, {la}, {lb}, {lc}"
                cases.append(f"CASE_MB({head}, {bx}, {by}, {tx}, {ty});")
                tx, ty = _TBLOCKS[(i // 3 + 2) % len(_TBLOCKS)]
                cases.append(f"CASE_SB({head}, {tx}, {ty});")
    return cases


# (BlockM, BlockN) of the reference's unit tests (test/unit/unit_test_params.hpp:89-141)
_UNIT_SIZES = ([(16, k) for k in (16, 32, 64, 128, 256)]
               + [(b, k) for b in (32, 64, 128, 256) for k in (8, 16, 32, 64, 128, 256)])
_UNIT_TYPES = ["f16", "h16", "f32", "i8", "bf16", "f64", "f8", "i32", "bf8"]
_UNIT_TBLOCKS = [(64, 1), (64, 2), (128, 1), (64, 4), (128, 2), (256, 1)]


def unit_kernel_cases():
    """The UNIT(...) lines for tests/dropin/unit_kernels.cpp, deterministic: every kernel x block
    size x layout, with element type and thread-block shape rotating; the map kernels (which copy
    their block element by element in every lane) on small blocks only."""
    cases = []

    def add(kind, kernel, size, layout, p1, p2):
        i = len(cases)
        t = _UNIT_TYPES[(i + i // len(_UNIT_TYPES)) % len(_UNIT_TYPES)]
        tx, ty = _UNIT_TBLOCKS[(i // 2 + i // 7) % len(_UNIT_TBLOCKS)]
        cases.append(f"UNIT({kind}, {kernel}, {size[0]}, {size[1]}, {t}, {layout}, {tx}, {ty}, {p1}, {p2});")

    for size in _UNIT_SIZES:
        for layout in "RC":
            for op in ("A", "B", "Acc"):
                n = len(cases)
                add("IDENT", "LoadStoreMatrixSync" + op, size, layout, 0, 0)
                # sharing dimension 0 / 1, index of the row / column of waves that does the work
                add("IDENT", "LoadStoreMatrixCoopSync" + op, size, layout, n % 2, (n // 2) % 3)
                add("FILL", "fillFragment" + op, size, layout, 5 - n % 11, 0)
                pad = ((4, 8), (3, 1), (4, 1), (3, 8))[n % 4]  # the reference's frame widths
                add("LOADC", "loadContamination" + op, size, layout, *pad)
                add("STOREC", "storeContamination" + op, size, layout, *pad)
    for size in ((16, 16), (32, 8), (16, 64), (32, 32), (64, 16)):
        for layout in "RC":
            for kernel in ("MapBlockToMatrix", "MapWaveToMatrix", "MapMatrixToData", "MapThreadToMatrix"):
                add("IDENT", kernel, size, layout, 0, 0)
            add("OVR_BLOCK_M", "MapBlockToMatrixOverrideM", size, layout, 1, 0)
            add("OVR_BLOCK_N", "MapBlockToMatrixOverrideN", size, layout, 1, 0)
            add("OVR_ELEM_M", "MapMatrixToDataOverrideM", size, layout, size[0] // 2, 0)
            add("OVR_ELEM_N", "MapMatrixToDataOverrideN", size, layout, size[1] // 2, 0)
    return cases


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


def coop_gemm_units():
    """The GEMM cases as dealt to the executables: (value of GEMM_KERNEL, cases) per unit.  The
    reference's three kernel headers share their include guards, so a unit holds one kernel."""
    cases = coop_gemm_cases()
    coop = [c for c in cases if c.startswith("CASE(")]
    ncoop = MATRIX_UNITS - 2
    return ([(0, coop[u::ncoop]) for u in range(ncoop)]
            + [(1, [c for c in cases if c.startswith("CASE_MB(")]),
               (2, [c for c in cases if c.startswith("CASE_SB(")])])


def unit_kernel_units():
    cases = unit_kernel_cases()
    return [(0, cases[u::MATRIX_UNITS]) for u in range(MATRIX_UNITS)]


def _build_case_units(source, stem, units, family_macro, extra_includes, verbose):
    """Compiles `source` once per unit (its case list passed as CASE_LIST), in parallel."""
    os.makedirs(BIN, exist_ok=True)
    procs = []
    for unit, (family, cases) in enumerate(units):
        lst = os.path.join(BIN, f"{stem}_cases_{unit}.inc")
        with open(lst, "w") as f:
            f.write("\n".join(cases) + "\n")
        exe = os.path.join(BIN, f"{stem}_{unit}")
        # the reference's test kernels are gated on the architecture ids they know: the device pass
        # reports gfx942's
        cmd = [_hipcc(), "--offload-arch=gfx950", "-std=c++17", "-O2", "-DROCWMMA_AMD_REPORT_ARCH_ID=0x942",
               f'-DCASE_LIST="{lst}"', f"-D{family_macro}={family}", "-I" + os.path.join(ROOT, "include")]
        cmd += ["-I" + d for d in extra_includes]
        cmd += ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
                os.path.join(HERE, source), "-o", exe]
        procs.append((exe, lst, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    out = []
    for exe, lst, proc in procs:
        log, _ = proc.communicate()
        if proc.returncode != 0:
            raise RuntimeError(f"{os.path.basename(exe)}: hipcc failed\n{log[-3000:]}")
        os.remove(lst)
        if verbose:
            print(exe)
        out.append(exe)
    return out


def build_coop_gemm_matrix(verbose=False):
    """Compiles the GEMM kernel-matrix executables; returns their paths."""
    if not (os.path.isdir(os.path.join(REFERENCE_TESTS, "gemm")) and _hipcc() is not None):
        return []
    return _build_case_units("coop_gemm_matrix.cpp", "coop_gemm_matrix", coop_gemm_units(), "GEMM_KERNEL",
                             [REFERENCE_TESTS, os.path.join(REFERENCE_TESTS, "gemm")], verbose)


def build_unit_kernels(verbose=False):
    """Compiles the unit-test-kernel executables; returns their paths."""
    if not (os.path.isdir(os.path.join(REFERENCE_TESTS, "unit")) and _hipcc() is not None):
        return []
    return _build_case_units("unit_kernels.cpp", "unit_kernels", unit_kernel_units(), "UNIT_FAMILY",
                             [REFERENCE_TESTS, os.path.join(REFERENCE_TESTS, "unit")], verbose)


def build_dlrm_kernels(verbose=False):
    """Compiles the reference's four DLRM test kernels (test/dlrm/device/*.hpp) with the host side in
    tests/dropin/dlrm_kernels.cpp; returns the executable's path in a list."""
    if not (os.path.isdir(os.path.join(REFERENCE_TESTS, "dlrm")) and _hipcc() is not None):
        return []
    os.makedirs(BIN, exist_ok=True)
    exe = os.path.join(BIN, "dlrm_kernels")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-std=c++17", "-O2", "-DROCWMMA_AMD_REPORT_ARCH_ID=0x942",
           "-I" + os.path.join(ROOT, "include"), "-I" + REFERENCE_TESTS, "-I" + os.path.join(REFERENCE_TESTS, "dlrm"),
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
           os.path.join(HERE, "dlrm_kernels.cpp"), "-o", exe]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"dlrm_kernels: hipcc failed\n{res.stdout[-3000:]}")
    if verbose:
        print(exe)
    return [exe]


if __name__ == "__main__":
    if not available():
        print("reference checkout or hipcc not present: nothing built")
        sys.exit(0)
    build(verbose=True)
    build_coop_gemm_matrix(verbose=True)
    build_unit_kernels(verbose=True)
    build_dlrm_kernels(verbose=True)
