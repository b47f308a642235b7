"""GEMM parity on the GPU: the HIP kernels (through the C ABI) against the CPU oracle on the same
seeded bits.  Bar: int8 -> int32 bit-exact; f16 / bf16 <= 1e-3 and fp8 <= 1e-2 in the reference's
compareEqual metric (max |a-b| / (|a|+|b|+1)); the exact-integer fill pattern must match bit for
bit for every type."""
import numpy as np
import pytest

import oracle as orc
import rocwmma_amd as rw
from util import CM, RM, exact_int_bits, normal_fp8_bits, to_device, to_host, tol_for, uniform_bits

pytestmark = pytest.mark.gpu

OUT_OF = {orc.F16: orc.F32, orc.BF16: orc.F32, orc.E4M3: orc.F32, orc.E5M2: orc.F32, orc.I8: orc.I32}


# kernel families a test runs through; GEMM_BLOCKED_256 forces the 256 x 256 configuration, which
# GEMM_BLOCKED only picks for problems that occupy at least half of the compute units
ALGOS = [rw.GEMM_WAVE_TILE, rw.GEMM_BLOCKED, rw.GEMM_BLOCKED_256]


def tile_dims(algo, m, n):
    """Problem size for `algo`: the forced 256 x 256 tile needs multiples of 256."""
    if algo == rw.GEMM_BLOCKED_256:
        return -(-m // 256) * 256, -(-n // 256) * 256
    return m, n


def run_gemm(dtype_in, dtype_out, la, lb, lc, m, n, k, a, b, c, alpha, beta, algo):
    import torch

    np_out = orc.storage_dtype(dtype_out)
    # D pre-filled with NaN / a sentinel so unwritten elements are caught
    if dtype_out == orc.F32:
        d0 = np.full(m * n, np.nan, dtype=np.float32)
    elif dtype_out == orc.I32:
        d0 = np.full(m * n, -123456789, dtype=np.int32)
    elif dtype_out == orc.I8:
        d0 = np.full(m * n, 0x55, dtype=np.int8)
    else:
        d0 = np.full(m * n, 0x7E00, dtype=np.uint16)
    d = to_device(d0)
    rw.gemm(dtype_in, dtype_out, la, lb, lc, m, n, k, to_device(a), to_device(b),
            None if c is None else to_device(c), d, alpha, beta, algo=algo)
    torch.cuda.synchronize()
    return to_host(d, np_out)


def check(dtype_in, dtype_out, got, want, tol):
    if tol == 0.0:
        assert np.array_equal(got, want), f"{(got != want).sum()} of {got.size} elements differ"
        return 0.0
    err, inf, nan = orc.compare_equal(dtype_out, got, dtype_out, want)
    assert not inf and not nan, (inf, nan)
    assert err <= tol, f"max relative error {err} > {tol}"
    return err


# ------------------------------------------------ type combinations of the reference's GEMM tests
@pytest.mark.parametrize("algo", ALGOS)
@pytest.mark.parametrize("la,lb", [(RM, CM), (CM, RM), (RM, RM), (CM, CM)])
@pytest.mark.parametrize("dtype_in,dtype_out,tol", [
    (orc.F16, orc.F16, 1e-3),    # <f16, f16, f32>
    (orc.BF16, orc.BF16, 4e-3),  # <bf16, bf16, f32>: one bf16 ulp (2^-8) of a value v costs v/(2v+1) * 2^-8 <= 2e-3
    (orc.F32, orc.F32, 1e-5),    # <f32, f32, f32> (wave-tile kernel only)
])
@pytest.mark.parametrize("beta", [-0.5, 0.0])
def test_narrow_output_and_f32_type_combinations(dtype_in, dtype_out, tol, la, lb, algo, beta):
    """Input/Output/Compute triples of test/gemm/gemm_common_test_params.hpp:51-111 beyond the
    f32-output ones: C and D in the input type, f32 compute."""
    if dtype_in == orc.F32 and algo != rw.GEMM_WAVE_TILE:
        pytest.skip("f32 inputs run on the wave-tile kernel only")
    m, n, k = 256, 384, 192
    m, n = tile_dims(algo, m, n)
    a = uniform_bits(51, dtype_in, m * k)
    b = uniform_bits(52, dtype_in, k * n)
    c = uniform_bits(53, dtype_out, m * n)
    got = run_gemm(dtype_in, dtype_out, la, lb, RM, m, n, k, a, b, c if beta else None, 1.5, beta, algo)
    want = orc.gemm(dtype_in, dtype_out, la, lb, RM, RM, m, n, k, a, b, c if beta else None, 1.5, beta)
    check(dtype_in, dtype_out, got, want, tol)


@pytest.mark.parametrize("algo", ALGOS + [rw.GEMM_AUTO])
@pytest.mark.parametrize("lc", [RM, CM])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (3.0, -2.0)])
def test_int8_output_triple(algo, lc, alpha, beta):
    """<int8, int8, int32> (test/gemm/gemm_common_test_params.hpp:51-56): 32-bit compute, C and D in
    int8; the result keeps the low eight bits of alpha * acc + beta * c.  Bit-exact.  Entries are
    small so that most results stay inside the int8 range and a lost bit anywhere shows."""
    m, n, k = 256, 256, 256
    rng = np.random.default_rng(61)
    a = rng.integers(-3, 4, size=m * k, dtype=np.int8)
    b = rng.integers(-3, 4, size=k * n, dtype=np.int8)
    c = rng.integers(-128, 128, size=m * n, dtype=np.int8)
    got = run_gemm(orc.I8, orc.I8, RM, CM, lc, m, n, k, a, b, c if beta else None, alpha, beta, algo)
    want = orc.gemm(orc.I8, orc.I8, RM, CM, lc, lc, m, n, k, a, b, c if beta else None, alpha, beta)
    assert np.array_equal(got, want), f"{(got != want).sum()} of {got.size} elements differ"


# ---------------------------------------------------------------- config 1: simple_hgemm workload
@pytest.mark.parametrize("algo", [rw.GEMM_WAVE_TILE, rw.GEMM_BLOCKED, rw.GEMM_AUTO])
def test_config1_256_cubed_f16_alpha_beta_2(algo):
    m = n = k = 256
    a = uniform_bits(0x5EED0001, orc.F16, m * k)
    b = uniform_bits(0x5EED0101, orc.F16, k * n)
    c = np.random.default_rng(0x5EED0201).uniform(-1, 1, m * n).astype(np.float32)
    got = run_gemm(orc.F16, orc.F32, RM, CM, RM, m, n, k, a, b, c, 2.0, 2.0, algo)
    want = orc.gemm(orc.F16, orc.F32, RM, CM, RM, RM, m, n, k, a, b, c, 2.0, 2.0)
    check(orc.F16, orc.F32, got, want, 1e-3)


# ---------------------------------------------------------------- all types x layouts, both families
@pytest.mark.parametrize("algo", ALGOS)
@pytest.mark.parametrize("lc", [RM, CM])
@pytest.mark.parametrize("lb", [RM, CM])
@pytest.mark.parametrize("la", [RM, CM])
@pytest.mark.parametrize("dtype_in", [orc.F16, orc.BF16])
def test_16bit_types_all_layouts(dtype_in, la, lb, lc, algo):
    m, n, k = 256, 384, 192
    m, n = tile_dims(algo, m, n)
    a = uniform_bits(21, dtype_in, m * k)
    b = uniform_bits(22, dtype_in, k * n)
    c = np.random.default_rng(23).uniform(-1, 1, m * n).astype(np.float32)
    got = run_gemm(dtype_in, orc.F32, la, lb, lc, m, n, k, a, b, c, 1.0, 1.0, algo)
    want = orc.gemm(dtype_in, orc.F32, la, lb, lc, lc, m, n, k, a, b, c, 1.0, 1.0)
    check(dtype_in, orc.F32, got, want, 1e-3)


@pytest.mark.parametrize("algo", ALGOS)
@pytest.mark.parametrize("dtype_in", [orc.I8, orc.E4M3, orc.E5M2])
def test_8bit_types_k_contiguous(dtype_in, algo):
    m, n, k = 256, 256, 512
    if dtype_in == orc.I8:
        a, b = uniform_bits(31, orc.I8, m * k), uniform_bits(32, orc.I8, k * n)
        c = uniform_bits(33, orc.I32, m * n)
        alpha, beta = 1.0, 0.0
    else:
        a, b = normal_fp8_bits(31, dtype_in, m * k), normal_fp8_bits(32, dtype_in, k * n)
        c = np.random.default_rng(33).uniform(-1, 1, m * n).astype(np.float32)
        alpha, beta = 1.0, 0.0
    out = OUT_OF[dtype_in]
    got = run_gemm(dtype_in, out, RM, CM, RM, m, n, k, a, b, c, alpha, beta, algo)
    want = orc.gemm(dtype_in, out, RM, CM, RM, RM, m, n, k, a, b, c, alpha, beta)
    check(dtype_in, out, got, want, tol_for(dtype_in))
    # beta != 0 path
    got = run_gemm(dtype_in, out, RM, CM, RM, m, n, k, a, b, c, 2.0, 3.0, algo)
    want = orc.gemm(dtype_in, out, RM, CM, RM, RM, m, n, k, a, b, c, 2.0, 3.0)
    check(dtype_in, out, got, want, tol_for(dtype_in))


@pytest.mark.parametrize("dtype_in", [orc.I8, orc.E4M3])
@pytest.mark.parametrize("la,lb", [(RM, RM), (CM, CM), (CM, RM)])
@pytest.mark.parametrize("algo", [rw.GEMM_AUTO, rw.GEMM_WAVE_TILE])
def test_8bit_types_other_layouts_small(dtype_in, la, lb, algo):
    """A small problem with a dim-major 8-bit operand: whatever AUTO picks for it (the blocked kernel's partly
    filled tiles), and the wave-tile kernel when asked for by name."""
    m, n, k = 64, 96, 256
    a = uniform_bits(41, orc.I8, m * k) if dtype_in == orc.I8 else normal_fp8_bits(41, dtype_in, m * k)
    b = uniform_bits(42, orc.I8, k * n) if dtype_in == orc.I8 else normal_fp8_bits(42, dtype_in, k * n)
    out = OUT_OF[dtype_in]
    got = run_gemm(dtype_in, out, la, lb, RM, m, n, k, a, b, None, 1.0, 0.0, algo)
    want = orc.gemm(dtype_in, out, la, lb, RM, RM, m, n, k, a, b, None, 1.0, 0.0)
    check(dtype_in, out, got, want, tol_for(dtype_in))


@pytest.mark.parametrize("dtype_in", [orc.I8, orc.E4M3, orc.E5M2])
@pytest.mark.parametrize("la,lb", [(RM, RM), (CM, CM), (CM, RM)])
@pytest.mark.parametrize("m,n,k", [(256, 256, 512), (512, 768, 384), (2176, 2304, 640), (128, 384, 320), (64, 192, 256),
                                   (1040, 912, 448)])
def test_8bit_types_other_layouts_blocked(dtype_in, la, lb, m, n, k):
    """8-bit operands whose K index is not the contiguous one go through transposing LDS reads:
    the 256-wide tile, the 128-wide tiles in both ring depths, 64-wide tiles and partly filled edge tiles.
    Random operands, so a lane or byte that lands in the wrong place shows."""
    a = uniform_bits(43, orc.I8, m * k) if dtype_in == orc.I8 else normal_fp8_bits(43, dtype_in, m * k)
    b = uniform_bits(44, orc.I8, k * n) if dtype_in == orc.I8 else normal_fp8_bits(44, dtype_in, k * n)
    out = OUT_OF[dtype_in]
    c = uniform_bits(45, out, m * n)
    got = run_gemm(dtype_in, out, la, lb, RM, m, n, k, a, b, c, 1.0, 1.0, rw.GEMM_BLOCKED)
    want = orc.gemm(dtype_in, out, la, lb, RM, RM, m, n, k, a, b, c, 1.0, 1.0)
    check(dtype_in, out, got, want, tol_for(dtype_in))


@pytest.mark.parametrize("algo", ALGOS)
@pytest.mark.parametrize("dtype_in", [orc.F16, orc.BF16, orc.E4M3, orc.E5M2, orc.I8])
def test_exact_integer_pattern_is_bit_exact(dtype_in, algo):
    """The reference's fill makes every partial sum an exact integer, so any summation order
    must reproduce the CPU result bit for bit (all types, not only int8)."""
    m, n, k = 256, 256, 1024
    a = exact_int_bits(dtype_in, m, k, RM)
    b = exact_int_bits(dtype_in, k, n, CM)
    out = OUT_OF[dtype_in]
    c = exact_int_bits(out, m, n, RM)
    got = run_gemm(dtype_in, out, RM, CM, RM, m, n, k, a, b, c, 2.0, 2.0, algo)
    want = orc.gemm(dtype_in, out, RM, CM, RM, RM, m, n, k, a, b, c, 2.0, 2.0)
    same = np.array_equal(got, want)
    assert same


def test_narrow_k_and_small_tiles_wave_tile():
    """K that only the half-width instructions divide, 16-wide blocks, f16 output."""
    for (m, n, k) in [(16, 48, 48), (32, 64, 48), (48, 16, 16), (64, 64, 80), (32, 32, 16)]:
        a = uniform_bits(51, orc.F16, m * k)
        b = uniform_bits(52, orc.F16, k * n)
        c = np.random.default_rng(53).uniform(-1, 1, m * n).astype(np.float32)
        got = run_gemm(orc.F16, orc.F32, RM, CM, RM, m, n, k, a, b, c, 2.0, 2.0, rw.GEMM_AUTO)
        want = orc.gemm(orc.F16, orc.F32, RM, CM, RM, RM, m, n, k, a, b, c, 2.0, 2.0)
        check(orc.F16, orc.F32, got, want, 1e-3)
    m, n, k = 64, 64, 64
    a, b = uniform_bits(54, orc.F16, m * k), uniform_bits(55, orc.F16, k * n)
    c = uniform_bits(56, orc.F16, m * n)
    got = run_gemm(orc.F16, orc.F16, RM, CM, RM, m, n, k, a, b, c, 2.0, 2.0, rw.GEMM_AUTO)
    want = orc.gemm(orc.F16, orc.F16, RM, CM, RM, RM, m, n, k, a, b, c, 2.0, 2.0)
    err, inf, nan = orc.compare_equal(orc.F16, got, orc.F16, want)
    assert not inf and not nan and err <= 10 * 2.0 ** -10


def test_leading_dimensions_larger_than_extent():
    """Padded leading dimensions: only the m x n window of D may be written."""
    import torch

    m, n, k = 256, 256, 128
    lda, ldb, ldc = k + 64, k + 32, n + 16
    rng = np.random.default_rng(61)
    A = orc.encode(orc.F16, rng.uniform(-1, 1, (m, lda)).astype(np.float32))
    B = orc.encode(orc.F16, rng.uniform(-1, 1, (n, ldb)).astype(np.float32))  # col-major B: n columns of ldb
    C = rng.uniform(-1, 1, (m, ldc)).astype(np.float32)
    for algo in ALGOS:
        d = torch.full((m, ldc), 777.0, device="cuda")
        rw.gemm(orc.F16, orc.F32, RM, CM, RM, m, n, k, to_device(A), to_device(B), to_device(C), d, 1.0, 1.0,
                lda=lda, ldb=ldb, ldc=ldc, ldd=ldc, algo=algo)
        torch.cuda.synchronize()
        got = d.cpu().numpy()
        want = orc.gemm(orc.F16, orc.F32, RM, CM, RM, RM, m, n, k, A[:, :k], B[:, :k], C[:, :n], 1.0, 1.0)
        check(orc.F16, orc.F32, np.ascontiguousarray(got[:, :n]).reshape(-1), want, 1e-3)
        assert np.all(got[:, n:] == 777.0)


@pytest.mark.parametrize("dtype_in,dtype_out", [(orc.F16, orc.F32), (orc.F16, orc.F16), (orc.I8, orc.I32)])
def test_c_may_alias_d(dtype_in, dtype_out):
    """In-place update (the same buffer as C and D), as the header allows: every element is read
    before it is written, by the same lane (blocked kernel: C staged through LDS for 32-bit outputs,
    through registers for 16-bit outputs)."""
    import torch

    m, n, k = 512, 768, 256
    a = uniform_bits(81, dtype_in, m * k)
    b = uniform_bits(82, dtype_in, k * n)
    c = uniform_bits(83, dtype_out, m * n)
    alpha, beta = (1.0, 1.0) if dtype_in == orc.I8 else (0.5, 1.5)
    want = orc.gemm(dtype_in, dtype_out, RM, CM, RM, RM, m, n, k, a, b, c, alpha, beta)
    for algo in ALGOS:
        cd = to_device(c.copy())
        rw.gemm(dtype_in, dtype_out, RM, CM, RM, m, n, k, to_device(a), to_device(b), cd, cd, alpha, beta, algo=algo)
        torch.cuda.synchronize()
        check(dtype_in, dtype_out, to_host(cd, orc.storage_dtype(dtype_out)), want, tol_for(dtype_in))


@pytest.mark.parametrize("la,lb", [(RM, CM), (CM, RM), (RM, RM), (CM, CM)])
def test_padded_leading_dimensions_every_layout_many_tiles(la, lb):
    """Padded lda / ldb / ldc / ldd with several macro tiles in both directions: the padding of D
    must stay untouched, the window must match the oracle."""
    import torch

    m, n, k = 512, 768, 320
    pad_a, pad_b, pad_c = 24, 40, 12
    rng = np.random.default_rng(91)
    a_rows, a_cols = (m, k) if la == RM else (k, m)
    b_rows, b_cols = (k, n) if lb == RM else (n, k)
    A = orc.encode(orc.F16, rng.uniform(-1, 1, (a_rows, a_cols + pad_a)).astype(np.float32))
    B = orc.encode(orc.F16, rng.uniform(-1, 1, (b_rows, b_cols + pad_b)).astype(np.float32))
    C = rng.uniform(-1, 1, (m, n + pad_c)).astype(np.float32)
    want = orc.gemm(orc.F16, orc.F32, la, lb, RM, RM, m, n, k, np.ascontiguousarray(A[:, :a_cols]),
                    np.ascontiguousarray(B[:, :b_cols]), np.ascontiguousarray(C[:, :n]), 1.0, -2.0)
    for algo in ALGOS:
        d = torch.full((m, n + pad_c), 777.0, device="cuda")
        rw.gemm(orc.F16, orc.F32, la, lb, RM, m, n, k, to_device(A), to_device(B), to_device(C), d, 1.0, -2.0,
                lda=a_cols + pad_a, ldb=b_cols + pad_b, ldc=n + pad_c, ldd=n + pad_c, algo=algo)
        torch.cuda.synchronize()
        got = d.cpu().numpy()
        check(orc.F16, orc.F32, np.ascontiguousarray(got[:, :n]).reshape(-1), want, 1e-3)
        assert np.all(got[:, n:] == 777.0)


@pytest.mark.parametrize("m,k", [(16, 1536), (32, 1536), (48, 1536), (80, 1536), (112, 1536), (128, 1536),
                                 (16, 1024), (32, 1024), (16, 2048), (32, 2048), (16, 4096), (32, 4096)])
@pytest.mark.parametrize("dtype_in", [orc.I8, orc.E4M3, orc.E5M2])
def test_skinny_weight_streaming_kernel(dtype_in, m, k):
    """M <= 128 token rows, 8-bit, A row / B col: served by the K-split weight-streaming kernel
    (AUTO).  int8 must be bit-exact; the wave-tile kernel gives the same answer."""
    n = 352  # k: 3, 2, 4 and 8 fragment steps per wave (the kernel fetches 1, 2, 4 or 8 at a time)
    if dtype_in == orc.I8:
        a, b = uniform_bits(71, orc.I8, m * k), uniform_bits(72, orc.I8, k * n)
        c = uniform_bits(73, orc.I32, m * n)
    else:
        a, b = normal_fp8_bits(71, dtype_in, m * k), normal_fp8_bits(72, dtype_in, k * n)
        c = np.random.default_rng(73).uniform(-1, 1, m * n).astype(np.float32)
    out = OUT_OF[dtype_in]
    for alpha, beta in [(1.0, 0.0), (2.0, -3.0)]:
        got = run_gemm(dtype_in, out, RM, CM, RM, m, n, k, a, b, c, alpha, beta, rw.GEMM_AUTO)
        want = orc.gemm(dtype_in, out, RM, CM, RM, RM, m, n, k, a, b, c, alpha, beta)
        check(dtype_in, out, got, want, tol_for(dtype_in))
        ref = run_gemm(dtype_in, out, RM, CM, RM, m, n, k, a, b, c, alpha, beta, rw.GEMM_WAVE_TILE)
        check(dtype_in, out, ref, want, tol_for(dtype_in))
        if m != 48:
            # every path but the 48-row one (K slices added to D with atomic adds) sums in a fixed order:
            # a second run gives the same bits, f32 included
            again = run_gemm(dtype_in, out, RM, CM, RM, m, n, k, a, b, c, alpha, beta, rw.GEMM_AUTO)
            assert np.array_equal(got.view(np.uint32), again.view(np.uint32))


@pytest.mark.parametrize("m,n,k", [(48, 352, 1024), (64, 352, 2048), (96, 352, 4096), (112, 1040, 2048),
                                   (80, 14336, 4096)])
@pytest.mark.parametrize("dtype_in", [orc.I8, orc.E4M3, orc.E5M2])
def test_sliced_weight_streaming_kernel(dtype_in, m, n, k):
    """48..112 token rows, 8-bit, A row / B col, K a multiple of 1024: a K slice of A stays in LDS, the K
    slices of an output belong to different workgroups and meet in D through atomic adds (AUTO).
    int8 must be bit-exact; beta != 0 goes through the kernel that initialises D; C may be D."""
    import torch

    if dtype_in == orc.I8:
        a, b = uniform_bits(81, orc.I8, m * k), uniform_bits(82, orc.I8, k * n)
        c = uniform_bits(83, orc.I32, m * n)
    else:
        a, b = normal_fp8_bits(81, dtype_in, m * k), normal_fp8_bits(82, dtype_in, k * n)
        c = np.random.default_rng(83).uniform(-1, 1, m * n).astype(np.float32)
    out = OUT_OF[dtype_in]
    for alpha, beta in [(1.0, 0.0), (2.0, -3.0)]:
        got = run_gemm(dtype_in, out, RM, CM, RM, m, n, k, a, b, c, alpha, beta, rw.GEMM_AUTO)
        want = orc.gemm(dtype_in, out, RM, CM, RM, RM, m, n, k, a, b, c, alpha, beta)
        check(dtype_in, out, got, want, tol_for(dtype_in))
    # in place: D holds C
    d = to_device(c)
    rw.gemm(dtype_in, out, RM, CM, RM, m, n, k, to_device(a), to_device(b), d, d, 2.0, -3.0)
    torch.cuda.synchronize()
    check(dtype_in, out, to_host(d, orc.storage_dtype(out)), want, tol_for(dtype_in))


@pytest.mark.parametrize("dtype_in", [orc.I8, orc.E4M3, orc.E5M2])
def test_sliced_kernel_exact_integer_pattern(dtype_in):
    """Integer-valued operands: every partial sum is exact, so the result must match bit for bit
    whatever order the K slices arrive in."""
    m, n, k = 64, 512, 4096
    a, b = exact_int_bits(dtype_in, m, k, RM), exact_int_bits(dtype_in, k, n, CM)
    out = OUT_OF[dtype_in]
    c = exact_int_bits(out, m, n, RM)
    got = run_gemm(dtype_in, out, RM, CM, RM, m, n, k, a, b, c, 2.0, 2.0, rw.GEMM_AUTO)
    want = orc.gemm(dtype_in, out, RM, CM, RM, RM, m, n, k, a, b, c, 2.0, 2.0)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("m,n,k", [(64, 192, 512), (192, 64, 256), (320, 448, 256), (64, 14336, 4096)])
@pytest.mark.parametrize("dtype_in,dtype_out", [(orc.F16, orc.F32), (orc.BF16, orc.BF16), (orc.I8, orc.I32),
                                                (orc.E4M3, orc.F32)])
def test_blocked_kernel_64x64_tiles(dtype_in, dtype_out, m, n, k):
    """Multiples of 64 that are not multiples of 128 (K-contiguous operands) run on the blocked
    kernel's 64 x 64 tile configuration instead of the wave-tile kernel."""
    if m * n * k > 1 << 30 and dtype_in not in (orc.I8, orc.F16):
        pytest.skip("full-size shape: one 16-bit and one 8-bit type")
    if dtype_in == orc.I8:
        a, b = uniform_bits(91, orc.I8, m * k), uniform_bits(92, orc.I8, k * n)
        c = uniform_bits(93, orc.I32, m * n)
    elif dtype_in == orc.E4M3:
        a, b = normal_fp8_bits(91, dtype_in, m * k), normal_fp8_bits(92, dtype_in, k * n)
        c = np.random.default_rng(93).uniform(-1, 1, m * n).astype(np.float32)
    else:
        a, b = uniform_bits(91, dtype_in, m * k), uniform_bits(92, dtype_in, k * n)
        c = (uniform_bits(93, dtype_out, m * n) if dtype_out != orc.F32
             else np.random.default_rng(93).uniform(-1, 1, m * n).astype(np.float32))
    tol = 4e-3 if dtype_out == orc.BF16 else tol_for(dtype_in)
    for alpha, beta in [(1.0, 0.0), (2.0, -1.0)]:
        got = run_gemm(dtype_in, dtype_out, RM, CM, RM, m, n, k, a, b, c, alpha, beta, rw.GEMM_BLOCKED)
        want = orc.gemm(dtype_in, dtype_out, RM, CM, RM, RM, m, n, k, a, b, c, alpha, beta)
        check(dtype_in, dtype_out, got, want, tol)


@pytest.mark.parametrize("m,n", [(256, 256), (1024, 1152), (1536, 1536)])
@pytest.mark.parametrize("dtype_in", [orc.F16, orc.I8, orc.E4M3])
def test_blocked_kernel_tile_ladder(dtype_in, m, n):
    """K-contiguous operands through every rung below the 256 x 256 tile on a 256-unit device:
    4 tiles of 128 x 128 -> 64 x 64 tiles, 72 -> 128 x 64, 144 -> 128 x 128."""
    k = 256
    if dtype_in == orc.I8:
        a, b = uniform_bits(61, orc.I8, m * k), uniform_bits(62, orc.I8, k * n)
    elif dtype_in == orc.E4M3:
        a, b = normal_fp8_bits(61, dtype_in, m * k), normal_fp8_bits(62, dtype_in, k * n)
    else:
        a, b = uniform_bits(61, dtype_in, m * k), uniform_bits(62, dtype_in, k * n)
    out = OUT_OF[dtype_in]
    got = run_gemm(dtype_in, out, RM, CM, RM, m, n, k, a, b, None, 1.0, 0.0, rw.GEMM_BLOCKED)
    want = orc.gemm(dtype_in, out, RM, CM, RM, RM, m, n, k, a, b, None, 1.0, 0.0)
    check(dtype_in, out, got, want, tol_for(dtype_in))


@pytest.mark.parametrize("la,lb", [(RM, CM), (CM, RM), (RM, RM)])
@pytest.mark.parametrize("dtype_in,m,n,k", [(orc.F16, 2176, 2176, 448), (orc.F16, 1088, 1088, 320), (orc.I8, 2176, 2304, 640),
                                            (orc.E4M3, 1088, 1216, 384), (orc.BF16, 2176, 2176, 96)])
def test_blocked_kernel_more_workgroups_than_compute_units(dtype_in, m, n, k, la, lb):
    """128 x 128 and 64 x 64 tilings with more tiles than a 256-unit device has compute units run on the
    ring of two 128-byte K stages (with K in whole stages; the last case, K = 96, stays on the ring of
    four); an odd number of stages and three layout pairs.  (Multiples of 64 that are not multiples of 128
    run 64 x 64 tiles with both operands K-contiguous and partly filled 128 x 128 tiles otherwise.)"""
    if dtype_in in (orc.E4M3,):
        a, b = normal_fp8_bits(81, dtype_in, m * k), normal_fp8_bits(82, dtype_in, k * n)
    else:
        a, b = uniform_bits(81, dtype_in, m * k), uniform_bits(82, dtype_in, k * n)
    out = OUT_OF[dtype_in]
    c = uniform_bits(83, out, m * n)
    got = run_gemm(dtype_in, out, la, lb, RM, m, n, k, a, b, c, 1.0, 1.0, rw.GEMM_BLOCKED)
    want = orc.gemm(dtype_in, out, la, lb, RM, RM, m, n, k, a, b, c, 1.0, 1.0)
    check(dtype_in, out, got, want, tol_for(dtype_in))


@pytest.mark.parametrize("la,lb,lc", [(RM, CM, RM), (CM, RM, RM), (RM, RM, CM), (CM, CM, CM)])
@pytest.mark.parametrize("dtype_in,dtype_out,m,n,k", [
    (orc.F16, orc.F32, 2560, 8192, 256),   # 10 x 32 tiles = 256 + 64: the last 64 tiles run as 128 half tiles
    (orc.I8, orc.I32, 4096, 5120, 384),    # 16 x 20 = 256 + 64
    (orc.E4M3, orc.F32, 4096, 5120, 256),
    (orc.BF16, orc.BF16, 5120, 4096, 256),  # (column-major C: the transposed problem is the one that is cut)
])
def test_blocked_kernel_last_round_cut_into_half_tiles(dtype_in, dtype_out, m, n, k, la, lb, lc):
    """256 x 256 tiles whose count leaves a last round of at most half of the compute units: the tiles of
    that round run as 256 x 128 tiles in the same launch (on a 256-unit device).  alpha, beta != 0 and every
    37th row checked over all columns: a half tile that lands on the wrong columns shows."""
    a = uniform_bits(61, dtype_in, m * k) if dtype_in in (orc.I8, orc.F16, orc.BF16) else normal_fp8_bits(61, dtype_in, m * k)
    b = uniform_bits(62, dtype_in, k * n) if dtype_in in (orc.I8, orc.F16, orc.BF16) else normal_fp8_bits(62, dtype_in, k * n)
    c = uniform_bits(63, dtype_out, m * n)
    got = run_gemm(dtype_in, dtype_out, la, lb, lc, m, n, k, a, b, c, 2.0, -1.0, rw.GEMM_BLOCKED)
    rows = np.arange(0, m, 37, dtype=np.uint32)
    want = orc.gemm(dtype_in, dtype_out, la, lb, lc, lc, m, n, k, a, b, c, 2.0, -1.0, rows=rows)
    if lc == RM:
        g2, w2 = got.reshape(m, n)[rows], want.reshape(m, n)[rows]
    else:
        g2, w2 = got.reshape(n, m)[:, rows], want.reshape(n, m)[:, rows]
    # (bf16 output: one bf16 ulp (2^-8) of a value v costs v / (2v + 1) * 2^-8 <= 2e-3 in the reference's metric)
    tol = 4e-3 if dtype_out == orc.BF16 else tol_for(dtype_in)
    check(dtype_in, dtype_out, np.ascontiguousarray(g2).ravel(), np.ascontiguousarray(w2).ravel(), tol)


@pytest.mark.parametrize("la,lb,lc", [(RM, CM, RM), (CM, RM, RM), (RM, RM, CM), (CM, CM, RM)])
@pytest.mark.parametrize("dtype_in,dtype_out,m,n,k", [
    (orc.F16, orc.F32, 144, 208, 256), (orc.F16, orc.F32, 2064, 2192, 192), (orc.F16, orc.F16, 400, 16, 128),
    (orc.BF16, orc.BF16, 16, 400, 320), (orc.I8, orc.I32, 272, 1040, 512), (orc.I8, orc.I8, 1936, 2320, 256),
    (orc.E4M3, orc.F32, 656, 48, 384), (orc.E5M2, orc.F32, 2160, 2064, 256)])
def test_blocked_kernel_partly_filled_edge_tiles(dtype_in, dtype_out, m, n, k, la, lb, lc):
    """M and N that are multiples of 16 but not of 64 run on 128 x 128 tiles whose last row and column
    are partly filled (operand reads beyond a matrix end cut off by the buffer bounds, C reads and D
    stores masked); one and many tiles, more tiles than compute units, with and without beta.  D is
    allocated to size and framed by a guard region that must stay untouched."""
    import torch

    if dtype_in in (orc.E4M3, orc.E5M2):
        a, b = normal_fp8_bits(85, dtype_in, m * k), normal_fp8_bits(86, dtype_in, k * n)
    elif dtype_in == orc.I8 and dtype_out == orc.I8:
        rng = np.random.default_rng(85)
        a, b = rng.integers(-3, 4, m * k, dtype=np.int8), rng.integers(-3, 4, k * n, dtype=np.int8)
    else:
        a, b = uniform_bits(85, dtype_in, m * k), uniform_bits(86, dtype_in, k * n)
    c = uniform_bits(87, dtype_out, m * n)
    tol = 4e-3 if dtype_out == orc.BF16 else tol_for(dtype_in)
    np_out = orc.storage_dtype(dtype_out)
    guard = 4096
    for alpha, beta in [(1.0, 0.0), (2.0, -1.0)]:
        frame = np.zeros(m * n + 2 * guard, dtype=np_out)
        frame[:] = 0x55 if np_out != np.float32 else 12345.0
        dev = to_device(frame)
        d = dev[guard:guard + m * n]
        rw.gemm(dtype_in, dtype_out, la, lb, lc, m, n, k, to_device(a), to_device(b), to_device(c), d, alpha, beta,
                algo=rw.GEMM_BLOCKED)
        torch.cuda.synchronize()
        host = to_host(dev, np_out)
        assert np.array_equal(host[:guard], frame[:guard]) and np.array_equal(host[-guard:], frame[-guard:]), "wrote outside D"
        want = orc.gemm(dtype_in, dtype_out, la, lb, lc, lc, m, n, k, a, b, c, alpha, beta)
        check(dtype_in, dtype_out, host[guard:guard + m * n], want, tol)


@pytest.mark.parametrize("m,n,k", [(16, 352, 2048), (16, 14336, 4096), (32, 352, 2048), (32, 352, 4096),
                                   (48, 1040, 1536), (80, 352, 4096), (112, 352, 1024)])
@pytest.mark.parametrize("dtype_in", [orc.F16, orc.BF16])
def test_skinny_and_sliced_kernels_16bit(dtype_in, m, n, k):
    """The weight-streaming kernels also take f16 / bf16 operands (f32 results): all of A in LDS
    while m * k * 2 <= 128 KiB, K slices over workgroups beyond that (AUTO); beta != 0 and C = D."""
    import torch

    a, b = uniform_bits(51, dtype_in, m * k), uniform_bits(52, dtype_in, k * n)
    c = np.random.default_rng(53).uniform(-1, 1, m * n).astype(np.float32)
    for alpha, beta in [(1.0, 0.0), (2.0, -3.0)]:
        got = run_gemm(dtype_in, orc.F32, RM, CM, RM, m, n, k, a, b, c, alpha, beta, rw.GEMM_AUTO)
        want = orc.gemm(dtype_in, orc.F32, RM, CM, RM, RM, m, n, k, a, b, c, alpha, beta)
        check(dtype_in, orc.F32, got, want, 1e-3)
    d = to_device(c)
    rw.gemm(dtype_in, orc.F32, RM, CM, RM, m, n, k, to_device(a), to_device(b), d, d, 2.0, -3.0)
    torch.cuda.synchronize()
    check(dtype_in, orc.F32, to_host(d, np.float32), want, 1e-3)
    # integer-valued operands: exact whatever the summation order
    ai, bi = exact_int_bits(dtype_in, m, k, RM), exact_int_bits(dtype_in, k, n, CM)
    got = run_gemm(dtype_in, orc.F32, RM, CM, RM, m, n, k, ai, bi, None, 1.0, 0.0, rw.GEMM_AUTO)
    assert np.array_equal(got, orc.gemm(dtype_in, orc.F32, RM, CM, RM, RM, m, n, k, ai, bi, None, 1.0, 0.0))


def _random_cases(count):
    rng = np.random.default_rng(20240607)
    out = []
    for i in range(count):
        dtype_in = [orc.F16, orc.BF16, orc.I8, orc.E4M3][i % 4]
        m = int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 192, 256, 320]))
        n = int(rng.choice([16, 64, 128, 192, 256, 352, 448, 512, 1040]))
        k = int(rng.choice([64, 128, 256, 512, 1024, 2048]))
        if dtype_in in (orc.I8, orc.E4M3) or rng.random() < 0.5:
            la, lb = RM, CM
        else:
            la, lb = [(RM, RM), (CM, CM), (CM, RM)][int(rng.integers(3))]
        out.append((dtype_in, m, n, k, la, lb, float(rng.choice([1.0, 2.0])), float(rng.choice([0.0, 1.0, -2.0]))))
    return out


@pytest.mark.parametrize("case", _random_cases(48), ids=lambda c: "-".join(str(x) for x in c))
def test_auto_dispatch_on_seeded_random_shapes(case):
    """Whatever kernel AUTO picks (weight-streaming, K-sliced, any rung of the blocked kernel's ladder,
    wave-tile) the result must match the oracle: shapes drawn so that every path is hit."""
    dtype_in, m, n, k, la, lb, alpha, beta = case
    out = OUT_OF[dtype_in]
    if dtype_in == orc.I8:
        a, b = uniform_bits(7, orc.I8, m * k), uniform_bits(8, orc.I8, k * n)
        c = uniform_bits(9, orc.I32, m * n)
    elif dtype_in == orc.E4M3:
        a, b = normal_fp8_bits(7, dtype_in, m * k), normal_fp8_bits(8, dtype_in, k * n)
        c = np.random.default_rng(9).uniform(-1, 1, m * n).astype(np.float32)
    else:
        a, b = uniform_bits(7, dtype_in, m * k), uniform_bits(8, dtype_in, k * n)
        c = np.random.default_rng(9).uniform(-1, 1, m * n).astype(np.float32)
    got = run_gemm(dtype_in, out, la, lb, RM, m, n, k, a, b, c, alpha, beta, rw.GEMM_AUTO)
    want = orc.gemm(dtype_in, out, la, lb, RM, RM, m, n, k, a, b, c, alpha, beta)
    check(dtype_in, out, got, want, tol_for(dtype_in))


# ---------------------------------------------------------------- config 3: quantised shapes
@pytest.mark.parametrize("m", [16, 128, 4096])
@pytest.mark.parametrize("dtype_in", [orc.I8, orc.E4M3])
def test_config3_quantised_inference_shapes(dtype_in, m):
    n, k = 14336, 4096
    if dtype_in == orc.I8:
        a, b = uniform_bits(0x5EED0003, orc.I8, m * k), uniform_bits(0x5EED0103, orc.I8, k * n)
    else:
        a, b = normal_fp8_bits(0x5EED0003, dtype_in, m * k), normal_fp8_bits(0x5EED0103, dtype_in, k * n)
    out = OUT_OF[dtype_in]
    got = run_gemm(dtype_in, out, RM, CM, RM, m, n, k, a, b, None, 1.0, 0.0, rw.GEMM_AUTO)
    # every element for M = 16 / 128; a seeded sample of 64 full rows for M = 4096
    rows = None if m <= 128 else np.sort(np.random.default_rng(7).choice(m, 64, replace=False)).astype(np.uint32)
    want = orc.gemm(dtype_in, out, RM, CM, RM, RM, m, n, k, a, b, None, 1.0, 0.0, rows=rows)
    if rows is None:
        check(dtype_in, out, got, want, tol_for(dtype_in))
    else:
        check(dtype_in, out, got.reshape(m, n)[rows].reshape(-1), want.reshape(m, n)[rows].reshape(-1),
              tol_for(dtype_in))


@pytest.mark.parametrize("dtype_in,dtype_out,m,n,k,beta", [
    (orc.I8, orc.I32, 128, 8448, 2048, 0.0), (orc.I8, orc.I32, 256, 4224, 2112, 2.0),
    (orc.E4M3, orc.F32, 128, 8448, 2048, 0.0), (orc.E5M2, orc.F32, 128, 8320, 2176, -0.5),
    (orc.F16, orc.F32, 128, 8448, 1024, 1.0), (orc.F16, orc.F16, 256, 4224, 1088, 0.0),
    (orc.BF16, orc.F32, 128, 8320, 1152, 0.0),
    # fp8 on 128 x 128 tiles of the same ring: more than half as many tiles as compute units, 4 KiB of K
    (orc.E4M3, orc.F32, 256, 8320, 4096, 0.5), (orc.E5M2, orc.F32, 384, 5632, 4224, 0.0),
])
def test_blocked_kernel_128x64_tiles_on_whole_line_stages(dtype_in, dtype_out, m, n, k, beta):
    """One round of 128 x 64 tiles (more than a quarter, at most the number of compute units) with at least
    2 KiB of K per row, both operands K-contiguous: the ring of four 128-byte stages.  K in whole stages and
    with half a stage left over (the latter falls back to the 64-byte ring), with and without C."""
    if dtype_in == orc.I8:
        a, b = uniform_bits(0x5EED0301, orc.I8, m * k), uniform_bits(0x5EED0302, orc.I8, k * n)
    elif dtype_in in (orc.E4M3, orc.E5M2):
        a, b = normal_fp8_bits(0x5EED0301, dtype_in, m * k), normal_fp8_bits(0x5EED0302, dtype_in, k * n)
    else:
        a, b = uniform_bits(0x5EED0301, dtype_in, m * k), uniform_bits(0x5EED0302, dtype_in, k * n)
    c = uniform_bits(0x5EED0303, dtype_out, m * n) if beta else None
    alpha = 1.0 if dtype_in == orc.I8 else 0.75
    got = run_gemm(dtype_in, dtype_out, RM, CM, RM, m, n, k, a, b, c, alpha, beta, rw.GEMM_AUTO)
    want = orc.gemm(dtype_in, dtype_out, RM, CM, RM, RM, m, n, k, a, b, c, alpha, beta)
    check(dtype_in, dtype_out, got, want, tol_for(dtype_in))


@pytest.mark.parametrize("dtype_in,dtype_out,m,n,k,beta", [
    (orc.I8, orc.I32, 64, 8448, 4096, 0.0), (orc.I8, orc.I32, 112, 4240, 4096, 2.0), (orc.I8, orc.I8, 80, 8320, 4224, 0.0),
    (orc.E4M3, orc.F32, 80, 8320, 4096, 0.5), (orc.E5M2, orc.F32, 16, 8448, 4224, 0.0),
    (orc.F16, orc.F32, 96, 8448, 2048, 1.0), (orc.F16, orc.F16, 64, 4176, 8192, 0.0),
    (orc.BF16, orc.F32, 144, 4224, 2112, 0.0),
])
def test_blocked_kernel_partly_filled_128x64_tiles_on_whole_line_stages(dtype_in, dtype_out, m, n, k, beta):
    """Row counts that leave a partly filled row of 128 x 64 tiles (and an n that leaves a partly filled
    column), one round of workgroups, at least 4 KiB of K per row, both operands K-contiguous."""
    if dtype_in == orc.I8:
        a, b = uniform_bits(0x5EED0311, orc.I8, m * k), uniform_bits(0x5EED0312, orc.I8, k * n)
    elif dtype_in in (orc.E4M3, orc.E5M2):
        a, b = normal_fp8_bits(0x5EED0311, dtype_in, m * k), normal_fp8_bits(0x5EED0312, dtype_in, k * n)
    else:
        a, b = uniform_bits(0x5EED0311, dtype_in, m * k), uniform_bits(0x5EED0312, dtype_in, k * n)
    c = uniform_bits(0x5EED0313, dtype_out, m * n) if beta else None
    alpha = 1.0 if dtype_in == orc.I8 else 0.75
    got = run_gemm(dtype_in, dtype_out, RM, CM, RM, m, n, k, a, b, c, alpha, beta, rw.GEMM_BLOCKED)
    want = orc.gemm(dtype_in, dtype_out, RM, CM, RM, RM, m, n, k, a, b, c, alpha, beta)
    check(dtype_in, dtype_out, got, want, tol_for(dtype_in))


@pytest.mark.parametrize("la,lb", [(RM, RM), (CM, CM)])
@pytest.mark.parametrize("dtype_in,m,n,k", [(orc.I8, 128, 8448, 4096), (orc.E4M3, 256, 4224, 4224), (orc.E5M2, 128, 8320, 4096)])
def test_8bit_types_one_operand_dim_major_on_whole_line_stages(dtype_in, m, n, k, la, lb):
    """128 x 64 / 64 x 128 tiles with one operand in the other major on the ring of four 128-byte stages:
    8-bit types, one round of workgroups, at least 4 KiB of K per row."""
    if dtype_in == orc.I8:
        a, b = uniform_bits(0x5EED0331, orc.I8, m * k), uniform_bits(0x5EED0332, orc.I8, k * n)
    else:
        a, b = normal_fp8_bits(0x5EED0331, dtype_in, m * k), normal_fp8_bits(0x5EED0332, dtype_in, k * n)
    out = OUT_OF[dtype_in]
    c = uniform_bits(0x5EED0333, out, m * n)
    alpha, beta = (1.0, -1.0) if dtype_in == orc.I8 else (0.5, 1.0)
    got = run_gemm(dtype_in, out, la, lb, RM, m, n, k, a, b, c, alpha, beta, rw.GEMM_BLOCKED)
    want = orc.gemm(dtype_in, out, la, lb, RM, RM, m, n, k, a, b, c, alpha, beta)
    check(dtype_in, out, got, want, tol_for(dtype_in))


@pytest.mark.parametrize("m", [128, 80])
def test_whole_line_128x64_tiles_padded_leading_dimensions_in_place(m):
    """The 128 x 64 tiles on 128-byte stages (whole, m = 128, and partly filled, m = 80) with padded lda / ldb /
    ldd and C = D: the window must match the oracle bit for bit (int8), the padding of D must stay untouched."""
    import torch

    n, k = 4240, 4096
    lda, ldb, ldd = k + 64, k + 128, n + 48
    rng = np.random.default_rng(0x5EED0321)
    A = rng.integers(-128, 128, (m, lda), dtype=np.int8)
    B = rng.integers(-128, 128, (n, ldb), dtype=np.int8)  # col-major B: n columns of ldb
    C = rng.integers(-1000, 1000, (m, ldd), dtype=np.int32)
    d = to_device(C.copy())
    rw.gemm(orc.I8, orc.I32, RM, CM, RM, m, n, k, to_device(A), to_device(B), d, d, 1.0, 3.0,
            lda=lda, ldb=ldb, ldc=ldd, ldd=ldd, algo=rw.GEMM_BLOCKED)
    torch.cuda.synchronize()
    got = d.cpu().numpy().reshape(m, ldd)
    want = orc.gemm(orc.I8, orc.I32, RM, CM, RM, RM, m, n, k, np.ascontiguousarray(A[:, :k]), np.ascontiguousarray(B[:, :k]),
                    np.ascontiguousarray(C[:, :n]), 1.0, 3.0)
    assert np.array_equal(np.ascontiguousarray(got[:, :n]).reshape(-1), want)
    assert np.array_equal(got[:, n:], C[:, n:])


# ---------------------------------------------------------------- config 2: 8192^3, 4 layouts x 2 types
@pytest.mark.parametrize("la", [RM, CM])
@pytest.mark.parametrize("lb", [RM, CM])
@pytest.mark.parametrize("dtype_in", [orc.F16, orc.BF16])
def test_config2_8192_cubed_sampled_rows(dtype_in, la, lb):
    """Full-size case: 64 seeded output rows are recomputed by the oracle (same dot-product
    loop, every column), plus a row-sum identity over the whole result."""
    import torch

    m = n = k = 8192
    g = torch.Generator(device="cuda").manual_seed(0x5EED0002 + 8 * dtype_in + 2 * la + lb)
    tdt = torch.float16 if dtype_in == orc.F16 else torch.bfloat16
    A = (torch.rand(m * k, device="cuda", generator=g) * 2 - 1).to(tdt)
    B = (torch.rand(k * n, device="cuda", generator=g) * 2 - 1).to(tdt)
    C = torch.rand(m * n, device="cuda", generator=g) * 2 - 1
    D = torch.full((m * n,), float("nan"), device="cuda")
    rw.gemm(dtype_in, orc.F32, la, lb, RM, m, n, k, A, B, C, D, 1.0, 1.0)
    torch.cuda.synchronize()
    assert not torch.isnan(D).any()
    rows = np.sort(np.random.default_rng(9).choice(m, 64, replace=False)).astype(np.uint32)
    a_bits = A.view(torch.int16).cpu().numpy().view(np.uint16)
    b_bits = B.view(torch.int16).cpu().numpy().view(np.uint16)
    c_host = C.cpu().numpy()
    want = orc.gemm(dtype_in, orc.F32, la, lb, RM, RM, m, n, k, a_bits, b_bits, c_host, 1.0, 1.0, rows=rows)
    got = D.cpu().numpy().reshape(m, n)[rows]
    check(dtype_in, orc.F32, got.reshape(-1), want.reshape(m, n)[rows].reshape(-1), 1e-3)
    # size-independent property: D 1 = A (B 1) + C 1 (float64 on the device, whole matrix)
    Am = (A.view(m, k) if la == RM else A.view(k, m).t()).double()
    Bm = (B.view(k, n) if lb == RM else B.view(n, k).t()).double()
    ones = torch.ones(n, 1, dtype=torch.float64, device="cuda")
    lhs = D.view(m, n).double() @ ones
    rhs = Am @ (Bm @ ones) + C.view(m, n).double() @ ones
    assert torch.allclose(lhs, rhs, rtol=0, atol=0.5), float((lhs - rhs).abs().max())
