"""Block-scaled (MX) fp8 GEMM on the GPU against the CPU oracle's restatement of the OCP definition,
on the same seeded bits.  Bar: fp8 <= 1e-2 in the reference's compareEqual metric; patterns whose
partial sums are exact (small integers times powers of two) must match bit for bit."""
import numpy as np
import pytest

import oracle as orc
import rocwmma_amd as rw
from util import CM, RM, exact_int_bits, to_device, to_host, uniform_bits

pytestmark = pytest.mark.gpu


def run_mx(dtype, la, lb, lc, m, n, k, a, sa, b, sb, c, alpha, beta, workspace):
    import torch

    d = to_device(np.full(m * n, np.nan, dtype=np.float32))
    ws = None
    if workspace:
        ws = torch.empty(rw.gemm_mx_workspace_size(m, n, k), dtype=torch.uint8, device="cuda")
    rw.gemm_mx(dtype, la, lb, lc, m, n, k, to_device(a), to_device(sa), to_device(b), to_device(sb),
               None if c is None else to_device(c), d, alpha, beta, workspace=ws)
    torch.cuda.synchronize()
    return to_host(d, np.float32)


def scales(seed, rows, k, lo, hi):
    return np.random.default_rng(seed).integers(lo, hi + 1, size=(rows, k // 32), dtype=np.uint8)


def check(got, want, tol):
    if tol == 0.0:
        assert np.array_equal(got, want), f"{(got != want).sum()} of {got.size} elements differ"
        return
    err, inf, nan = orc.compare_equal(orc.F32, got, orc.F32, want)
    assert not inf and not nan, (inf, nan)
    assert err <= tol, f"max relative error {err} > {tol}"


@pytest.mark.parametrize("workspace", [False, True])
@pytest.mark.parametrize("la,lb", [(RM, CM), (CM, RM), (RM, RM), (CM, CM)])
@pytest.mark.parametrize("dtype", [orc.E4M3, orc.E5M2])
@pytest.mark.parametrize("m,n,k", [(48, 80, 384), (64, 96, 192), (256, 512, 512), (256, 256, 128), (512, 256, 896)])
def test_exact_pattern_with_power_of_two_scales_is_bit_exact(dtype, la, lb, m, n, k, workspace):
    """Elements 0, -1, -2 (the reference's device fill, test/device/common.hpp:204-219) and scales
    1/2, 1, 2: every partial sum is an integer multiple of 1/4 below 2^24 of them, so any order of
    accumulation gives the same bits.  A scale applied to the wrong block, row or operand does not."""
    a = exact_int_bits(dtype, m, k, la)
    b = exact_int_bits(dtype, k, n, lb)
    sa, sb = scales(11, m, k, 126, 128), scales(12, n, k, 126, 128)
    c = exact_int_bits(orc.F32, m, n, RM)
    got = run_mx(dtype, la, lb, RM, m, n, k, a, sa, b, sb, c, 2.0, 3.0, workspace)
    want = orc.gemm_mx(dtype, la, lb, RM, RM, m, n, k, a, sa, b, sb, c, 2.0, 3.0)
    check(got, want, 0.0)


@pytest.mark.parametrize("dtype", [orc.E4M3, orc.E5M2])
@pytest.mark.parametrize("m,n,k", [(2048, 4352, 256), (4352, 2048, 384)])
def test_large_tile_with_half_tiles_for_the_last_round(dtype, m, n, k):
    """136 tiles of 256 x 256: on a 256-unit device the 256 x 256 / 16x16x128 configuration with every
    tile of the (only, partly filled) round cut into half tiles.  Exact pattern, bit for bit."""
    a = exact_int_bits(dtype, m, k, RM)
    b = exact_int_bits(dtype, k, n, CM)
    sa, sb = scales(81, m, k, 126, 128), scales(82, n, k, 126, 128)
    got = run_mx(dtype, RM, CM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0, True)
    want = orc.gemm_mx(dtype, RM, CM, RM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0)
    check(got, want, 0.0)


@pytest.mark.parametrize("dtype", [orc.E4M3, orc.E5M2])
@pytest.mark.parametrize("m,n,k", [(48, 14336, 512), (128, 1040, 640), (208, 304, 128), (1024, 768, 1152)])
def test_mid_size_shapes_on_edge_tiles(dtype, m, n, k):
    """More than 32 rows, not enough 256 x 256 tiles for half of the device: 128 x 128 tiles of 32x32x64
    blocks, the last row and column of tiles partly filled.  Exact pattern bit for bit; random operands
    within the fp8 tolerance."""
    a = exact_int_bits(dtype, m, k, RM)
    b = exact_int_bits(dtype, k, n, CM)
    sa, sb = scales(91, m, k, 126, 128), scales(92, n, k, 126, 128)
    c = exact_int_bits(orc.F32, m, n, RM)
    got = run_mx(dtype, RM, CM, RM, m, n, k, a, sa, b, sb, c, 2.0, 3.0, True)
    want = orc.gemm_mx(dtype, RM, CM, RM, RM, m, n, k, a, sa, b, sb, c, 2.0, 3.0)
    check(got, want, 0.0)
    a = uniform_bits(93, dtype, m * k)
    b = uniform_bits(94, dtype, k * n)
    sa, sb = scales(95, m, k, 124, 130), scales(96, n, k, 124, 130)
    got = run_mx(dtype, RM, CM, RM, m, n, k, a, sa, b, sb, None, 0.5, 0.0, True)
    want = orc.gemm_mx(dtype, RM, CM, RM, RM, m, n, k, a, sa, b, sb, None, 0.5, 0.0)
    check(got, want, 1e-2)


@pytest.mark.parametrize("workspace", [False, True])
@pytest.mark.parametrize("la,lb,lc", [(RM, CM, RM), (RM, CM, CM), (CM, RM, CM), (CM, CM, RM), (RM, RM, CM)])
@pytest.mark.parametrize("dtype", [orc.E4M3, orc.E5M2])
def test_random_operands_and_scales(dtype, la, lb, lc, workspace):
    m, n, k = 256, 512, 640
    a = uniform_bits(21, dtype, m * k)
    b = uniform_bits(22, dtype, k * n)
    sa, sb = scales(23, m, k, 124, 130), scales(24, n, k, 124, 130)
    c = uniform_bits(25, orc.F32, m * n)
    for beta in (0.0, -0.5):
        got = run_mx(dtype, la, lb, lc, m, n, k, a, sa, b, sb, c if beta else None, 1.5, beta, workspace)
        want = orc.gemm_mx(dtype, la, lb, lc, lc, m, n, k, a, sa, b, sb, c if beta else None, 1.5, beta)
        check(got, want, 1e-2)


@pytest.mark.parametrize("workspace", [False, True])
def test_wide_range_of_scales_against_the_size_of_the_terms(workspace):
    """Scales from 2^-7 to 2^7 per operand: a result is then a small difference of terms up to 2^14
    times larger, and two float32 summations in different orders agree to a few ulp of the LARGEST
    partial sums, not of the result.  So the error is measured against the sum of the terms'
    magnitudes (float64).  Measured: 2^-16.2 of that sum, the same for both kernels (the matrix core
    adds the 128 products of an instruction aligned to the largest of them and drops what falls
    below its adder width); the bound of 2^-14 still catches any scale applied to the wrong block (a
    factor of two on one block moves a result by about 1/20 of that sum)."""
    m, n, k = 256, 256, 640
    dtype = orc.E4M3
    a = uniform_bits(61, dtype, m * k)
    b = uniform_bits(62, dtype, k * n)
    sa, sb = scales(63, m, k, 120, 134), scales(64, n, k, 120, 134)
    got = run_mx(dtype, RM, CM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0, workspace).reshape(m, n).astype(np.float64)
    af = orc.mx_dequantise(dtype, a, sa, RM, m, k).astype(np.float64)
    bf = orc.mx_dequantise(dtype, b, sb, RM, n, k).astype(np.float64)
    want = af @ bf.T
    size = np.abs(af) @ np.abs(bf).T
    assert np.max(np.abs(got - want) / size) < 2.0 ** -14


@pytest.mark.parametrize("dtype", [orc.E4M3, orc.E5M2])
@pytest.mark.parametrize("m,n,k", [(16, 14336, 4096), (32, 1024, 4096), (16, 200 * 16, 1024), (32, 80, 2048)])
def test_few_token_rows_on_the_weight_streaming_kernel(dtype, m, n, k):
    """Up to 32 token rows against a wide block-scaled weight matrix (row-major A, col-major B): the
    weight-streaming kernel with the scaled instruction.  Exact pattern bit for bit, random operands
    within the fp8 tolerance, with and without C."""
    a = exact_int_bits(dtype, m, k, RM)
    b = exact_int_bits(dtype, k, n, CM)
    sa, sb = scales(71, m, k, 126, 128), scales(72, n, k, 126, 128)
    c = exact_int_bits(orc.F32, m, n, RM)
    got = run_mx(dtype, RM, CM, RM, m, n, k, a, sa, b, sb, c, 2.0, 3.0, False)
    want = orc.gemm_mx(dtype, RM, CM, RM, RM, m, n, k, a, sa, b, sb, c, 2.0, 3.0)
    check(got, want, 0.0)
    a = uniform_bits(73, dtype, m * k)
    b = uniform_bits(74, dtype, k * n)
    sa, sb = scales(75, m, k, 124, 130), scales(76, n, k, 124, 130)
    got = run_mx(dtype, RM, CM, RM, m, n, k, a, sa, b, sb, None, 0.5, 0.0, False)
    want = orc.gemm_mx(dtype, RM, CM, RM, RM, m, n, k, a, sa, b, sb, None, 0.5, 0.0)
    check(got, want, 1e-2)


def test_unit_scales_give_the_unscaled_gemm():
    import torch

    m, n, k = 256, 256, 1024
    dtype = orc.E4M3
    a = uniform_bits(31, dtype, m * k)
    b = uniform_bits(32, dtype, k * n)
    one_a = np.full((m, k // 32), 127, dtype=np.uint8)
    one_b = np.full((n, k // 32), 127, dtype=np.uint8)
    for workspace in (False, True):
        got = run_mx(dtype, RM, CM, RM, m, n, k, a, one_a, b, one_b, None, 1.0, 0.0, workspace)
        d = to_device(np.zeros(m * n, dtype=np.float32))
        rw.gemm(dtype, orc.F32, RM, CM, RM, m, n, k, to_device(a), to_device(b), None, d, 1.0, 0.0)
        torch.cuda.synchronize()
        check(got, to_host(d, np.float32), 1e-5)


def test_padded_leading_dimensions_of_the_scale_matrices():
    import torch

    m, n, k = 256, 256, 512
    dtype = orc.E5M2
    a = uniform_bits(41, dtype, m * k)
    b = uniform_bits(42, dtype, k * n)
    sa, sb = scales(43, m, k, 124, 130), scales(44, n, k, 124, 130)
    want = orc.gemm_mx(dtype, RM, CM, RM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0)
    pad_a = np.full((m, k // 32 + 5), 255, dtype=np.uint8)  # (NaN scales in the padding: never read)
    pad_b = np.full((n, k // 32 + 3), 255, dtype=np.uint8)
    pad_a[:, :k // 32] = sa
    pad_b[:, :k // 32] = sb
    for workspace in (False, True):
        d = to_device(np.full(m * n, np.nan, dtype=np.float32))
        ws = torch.empty(rw.gemm_mx_workspace_size(m, n, k), dtype=torch.uint8, device="cuda") if workspace else None
        rw.gemm_mx(dtype, RM, CM, RM, m, n, k, to_device(a), to_device(pad_a), to_device(b), to_device(pad_b), None, d,
                   1.0, 0.0, workspace=ws, ld_scale_a=k // 32 + 5, ld_scale_b=k // 32 + 3)
        torch.cuda.synchronize()
        check(to_host(d, np.float32), want, 1e-2)


def test_full_size_quantised_inference_shape_sampled_rows():
    """4096 x 14336 x 4096 (the fp8 shape of the quantised-inference configuration) with block scales:
    64 oracle rows and the row sums of every row against float64 sums of the dequantised operands."""
    import torch

    m, n, k = 4096, 14336, 4096
    dtype = orc.E4M3
    a = uniform_bits(51, dtype, m * k)
    b = uniform_bits(52, dtype, k * n)
    sa, sb = scales(53, m, k, 124, 130), scales(54, n, k, 124, 130)
    got = run_mx(dtype, RM, CM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0, True).reshape(m, n)
    rows = np.random.default_rng(55).choice(m, size=64, replace=False).astype(np.uint32)
    want = orc.gemm_mx(dtype, RM, CM, RM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0, rows=np.sort(rows)).reshape(m, n)
    check(np.ascontiguousarray(got[np.sort(rows)]), np.ascontiguousarray(want[np.sort(rows)]), 1e-2)
    # every row and column takes part: D summed over columns = A_deq * (B_deq summed over columns)
    af = orc.mx_dequantise(dtype, a, sa, RM, m, k).astype(np.float64)
    bsum = orc.mx_dequantise(dtype, b, sb, RM, n, k).astype(np.float64).sum(axis=0)
    ref = af @ bsum
    size = np.abs(af) @ np.abs(orc.mx_dequantise(dtype, b, sb, RM, n, k).astype(np.float64)).sum(axis=0)
    assert np.max(np.abs(got.astype(np.float64).sum(axis=1) - ref) / size) < 1e-5


@pytest.mark.parametrize("m,n,k", [(4096, 2048, 512), (128, 1040, 640), (512, 768, 256)])
def test_scales_packed_once_and_reused(m, n, k):
    """rocwmma_amd_gemm_mx_pack_scales + rocwmma_amd_gemm_mx_packed against rocwmma_amd_gemm_mx with a workspace
    (which packs on every call), bit for bit, on the 256 x 256 tiles and on the mid-size tiles; then new token
    scales packed into the same workspace without touching the weights' part."""
    import torch

    rng = np.random.default_rng(77)
    a, b = exact_int_bits(orc.E4M3, m, k, RM), exact_int_bits(orc.E4M3, k, n, CM)
    sa, sb = scales(71, m, k, 125, 129), scales(72, n, k, 125, 129)
    want = run_mx(orc.E4M3, RM, CM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0, True)
    ws = torch.randint(0, 255, (rw.gemm_mx_workspace_size(m, n, k),), dtype=torch.uint8, device="cuda")
    rw.gemm_mx_pack_scales(RM, CM, RM, m, n, k, to_device(sa), to_device(sb), ws)
    da, db = to_device(a), to_device(b)
    for _ in range(2):  # the GEMM leaves the workspace as it is
        d = to_device(np.full(m * n, np.nan, dtype=np.float32))
        rw.gemm_mx_packed(orc.E4M3, RM, CM, RM, m, n, k, da, db, None, d, 1.0, 0.0, ws)
        assert np.array_equal(to_host(d, np.float32).view(np.uint32), want.view(np.uint32))
    # new tokens' scales only: the weights' packed scales stay
    sa2 = scales(73, m, k, 125, 129)
    rw.gemm_mx_pack_scales(RM, CM, RM, m, n, k, to_device(sa2), None, ws)
    d = to_device(np.full(m * n, np.nan, dtype=np.float32))
    rw.gemm_mx_packed(orc.E4M3, RM, CM, RM, m, n, k, da, db, None, d, 1.0, 0.0, ws)
    want2 = run_mx(orc.E4M3, RM, CM, RM, m, n, k, a, sa2, b, sb, None, 1.0, 0.0, True)
    assert np.array_equal(to_host(d, np.float32).view(np.uint32), want2.view(np.uint32))
    want_cpu = orc.gemm_mx(orc.E4M3, RM, CM, RM, RM, m, n, k, a, sa2, b, sb, None, 1.0, 0.0, rows=np.arange(0, m, 61, dtype=np.uint32))
    rows = np.arange(0, m, 61)
    assert np.array_equal(want2.reshape(m, n)[rows], want_cpu.reshape(m, n)[rows])


def test_packed_entry_points_reject_what_the_blocked_kernels_do_not_take():
    import torch

    m, n, k = 128, 256, 256
    ws = torch.empty(rw.gemm_mx_workspace_size(m, n, k), dtype=torch.uint8, device="cuda")
    sa, sb = to_device(scales(1, m, k, 127, 127)), to_device(scales(2, n, k, 127, 127))
    with pytest.raises(rw.RocwmmaError) as e:  # both operands row-major: one block per wave only
        rw.gemm_mx_pack_scales(RM, RM, RM, m, n, k, sa, sb, ws)
    assert e.value.status == 3
    with pytest.raises(rw.RocwmmaError) as e:  # nothing to pack
        rw.gemm_mx_pack_scales(RM, CM, RM, m, n, k, None, None, ws)
    assert e.value.status == 1
    with pytest.raises(rw.RocwmmaError) as e:  # workspace too small
        rw.gemm_mx_pack_scales(RM, CM, RM, m, n, k, sa, sb, ws[:256])
    assert e.value.status == 1
    a = to_device(exact_int_bits(orc.E4M3, m, k, RM))
    b = to_device(exact_int_bits(orc.E4M3, k, n, CM))
    d = torch.empty(m * n, device="cuda")
    with pytest.raises(rw.RocwmmaError) as e:  # k not in whole 128-byte stages
        rw.gemm_mx_packed(orc.E4M3, RM, CM, RM, m, n, 192, a, b, None, d, 1.0, 0.0, ws)
    assert e.value.status == 3


@pytest.mark.parametrize("workspace", [False, True])
@pytest.mark.parametrize("m,n,k", [(64, 96, 256), (256, 256, 256)])
def test_end_points_of_the_scale_range_in_live_positions(m, n, k, workspace):
    """E8M0 bytes 0 (2^-127) and 254 (2^127) on blocks that hold non-zero elements: A's blocks of every third row at
    2^-127 (and of the rows behind them at 2^-126) against B's at 2^127 in the first K block, unit scales elsewhere.
    Elements 0, -1, -2 in A and 0, -1 in B, so every product and every partial sum is exact and must match bit for
    bit; a kernel that flushed the small scale or saturated the large one before multiplying would not."""
    a = exact_int_bits(orc.E4M3, m, k, RM)
    bmat = -((np.arange(k)[:, None] + np.arange(n)[None, :]) % 2).astype(np.float32)  # k x n, values 0 / -1
    b = orc.encode(orc.E4M3, np.ascontiguousarray(bmat.T).reshape(-1))  # col-major
    sa = np.full((m, k // 32), 127, dtype=np.uint8)
    sb = np.full((n, k // 32), 127, dtype=np.uint8)
    sa[::3, 0] = 0
    sb[:, 0] = 254
    sa[1::3, 0] = 1  # 2^-126 against 2^127: the block's products are doubled
    sa[2::3, 0] = 2  # and here times four (a unit scale against 2^127 would overflow)
    got = run_mx(orc.E4M3, RM, CM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0, workspace)
    # (the oracle dequantises each operand on its own; every element times its scale is representable here)
    want = orc.gemm_mx(orc.E4M3, RM, CM, RM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0)
    assert np.isfinite(want).all() and np.abs(want).max() < 2.0 ** 24
    # rows whose first block is scaled by 2^-127 * 2^127 = 1 equal the product with unit scales everywhere
    unit = orc.gemm_mx(orc.E4M3, RM, CM, RM, RM, m, n, k, a, np.full_like(sa, 127), b, np.full_like(sb, 127), None, 1.0, 0.0)
    assert np.array_equal(want.reshape(m, n)[::3], unit.reshape(m, n)[::3])
    assert np.array_equal(got, want)


@pytest.mark.parametrize("workspace", [False, True])
def test_nan_scale_poisons_its_row_only(workspace):
    """Scale byte 255 is NaN: every output that block contributes to is NaN, every other output is untouched."""
    m, n, k = 64, 96, 256
    a, b = exact_int_bits(orc.E4M3, m, k, RM), exact_int_bits(orc.E4M3, k, n, CM)
    sa, sb = scales(31, m, k, 126, 128), scales(32, n, k, 126, 128)
    sa[5, 1] = 255
    sb[17, 0] = 255
    got = run_mx(orc.E4M3, RM, CM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0, workspace).reshape(m, n)
    want = orc.gemm_mx(orc.E4M3, RM, CM, RM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0).reshape(m, n)
    assert np.isnan(want[5]).all() and np.isnan(want[:, 17]).all() and np.isnan(want).sum() == n + m - 1
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(want)], want[~np.isnan(want)])


@pytest.mark.parametrize("dtype", [orc.E4M3, orc.E5M2])
@pytest.mark.parametrize("m,n,k", [(128, 4160, 4096), (48, 8192, 4224), (112, 14336, 4096)])
def test_one_round_of_narrow_tiles_on_the_ring_of_four_line_stages(dtype, m, n, k):
    """One round of 128 x 64 tiles with at least 4 KiB of K per row (on a 256-unit device): the scaled tile on the
    ring of four 128-byte stages, whose scale loads join the count of operations in flight.  An even and an odd
    number of stages, a partly filled row of tiles, every scale different: exact pattern bit for bit, random
    operands within the fp8 tolerance against sampled oracle rows."""
    a = exact_int_bits(dtype, m, k, RM)
    b = exact_int_bits(dtype, k, n, CM)
    sa, sb = scales(101, m, k, 125, 129), scales(102, n, k, 125, 129)
    rows = np.arange(0, m, 5, dtype=np.uint32)
    got = run_mx(dtype, RM, CM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0, True)
    want = orc.gemm_mx(dtype, RM, CM, RM, RM, m, n, k, a, sa, b, sb, None, 1.0, 0.0, rows=rows)
    check(np.ascontiguousarray(got.reshape(m, n)[rows]).ravel(), np.ascontiguousarray(want.reshape(m, n)[rows]).ravel(), 0.0)
    a, b = uniform_bits(103, dtype, m * k), uniform_bits(104, dtype, k * n)
    c = uniform_bits(105, orc.F32, m * n)
    got = run_mx(dtype, RM, CM, RM, m, n, k, a, sa, b, sb, c, 0.5, 2.0, True)
    want = orc.gemm_mx(dtype, RM, CM, RM, RM, m, n, k, a, sa, b, sb, c, 0.5, 2.0, rows=rows)
    check(np.ascontiguousarray(got.reshape(m, n)[rows]).ravel(), np.ascontiguousarray(want.reshape(m, n)[rows]).ravel(), 1e-2)
