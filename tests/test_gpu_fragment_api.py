"""On-GPU semantics of the public fragment API, through the C ABI self-test kernels.

Mirrors the reference's unit tests: load/store identity for matrix_a, matrix_b and accumulator
fragments in both layouts (test/unit/load_store_matrix_sync_test), the cooperative twin
(test/unit/load_store_matrix_coop_sync_test), untouched padding (test/unit/contamination_test),
and the perf_hgemm data flow (cooperative loads + transforms + mma_sync) against the CPU oracle."""
import numpy as np
import pytest

import oracle as orc
import rocwmma_amd as rw
from util import CM, RM, to_device, to_host, uniform_bits

pytestmark = pytest.mark.gpu

NP = {rw.F16: np.uint16, rw.I8: np.int8, rw.F32: np.float32}


def _shape(context, block, blockk):
    if context == 0:
        return block, blockk          # matrix_a: BlockM x BlockK
    if context == 1:
        return blockk, block          # matrix_b: BlockK x BlockN
    return block, block               # accumulator: BlockM x BlockN


@pytest.mark.parametrize("coop", [0, 1])
@pytest.mark.parametrize("layout", [RM, CM])
@pytest.mark.parametrize("context", [0, 1, 2])
@pytest.mark.parametrize("dtype,block,blockk", [
    (rw.F16, 16, 16), (rw.F16, 32, 16), (rw.F16, 16, 64), (rw.F16, 32, 64), (rw.F16, 64, 16),
    (rw.I8, 16, 64), (rw.I8, 32, 64), (rw.I8, 32, 128), (rw.I8, 16, 16),
    (rw.F32, 16, 16), (rw.F32, 32, 16), (rw.F32, 64, 64),
    # the rest of the reference's unit-test matrix (test/unit/unit_test_params.hpp:89-141):
    # BlockK 8 .. 256 and blocks up to 256
    (rw.F16, 32, 8), (rw.F16, 64, 32), (rw.F16, 16, 256), (rw.F16, 128, 8), (rw.F16, 128, 32), (rw.F16, 256, 8),
    (rw.F16, 256, 32), (rw.I8, 64, 8), (rw.I8, 16, 256), (rw.I8, 128, 32), (rw.I8, 256, 8),
    (rw.F32, 32, 8), (rw.F32, 16, 128), (rw.F32, 128, 8), (rw.F32, 256, 32),
])
def test_load_store_identity_and_no_contamination(dtype, block, blockk, context, layout, coop):
    import torch

    if context == 2 and block > 64:
        pytest.skip("an accumulator block above 64 x 64 does not fit a wave's registers")
    h, w = _shape(context, block, blockk)
    tiles_r, tiles_c = 3, 2
    rows, cols = tiles_r * h, tiles_c * w
    pad = 16  # elements of padding in the leading dimension: must stay untouched
    ld = -(-(cols if layout == RM else rows) // 16) * 16 + pad  # multiple of 16 elements (alignment rule of the ABI)
    outer = rows if layout == RM else cols
    np_t = NP[dtype]
    if dtype == rw.F32:
        src = np.random.default_rng(1).uniform(-1, 1, outer * ld).astype(np.float32)
    else:
        src = uniform_bits(1, {rw.F16: orc.F16, rw.I8: orc.I8}[dtype], outer * ld)
    sentinel = np.full(outer * ld, 0x5A if dtype == rw.I8 else (0x7B5A if dtype == rw.F16 else 12345.0), dtype=np_t)
    d_in, d_out = to_device(src), to_device(sentinel)
    rw.selftest_roundtrip(context, dtype, layout, block, blockk, coop, rows, cols, d_in, d_out, ld)
    torch.cuda.synchronize()
    got = to_host(d_out, np_t).reshape(outer, ld)
    want = src.reshape(outer, ld)
    inner = cols if layout == RM else rows
    assert np.array_equal(got[:, :inner], want[:, :inner]), "tile data changed by load -> store"
    assert np.array_equal(got[:, inner:], sentinel.reshape(outer, ld)[:, inner:]), "padding was written"


@pytest.mark.parametrize("la", [RM, CM])
@pytest.mark.parametrize("lb", [RM, CM])
def test_cooperative_lds_gemm_flow_matches_oracle(la, lb):
    """perf_hgemm's structure written with the public API only (coop loads, applyDataLayout,
    applyTranspose, LDS, mma_sync)."""
    import torch

    m, n, k = 128, 256, 160
    a = uniform_bits(11, orc.F16, m * k)
    b = uniform_bits(12, orc.F16, k * n)
    c = np.random.default_rng(13).uniform(-1, 1, m * n).astype(np.float32)
    d = torch.full((m * n,), float("nan"), device="cuda")
    rw.selftest_coop_gemm(la, lb, m, n, k, to_device(a), to_device(b), to_device(c), d, 2.0, -1.5)
    torch.cuda.synchronize()
    want = orc.gemm(orc.F16, orc.F32, la, lb, RM, RM, m, n, k, a, b, c, 2.0, -1.5)
    err, inf, nan = orc.compare_equal(orc.F32, d.cpu().numpy(), orc.F32, want)
    assert not inf and not nan and err <= 1e-3, err


@pytest.mark.parametrize("la", [RM, CM])
@pytest.mark.parametrize("lb", [RM, CM])
def test_cooperative_flow_exact_on_integer_pattern(la, lb):
    """With the reference's own integer fill every summation order gives the same bits."""
    import torch

    from util import exact_int_bits

    m, n, k = 128, 128, 256
    a = exact_int_bits(orc.F16, m, k, la)
    b = exact_int_bits(orc.F16, k, n, lb)
    c = exact_int_bits(orc.F32, m, n, RM)
    d = torch.full((m * n,), float("nan"), device="cuda")
    rw.selftest_coop_gemm(la, lb, m, n, k, to_device(a), to_device(b), to_device(c), d, 2.0, 2.0)
    torch.cuda.synchronize()
    want = orc.gemm(orc.F16, orc.F32, la, lb, RM, RM, m, n, k, a, b, c, 2.0, 2.0)
    same = np.array_equal(d.cpu().numpy(), want)
    assert same


@pytest.mark.parametrize("la", [RM, CM])
@pytest.mark.parametrize("lb", [RM, CM])
def test_blocked_gemm_through_the_public_api_only(la, lb):
    """The blocked GEMM laid out for gfx950 and written against the fragment API alone (cooperative loads and stores,
    applyDataLayout, applyTranspose, padded LDS slabs, mma_sync on 16 x 16 x 32 blocks): against the oracle, and bit
    for bit on the reference's integer fill; a K of three stages walks both LDS buffers and the tail."""
    import torch

    from util import exact_int_bits

    m, n, k = 512, 256, 192
    a = uniform_bits(21, orc.F16, m * k)
    b = uniform_bits(22, orc.F16, k * n)
    c = np.random.default_rng(23).uniform(-1, 1, m * n).astype(np.float32)
    d = torch.full((m * n,), float("nan"), device="cuda")
    rw.selftest_tiled_gemm(la, lb, m, n, k, to_device(a), to_device(b), to_device(c), d, 2.0, -1.5)
    torch.cuda.synchronize()
    want = orc.gemm(orc.F16, orc.F32, la, lb, RM, RM, m, n, k, a, b, c, 2.0, -1.5)
    err, inf, nan = orc.compare_equal(orc.F32, d.cpu().numpy(), orc.F32, want)
    assert not inf and not nan and err <= 1e-3, err
    a, b, c = exact_int_bits(orc.F16, m, k, la), exact_int_bits(orc.F16, k, n, lb), exact_int_bits(orc.F32, m, n, RM)
    d.fill_(float("nan"))
    rw.selftest_tiled_gemm(la, lb, m, n, k, to_device(a), to_device(b), to_device(c), d, 2.0, 2.0)
    torch.cuda.synchronize()
    assert np.array_equal(d.cpu().numpy(), orc.gemm(orc.F16, orc.F32, la, lb, RM, RM, m, n, k, a, b, c, 2.0, 2.0))
    with pytest.raises(rw.RocwmmaError) as e:  # whole 256 x 256 tiles and 64-wide stages only
        rw.selftest_tiled_gemm(la, lb, 384, n, k, to_device(a), to_device(b), to_device(c), d, 1.0, 0.0)
    assert e.value.status == 3
