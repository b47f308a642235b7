"""Stream-K GEMM entry point (rocwmma_amd_gemm_streamk) on the GPU: parity with the CPU oracle and with
the one-tile-per-workgroup kernel on the same bits, on shapes whose tiles are shared by many
workgroups (few tiles, long K), by two (a half round left over) and by none.  int8 -> int32 bit-exact;
f16 / bf16 <= 1e-3, fp8 <= 1e-2 in the reference's compareEqual metric; results identical from run
to run."""
import numpy as np
import pytest

import oracle as orc
import rocwmma_amd as rw
from util import CM, RM, normal_fp8_bits, to_device, to_host, tol_for, uniform_bits

pytestmark = pytest.mark.gpu

OUT_OF = {orc.F16: orc.F32, orc.BF16: orc.F32, orc.E4M3: orc.F32, orc.E5M2: orc.F32, orc.I8: orc.I32}


@pytest.fixture(scope="module")
def workspace():
    import torch

    size = rw.gemm_streamk_workspace_size()
    assert size >= 256 * 256 * 4
    # garbage on purpose: the entry point must not depend on the workspace's contents
    # (bytes below 0x45: the garbage cannot spell the time-out value)
    return torch.randint(0, 0x45, (size,), dtype=torch.uint8, device="cuda")


TIMED_OUT = 0x54494D45  # what a wait that ran out leaves in the workspace (include/rocwmma_amd.h)


def marker_word(workspace):
    """The word behind the flags that records a wait that ran out (offset documented in include/rocwmma_amd.h)."""
    cus = rw.device_info()["compute_units"]
    return workspace[cus * 256 * 256 * 4:].view(__import__("torch").int32)[cus:cus + 1]


def run_streamk(dtype_in, la, lb, lc, m, n, k, a, b, c, alpha, beta, workspace):
    import torch

    dtype_out = OUT_OF[dtype_in]
    sentinel = np.full(m * n, -123456789, dtype=np.int32) if dtype_out == orc.I32 else np.full(m * n, np.nan, dtype=np.float32)
    d = to_device(sentinel)
    rw.gemm_streamk(dtype_in, dtype_out, la, lb, lc, m, n, k, to_device(a), to_device(b),
                    None if c is None else to_device(c), d, alpha, beta, workspace)
    assert not rw.gemm_streamk_timed_out(workspace), "a stream-K owner gave up waiting for a contributor"
    return to_host(d, orc.storage_dtype(dtype_out))


def inputs(dtype_in, m, n, k, seed):
    if dtype_in in (orc.E4M3, orc.E5M2):
        a, b = normal_fp8_bits(seed, dtype_in, m * k), normal_fp8_bits(seed + 1, dtype_in, k * n)
    else:
        a, b = uniform_bits(seed, dtype_in, m * k), uniform_bits(seed + 1, dtype_in, k * n)
    c = uniform_bits(seed + 2, OUT_OF[dtype_in], m * n)
    return a, b, c


def check(dtype_in, got, want):
    tol = tol_for(dtype_in)
    if tol == 0.0:
        assert np.array_equal(got, want), f"{(got != want).sum()} of {got.size} elements differ"
        return
    err, inf, nan = orc.compare_equal(OUT_OF[dtype_in], got, OUT_OF[dtype_in], want)
    assert not inf and not nan and err <= tol, (err, inf, nan)


@pytest.mark.parametrize("dtype_in,la,lb,lc", [
    (orc.F16, RM, CM, RM), (orc.F16, RM, RM, RM), (orc.F16, CM, RM, RM), (orc.F16, CM, CM, CM),
    (orc.BF16, RM, CM, RM), (orc.BF16, CM, RM, CM), (orc.I8, RM, CM, RM), (orc.I8, RM, CM, CM),
    (orc.E4M3, RM, CM, RM), (orc.E5M2, RM, CM, RM),
    # 8-bit operands with a dim-major side (int8 on 16-wide blocks, fp8 on 32 x 32 x 64)
    (orc.I8, RM, RM, RM), (orc.I8, CM, RM, CM), (orc.I8, CM, CM, RM),
    (orc.E4M3, RM, RM, RM), (orc.E4M3, CM, RM, RM), (orc.E4M3, CM, CM, CM), (orc.E5M2, CM, RM, RM),
])
@pytest.mark.parametrize("m,n,k", [(1024, 1024, 2048), (1280, 768, 4096)])
def test_tiles_shared_by_many_workgroups_against_oracle(dtype_in, la, lb, lc, m, n, k, workspace):
    """Fewer tiles than compute units: every tile's K range is spread over many workgroups."""
    a, b, c = inputs(dtype_in, m, n, k, 0x5EED0700 + m)
    alpha, beta = (2.0, -1.0) if dtype_in == orc.I8 else (1.5, 0.5)
    got = run_streamk(dtype_in, la, lb, lc, m, n, k, a, b, c, alpha, beta, workspace)
    want = orc.gemm(dtype_in, OUT_OF[dtype_in], la, lb, lc, lc, m, n, k, a, b, c, alpha, beta)
    check(dtype_in, got, want)
    # the same call again: identical bits (fixed summation order), also with beta = 0 and no C
    again = run_streamk(dtype_in, la, lb, lc, m, n, k, a, b, c, alpha, beta, workspace)
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    got0 = run_streamk(dtype_in, la, lb, lc, m, n, k, a, b, None, alpha, 0.0, workspace)
    want0 = orc.gemm(dtype_in, OUT_OF[dtype_in], la, lb, lc, lc, m, n, k, a, b, None, alpha, 0.0)
    check(dtype_in, got0, want0)


@pytest.mark.parametrize("dtype_in", [orc.I8, orc.F16])
def test_half_round_left_over_against_plain_kernel(dtype_in, workspace):
    """896 tiles on 256 compute units (the quantised-inference shape M = 4096, N = 14336): three whole
    rounds and 128 tiles shared by two workgroups each.  Against the one-tile kernel on the same bits
    (int8: every element equal) and against the oracle on sampled rows."""
    import torch

    m, n, k = 4096, 14336, 512
    a, b, c = inputs(dtype_in, m, n, k, 0x5EED0711)
    got = run_streamk(dtype_in, RM, CM, RM, m, n, k, a, b, c, 1.0, 1.0, workspace)
    out = OUT_OF[dtype_in]
    d = to_device(np.zeros(m * n, dtype=orc.storage_dtype(out)))
    rw.gemm(dtype_in, out, RM, CM, RM, m, n, k, to_device(a), to_device(b), to_device(c), d, 1.0, 1.0, algo=rw.GEMM_BLOCKED_256)
    torch.cuda.synchronize()
    plain = to_host(d, orc.storage_dtype(out))
    check(dtype_in, got, plain)
    rows = np.arange(0, m, m // 32, dtype=np.uint32)
    want = orc.gemm(dtype_in, out, RM, CM, RM, RM, m, n, k, a, b, c, 1.0, 1.0, rows=rows)
    check(dtype_in, got.reshape(m, n)[rows].ravel(), want.reshape(m, n)[rows].ravel())


def test_whole_rounds_only(workspace):
    """A tile count that is a multiple of the unit count: one round is still run through the shared
    path (each workgroup owns one whole tile of it)."""
    m, n, k = 4096, 4096, 256
    a, b, c = inputs(orc.I8, m, n, k, 0x5EED0722)
    got = run_streamk(orc.I8, RM, CM, RM, m, n, k, a, b, c, 1.0, 0.0, workspace)
    rows = np.arange(0, m, m // 64, dtype=np.uint32)
    want = orc.gemm(orc.I8, orc.I32, RM, CM, RM, RM, m, n, k, a, b, c, 1.0, 0.0, rows=rows)
    assert np.array_equal(got.reshape(m, n)[rows], want.reshape(m, n)[rows])


def test_argument_errors(workspace):
    import torch

    m = n = 1024
    k = 2048
    a, b, c = inputs(orc.F16, m, n, k, 1)
    da, db, dc = to_device(a), to_device(b), to_device(c)
    d = torch.empty(m * n, device="cuda")
    with pytest.raises(rw.RocwmmaError) as e:  # workspace too small
        rw.gemm_streamk(rw.F16, rw.F32, RM, CM, RM, m, n, k, da, db, dc, d, 1.0, 0.0, workspace[:4096])
    assert e.value.status == 1
    with pytest.raises(rw.RocwmmaError) as e:  # not whole 256 x 256 tiles
        rw.gemm_streamk(rw.F16, rw.F32, RM, CM, RM, 128, n, k, da, db, dc, d, 1.0, 0.0, workspace)
    assert e.value.status == 3
    with pytest.raises(rw.RocwmmaError) as e:  # too little work to share (fewer K stages than compute units)
        rw.gemm_streamk(rw.F16, rw.F32, RM, CM, RM, 256, 256, 256, da, db, dc, d, 1.0, 0.0, workspace)
    assert e.value.status == 3


def test_timed_out_query_reports_once_and_launches_do_not_clear_it(workspace):
    """No kernel is made to wait: the host itself writes the value a wait that ran out would leave, behind
    a finished launch.  The next launch must not clear it; the query reports it once and clears it."""
    import torch

    m, n, k = 1024, 1024, 2048
    a, b, c = inputs(orc.I8, m, n, k, 0x5EED0733)
    want = run_streamk(orc.I8, RM, CM, RM, m, n, k, a, b, c, 1.0, 0.0, workspace)  # (asserts: no time-out)
    assert not rw.gemm_streamk_timed_out(workspace)
    marker_word(workspace).fill_(TIMED_OUT)
    torch.cuda.synchronize()
    d = to_device(np.zeros(m * n, dtype=np.int32))
    rw.gemm_streamk(orc.I8, orc.I32, RM, CM, RM, m, n, k, to_device(a), to_device(b), None, d, 1.0, 0.0, workspace)
    assert np.array_equal(to_host(d, np.int32), want)
    assert rw.gemm_streamk_timed_out(workspace), "a later launch hid an earlier time-out"
    assert not rw.gemm_streamk_timed_out(workspace), "the query reports a time-out once"
    with pytest.raises(rw.RocwmmaError) as e:  # a workspace that cannot hold the marker
        rw.gemm_streamk_timed_out(workspace[:4096])
    assert e.value.status == 1
