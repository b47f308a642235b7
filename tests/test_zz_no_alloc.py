"""The entry point that allocates nothing (rocwmma_amd_gemm_streamk_static: stream-K GEMM on the
library's own static device scratch) against the entry point it is a variant of
(rocwmma_amd_gemm_streamk with a caller-provided workspace), through the C ABI, on two calls in a
row, the second on a smaller input: the scratch keeps the first call's contents, and the second call
must not see them.  Same kernels, same summation order: the results must be identical bit for bit
(int8 -> int32 and f16 -> f32 alike), and they are checked against the CPU oracle as well."""
import numpy as np
import pytest

import oracle as orc
import rocwmma_amd as rw
from util import CM, RM, to_device, to_host, uniform_bits

pytestmark = pytest.mark.gpu


def _both(dtype_in, dtype_out, la, lb, m, n, k, seed, alpha, beta, workspace):
    import torch

    a, b = uniform_bits(seed, dtype_in, m * k), uniform_bits(seed + 1, dtype_in, k * n)
    c = uniform_bits(seed + 2, dtype_out, m * n)
    da, db, dc = to_device(a), to_device(b), to_device(c)
    fill = np.full(m * n, -7, dtype=np.int32) if dtype_out == orc.I32 else np.full(m * n, np.nan, dtype=np.float32)
    d_static, d_ws = to_device(fill), to_device(fill)
    rw.gemm_streamk_static(dtype_in, dtype_out, la, lb, RM, m, n, k, da, db, dc, d_static, alpha, beta)
    rw.gemm_streamk(dtype_in, dtype_out, la, lb, RM, m, n, k, da, db, dc, d_ws, alpha, beta, workspace)
    torch.cuda.synchronize()
    got = to_host(d_static, orc.storage_dtype(dtype_out))
    ref = to_host(d_ws, orc.storage_dtype(dtype_out))
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), f"{(got.view(np.uint32) != ref.view(np.uint32)).sum()} elements differ"
    want = orc.gemm(dtype_in, dtype_out, la, lb, RM, RM, m, n, k, a, b, c, alpha, beta)
    if dtype_out == orc.I32:
        assert np.array_equal(got, want)
    else:
        err, inf, nan = orc.compare_equal(dtype_out, got, dtype_out, want)
        assert not inf and not nan and err <= 1e-3, (err, inf, nan)


@pytest.mark.parametrize("dtype_in,dtype_out,la,lb", [(orc.I8, orc.I32, RM, CM), (orc.F16, orc.F32, RM, CM), (orc.F16, orc.F32, CM, RM)])
def test_static_scratch_entry_point_two_calls_in_a_row(dtype_in, dtype_out, la, lb):
    import torch

    workspace = torch.empty(rw.gemm_streamk_workspace_size(), dtype=torch.uint8, device="cuda")
    alpha, beta = (2.0, -1.0) if dtype_in == orc.I8 else (1.5, 0.5)
    # first call: 20 tiles, every one shared by a dozen workgroups; second call, smaller: 12 tiles
    _both(dtype_in, dtype_out, la, lb, 1280, 1024, 4096, 0x5EED0900, alpha, beta, workspace)
    _both(dtype_in, dtype_out, la, lb, 768, 1024, 3072, 0x5EED0910, alpha, beta, workspace)
    assert not rw.gemm_streamk_timed_out(None), "a stream-K owner on the static scratch gave up waiting"


def test_static_scratch_entry_point_leaves_free_device_memory_unchanged():
    """After a warm-up call (which resolves the scratch's address and sets the kernel's LDS attribute), calls of
    the entry point must not change what the device reports as free memory."""
    import torch

    m, n, k = 1024, 1024, 2048
    a, b = to_device(uniform_bits(1, orc.I8, m * k)), to_device(uniform_bits(2, orc.I8, k * n))
    d = torch.empty(m * n, dtype=torch.int32, device="cuda")
    call = lambda: rw.gemm_streamk_static(orc.I8, orc.I32, RM, CM, RM, m, n, k, a, b, None, d, 1.0, 0.0)
    call()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    call()
    call()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
