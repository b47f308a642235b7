"""GEMV parity: Y = alpha*A*X + beta*Y (f16 A row-major, 1..8 right-hand sides) against the CPU
oracle (gemm_CPU with n columns == sgemv_cpu_h, samples/simple_sgemv.cpp:46-66)."""
import numpy as np
import pytest

import oracle as orc
import rocwmma_amd as rw
from util import CM, RM, to_device, uniform_bits

pytestmark = pytest.mark.gpu


def run(m, k, ncols, alpha, beta, seed, lda=None):
    import torch

    lda = lda or k
    a = uniform_bits(seed, orc.F16, m * lda)
    x = uniform_bits(seed + 1, orc.F16, k * ncols)
    y0 = np.random.default_rng(seed + 2).uniform(-1, 1, m * ncols).astype(np.float32)
    y = to_device(y0.copy()) if beta != 0 else torch.full((m * ncols,), float("nan"), device="cuda")
    rw.gemv(m, k, ncols, to_device(a), to_device(x), y, alpha, beta, lda=lda)
    torch.cuda.synchronize()
    a_used = np.ascontiguousarray(a.reshape(m, lda)[:, :k])
    want = orc.gemm(orc.F16, orc.F32, RM, CM, CM, CM, m, ncols, k, a_used, x, y0 if beta != 0 else None, alpha, beta)
    err, inf, nan = orc.compare_equal(orc.F32, y.cpu().numpy(), orc.F32, want)
    assert not inf and not nan and err <= 1e-3, (err, inf, nan)


@pytest.mark.parametrize("ncols", [1, 4, 8])
@pytest.mark.parametrize("m,k", [(8192, 8192), (14336, 4096)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_config4_full_shapes(m, k, ncols, beta):
    run(m, k, ncols, 1.0, beta, 0x5EED0004 + ncols)


@pytest.mark.parametrize("m,k,ncols", [(1, 8, 1), (3, 520, 2), (37, 1000, 4), (130, 72, 8), (255, 4104, 1),
                                       (2, 16, 1), (5, 24, 1), (64, 16384, 8), (100, 32776, 4), (9, 65536, 2),
                                       (1000, 8, 8), (4100, 264, 2),
                                       # m a multiple of 16 and k a multiple of 4096
                                       (48, 4096, 4), (16, 8192, 8), (2064, 4096, 8), (80, 8192, 4),
                                       # 8 columns, m % 4 == 0, k % 1024 == 0 but not % 4096; one row quad
                                       (100, 3072, 8), (4, 1024, 8), (1028, 2048, 8), (100, 3072, 4), (12, 1024, 4)])
def test_ragged_shapes(m, k, ncols):
    run(m, k, ncols, 2.1, 2.1, 99)


def test_padded_leading_dimension():
    run(64, 512, 4, 1.0, 0.0, 5, lda=640)
    run(64, 4096, 8, 1.0, 0.5, 6, lda=4096 + 64)


def test_equals_gemm_with_n_columns():
    """GEMV is GEMM with n columns: same inputs through the GEMM entry point (padded to 16
    columns of zeros) give the same answer up to summation order."""
    import torch

    m, k, ncols = 256, 512, 8
    a = uniform_bits(1, orc.F16, m * k)
    x = uniform_bits(2, orc.F16, k * ncols)
    y = torch.zeros(m * ncols, device="cuda")
    rw.gemv(m, k, ncols, to_device(a), to_device(x), y)
    xpad = np.zeros(k * 16, dtype=np.uint16)
    xpad[: k * ncols] = x
    d = torch.zeros(m * 16, device="cuda")
    rw.gemm(rw.F16, rw.F32, RM, CM, CM, m, 16, k, to_device(a), to_device(xpad), None, d, 1.0, 0.0)
    torch.cuda.synchronize()
    assert torch.allclose(y, d[: m * ncols], rtol=0, atol=1e-3)
    assert float(d[m * ncols:].abs().max()) == 0.0
