"""The benchmark build of the blocked GEMM's 256 x 256 kernel (time stamps in its main loop,
librocwmma_amd_aux.so): its result must be the product kernel's bit for bit, and its trace must add up."""
import numpy as np
import pytest

import rocwmma_amd as rw
from util import CM, RM

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,la,lb", [(rw.F16, RM, CM), (rw.F16, RM, RM), (rw.BF16, CM, CM), (rw.I8, RM, CM), (rw.I8, CM, RM)])
def test_traced_kernel_matches_the_product_kernel_and_its_trace_adds_up(dtype, la, lb):
    import torch

    m, n, k = 512, 768, 1024
    g = torch.Generator(device="cuda").manual_seed(0x5EED0401)
    if dtype == rw.I8:
        a = torch.randint(-128, 128, (m * k,), device="cuda", dtype=torch.int8, generator=g)
        b = torch.randint(-128, 128, (k * n,), device="cuda", dtype=torch.int8, generator=g)
        c = torch.randint(-1000, 1000, (m * n,), device="cuda", dtype=torch.int32, generator=g)
        out, alpha, beta = rw.I32, 1.0, 2.0
    else:
        tdt = torch.float16 if dtype == rw.F16 else torch.bfloat16
        a = (torch.rand(m * k, device="cuda", generator=g) * 2 - 1).to(tdt)
        b = (torch.rand(k * n, device="cuda", generator=g) * 2 - 1).to(tdt)
        c = torch.rand(m * n, device="cuda", generator=g) * 2 - 1
        out, alpha, beta = rw.F32, 0.5, 1.5
    want = torch.empty_like(c)
    rw.gemm(dtype, out, la, lb, RM, m, n, k, a, b, c, want, alpha, beta, algo=rw.GEMM_BLOCKED_256)
    got = torch.full_like(c, 7)
    tiles, waves = (m // 256) * (n // 256), 8
    trace = torch.full((tiles * waves * 8,), -1, device="cuda", dtype=torch.int64)
    rw.bench_phase_trace(dtype, la, lb, m, n, k, a, b, c, got, alpha, beta, trace)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    t = trace.cpu().numpy().reshape(tiles, waves, 8)
    stages = k * a.element_size() // 128
    assert np.all(t[:, :, 5] == stages)
    parts = t[:, :, 0] + t[:, :, 1] + t[:, :, 2] + t[:, :, 3]
    assert np.all(t[:, :, :5] > 0)
    # the four parts are the loop's time stamps end to end: they add up to the loop within the few clocks
    # between the last stamp of the loop and the one that closes it
    assert np.all(parts <= t[:, :, 4]) and np.all(t[:, :, 4] - parts < 4000)
    # every stage holds 64 MFMAs of 16 clocks per wave
    assert np.all(t[:, :, 4] >= stages * 1024)


def test_phase_trace_argument_checks():
    import torch

    a = torch.zeros(256 * 256, device="cuda", dtype=torch.float16)
    c = torch.zeros(256 * 256, device="cuda")
    small = torch.zeros(8, device="cuda", dtype=torch.int64)
    with pytest.raises(rw.RocwmmaError):  # trace buffer too small
        rw.bench_phase_trace(rw.F16, RM, CM, 256, 256, 256, a, a, c, c, 1.0, 0.0, small)
    trace = torch.zeros(64, device="cuda", dtype=torch.int64)
    with pytest.raises(rw.RocwmmaError):  # not whole 256 x 256 tiles
        rw.bench_phase_trace(rw.F16, RM, CM, 128, 256, 256, a, a, c, c, 1.0, 0.0, trace)
    with pytest.raises(rw.RocwmmaError):  # fp8 is not built with time stamps
        rw.bench_phase_trace(rw.E4M3, RM, CM, 256, 256, 256, a, a, c, c, 1.0, 0.0, trace)
