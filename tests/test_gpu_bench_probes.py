"""The measurement probes of the auxiliary library (include/rocwmma_amd_aux.h) on the GPU: they launch, report
the operation and byte counts the benchmark divides by, leave their outputs finite, and reject what they cannot
run.  (They have no numerical result to compare: what they are for is their duration.)"""
import numpy as np
import pytest

import rocwmma_amd as rw

pytestmark = pytest.mark.gpu


def test_matrix_pipes_next_to_their_operand_streams():
    import torch

    units = rw.device_info()["compute_units"]
    s = 8192
    a = (torch.rand(s * s, device="cuda") * 2 - 1).to(torch.float16)
    table = a[:32768].contiguous().view(torch.uint8)
    out = torch.full((units * 512,), float("nan"), device="cuda")
    for streams in (0, 1, 3):
        ops = rw.bench_mfma_streams(streams, 1, a, a, table, out)
        torch.cuda.synchronize()
        assert ops == 2.0 * 256 * 256 * 8192 * units
        assert bool(torch.isfinite(out).all())
    assert rw.bench_mfma_streams(3, 2, a, a, table, out) == 2 * 2.0 * 256 * 256 * 8192 * units
    torch.cuda.synchronize()
    # the 8-bit kinds walk rows of the same 16 KiB: twice the K
    a8 = torch.randint(-128, 128, (s * s * 2,), device="cuda", dtype=torch.int8)
    f8 = (torch.randn(s * s * 2, device="cuda") * 0.1).to(torch.float8_e4m3fn)
    for kind, panel in ((rw.STREAMS_I8, a8), (rw.STREAMS_FP8, f8)):
        for streams in (0, 1, 3):
            out.fill_(float("nan"))
            ops = rw.bench_mfma_streams(streams, 1, panel, panel, panel.view(torch.uint8)[:65536].contiguous(), out, kind)
            torch.cuda.synchronize()
            assert ops == 2.0 * 256 * 256 * 16384 * units
            assert bool(torch.isfinite(out).all())
    with pytest.raises(rw.RocwmmaError) as e:  # unknown instruction kind
        rw.bench_mfma_streams(0, 1, a, a, table, out, 3)
    assert e.value.status == 1
    for bad in (2, 4, -1):  # copies without reads, unknown bits
        with pytest.raises(rw.RocwmmaError) as e:
            rw.bench_mfma_streams(bad, 1, a, a, table, out)
        assert e.value.status == 1
    with pytest.raises(rw.RocwmmaError) as e:  # copies need the panels
        rw.bench_mfma_streams(3, 1, None, None, table, out)
    assert e.value.status == 1
    with pytest.raises(rw.RocwmmaError) as e:  # more tiles than the walked problem has
        rw.bench_mfma_streams(0, 1024 // units + 1, a, a, table, out)
    assert e.value.status == 3


def test_memory_stream_probes_move_what_they_say():
    import torch

    n = 4 << 20
    src = torch.randint(0, 255, (2 * n,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros(n + 64, dtype=torch.uint8, device="cuda")
    rw.bench_stream(rw.STREAM_COPY, src, dst, n)
    torch.cuda.synchronize()
    assert torch.equal(dst[:n], src[:n]) and int(dst[n:].sum()) == 0
    dst.zero_()
    rw.bench_stream(rw.STREAM_COPY_READ_MORE, src, dst, n)
    torch.cuda.synchronize()
    assert torch.equal(dst[:n], src[:n]) and int(dst[n + 4:].sum()) == 0
    rw.bench_stream(rw.STREAM_WRITE, None, dst, n)
    torch.cuda.synchronize()
    assert np.array_equal(dst[:16].cpu().numpy().view(np.uint32), np.array([1, 2, 3, 4], dtype=np.uint32))
    assert int(dst[n:].sum()) == 0
    rw.bench_stream(rw.STREAM_READ, src, dst, n)
    torch.cuda.synchronize()
    # the cache-resident read: reads its bytes over and over and writes nothing but (practically never) its sink word
    dst.zero_()
    rw.bench_stream(rw.STREAM_READ_RESIDENT, src, dst, n)
    torch.cuda.synchronize()
    assert int(dst[4:].sum()) == 0
    with pytest.raises(rw.RocwmmaError) as e:
        rw.bench_stream(5, src, dst, n)
    assert e.value.status == 1
    with pytest.raises(rw.RocwmmaError) as e:  # whole 64 KiB trips only
        rw.bench_stream(rw.STREAM_COPY, src, dst, n + 32768)
    assert e.value.status == 3
