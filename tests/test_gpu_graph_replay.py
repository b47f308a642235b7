"""Every entry-point family recorded into a HIP graph and replayed: a caller that captures its launches
(serving loops do) must get, on every replay, what the same call gives when it is launched directly.

The entry points enqueue kernels only (the stream-K flags and the K-sliced kernel's D = beta * C are
set by small kernels, not by memsets), so a capture holds everything a call does.  Each case runs
directly first, is then captured once and replayed three times; between replays the output is
overwritten and the program does other work and synchronises.  The paths tested sum in a fixed order
(the K-sliced kernel's atomic adds are tested on int32, where any order is exact), so a replay must
reproduce the direct result bit for bit."""
import numpy as np
import pytest

import oracle as orc
import rocwmma_amd as rw
from util import CM, RM, normal_fp8_bits, to_device, uniform_bits

pytestmark = pytest.mark.gpu


def _replays_match(call, outputs):
    """call(): enqueues the work on the current stream, writing `outputs` (device tensors)."""
    import torch

    def poison():
        for t in outputs:
            t.fill_(-3 if not t.is_floating_point() else float("nan"))

    poison()
    call()
    torch.cuda.synchronize()
    direct = [t.clone() for t in outputs]
    for t in direct:
        assert not (t.is_floating_point() and bool(torch.isnan(t.float()).any())), "direct call left output unwritten"

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    other = torch.arange(1 << 16, device="cuda", dtype=torch.float32)
    for replay in range(3):
        poison()
        other.mul_(1.0001)  # the program's own work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for t, want in zip(outputs, direct):
            same = torch.equal(t.view(torch.uint8), want.view(torch.uint8))
            assert same, f"replay {replay}: {(t.view(torch.uint8) != want.view(torch.uint8)).sum().item()} bytes differ"


@pytest.mark.parametrize("dtype_in,dtype_out,m,n,k,algo", [
    (orc.F16, orc.F32, 256, 256, 256, rw.GEMM_AUTO),  # blocked kernel, small tiles
    (orc.F16, orc.F32, 256, 256, 512, rw.GEMM_BLOCKED_256),  # the 256 x 256 configuration
    (orc.BF16, orc.F32, 512, 768, 1024, rw.GEMM_AUTO),
    (orc.F16, orc.F32, 64, 64, 64, rw.GEMM_WAVE_TILE),
    (orc.I8, orc.I32, 16, 352, 1024, rw.GEMM_AUTO),  # weight-streaming kernel
    (orc.E4M3, orc.F32, 32, 352, 2048, rw.GEMM_AUTO),
    (orc.I8, orc.I32, 48, 352, 1024, rw.GEMM_AUTO),  # K-sliced kernel: D = beta * C by a kernel, then atomic adds
    (orc.I8, orc.I32, 128, 1024, 4096, rw.GEMM_AUTO),  # 128 x 64 tiles on the ring of four 128-byte stages
])
def test_gemm_replays(dtype_in, dtype_out, m, n, k, algo):
    import torch

    if dtype_in in (orc.E4M3, orc.E5M2):
        a, b = normal_fp8_bits(11, dtype_in, m * k), normal_fp8_bits(12, dtype_in, k * n)
    else:
        a, b = uniform_bits(11, dtype_in, m * k), uniform_bits(12, dtype_in, k * n)
    c = uniform_bits(13, dtype_out, m * n) if dtype_out == orc.I32 else np.random.default_rng(13).uniform(-1, 1, m * n).astype(np.float32)
    da, db, dc = to_device(a), to_device(b), to_device(c)
    d = torch.empty(m * n, device="cuda", dtype=torch.int32 if dtype_out == orc.I32 else torch.float32)
    _replays_match(lambda: rw.gemm(dtype_in, dtype_out, RM, CM, RM, m, n, k, da, db, dc, d, 2.0, -1.0, algo=algo), [d])
    # and the replayed result is the right one
    want = orc.gemm(dtype_in, dtype_out, RM, CM, RM, RM, m, n, k, a, b, c, 2.0, -1.0)
    got = d.cpu().numpy()
    if dtype_out == orc.I32:
        assert np.array_equal(got, want)
    else:
        err, inf, nan = orc.compare_equal(dtype_out, got, dtype_out, want)
        assert not inf and not nan and err <= (1e-2 if dtype_in == orc.E4M3 else 1e-3), (err, inf, nan)


@pytest.mark.parametrize("static", [False, True])
def test_stream_k_replays(static):
    """The stream-K kernel's flags are cleared by a kernel in front of it: every replay starts from zero."""
    import torch

    m, n, k = 1280, 1024, 4096
    a, b = uniform_bits(21, orc.I8, m * k), uniform_bits(22, orc.I8, k * n)
    da, db = to_device(a), to_device(b)
    d = torch.empty(m * n, device="cuda", dtype=torch.int32)
    workspace = torch.empty(rw.gemm_streamk_workspace_size(), dtype=torch.uint8, device="cuda")
    if static:
        call = lambda: rw.gemm_streamk_static(orc.I8, orc.I32, RM, CM, RM, m, n, k, da, db, None, d, 1.0, 0.0)
    else:
        call = lambda: rw.gemm_streamk(orc.I8, orc.I32, RM, CM, RM, m, n, k, da, db, None, d, 1.0, 0.0, workspace)
    _replays_match(call, [d])
    assert np.array_equal(d.cpu().numpy(), orc.gemm(orc.I8, orc.I32, RM, CM, RM, RM, m, n, k, a, b, None, 1.0, 0.0))


@pytest.mark.parametrize("m,k,ncols", [(512, 1024, 1), (512, 2048, 2), (512, 2048, 4), (256, 4096, 8)])
def test_gemv_replays(m, k, ncols):
    import torch

    a, x = uniform_bits(31, orc.F16, m * k), uniform_bits(32, orc.F16, k * ncols)
    da, dx = to_device(a), to_device(x)
    y = torch.empty(m * ncols, device="cuda", dtype=torch.float32)
    _replays_match(lambda: rw.gemv(m, k, ncols, da, dx, y, 1.5, 0.0), [y])
    # Y (m x ncols, column-major) = the row-major result of X^T (ncols x k) * A^T
    want = orc.gemm(orc.F16, orc.F32, RM, CM, RM, RM, ncols, m, k, x, a, None, 1.5, 0.0)
    err, inf, nan = orc.compare_equal(orc.F32, y.cpu().numpy(), orc.F32, want)
    assert not inf and not nan and err <= 1e-3, (err, inf, nan)


@pytest.mark.parametrize("batch,m,k", [(6, 27, 128), (64, 27, 128), (2048, 27, 128), (3, 300, 200)])
def test_dlrm_replays(batch, m, k):
    """One wave per sample, and (300 rows) the tiled kernels for samples that do not fit a wave."""
    import torch

    width = k + m * (m - 1) // 2
    feats, up = uniform_bits(41, orc.F16, batch * m * k), uniform_bits(42, orc.F16, batch * width)
    dfe, dup = to_device(feats), to_device(up)
    out = torch.empty(batch * width, device="cuda", dtype=torch.int16)
    grad = torch.empty(batch * m * k, device="cuda", dtype=torch.int16)
    mlp = torch.empty(batch * k, device="cuda", dtype=torch.int16)

    def call():
        rw.dlrm_fwd(dfe, out, m, k, batch)
        rw.dlrm_bwd(dfe, dup, grad, mlp, m, k, batch)

    _replays_match(call, [out, grad, mlp])


@pytest.mark.parametrize("batch,m,k", [(64, 27, 128), (5, 128, 128), (3, 300, 200)])
def test_dlrm_float32_replays(batch, m, k):
    """One wave per sample, and (300 rows) the tiled kernels for samples that do not fit a wave."""
    import torch

    width = k + m * (m - 1) // 2
    rng = np.random.default_rng(43)
    dfe = to_device(rng.uniform(-1, 1, batch * m * k).astype(np.float32))
    dup = to_device(rng.uniform(-1, 1, batch * width).astype(np.float32))
    out = torch.empty(batch * width, device="cuda")
    grad = torch.empty(batch * m * k, device="cuda")
    mlp = torch.empty(batch * k, device="cuda")

    def call():
        rw.dlrm_fwd(dfe, out, m, k, batch, rw.F32)
        rw.dlrm_bwd(dfe, dup, grad, mlp, m, k, batch, rw.F32)

    _replays_match(call, [out, grad, mlp])


def test_block_scaled_gemm_replays():
    """Two launches per call (scale re-ordering into the workspace, then the GEMM): both are in the graph."""
    import torch

    m, n, k = 256, 512, 1024
    a, b = normal_fp8_bits(51, orc.E4M3, m * k, 1.0), normal_fp8_bits(52, orc.E4M3, k * n, 1.0)
    rng = np.random.default_rng(53)
    sa = rng.integers(124, 131, m * (k // 32)).astype(np.uint8)
    sb = rng.integers(124, 131, n * (k // 32)).astype(np.uint8)
    da, db, dsa, dsb = to_device(a), to_device(b), to_device(sa), to_device(sb)
    d = torch.empty(m * n, device="cuda", dtype=torch.float32)
    workspace = torch.empty(rw.gemm_mx_workspace_size(m, n, k), dtype=torch.uint8, device="cuda")
    _replays_match(lambda: rw.gemm_mx(orc.E4M3, RM, CM, RM, m, n, k, da, dsa, db, dsb, None, d, 1.0, 0.0, workspace=workspace), [d])
