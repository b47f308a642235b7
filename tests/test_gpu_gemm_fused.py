"""GEMM with the fused epilogue D = act(alpha*A*B + beta*C + bias[column]) on the GPU against the CPU
oracle (gemm_CPU's loop nest, then bias and activation in float64, rounded once to the output type).
Bar: f16 <= 1e-3, bf16 <= 4e-3 (one bf16 ulp of the output), fp8 <= 1e-2 in the compareEqual metric."""
import numpy as np
import pytest

import oracle as orc
import rocwmma_amd as rw
from util import CM, RM, to_device, to_host, uniform_bits

pytestmark = pytest.mark.gpu

TRIPLES = [(orc.F16, orc.F32, 1e-3), (orc.F16, orc.F16, 1e-3), (orc.BF16, orc.BF16, 4e-3), (orc.BF16, orc.F32, 1e-3),
           (orc.E4M3, orc.F32, 1e-2), (orc.E5M2, orc.F32, 1e-2)]


def run(dtype_in, dtype_out, la, lb, lc, m, n, k, a, b, c, alpha, beta, bias, act):
    import torch

    np_out = orc.storage_dtype(dtype_out)
    d0 = np.full(m * n, np.nan, dtype=np.float32) if dtype_out == orc.F32 else np.full(m * n, 0x7E00, dtype=np.uint16)
    d = to_device(d0)
    rw.gemm_bias_act(dtype_in, dtype_out, la, lb, lc, m, n, k, to_device(a), to_device(b),
                     None if c is None else to_device(c), d, alpha, beta, None if bias is None else to_device(bias), act)
    torch.cuda.synchronize()
    return to_host(d, np_out)


def check(dtype_out, got, want, tol):
    err, inf, nan = orc.compare_equal(dtype_out, got, dtype_out, want)
    assert not inf and not nan, (inf, nan)
    assert err <= tol, f"max relative error {err} > {tol}"


def case(seed, dtype_in, dtype_out, m, n, k):
    a = uniform_bits(seed, dtype_in, m * k)
    b = uniform_bits(seed + 1, dtype_in, k * n)
    c = uniform_bits(seed + 2, dtype_out, m * n)
    bias = np.random.default_rng(seed + 3).uniform(-2.0, 2.0, n).astype(np.float32)
    return a, b, c, bias


@pytest.mark.parametrize("act", [rw.ACT_NONE, rw.ACT_RELU, rw.ACT_GELU])
@pytest.mark.parametrize("la,lb", [(RM, CM), (CM, RM), (RM, RM), (CM, CM)])
@pytest.mark.parametrize("dtype_in,dtype_out,tol", TRIPLES)
def test_bias_and_activation_on_edge_tiles(dtype_in, dtype_out, tol, la, lb, act):
    """128 x 128 tiles with partly filled last row and column of tiles (m, n multiples of 16 only)."""
    m, n, k = 208, 304, 256
    a, b, c, bias = case(100, dtype_in, dtype_out, m, n, k)
    for beta, bv in ((0.0, bias), (-0.5, bias), (0.75, None)):
        got = run(dtype_in, dtype_out, la, lb, RM, m, n, k, a, b, c if beta else None, 0.25, beta, bv, act)
        want = orc.gemm_bias_act(dtype_in, dtype_out, la, lb, RM, m, n, k, a, b, c if beta else None, 0.25, beta, bv, act)
        check(dtype_out, got, want, tol)


@pytest.mark.parametrize("act", [rw.ACT_RELU, rw.ACT_GELU])
@pytest.mark.parametrize("la,lb", [(RM, CM), (CM, RM)])
@pytest.mark.parametrize("dtype_in,dtype_out,tol", TRIPLES)
def test_bias_and_activation_on_the_large_tile(dtype_in, dtype_out, tol, la, lb, act):
    """2048 x 4352 x 256: 136 tiles of 256 x 256 on 256 compute units, i.e. the large tile with the
    last (only) round cut into half tiles on a 256-unit device."""
    m, n, k = 2048, 4352, 256
    a, b, c, bias = case(200, dtype_in, dtype_out, m, n, k)
    rows = np.arange(0, m, 37, dtype=np.uint32)
    for beta in (0.0, 1.0):
        got = run(dtype_in, dtype_out, la, lb, RM, m, n, k, a, b, c if beta else None, 0.5, beta, bias, act)
        want = orc.gemm_bias_act(dtype_in, dtype_out, la, lb, RM, m, n, k, a, b, c if beta else None, 0.5, beta, bias, act,
                                 rows=rows)
        check(dtype_out, np.ascontiguousarray(got.reshape(m, n)[rows]), np.ascontiguousarray(want.reshape(m, n)[rows]), tol)


@pytest.mark.parametrize("lc", [RM, CM])
@pytest.mark.parametrize("dtype_in,dtype_out,tol", TRIPLES[:3])
def test_shapes_and_layouts_left_to_the_wave_tile_kernel(dtype_in, dtype_out, tol, lc):
    """K that is not in whole stages, and column-major C/D (bias still per column of D)."""
    m, n, k = 64, 96, 48 if lc == RM else 128
    a, b, c, bias = case(300, dtype_in, dtype_out, m, n, k)
    got = run(dtype_in, dtype_out, RM, CM, lc, m, n, k, a, b, c, 1.0, 1.0, bias, rw.ACT_GELU)
    want = orc.gemm_bias_act(dtype_in, dtype_out, RM, CM, lc, m, n, k, a, b, c, 1.0, 1.0, bias, rw.ACT_GELU)
    check(dtype_out, got, want, tol)


def test_no_bias_and_no_activation_is_the_plain_gemm_bit_for_bit():
    import torch

    m, n, k = 512, 768, 512
    a, b, c, _ = case(400, orc.F16, orc.F32, m, n, k)
    got = run(orc.F16, orc.F32, RM, CM, RM, m, n, k, a, b, c, 1.5, -0.5, None, rw.ACT_NONE)
    d = to_device(np.zeros(m * n, dtype=np.float32))
    rw.gemm(orc.F16, orc.F32, RM, CM, RM, m, n, k, to_device(a), to_device(b), to_device(c), d, 1.5, -0.5, algo=rw.GEMM_BLOCKED)
    torch.cuda.synchronize()
    want = orc.gemm(orc.F16, orc.F32, RM, CM, RM, RM, m, n, k, a, b, c, 1.5, -0.5)
    check(orc.F32, got, want, 1e-3)
    assert np.array_equal(got.view(np.uint32), to_host(d, np.float32).view(np.uint32))


@pytest.mark.parametrize("act", [rw.ACT_RELU, rw.ACT_GELU])
@pytest.mark.parametrize("m,n,k", [(208, 304, 256), (64, 96, 48)])
def test_activations_at_non_finite_and_large_arguments(act, m, n, k):
    """What the activations do at +-Inf, NaN and large |x| (fed in through C with beta = 1), on the blocked kernel
    and on the wave-tile kernel: ReLU(-Inf) = 0, ReLU(+Inf) = +Inf, ReLU(NaN) = NaN; GELU(+Inf) = +Inf,
    GELU(NaN) = NaN, GELU(-Inf) = NaN (x * Phi(x) = -Inf * 0, in the oracle's float64 formula as well),
    GELU(x) = x for large x and -0 for large negative x."""
    a, b, c, bias = case(500, orc.F16, orc.F32, m, n, k)
    c = c.copy()
    special = np.array([np.inf, -np.inf, np.nan, 1e30, -1e30, 40.0, -40.0, 6.0, -6.0], dtype=np.float32)
    c[: special.size * 7 : 7] = special
    got = run(orc.F16, orc.F32, RM, CM, RM, m, n, k, a, b, c, 1.0, 1.0, bias, act)
    want = orc.gemm_bias_act(orc.F16, orc.F32, RM, CM, RM, m, n, k, a, b, c, 1.0, 1.0, bias, act)
    assert np.array_equal(np.isnan(got), np.isnan(want)), (got[: special.size * 7 : 7], want[: special.size * 7 : 7])
    assert np.array_equal(np.isinf(got), np.isinf(want))
    ok = np.isfinite(want)
    assert np.array_equal(np.sign(got[np.isinf(want)]), np.sign(want[np.isinf(want)]))
    err, inf, nan = orc.compare_equal(orc.F32, got[ok], orc.F32, want[ok])
    assert not inf and not nan and err <= 1e-3, (err, inf, nan)
    sp = got[: special.size * 7 : 7]
    if act == rw.ACT_RELU:
        assert sp[0] == np.inf and sp[1] == 0.0 and np.isnan(sp[2]) and sp[4] == 0.0
    else:
        assert sp[0] == np.inf and np.isnan(sp[1]) and np.isnan(sp[2]) and sp[3] > 9e29 and abs(sp[4]) == 0.0 and abs(sp[6]) == 0.0
