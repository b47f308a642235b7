"""DLRM dot-interaction parity: the HIP kernels against the reference's golden files and the
CPU oracle (dlrm_fwd_CPU / dlrm_bwd_CPU, test/reference_impl.hpp:83-179).
Tolerance: 10 * eps(f16) in the compareEqual metric (test/dlrm/dlrm_kernel_base_impl.hpp:472-478)."""
import os

import numpy as np
import pytest

import oracle as orc
import rocwmma_amd as rw
from util import to_device, uniform_bits

pytestmark = pytest.mark.gpu
TOL = 10 * 2.0 ** -10


def gpu_fwd(inp, m, k, b):
    import torch

    width = k + m * (m - 1) // 2
    out = to_device(np.full(b * width, 0x7E00, dtype=np.uint16))
    rw.dlrm_fwd(to_device(inp), out, m, k, b)
    torch.cuda.synchronize()
    return out.cpu().numpy().view(np.uint16).reshape(b, width)


def gpu_bwd(inp, up, m, k, b):
    import torch

    grad = to_device(np.full(b * m * k, 0x7E00, dtype=np.uint16))
    mlp = to_device(np.full(b * k, 0x7E00, dtype=np.uint16))
    rw.dlrm_bwd(to_device(inp), to_device(up), grad, mlp, m, k, b)
    torch.cuda.synchronize()
    return (grad.cpu().numpy().view(np.uint16).reshape(b, m, k), mlp.cpu().numpy().view(np.uint16).reshape(b, k))


def close(got, want, tol=TOL):
    err, inf, nan = orc.compare_equal(orc.F16, got, orc.F16, want)
    assert not inf and not nan and err <= tol, (err, inf, nan)
    return err


def _golden(golden_dir, name, shape):
    return np.fromfile(os.path.join(golden_dir, f"dlrm_{name}.bin"), dtype=np.uint16).reshape(shape)


def test_forward_against_reference_golden_files(golden_dir):
    b, m, k = 64, 27, 128
    inp = _golden(golden_dir, "input_fp16", (b, m, k))
    want = _golden(golden_dir, "output_fp16", (b, k + m * (m - 1) // 2))
    got = gpu_fwd(inp, m, k, b)
    close(got, want)
    assert np.array_equal(got[:, :k], inp[:, 0, :])
    close(got, orc.dlrm_fwd(inp, m, k, b))


def test_backward_against_reference_golden_files(golden_dir):
    b, m, k = 64, 27, 128
    inp = _golden(golden_dir, "input_fp16", (b, m, k))
    up = _golden(golden_dir, "input_grad_fp16", (b, k + m * (m - 1) // 2))
    grad, mlp = gpu_bwd(inp, up, m, k, b)
    assert np.array_equal(mlp, _golden(golden_dir, "output_mlp_input_grad_fp16", (b, k)))
    close(grad, _golden(golden_dir, "output_input_grad_fp16", (b, m, k)))
    wgrad, wmlp = orc.dlrm_bwd(inp, up, m, k, b)
    close(grad, wgrad)
    assert np.array_equal(mlp, wmlp)


@pytest.mark.parametrize("b,m,k", [(2048, 27, 128), (13, 27, 128), (1, 27, 128), (40, 32, 128), (24, 5, 64),
                                   (9, 16, 32), (17, 2, 256), (8, 1, 128)])
def test_forward_and_backward_against_oracle(b, m, k):
    width = k + m * (m - 1) // 2
    inp = uniform_bits(0x5EED0005 + b, orc.F16, b * m * k)
    up = uniform_bits(0x5EED0105 + b, orc.F16, b * width)
    got = gpu_fwd(inp, m, k, b)
    close(got, orc.dlrm_fwd(inp, m, k, b))
    grad, mlp = gpu_bwd(inp, up, m, k, b)
    wgrad, wmlp = orc.dlrm_bwd(inp, up, m, k, b)
    close(grad, wgrad)
    assert np.array_equal(mlp, wmlp)


def test_backward_is_linear_and_forward_is_symmetric_at_large_batch():
    """Size-independent properties at a batch the oracle would take long on.  Doubling the
    upstream gradient doubles grad exactly (power-of-two scaling commutes with every rounding
    in the normal range); swapping two feature rows swaps the matching Gram entries."""
    b, m, k = 16384, 27, 128
    width = k + m * (m - 1) // 2
    inp = uniform_bits(1, orc.F16, b * m * k)
    up = uniform_bits(2, orc.F16, b * width)
    g1, _ = gpu_bwd(inp, up, m, k, b)
    dbl = (up.view(np.float16) * np.float16(2.0)).view(np.uint16)
    g2, _ = gpu_bwd(inp, dbl, m, k, b)
    v1, v2 = g1.view(np.float16).astype(np.float32), g2.view(np.float16).astype(np.float32)
    normal = np.abs(v1) >= 2.0 ** -13
    mismatches = int((v2[normal] != 2.0 * v1[normal]).sum())
    assert mismatches == 0
    assert float(np.abs(v2[~normal] - 2.0 * v1[~normal]).max(initial=0.0)) <= 2.0 ** -23
    f1 = gpu_fwd(inp, m, k, b)
    perm = inp.reshape(b, m, k).copy()
    perm[:, [1, 2]] = perm[:, [2, 1]]
    f2 = gpu_fwd(perm, m, k, b)
    checks = [np.array_equal(f2[:, k + 0], f1[:, k + 1]),   # new Z[1,0] = F2.F0 = old Z[2,0]
              np.array_equal(f2[:, k + 1], f1[:, k + 0]),   # new Z[2,0] = F1.F0 = old Z[1,0]
              np.array_equal(f2[:, k + 2], f1[:, k + 2])]   # Z[2,1] is symmetric under the swap
    assert checks == [True, True, True]


@pytest.mark.parametrize("b", [4, 9])
def test_backward_samples_are_independent_of_non_finite_neighbours(b):
    """The backward kernel contracts over 32 feature rows of a sample's LDS tile; with m < 32 the rows
    behind the m-th belong to the next sample.  G is zero there, but 0 * NaN is NaN: a NaN or Inf in
    sample s + 1 must leave the gradient of sample s untouched, as in the reference's CPU loops,
    which never read another sample (test/reference_impl.hpp:121-179)."""
    m, k = 27, 128
    width = k + m * (m - 1) // 2
    inp = uniform_bits(71, orc.F16, b * m * k).reshape(b, m, k).copy()
    up = uniform_bits(72, orc.F16, b * width)
    clean, _ = gpu_bwd(inp, up, m, k, b)
    poisoned = inp.copy()
    poisoned[1::2, :, :] = 0x7E00  # every odd sample: all NaN
    poisoned[1::2, 0, 1] = 0x7C00  # and an Inf
    grad, _ = gpu_bwd(poisoned, up, m, k, b)
    assert np.array_equal(grad[0::2], clean[0::2])
    wgrad, _ = orc.dlrm_bwd(poisoned, up, m, k, b)
    assert np.array_equal(np.isnan(orc.decode(orc.F16, grad.reshape(-1))), np.isnan(orc.decode(orc.F16, wgrad.reshape(-1))))


@pytest.mark.parametrize("b,m,k", [(5, 128, 128), (3, 128, 256), (4, 33, 64), (7, 64, 32), (6, 100, 128), (2, 96, 256), (9, 40, 128)])
def test_more_than_32_feature_rows_run_as_tiles_of_32(b, m, k):
    """32 < m <= 128 (the reference's DLRM tests run m = 128, test/dlrm/test/dlrm_test_params.hpp:51-58): forward
    and backward against the oracle; one and two samples per workgroup, odd batch sizes and odd row widths
    (m = 33: width 592, m = 100 with k = 128: 5078), m that is not a multiple of 32."""
    inp = uniform_bits(700 + m, orc.F16, b * m * k).reshape(b, m, k)
    width = k + m * (m - 1) // 2
    up = uniform_bits(701 + m, orc.F16, b * width).reshape(b, width)
    got = gpu_fwd(inp, m, k, b)
    want = orc.dlrm_fwd(inp, m, k, b)
    close(got, want)
    assert np.array_equal(got[:, :k], inp[:, 0, :])
    grad, mlp = gpu_bwd(inp, up, m, k, b)
    wgrad, wmlp = orc.dlrm_bwd(inp, up, m, k, b)
    close(grad, wgrad)
    assert np.array_equal(mlp, wmlp)


def test_tiled_backward_samples_are_independent_of_non_finite_neighbours():
    """As for m <= 32: rows of the next sample that a tile's operand reads beyond m must not leak (0 * Inf)."""
    b, m, k = 4, 40, 128
    inp = uniform_bits(801, orc.F16, b * m * k).reshape(b, m, k).copy()
    width = k + m * (m - 1) // 2
    up = uniform_bits(802, orc.F16, b * width).reshape(b, width)
    want, _ = orc.dlrm_bwd(inp, up, m, k, b)
    poisoned = inp.copy()
    poisoned[2] = 0x7C00  # +Inf everywhere in sample 2
    grad, _ = gpu_bwd(poisoned, up, m, k, b)
    for s in (0, 1, 3):
        close(grad[s], want[s])


# ---------------------------------------------------------------- float32 (rocwmma_amd_dlrm_fwd_ex / _bwd_ex)
# The reference's tolerance for float32_t is 10 * eps in the compareEqual metric (test/dlrm/dlrm_kernel_base_impl.hpp:472-478).
# On random data in [-1, 1] no float32 summation of 128 and more such terms meets that against another order: the
# reference's own CPU loop is 13-31 eps from the exact (float64) result at these sizes, and its fp32 fixtures are 9.8 eps
# from its CPU loop.  So the kernels are held to the accuracy of that loop (error against the exact result at most 1.5 x
# the loop's, plus 2 eps) and to 64 eps against loop and fixtures (an indexing mistake is off by O(0.1)); integer-valued
# data, where every sum is exact, must match the loop bit for bit.
EPS32 = 2.0 ** -23
TOL32_PAIR = 64 * EPS32


def exact_fwd(inp, m, k):
    F = inp.astype(np.float64)
    Z = np.einsum("bik,bjk->bij", F, F)
    il, jl = np.tril_indices(m, -1)
    return np.concatenate([F[:, 0, :], Z[:, il, jl]], axis=1)


def exact_bwd(inp, up, m, k):
    b = inp.shape[0]
    il, jl = np.tril_indices(m, -1)
    G = np.zeros((b, m, m))
    G[:, il, jl] = up[:, k:].astype(np.float64)
    return (G + G.transpose(0, 2, 1)) @ inp.astype(np.float64)


def rel_to_exact(got, exact):
    got = got.astype(np.float64)
    return float(np.max(np.abs(got - exact) / (np.abs(got) + np.abs(exact) + 1.0)))


def as_accurate_as_the_cpu_loop(got, cpu, exact):
    assert np.isfinite(got).all()
    assert rel_to_exact(got, exact) <= 1.5 * rel_to_exact(cpu, exact) + 2 * EPS32, (rel_to_exact(got, exact), rel_to_exact(cpu, exact))


def gpu_fwd32(inp, m, k, b):
    import torch

    width = k + m * (m - 1) // 2
    out = to_device(np.full(b * width, np.nan, dtype=np.float32))
    rw.dlrm_fwd(to_device(np.ascontiguousarray(inp, dtype=np.float32)), out, m, k, b, rw.F32)
    torch.cuda.synchronize()
    return out.cpu().numpy().reshape(b, width)


def gpu_bwd32(inp, up, m, k, b):
    import torch

    grad = to_device(np.full(b * m * k, np.nan, dtype=np.float32))
    mlp = to_device(np.full(b * k, np.nan, dtype=np.float32))
    rw.dlrm_bwd(to_device(np.ascontiguousarray(inp, dtype=np.float32)), to_device(np.ascontiguousarray(up, dtype=np.float32)),
                grad, mlp, m, k, b, rw.F32)
    torch.cuda.synchronize()
    return grad.cpu().numpy().reshape(b, m, k), mlp.cpu().numpy().reshape(b, k)


def close32(got, want, tol=TOL32_PAIR):
    err, inf, nan = orc.compare_equal(orc.F32, np.ascontiguousarray(got), orc.F32, np.ascontiguousarray(want))
    assert not inf and not nan and err <= tol, (err, inf, nan)
    return err


def _golden32(golden_dir, name, shape):
    return np.fromfile(os.path.join(golden_dir, f"dlrm_{name}.bin"), dtype=np.float32).reshape(shape)


def test_float32_against_reference_golden_files(golden_dir):
    """The first 16 samples of the reference's fp32 data files (test/dlrm/data/*_fp32), forward and backward."""
    b, m, k = 16, 27, 128
    width = k + m * (m - 1) // 2
    inp = _golden32(golden_dir, "input_fp32", (b, m, k))
    got = gpu_fwd32(inp, m, k, b)
    want = orc.dlrm_fwd(inp, m, k, b, orc.F32)
    as_accurate_as_the_cpu_loop(got, want, exact_fwd(inp, m, k))
    close32(got, _golden32(golden_dir, "output_fp32", (b, width)))
    close32(got, want)
    assert np.array_equal(got[:, :k], inp[:, 0, :])
    up = _golden32(golden_dir, "input_grad_fp32", (b, width))
    grad, mlp = gpu_bwd32(inp, up, m, k, b)
    assert np.array_equal(mlp, _golden32(golden_dir, "output_mlp_input_grad_fp32", (b, k)))
    wgrad, wmlp = orc.dlrm_bwd(inp, up, m, k, b, orc.F32)
    as_accurate_as_the_cpu_loop(grad, wgrad, exact_bwd(inp, up, m, k))
    close32(grad, _golden32(golden_dir, "output_input_grad_fp32", (b, m, k)))
    close32(grad, wgrad)
    assert np.array_equal(mlp, wmlp)


@pytest.mark.parametrize("b,m,k", [(64, 32, 32), (64, 32, 128), (64, 128, 128), (2048, 27, 128), (13, 27, 128), (1, 27, 128),
                                   (24, 5, 64), (17, 2, 256), (8, 1, 128), (3, 128, 256), (4, 33, 64), (6, 100, 128)])
def test_float32_forward_and_backward_against_oracle(b, m, k):
    """The reference's float32 test sizes that fit a sample into LDS ((32, 32), (32, 128), (128, 128), batch 64:
    test/dlrm/test/dlrm_test_params.hpp:55-58), the benchmark's shape, odd batches, m that is not a multiple of 32,
    one / two / four samples per workgroup."""
    rng = np.random.default_rng(900 + m + k)
    width = k + m * (m - 1) // 2
    inp = rng.uniform(-1, 1, (b, m, k)).astype(np.float32)
    up = rng.uniform(-1, 1, (b, width)).astype(np.float32)
    got = gpu_fwd32(inp, m, k, b)
    want = orc.dlrm_fwd(inp, m, k, b, orc.F32)
    as_accurate_as_the_cpu_loop(got, want, exact_fwd(inp, m, k))
    close32(got, want)
    assert np.array_equal(got[:, :k], inp[:, 0, :])
    grad, mlp = gpu_bwd32(inp, up, m, k, b)
    wgrad, wmlp = orc.dlrm_bwd(inp, up, m, k, b, orc.F32)
    as_accurate_as_the_cpu_loop(grad, wgrad, exact_bwd(inp, up, m, k))
    close32(grad, wgrad)
    assert np.array_equal(mlp, wmlp)


def test_float32_exact_on_small_integers_and_independent_samples():
    """Integer-valued features and gradients make every sum exact in float32: bit-for-bit against the oracle.  A NaN /
    Inf sample next to a finite one must not leak into it (the kernels never read another sample's rows)."""
    b, m, k = 6, 27, 128
    rng = np.random.default_rng(31)
    width = k + m * (m - 1) // 2
    inp = rng.integers(-3, 4, (b, m, k)).astype(np.float32)
    up = rng.integers(-3, 4, (b, width)).astype(np.float32)
    assert np.array_equal(gpu_fwd32(inp, m, k, b), orc.dlrm_fwd(inp, m, k, b, orc.F32))
    grad, _ = gpu_bwd32(inp, up, m, k, b)
    assert np.array_equal(grad, orc.dlrm_bwd(inp, up, m, k, b, orc.F32)[0])
    poisoned = inp.copy()
    poisoned[1::2] = np.nan
    poisoned[1::2, 0, 1] = np.inf
    pgrad, _ = gpu_bwd32(poisoned, up, m, k, b)
    assert np.array_equal(pgrad[0::2], grad[0::2])
    pfwd = gpu_fwd32(poisoned, m, k, b)
    assert np.array_equal(pfwd[0::2], orc.dlrm_fwd(inp, m, k, b, orc.F32)[0::2])


def test_typed_entry_points_take_f16_and_reject_other_types():
    b, m, k = 8, 27, 128
    inp = uniform_bits(5, orc.F16, b * m * k).reshape(b, m, k)
    width = k + m * (m - 1) // 2
    out = to_device(np.zeros(b * width, dtype=np.uint16))
    rw.dlrm_fwd(to_device(inp), out, m, k, b, rw.F16)
    import torch

    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16).reshape(b, width), gpu_fwd(inp, m, k, b))
    with pytest.raises(rw.RocwmmaError) as e:
        rw.dlrm_fwd(to_device(inp), out, m, k, b, rw.BF16)
    assert e.value.status == 2  # ROCWMMA_AMD_UNSUPPORTED_TYPE


# ---------------------------------------------------------------- samples that do not fit one wave (tiles of 128 x 128)
# More than 128 feature rows or a feature width other than 32 / 64 / 128 / 256, up to the reference's largest test
# size (m, k) = (1024, 1024) (test/dlrm/test/dlrm_test_params.hpp:51-68).
def exact_fwd_mm(inp, m, k):
    F = inp.astype(np.float64)
    Z = F @ F.transpose(0, 2, 1)
    il, jl = np.tril_indices(m, -1)
    return np.concatenate([F[:, 0, :], Z[:, il, jl]], axis=1)


GENERAL_SHAPES = [(3, 160, 128), (11, 129, 64), (5, 27, 96), (2, 200, 40), (3, 1, 24), (4, 2, 8), (2, 300, 512),
                  (2, 130, 1032), (3, 257, 264), (1, 1024, 1024)]


@pytest.mark.parametrize("b,m,k", GENERAL_SHAPES)
def test_samples_larger_than_a_wave_run_as_tiles_of_128(b, m, k):
    """f16, forward and backward against the oracle: m just above 128 and not a multiple of anything, k that is no power
    of two (96, 40, 24, 8: whole 16-byte pieces is all that is asked), k that ends inside a step of the K loop
    (1032, 264), one and two feature rows, more than one tile in every direction, a batch that is no multiple of the
    eight XCDs the samples are dealt to, the reference's largest size."""
    width = k + m * (m - 1) // 2
    inp = uniform_bits(1100 + m, orc.F16, b * m * k).reshape(b, m, k)
    up = uniform_bits(1101 + m, orc.F16, b * width).reshape(b, width)
    got = gpu_fwd(inp, m, k, b)
    close(got, orc.dlrm_fwd(inp, m, k, b))
    assert np.array_equal(got[:, :k], inp[:, 0, :])
    grad, mlp = gpu_bwd(inp, up, m, k, b)
    wgrad, wmlp = orc.dlrm_bwd(inp, up, m, k, b)
    close(grad, wgrad)
    assert np.array_equal(mlp, wmlp)


@pytest.mark.parametrize("b,m,k", GENERAL_SHAPES + [(4, 27, 100), (2, 130, 36)])
def test_float32_samples_larger_than_a_wave(b, m, k):
    """float32, same shapes plus widths that are multiples of 4 only.  The rounding error of a float32 sum grows with
    its length: against the CPU loop the bound is 64 eps up to 256 terms and a quarter eps per term beyond."""
    rng = np.random.default_rng(1200 + m + k)
    width = k + m * (m - 1) // 2
    inp = rng.uniform(-1, 1, (b, m, k)).astype(np.float32)
    up = rng.uniform(-1, 1, (b, width)).astype(np.float32)
    tol = max(64, max(m, k) // 4) * EPS32
    got = gpu_fwd32(inp, m, k, b)
    want = orc.dlrm_fwd(inp, m, k, b, orc.F32)
    as_accurate_as_the_cpu_loop(got, want, exact_fwd_mm(inp, m, k))
    close32(got, want, tol)
    assert np.array_equal(got[:, :k], inp[:, 0, :])
    grad, mlp = gpu_bwd32(inp, up, m, k, b)
    wgrad, wmlp = orc.dlrm_bwd(inp, up, m, k, b, orc.F32)
    as_accurate_as_the_cpu_loop(grad, wgrad, exact_bwd(inp, up, m, k))
    close32(grad, wgrad, tol)
    assert np.array_equal(mlp, wmlp)


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_reference_largest_size_is_exact_on_small_integers(dtype):
    """The reference's largest DLRM test case at full size, (m, k, batch) = (1024, 1024, 64) with values -1 / 0 / 1 as its
    tests fill them (test/dlrm/test/dlrm_test_params.hpp:51-68): every sum is an integer of at most 1024, exact in f16
    and float32, so forward and backward must equal a float64 matrix product bit for bit (torch on the device is the
    calculator here; the CPU loops would take ten minutes)."""
    import torch

    b, m, k = 64, 1024, 1024
    width = k + m * (m - 1) // 2
    gen = torch.Generator(device="cuda").manual_seed(77)
    tdt = torch.float16 if dtype == "f16" else torch.float32
    code = rw.F16 if dtype == "f16" else rw.F32
    F = torch.randint(-1, 2, (b, m, k), generator=gen, device="cuda").to(tdt)
    up = torch.randint(-1, 2, (b, width), generator=gen, device="cuda").to(tdt)
    out = torch.full((b, width), float("nan"), dtype=tdt, device="cuda")
    rw.dlrm_fwd(F, out, m, k, b, code)
    il = torch.tril_indices(m, m, -1, device="cuda")
    for s0 in range(0, b, 8):  # (eight samples at a time: float64 copies are 8 MiB a sample)
        F64 = F[s0:s0 + 8].double()
        Z = torch.bmm(F64, F64.transpose(1, 2))
        assert torch.equal(out[s0:s0 + 8, k:].double(), Z[:, il[0], il[1]]), s0
    assert torch.equal(out[:, :k], F[:, 0, :])
    grad = torch.full((b, m, k), float("nan"), dtype=tdt, device="cuda")
    mlp = torch.full((b, k), float("nan"), dtype=tdt, device="cuda")
    rw.dlrm_bwd(F, up, grad, mlp, m, k, b, code)
    for s0 in range(0, b, 8):
        G = torch.zeros((8, m, m), dtype=torch.float64, device="cuda")
        G[:, il[0], il[1]] = up[s0:s0 + 8, k:].double()
        want = torch.bmm(G + G.transpose(1, 2), F[s0:s0 + 8].double())
        assert torch.equal(grad[s0:s0 + 8].double(), want), s0
    assert torch.equal(mlp, up[:, :k])


def test_large_samples_are_independent_of_non_finite_neighbours():
    """Rows beyond a sample's last belong to the next sample: the tiles must not read them (0 * Inf would leak)."""
    b, m, k = 3, 150, 72
    inp = uniform_bits(1301, orc.F16, b * m * k).reshape(b, m, k).copy()
    width = k + m * (m - 1) // 2
    up = uniform_bits(1302, orc.F16, b * width).reshape(b, width)
    want_f = orc.dlrm_fwd(inp, m, k, b)
    want_g, _ = orc.dlrm_bwd(inp, up, m, k, b)
    poisoned = inp.copy()
    poisoned[1] = 0x7C00  # +Inf everywhere in the middle sample
    got_f = gpu_fwd(poisoned, m, k, b)
    got_g, _ = gpu_bwd(poisoned, up, m, k, b)
    for s in (0, 2):
        close(got_f[s], want_f[s])
        close(got_g[s], want_g[s])
