"""Shared helpers of the test-suite: seeded inputs as storage bit patterns (the same bits go to
the GPU and to the CPU oracle) and numpy <-> device plumbing (torch is used for memory only)."""
import numpy as np

import oracle as orc

RM, CM = orc.ROW_MAJOR, orc.COL_MAJOR


def uniform_bits(seed, dtype, count, lo=-1.0, hi=1.0):
    """count values, i.i.d. uniform[lo, hi] from the seed, rounded once to `dtype` storage."""
    rng = np.random.default_rng(seed)
    if dtype == orc.I8:
        return rng.integers(-128, 128, size=count, dtype=np.int8)
    if dtype == orc.I32:
        return rng.integers(-1000, 1000, size=count, dtype=np.int32)
    vals = rng.uniform(lo, hi, size=count).astype(np.float32)
    return orc.encode(dtype, vals)


def normal_fp8_bits(seed, dtype, count, scale=0.1):
    """N(0,1) * scale rounded to fp8 (round-to-nearest-even, saturating)."""
    rng = np.random.default_rng(seed)
    return orc.encode(dtype, (rng.standard_normal(count) * scale).astype(np.float32))


def exact_int_bits(dtype, rows, cols, layout):
    """The reference's device fill pattern, value = -((i*cols + j) % 3)
    (test/device/common.hpp:204-219): every GEMM partial sum is an exact small integer."""
    i = np.arange(rows)[:, None]
    j = np.arange(cols)[None, :]
    mat = -((i * cols + j) % 3).astype(np.float32)
    flat = np.ascontiguousarray(mat if layout == RM else mat.T).reshape(-1)
    if dtype == orc.I8:
        return flat.astype(np.int8)
    if dtype == orc.F32:
        return flat
    if dtype == orc.I32:
        return flat.astype(np.int32)
    return orc.encode(dtype, flat)


def to_device(bits):
    """numpy storage array -> device tensor with the same bytes."""
    import torch

    arr = np.ascontiguousarray(bits)
    if arr.dtype == np.uint16:
        arr = arr.view(np.int16)
    return torch.from_numpy(arr).cuda()


def to_host(tensor, np_dtype):
    arr = tensor.cpu().numpy()
    return arr.view(np_dtype) if arr.dtype != np_dtype else arr


def tol_for(dtype_in):
    """Max relative error (compareEqual metric) allowed against the CPU oracle."""
    if dtype_in in (orc.E4M3, orc.E5M2):
        return 1e-2
    if dtype_in == orc.I8:
        return 0.0
    return 1e-3


def dropin_missing(what):
    """The drop-in executables are built where the reference checkout is (tests/dropin/build_samples.py) and
    travel with the tree, so on a GPU box their absence is an error, not a reason to skip: a tree
    without them would otherwise pass with the drop-in proof silently left out.
    ROCWMMA_AMD_REQUIRE_DROPIN=0 turns the failure into a skip (a checkout without the reference)."""
    import os

    import pytest

    msg = f"{what} not built (tests/dropin/build_samples.py, needs the reference checkout)"
    if os.environ.get("ROCWMMA_AMD_REQUIRE_DROPIN", "1") == "0":
        pytest.skip(msg)
    pytest.fail(msg + "; set ROCWMMA_AMD_REQUIRE_DROPIN=0 to skip instead")
