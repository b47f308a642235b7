"""Host-only checks of the C-ABI library: it loads, exports every symbol the header declares,
and rejects bad arguments with status codes before touching a device.  No GPU needed."""
import ctypes
import os
import re

import pytest

import rocwmma_amd as rw

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(rw.library_path()):
        import __graft_entry__ as g

        g.build()
    return rw.library()


def _declared(header_name):
    header = open(os.path.join(ROOT, "include", header_name)).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)  # declarations only, not prose
    return set(re.findall(r"\b(rocwmma_amd_[a-z0-9_]+)\s*\(", header))


def test_exports_every_declared_symbol(lib):
    declared = _declared("rocwmma_amd.h")
    assert declared, "no declarations found"
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in include/rocwmma_amd.h but not exported"
    assert declared == set(rw.api.EXPORTS)


def test_aux_library_exports_every_declared_symbol_and_product_library_none_of_them(lib):
    """Test and benchmark support lives in a library of its own, not in the product ABI."""
    aux = rw.aux_library()
    declared = _declared("rocwmma_amd_aux.h")
    assert declared == set(rw.api.AUX_EXPORTS)
    for name in sorted(declared):
        assert hasattr(aux, name), f"{name} declared in include/rocwmma_amd_aux.h but not exported"
        with pytest.raises(AttributeError):
            getattr(lib, name)


def test_version_and_status_strings(lib):
    assert rw.version() == 10700
    assert rw.status_string(0) == "success"
    assert "16-byte" in rw.status_string(4)
    assert rw.status_string(99) == "unknown status"


def _gemm(lib, *, dtype_in=rw.F16, dtype_out=rw.F32, la=0, lb=1, lc=0, m=32, n=32, k=32, a=4096, lda=None,
          b=8192, ldb=None, c=12288, ldc=None, d=16384, ldd=None, alpha=1.0, beta=1.0):
    lda = lda if lda is not None else (k if la == 0 else m)
    ldb = ldb if ldb is not None else (n if lb == 0 else k)
    ldc = ldc if ldc is not None else (n if lc == 0 else m)
    ldd = ldd if ldd is not None else (n if lc == 0 else m)
    return lib.rocwmma_amd_gemm(dtype_in, dtype_out, la, lb, lc, m, n, k, a, lda, b, ldb, c, ldc, d, ldd,
                                alpha, beta, None)


def test_gemm_argument_validation(lib):
    # (fake, never dereferenced pointers: every case is rejected before any launch)
    assert _gemm(lib, a=None) == 1
    assert _gemm(lib, m=0) == 1
    assert _gemm(lib, la=7) == 1
    assert _gemm(lib, c=None, beta=1.0) == 1
    assert _gemm(lib, dtype_in=rw.I32) == 2
    assert _gemm(lib, dtype_in=rw.BF16, dtype_out=rw.F16) == 2
    assert _gemm(lib, dtype_in=rw.I8, dtype_out=rw.F32) == 2
    assert _gemm(lib, dtype_in=rw.I8, dtype_out=rw.I32, alpha=0.5) == 1
    assert _gemm(lib, m=24) == 3
    assert _gemm(lib, k=8) == 3
    assert _gemm(lib, lda=16) == 5
    assert _gemm(lib, a=4098) == 4
    assert _gemm(lib, lda=36) == 4                  # 36 halves = 72 B: not 16-byte aligned
    # valid arguments: NO_DEVICE where no GPU is visible.  Where one is, such a call would launch a kernel on
    # the fake pointers and fault the card, so it is only made without one.
    import torch

    if not torch.cuda.is_available():
        assert _gemm(lib) == 6
        assert _gemm(lib, ldd=36, ldc=36) == 6      # 36 floats = 144 B: aligned, passes on to the device check


def test_fused_and_block_scaled_gemm_argument_validation(lib):
    f = lib.rocwmma_amd_gemm_bias_act
    ok = dict(m=32, n=32, k=32, a=4096, lda=32, b=8192, ldb=32, c=12288, ldc=32, d=16384, ldd=32)

    def fused(dtype_in=rw.F16, dtype_out=rw.F32, bias=20480, act=rw.ACT_GELU, **kw):
        v = dict(ok, **kw)
        return f(dtype_in, dtype_out, 0, 1, 0, v["m"], v["n"], v["k"], v["a"], v["lda"], v["b"], v["ldb"], v["c"], v["ldc"],
                 v["d"], v["ldd"], 1.0, 1.0, bias, act, None)

    assert fused(dtype_in=rw.I8, dtype_out=rw.I32) == 2      # float types only
    assert fused(dtype_in=rw.F32) == 2
    assert fused(act=7) == 1
    assert fused(bias=20484) == 4                              # bias must be 16-byte aligned
    assert fused(a=None) == 1
    assert fused(m=24) == 3

    g = lib.rocwmma_amd_gemm_mx

    def mx(dtype_in=rw.E4M3, m=32, n=32, k=128, sa=20480, lsa=4, sb=24576, lsb=4, ws=None, wsb=0):
        return g(dtype_in, 0, 1, 0, m, n, k, 4096, k, sa, lsa, 8192, k, sb, lsb, 12288, n, 16384, n, 1.0, 1.0, ws, wsb, None)

    assert mx(dtype_in=rw.F16) == 2                            # fp8 / bf8 only
    assert mx(dtype_in=rw.I8) == 2
    assert mx(sa=None) == 1
    assert mx(k=96) == 3                                       # K in whole instructions (64 at least)
    assert mx(lsa=3) == 5                                      # scale leading dimension below k / 32
    assert lib.rocwmma_amd_gemm_mx_workspace_size(256, 512, 512) == (4 + 8) * 2 * 64 * 8
    import torch

    if not torch.cuda.is_available():
        assert fused() == 6 and mx() == 6


def test_gemv_and_dlrm_argument_validation(lib):
    f = lib.rocwmma_amd_gemv
    assert f(64, 64, 3, 4096, 64, 8192, 64, 12288, 64, 1.0, 0.0, None) == 3
    assert f(64, 60, 1, 4096, 64, 8192, 64, 12288, 64, 1.0, 0.0, None) == 3
    assert f(64, 64, 1, 4096, 32, 8192, 64, 12288, 64, 1.0, 0.0, None) == 5
    assert f(64, 64, 1, 4098, 64, 8192, 64, 12288, 64, 1.0, 0.0, None) == 4
    assert f(64, 64, 1, None, 64, 8192, 64, 12288, 64, 1.0, 0.0, None) == 1
    g = lib.rocwmma_amd_dlrm_fwd
    assert g(None, 4096, 27, 128, 8, None) == 1
    assert g(4096, 8192, 40000, 128, 8, None) == 3
    assert g(4096, 8192, 32768, 65536, 8, None) == 3  # (a sample of 4 GiB: beyond the kernels' 32-bit offsets)
    assert g(4096, 8192, 27, 100, 8, None) == 3  # (rows of f16 must be whole 16-byte pieces)
    assert g(4096, 8192, 27, 128, 0, None) == 1 and g(4096, 8192, 27, 0, 8, None) == 1
    h = lib.rocwmma_amd_dlrm_bwd
    assert h(4096, 8192, 12288, None, 27, 128, 8, None) == 1
    assert h(4096, 8192, 12290, 16384, 27, 128, 8, None) == 4
    # the entry points with an element type: float32 and f16 only, same checks
    gx, hx = lib.rocwmma_amd_dlrm_fwd_ex, lib.rocwmma_amd_dlrm_bwd_ex
    F16, BF16, F32, I8 = 0, 1, 5, 4
    assert gx(BF16, 4096, 8192, 27, 128, 8, None) == 2 and hx(I8, 4096, 8192, 12288, 16384, 27, 128, 8, None) == 2
    for t in (F16, F32):
        assert gx(t, None, 4096, 27, 128, 8, None) == 1
        assert gx(t, 4096, 8192, 40000, 128, 8, None) == 3
        assert gx(t, 4096, 8192, 27, 102, 8, None) == 3 and hx(t, 4096, 8192, 12288, 16384, 200, 1026, 8, None) == 3
        assert hx(t, 4096, 8192, 12288, None, 27, 128, 8, None) == 1
        assert hx(t, 4096, 8192, 12290, 16384, 27, 128, 8, None) == 4


def test_product_code_never_touches_the_oracle():
    """The shipped package and the C sources must not import, link or mention the oracle."""
    for base in ("rocwmma_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, base)):
            for fn in files:
                if fn.endswith((".py", ".hip", ".hpp", ".h", ".cpp")):
                    text = open(os.path.join(dirpath, fn), errors="ignore").read()
                    assert "liboracle" not in text and "import oracle" not in text, os.path.join(dirpath, fn)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more exits with a message instead of running."""
    import subprocess
    import sys

    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True, timeout=120)
    assert res.returncode != 0
    assert "one GPU" in res.stdout
