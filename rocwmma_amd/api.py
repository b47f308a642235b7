"""ctypes binding of librocwmma_amd.so plus thin torch-tensor wrappers.

The wrappers mirror the argument lists of the reference's workload hosts
(samples/simple_hgemm.cpp:141 gemm_test, samples/perf_hgemm.cpp:716 gemm_test,
samples/simple_sgemv.cpp sgemv_test, samples/simple_dlrm.cpp:443 dlrm_test) but take device
tensors, run on torch's current stream and raise RocwmmaError instead of exiting.
torch is used for device memory and streams only."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_NAME = "librocwmma_amd.so"

F16, BF16, E4M3, E5M2, I8, F32, I32 = range(7)
ROW_MAJOR, COL_MAJOR = 0, 1
GEMM_AUTO, GEMM_WAVE_TILE, GEMM_BLOCKED, GEMM_BLOCKED_256 = 0, 1, 2, 3

EXPORTS = [
    "rocwmma_amd_version", "rocwmma_amd_status_string", "rocwmma_amd_device_info", "rocwmma_amd_gemm",
    "rocwmma_amd_gemm_ex", "rocwmma_amd_gemv", "rocwmma_amd_dlrm_fwd", "rocwmma_amd_dlrm_bwd",
    "rocwmma_amd_gemm_streamk", "rocwmma_amd_gemm_streamk_workspace_size", "rocwmma_amd_gemm_streamk_static",
    "rocwmma_amd_gemm_mx", "rocwmma_amd_gemm_mx_workspace_size", "rocwmma_amd_gemm_bias_act",
    "rocwmma_amd_gemm_streamk_timed_out", "rocwmma_amd_gemm_mx_pack_scales", "rocwmma_amd_gemm_mx_packed",
    "rocwmma_amd_dlrm_fwd_ex", "rocwmma_amd_dlrm_bwd_ex",
]
ACT_NONE, ACT_RELU, ACT_GELU = range(3)
# librocwmma_amd_aux.so: test and benchmark support (include/rocwmma_amd_aux.h)
_AUX_LIB_NAME = "librocwmma_amd_aux.so"
AUX_EXPORTS = ["rocwmma_amd_selftest_roundtrip", "rocwmma_amd_selftest_coop_gemm", "rocwmma_amd_selftest_tiled_gemm", "rocwmma_amd_bench_mfma_ceiling",
               "rocwmma_amd_bench_stream", "rocwmma_amd_bench_mfma_streams"]
(MFMA_F16_16X16X32, MFMA_F16_32X32X16, MFMA_BF16_16X16X32, MFMA_BF16_32X32X16, MFMA_I8_16X16X64, MFMA_I8_32X32X32,
 MFMA_F8_16X16X128, MFMA_F8_32X32X64, MFMA_F8_16X16X128_SCALED) = range(9)


class RocwmmaError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        super().__init__(f"{where}: status {status} ({status_string(status)})")


def library_path():
    return os.path.join(HERE, _LIB_NAME)


_lib = None


def library():
    """Loads the built library.  It is never built implicitly on import: run
    ``python -c "import __graft_entry__ as g; g.build()"`` (or rocwmma_amd/build.py) first."""
    global _lib
    if _lib is None:
        path = library_path()
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `python rocwmma_amd/build.py`")
        # PyTorch brings a HIP runtime of its own.  Loaded first, this library would bind to the system's,
        # and a device made current through one runtime is not current in the other (device_info then
        # reports that no gfx950 device is current): where PyTorch is installed it is imported first.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = ctypes.CDLL(path)
        i, u, vp, f = ctypes.c_int, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_float
        L.rocwmma_amd_version.restype = i
        L.rocwmma_amd_status_string.argtypes = [i]
        L.rocwmma_amd_status_string.restype = ctypes.c_char_p
        L.rocwmma_amd_device_info.argtypes = [ctypes.POINTER(i)] * 3
        L.rocwmma_amd_device_info.restype = i
        gemm_args = [i, i, i, i, i, u, u, u, vp, u, vp, u, vp, u, vp, u, f, f, vp]
        L.rocwmma_amd_gemm.argtypes = gemm_args
        L.rocwmma_amd_gemm.restype = i
        L.rocwmma_amd_gemm_ex.argtypes = [i] + gemm_args
        L.rocwmma_amd_gemm_ex.restype = i
        L.rocwmma_amd_gemm_streamk.argtypes = gemm_args[:-1] + [vp, ctypes.c_size_t, vp]
        L.rocwmma_amd_gemm_streamk.restype = i
        L.rocwmma_amd_gemm_streamk_static.argtypes = gemm_args
        L.rocwmma_amd_gemm_streamk_static.restype = i
        L.rocwmma_amd_gemm_streamk_timed_out.argtypes = [vp, ctypes.c_size_t, vp, ctypes.POINTER(i)]
        L.rocwmma_amd_gemm_streamk_timed_out.restype = i
        L.rocwmma_amd_gemm_bias_act.argtypes = gemm_args[:-1] + [vp, i, vp]
        L.rocwmma_amd_gemm_bias_act.restype = i
        L.rocwmma_amd_gemm_mx.argtypes = [i, i, i, i, u, u, u, vp, u, vp, u, vp, u, vp, u, vp, u, vp, u, f, f, vp, ctypes.c_size_t, vp]
        L.rocwmma_amd_gemm_mx_workspace_size.argtypes = [u, u, u]
        L.rocwmma_amd_gemm_mx_workspace_size.restype = ctypes.c_size_t
        L.rocwmma_amd_gemm_mx.restype = i
        L.rocwmma_amd_gemm_mx_pack_scales.argtypes = [i, i, i, u, u, u, vp, u, vp, u, vp, ctypes.c_size_t, vp]
        L.rocwmma_amd_gemm_mx_pack_scales.restype = i
        L.rocwmma_amd_gemm_mx_packed.argtypes = [i, i, i, i, u, u, u, vp, u, vp, u, vp, u, vp, u, f, f, vp, ctypes.c_size_t, vp]
        L.rocwmma_amd_gemm_mx_packed.restype = i
        L.rocwmma_amd_gemm_streamk_workspace_size.argtypes = []
        L.rocwmma_amd_gemm_streamk_workspace_size.restype = ctypes.c_size_t
        L.rocwmma_amd_gemv.argtypes = [u, u, u, vp, u, vp, u, vp, u, f, f, vp]
        L.rocwmma_amd_gemv.restype = i
        L.rocwmma_amd_dlrm_fwd.argtypes = [vp, vp, u, u, u, vp]
        L.rocwmma_amd_dlrm_fwd.restype = i
        L.rocwmma_amd_dlrm_bwd.argtypes = [vp, vp, vp, vp, u, u, u, vp]
        L.rocwmma_amd_dlrm_bwd.restype = i
        L.rocwmma_amd_dlrm_fwd_ex.argtypes = [i, vp, vp, u, u, u, vp]
        L.rocwmma_amd_dlrm_fwd_ex.restype = i
        L.rocwmma_amd_dlrm_bwd_ex.argtypes = [i, vp, vp, vp, vp, u, u, u, vp]
        L.rocwmma_amd_dlrm_bwd_ex.restype = i
        _lib = L
    return _lib


def aux_library_path():
    return os.path.join(HERE, _AUX_LIB_NAME)


_aux = None


def aux_library():
    """Loads the test / benchmark support library (self-test kernels, measurement probes)."""
    global _aux
    if _aux is None:
        path = aux_library_path()
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `python rocwmma_amd/build.py`")
        L = ctypes.CDLL(path)
        i, u, vp, f = ctypes.c_int, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_float
        L.rocwmma_amd_selftest_roundtrip.argtypes = [i, i, i, i, i, i, u, u, vp, vp, u, vp]
        L.rocwmma_amd_selftest_roundtrip.restype = i
        L.rocwmma_amd_selftest_coop_gemm.argtypes = [i, i, u, u, u, vp, vp, vp, vp, f, f, vp]
        L.rocwmma_amd_selftest_coop_gemm.restype = i
        L.rocwmma_amd_selftest_tiled_gemm.argtypes = [i, i, u, u, u, vp, vp, vp, vp, f, f, vp]
        L.rocwmma_amd_selftest_tiled_gemm.restype = i
        L.rocwmma_amd_bench_mfma_ceiling.argtypes = [i, u, u, vp, vp, ctypes.POINTER(ctypes.c_double), vp]
        L.rocwmma_amd_bench_mfma_ceiling.restype = i
        L.rocwmma_amd_bench_stream.argtypes = [i, vp, vp, ctypes.c_size_t, vp]
        L.rocwmma_amd_bench_mfma_streams.argtypes = [i, i, u, vp, vp, vp, vp, ctypes.POINTER(ctypes.c_double), vp]
        L.rocwmma_amd_bench_mfma_streams.restype = i
        L.rocwmma_amd_bench_stream.restype = i
        _aux = L
    return _aux


def version():
    return library().rocwmma_amd_version()


def status_string(status):
    return library().rocwmma_amd_status_string(int(status)).decode()


def device_info():
    cu, mhz, ok = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    rc = library().rocwmma_amd_device_info(ctypes.byref(cu), ctypes.byref(mhz), ctypes.byref(ok))
    if rc != 0:
        raise RocwmmaError(rc, "device_info")
    return {"compute_units": cu.value, "clock_mhz": mhz.value, "is_gfx950": bool(ok.value)}


def _check(rc, where):
    if rc != 0:
        raise RocwmmaError(rc, where)


_raw_stream = None


def _stream():
    """The current PyTorch stream of the current device as a raw handle."""
    global _raw_stream
    if _raw_stream is None:
        import torch

        fast = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        if fast is not None:
            # (no Stream object per call: a launch from Python costs a few microseconds, and this is one of them)
            _raw_stream = lambda: fast(torch.cuda.current_device())
        else:
            _raw_stream = lambda: torch.cuda.current_stream().cuda_stream
    return ctypes.c_void_p(_raw_stream())


def _ptr(t):
    """Device tensor (its data pointer), raw address (int / c_void_p) or None."""
    if t is None or isinstance(t, ctypes.c_void_p):
        return t
    if isinstance(t, int):
        return ctypes.c_void_p(t)
    return ctypes.c_void_p(t.data_ptr())


def gemm_raw(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, a, lda, b, ldb, c, ldc, d, ldd,
             alpha, beta, algo=GEMM_AUTO, stream=None):
    """Straight call of rocwmma_amd_gemm_ex with raw device pointers (ints / c_void_p)."""
    rc = library().rocwmma_amd_gemm_ex(algo, dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k,
                                       a, lda, b, ldb, c, ldc, d, ldd, alpha, beta,
                                       stream if stream is not None else _stream())
    _check(rc, "gemm")


def gemm(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, a, b, c, d, alpha, beta,
         lda=None, ldb=None, ldc=None, ldd=None, algo=GEMM_AUTO):
    """D = alpha*A*B + beta*C on device tensors (any shape; only data_ptr is used), natural
    leading dimensions unless given.  Kernel argument order of the reference
    (m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta)."""
    lda = lda if lda is not None else (k if layout_a == ROW_MAJOR else m)
    ldb = ldb if ldb is not None else (n if layout_b == ROW_MAJOR else k)
    nat = n if layout_c == ROW_MAJOR else m
    ldc = ldc if ldc is not None else nat
    ldd = ldd if ldd is not None else nat
    gemm_raw(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, _ptr(a), lda, _ptr(b), ldb,
             _ptr(c), ldc, _ptr(d), ldd, alpha, beta, algo)
    return d


def gemm_streamk_workspace_size():
    return library().rocwmma_amd_gemm_streamk_workspace_size()


def gemm_streamk(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, a, b, c, d, alpha, beta, workspace,
                 lda=None, ldb=None, ldc=None, ldd=None):
    """rocwmma_amd_gemm_streamk on device tensors; `workspace` is a device tensor of at least
    gemm_streamk_workspace_size() bytes."""
    lda = lda if lda is not None else (k if layout_a == ROW_MAJOR else m)
    ldb = ldb if ldb is not None else (n if layout_b == ROW_MAJOR else k)
    nat = n if layout_c == ROW_MAJOR else m
    ldc = ldc if ldc is not None else nat
    ldd = ldd if ldd is not None else nat
    rc = library().rocwmma_amd_gemm_streamk(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, _ptr(a), lda,
                                            _ptr(b), ldb, _ptr(c), ldc, _ptr(d), ldd, alpha, beta, _ptr(workspace),
                                            workspace.numel() * workspace.element_size(), _stream())
    _check(rc, "gemm_streamk")
    return d


def gemm_streamk_static(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, a, b, c, d, alpha, beta,
                        lda=None, ldb=None, ldc=None, ldd=None):
    """rocwmma_amd_gemm_streamk_static on device tensors (the library's own scratch, no allocation)."""
    lda = lda if lda is not None else (k if layout_a == ROW_MAJOR else m)
    ldb = ldb if ldb is not None else (n if layout_b == ROW_MAJOR else k)
    nat = n if layout_c == ROW_MAJOR else m
    ldc = ldc if ldc is not None else nat
    ldd = ldd if ldd is not None else nat
    rc = library().rocwmma_amd_gemm_streamk_static(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, _ptr(a),
                                                   lda, _ptr(b), ldb, _ptr(c), ldc, _ptr(d), ldd, alpha, beta, _stream())
    _check(rc, "gemm_streamk_static")
    return d


def gemm_streamk_timed_out(workspace=None):
    """rocwmma_amd_gemm_streamk_timed_out: True when an owner's bounded wait ran out in a stream-K launch on
    `workspace` (None: the library's static scratch) since the last query.  Waits for torch's current stream."""
    flag = ctypes.c_int(-1)
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _check(library().rocwmma_amd_gemm_streamk_timed_out(_ptr(workspace), nbytes, _stream(), ctypes.byref(flag)),
           "gemm_streamk_timed_out")
    return bool(flag.value)


def gemm_bias_act(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, a, b, c, d, alpha, beta, bias, activation,
                  lda=None, ldb=None, ldc=None, ldd=None):
    """rocwmma_amd_gemm_bias_act on device tensors: D = act(alpha*A*B + beta*C + bias[column]);
    `bias` is a float32 device tensor of n values or None."""
    lda = lda if lda is not None else (k if layout_a == ROW_MAJOR else m)
    ldb = ldb if ldb is not None else (n if layout_b == ROW_MAJOR else k)
    nat = n if layout_c == ROW_MAJOR else m
    ldc = ldc if ldc is not None else nat
    ldd = ldd if ldd is not None else nat
    rc = library().rocwmma_amd_gemm_bias_act(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, _ptr(a), lda,
                                             _ptr(b), ldb, _ptr(c), ldc, _ptr(d), ldd, alpha, beta, _ptr(bias), activation,
                                             _stream())
    _check(rc, "gemm_bias_act")
    return d


def gemm_mx_workspace_size(m, n, k):
    return int(library().rocwmma_amd_gemm_mx_workspace_size(m, n, k))


def gemm_mx(dtype_in, layout_a, layout_b, layout_c, m, n, k, a, scale_a, b, scale_b, c, d, alpha, beta,
            workspace=None, lda=None, ldb=None, ldc=None, ldd=None, ld_scale_a=None, ld_scale_b=None):
    """rocwmma_amd_gemm_mx on device tensors: fp8 / bf8 operands with one E8M0 scale byte per 32
    elements along K (scale_a: m x k/32, scale_b: n x k/32, K blocks contiguous), f32 C / D.
    `workspace`: None (one-block-per-wave kernel) or a device tensor of at least
    gemm_mx_workspace_size(m, n, k) bytes (blocked kernel where the shape allows)."""
    lda = lda if lda is not None else (k if layout_a == ROW_MAJOR else m)
    ldb = ldb if ldb is not None else (n if layout_b == ROW_MAJOR else k)
    nat = n if layout_c == ROW_MAJOR else m
    ldc = ldc if ldc is not None else nat
    ldd = ldd if ldd is not None else nat
    ld_scale_a = ld_scale_a if ld_scale_a is not None else k // 32
    ld_scale_b = ld_scale_b if ld_scale_b is not None else k // 32
    rc = library().rocwmma_amd_gemm_mx(dtype_in, layout_a, layout_b, layout_c, m, n, k, _ptr(a), lda, _ptr(scale_a),
                                       ld_scale_a, _ptr(b), ldb, _ptr(scale_b), ld_scale_b, _ptr(c), ldc, _ptr(d), ldd,
                                       alpha, beta, _ptr(workspace),
                                       0 if workspace is None else workspace.numel() * workspace.element_size(), _stream())
    _check(rc, "gemm_mx")
    return d


def gemm_mx_pack_scales(layout_a, layout_b, layout_c, m, n, k, scale_a, scale_b, workspace, ld_scale_a=None, ld_scale_b=None):
    """rocwmma_amd_gemm_mx_pack_scales: re-orders the scales of a problem into `workspace` for gemm_mx_packed;
    scale_a or scale_b may be None (that operand's part of the workspace is left as it is)."""
    rc = library().rocwmma_amd_gemm_mx_pack_scales(layout_a, layout_b, layout_c, m, n, k, _ptr(scale_a),
                                                   ld_scale_a if ld_scale_a is not None else k // 32, _ptr(scale_b),
                                                   ld_scale_b if ld_scale_b is not None else k // 32, _ptr(workspace),
                                                   workspace.numel() * workspace.element_size(), _stream())
    _check(rc, "gemm_mx_pack_scales")
    return workspace


def gemm_mx_packed(dtype_in, layout_a, layout_b, layout_c, m, n, k, a, b, c, d, alpha, beta, workspace,
                   lda=None, ldb=None, ldc=None, ldd=None):
    """rocwmma_amd_gemm_mx_packed: the block-scaled GEMM on a workspace filled by gemm_mx_pack_scales."""
    lda = lda if lda is not None else (k if layout_a == ROW_MAJOR else m)
    ldb = ldb if ldb is not None else (n if layout_b == ROW_MAJOR else k)
    nat = n if layout_c == ROW_MAJOR else m
    ldc = ldc if ldc is not None else nat
    ldd = ldd if ldd is not None else nat
    rc = library().rocwmma_amd_gemm_mx_packed(dtype_in, layout_a, layout_b, layout_c, m, n, k, _ptr(a), lda, _ptr(b), ldb,
                                              _ptr(c), ldc, _ptr(d), ldd, alpha, beta, _ptr(workspace),
                                              workspace.numel() * workspace.element_size(), _stream())
    _check(rc, "gemm_mx_packed")
    return d


def gemv(m, k, ncols, a, x, y, alpha=1.0, beta=0.0, lda=None, ldx=None, ldy=None):
    """Y = alpha*A*X + beta*Y in place; A f16 row-major m x k, X f16 k x ncols column-major,
    Y f32 m x ncols column-major."""
    rc = library().rocwmma_amd_gemv(m, k, ncols, _ptr(a), lda or k, _ptr(x), ldx or k, _ptr(y), ldy or m,
                                    alpha, beta, _stream())
    _check(rc, "gemv")
    return y


def dlrm_fwd(inp, out, m, k, batch, dtype=None):
    """DLRM dot interaction, forward; dtype None: the f16 entry point, else rocwmma_amd_dlrm_fwd_ex (F16 or F32)."""
    if dtype is None:
        _check(library().rocwmma_amd_dlrm_fwd(_ptr(inp), _ptr(out), m, k, batch, _stream()), "dlrm_fwd")
    else:
        _check(library().rocwmma_amd_dlrm_fwd_ex(dtype, _ptr(inp), _ptr(out), m, k, batch, _stream()), "dlrm_fwd_ex")
    return out


def dlrm_bwd(inp, upstream, grad, mlp_grad, m, k, batch, dtype=None):
    """DLRM dot interaction, backward; dtype None: the f16 entry point, else rocwmma_amd_dlrm_bwd_ex (F16 or F32)."""
    if dtype is None:
        _check(library().rocwmma_amd_dlrm_bwd(_ptr(inp), _ptr(upstream), _ptr(grad), _ptr(mlp_grad), m, k, batch,
                                              _stream()), "dlrm_bwd")
    else:
        _check(library().rocwmma_amd_dlrm_bwd_ex(dtype, _ptr(inp), _ptr(upstream), _ptr(grad), _ptr(mlp_grad), m, k, batch,
                                                 _stream()), "dlrm_bwd_ex")
    return grad, mlp_grad


def selftest_roundtrip(context, dtype, layout, block, blockk, coop, rows, cols, inp, out, ld):
    _check(aux_library().rocwmma_amd_selftest_roundtrip(context, dtype, layout, block, blockk, int(coop), rows, cols,
                                                    _ptr(inp), _ptr(out), ld, _stream()), "selftest_roundtrip")
    return out


def selftest_coop_gemm(layout_a, layout_b, m, n, k, a, b, c, d, alpha, beta):
    _check(aux_library().rocwmma_amd_selftest_coop_gemm(layout_a, layout_b, m, n, k, _ptr(a), _ptr(b), _ptr(c), _ptr(d),
                                                    alpha, beta, _stream()), "selftest_coop_gemm")
    return d


def selftest_tiled_gemm(layout_a, layout_b, m, n, k, a, b, c, d, alpha, beta):
    _check(aux_library().rocwmma_amd_selftest_tiled_gemm(layout_a, layout_b, m, n, k, _ptr(a), _ptr(b), _ptr(c), _ptr(d),
                                                     alpha, beta, _stream()), "selftest_tiled_gemm")
    return d


STREAM_READ, STREAM_WRITE, STREAM_COPY, STREAM_COPY_READ_MORE, STREAM_READ_RESIDENT = 0, 1, 2, 3, 4
STREAM_RESIDENT_PASSES = 256  # ROCWMMA_AMD_STREAM_RESIDENT_PASSES: mode 4 reads its bytes this many times


def bench_stream(mode, src, dst, nbytes, stream=None):
    """Launches the memory-stream ceiling probe (plain read / write / copy of nbytes bytes); src / dst are
    device tensors or raw addresses."""
    _check(aux_library().rocwmma_amd_bench_stream(mode, _ptr(src), _ptr(dst), nbytes,
                                                  stream if stream is not None else _stream()), "bench_stream")


STREAMS_F16, STREAMS_I8, STREAMS_FP8 = 0, 1, 2


def bench_mfma_streams(streams, tiles_per_workgroup, a, b, operands, out, kind=STREAMS_F16):
    """Launches the matrix-pipes-next-to-their-operand-streams probe (include/rocwmma_amd_aux.h); returns the
    operation count of the launch."""
    ops = ctypes.c_double(0.0)
    _check(aux_library().rocwmma_amd_bench_mfma_streams(kind, streams, tiles_per_workgroup, _ptr(a), _ptr(b), _ptr(operands),
                                                        _ptr(out), ctypes.byref(ops), _stream()), "bench_mfma_streams")
    return ops.value


def bench_mfma_ceiling(shape, trips, waves_per_simd, operands, out):
    """Launches the matrix-pipe ceiling probe; returns the operation count of the launch."""
    ops = ctypes.c_double(0.0)
    _check(aux_library().rocwmma_amd_bench_mfma_ceiling(shape, trips, waves_per_simd, _ptr(operands), _ptr(out),
                                                        ctypes.byref(ops), _stream()), "bench_mfma_ceiling")
    return ops.value
