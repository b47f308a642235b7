"""ctypes binding of the C oracle.  Arrays are numpy; element types are raw bit patterns
(uint16 for f16/bf16, uint8 for fp8, int8, float32, int32)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F16, BF16, E4M3, E5M2, I8, F32, I32 = range(7)
ROW_MAJOR, COL_MAJOR = 0, 1

_NP_STORAGE = {F16: np.uint16, BF16: np.uint16, E4M3: np.uint8, E5M2: np.uint8,
               I8: np.int8, F32: np.float32, I32: np.int32}


def build(force=False):
    """Compile liboracle.so with the committed Makefile."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, u32, dbl, i = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_double, ctypes.c_int
        L.oracle_gemm_naive.argtypes = [i, i, i, i, i, i, u32, u32, u32, vp, vp, vp, vp, dbl, dbl]
        L.oracle_gemm_naive.restype = i
        L.oracle_gemm.argtypes = L.oracle_gemm_naive.argtypes
        L.oracle_gemm.restype = i
        L.oracle_gemm_rows.argtypes = L.oracle_gemm_naive.argtypes + [vp, u32]
        L.oracle_gemm_rows.restype = i
        L.oracle_dlrm_fwd_f16.argtypes = [vp, vp, u32, u32, u32]
        L.oracle_dlrm_fwd_f16.restype = None
        L.oracle_dlrm_bwd_f16.argtypes = [vp, vp, vp, vp, u32, u32, u32]
        L.oracle_dlrm_bwd_f16.restype = None
        L.oracle_dlrm_fwd_f32.argtypes = [vp, vp, u32, u32, u32]
        L.oracle_dlrm_fwd_f32.restype = None
        L.oracle_dlrm_bwd_f32.argtypes = [vp, vp, vp, vp, u32, u32, u32]
        L.oracle_dlrm_bwd_f32.restype = None
        L.oracle_compare_equal.argtypes = [i, vp, i, vp, ctypes.c_size_t, ctypes.POINTER(i)]
        L.oracle_compare_equal.restype = dbl
        L.oracle_encode.argtypes = [i, vp, vp, ctypes.c_size_t]
        L.oracle_encode.restype = None
        L.oracle_decode.argtypes = [i, vp, vp, ctypes.c_size_t]
        L.oracle_decode.restype = None
        L.oracle_num_threads.restype = i
        _lib = L
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def storage_dtype(dtype):
    return _NP_STORAGE[dtype]


def encode(dtype, values):
    """float32 array -> storage bits, round-to-nearest-even (fp8 saturating)."""
    src = np.ascontiguousarray(values, dtype=np.float32)
    if dtype == F32:
        return src.copy()
    if dtype == I8:
        return src.astype(np.int8)
    out = np.empty(src.shape, dtype=_NP_STORAGE[dtype])
    lib().oracle_encode(dtype, _ptr(src), _ptr(out), src.size)
    return out


def decode(dtype, bits):
    """storage bits -> float32 (exact)."""
    src = np.ascontiguousarray(bits, dtype=_NP_STORAGE[dtype])
    out = np.empty(src.shape, dtype=np.float32)
    lib().oracle_decode(dtype, _ptr(src), _ptr(out), src.size)
    return out


def _ld_shape(layout, rows, cols):
    return (rows, cols) if layout == ROW_MAJOR else (cols, rows)


def gemm(dtype_in, dtype_out, layA, layB, layC, layD, m, n, k, a, b, c, alpha, beta,
         rows=None, naive=False):
    """D = alpha*A*B + beta*C following gemm_CPU (test/reference_impl.hpp:36-81).

    a, b, c are flat or 2-D numpy arrays of storage bits in the stated layouts with natural
    leading dimensions.  Returns D as a flat array of m*n storage elements.  With ``rows``
    only those output rows are computed (other entries of the result are zero)."""
    a = np.ascontiguousarray(a, dtype=_NP_STORAGE[dtype_in]).reshape(-1)
    b = np.ascontiguousarray(b, dtype=_NP_STORAGE[dtype_in]).reshape(-1)
    assert a.size == m * k and b.size == k * n
    if c is not None:
        c = np.ascontiguousarray(c, dtype=_NP_STORAGE[dtype_out]).reshape(-1)
        assert c.size == m * n
    d = np.zeros(m * n, dtype=_NP_STORAGE[dtype_out])
    L = lib()
    if naive:
        assert rows is None
        rc = L.oracle_gemm_naive(dtype_in, dtype_out, layA, layB, layC, layD, m, n, k,
                                 _ptr(a), _ptr(b), _ptr(c), _ptr(d), alpha, beta)
    elif rows is None:
        rc = L.oracle_gemm(dtype_in, dtype_out, layA, layB, layC, layD, m, n, k,
                           _ptr(a), _ptr(b), _ptr(c), _ptr(d), alpha, beta)
    else:
        rows = np.ascontiguousarray(rows, dtype=np.uint32)
        rc = L.oracle_gemm_rows(dtype_in, dtype_out, layA, layB, layC, layD, m, n, k,
                                _ptr(a), _ptr(b), _ptr(c), _ptr(d), alpha, beta,
                                _ptr(rows), rows.size)
    if rc != 0:
        raise ValueError(f"oracle_gemm: unsupported combination (rc={rc})")
    return d


MX_BLOCK = 32  # elements along K that share one scale (OCP Microscaling Formats v1.0, section 5)


def mx_scale_values(scales):
    """E8M0 scale bytes -> float32 factors 2^(e - 127) (e = 255 encodes NaN)."""
    e = np.ascontiguousarray(scales, dtype=np.uint8).astype(np.int32)
    out = np.ldexp(np.float32(1.0), e - 127).astype(np.float32)
    out[e == 255] = np.nan
    return out


def mx_dequantise(dtype, bits, scales, layout, rows, k):
    """Values of a block-scaled operand: `bits` holds a rows x k matrix (`layout` says whether rows
    or K are contiguous: ROW_MAJOR = K contiguous), `scales` a rows x k/32 byte matrix (K blocks
    contiguous).  Returns float32 in the same layout as `bits`.  The product element * 2^(e-127) is
    exact in float32 for every finite fp8 value and every scale whose result stays normal."""
    vals = decode(dtype, bits).reshape((rows, k) if layout == ROW_MAJOR else (k, rows))
    fac = np.repeat(mx_scale_values(scales).reshape(rows, k // MX_BLOCK), MX_BLOCK, axis=1)
    return (vals * (fac if layout == ROW_MAJOR else fac.T)).astype(np.float32)


def gemm_mx(dtype_in, layA, layB, layC, layD, m, n, k, a, scale_a, b, scale_b, c, alpha, beta, rows=None):
    """Block-scaled GEMM.  The reference has no such path; the definition is that of the OCP
    Microscaling Formats specification v1.0 (section 6.2: the dot product of two MX vectors is the
    sum over blocks of scaleA * scaleB * sum of element products), restated as: dequantise both
    operands (exact, see mx_dequantise), then gemm_CPU's loop nest in float32
    (test/reference_impl.hpp:36-81) on the dequantised values."""
    af = mx_dequantise(dtype_in, a, scale_a, layA, m, k)
    # B is k x n: its "rows" in the sense of mx_dequantise are its columns
    bf = mx_dequantise(dtype_in, b, scale_b, ROW_MAJOR if layB == COL_MAJOR else COL_MAJOR, n, k)
    return gemm(F32, F32, layA, layB, layC, layD, m, n, k, af, bf, c, alpha, beta, rows=rows)


ACT_NONE, ACT_RELU, ACT_GELU = range(3)


def gemm_bias_act(dtype_in, dtype_out, layA, layB, layC, m, n, k, a, b, c, alpha, beta, bias, activation, rows=None):
    """D = act(alpha*A*B + beta*C + bias[column]).  The reference has no fused epilogue: this is
    gemm_CPU (test/reference_impl.hpp:36-81) with a float32 result, followed by the bias and the
    activation in float64 (ReLU: max(x, 0); GELU: x (1 + erf(x / sqrt 2)) / 2), rounded once to
    `dtype_out`.  C and D share layC."""
    from scipy.special import erf

    cf = None if c is None else decode(dtype_out, c)
    acc = gemm(dtype_in, F32, layA, layB, layC, layC, m, n, k, a, b, cf, alpha, beta, rows=rows).astype(np.float64)
    acc = acc.reshape((m, n) if layC == ROW_MAJOR else (n, m))
    if bias is not None:
        bv = np.asarray(bias, dtype=np.float32).astype(np.float64)
        acc = acc + (bv[None, :] if layC == ROW_MAJOR else bv[:, None])
    if activation == ACT_RELU:
        acc = np.maximum(acc, 0.0)
    elif activation == ACT_GELU:
        acc = 0.5 * acc * (1.0 + erf(acc / np.sqrt(2.0)))
    out = encode(dtype_out, acc.astype(np.float32).reshape(-1))
    if rows is not None:  # rows that were not computed stay zero, as in gemm()
        keep = np.zeros(m, dtype=bool)
        keep[np.asarray(rows)] = True
        mask = np.broadcast_to(keep[:, None] if layC == ROW_MAJOR else keep[None, :], acc.shape).reshape(-1)
        out = np.where(mask, out, np.zeros_like(out))
    return out


def dlrm_fwd(inp, m, k, batch, dtype=F16):
    """dlrm_fwd_CPU (test/reference_impl.hpp:83-119) on f16 bit patterns (dtype F16) or float32 values (F32)."""
    width = m * (m - 1) // 2 + k
    if dtype == F32:
        inp = np.ascontiguousarray(inp, dtype=np.float32).reshape(-1)
        assert inp.size == batch * m * k
        out = np.zeros(batch * width, dtype=np.float32)
        lib().oracle_dlrm_fwd_f32(_ptr(inp), _ptr(out), m, k, batch)
        return out.reshape(batch, width)
    assert dtype == F16
    inp = np.ascontiguousarray(inp, dtype=np.uint16).reshape(-1)
    assert inp.size == batch * m * k
    out = np.zeros(batch * width, dtype=np.uint16)
    lib().oracle_dlrm_fwd_f16(_ptr(inp), _ptr(out), m, k, batch)
    return out.reshape(batch, width)


def dlrm_bwd(inp, upstream, m, k, batch, dtype=F16):
    """dlrm_bwd_CPU (test/reference_impl.hpp:121-179) on f16 bit patterns (dtype F16) or float32 values (F32).
    Returns (grad[batch,m,k], bottom_mlp_grad[batch,k])."""
    width = m * (m - 1) // 2 + k
    np_t = np.float32 if dtype == F32 else np.uint16
    assert dtype in (F16, F32)
    inp = np.ascontiguousarray(inp, dtype=np_t).reshape(-1)
    upstream = np.ascontiguousarray(upstream, dtype=np_t).reshape(-1)
    assert inp.size == batch * m * k and upstream.size == batch * width
    grad = np.zeros(batch * m * k, dtype=np_t)
    mlp = np.zeros(batch * k, dtype=np_t)
    fn = lib().oracle_dlrm_bwd_f32 if dtype == F32 else lib().oracle_dlrm_bwd_f16
    fn(_ptr(inp), _ptr(upstream), _ptr(mlp), _ptr(grad), m, k, batch)
    return grad.reshape(batch, m, k), mlp.reshape(batch, k)


def compare_equal(dtype_a, a, dtype_b, b):
    """compareEqual metric (test/common.hpp:436-523): returns (max_rel_err, saw_inf, saw_nan)."""
    a = np.ascontiguousarray(a, dtype=_NP_STORAGE[dtype_a]).reshape(-1)
    b = np.ascontiguousarray(b, dtype=_NP_STORAGE[dtype_b]).reshape(-1)
    assert a.size == b.size
    flags = ctypes.c_int(0)
    err = lib().oracle_compare_equal(dtype_a, _ptr(a), dtype_b, _ptr(b), a.size, ctypes.byref(flags))
    return err, bool(flags.value & 1), bool(flags.value & 2)


def num_threads():
    return lib().oracle_num_threads()
