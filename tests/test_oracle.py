"""Pins the CPU oracle: golden files, closed forms, brute force, codec tables.

Each check is chosen so that a plausible mistake in the restatement (dropped term, wrong
index, transposed operand, wrong rounding) fails it.  No GPU needed."""
import os

import numpy as np
import pytest

import oracle as orc

RM, CM = orc.ROW_MAJOR, orc.COL_MAJOR


def _rand_bits(rng, dtype, shape):
    if dtype == orc.I8:
        return rng.integers(-128, 128, size=shape, dtype=np.int8)
    vals = rng.uniform(-1.0, 1.0, size=shape).astype(np.float32)
    return orc.encode(dtype, vals)


def _as_matrix(bits_f32, layout, rows, cols):
    """float matrix (rows x cols) from a flat buffer in the given layout."""
    return bits_f32.reshape(rows, cols) if layout == RM else bits_f32.reshape(cols, rows).T


def _store(mat, layout):
    return np.ascontiguousarray(mat if layout == RM else mat.T).reshape(-1)


# ---------------------------------------------------------------- codecs
def test_f16_codec_all_codes_against_numpy():
    codes = np.arange(65536, dtype=np.uint16)
    ours = orc.decode(orc.F16, codes)
    theirs = codes.view(np.float16).astype(np.float32)
    both_nan = np.isnan(ours) & np.isnan(theirs)
    assert np.array_equal(ours[~both_nan], theirs[~both_nan])
    # encode: round trip every finite code, and RNE on random floats + exact midpoints
    finite = np.isfinite(theirs)
    assert np.array_equal(orc.encode(orc.F16, theirs[finite]), codes[finite])
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.uniform(-70000, 70000, 20000), rng.normal(0, 1e-5, 20000),
                        rng.normal(0, 1, 20000)]).astype(np.float32)
    with np.errstate(over="ignore"):
        assert np.array_equal(orc.encode(orc.F16, x), x.astype(np.float16).view(np.uint16))
    pos = theirs[(codes < 0x7BFF)]
    nxt = codes[(codes < 0x7BFF)] + 1
    mid = ((pos.astype(np.float64) + nxt.view(np.float16).astype(np.float64)) / 2).astype(np.float32)
    assert np.array_equal(orc.encode(orc.F16, mid), mid.astype(np.float16).view(np.uint16))


def test_bf16_codec():
    codes = np.arange(65536, dtype=np.uint16)
    ours = orc.decode(orc.BF16, codes)
    theirs = (codes.astype(np.uint32) << 16).view(np.float32)
    nan = np.isnan(theirs)
    assert np.array_equal(ours[~nan], theirs[~nan])
    rng = np.random.default_rng(2)
    x = rng.normal(0, 10, 50000).astype(np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    rne = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(orc.encode(orc.BF16, x), rne)
    # ties: exactly half-way values must go to the even neighbour
    ties = ((np.arange(0x3F80, 0x3FA0, dtype=np.uint32) << 16) | 0x8000).view(np.float32)
    enc = orc.encode(orc.BF16, ties)
    assert np.all(enc % 2 == 0)


def _ocp_e4m3_value(code):
    s = -1.0 if code & 0x80 else 1.0
    e, m = (code >> 3) & 0xF, code & 7
    if e == 0xF and m == 7:
        return float("nan")
    if e == 0:
        return s * m * 2.0 ** -9
    return s * (1 + m / 8.0) * 2.0 ** (e - 7)


def _ocp_e5m2_value(code):
    s = -1.0 if code & 0x80 else 1.0
    e, m = (code >> 2) & 0x1F, code & 3
    if e == 0x1F:
        return s * float("inf") if m == 0 else float("nan")
    if e == 0:
        return s * m * 2.0 ** -16
    return s * (1 + m / 4.0) * 2.0 ** (e - 15)


@pytest.mark.parametrize("dtype,fn,maxfinite", [(orc.E4M3, _ocp_e4m3_value, 448.0),
                                                (orc.E5M2, _ocp_e5m2_value, 57344.0)])
def test_fp8_codec_against_ocp_closed_form(dtype, fn, maxfinite):
    codes = np.arange(256, dtype=np.uint8)
    table = np.array([fn(int(c)) for c in codes], dtype=np.float64)
    ours = orc.decode(dtype, codes).astype(np.float64)
    ok = ~np.isnan(table)
    assert np.array_equal(ours[ok], table[ok]) and np.all(np.isnan(ours[~ok]))
    assert np.nanmax(np.where(np.isinf(table), np.nan, table)) == maxfinite
    fin = np.isfinite(table)
    # every finite code round-trips (-0 keeps its sign bit)
    assert np.array_equal(orc.encode(dtype, table[fin].astype(np.float32)), codes[fin])
    # brute-force nearest-even on a dense grid, incl. all midpoints, with saturation
    pos = np.sort(table[fin & (table >= 0) & (codes < 0x80)])
    mids = (pos[:-1] + pos[1:]) / 2
    grid = np.concatenate([mids, mids * (1 + 1e-6), mids * (1 - 1e-6), pos,
                           [maxfinite * 1.01, maxfinite * 2, 1e30, np.inf]]).astype(np.float32)
    enc = orc.encode(dtype, grid)
    poscodes = np.array([c for c in range(0x80) if np.isfinite(fn(c))])
    posvals = np.array([fn(int(c)) for c in poscodes])
    for x, e in zip(grid.astype(np.float64), enc):
        if x >= maxfinite:
            want = poscodes[np.argmax(posvals)]
        else:
            dist = np.abs(posvals - x)
            best = np.flatnonzero(dist == dist.min())
            want = poscodes[best[0]] if len(best) == 1 else [c for c in poscodes[best] if c % 2 == 0][0]
        assert e == want, (x, e, want)
    neg = orc.encode(dtype, -grid)
    assert np.array_equal(neg, enc | 0x80)


# ---------------------------------------------------------------- GEMM
@pytest.mark.parametrize("dtype_in,dtype_out", [(orc.F16, orc.F32), (orc.BF16, orc.F32),
                                                (orc.E4M3, orc.F32), (orc.E5M2, orc.F32),
                                                (orc.I8, orc.I32), (orc.F16, orc.F16)])
@pytest.mark.parametrize("layA", [RM, CM])
@pytest.mark.parametrize("layB", [RM, CM])
def test_gemm_fast_equals_reference_loop_nest(dtype_in, dtype_out, layA, layB):
    """The column-blocked form must reproduce the verbatim loop nest bit for bit."""
    rng = np.random.default_rng(10 + dtype_in)
    m, n, k = 37, 70, 53
    a = _rand_bits(rng, dtype_in, m * k)
    b = _rand_bits(rng, dtype_in, k * n)
    if dtype_out == orc.I32:
        c = rng.integers(-1000, 1000, m * n, dtype=np.int32)
        alpha, beta = 3, -2
    else:
        c = _rand_bits(rng, dtype_out, m * n)
        alpha, beta = 2.0, 0.5
    for layC, layD in [(RM, RM), (CM, RM), (RM, CM)]:
        d0 = orc.gemm(dtype_in, dtype_out, layA, layB, layC, layD, m, n, k, a, b, c, alpha, beta, naive=True)
        d1 = orc.gemm(dtype_in, dtype_out, layA, layB, layC, layD, m, n, k, a, b, c, alpha, beta)
        assert np.array_equal(d0, d1)
    rows = np.array([0, 5, 36], dtype=np.uint32)
    d2 = orc.gemm(dtype_in, dtype_out, layA, layB, RM, RM, m, n, k, a, b, c, alpha, beta, rows=rows)
    d0 = orc.gemm(dtype_in, dtype_out, layA, layB, RM, RM, m, n, k, a, b, c, alpha, beta, naive=True)
    assert np.array_equal(d2.reshape(m, n)[rows], d0.reshape(m, n)[rows])
    untouched = np.setdiff1d(np.arange(m), rows)
    assert not d2.reshape(m, n)[untouched].any()


@pytest.mark.parametrize("layA", [RM, CM])
@pytest.mark.parametrize("layB", [RM, CM])
@pytest.mark.parametrize("layC", [RM, CM])
def test_gemm_against_float64_and_layout_semantics(layA, layB, layC):
    """Independent check of indexing: build matrices in numpy, store them in each layout,
    compare with a float64 product (tolerance = f32 accumulation noise).  A transposed or
    mis-strided operand fails by O(1)."""
    rng = np.random.default_rng(3)
    m, n, k = 48, 33, 65
    A = rng.uniform(-1, 1, (m, k)).astype(np.float16)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float16)
    C = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    d = orc.gemm(orc.F16, orc.F32, layA, layB, layC, RM, m, n, k,
                 _store(A.view(np.uint16), layA), _store(B.view(np.uint16), layB), _store(C, layC), 2.0, -3.0)
    want = 2.0 * (A.astype(np.float64) @ B.astype(np.float64)) - 3.0 * C
    assert np.abs(d.reshape(m, n) - want).max() < 1e-4


def test_gemm_closed_forms():
    n = 64
    rng = np.random.default_rng(4)
    eye = orc.encode(orc.F16, np.eye(n, dtype=np.float32))
    Bv = rng.uniform(-1, 1, (n, n)).astype(np.float16)
    Cv = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    # A = I  =>  D = alpha*B + beta*C exactly (one product per sum is non-zero)
    d = orc.gemm(orc.F16, orc.F32, RM, CM, RM, RM, n, n, n, eye, _store(Bv.view(np.uint16), CM), Cv, 2.0, 2.0)
    want = np.float32(2.0) * Bv.astype(np.float32) + np.float32(2.0) * Cv
    assert np.array_equal(d.reshape(n, n), want)
    # all ones => alpha*K + beta
    ones = orc.encode(orc.BF16, np.ones(n * 200, dtype=np.float32))
    d = orc.gemm(orc.BF16, orc.F32, RM, RM, RM, RM, n, n, 200, ones, ones[: 200 * n],
                 np.ones(n * n, np.float32), 2.0, 3.0)
    assert np.all(d == 2.0 * 200 + 3.0)


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16, orc.E4M3, orc.E5M2])
def test_gemm_exact_integer_pattern(dtype):
    """The reference's own fill pattern ((i*n+j)%3 negated, test/device/common.hpp:204-219)
    keeps every partial sum an exactly representable integer, so the oracle must equal an
    int64 computation exactly, whatever the summation order."""
    m, n, k = 32, 48, 256
    ia = -((np.arange(m)[:, None] * k + np.arange(k)[None, :]) % 3)
    ib = -((np.arange(k)[:, None] * n + np.arange(n)[None, :]) % 3)
    ic = -((np.arange(m)[:, None] * n + np.arange(n)[None, :]) % 3)
    a = orc.encode(dtype, ia.astype(np.float32))
    b = orc.encode(dtype, ib.astype(np.float32))
    d = orc.gemm(dtype, orc.F32, RM, RM, RM, RM, m, n, k, a, b, ic.astype(np.float32), 2.0, 2.0)
    want = 2 * (ia.astype(np.int64) @ ib.astype(np.int64)) + 2 * ic
    assert np.array_equal(d.reshape(m, n).astype(np.int64), want)


def test_gemm_int8_exact_against_int64():
    rng = np.random.default_rng(5)
    m, n, k = 24, 40, 4096
    A = rng.integers(-128, 128, (m, k), dtype=np.int8)
    B = rng.integers(-128, 128, (k, n), dtype=np.int8)
    d = orc.gemm(orc.I8, orc.I32, RM, CM, RM, RM, m, n, k, A, _store(B, CM), None, 1, 0)
    want = A.astype(np.int64) @ B.astype(np.int64)
    assert np.array_equal(d.reshape(m, n).astype(np.int64), want)


def test_gemm_int8_output_keeps_low_byte_against_int64():
    """<int8, int8, int32>: D = int8(alpha * acc + beta * c) keeps the low eight bits of the exact
    integer result (two's complement), for the fast and the verbatim loop alike and in both C/D
    layouts; the saturating alternative differs on this data, so the check has teeth."""
    rng = np.random.default_rng(15)
    m, n, k = 24, 40, 96
    A = rng.integers(-128, 128, (m, k), dtype=np.int8)
    B = rng.integers(-128, 128, (k, n), dtype=np.int8)
    C = rng.integers(-128, 128, (m, n), dtype=np.int8)
    exact = 3 * (A.astype(np.int64) @ B.astype(np.int64)) - 2 * C.astype(np.int64)
    want = ((exact + 128) % 256 - 128).astype(np.int8)
    assert not np.array_equal(want, np.clip(exact, -128, 127).astype(np.int8))
    for lc in (RM, CM):
        for naive in (False, True):
            d = orc.gemm(orc.I8, orc.I8, RM, CM, lc, lc, m, n, k, A, _store(B, CM), _store(C, lc), 3, -2, naive=naive)
            got = d.reshape(m, n) if lc == RM else d.reshape(n, m).T
            assert np.array_equal(got, want)


def test_gemm_accumulation_order_is_sequential_f32():
    """Pins 'one f32 accumulator, increasing h, separate multiply and add' against a
    pure-Python loop on a case where the order matters (large cancellation)."""
    rng = np.random.default_rng(6)
    k = 300
    a = (rng.uniform(-1, 1, k) * 2.0 ** rng.integers(-8, 8, k)).astype(np.float16)
    b = (rng.uniform(-1, 1, k) * 2.0 ** rng.integers(-8, 8, k)).astype(np.float16)
    acc = np.float32(0)
    for h in range(k):
        acc = np.float32(acc + np.float32(np.float32(a[h]) * np.float32(b[h])))
    d = orc.gemm(orc.F16, orc.F32, RM, CM, RM, RM, 1, 1, k, a.view(np.uint16), b.view(np.uint16), None, 1.0, 0.0)
    assert d[0] == acc
    # reversed order differs on this data, so the check has teeth
    acc_r = np.float32(0)
    for h in reversed(range(k)):
        acc_r = np.float32(acc_r + np.float32(np.float32(a[h]) * np.float32(b[h])))
    assert acc_r != acc


# ---------------------------------------------------------------- compare metric
# ---- block-scaled GEMM (the reference has none: pinned on the OCP definition) ------------------
def _mx_case(seed, m, n, k, dtype, lo=120, hi=134):
    rng = np.random.default_rng(seed)
    a = orc.encode(dtype, rng.uniform(-1, 1, m * k).astype(np.float32))
    b = orc.encode(dtype, rng.uniform(-1, 1, k * n).astype(np.float32))
    sa = rng.integers(lo, hi + 1, size=(m, k // 32), dtype=np.uint8)
    sb = rng.integers(lo, hi + 1, size=(n, k // 32), dtype=np.uint8)
    return a, sa, b, sb


def test_mx_scale_decoding():
    """E8M0: 2^(e - 127); 127 is one, 0 the smallest (a float32 subnormal), 255 NaN."""
    v = orc.mx_scale_values(np.array([0, 1, 126, 127, 128, 254, 255], dtype=np.uint8))
    assert v[3] == 1.0 and v[2] == 0.5 and v[4] == 2.0
    assert v[0] == np.float32(2.0) ** -127 and v[1] == np.float32(2.0) ** -126
    assert v[5] == np.float32(2.0) ** 127 and np.isnan(v[6])


@pytest.mark.parametrize("dtype", [orc.E4M3, orc.E5M2])
def test_mx_gemm_with_unit_scales_is_the_unscaled_gemm(dtype):
    m, n, k = 48, 32, 128
    a, _, b, _ = _mx_case(1, m, n, k, dtype)
    one = np.full((max(m, n), k // 32), 127, dtype=np.uint8)
    for la, lb in [(orc.ROW_MAJOR, orc.COL_MAJOR), (orc.COL_MAJOR, orc.ROW_MAJOR)]:
        got = orc.gemm_mx(dtype, la, lb, 0, 0, m, n, k, a, one[:m], b, one[:n], None, 1.0, 0.0)
        want = orc.gemm(dtype, orc.F32, la, lb, 0, 0, m, n, k, a, b, None, 1.0, 0.0)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("la,lb", [(0, 1), (1, 0), (0, 0), (1, 1)])
def test_mx_gemm_against_float64_block_formula(la, lb):
    """Independent statement of the definition: per K block, scaleA * scaleB * (sum of element
    products), summed over blocks, in float64.  A swapped scale matrix, a scale applied to the wrong
    block or operand, or a wrong bias all fail this."""
    m, n, k = 32, 48, 256
    dtype = orc.E4M3
    a, sa, b, sb = _mx_case(2, m, n, k, dtype)
    c = np.random.default_rng(3).uniform(-1, 1, m * n).astype(np.float32)
    got = orc.gemm_mx(dtype, la, lb, 0, 0, m, n, k, a, sa, b, sb, c, 2.0, -0.5).reshape(m, n).astype(np.float64)
    A = orc.decode(dtype, a).astype(np.float64).reshape((m, k) if la == 0 else (k, m))
    A = A if la == 0 else A.T
    B = orc.decode(dtype, b).astype(np.float64).reshape((k, n) if lb == 0 else (n, k))
    B = B if lb == 0 else B.T  # k x n
    want = np.zeros((m, n))
    size = np.zeros((m, n))  # sum of the terms' magnitudes: what float32 rounding errors scale with
    for kb in range(k // 32):
        part = A[:, kb * 32:(kb + 1) * 32] @ B[kb * 32:(kb + 1) * 32, :]
        mag = np.abs(A[:, kb * 32:(kb + 1) * 32]) @ np.abs(B[kb * 32:(kb + 1) * 32, :])
        fa = 2.0 ** (sa[:, kb].astype(np.float64) - 127)
        fb = 2.0 ** (sb[:, kb].astype(np.float64) - 127)
        want += part * fa[:, None] * fb[None, :]
        size += mag * fa[:, None] * fb[None, :]
    want = 2.0 * want - 0.5 * c.reshape(m, n)
    # (float32 summation of k terms: a few ulp of the running sum per term, far below k * 2^-24 * size)
    assert np.max(np.abs(got - want) / (2.0 * size + 1.0)) < 2e-6


def test_mx_gemm_scales_are_exact_powers_of_two():
    """Raising every scale of A by one doubles the product exactly; raising one K block's scale of
    one row changes that row only."""
    m, n, k = 16, 16, 128
    dtype = orc.E5M2
    a, sa, b, sb = _mx_case(4, m, n, k, dtype)
    base = orc.gemm_mx(dtype, 0, 1, 0, 0, m, n, k, a, sa, b, sb, None, 1.0, 0.0)
    twice = orc.gemm_mx(dtype, 0, 1, 0, 0, m, n, k, a, sa + 1, b, sb, None, 1.0, 0.0)
    assert np.array_equal(twice, 2.0 * base)
    sa2 = sa.copy()
    sa2[5, 2] += 3
    one = orc.gemm_mx(dtype, 0, 1, 0, 0, m, n, k, a, sa2, b, sb, None, 1.0, 0.0).reshape(m, n)
    differs = np.any(one != base.reshape(m, n), axis=1)
    assert differs[5] and differs.sum() == 1


def test_fused_epilogue_restatement():
    """gemm_bias_act = gemm, then bias per column and activation: without either it is gemm bit for
    bit; ReLU output is the positive part; GELU against math.erf element by element; the bias follows
    the columns of D whatever D's layout."""
    import math

    m, n, k = 32, 48, 64
    rng = np.random.default_rng(7)
    a = orc.encode(orc.F16, rng.uniform(-1, 1, m * k).astype(np.float32))
    b = orc.encode(orc.F16, rng.uniform(-1, 1, k * n).astype(np.float32))
    c = rng.uniform(-1, 1, m * n).astype(np.float32)
    bias = rng.uniform(-2, 2, n).astype(np.float32)
    plain = orc.gemm(orc.F16, orc.F32, 0, 1, 0, 0, m, n, k, a, b, c, 2.0, 0.5)
    assert np.array_equal(orc.gemm_bias_act(orc.F16, orc.F32, 0, 1, 0, m, n, k, a, b, c, 2.0, 0.5, None, orc.ACT_NONE), plain)
    with_bias = orc.gemm_bias_act(orc.F16, orc.F32, 0, 1, 0, m, n, k, a, b, c, 2.0, 0.5, bias, orc.ACT_NONE).reshape(m, n)
    assert np.allclose(with_bias - plain.reshape(m, n), np.broadcast_to(bias, (m, n)), atol=1e-5)
    relu = orc.gemm_bias_act(orc.F16, orc.F32, 0, 1, 0, m, n, k, a, b, c, 2.0, 0.5, bias, orc.ACT_RELU).reshape(m, n)
    assert np.array_equal(relu, np.maximum(with_bias, 0.0))
    gelu = orc.gemm_bias_act(orc.F16, orc.F32, 0, 1, 0, m, n, k, a, b, c, 2.0, 0.5, bias, orc.ACT_GELU).reshape(m, n)
    ref = np.array([[0.5 * x * (1.0 + math.erf(x / math.sqrt(2.0))) for x in row] for row in with_bias.astype(np.float64)])
    assert np.max(np.abs(gelu - ref)) < 1e-5
    # column-major D: same values, transposed storage (c given in D's layout)
    c_cm = np.ascontiguousarray(c.reshape(m, n).T).reshape(-1)
    gelu_cm = orc.gemm_bias_act(orc.F16, orc.F32, 0, 1, 1, m, n, k, a, b, c_cm, 2.0, 0.5, bias, orc.ACT_GELU).reshape(n, m)
    assert np.array_equal(gelu_cm.T, gelu)


def test_compare_equal_metric():
    a = np.array([1.0, 2.0, -3.0, 0.0], dtype=np.float32)
    b = np.array([1.0, 2.5, -3.0, 0.0], dtype=np.float32)
    err, inf, nan = orc.compare_equal(orc.F32, a, orc.F32, b)
    assert err == pytest.approx(0.5 / (2.0 + 2.5 + 1.0)) and not inf and not nan
    b[0] = np.inf
    assert orc.compare_equal(orc.F32, a, orc.F32, b)[1]
    b[0] = np.nan
    assert orc.compare_equal(orc.F32, a, orc.F32, b)[2]


# ---------------------------------------------------------------- DLRM golden files
def _golden(golden_dir, name, shape):
    return np.fromfile(os.path.join(golden_dir, f"dlrm_{name}.bin"), dtype=np.uint16).reshape(shape)


B_, M_, K_ = 64, 27, 128
W_ = M_ * (M_ - 1) // 2 + K_


def test_dlrm_fwd_against_reference_golden_files(golden_dir):
    inp = _golden(golden_dir, "input_fp16", (B_, M_, K_))
    want = _golden(golden_dir, "output_fp16", (B_, W_))
    got = orc.dlrm_fwd(inp, M_, K_, B_)
    err, inf, nan = orc.compare_equal(orc.F16, got, orc.F16, want)
    assert not inf and not nan
    assert err <= 10 * 2.0 ** -10          # the reference's tolerance, 10 * eps(f16)
    assert err <= 5e-4                     # observed 2.3e-4: generator used another sum order
    assert np.array_equal(got[:, :K_], inp[:, 0, :])          # MLP row copied bit for bit
    assert (got == want).mean() > 0.99
    # ordering pin: the [tril | mlp] order or a column-major tril would be off by O(1)
    swapped = np.concatenate([got[:, K_:], got[:, :K_]], axis=1)
    assert orc.compare_equal(orc.F16, swapped, orc.F16, want)[0] > 0.1


def test_dlrm_bwd_against_reference_golden_files(golden_dir):
    inp = _golden(golden_dir, "input_fp16", (B_, M_, K_))
    up = _golden(golden_dir, "input_grad_fp16", (B_, W_))
    want_grad = _golden(golden_dir, "output_input_grad_fp16", (B_, M_, K_))
    want_mlp = _golden(golden_dir, "output_mlp_input_grad_fp16", (B_, K_))
    grad, mlp = orc.dlrm_bwd(inp, up, M_, K_, B_)
    assert np.array_equal(mlp, want_mlp) and np.array_equal(mlp, up[:, :K_])
    err, inf, nan = orc.compare_equal(orc.F16, grad, orc.F16, want_grad)
    assert not inf and not nan and err <= 10 * 2.0 ** -10
    # adding the MLP gradient into row 0 (a plausible mis-reading) is off by O(1)
    g = grad.view(np.float16).astype(np.float32)
    g[:, 0, :] += mlp.view(np.float16).astype(np.float32)
    assert orc.compare_equal(orc.F16, orc.encode(orc.F16, g), orc.F16, want_grad)[0] > 0.1


def test_dlrm_float32_against_reference_golden_files(golden_dir):
    """The float32 form of the two loops against the first 16 samples of the reference's fp32 data files
    (test/dlrm/data/*_fp32; tests/golden/extract_fp32.py).  The fixtures come from another summation order: 9.8 eps in
    the compareEqual metric, inside the reference's 10 * eps for float32_t."""
    b, m, k = 16, M_, K_
    g = lambda name, shape: np.fromfile(os.path.join(golden_dir, f"dlrm_{name}.bin"), dtype=np.float32).reshape(shape)
    inp, up = g("input_fp32", (b, m, k)), g("input_grad_fp32", (b, W_))
    got = orc.dlrm_fwd(inp, m, k, b, orc.F32)
    err, inf, nan = orc.compare_equal(orc.F32, got, orc.F32, g("output_fp32", (b, W_)))
    assert not inf and not nan and err <= 10 * 2.0 ** -23
    assert np.array_equal(got[:, :k], inp[:, 0, :])
    swapped = np.concatenate([got[:, k:], got[:, :k]], axis=1)
    assert orc.compare_equal(orc.F32, swapped, orc.F32, g("output_fp32", (b, W_)))[0] > 0.1
    grad, mlp = orc.dlrm_bwd(inp, up, m, k, b, orc.F32)
    assert np.array_equal(mlp, g("output_mlp_input_grad_fp32", (b, k))) and np.array_equal(mlp, up[:, :k])
    err, inf, nan = orc.compare_equal(orc.F32, grad, orc.F32, g("output_input_grad_fp32", (b, m, k)))
    assert not inf and not nan and err <= 10 * 2.0 ** -23
    with_mlp = grad.copy()
    with_mlp[:, 0, :] += mlp
    assert orc.compare_equal(orc.F32, with_mlp, orc.F32, g("output_input_grad_fp32", (b, m, k)))[0] > 0.1


def test_dlrm_float32_equals_the_f16_loops_on_f16_representable_data():
    """On inputs that are exactly representable in f16 the two element types run the same float accumulation: the f16
    results are the float32 results rounded once."""
    rng = np.random.default_rng(11)
    b, m, k = 4, 27, 64
    F = rng.uniform(-1, 1, (b, m, k)).astype(np.float16)
    up = rng.uniform(-1, 1, (b, m * (m - 1) // 2 + k)).astype(np.float16)
    out16 = orc.dlrm_fwd(F.view(np.uint16), m, k, b)
    out32 = orc.dlrm_fwd(F.astype(np.float32), m, k, b, orc.F32)
    assert np.array_equal(out16, orc.encode(orc.F16, out32.reshape(-1)).reshape(out16.shape))
    g16, m16 = orc.dlrm_bwd(F.view(np.uint16), up.view(np.uint16), m, k, b)
    g32, m32 = orc.dlrm_bwd(F.astype(np.float32), up.astype(np.float32), m, k, b, orc.F32)
    assert np.array_equal(g16, orc.encode(orc.F16, g32.reshape(-1)).reshape(g16.shape))
    assert np.array_equal(m16.view(np.float16).astype(np.float32), m32)


def test_dlrm_fwd_bwd_against_numpy_float64():
    rng = np.random.default_rng(7)
    b, m, k = 5, 27, 128
    F = rng.uniform(-1, 1, (b, m, k)).astype(np.float16)
    out = orc.dlrm_fwd(F.view(np.uint16), m, k, b).view(np.float16).astype(np.float64)
    Z = np.einsum("bik,bjk->bij", F.astype(np.float64), F.astype(np.float64))
    il, jl = np.tril_indices(m, -1)
    want = np.concatenate([F[:, 0, :].astype(np.float64), Z[:, il, jl]], axis=1)
    assert np.abs(out - want).max() < 2e-2 and np.abs(out - want).max() / 20 < 1e-3
    up = rng.uniform(-1, 1, (b, m * (m - 1) // 2 + k)).astype(np.float16)
    grad, mlp = orc.dlrm_bwd(F.view(np.uint16), up.view(np.uint16), m, k, b)
    G = np.zeros((b, m, m))
    G[:, il, jl] = up[:, k:].astype(np.float64)
    G = G + G.transpose(0, 2, 1)
    wantg = G @ F.astype(np.float64)
    assert np.abs(grad.view(np.float16).astype(np.float64) - wantg).max() < 2e-2
    # linearity in the upstream gradient (exact for power-of-two scaling)
    grad2, _ = orc.dlrm_bwd(F.view(np.uint16), (up * np.float16(0.5)).view(np.uint16), m, k, b)
    assert np.array_equal(grad2.view(np.float16), grad.view(np.float16) * np.float16(0.5))
