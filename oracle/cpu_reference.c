/*
 * CPU oracle -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's OpenMP CPU reference for the GEMM /
 * GEMV / DLRM path.  It is the checker the GPU results are compared with and the
 * "cpu_baseline" leg of the benchmark.  Nothing the library ships may link,
 * import or call this file.
 *
 * Reference followed (paths relative to the rocWMMA source tree):
 *   gemm_CPU        test/reference_impl.hpp:36-81   (sample twin samples/common.hpp:297-342)
 *   dlrm_fwd_CPU    test/reference_impl.hpp:83-119
 *   dlrm_bwd_CPU    test/reference_impl.hpp:121-179
 *   sgemv_cpu_h     samples/simple_sgemv.cpp:46-66  (== gemm with n columns)
 *   compareEqual    test/common.hpp:436-523         (sample twin samples/common.hpp:345-416)
 *
 * Arithmetic contract restated from those loops:
 *   - every input element is converted to ComputeT (f32, or i32 for int8) first;
 *   - products are formed in ComputeT and summed into one ComputeT accumulator in
 *     increasing h (k index), starting from 0, one rounding per multiply and one per
 *     add (no fused multiply-add: this file must be built with -ffp-contract=off);
 *   - GEMM output = OutputT(alpha * accum + beta * ComputeT(c));
 *   - DLRM accumulates in float and casts once to the storage type; the backward
 *     pass first materialises the symmetric zero-diagonal matrix in the storage type.
 *
 * Element types are passed as raw bit patterns so the file needs no _Float16
 * support from the compiler.  Decoders are exact; encoders round to nearest even.
 *
 * Parity pins (see tests/test_oracle.py):
 *   - oracle_gemm_fast (column-blocked, same per-element order) == oracle_gemm_naive
 *     (the reference loop nest verbatim) bit for bit;
 *   - identity / all-ones / exact-integer closed forms, int8 against numpy int64;
 *   - f16 / bf16 / e4m3 / e5m2 codecs against numpy / the OCP closed form, all codes;
 *   - DLRM forward and backward against the reference's golden files
 *     the five fp16 files of test/dlrm/data (committed under tests/golden/ as dlrm_<name>.bin);
 *   - the float32 forms of the two DLRM loops against the first 16 samples of the five fp32 files of the same
 *     directory, and against the f16 forms on f16-representable inputs (equal after one rounding).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- element type codes (shared with include/rocwmma_amd.h) ------------------ */
enum
{
    ORC_F16  = 0,
    ORC_BF16 = 1,
    ORC_E4M3 = 2, /* OCP FP8 E4M3 (no inf, S.1111.111 = NaN, max 448) */
    ORC_E5M2 = 3, /* OCP FP8 E5M2 (IEEE-like) */
    ORC_I8   = 4,
    ORC_F32  = 5,
    ORC_I32  = 6
};

enum
{
    ORC_ROW_MAJOR = 0,
    ORC_COL_MAJOR = 1
};

/* ---- codecs ------------------------------------------------------------------ */
static inline float bits_to_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint32_t f32_to_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

float oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp  = (h >> 10) & 0x1Fu;
    uint32_t man  = h & 0x3FFu;
    if(exp == 0x1Fu)
        return bits_to_f32(sign | 0x7F800000u | (man << 13));
    if(exp == 0)
    {
        /* subnormal or zero: value = man * 2^-24, exact in float */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* Generic round-to-nearest-even narrowing of an f32 to a small binary format with
 * `ebits` exponent bits, `mbits` mantissa bits and IEEE-style subnormals.
 * Returns magnitude code (without sign) as if the format had inf at all-ones exponent;
 * the callers patch the special cases. */
static uint32_t narrow_rne(float f, int ebits, int mbits, int* overflow)
{
    uint32_t u    = f32_to_bits(f) & 0x7FFFFFFFu;
    int      bias = (1 << (ebits - 1)) - 1;
    int      e    = (int)(u >> 23) - 127; /* unbiased, for normal f32 */
    uint32_t m    = u & 0x7FFFFFu;
    *overflow     = 0;
    if((u >> 23) == 0)
        return 0; /* f32 subnormal: far below any target subnormal -> 0 */
    m |= 0x800000u; /* implicit one, 24-bit significand */
    int shift = 23 - mbits; /* bits to drop for a normal result */
    int te    = e + bias; /* target biased exponent */
    if(te <= 0)
    {
        /* subnormal in target: shift further */
        shift += 1 - te;
        te = 0;
        if(shift > 25)
            return 0;
    }
    uint32_t kept = m >> shift;
    uint32_t rem  = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if(rem > half || (rem == half && (kept & 1u)))
        kept++;
    uint32_t code;
    if(te == 0)
    {
        /* kept may have carried into the normal range (== 1<<mbits): encoding is continuous */
        code = kept;
    }
    else
    {
        /* kept includes the implicit bit at position mbits; carry to 1<<(mbits+1) bumps exponent */
        code = ((uint32_t)te << mbits) + (kept - (1u << mbits));
    }
    uint32_t maxcode = ((uint32_t)((1 << ebits) - 1) << mbits); /* first inf/NaN code */
    if(code >= maxcode)
        *overflow = 1;
    return code;
}

uint16_t oracle_f32_to_f16(float f)
{
    uint32_t u    = f32_to_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    if((u & 0x7F800000u) == 0x7F800000u)
    {
        if(u & 0x7FFFFFu)
            return (uint16_t)(sign | 0x7E00u | ((u >> 13) & 0x3FFu));
        return (uint16_t)(sign | 0x7C00u);
    }
    int      ovf;
    uint32_t code = narrow_rne(f, 5, 10, &ovf);
    if(ovf)
        code = 0x7C00u;
    return (uint16_t)(sign | code);
}

float oracle_bf16_to_f32(uint16_t b)
{
    return bits_to_f32((uint32_t)b << 16);
}

uint16_t oracle_f32_to_bf16(float f)
{
    uint32_t u = f32_to_bits(f);
    if((u & 0x7F800000u) == 0x7F800000u && (u & 0x7FFFFFu))
        return (uint16_t)((u >> 16) | 0x40u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

/* OCP OFP8 E4M3: bias 7, subnormals m*2^-9, no infinities, 0x7F/0xFF = NaN, max 448 */
float oracle_e4m3_to_f32(uint8_t v)
{
    uint32_t sign = v & 0x80u;
    uint32_t exp  = (v >> 3) & 0xFu;
    uint32_t man  = v & 0x7u;
    float    r;
    if(exp == 0xFu && man == 0x7u)
        return bits_to_f32(0x7FC00000u | (sign << 24));
    if(exp == 0)
        r = (float)man * 0.001953125f; /* 2^-9 */
    else
        r = bits_to_f32(((exp + 120u) << 23) | (man << 20));
    return sign ? -r : r;
}

/* round-to-nearest-even with saturation to +-448 (the OCP "satfinite" conversion) */
uint8_t oracle_f32_to_e4m3(float f)
{
    uint32_t u    = f32_to_bits(f);
    uint8_t  sign = (uint8_t)((u >> 24) & 0x80u);
    if((u & 0x7F800000u) == 0x7F800000u)
    {
        if(u & 0x7FFFFFu)
            return (uint8_t)(sign | 0x7Fu);
        return (uint8_t)(sign | 0x7Eu); /* inf saturates */
    }
    int      ovf;
    uint32_t code = narrow_rne(f, 4, 3, &ovf);
    /* E4M3 uses the all-ones exponent for finite values up to mantissa 110 */
    if(code > 0x7Eu)
        code = 0x7Eu;
    return (uint8_t)(sign | code);
}

/* OCP OFP8 E5M2: bias 15, IEEE-like inf / NaN */
float oracle_e5m2_to_f32(uint8_t v)
{
    return oracle_f16_to_f32((uint16_t)((uint16_t)v << 8));
}

uint8_t oracle_f32_to_e5m2(float f)
{
    uint32_t u    = f32_to_bits(f);
    uint8_t  sign = (uint8_t)((u >> 24) & 0x80u);
    if((u & 0x7F800000u) == 0x7F800000u)
    {
        if(u & 0x7FFFFFu)
            return (uint8_t)(sign | 0x7Fu);
        return (uint8_t)(sign | 0x7Bu); /* inf saturates to max finite 57344 */
    }
    int      ovf;
    uint32_t code = narrow_rne(f, 5, 2, &ovf);
    if(ovf)
        code = 0x7Bu;
    return (uint8_t)(sign | code);
}

/* vectorised helpers for the tests / data generators */
void oracle_encode(int dtype, const float* src, void* dst, size_t n)
{
    size_t i;
    switch(dtype)
    {
    case ORC_F16:
        for(i = 0; i < n; i++)
            ((uint16_t*)dst)[i] = oracle_f32_to_f16(src[i]);
        break;
    case ORC_BF16:
        for(i = 0; i < n; i++)
            ((uint16_t*)dst)[i] = oracle_f32_to_bf16(src[i]);
        break;
    case ORC_E4M3:
        for(i = 0; i < n; i++)
            ((uint8_t*)dst)[i] = oracle_f32_to_e4m3(src[i]);
        break;
    case ORC_E5M2:
        for(i = 0; i < n; i++)
            ((uint8_t*)dst)[i] = oracle_f32_to_e5m2(src[i]);
        break;
    default:
        break;
    }
}

static size_t elem_size(int dtype)
{
    switch(dtype)
    {
    case ORC_F16:
    case ORC_BF16:
        return 2;
    case ORC_E4M3:
    case ORC_E5M2:
    case ORC_I8:
        return 1;
    default:
        return 4;
    }
}

static inline float decode_one(int dtype, const void* p, size_t i)
{
    switch(dtype)
    {
    case ORC_F16:
        return oracle_f16_to_f32(((const uint16_t*)p)[i]);
    case ORC_BF16:
        return oracle_bf16_to_f32(((const uint16_t*)p)[i]);
    case ORC_E4M3:
        return oracle_e4m3_to_f32(((const uint8_t*)p)[i]);
    case ORC_E5M2:
        return oracle_e5m2_to_f32(((const uint8_t*)p)[i]);
    case ORC_I8:
        return (float)((const int8_t*)p)[i];
    case ORC_F32:
        return ((const float*)p)[i];
    case ORC_I32:
        return (float)((const int32_t*)p)[i];
    default:
        return 0.0f;
    }
}

void oracle_decode(int dtype, const void* src, float* dst, size_t n)
{
    size_t i;
#pragma omp parallel for
    for(i = 0; i < n; i++)
        dst[i] = decode_one(dtype, src, i);
}

static inline size_t idx2(int layout, size_t row, size_t col, size_t ld)
{
    return layout == ORC_ROW_MAJOR ? row * ld + col : col * ld + row;
}

/* ---- GEMM: the reference loop nest verbatim (test/reference_impl.hpp:66-80) ---- */
/* dtype_out: ORC_F32 (ComputeT f32) or ORC_I32 (ComputeT i32, dtype_in must be ORC_I8),
 * or ORC_F16 / ORC_BF16 (ComputeT f32, narrow output), or ORC_I8 (ComputeT i32, narrow output:
 * the reference's <int8, int8, int32> triple, static_cast<int8_t> of the 32-bit result, which
 * keeps its low eight bits).  alpha/beta are passed as double
 * and converted to ComputeT, like the reference's by-value ComputeT arguments. */
int oracle_gemm_naive(int         dtype_in,
                      int         dtype_out,
                      int         layA,
                      int         layB,
                      int         layC,
                      int         layD,
                      uint32_t    m,
                      uint32_t    n,
                      uint32_t    k,
                      const void* a,
                      const void* b,
                      const void* c,
                      void*       d,
                      double      alpha,
                      double      beta)
{
    size_t lda = layA == ORC_ROW_MAJOR ? k : m;
    size_t ldb = layB == ORC_ROW_MAJOR ? n : k;
    size_t ldc = layC == ORC_ROW_MAJOR ? n : m;
    size_t ldd = layD == ORC_ROW_MAJOR ? n : m;
    long   i;
    if(dtype_out == ORC_I32 || dtype_out == ORC_I8)
    {
        if(dtype_in != ORC_I8)
            return -1;
        const int     out8 = dtype_out == ORC_I8;
        const int8_t* A    = (const int8_t*)a;
        const int8_t* B    = (const int8_t*)b;
        int32_t       al = (int32_t)alpha, be = (int32_t)beta;
#pragma omp parallel for
        for(i = 0; i < (long)m; ++i)
            for(size_t j = 0; j < n; ++j)
            {
                int32_t accum = 0;
                for(size_t h = 0; h < k; ++h)
                    accum += (int32_t)A[idx2(layA, i, h, lda)] * (int32_t)B[idx2(layB, h, j, ldb)];
                int32_t cv = 0;
                if(c)
                    cv = out8 ? (int32_t)((const int8_t*)c)[idx2(layC, i, j, ldc)]
                              : ((const int32_t*)c)[idx2(layC, i, j, ldc)];
                /* unsigned arithmetic: same two's-complement result, no UB on wrap */
                const uint32_t res = (uint32_t)al * (uint32_t)accum + (uint32_t)be * (uint32_t)cv;
                if(out8)
                    ((int8_t*)d)[idx2(layD, i, j, ldd)] = (int8_t)(uint8_t)(res & 0xffu);
                else
                    ((int32_t*)d)[idx2(layD, i, j, ldd)] = (int32_t)res;
            }
        return 0;
    }
    if(dtype_out != ORC_F32 && dtype_out != ORC_F16 && dtype_out != ORC_BF16)
        return -1;
    {
        float al = (float)alpha, be = (float)beta;
#pragma omp parallel for
        for(i = 0; i < (long)m; ++i)
            for(size_t j = 0; j < n; ++j)
            {
                float accum = 0.0f;
                for(size_t h = 0; h < k; ++h)
                    accum += decode_one(dtype_in, a, idx2(layA, i, h, lda))
                             * decode_one(dtype_in, b, idx2(layB, h, j, ldb));
                float cv = c ? decode_one(dtype_out, c, idx2(layC, i, j, ldc)) : 0.0f;
                float r  = al * accum + be * cv;
                size_t o = idx2(layD, i, j, ldd);
                if(dtype_out == ORC_F32)
                    ((float*)d)[o] = r;
                else if(dtype_out == ORC_F16)
                    ((uint16_t*)d)[o] = oracle_f32_to_f16(r);
                else
                    ((uint16_t*)d)[o] = oracle_f32_to_bf16(r);
            }
    }
    return 0;
}

/* ---- GEMM, fast form -----------------------------------------------------------
 * Same arithmetic per output element (ComputeT(a)*ComputeT(b) summed in increasing h
 * into one accumulator that starts at 0), restructured for speed only:
 *   - A and B are decoded to ComputeT once, A as [i][h], B as [h][j];
 *   - for each i the j loop is blocked so the compiler can keep JB independent
 *     accumulators in vector registers; no accumulator ever sees a different order.
 * `rows` (may be NULL) restricts the computation to the listed output rows; results
 * are written to d at their normal positions, other rows of d are left untouched.
 */
#define JB 64

static int gemm_fast_f32(int             dtype_in,
                         int             dtype_out,
                         int             layA,
                         int             layB,
                         int             layC,
                         int             layD,
                         uint32_t        m,
                         uint32_t        n,
                         uint32_t        k,
                         const void*     a,
                         const void*     b,
                         const void*     c,
                         void*           d,
                         float           al,
                         float           be,
                         const uint32_t* rows,
                         uint32_t        nrows)
{
    size_t lda = layA == ORC_ROW_MAJOR ? k : m;
    size_t ldb = layB == ORC_ROW_MAJOR ? n : k;
    size_t ldc = layC == ORC_ROW_MAJOR ? n : m;
    size_t ldd = layD == ORC_ROW_MAJOR ? n : m;
    size_t npad = ((size_t)n + JB - 1) / JB * JB;
    float* Bf   = (float*)calloc((size_t)k * npad, sizeof(float));
    if(!Bf)
        return -2;
    long h;
#pragma omp parallel for
    for(h = 0; h < (long)k; ++h)
        for(size_t j = 0; j < n; ++j)
            Bf[(size_t)h * npad + j] = decode_one(dtype_in, b, idx2(layB, h, j, ldb));

    uint32_t count = rows ? nrows : m;
    long     r;
#pragma omp parallel
    {
        float* Af = (float*)malloc((size_t)k * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for(r = 0; r < (long)count; ++r)
        {
            size_t i = rows ? rows[r] : (size_t)r;
            for(size_t hh = 0; hh < k; ++hh)
                Af[hh] = decode_one(dtype_in, a, idx2(layA, i, hh, lda));
            for(size_t j0 = 0; j0 < n; j0 += JB)
            {
                float acc[JB];
                for(int jj = 0; jj < JB; ++jj)
                    acc[jj] = 0.0f;
                for(size_t hh = 0; hh < k; ++hh)
                {
                    const float  av = Af[hh];
                    const float* bp = Bf + hh * npad + j0;
                    for(int jj = 0; jj < JB; ++jj)
                        acc[jj] += av * bp[jj];
                }
                size_t jend = j0 + JB < n ? JB : n - j0;
                for(size_t jj = 0; jj < jend; ++jj)
                {
                    size_t j   = j0 + jj;
                    float  cv  = c ? decode_one(dtype_out, c, idx2(layC, i, j, ldc)) : 0.0f;
                    float  res = al * acc[jj] + be * cv;
                    size_t o   = idx2(layD, i, j, ldd);
                    if(dtype_out == ORC_F32)
                        ((float*)d)[o] = res;
                    else if(dtype_out == ORC_F16)
                        ((uint16_t*)d)[o] = oracle_f32_to_f16(res);
                    else
                        ((uint16_t*)d)[o] = oracle_f32_to_bf16(res);
                }
            }
        }
        free(Af);
    }
    free(Bf);
    return 0;
}

static int gemm_fast_i32(int             layA,
                         int             layB,
                         int             layC,
                         int             layD,
                         uint32_t        m,
                         uint32_t        n,
                         uint32_t        k,
                         const int8_t*   A,
                         const int8_t*   B,
                         const void*     C,
                         void*           D,
                         int             out8, /* C and D hold int8 (low eight bits of the result) */
                         int32_t         al,
                         int32_t         be,
                         const uint32_t* rows,
                         uint32_t        nrows)
{
    size_t lda = layA == ORC_ROW_MAJOR ? k : m;
    size_t ldb = layB == ORC_ROW_MAJOR ? n : k;
    size_t ldc = layC == ORC_ROW_MAJOR ? n : m;
    size_t ldd = layD == ORC_ROW_MAJOR ? n : m;
    size_t npad = ((size_t)n + JB - 1) / JB * JB;
    int16_t* Bw = (int16_t*)calloc((size_t)k * npad, sizeof(int16_t));
    if(!Bw)
        return -2;
    long h;
#pragma omp parallel for
    for(h = 0; h < (long)k; ++h)
        for(size_t j = 0; j < n; ++j)
            Bw[(size_t)h * npad + j] = B[idx2(layB, h, j, ldb)];
    uint32_t count = rows ? nrows : m;
    long     r;
#pragma omp parallel
    {
        int32_t* Aw = (int32_t*)malloc((size_t)k * sizeof(int32_t));
#pragma omp for schedule(dynamic, 1)
        for(r = 0; r < (long)count; ++r)
        {
            size_t i = rows ? rows[r] : (size_t)r;
            for(size_t hh = 0; hh < k; ++hh)
                Aw[hh] = A[idx2(layA, i, hh, lda)];
            for(size_t j0 = 0; j0 < n; j0 += JB)
            {
                int32_t acc[JB];
                for(int jj = 0; jj < JB; ++jj)
                    acc[jj] = 0;
                for(size_t hh = 0; hh < k; ++hh)
                {
                    const int32_t  av = Aw[hh];
                    const int16_t* bp = Bw + hh * npad + j0;
                    for(int jj = 0; jj < JB; ++jj)
                        acc[jj] += av * (int32_t)bp[jj];
                }
                size_t jend = j0 + JB < n ? JB : n - j0;
                for(size_t jj = 0; jj < jend; ++jj)
                {
                    size_t  j  = j0 + jj;
                    int32_t cv = 0;
                    if(C)
                        cv = out8 ? (int32_t)((const int8_t*)C)[idx2(layC, i, j, ldc)]
                                  : ((const int32_t*)C)[idx2(layC, i, j, ldc)];
                    const uint32_t res = (uint32_t)al * (uint32_t)acc[jj] + (uint32_t)be * (uint32_t)cv;
                    if(out8)
                        ((int8_t*)D)[idx2(layD, i, j, ldd)] = (int8_t)(uint8_t)(res & 0xffu);
                    else
                        ((int32_t*)D)[idx2(layD, i, j, ldd)] = (int32_t)res;
                }
            }
        }
        free(Aw);
    }
    free(Bw);
    return 0;
}

int oracle_gemm_rows(int             dtype_in,
                     int             dtype_out,
                     int             layA,
                     int             layB,
                     int             layC,
                     int             layD,
                     uint32_t        m,
                     uint32_t        n,
                     uint32_t        k,
                     const void*     a,
                     const void*     b,
                     const void*     c,
                     void*           d,
                     double          alpha,
                     double          beta,
                     const uint32_t* rows,
                     uint32_t        nrows)
{
    if(dtype_out == ORC_I32 || dtype_out == ORC_I8)
    {
        if(dtype_in != ORC_I8)
            return -1;
        return gemm_fast_i32(layA, layB, layC, layD, m, n, k, (const int8_t*)a, (const int8_t*)b, c, d,
                             dtype_out == ORC_I8, (int32_t)alpha, (int32_t)beta, rows, nrows);
    }
    if(dtype_out != ORC_F32 && dtype_out != ORC_F16 && dtype_out != ORC_BF16)
        return -1;
    return gemm_fast_f32(dtype_in, dtype_out, layA, layB, layC, layD, m, n, k, a, b, c, d,
                         (float)alpha, (float)beta, rows, nrows);
}

int oracle_gemm(int         dtype_in,
                int         dtype_out,
                int         layA,
                int         layB,
                int         layC,
                int         layD,
                uint32_t    m,
                uint32_t    n,
                uint32_t    k,
                const void* a,
                const void* b,
                const void* c,
                void*       d,
                double      alpha,
                double      beta)
{
    return oracle_gemm_rows(dtype_in, dtype_out, layA, layB, layC, layD, m, n, k, a, b, c, d, alpha,
                            beta, NULL, 0);
}

/* ---- DLRM forward (test/reference_impl.hpp:83-119), DataT = f16 bits ------------ */
void oracle_dlrm_fwd_f16(
    const uint16_t* input, uint16_t* output, uint32_t m, uint32_t k, uint32_t batch)
{
    size_t batchOffset       = (size_t)m * k;
    size_t outputBatchOffset = ((size_t)m * (m - 1)) / 2 + k;
    long   b;
#pragma omp parallel for
    for(b = 0; b < (long)batch; b++)
    {
        size_t outputIdx = b * outputBatchOffset;
        for(uint32_t i = 0; i < k; i++)
            output[outputIdx++] = input[b * batchOffset + i];
        for(uint32_t i = 0; i < m; i++)
            for(uint32_t j = 0; j < m; j++)
            {
                if(j >= i)
                    continue; /* the reference computes and discards these */
                float accum = 0.0f;
                for(uint32_t h = 0; h < k; h++)
                    accum += oracle_f16_to_f32(input[b * batchOffset + (size_t)i * k + h])
                             * oracle_f16_to_f32(input[b * batchOffset + (size_t)j * k + h]);
                output[outputIdx++] = oracle_f32_to_f16(accum);
            }
    }
}

/* ---- DLRM backward (test/reference_impl.hpp:121-179), DataT = f16 bits ---------- */
void oracle_dlrm_bwd_f16(const uint16_t* input,
                         const uint16_t* upstreamGrad,
                         uint16_t*       bottomMlpGrad,
                         uint16_t*       output,
                         uint32_t        m,
                         uint32_t        k,
                         uint32_t        batch)
{
    size_t batchOffset = (size_t)m * k;
    size_t accOffset   = (size_t)m * m;
    size_t trilSize    = ((size_t)m * (m - 1)) / 2 + k;
    long   b;
#pragma omp parallel
    {
        /* the reference materialises acc in DataT (f16); values are copies, so holding the
         * decoded floats is identical */
        float* acc = (float*)malloc(accOffset * sizeof(float));
        float* in  = (float*)malloc(batchOffset * sizeof(float));
#pragma omp for
        for(b = 0; b < (long)batch; b++)
        {
            for(uint32_t j = 0; j < k; j++)
                bottomMlpGrad[b * (size_t)k + j] = upstreamGrad[b * trilSize + j];
            size_t upstreamIdx = b * trilSize + k;
            for(uint32_t i = 0; i < m; i++)
                for(uint32_t j = 0; j <= i; j++)
                {
                    if(i == j)
                        acc[(size_t)i * m + j] = 0.0f;
                    else
                    {
                        float g                = oracle_f16_to_f32(upstreamGrad[upstreamIdx++]);
                        acc[(size_t)i * m + j] = g;
                        acc[(size_t)j * m + i] = g;
                    }
                }
            for(size_t e = 0; e < batchOffset; e++)
                in[e] = oracle_f16_to_f32(input[b * batchOffset + e]);
            for(uint32_t i = 0; i < m; i++)
                for(uint32_t j = 0; j < k; j++)
                {
                    float accum = 0.0f;
                    for(uint32_t h = 0; h < m; h++)
                        accum += acc[(size_t)i * m + h] * in[(size_t)h * k + j];
                    output[b * batchOffset + (size_t)i * k + j] = oracle_f32_to_f16(accum);
                }
        }
        free(acc);
        free(in);
    }
}

/* ---- DLRM forward / backward, DataT = float (the same loops with the identity for the conversions; the
 * reference's DLRM tests instantiate float32_t as well, test/dlrm/test/dlrm_test_params.hpp:51, and its data
 * directory holds fp32 fixtures next to the fp16 ones) ----------------------------------------------------- */
void oracle_dlrm_fwd_f32(const float* input, float* output, uint32_t m, uint32_t k, uint32_t batch)
{
    size_t batchOffset       = (size_t)m * k;
    size_t outputBatchOffset = ((size_t)m * (m - 1)) / 2 + k;
    long   b;
#pragma omp parallel for
    for(b = 0; b < (long)batch; b++)
    {
        size_t outputIdx = b * outputBatchOffset;
        for(uint32_t i = 0; i < k; i++)
            output[outputIdx++] = input[b * batchOffset + i];
        for(uint32_t i = 0; i < m; i++)
            for(uint32_t j = 0; j < i; j++) /* (the reference computes and discards j >= i) */
            {
                float accum = 0.0f;
                for(uint32_t h = 0; h < k; h++)
                    accum += input[b * batchOffset + (size_t)i * k + h] * input[b * batchOffset + (size_t)j * k + h];
                output[outputIdx++] = accum;
            }
    }
}

void oracle_dlrm_bwd_f32(const float* input,
                         const float* upstreamGrad,
                         float*       bottomMlpGrad,
                         float*       output,
                         uint32_t     m,
                         uint32_t     k,
                         uint32_t     batch)
{
    size_t batchOffset = (size_t)m * k;
    size_t accOffset   = (size_t)m * m;
    size_t trilSize    = ((size_t)m * (m - 1)) / 2 + k;
    long   b;
#pragma omp parallel
    {
        float* acc = (float*)malloc(accOffset * sizeof(float));
#pragma omp for
        for(b = 0; b < (long)batch; b++)
        {
            for(uint32_t j = 0; j < k; j++)
                bottomMlpGrad[b * (size_t)k + j] = upstreamGrad[b * trilSize + j];
            size_t upstreamIdx = b * trilSize + k;
            for(uint32_t i = 0; i < m; i++)
                for(uint32_t j = 0; j <= i; j++)
                {
                    if(i == j)
                        acc[(size_t)i * m + j] = 0.0f;
                    else
                    {
                        float g                = upstreamGrad[upstreamIdx++];
                        acc[(size_t)i * m + j] = g;
                        acc[(size_t)j * m + i] = g;
                    }
                }
            for(uint32_t i = 0; i < m; i++)
                for(uint32_t j = 0; j < k; j++)
                {
                    float accum = 0.0f;
                    for(uint32_t h = 0; h < m; h++)
                        accum += acc[(size_t)i * m + h] * input[b * batchOffset + (size_t)h * k + j];
                    output[b * batchOffset + (size_t)i * k + j] = accum;
                }
        }
        free(acc);
    }
}

/* ---- compareEqual (test/common.hpp:436-523) ---------------------------------- */
/* Returns max over elements of |a-b| / (|a|+|b|+1) evaluated in double after a float
 * conversion of each side.  *flags: bit0 = an inf was met, bit1 = a NaN was met. */
double oracle_compare_equal(int dtype_a, const void* a, int dtype_b, const void* b, size_t n, int* flags)
{
    double max_rel = 0.0;
    int    is_inf = 0, is_nan = 0;
    long   i;
#pragma omp parallel for reduction(max : max_rel) reduction(| : is_inf) reduction(| : is_nan)
    for(i = 0; i < (long)n; ++i)
    {
        double va = (double)decode_one(dtype_a, a, i);
        double vb = (double)decode_one(dtype_b, b, i);
        if(dtype_a == ORC_I32)
            va = (double)((const int32_t*)a)[i];
        if(dtype_b == ORC_I32)
            vb = (double)((const int32_t*)b)[i];
        double num = fabs(va - vb);
        double den = fabs(va) + fabs(vb) + 1.0;
        if(isinf(num) || isinf(den))
            is_inf |= 1;
        else
        {
            double rel = num / den;
            if(isnan(rel))
                is_nan |= 1;
            else if(rel > max_rel)
                max_rel = rel;
        }
    }
    if(flags)
        *flags = (is_inf ? 1 : 0) | (is_nan ? 2 : 0);
    return max_rel;
}

int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

size_t oracle_elem_size(int dtype)
{
    return elem_size(dtype);
}
