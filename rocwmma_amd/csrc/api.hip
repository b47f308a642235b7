// extern "C" entry points of librocwmma_amd.so: argument validation and dispatch to the kernel
// families.  Declarations and the reference interfaces they stand in for: include/rocwmma_amd.h.
#include "common.hpp"

#include <atomic>
#include <cmath>
#include <cstring>
#include <utility>

namespace rocwmma_amd
{
    int launchGemv(uint32_t m, uint32_t k, uint32_t ncols, const void* a, uint32_t lda, const void* x, uint32_t ldx,
                   float* y, uint32_t ldy, float alpha, float beta, hipStream_t stream);
    int launchDlrmFwd(const void* input, void* output, uint32_t m, uint32_t k, uint32_t batch, hipStream_t stream);
    int launchDlrmFwdF32(const void* input, void* output, uint32_t m, uint32_t k, uint32_t batch, hipStream_t stream);
    int launchDlrmFwdGeneral(int dtype, const void* input, void* output, uint32_t m, uint32_t k, uint32_t batch, hipStream_t stream);
    int launchDlrmBwdGeneral(int dtype, const void* input, const void* upstream, void* grad, void* mlpGrad, uint32_t m, uint32_t k,
                             uint32_t batch, hipStream_t stream);
    int launchDlrmBwdF32(const void* input, const void* upstream, void* grad, void* mlpGrad, uint32_t m, uint32_t k, uint32_t batch,
                         hipStream_t stream);
    int launchDlrmBwd(const void* input, const void* upstream, void* grad, void* mlpGrad, uint32_t m, uint32_t k,
                      uint32_t batch, hipStream_t stream);

    namespace
    {
        bool validLayout(int l)
        {
            return l == ROCWMMA_AMD_ROW_MAJOR || l == ROCWMMA_AMD_COL_MAJOR;
        }

        // Whether the current device is a gfx950.  The answer never changes for a device, so it
        // is remembered per device ordinal (0 = not asked yet, 1 = yes, 2 = no).
        bool isGfx950Current()
        {
            constexpr int           kMaxDevices = 64;
            static std::atomic<int> known[kMaxDevices];
            int                     dev = 0;
            if(hipGetDevice(&dev) != hipSuccess)
                return false;
            if(dev >= 0 && dev < kMaxDevices)
            {
                const int cached = known[dev].load(std::memory_order_relaxed);
                if(cached != 0)
                    return cached == 1;
            }
            hipDeviceProp_t props;
            if(hipGetDeviceProperties(&props, dev) != hipSuccess)
                return false;
            const bool yes = std::strncmp(props.gcnArchName, "gfx950", 6) == 0;
            if(dev >= 0 && dev < kMaxDevices)
                known[dev].store(yes ? 1 : 2, std::memory_order_relaxed);
            return yes;
        }

        // Pure argument checks of the GEMM entry points (no device access): shared by the
        // entry points and testable without a GPU.
        int checkGemm(int dtypeIn, int dtypeOut, int layoutA, int layoutB, int layoutC, uint32_t m, uint32_t n, uint32_t k,
                      const void* a, uint32_t lda, const void* b, uint32_t ldb, const void* c, uint32_t ldc, void* d,
                      uint32_t ldd, float alpha, float beta)
        {
            if(!a || !b || !d || m == 0u || n == 0u || k == 0u)
                return ROCWMMA_AMD_INVALID_ARGUMENT;
            if(!validLayout(layoutA) || !validLayout(layoutB) || !validLayout(layoutC))
                return ROCWMMA_AMD_INVALID_ARGUMENT;
            if(!c && beta != 0.0f)
                return ROCWMMA_AMD_INVALID_ARGUMENT;
            const bool floatIn = dtypeIn == ROCWMMA_AMD_F16 || dtypeIn == ROCWMMA_AMD_BF16 || dtypeIn == ROCWMMA_AMD_E4M3
                                 || dtypeIn == ROCWMMA_AMD_E5M2;
            const bool okTypes = (floatIn && dtypeOut == ROCWMMA_AMD_F32)
                                 || (dtypeIn == ROCWMMA_AMD_F16 && dtypeOut == ROCWMMA_AMD_F16)
                                 || (dtypeIn == ROCWMMA_AMD_BF16 && dtypeOut == ROCWMMA_AMD_BF16)
                                 || (dtypeIn == ROCWMMA_AMD_F32 && dtypeOut == ROCWMMA_AMD_F32)
                                 || (dtypeIn == ROCWMMA_AMD_I8 && (dtypeOut == ROCWMMA_AMD_I32 || dtypeOut == ROCWMMA_AMD_I8));
            if(!okTypes)
                return ROCWMMA_AMD_UNSUPPORTED_TYPE;
            if(dtypeIn == ROCWMMA_AMD_I8 && (alpha != std::nearbyint(alpha) || beta != std::nearbyint(beta)))
                return ROCWMMA_AMD_INVALID_ARGUMENT;
            const uint32_t inSize  = dtypeSize(dtypeIn);
            const uint32_t outSize = dtypeSize(dtypeOut);
            if(m % 16u != 0u || n % 16u != 0u || (k * inSize) % 32u != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            const uint32_t minLda = layoutA == ROCWMMA_AMD_ROW_MAJOR ? k : m;
            const uint32_t minLdb = layoutB == ROCWMMA_AMD_ROW_MAJOR ? n : k;
            const uint32_t minLdc = layoutC == ROCWMMA_AMD_ROW_MAJOR ? n : m;
            if(lda < minLda || ldb < minLdb || ldd < minLdc || (c && ldc < minLdc))
                return ROCWMMA_AMD_BAD_LEADING_DIM;
            if(!aligned16(a) || !aligned16(b) || !aligned16(d) || (c && !aligned16(c)))
                return ROCWMMA_AMD_BAD_ALIGNMENT;
            if((lda * inSize) % 16u != 0u || (ldb * inSize) % 16u != 0u || (ldd * outSize) % 16u != 0u
               || (c && (ldc * outSize) % 16u != 0u))
                return ROCWMMA_AMD_BAD_ALIGNMENT;
            return ROCWMMA_AMD_OK;
        }

        int flip(int layout)
        {
            return layout == ROCWMMA_AMD_ROW_MAJOR ? ROCWMMA_AMD_COL_MAJOR : ROCWMMA_AMD_ROW_MAJOR;
        }

        // The blocked kernels write row-major C/D; a column-major result is the row-major result of
        // the transposed problem D^T = B^T * A^T.
        void transposeForColMajorC(GemmArgs& g, int& layoutA, int& layoutB)
        {
            if(g.layoutC != ROCWMMA_AMD_COL_MAJOR)
                return;
            std::swap(g.m, g.n);
            std::swap(g.a, g.b);
            std::swap(g.lda, g.ldb);
            const int la = flip(layoutB), lb = flip(layoutA);
            layoutA      = la;
            layoutB      = lb;
            g.layoutC    = ROCWMMA_AMD_ROW_MAJOR;
        }
    } // namespace
} // namespace rocwmma_amd

using namespace rocwmma_amd;

extern "C" {

int rocwmma_amd_version(void)
{
    return ROCWMMA_VERSION_MAJOR * 10000 + ROCWMMA_VERSION_MINOR * 100 + ROCWMMA_VERSION_PATCH;
}

const char* rocwmma_amd_status_string(int status)
{
    switch(status)
    {
    case ROCWMMA_AMD_OK:
        return "success";
    case ROCWMMA_AMD_INVALID_ARGUMENT:
        return "invalid argument (null pointer, zero size or bad enum)";
    case ROCWMMA_AMD_UNSUPPORTED_TYPE:
        return "unsupported element type combination";
    case ROCWMMA_AMD_UNSUPPORTED_SHAPE:
        return "unsupported size: not a multiple of the block the kernel needs";
    case ROCWMMA_AMD_BAD_ALIGNMENT:
        return "pointer or leading dimension is not 16-byte aligned";
    case ROCWMMA_AMD_BAD_LEADING_DIM:
        return "leading dimension smaller than the matrix extent";
    case ROCWMMA_AMD_NO_DEVICE:
        return "no gfx950 device is current";
    case ROCWMMA_AMD_LAUNCH_FAILED:
        return "kernel launch failed";
    case ROCWMMA_AMD_SCRATCH_TOO_SMALL:
        return "the library's static scratch is too small for this device";
    default:
        return "unknown status";
    }
}

int rocwmma_amd_device_info(int* compute_units, int* clock_mhz, int* is_gfx950)
{
    int dev = 0;
    if(hipGetDevice(&dev) != hipSuccess)
        return ROCWMMA_AMD_NO_DEVICE;
    hipDeviceProp_t props;
    if(hipGetDeviceProperties(&props, dev) != hipSuccess)
        return ROCWMMA_AMD_NO_DEVICE;
    if(compute_units)
        *compute_units = props.multiProcessorCount;
    if(clock_mhz)
        *clock_mhz = props.clockRate / 1000;
    if(is_gfx950)
        *is_gfx950 = std::strncmp(props.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
    return ROCWMMA_AMD_OK;
}

int rocwmma_amd_gemm_ex(int         algo,
                        int         dtype_in,
                        int         dtype_out,
                        int         layout_a,
                        int         layout_b,
                        int         layout_c,
                        uint32_t    m,
                        uint32_t    n,
                        uint32_t    k,
                        const void* a,
                        uint32_t    lda,
                        const void* b,
                        uint32_t    ldb,
                        const void* c,
                        uint32_t    ldc,
                        void*       d,
                        uint32_t    ldd,
                        float       alpha,
                        float       beta,
                        void*       stream)
{
    int rc = checkGemm(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, a, lda, b, ldb, c, ldc, d, ldd, alpha, beta);
    if(rc != ROCWMMA_AMD_OK)
        return rc;
    if(algo != ROCWMMA_AMD_GEMM_AUTO && algo != ROCWMMA_AMD_GEMM_WAVE_TILE && algo != ROCWMMA_AMD_GEMM_BLOCKED
       && algo != ROCWMMA_AMD_GEMM_BLOCKED_256)
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;

    GemmArgs args{m, n, k, a, b, c, d, lda, ldb, c ? ldc : ldd, ldd, alpha, beta, layout_c};
    if(algo == ROCWMMA_AMD_GEMM_AUTO && m <= 128u)
    {
        // few token rows against a wide 8-bit weight matrix: the weight-streaming kernels (<= 32 rows;
        // 48 rows with the K slices spread over workgroups)
        rc = launchGemmSkinny(dtype_in, dtype_out, layout_a, layout_b, args, asStream(stream));
        if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE && rc != ROCWMMA_AMD_UNSUPPORTED_TYPE)
            return rc;
    }
    if(algo != ROCWMMA_AMD_GEMM_WAVE_TILE)
    {
        GemmArgs blocked = args;
        int      la = layout_a, lb = layout_b;
        transposeForColMajorC(blocked, la, lb);
        rc = launchGemmBlocked(dtype_in, dtype_out, la, lb, blocked, asStream(stream), algo == ROCWMMA_AMD_GEMM_BLOCKED_256);
        if(rc == ROCWMMA_AMD_OK || algo == ROCWMMA_AMD_GEMM_BLOCKED || algo == ROCWMMA_AMD_GEMM_BLOCKED_256)
            return rc;
        if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE && rc != ROCWMMA_AMD_UNSUPPORTED_TYPE)
            return rc;
    }
    return launchGemmWaveTile(dtype_in, dtype_out, layout_a, layout_b, args, asStream(stream));
}

size_t rocwmma_amd_gemm_streamk_workspace_size(void)
{
    return streamKWorkspaceBytes(computeUnits());
}

int rocwmma_amd_gemm_streamk(int         dtype_in,
                             int         dtype_out,
                             int         layout_a,
                             int         layout_b,
                             int         layout_c,
                             uint32_t    m,
                             uint32_t    n,
                             uint32_t    k,
                             const void* a,
                             uint32_t    lda,
                             const void* b,
                             uint32_t    ldb,
                             const void* c,
                             uint32_t    ldc,
                             void*       d,
                             uint32_t    ldd,
                             float       alpha,
                             float       beta,
                             void*       workspace,
                             size_t      workspace_bytes,
                             void*       stream)
{
    int rc = checkGemm(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, a, lda, b, ldb, c, ldc, d, ldd, alpha, beta);
    if(rc != ROCWMMA_AMD_OK)
        return rc;
    if(!workspace)
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    GemmArgs args{m, n, k, a, b, c, d, lda, ldb, c ? ldc : ldd, ldd, alpha, beta, layout_c};
    int      la = layout_a, lb = layout_b;
    transposeForColMajorC(args, la, lb);
    return launchGemmStreamK(dtype_in, dtype_out, la, lb, args, workspace, workspace_bytes, asStream(stream));
}

int rocwmma_amd_gemm_streamk_timed_out(void* workspace, size_t workspace_bytes, void* stream, int* timed_out)
{
    if(!timed_out || (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0u))
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    return streamKTimedOut(workspace, workspace_bytes, asStream(stream), timed_out);
}

int rocwmma_amd_gemm_streamk_static(int         dtype_in,
                                    int         dtype_out,
                                    int         layout_a,
                                    int         layout_b,
                                    int         layout_c,
                                    uint32_t    m,
                                    uint32_t    n,
                                    uint32_t    k,
                                    const void* a,
                                    uint32_t    lda,
                                    const void* b,
                                    uint32_t    ldb,
                                    const void* c,
                                    uint32_t    ldc,
                                    void*       d,
                                    uint32_t    ldd,
                                    float       alpha,
                                    float       beta,
                                    void*       stream)
{
    int rc = checkGemm(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, a, lda, b, ldb, c, ldc, d, ldd, alpha, beta);
    if(rc != ROCWMMA_AMD_OK)
        return rc;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    GemmArgs args{m, n, k, a, b, c, d, lda, ldb, c ? ldc : ldd, ldd, alpha, beta, layout_c};
    int      la = layout_a, lb = layout_b;
    transposeForColMajorC(args, la, lb);
    return launchGemmStreamKStatic(dtype_in, dtype_out, la, lb, args, asStream(stream));
}

int rocwmma_amd_gemm_bias_act(int          dtype_in,
                              int          dtype_out,
                              int          layout_a,
                              int          layout_b,
                              int          layout_c,
                              uint32_t     m,
                              uint32_t     n,
                              uint32_t     k,
                              const void*  a,
                              uint32_t     lda,
                              const void*  b,
                              uint32_t     ldb,
                              const void*  c,
                              uint32_t     ldc,
                              void*        d,
                              uint32_t     ldd,
                              float        alpha,
                              float        beta,
                              const float* bias,
                              int          activation,
                              void*        stream)
{
    int rc = checkGemm(dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, a, lda, b, ldb, c, ldc, d, ldd, alpha, beta);
    if(rc != ROCWMMA_AMD_OK)
        return rc;
    if(dtype_in == ROCWMMA_AMD_I8 || dtype_in == ROCWMMA_AMD_F32)
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    if(activation != ROCWMMA_AMD_ACT_NONE && activation != ROCWMMA_AMD_ACT_RELU && activation != ROCWMMA_AMD_ACT_GELU)
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(bias && !aligned16(bias))
        return ROCWMMA_AMD_BAD_ALIGNMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    GemmArgs args{m, n, k, a, b, c, d, lda, ldb, c ? ldc : ldd, ldd, alpha, beta, layout_c, bias, activation};
    rc = launchGemmBlockedFused(dtype_in, dtype_out, layout_a, layout_b, args, asStream(stream));
    if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE && rc != ROCWMMA_AMD_UNSUPPORTED_TYPE)
        return rc;
    return launchGemmWaveTile(dtype_in, dtype_out, layout_a, layout_b, args, asStream(stream));
}

namespace
{
    // The blocked block-scaled kernels take: row-major A / col-major B for a row-major C (the transposed
    // problem for a col-major C), k in whole 128-byte stages, operand spans inside a copy's window.
    // Fills in the problem as those kernels see it (and the scales swapped with it).
    bool mxBlockedProblem(int layout_a, int layout_b, GemmArgs const& args, MxScales const& scales, GemmArgs& blocked, MxScales& sc)
    {
        blocked = args;
        sc      = scales;
        int la = layout_a, lb = layout_b;
        if(blocked.layoutC == ROCWMMA_AMD_COL_MAJOR)
        {
            std::swap(sc.a, sc.b);
            std::swap(sc.lda, sc.ldb);
        }
        transposeForColMajorC(blocked, la, lb);
        return la == ROCWMMA_AMD_ROW_MAJOR && lb == ROCWMMA_AMD_COL_MAJOR && args.k % 128u == 0u
               && static_cast<uint64_t>(blocked.lda) * 128u < 0x7FFF0000ull && static_cast<uint64_t>(blocked.ldb) * 128u < 0x7FFF0000ull;
    }

    bool mxWorkspaceFits(const void* workspace, size_t bytes, uint32_t m, uint32_t n, uint32_t k)
    {
        return workspace && bytes >= mxPackedScaleBytes(m, n, k) && (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0u;
    }
} // namespace

size_t rocwmma_amd_gemm_mx_workspace_size(uint32_t m, uint32_t n, uint32_t k)
{
    return mxPackedScaleBytes(m, n, k);
}

int rocwmma_amd_gemm_mx(int         dtype_in,
                        int         layout_a,
                        int         layout_b,
                        int         layout_c,
                        uint32_t    m,
                        uint32_t    n,
                        uint32_t    k,
                        const void* a,
                        uint32_t    lda,
                        const void* scale_a,
                        uint32_t    ld_scale_a,
                        const void* b,
                        uint32_t    ldb,
                        const void* scale_b,
                        uint32_t    ld_scale_b,
                        const void* c,
                        uint32_t    ldc,
                        void*       d,
                        uint32_t    ldd,
                        float       alpha,
                        float       beta,
                        void*       workspace,
                        size_t      workspace_bytes,
                        void*       stream)
{
    if(dtype_in != ROCWMMA_AMD_E4M3 && dtype_in != ROCWMMA_AMD_E5M2)
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    int rc = checkGemm(dtype_in, ROCWMMA_AMD_F32, layout_a, layout_b, layout_c, m, n, k, a, lda, b, ldb, c, ldc, d, ldd, alpha, beta);
    if(rc != ROCWMMA_AMD_OK)
        return rc;
    if(!scale_a || !scale_b)
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(k % 64u != 0u)
        return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
    if(ld_scale_a < k / 32u || ld_scale_b < k / 32u)
        return ROCWMMA_AMD_BAD_LEADING_DIM;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    GemmArgs args{m, n, k, a, b, c, d, lda, ldb, c ? ldc : ldd, ldd, alpha, beta, layout_c};
    MxScales scales{static_cast<const uint8_t*>(scale_a), static_cast<const uint8_t*>(scale_b), ld_scale_a, ld_scale_b};
    if(m <= 32u)
    {
        // few token rows against a wide weight matrix: the weight-streaming kernel
        rc = launchGemmMxSkinny(dtype_in, layout_a, layout_b, args, scales, asStream(stream));
        if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE && rc != ROCWMMA_AMD_UNSUPPORTED_TYPE)
            return rc;
    }
    if(mxWorkspaceFits(workspace, workspace_bytes, m, n, k))
    {
        GemmArgs blocked;
        MxScales sc;
        if(mxBlockedProblem(layout_a, layout_b, args, scales, blocked, sc))
        {
            char* packedA = static_cast<char*>(workspace);
            char* packedB = packedA + mxPackedScaleOffsetB(blocked.m, k);
            rc            = launchMxPackScales(sc, blocked.m, blocked.n, k, packedA, packedB, !gemmMxBlockedUsesLargeTile(blocked),
                                               asStream(stream));
            if(rc != ROCWMMA_AMD_OK)
                return rc;
            rc = launchGemmMxBlocked(dtype_in, blocked, packedA, packedB, asStream(stream));
            if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                return rc;
        }
    }
    return launchGemmMxWaveTile(dtype_in, layout_a, layout_b, args, scales, asStream(stream));
}

int rocwmma_amd_gemm_mx_pack_scales(int         layout_a,
                                    int         layout_b,
                                    int         layout_c,
                                    uint32_t    m,
                                    uint32_t    n,
                                    uint32_t    k,
                                    const void* scale_a,
                                    uint32_t    ld_scale_a,
                                    const void* scale_b,
                                    uint32_t    ld_scale_b,
                                    void*       workspace,
                                    size_t      workspace_bytes,
                                    void*       stream)
{
    if(!validLayout(layout_a) || !validLayout(layout_b) || !validLayout(layout_c) || m == 0u || n == 0u || k == 0u
       || (!scale_a && !scale_b))
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(m % 16u != 0u || n % 16u != 0u || k % 128u != 0u)
        return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
    if((scale_a && ld_scale_a < k / 32u) || (scale_b && ld_scale_b < k / 32u))
        return ROCWMMA_AMD_BAD_LEADING_DIM;
    if(!mxWorkspaceFits(workspace, workspace_bytes, m, n, k))
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    // (only the shape, the layouts and the scales matter here: dense leading dimensions stand in for the operands')
    GemmArgs args{m, n, k, nullptr, nullptr, nullptr, nullptr, layout_a == ROCWMMA_AMD_ROW_MAJOR ? k : m,
                  layout_b == ROCWMMA_AMD_ROW_MAJOR ? n : k, 0u, 0u, 1.0f, 0.0f, layout_c};
    MxScales scales{static_cast<const uint8_t*>(scale_a), static_cast<const uint8_t*>(scale_b), ld_scale_a, ld_scale_b};
    GemmArgs blocked;
    MxScales sc;
    if(!mxBlockedProblem(layout_a, layout_b, args, scales, blocked, sc))
        return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
    char* packedA = static_cast<char*>(workspace);
    char* packedB = packedA + mxPackedScaleOffsetB(blocked.m, k);
    return launchMxPackScales(sc, blocked.m, blocked.n, k, packedA, packedB, !gemmMxBlockedUsesLargeTile(blocked), asStream(stream));
}

int rocwmma_amd_gemm_mx_packed(int         dtype_in,
                               int         layout_a,
                               int         layout_b,
                               int         layout_c,
                               uint32_t    m,
                               uint32_t    n,
                               uint32_t    k,
                               const void* a,
                               uint32_t    lda,
                               const void* b,
                               uint32_t    ldb,
                               const void* c,
                               uint32_t    ldc,
                               void*       d,
                               uint32_t    ldd,
                               float       alpha,
                               float       beta,
                               const void* workspace,
                               size_t      workspace_bytes,
                               void*       stream)
{
    if(dtype_in != ROCWMMA_AMD_E4M3 && dtype_in != ROCWMMA_AMD_E5M2)
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    int rc = checkGemm(dtype_in, ROCWMMA_AMD_F32, layout_a, layout_b, layout_c, m, n, k, a, lda, b, ldb, c, ldc, d, ldd, alpha, beta);
    if(rc != ROCWMMA_AMD_OK)
        return rc;
    if(m % 16u != 0u || n % 16u != 0u || k % 128u != 0u)
        return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
    if(!mxWorkspaceFits(workspace, workspace_bytes, m, n, k))
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    GemmArgs args{m, n, k, a, b, c, d, lda, ldb, c ? ldc : ldd, ldd, alpha, beta, layout_c};
    GemmArgs blocked;
    MxScales sc, none{};
    if(!mxBlockedProblem(layout_a, layout_b, args, none, blocked, sc))
        return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
    const char* packedA = static_cast<const char*>(workspace);
    const char* packedB = packedA + mxPackedScaleOffsetB(blocked.m, k);
    return launchGemmMxBlocked(dtype_in, blocked, packedA, packedB, asStream(stream));
}

int rocwmma_amd_gemm(int         dtype_in,
                     int         dtype_out,
                     int         layout_a,
                     int         layout_b,
                     int         layout_c,
                     uint32_t    m,
                     uint32_t    n,
                     uint32_t    k,
                     const void* a,
                     uint32_t    lda,
                     const void* b,
                     uint32_t    ldb,
                     const void* c,
                     uint32_t    ldc,
                     void*       d,
                     uint32_t    ldd,
                     float       alpha,
                     float       beta,
                     void*       stream)
{
    return rocwmma_amd_gemm_ex(ROCWMMA_AMD_GEMM_AUTO, dtype_in, dtype_out, layout_a, layout_b, layout_c, m, n, k, a, lda, b,
                               ldb, c, ldc, d, ldd, alpha, beta, stream);
}

int rocwmma_amd_gemv(uint32_t    m,
                     uint32_t    k,
                     uint32_t    ncols,
                     const void* a,
                     uint32_t    lda,
                     const void* x,
                     uint32_t    ldx,
                     float*      y,
                     uint32_t    ldy,
                     float       alpha,
                     float       beta,
                     void*       stream)
{
    if(!a || !x || !y || m == 0u || k == 0u)
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(ncols != 1u && ncols != 2u && ncols != 4u && ncols != 8u)
        return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
    if(k % 8u != 0u)
        return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
    if(lda < k || ldx < k || ldy < m)
        return ROCWMMA_AMD_BAD_LEADING_DIM;
    if(!aligned16(a) || !aligned16(x) || lda % 8u != 0u || ldx % 8u != 0u || (reinterpret_cast<uintptr_t>(y) & 3u))
        return ROCWMMA_AMD_BAD_ALIGNMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    return launchGemv(m, k, ncols, a, lda, x, ldx, y, ldy, alpha, beta, asStream(stream));
}

// The one-wave-per-sample kernels take these shapes; the tiled kernels of dlrm_general.hip take the others.
static bool dlrmSampleFitsAWave(uint32_t m, uint32_t k)
{
    return m <= 128u && (k == 32u || k == 64u || k == 128u || k == 256u);
}

static int checkDlrm(int dtype, uint32_t m, uint32_t k, uint32_t batch)
{
    if(m == 0u || k == 0u || batch == 0u)
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    // the tiled kernels read rows in 16-byte pieces and address a sample's features with 32-bit byte offsets
    const uint32_t size = dtype == ROCWMMA_AMD_F16 ? 2u : 4u;
    if(!dlrmSampleFitsAWave(m, k) && (m > 32768u || k % (16u / size) != 0u || static_cast<uint64_t>(m) * k * size >= (1ull << 31)))
        return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
    return ROCWMMA_AMD_OK;
}

int rocwmma_amd_dlrm_fwd(const void* input, void* output, uint32_t m, uint32_t k, uint32_t batch, void* stream)
{
    if(!input || !output)
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    int rc = checkDlrm(ROCWMMA_AMD_F16, m, k, batch);
    if(rc != ROCWMMA_AMD_OK)
        return rc;
    if(!aligned16(input) || !aligned16(output))
        return ROCWMMA_AMD_BAD_ALIGNMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    if(dlrmSampleFitsAWave(m, k))
    {
        rc = launchDlrmFwd(input, output, m, k, batch, asStream(stream));
        if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE) // (a sample larger than the LDS: tiles)
            return rc;
    }
    return launchDlrmFwdGeneral(ROCWMMA_AMD_F16, input, output, m, k, batch, asStream(stream));
}

int rocwmma_amd_dlrm_bwd(const void* input,
                         const void* upstream_grad,
                         void*       grad,
                         void*       bottom_mlp_grad,
                         uint32_t    m,
                         uint32_t    k,
                         uint32_t    batch,
                         void*       stream)
{
    if(!input || !upstream_grad || !grad || !bottom_mlp_grad)
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    int rc = checkDlrm(ROCWMMA_AMD_F16, m, k, batch);
    if(rc != ROCWMMA_AMD_OK)
        return rc;
    if(!aligned16(input) || !aligned16(upstream_grad) || !aligned16(grad) || !aligned16(bottom_mlp_grad))
        return ROCWMMA_AMD_BAD_ALIGNMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    if(dlrmSampleFitsAWave(m, k))
    {
        rc = launchDlrmBwd(input, upstream_grad, grad, bottom_mlp_grad, m, k, batch, asStream(stream));
        if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
            return rc;
    }
    return launchDlrmBwdGeneral(ROCWMMA_AMD_F16, input, upstream_grad, grad, bottom_mlp_grad, m, k, batch, asStream(stream));
}

int rocwmma_amd_dlrm_fwd_ex(int dtype, const void* input, void* output, uint32_t m, uint32_t k, uint32_t batch, void* stream)
{
    if(dtype == ROCWMMA_AMD_F16)
        return rocwmma_amd_dlrm_fwd(input, output, m, k, batch, stream);
    if(dtype != ROCWMMA_AMD_F32)
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    if(!input || !output)
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    int rc = checkDlrm(ROCWMMA_AMD_F32, m, k, batch);
    if(rc != ROCWMMA_AMD_OK)
        return rc;
    if(!aligned16(input) || !aligned16(output))
        return ROCWMMA_AMD_BAD_ALIGNMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    if(dlrmSampleFitsAWave(m, k))
        return launchDlrmFwdF32(input, output, m, k, batch, asStream(stream));
    return launchDlrmFwdGeneral(ROCWMMA_AMD_F32, input, output, m, k, batch, asStream(stream));
}

int rocwmma_amd_dlrm_bwd_ex(int         dtype,
                            const void* input,
                            const void* upstream_grad,
                            void*       grad,
                            void*       bottom_mlp_grad,
                            uint32_t    m,
                            uint32_t    k,
                            uint32_t    batch,
                            void*       stream)
{
    if(dtype == ROCWMMA_AMD_F16)
        return rocwmma_amd_dlrm_bwd(input, upstream_grad, grad, bottom_mlp_grad, m, k, batch, stream);
    if(dtype != ROCWMMA_AMD_F32)
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    if(!input || !upstream_grad || !grad || !bottom_mlp_grad)
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    int rc = checkDlrm(ROCWMMA_AMD_F32, m, k, batch);
    if(rc != ROCWMMA_AMD_OK)
        return rc;
    if(!aligned16(input) || !aligned16(upstream_grad) || !aligned16(grad) || !aligned16(bottom_mlp_grad))
        return ROCWMMA_AMD_BAD_ALIGNMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    if(dlrmSampleFitsAWave(m, k))
        return launchDlrmBwdF32(input, upstream_grad, grad, bottom_mlp_grad, m, k, batch, asStream(stream));
    return launchDlrmBwdGeneral(ROCWMMA_AMD_F32, input, upstream_grad, grad, bottom_mlp_grad, m, k, batch, asStream(stream));
}

} // extern "C"
