// Host-side helpers shared by the workload translation units of librocwmma_amd.so.
#ifndef ROCWMMA_AMD_CSRC_COMMON_HPP
#define ROCWMMA_AMD_CSRC_COMMON_HPP

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <hip/hip_runtime.h>

#include <rocwmma/rocwmma.hpp>
#include <rocwmma_amd.h>

static_assert(ROCWMMA_AMD_GFX950_NATIVE == 1,
              "the toolchain's own rocWMMA headers were picked up: put -I<repo>/include first");

namespace rocwmma_amd
{
    inline hipStream_t asStream(void* stream)
    {
        return reinterpret_cast<hipStream_t>(stream);
    }

    inline bool aligned16(const void* p)
    {
        return (reinterpret_cast<uintptr_t>(p) & 15u) == 0u;
    }

    inline uint32_t dtypeSize(int dtype)
    {
        switch(dtype)
        {
        case ROCWMMA_AMD_F16:
        case ROCWMMA_AMD_BF16:
            return 2;
        case ROCWMMA_AMD_E4M3:
        case ROCWMMA_AMD_E5M2:
        case ROCWMMA_AMD_I8:
            return 1;
        case ROCWMMA_AMD_F32:
        case ROCWMMA_AMD_I32:
            return 4;
        default:
            return 0;
        }
    }

    // Compute units of the current device (immutable per device, so remembered per ordinal).
    inline uint32_t computeUnits()
    {
        constexpr int             kMaxDevices = 64;
        static std::atomic<int>   known[kMaxDevices];
        int                       dev = 0;
        if(hipGetDevice(&dev) != hipSuccess)
            return 256u;
        if(dev >= 0 && dev < kMaxDevices && known[dev].load(std::memory_order_relaxed) > 0)
            return static_cast<uint32_t>(known[dev].load(std::memory_order_relaxed));
        int cus = 0;
        if(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            return 256u;
        if(dev >= 0 && dev < kMaxDevices)
            known[dev].store(cus, std::memory_order_relaxed);
        return static_cast<uint32_t>(cus);
    }

    inline int launchStatus()
    {
        return hipGetLastError() == hipSuccess ? ROCWMMA_AMD_OK : ROCWMMA_AMD_LAUNCH_FAILED;
    }

    // Argument block every GEMM kernel family takes: the reference kernels' argument list
    // (m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta) plus the run-time C/D layout.
    struct GemmArgs
    {
        uint32_t    m, n, k;
        const void* a;
        const void* b;
        const void* c;
        void*       d;
        uint32_t    lda, ldb, ldc, ldd;
        float       alpha, beta;
        int         layoutC;
        // fused epilogue (rocwmma_amd_gemm_bias_act): D = act(alpha * A * B + beta * C + bias[column])
        const float* bias       = nullptr; // one value per column of D, or nullptr
        int          activation = ROCWMMA_AMD_ACT_NONE;
    };

    ROCWMMA_DEVICE ROCWMMA_INLINE float applyActivation(float v, int activation)
    {
        if(activation == ROCWMMA_AMD_ACT_RELU)
            return v < 0.0f ? 0.0f : v; // (a NaN stays a NaN, as with a maximum that propagates NaNs)
        if(activation == ROCWMMA_AMD_ACT_GELU)
        {
            // x * Phi(x) with Phi(x) = erfc(-x / sqrt 2) / 2 and, for z >= 0, erfc(z) = (a1 t + ... + a5 t^5)
            // exp(-z^2), t = 1 / (1 + p z) (Abramowitz & Stegun 7.1.26, absolute error below 1.5e-7): one
            // reciprocal, one exponential and a dozen multiply-adds, a third of the library erff.
            const float z    = fabsf(v) * 0.70710678118654752f;
            const float t    = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * z);
            const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
            const float half = 0.5f * poly * __builtin_amdgcn_exp2f(-1.4426950408889634f * z * z);
            return v * (v >= 0.0f ? 1.0f - half : half);
        }
        return v;
    }

    // Block scales of a microscaled GEMM: one E8M0 byte per 32 elements along K of every row of A
    // (a: m x k/32, leading dimension lda) and every column of B (b: n x k/32, leading dimension ldb).
    struct MxScales
    {
        const uint8_t* a;
        const uint8_t* b;
        uint32_t       lda, ldb;
    };

    // Family launchers (one translation unit each).  Return a rocwmma_amd_status;
    // ROCWMMA_AMD_UNSUPPORTED_SHAPE / _TYPE mean "this family has no kernel for it".
    int launchGemmWaveTile(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& args, hipStream_t stream);
    // forceLargeTile: the 256 x 256 tile or nothing (ROCWMMA_AMD_GEMM_BLOCKED_256)
    int launchGemmBlocked(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& args, hipStream_t stream,
                          bool forceLargeTile = false);
    int launchGemmSkinny(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& args, hipStream_t stream);
    // Stream-K: the 256 x 256 tiling with the tile count balanced over persistent workgroups.  The
    // workspace holds one slot of raw accumulators per workgroup plus flags (streamKWorkspaceBytes).
    constexpr uint32_t kStreamKSlotBytes = 256u * 256u * 4u;
    size_t streamKWorkspaceBytes(uint32_t workgroups);
    int    launchGemmStreamK(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& args, void* workspace,
                             size_t workspaceBytes, hipStream_t stream);
    // Whether an owner's bounded wait ran out in a launch on this workspace (nullptr: the library's own scratch) since
    // the last query; waits for `stream` first.
    int    streamKTimedOut(void* workspace, size_t workspaceBytes, hipStream_t stream, int* timedOut);
    // the same on the library's own scratch (a static device array): allocates nothing
    int    launchGemmStreamKStatic(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& args, hipStream_t stream);

    // Scales of the blocked block-scaled kernel, re-ordered into the order its lanes load them in:
    // per operand, groups of 64 rows of A (columns of B) x pairs of 128-byte K stages x 64 lanes x 4
    // blocks of 16 rows x 2 stages, one byte each -- 8 contiguous bytes per lane, group and stage pair.
    // A's part comes first; B's starts at the next multiple of 256 bytes.
    inline size_t mxPackedScaleBytesOf(uint32_t rows, uint32_t k)
    {
        return static_cast<size_t>((rows + 63u) / 64u) * ((k + 255u) / 256u) * 64u * 8u;
    }
    inline size_t mxPackedScaleOffsetB(uint32_t m, uint32_t k)
    {
        return (mxPackedScaleBytesOf(m, k) + 255u) & ~static_cast<size_t>(255u);
    }
    inline size_t mxPackedScaleBytes(uint32_t m, uint32_t n, uint32_t k)
    {
        return mxPackedScaleOffsetB(m, k) + mxPackedScaleBytesOf(n, k);
    }
    // Re-orders both operands' scales (one launch).  wide32: for the tiles of 32-wide blocks (lane l = row
    // l % 32 of a block and K block l / 32 of a 64-byte step; 8 bytes per lane = [block 0..1][step 0..3])
    // instead of 16-wide ones (lane l = row l % 16, K block l / 16 of a 128-byte stage; [block 0..3][stage 0..1]).
    int launchMxPackScales(MxScales const& scales, uint32_t m, uint32_t n, uint32_t k, void* packedA, void* packedB, bool wide32,
                           hipStream_t stream);
    // The blocked kernel on packed scales: row-major A, col-major B, row-major C/D, m and n multiples of 16,
    // k a multiple of 128.  256 x 256 tiles of 16-wide blocks when gemmMxBlockedUsesLargeTile(), else 128 x 128
    // tiles of 32-wide blocks: the scales must have been packed for that.
    bool gemmMxBlockedUsesLargeTile(GemmArgs const& args);
    // True when launchGemmBlocked runs a problem with K-contiguous operands (A row-major, B col-major) of
    // `elemBytes`-byte elements on partly filled 128 x 64 tiles over the ring of four 128-byte stages:
    // one round of workgroups with enough K to stream.  (The weight-streaming kernels leave those to it.)
    bool gemmBlockedTakesPartlyFilledLineTiles(uint32_t m, uint32_t n, uint32_t k, uint32_t elemBytes);
    int  launchGemmMxBlocked(int dtypeIn, GemmArgs const& args, const void* packedA, const void* packedB, hipStream_t stream);

    // The blocked kernel with the fused epilogue (float types, row-major C/D; args.bias / args.activation)
    int launchGemmBlockedFused(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& args, hipStream_t stream);

    // Block-scaled weight streaming: up to 32 token rows, row-major A, col-major B, row-major C/D
    int launchGemmMxSkinny(int dtypeIn, int layoutA, int layoutB, GemmArgs const& args, MxScales const& scales, hipStream_t stream);
    // Block-scaled fp8 / bf8 GEMM (f32 C/D): one block per wave, every layout pair
    int launchGemmMxWaveTile(int dtypeIn, int layoutA, int layoutB, GemmArgs const& args, MxScales const& scales, hipStream_t stream);

} // namespace rocwmma_amd

#endif // ROCWMMA_AMD_CSRC_COMMON_HPP
