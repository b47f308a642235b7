// Drop-in check: the reference's three GEMM test kernels, the cooperative, LDS double-buffered
// multi-block one (reference: test/gemm/gemm_PGR1_LB2_MP0_MB_CP/device/kernel_device_func.hpp:70-283,
// with its mapping / scheduling / driver helpers test/gemm/gemm_{config,global_mapping,local_mapping,
// coop_schedule,driver}.hpp) and the two without LDS (test/gemm/gemm_PGR0_LB0_MP0_{MB,SB}_NC/device/
// kernel_device_func.hpp), are compiled unchanged against this repository's headers and run over
// a matrix of block sizes, element types, operand layouts, LDS layouts, cooperation levels,
// blocks per wave and thread-block shapes.
//
// This file is only the host side: it fills the operands with small integers, so that every
// partial sum is exact in every element type and accumulation order, launches the kernel the way
// the reference's harness does (test/gemm/gemm_PGR1_LB2_MP0_MB_CP/detail/kernel_impl.hpp:134-194:
// grid, block and LDS size), and compares D with a plain CPU loop bit for bit (compute types of 16
// bits: within the reference's 100 eps).
//
// The reference's kernel headers are found on the include path at build time; nothing of them is
// copied here.  The case list is split over several translation units (CASE_LIST names the list of
// one of them) to keep compile times short.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <iostream>
#include <type_traits>
#include <vector>

#include <rocwmma/rocwmma.hpp>
#include <rocwmma/rocwmma_coop.hpp>
#include <rocwmma/rocwmma_transforms.hpp>

// The reference's three kernel headers share their include guards, so a translation unit holds one
// of them: GEMM_KERNEL = 0 cooperative, 1 multi-block without LDS, 2 single-block without LDS.
#ifndef GEMM_KERNEL
#define GEMM_KERNEL 0
#endif
#if GEMM_KERNEL == 0
#include "gemm_PGR1_LB2_MP0_MB_CP/device/kernel_device_func.hpp"
#elif GEMM_KERNEL == 1
#include "gemm_PGR0_LB0_MP0_MB_NC/device/kernel_device_func.hpp"
#else
#include "gemm_PGR0_LB0_MP0_SB_NC/device/kernel_device_func.hpp"
#endif

#ifndef CASE_LIST
#error "compile with -DCASE_LIST=\"file\" naming the list of CASE(...) lines (see tests/dropin/build_samples.py)"
#endif

namespace
{
    using namespace rocwmma;

    constexpr uint32_t kArch = 0x942; // the newest architecture id the reference's guards know

    int gPassed = 0, gFailed = 0, gSkipped = 0;

    template <typename T>
    T fromInt(int v)
    {
        return static_cast<T>(static_cast<float>(v));
    }
    template <>
    int8_t fromInt<int8_t>(int v)
    {
        return static_cast<int8_t>(v);
    }
    template <>
    int32_t fromInt<int32_t>(int v)
    {
        return v;
    }

    template <typename T>
    double toDouble(T const& v)
    {
        return static_cast<double>(static_cast<float>(v));
    }
    template <>
    double toDouble<int32_t>(int32_t const& v)
    {
        return v;
    }

    template <typename Layout>
    size_t at(uint32_t row, uint32_t col, uint32_t ld)
    {
        return std::is_same<Layout, row_major>::value ? static_cast<size_t>(row) * ld + col
                                                      : static_cast<size_t>(col) * ld + row;
    }
    template <typename Layout>
    uint32_t naturalLd(uint32_t rows, uint32_t cols)
    {
        return std::is_same<Layout, row_major>::value ? cols : rows;
    }

#define HIP_OK(expr)                                                                     \
    do                                                                                   \
    {                                                                                    \
        hipError_t e_ = (expr);                                                          \
        if(e_ != hipSuccess)                                                             \
        {                                                                                \
            std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            std::exit(2);                                                                \
        }                                                                                \
    } while(0)

    // Fills, launches, checks.  The three kernels share the argument list and the grid rule; they
    // differ in the macro tile a workgroup covers and in their LDS need.
    template <typename InputT, typename OutputT, typename ComputeT, typename LayoutA, typename LayoutB, typename LayoutC>
    void runGemm(const char* name,
                 void (*kernel)(uint32_t, uint32_t, uint32_t, InputT const*, InputT const*, OutputT const*, OutputT*,
                                uint32_t, uint32_t, uint32_t, uint32_t, ComputeT, ComputeT),
                 uint32_t macroM,
                 uint32_t macroN,
                 uint32_t blockK,
                 uint32_t ldsBytes,
                 uint32_t tx,
                 uint32_t ty,
                 bool     enabled)
    {
        if(!enabled)
        {
            std::printf("SKIPPED %s (disabled by the kernel's own guard)\n", name);
            ++gSkipped;
            return;
        }
        const uint32_t m = 2u * macroM, n = 3u * macroN, k = 5u * blockK;
        const uint32_t lda = naturalLd<LayoutA>(m, k), ldb = naturalLd<LayoutB>(k, n);
        const uint32_t ldc = naturalLd<LayoutC>(m, n), ldd = ldc;
        const int      alpha = 2, beta = 3;

        std::vector<InputT>  a(static_cast<size_t>(m) * k), b(static_cast<size_t>(k) * n);
        std::vector<OutputT> c(static_cast<size_t>(m) * n), d(static_cast<size_t>(m) * n), want(c.size());
        std::vector<int>     ai(a.size()), bi(b.size()), ci(c.size());
        for(uint32_t i = 0; i < m; ++i)
            for(uint32_t h = 0; h < k; ++h)
            {
                const int v               = static_cast<int>((i * 7u + h * 3u + (i * h) % 5u) % 5u) - 2;
                ai[at<LayoutA>(i, h, lda)] = v;
                a[at<LayoutA>(i, h, lda)]  = fromInt<InputT>(v);
            }
        for(uint32_t h = 0; h < k; ++h)
            for(uint32_t j = 0; j < n; ++j)
            {
                const int v               = static_cast<int>((h * 5u + j * 11u + (h * j) % 3u) % 5u) - 2;
                bi[at<LayoutB>(h, j, ldb)] = v;
                b[at<LayoutB>(h, j, ldb)]  = fromInt<InputT>(v);
            }
        for(uint32_t i = 0; i < m; ++i)
            for(uint32_t j = 0; j < n; ++j)
            {
                const int v               = static_cast<int>((i * 13u + j * 17u) % 7u) - 3;
                ci[at<LayoutC>(i, j, ldc)] = v;
                c[at<LayoutC>(i, j, ldc)]  = fromInt<OutputT>(v);
            }
        for(uint32_t i = 0; i < m; ++i)
            for(uint32_t j = 0; j < n; ++j)
            {
                int acc = 0;
                for(uint32_t h = 0; h < k; ++h)
                    acc += ai[at<LayoutA>(i, h, lda)] * bi[at<LayoutB>(h, j, ldb)];
                want[at<LayoutC>(i, j, ldd)] = fromInt<OutputT>(alpha * acc + beta * ci[at<LayoutC>(i, j, ldc)]);
            }

        InputT * dA, *dB;
        OutputT *dC, *dD;
        HIP_OK(hipMalloc(&dA, a.size() * sizeof(InputT)));
        HIP_OK(hipMalloc(&dB, b.size() * sizeof(InputT)));
        HIP_OK(hipMalloc(&dC, c.size() * sizeof(OutputT)));
        HIP_OK(hipMalloc(&dD, d.size() * sizeof(OutputT)));
        HIP_OK(hipMemcpy(dA, a.data(), a.size() * sizeof(InputT), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dB, b.data(), b.size() * sizeof(InputT), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dC, c.data(), c.size() * sizeof(OutputT), hipMemcpyHostToDevice));
        HIP_OK(hipMemset(dD, 0x7f, d.size() * sizeof(OutputT))); // a value no case produces

        const dim3 grid((m + macroM - 1u) / macroM, (n + macroN - 1u) / macroN), block(tx, ty);
        hipLaunchKernelGGL(kernel, grid, block, ldsBytes, 0, m, n, k, dA, dB, dC, dD, lda, ldb, ldc, ldd,
                           static_cast<ComputeT>(alpha), static_cast<ComputeT>(beta));
        HIP_OK(hipGetLastError());
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(d.data(), dD, d.size() * sizeof(OutputT), hipMemcpyDeviceToHost));
        HIP_OK(hipFree(dA));
        HIP_OK(hipFree(dB));
        HIP_OK(hipFree(dC));
        HIP_OK(hipFree(dD));

        // 32-bit compute types: bit for bit.  Narrower compute types are widened and narrowed again
        // around every matrix instruction, so a partial sum beyond the exact-integer range of the
        // type rounds: the reference's bound for them, 100 eps in max |a-b| / (|a|+|b|+1)
        // (test/gemm/gemm_kernel_base_impl.hpp:915-927).
        const double tolerance = sizeof(ComputeT) < 4u ? 100.0 * std::ldexp(1.0, std::is_same<ComputeT, bfloat16_t>::value ? -7 : -10)
                                                       : 0.0;
        size_t bad = 0, firstBad = 0;
        for(size_t e = 0; e < d.size(); ++e)
            if(!(std::fabs(toDouble(d[e]) - toDouble(want[e]))
                 <= tolerance * (std::fabs(toDouble(d[e])) + std::fabs(toDouble(want[e])) + 1.0)))
            {
                if(bad == 0)
                    firstBad = e;
                ++bad;
            }
        if(bad == 0)
        {
            std::printf("PASSED %s (%ux%ux%u)\n", name, m, n, k);
            ++gPassed;
        }
        else
        {
            std::printf("FAILED %s (%ux%ux%u): %zu of %zu elements differ, first at %zu: got %g want %g\n", name, m,
                        n, k, bad, d.size(), firstBad, toDouble(d[firstBad]), toDouble(want[firstBad]));
            ++gFailed;
        }
        std::fflush(stdout);
    }

#if GEMM_KERNEL == 0
    namespace Block = CooperativeGemm::BlockLevel;
    namespace Wave  = CooperativeGemm::WaveLevel;
    namespace Wg    = CooperativeGemm::WorkgroupLevel;
#endif
    using R         = row_major;
    using C         = col_major;
    using f16       = float16_t;
    using bf16      = bfloat16_t;
    using h16       = hfloat16_t;
    using f32       = float32_t;
    using f64       = float64_t;
    using f8        = float8_t;
    using bf8       = bfloat8_t;
    using i8        = int8_t;
    using i32       = int32_t;

// The guards' enableBuild() also asks whether the *current compilation pass* targets that
// architecture, which the host pass never does; enableRun() is what the reference's harness asks.
// Grid, block and LDS size as in the reference's harness (test/gemm/gemm_PGR1_LB2_MP0_MB_CP/detail/
// kernel_impl.hpp:134-194 and its two siblings).

// cooperative, LDS double-buffered, multi-block
#define CASE(BM, BN, BK, IN, OUT, COMP, LA, LB, LC, LLDS, CFG, BX, BY, TX, TY)                                        \
    runGemm<IN, OUT, COMP, LA, LB, LC>(                                                                               \
        "coop " #BM "x" #BN "x" #BK " " #IN "->" #OUT " A:" #LA " B:" #LB " C:" #LC " lds:" #LLDS " " #CFG " " #BX    \
        "x" #BY " tb(" #TX "," #TY ")",                                                                               \
        gemm_PGR1_LB2_MP0_MB_CP<BM, BN, BK, IN, OUT, COMP, LA, LB, LC, LC, LLDS, CFG, BX, BY, TX, TY, 64u, kArch>,    \
        BM * BX * (TX / 64u), BN * BY * TY, BK,                                                                      \
        2u * sizeof(IN) * (BM * BX * (TX / 64u) + BN * BY * TY) * BK, TX, TY,                                        \
        gemm_PGR1_LB2_MP0_MB_CP_guard<BM, BN, BK, IN, OUT, COMP, LA, LB, LC, LC, LLDS, CFG, BX, BY, TX, TY, 64u,      \
                                      kArch>::enableRun())

// no LDS, BX x BY blocks per wave
#define CASE_MB(BM, BN, BK, IN, OUT, COMP, LA, LB, LC, BX, BY, TX, TY)                                            \
    runGemm<IN, OUT, COMP, LA, LB, LC>(                                                                           \
        "multi-block " #BM "x" #BN "x" #BK " " #IN "->" #OUT " A:" #LA " B:" #LB " C:" #LC " " #BX "x" #BY        \
        " tb(" #TX "," #TY ")",                                                                                   \
        gemm_PGR0_LB0_MP0_MB_NC<BM, BN, BK, IN, OUT, COMP, LA, LB, LC, LC, BX, BY, TX, TY, 64u, kArch>,           \
        BM * BX * (TX / 64u), BN * BY * TY, BK, 0u, TX, TY,                                                       \
        gemm_PGR0_LB0_MP0_MB_NC_guard<BM, BN, BK, IN, OUT, COMP, BX, BY, TX, TY, 64u, kArch>::enableRun())

// no LDS, one block per wave
#define CASE_SB(BM, BN, BK, IN, OUT, COMP, LA, LB, LC, TX, TY)                                             \
    runGemm<IN, OUT, COMP, LA, LB, LC>(                                                                    \
        "single-block " #BM "x" #BN "x" #BK " " #IN "->" #OUT " A:" #LA " B:" #LB " C:" #LC " tb(" #TX     \
        "," #TY ")",                                                                                       \
        gemm_PGR0_LB0_MP0_SB_NC<BM, BN, BK, IN, OUT, COMP, LA, LB, LC, LC, TX, TY, 64u, kArch>,            \
        BM * (TX / 64u), BN * TY, BK, 0u, TX, TY,                                                          \
        gemm_PGR0_LB0_MP0_SB_NC_guard<BM, BN, BK, IN, OUT, COMP, TX, TY, 64u, kArch>::enableRun())
} // namespace

int main()
{
    // the list of CASE(...) lines of this translation unit, written by tests/dropin/build_samples.py
#include CASE_LIST
    std::printf("SUMMARY: %d passed, %d failed, %d skipped\n", gPassed, gFailed, gSkipped);
    return gFailed == 0 ? 0 : 1;
}
