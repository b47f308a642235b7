// Drop-in check: the device kernels of the reference's unit tests that use only the public API
// (reference tree, test/unit/*/device/*.hpp: load / store, cooperative load / store, fill,
// load and store contamination, MappingUtil coordinate maps and their overrides) are compiled
// unchanged against this repository's headers and run.
//
// This file is only the host side.  All those kernels share one signature
// (m, n, in, out, ld, param1, param2) and one launch rule: thread block (TBlockX, TBlockY), every
// wave owns one BlockM x BlockN block, grid = (m / (BlockM * TBlockX / 64), n / (BlockN * TBlockY))
// (reference: test/unit/unit_kernel_base_impl.hpp:64-80).  What each kind must produce:
//
//   IDENT   out == in                                   (load/store, coop load/store, map kernels)
//   FILL    out == param1 everywhere
//   LOADC   `in` is the matrix inside a frame of param1 rows / param2 columns of a marker value;
//           out == the inner matrix, no marker          (contamination_test/detail/load_contamination.hpp)
//   STOREC  `out` has such a frame; inner part == in, frame still all marker
//   OVR_*   the block row / column (or element row / column) every wave reads from is overridden
//           by param1; out block (i, j) == in block (param1, j) and so on
//
// The case list (CASE_LIST names the file) is written by tests/dropin/build_samples.py.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <iostream>
#include <type_traits>
#include <vector>

#include <rocwmma/rocwmma.hpp>
#include <rocwmma/rocwmma_coop.hpp>

#include "contamination_test/device/load_contamination.hpp"
#include "contamination_test/device/store_contamination.hpp"
#include "fill_fragment_test/device/fill_fragment.hpp"
#include "load_store_matrix_coop_sync_test/device/load_store_matrix_coop_sync.hpp"
#include "load_store_matrix_sync_test/device/load_store_matrix_sync.hpp"
#include "map_util_test/device/map_block_to_matrix.hpp"
#include "map_util_test/device/map_block_to_matrix_override.hpp"
#include "map_util_test/device/map_matrix_to_data.hpp"
#include "map_util_test/device/map_matrix_to_data_override.hpp"
#include "map_util_test/device/map_thread_to_matrix.hpp"
#include "map_util_test/device/map_wave_to_matrix.hpp"

#ifndef CASE_LIST
#error "compile with -DCASE_LIST=\"file\" naming the list of UNIT(...) lines (see tests/dropin/build_samples.py)"
#endif

namespace
{
    using namespace rocwmma;

    constexpr uint32_t kArch = 0x942; // the newest architecture id the reference's guards know

    int gPassed = 0, gFailed = 0, gSkipped = 0;

    enum Kind
    {
        IDENT,
        FILL,
        LOADC,
        STOREC,
        OVR_BLOCK_M,
        OVR_BLOCK_N,
        OVR_ELEM_M,
        OVR_ELEM_N
    };

    template <typename T>
    T fromInt(int v)
    {
        if constexpr(std::is_integral<T>::value)
            return static_cast<T>(v);
        else
            return static_cast<T>(static_cast<float>(v));
    }
    template <typename T>
    double toDouble(T const& v)
    {
        if constexpr(std::is_integral<T>::value || std::is_same<T, double>::value)
            return static_cast<double>(v);
        else
            return static_cast<double>(static_cast<float>(v));
    }

#define HIP_OK(expr)                                                                         \
    do                                                                                       \
    {                                                                                        \
        hipError_t e_ = (expr);                                                              \
        if(e_ != hipSuccess)                                                                 \
        {                                                                                    \
            std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            std::exit(2);                                                                    \
        }                                                                                    \
    } while(0)

    constexpr int kMarker = 7; // the pattern below stays within -6 .. 6

    int pattern(uint32_t row, uint32_t col)
    {
        return static_cast<int>((row * 31u + col * 7u + (row * col) % 11u) % 13u) - 6;
    }

    template <typename T, typename Layout>
    void runUnit(Kind        kind,
                 const char* name,
                 void (*kernel)(uint32_t, uint32_t, T const*, T*, uint32_t, T, T),
                 uint32_t blockM,
                 uint32_t blockN,
                 uint32_t tx,
                 uint32_t ty,
                 int      p1,
                 int      p2,
                 bool     enabled)
    {
        if(!enabled)
        {
            std::printf("SKIPPED %s (disabled by the kernel's own guard)\n", name);
            ++gSkipped;
            return;
        }
        constexpr bool rowMajor = std::is_same<Layout, row_major>::value;
        const uint32_t tileM = blockM * (tx / 64u), tileN = blockN * ty;
        const uint32_t m = 2u * tileM, n = 2u * tileN;
        const uint32_t ld = rowMajor ? n : m;
        // frames: rows above / below = fr, columns left / right = fc
        const uint32_t inFr = kind == LOADC ? p1 : 0u, inFc = kind == LOADC ? p2 : 0u;
        const uint32_t outFr = kind == STOREC ? p1 : 0u, outFc = kind == STOREC ? p2 : 0u;
        auto index = [&](uint32_t r, uint32_t c, uint32_t fr, uint32_t fc) {
            const uint32_t rows = m + 2u * fr, cols = n + 2u * fc;
            return rowMajor ? static_cast<size_t>(r) * cols + c : static_cast<size_t>(c) * rows + r;
        };
        std::vector<T> in(static_cast<size_t>(m + 2u * inFr) * (n + 2u * inFc), fromInt<T>(kMarker));
        std::vector<T> out(static_cast<size_t>(m + 2u * outFr) * (n + 2u * outFc), fromInt<T>(kMarker));
        for(uint32_t r = 0; r < m; ++r)
            for(uint32_t c = 0; c < n; ++c)
                in[index(r + inFr, c + inFc, inFr, inFc)] = fromInt<T>(pattern(r, c));

        T *dIn, *dOut;
        HIP_OK(hipMalloc(&dIn, in.size() * sizeof(T)));
        HIP_OK(hipMalloc(&dOut, out.size() * sizeof(T)));
        HIP_OK(hipMemcpy(dIn, in.data(), in.size() * sizeof(T), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dOut, out.data(), out.size() * sizeof(T), hipMemcpyHostToDevice));
        hipLaunchKernelGGL(kernel, dim3(m / tileM, n / tileN), dim3(tx, ty), 0, 0, m, n, dIn, dOut, ld,
                           fromInt<T>(p1), fromInt<T>(p2));
        HIP_OK(hipGetLastError());
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(out.data(), dOut, out.size() * sizeof(T), hipMemcpyDeviceToHost));
        HIP_OK(hipFree(dIn));
        HIP_OK(hipFree(dOut));

        size_t bad = 0;
        double got0 = 0, want0 = 0;
        auto   expect = [&](size_t at, double want) {
            if(!(toDouble(out[at]) == want))
            {
                if(bad == 0)
                {
                    got0  = toDouble(out[at]);
                    want0 = want;
                }
                ++bad;
            }
        };
        for(uint32_t r = 0; r < m + 2u * outFr; ++r)
            for(uint32_t c = 0; c < n + 2u * outFc; ++c)
            {
                const size_t at    = index(r, c, outFr, outFc);
                const bool   frame = r < outFr || r >= m + outFr || c < outFc || c >= n + outFc;
                if(frame)
                {
                    expect(at, kMarker);
                    continue;
                }
                uint32_t sr = r - outFr, sc = c - outFc;
                switch(kind)
                {
                case FILL:
                    expect(at, p1);
                    continue;
                case OVR_BLOCK_M:
                    sr = p1 * blockM + sr % blockM;
                    break;
                case OVR_BLOCK_N:
                    sc = p1 * blockN + sc % blockN;
                    break;
                case OVR_ELEM_M:
                    sr = p1 + sr % blockM;
                    break;
                case OVR_ELEM_N:
                    sc = p1 + sc % blockN;
                    break;
                default:
                    break;
                }
                expect(at, pattern(sr, sc));
            }
        if(bad == 0)
        {
            std::printf("PASSED %s (%ux%u)\n", name, m, n);
            ++gPassed;
        }
        else
        {
            std::printf("FAILED %s (%ux%u): %zu elements differ, first: got %g want %g\n", name, m, n, bad, got0,
                        want0);
            ++gFailed;
        }
        std::fflush(stdout);
    }

    using R    = row_major;
    using C    = col_major;
    using f16  = float16_t;
    using bf16 = bfloat16_t;
    using h16  = hfloat16_t;
    using f32  = float32_t;
    using f64  = float64_t;
    using f8   = float8_t;
    using bf8  = bfloat8_t;
    using i8   = int8_t;
    using i32  = int32_t;

#define UNIT(KIND, KERNEL, BM, BN, T, L, TX, TY, P1, P2)                                                        \
    runUnit<T, L>(KIND, #KERNEL "<" #BM "," #BN "," #T "," #L "> tb(" #TX "," #TY ") params(" #P1 "," #P2 ")", \
                  KERNEL<BM, BN, T, L>, BM, BN, TX, TY, P1, P2, FragSize_guard<BM, BN, T, L, 64u, kArch>::enable())
} // namespace

int main()
{
#include CASE_LIST
    std::printf("SUMMARY: %d passed, %d failed, %d skipped\n", gPassed, gFailed, gSkipped);
    return gFailed == 0 ? 0 : 1;
}
