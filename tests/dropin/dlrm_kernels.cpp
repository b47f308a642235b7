// Drop-in check: the device kernels of the reference's DLRM dot-interaction tests (reference tree,
// test/dlrm/device/dlrm_dot_fwd.hpp, dlrm_dot_bwd.hpp and their LDS variants dlrm_dot_fwd_lds.hpp,
// dlrm_dot_bwd_lds.hpp with test/dlrm/lds_mapping_util.hpp) are compiled unchanged against this
// repository's headers and run.
//
// This file is only the host side.  Launch geometry as the reference's test base uses it
// (test/dlrm/dlrm_kernel_base_impl.hpp:78-99, 300-395): thread block (128, 1); forward grid
// (m / (2 * Tile), m / Tile, b); backward: the triangle is first unpacked into a symmetric m x m
// matrix per sample by trilReconstruct, grid (m * m / 128, 1, b), then the gradient kernel runs on
// grid (m / (2 * Tile), k / Tile, b).  The LDS variants get
// 2 * sizeof(DataT) * (2 + 1) * Tile * Tile bytes of dynamic LDS (test/dlrm/detail/dlrm_dot_lds.hpp:48-54:
// two buffers, each the register files of two waves' A blocks and one B block).
//
// Inputs are -1, 0, 1 so that every sum is an integer below 2048 and the f16 results are exact:
// the outputs are compared for equality with plain CPU loops.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <initializer_list>
#include <vector>

#include <rocwmma/rocwmma.hpp>
#include <rocwmma/rocwmma_coop.hpp>

#include "device/dlrm_dot_bwd.hpp"
#include "device/dlrm_dot_bwd_lds.hpp"
#include "device/dlrm_dot_fwd.hpp"
#include "device/dlrm_dot_fwd_lds.hpp"

namespace
{
    using namespace rocwmma;

    int gPassed = 0, gFailed = 0;

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

    int pattern(uint32_t seed, size_t i)
    {
        uint32_t x = static_cast<uint32_t>(i) * 2654435761u + seed * 40503u;
        x ^= x >> 15;
        x *= 2246822519u;
        x ^= x >> 13;
        return static_cast<int>(x % 3u) - 1;
    }

    template <typename T>
    struct DeviceBuffer
    {
        T*     ptr = nullptr;
        size_t count;
        explicit DeviceBuffer(size_t n)
            : count(n)
        {
            HIP_OK(hipMalloc(&ptr, n * sizeof(T)));
            HIP_OK(hipMemset(ptr, 0xff, n * sizeof(T))); // NaN for f16 / f32: unwritten output shows
        }
        ~DeviceBuffer()
        {
            (void)hipFree(ptr);
        }
        void upload(std::vector<T> const& h)
        {
            HIP_OK(hipMemcpy(ptr, h.data(), count * sizeof(T), hipMemcpyHostToDevice));
        }
        std::vector<T> download() const
        {
            std::vector<T> h(count);
            HIP_OK(hipMemcpy(h.data(), ptr, count * sizeof(T), hipMemcpyDeviceToHost));
            return h;
        }
    };

    template <typename T>
    size_t countDifferent(std::vector<T> const& got, std::vector<float> const& want, float* got0, float* want0)
    {
        size_t bad = 0;
        for(size_t i = 0; i < want.size(); ++i)
        {
            const float g = static_cast<float>(got[i]);
            if(!(g == want[i]))
            {
                if(bad == 0)
                {
                    *got0  = g;
                    *want0 = want[i];
                }
                ++bad;
            }
        }
        return bad;
    }

    void report(const char* what, const char* type, uint32_t tile, bool lds, uint32_t m, uint32_t k, uint32_t b,
                size_t bad, float got0, float want0)
    {
        if(bad == 0)
        {
            std::printf("PASSED %s<%s, %u>%s m=%u k=%u b=%u\n", what, type, tile, lds ? " (LDS)" : "", m, k, b);
            ++gPassed;
        }
        else
        {
            std::printf("FAILED %s<%s, %u>%s m=%u k=%u b=%u: %zu elements differ, first: got %g want %g\n", what,
                        type, tile, lds ? " (LDS)" : "", m, k, b, bad, got0, want0);
            ++gFailed;
        }
        std::fflush(stdout);
    }

    template <typename DataT, uint32_t Tile>
    void runForward(const char* type, uint32_t m, uint32_t k, uint32_t b)
    {
        const uint32_t inStride = m * k, outStride = m * (m - 1u) / 2u + k, accStride = m * m;
        std::vector<DataT> in(static_cast<size_t>(b) * inStride);
        for(size_t i = 0; i < in.size(); ++i)
            in[i] = static_cast<DataT>(static_cast<float>(pattern(1u, i)));

        std::vector<float> want(static_cast<size_t>(b) * outStride);
        for(uint32_t s = 0; s < b; ++s)
        {
            const DataT* f = in.data() + static_cast<size_t>(s) * inStride;
            float*       o = want.data() + static_cast<size_t>(s) * outStride;
            for(uint32_t h = 0; h < k; ++h)
                o[h] = static_cast<float>(f[h]);
            size_t at = k;
            for(uint32_t i = 1; i < m; ++i)
                for(uint32_t j = 0; j < i; ++j)
                {
                    float sum = 0.f;
                    for(uint32_t h = 0; h < k; ++h)
                        sum += static_cast<float>(f[i * k + h]) * static_cast<float>(f[j * k + h]);
                    o[at++] = sum;
                }
        }

        const dim3     grid((m + 2u * Tile - 1u) / (2u * Tile), (m + Tile - 1u) / Tile, b), block(128, 1);
        const uint32_t ldsBytes = 2u * sizeof(DataT) * 3u * Tile * Tile;
        for(bool lds : {false, true})
        {
            DeviceBuffer<DataT> dIn(in.size()), dOut(want.size());
            DeviceBuffer<float> dAcc(static_cast<size_t>(b) * accStride);
            dIn.upload(in);
            if(lds)
                hipLaunchKernelGGL((dlrmDotFwdLds<DataT, Tile, LdsRF>), grid, block, ldsBytes, 0,
                                   dIn.ptr, dOut.ptr, dAcc.ptr, m, k, b, inStride, outStride, accStride);
            else
                hipLaunchKernelGGL((dlrmDotFwd<DataT, Tile>), grid, block, 0, 0, dIn.ptr, dOut.ptr, dAcc.ptr, m, k,
                                   b, inStride, outStride, accStride);
            HIP_OK(hipGetLastError());
            HIP_OK(hipDeviceSynchronize());

            float        got0 = 0, want0 = 0;
            const size_t bad = countDifferent(dOut.download(), want, &got0, &want0);
            report("dlrmDotFwd", type, Tile, lds, m, k, b, bad, got0, want0);
        }
    }

    template <typename DataT, uint32_t Tile>
    void runBackward(const char* type, uint32_t m, uint32_t k, uint32_t b)
    {
        const uint32_t inStride = m * k, upStride = m * (m - 1u) / 2u + k, accStride = m * m;
        std::vector<DataT> in(static_cast<size_t>(b) * inStride), up(static_cast<size_t>(b) * upStride);
        for(size_t i = 0; i < in.size(); ++i)
            in[i] = static_cast<DataT>(static_cast<float>(pattern(2u, i)));
        for(size_t i = 0; i < up.size(); ++i)
            up[i] = static_cast<DataT>(static_cast<float>(pattern(3u, i)));

        std::vector<float> wantGrad(in.size()), wantMlp(static_cast<size_t>(b) * k);
        std::vector<float> sym(accStride);
        for(uint32_t s = 0; s < b; ++s)
        {
            const DataT* f = in.data() + static_cast<size_t>(s) * inStride;
            const DataT* u = up.data() + static_cast<size_t>(s) * upStride;
            for(uint32_t h = 0; h < k; ++h)
                wantMlp[static_cast<size_t>(s) * k + h] = static_cast<float>(u[h]);
            size_t at = k;
            for(uint32_t i = 0; i < m; ++i)
            {
                sym[i * m + i] = 0.f;
                for(uint32_t j = 0; j < i; ++j)
                    sym[i * m + j] = sym[j * m + i] = static_cast<float>(u[at++]);
            }
            for(uint32_t i = 0; i < m; ++i)
            {
                float* g = wantGrad.data() + static_cast<size_t>(s) * inStride + i * k; // starts at 0
                for(uint32_t j = 0; j < m; ++j)
                    for(uint32_t h = 0; h < k; ++h)
                        g[h] += sym[i * m + j] * static_cast<float>(f[j * k + h]);
            }
        }

        const dim3 trilGrid((m * m + 127u) / 128u, 1, b), block(128, 1);
        const dim3 grid((m + 2u * Tile - 1u) / (2u * Tile), (k + Tile - 1u) / Tile, b);
        const uint32_t ldsBytes = 2u * sizeof(DataT) * 3u * Tile * Tile;
        for(bool lds : {false, true})
        {
            DeviceBuffer<DataT> dIn(in.size()), dUp(up.size()), dGrad(in.size()), dMlp(wantMlp.size());
            DeviceBuffer<DataT> dAcc(static_cast<size_t>(b) * accStride);
            dIn.upload(in);
            dUp.upload(up);
            if(lds)
                hipLaunchKernelGGL((trilReconstructLds<DataT>), trilGrid, block, 0, 0, dUp.ptr, dAcc.ptr, m, k, b,
                                   upStride, accStride);
            else
                hipLaunchKernelGGL((trilReconstruct<DataT>), trilGrid, block, 0, 0, dUp.ptr, dAcc.ptr, m, k, b,
                                   upStride, accStride);
            HIP_OK(hipGetLastError());
            HIP_OK(hipDeviceSynchronize());
            if(lds)
                hipLaunchKernelGGL((dlrmDotBwdLds<DataT, Tile, LdsRF>), grid, block, ldsBytes, 0,
                                   dIn.ptr, dUp.ptr, dGrad.ptr, dMlp.ptr, dAcc.ptr, m, k, b, inStride, upStride,
                                   accStride);
            else
                hipLaunchKernelGGL((dlrmDotBwd<DataT, Tile>), grid, block, 0, 0, dIn.ptr, dUp.ptr, dGrad.ptr,
                                   dMlp.ptr, dAcc.ptr, m, k, b, inStride, upStride, accStride);
            HIP_OK(hipGetLastError());
            HIP_OK(hipDeviceSynchronize());

            float  got0 = 0, want0 = 0;
            size_t bad = countDifferent(dGrad.download(), wantGrad, &got0, &want0);
            bad += countDifferent(dMlp.download(), wantMlp, &got0, &want0);
            report("dlrmDotBwd", type, Tile, lds, m, k, b, bad, got0, want0);
        }
    }

    template <typename DataT, uint32_t Tile>
    void runAll(const char* type)
    {
        // the reference's problem sizes (test/dlrm/test/*.cpp: m, k in {32, 128, 1024}), with fewer samples
        const uint32_t sizes[][3] = {{32, 32, 8}, {32, 128, 8}, {128, 128, 8}, {1024, 1024, 1}};
        for(auto const& s : sizes)
        {
            if(s[0] % Tile != 0u || s[1] % Tile != 0u)
                continue;
            runForward<DataT, Tile>(type, s[0], s[1], s[2]);
            runBackward<DataT, Tile>(type, s[0], s[1], s[2]);
        }
    }
} // namespace

int main()
{
    runAll<float16_t, 16>("f16");
    runAll<float16_t, 32>("f16");
    runAll<float32_t, 16>("f32");
    runAll<float32_t, 32>("f32");
    std::printf("SUMMARY: %d passed, %d failed, 0 skipped\n", gPassed, gFailed);
    return gFailed == 0 ? 0 : 1;
}
