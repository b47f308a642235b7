// Blocked GEMM for gfx950: the kernels around gemmTile (one macro tile per workgroup; two tilings in one
// launch for a last round that would be at most half full) and their launch helpers.  Included by the
// translation units that instantiate tile configurations (gemm_blocked.hip, gemm_fused.hip).
#ifndef ROCWMMA_AMD_CSRC_GEMM_BLOCKED_LAUNCH_HPP
#define ROCWMMA_AMD_CSRC_GEMM_BLOCKED_LAUNCH_HPP

#include "gemm_blocked_core.hpp"

namespace rocwmma_amd
{
    namespace
    {
        template <typename Cfg>
        __global__ void __launch_bounds__(Cfg::Threads) __attribute__((amdgpu_waves_per_eu(Cfg::WavesPerSimd, Cfg::WavesPerSimd)))
        gemmBlockedKernel(uint32_t                   m,
                          uint32_t                   n,
                          uint32_t                   k,
                          typename Cfg::InT const*   a,
                          typename Cfg::InT const*   b,
                          typename Cfg::OutT const*  c,
                          typename Cfg::OutT*        d,
                          uint32_t                   lda,
                          uint32_t                   ldb,
                          uint32_t                   ldc,
                          uint32_t                   ldd,
                          typename Cfg::CompT        alpha,
                          typename Cfg::CompT        beta,
                          TileExtras                 ex) // block scales, fused epilogue (configurations that have them)
        {
            uint32_t tm, tn;
            tileOfWorkgroup(blockIdx.x, ceilDiv(m, Cfg::MacroM), ceilDiv(n, Cfg::MacroN), tm, tn);
            gemmTile<Cfg>(tm, tn, 0u, k / Cfg::MacroK, m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta, StreamKPart{}, ex);
        }

        // Two tilings in one launch: the first `fullTiles` workgroups run Full tiles, the others the two
        // halves (same rows, half the columns each) of the remaining Full tiles, in the same tile order.
        // Used when the Full tiles alone would leave the last round of workgroups at most half occupied.
        template <typename Full, typename Half>
        __global__ void __launch_bounds__(Full::Threads) __attribute__((amdgpu_waves_per_eu(Full::WavesPerSimd, Full::WavesPerSimd)))
        gemmBlockedSplitTailKernel(uint32_t                   m,
                                   uint32_t                   n,
                                   uint32_t                   k,
                                   typename Full::InT const*  a,
                                   typename Full::InT const*  b,
                                   typename Full::OutT const* c,
                                   typename Full::OutT*       d,
                                   uint32_t                   lda,
                                   uint32_t                   ldb,
                                   uint32_t                   ldc,
                                   uint32_t                   ldd,
                                   typename Full::CompT       alpha,
                                   typename Full::CompT       beta,
                                   uint32_t                   fullTiles,
                                   TileExtras                 ex)
        {
            // (The half tiles go last.  Running half of them first, on half of the compute units of every
            // XCD or on XCDs 0-3, so that one half of the device writes its results while the other is in
            // its main loop, was 3-4 % slower either way.)
            const uint32_t tilesM = m / Full::MacroM, tilesN = n / Full::MacroN;
            uint32_t       tm, tn;
            if(blockIdx.x < fullTiles)
            {
                tileOfWorkgroup(blockIdx.x, tilesM, tilesN, tm, tn);
                gemmTile<Full>(tm, tn, 0u, k / Full::MacroK, m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta, StreamKPart{}, ex);
            }
            else
            {
                const uint32_t j = blockIdx.x - fullTiles;
                tileOfWorkgroup(fullTiles + j / 2u, tilesM, tilesN, tm, tn);
                gemmTile<Half>(tm, 2u * tn + (j & 1u), 0u, k / Half::MacroK, m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha,
                               beta, StreamKPart{}, ex);
            }
        }

        // Launches Full tiles with the tiles of the last round cut into Half tiles when that round would be
        // at most half full: T = q * units + r tiles with 0 < r <= units / 2 would otherwise end with a round
        // that occupies at most half of the compute units for the time of a whole tile (4096 x 14336: 896
        // tiles on 256 units, 3.5 rounds; 6144^3: 2.25 rounds).
        template <typename Full, typename Half>
        int launchSplitTail(GemmArgs const& g, hipStream_t stream, TileExtras const& ex = TileExtras{})
        {
            static_assert(Full::MacroM == Half::MacroM && Full::MacroN == 2u * Half::MacroN && Full::MacroK == Half::MacroK
                              && Full::Threads == Half::Threads && Full::Stages == Half::Stages
                              && Full::WavesPerSimd == Half::WavesPerSimd && !Full::Edges && !Half::Edges,
                          "half tiles: same rows, half the columns, same pipeline");
            if(g.m % Full::MacroM != 0u || g.n % Full::MacroN != 0u || g.k % Full::MacroK != 0u
               || g.k < (Full::Stages - 1u) * Full::MacroK)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            const uint32_t tilesM = g.m / Full::MacroM, tilesN = g.n / Full::MacroN, units = computeUnits();
            const uint32_t total = tilesM * tilesN, rest = total % units;
            if(total < units || rest == 0u || 2u * rest > units)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            {
                const uint64_t spanA = static_cast<uint64_t>(g.lda) * sizeof(typename Full::InT)
                                       * (Full::AKMajor ? Full::MacroM : Full::MacroK);
                const uint64_t spanB = static_cast<uint64_t>(g.ldb) * sizeof(typename Full::InT)
                                       * (Full::BKMajor ? Full::MacroN : Full::MacroK);
                if(spanA >= 0x7FFF0000ull || spanB >= 0x7FFF0000ull)
                    return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            }
            auto               kernel = gemmBlockedSplitTailKernel<Full, Half>;
            constexpr uint32_t lds    = Full::LdsBytes > Half::LdsBytes ? Full::LdsBytes : Half::LdsBytes;
            if(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   static_cast<int>(lds))
               != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            const uint32_t fullTiles = total - rest;
            hipLaunchKernelGGL(kernel, dim3(fullTiles + 2u * rest), dim3(Full::Threads), lds, stream, g.m, g.n, g.k,
                               static_cast<typename Full::InT const*>(g.a), static_cast<typename Full::InT const*>(g.b),
                               static_cast<typename Full::OutT const*>(g.c), static_cast<typename Full::OutT*>(g.d), g.lda,
                               g.ldb, g.ldc, g.ldd, static_cast<typename Full::CompT>(g.alpha),
                               static_cast<typename Full::CompT>(g.beta), fullTiles, ex);
            return launchStatus();
        }

        template <typename Cfg>
        int launchCfg(GemmArgs const& g, hipStream_t stream, TileExtras const& ex = TileExtras{})
        {
            if((!Cfg::Edges && (g.m % Cfg::MacroM != 0u || g.n % Cfg::MacroN != 0u)) || g.k % Cfg::MacroK != 0u
               || g.k < (Cfg::Stages - 1u) * Cfg::MacroK)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            // a stage's copies address their source inside a 2 GiB window from the stage origin
            {
                const uint64_t spanA = static_cast<uint64_t>(g.lda) * sizeof(typename Cfg::InT)
                                       * (Cfg::AKMajor ? Cfg::MacroM : Cfg::MacroK);
                const uint64_t spanB = static_cast<uint64_t>(g.ldb) * sizeof(typename Cfg::InT)
                                       * (Cfg::BKMajor ? Cfg::MacroN : Cfg::MacroK);
                if(spanA >= 0x7FFF0000ull || spanB >= 0x7FFF0000ull)
                    return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            }
            auto kernel = gemmBlockedKernel<Cfg>;
            // more than 64 KiB of dynamic LDS needs an explicit opt-in (idempotent, no allocation)
            if(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize,
                                   static_cast<int>(Cfg::LdsBytes))
               != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            const uint32_t tiles = ceilDiv(g.m, Cfg::MacroM) * ceilDiv(g.n, Cfg::MacroN);
            hipLaunchKernelGGL(kernel,
                               dim3(tiles),
                               dim3(Cfg::Threads),
                               Cfg::LdsBytes,
                               stream,
                               g.m,
                               g.n,
                               g.k,
                               static_cast<typename Cfg::InT const*>(g.a),
                               static_cast<typename Cfg::InT const*>(g.b),
                               static_cast<typename Cfg::OutT const*>(g.c),
                               static_cast<typename Cfg::OutT*>(g.d),
                               g.lda,
                               g.ldb,
                               g.ldc,
                               g.ldd,
                               static_cast<typename Cfg::CompT>(g.alpha),
                               static_cast<typename Cfg::CompT>(g.beta),
                               ex);
            return launchStatus();
        }

        // The 4-wave configurations come with either LDS pipeline.  With at most one workgroup per
        // compute unit a launch is one round of latency-bound workgroups, and the ring of four 64-byte
        // stages (copies three stages ahead) hides more of it: 128 x 14336 x 4096 int8 25.8 against 29.7 us,
        // 2048^3 f16 24 against 27 us.  With more workgroups than compute units the units stream operands
        // all the time, the L2 request rate limits them, and the ring of two 128-byte stages (whole-line
        // requests) wins: 512 x 14336 x 4096 int8 51 -> 44 us, f16 with a row-major B 101 -> 85 us,
        // 192 x 14336 x 4096 f16 (64 x 64 tiles) 74 -> 56 us.  Results are identical bit for bit.
        template <typename Ring4, typename Ring2>
        int launchByRounds(GemmArgs const& g, hipStream_t stream, TileExtras const& ex = TileExtras{})
        {
            static_assert(Ring4::MacroM == Ring2::MacroM && Ring4::MacroN == Ring2::MacroN, "same tiling");
            if(ceilDiv(g.m, Ring4::MacroM) * ceilDiv(g.n, Ring4::MacroN) > computeUnits())
            {
                const int rc = launchCfg<Ring2>(g, stream, ex);
                if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE) // (K not in whole 128-byte stages)
                    return rc;
            }
            return launchCfg<Ring4>(g, stream, ex);
        }
    } // namespace
} // namespace rocwmma_amd

#endif // ROCWMMA_AMD_CSRC_GEMM_BLOCKED_LAUNCH_HPP
