// Blocked GEMM for gfx950: D = alpha * A * B + beta * C, C/D row-major.
//
// The workload of the reference's perf_hgemm sample (gemm_rocwmma_d,
// samples/perf_hgemm.cpp:518-714: macro tile per workgroup, wave tile of MFMA blocks per wave,
// two LDS buffers, next K slab prefetched while the current one is multiplied), re-tiled and
// re-plumbed for CDNA4:
//
//   reference (gfx9 params)                      this kernel
//   macro tile 128 x 128 x 16, 4 waves           256 x 256 x (128 bytes of K), 4 waves (2 x 2)
//   wave tile 2 x 2 blocks of 32x32x16 (2 MFMA)  4 x 4 blocks of 32x32, one wide-K MFMA per step
//   global -> VGPR -> shuffle -> LDS             global -> LDS directly (global_load_lds_dwordx4)
//   LDS -> VGPR -> shuffle (AOS<->SOA)           swizzled ds_read_b128, or ds_read_b64_tr_b16
//                                                for operands whose K is not contiguous
//   8 MFMA between barriers                      64 MFMA (256 passes) between barriers
//   grid (m/128, n/128)                          1-D grid, tiles dealt to XCDs in L2-friendly patches
//
// Column-major C/D is handled by the caller as the transposed problem (D^T = B^T A^T).
#include "common.hpp"
#include <rocwmma/rocwmma_lds.hpp>

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        constexpr uint32_t kXcds = 8; // MI355X: 8 accelerator complex dies, one L2 each

        template <typename InT_,
                  typename OutT_,
                  typename CompT_,
                  bool     AKMajor_, // A row-major  (K contiguous)
                  bool     BKMajor_, // B col-major  (K contiguous)
                  uint32_t WavesM_,
                  uint32_t WavesN_,
                  uint32_t BlocksM_,
                  uint32_t BlocksN_>
        struct BlockedConfig
        {
            using InT   = InT_;
            using OutT  = OutT_;
            using CompT = CompT_;

            static constexpr bool     AKMajor  = AKMajor_;
            static constexpr bool     BKMajor  = BKMajor_;
            static constexpr uint32_t WavesM   = WavesM_;
            static constexpr uint32_t WavesN   = WavesN_;
            static constexpr uint32_t BlocksM  = BlocksM_;
            static constexpr uint32_t BlocksN  = BlocksN_;
            static constexpr uint32_t Waves    = WavesM * WavesN;
            static constexpr uint32_t Threads  = Waves * 64u;
            static constexpr uint32_t Block    = 32u; // MFMA edge
            static constexpr uint32_t WaveM    = BlocksM * Block;
            static constexpr uint32_t WaveN    = BlocksN * Block;
            static constexpr uint32_t MacroM   = WavesM * WaveM;
            static constexpr uint32_t MacroN   = WavesN * WaveN;
            static constexpr uint32_t TileKB   = 128u; // bytes of K per LDS tile
            static constexpr uint32_t MacroK   = TileKB / sizeof(InT);

            // Fragments of one MFMA step.  BlockK = K of the widest single instruction.
            static constexpr uint32_t KPack      = detail::maxKPack(detail::packClassOf<InT>());
            static constexpr uint32_t BlockK     = KPack * 2u; // 32-wide blocks: 2 lane groups along K
            static constexpr uint32_t KPackBytes = KPack * sizeof(InT);
            static constexpr uint32_t KSteps     = MacroK / BlockK;

            using FragA   = fragment<matrix_a, Block, Block, BlockK, InT, row_major>;
            using FragB   = fragment<matrix_b, Block, Block, BlockK, InT, col_major>;
            using FragAcc = fragment<accumulator, Block, Block, BlockK, CompT>;
            using FragC   = fragment<accumulator, Block, Block, BlockK, OutT, row_major>;

            using TileAK = lds::KMajorTile<MacroM>;
            using TileBK = lds::KMajorTile<MacroN>;
            using TileAD = lds::DimMajorTile<MacroM>;
            using TileBD = lds::DimMajorTile<MacroN>;

            static constexpr uint32_t BytesA   = MacroM * TileKB;
            static constexpr uint32_t BytesB   = MacroN * TileKB;
            static constexpr uint32_t StageB   = BytesA + BytesB;
            static constexpr uint32_t Stages   = 2u;
            static constexpr uint32_t LdsBytes = Stages * StageB;

            static_assert(AKMajor || sizeof(InT) == 2, "transposing LDS reads exist for 16-bit types only");
            static_assert(BKMajor || sizeof(InT) == 2, "transposing LDS reads exist for 16-bit types only");
            static_assert(LdsBytes <= Constants::AMDGCN_LDS_MAX_SIZE_BYTES, "macro tile does not fit the LDS");
        };

        // Deals the 1-D grid to tiles so that the workgroups resident on one XCD (ids congruent
        // mod 8 land on the same XCD) form a compact patch of the tile grid and share A / B
        // panels through that XCD's L2.
        ROCWMMA_DEVICE inline void tileOfWorkgroup(uint32_t wg, uint32_t tilesM, uint32_t tilesN, uint32_t& tm, uint32_t& tn)
        {
            const uint32_t total = tilesM * tilesN;
            uint32_t       id    = wg;
            if(total % kXcds == 0u)
                id = (wg % kXcds) * (total / kXcds) + wg / kXcds;
            // panels of 8 tile rows, walked column by column
            constexpr uint32_t panel      = 8u;
            const uint32_t     perPanel   = panel * tilesN;
            const uint32_t     panelIdx   = id / perPanel;
            const uint32_t     firstRow   = panelIdx * panel;
            const uint32_t     rowsHere   = (tilesM - firstRow) < panel ? (tilesM - firstRow) : panel;
            const uint32_t     inPanel    = id - panelIdx * perPanel;
            tm                            = firstRow + inPanel % rowsHere;
            tn                            = inPanel / rowsHere;
        }

        template <typename Cfg>
        __global__ void __launch_bounds__(Cfg::Threads) gemmBlockedKernel(uint32_t                   m,
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
                                                                           typename Cfg::CompT        beta)
        {
            using InT   = typename Cfg::InT;
            using OutT  = typename Cfg::OutT;
            using CompT = typename Cfg::CompT;

            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];

            const uint32_t lane   = threadIdx.x & 63u;
            const uint32_t wave   = threadIdx.x >> 6;
            const uint32_t waveM  = wave / Cfg::WavesN;
            const uint32_t waveN  = wave % Cfg::WavesN;

            uint32_t tm, tn;
            tileOfWorkgroup(blockIdx.x, m / Cfg::MacroM, n / Cfg::MacroN, tm, tn);
            const uint32_t row0 = tm * Cfg::MacroM;
            const uint32_t col0 = tn * Cfg::MacroN;

            // Global sources of the first K tile (byte pointers)
            const char* aSrc;
            const char* bSrc;
            uint32_t    aStep, bStep; // bytes to the next K tile
            const uint32_t ldaB = lda * sizeof(InT);
            const uint32_t ldbB = ldb * sizeof(InT);
            if constexpr(Cfg::AKMajor)
            {
                aSrc  = reinterpret_cast<const char*>(a) + static_cast<size_t>(row0) * ldaB;
                aStep = Cfg::TileKB;
            }
            else
            {
                aSrc  = reinterpret_cast<const char*>(a) + static_cast<size_t>(row0) * sizeof(InT);
                aStep = Cfg::MacroK * ldaB;
            }
            if constexpr(Cfg::BKMajor)
            {
                bSrc  = reinterpret_cast<const char*>(b) + static_cast<size_t>(col0) * ldbB;
                bStep = Cfg::TileKB;
            }
            else
            {
                bSrc  = reinterpret_cast<const char*>(b) + static_cast<size_t>(col0) * sizeof(InT);
                bStep = Cfg::MacroK * ldbB;
            }

            auto issueTile = [&](uint32_t stage) {
                char* ldsA = ldsRaw + stage * Cfg::StageB;
                char* ldsB = ldsA + Cfg::BytesA;
                if constexpr(Cfg::AKMajor)
                    Cfg::TileAK::template asyncLoad<Cfg::Waves>(ldsA, aSrc, ldaB, wave, lane);
                else
                    Cfg::TileAD::template asyncLoad<Cfg::Waves>(ldsA, aSrc, ldaB, wave, lane);
                if constexpr(Cfg::BKMajor)
                    Cfg::TileBK::template asyncLoad<Cfg::Waves>(ldsB, bSrc, ldbB, wave, lane);
                else
                    Cfg::TileBD::template asyncLoad<Cfg::Waves>(ldsB, bSrc, ldbB, wave, lane);
                aSrc += aStep;
                bSrc += bStep;
            };

            typename Cfg::FragAcc acc[Cfg::BlocksM][Cfg::BlocksN];
#pragma unroll
            for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
#pragma unroll
                for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
                    fill_fragment(acc[i][j], static_cast<CompT>(0));

            auto computeTile = [&](uint32_t stage) {
                const char* ldsA = ldsRaw + stage * Cfg::StageB;
                const char* ldsB = ldsA + Cfg::BytesA;
#pragma unroll
                for(uint32_t ks = 0; ks < Cfg::KSteps; ++ks)
                {
                    typename Cfg::FragA fa[Cfg::BlocksM];
                    typename Cfg::FragB fb[Cfg::BlocksN];
#pragma unroll
                    for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
                    {
                        const uint32_t r = waveM * Cfg::WaveM + i * Cfg::Block;
                        if constexpr(Cfg::AKMajor)
                            Cfg::TileAK::template readBlock32<Cfg::KPackBytes>(fa[i].x, ldsA, r, ks, lane);
                        else
                            Cfg::TileAD::readBlock32(fa[i].x, ldsA, r, ks, lane);
                    }
#pragma unroll
                    for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
                    {
                        const uint32_t cc = waveN * Cfg::WaveN + j * Cfg::Block;
                        if constexpr(Cfg::BKMajor)
                            Cfg::TileBK::template readBlock32<Cfg::KPackBytes>(fb[j].x, ldsB, cc, ks, lane);
                        else
                            Cfg::TileBD::readBlock32(fb[j].x, ldsB, cc, ks, lane);
                    }
#pragma unroll
                    for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
#pragma unroll
                        for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
                            mma_sync(acc[i][j], fa[i], fb[j], acc[i][j]);
                }
            };

            // Prologue: first K tile into stage 0
            const uint32_t kTiles = k / Cfg::MacroK;
            issueTile(0);
            lds::asyncCopyWait();
            synchronize_workgroup();

            for(uint32_t kt = 0; kt + 1 < kTiles; ++kt)
            {
                const uint32_t stage = kt & 1u;
                issueTile(stage ^ 1u); // next tile streams into the other buffer ...
                computeTile(stage); // ... while this one is multiplied
                lds::asyncCopyWait();
                synchronize_workgroup();
            }
            computeTile((kTiles - 1u) & 1u);

            // Epilogue: D = alpha * acc + beta * C, block by block (16-byte accesses per lane)
            const uint32_t wRow = row0 + waveM * Cfg::WaveM;
            const uint32_t wCol = col0 + waveN * Cfg::WaveN;
#pragma unroll
            for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
            {
#pragma unroll
                for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
                {
                    const size_t rr = wRow + i * Cfg::Block;
                    const size_t cc = wCol + j * Cfg::Block;
                    typename Cfg::FragC fc;
                    if(beta != static_cast<CompT>(0))
                    {
                        load_matrix_sync(fc, c + rr * ldc + cc, ldc);
#pragma unroll
                        for(uint32_t e = 0; e < fc.num_elements; ++e)
                            fc.x[e] = static_cast<OutT>(alpha * acc[i][j].x[e] + beta * static_cast<CompT>(fc.x[e]));
                    }
                    else
                    {
#pragma unroll
                        for(uint32_t e = 0; e < fc.num_elements; ++e)
                            fc.x[e] = static_cast<OutT>(alpha * acc[i][j].x[e]);
                    }
                    store_matrix_sync(d + rr * ldd + cc, fc, ldd);
                }
            }
        }

        template <typename Cfg>
        int launchCfg(GemmArgs const& g, hipStream_t stream)
        {
            if(g.m % Cfg::MacroM != 0u || g.n % Cfg::MacroN != 0u || g.k % Cfg::MacroK != 0u || g.k < Cfg::MacroK)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            auto kernel = gemmBlockedKernel<Cfg>;
            // more than 64 KiB of dynamic LDS needs an explicit opt-in (idempotent, no allocation)
            if(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize,
                                   static_cast<int>(Cfg::LdsBytes))
               != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            const uint32_t tiles = (g.m / Cfg::MacroM) * (g.n / Cfg::MacroN);
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
                               static_cast<typename Cfg::CompT>(g.beta));
            return launchStatus();
        }

        // Tile ladder: the 256 x 256 macro tile when the problem fills it, else 128 x 128.
        template <typename InT, typename OutT, typename CompT, bool AK, bool BK>
        int pickTile(GemmArgs const& g, hipStream_t stream)
        {
            using Big   = BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 4, 4>;
            using Small = BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 2>;
            if(g.m % Big::MacroM == 0u && g.n % Big::MacroN == 0u)
            {
                int rc = launchCfg<Big>(g, stream);
                if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                    return rc;
            }
            return launchCfg<Small>(g, stream);
        }

        template <typename InT, typename OutT, typename CompT>
        int pickLayout16(int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream)
        {
            const bool ak = layoutA == ROCWMMA_AMD_ROW_MAJOR;
            const bool bk = layoutB == ROCWMMA_AMD_COL_MAJOR;
            if(ak && bk)
                return pickTile<InT, OutT, CompT, true, true>(g, stream);
            if(ak && !bk)
                return pickTile<InT, OutT, CompT, true, false>(g, stream);
            if(!ak && bk)
                return pickTile<InT, OutT, CompT, false, true>(g, stream);
            return pickTile<InT, OutT, CompT, false, false>(g, stream);
        }

        template <typename InT, typename OutT, typename CompT>
        int pickLayout8(int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream)
        {
            // 8-bit operands: only the K-contiguous pairing (row-major A, col-major B)
            if(layoutA == ROCWMMA_AMD_ROW_MAJOR && layoutB == ROCWMMA_AMD_COL_MAJOR)
                return pickTile<InT, OutT, CompT, true, true>(g, stream);
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        }
    } // namespace

    int launchGemmBlocked(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream)
    {
        if(g.layoutC != ROCWMMA_AMD_ROW_MAJOR)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE; // caller transposes the problem first
        if(dtypeIn == ROCWMMA_AMD_F16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout16<float16_t, float32_t, float32_t>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_BF16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout16<bfloat16_t, float32_t, float32_t>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_F16 && dtypeOut == ROCWMMA_AMD_F16)
            return pickLayout16<float16_t, float16_t, float32_t>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_I8 && dtypeOut == ROCWMMA_AMD_I32)
            return pickLayout8<int8_t, int32_t, int32_t>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_E4M3 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout8<float8_t, float32_t, float32_t>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_E5M2 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout8<bfloat8_t, float32_t, float32_t>(layoutA, layoutB, g, stream);
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    }

} // namespace rocwmma_amd
