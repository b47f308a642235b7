// Device side of the API-semantics tests: tiny kernels written ONLY against the public
// rocwmma:: API (fragment, load/store_matrix_sync, the cooperative loaders, the transforms,
// mma_sync).  The host tests compare their output with the CPU oracle / with the input.
//
// roundtrip  : out tile = store(load(in tile)), one fragment per wave, or one fragment per
//              workgroup of four waves through the cooperative pair.  Mirrors the reference
//              unit tests test/unit/load_store_matrix_sync_test/device/load_store_matrix_sync.hpp:35-117
//              and test/unit/load_store_matrix_coop_sync_test.  Elements outside the tiles are
//              never written, which the host checks with a padding ring (contamination test,
//              reference test/unit/contamination_test).
// coop gemm  : the data flow of the reference's perf_hgemm sample (samples/perf_hgemm.cpp:328-409,
//              518-714) at a small fixed tiling: cooperative global read of macro-tile
//              fragments, applyDataLayout / applyTranspose, cooperative LDS write, LDS read of
//              MFMA fragments, mma_sync, fragment-wise epilogue.
#include "common.hpp"
#include <rocwmma/rocwmma_coop.hpp>
#include <rocwmma/rocwmma_transforms.hpp>

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        template <typename FragT, bool Coop>
        __global__ void __launch_bounds__(256)
            roundtripKernel(uint32_t rows, uint32_t cols, GetDataType_t<FragT> const* in, GetDataType_t<FragT>* out, uint32_t ld)
        {
            using Shape  = GetIOShape_t<FragT>;
            using Layout = GetDataLayout_t<FragT>;
            // non-coop: blockDim = (128, 2) -> 2 x 2 waves, one fragment each
            // coop    : blockDim = (256, 1) -> one fragment per workgroup
            uint32_t tileRow, tileCol;
            if constexpr(Coop)
            {
                tileRow = blockIdx.x;
                tileCol = blockIdx.y;
            }
            else
            {
                tileRow = (blockIdx.x * blockDim.x + threadIdx.x) / Constants::AMDGCN_WAVE_SIZE;
                tileCol = blockIdx.y * blockDim.y + threadIdx.y;
            }
            const uint32_t r0 = tileRow * Shape::BlockHeight;
            const uint32_t c0 = tileCol * Shape::BlockWidth;
            if(r0 + Shape::BlockHeight > rows || c0 + Shape::BlockWidth > cols)
                return;
            const uint32_t off = Layout::fromMatrixCoord(make_coord2d(r0, c0), ld);
            FragT          frag;
            if constexpr(Coop)
            {
                load_matrix_coop_sync(frag, in + off, ld);
                store_matrix_coop_sync(out + off, frag, ld);
            }
            else
            {
                load_matrix_sync(frag, in + off, ld);
                store_matrix_sync(out + off, frag, ld);
            }
        }

        template <typename FragT>
        int launchRoundtrip(int coop, uint32_t rows, uint32_t cols, const void* in, void* out, uint32_t ld, hipStream_t stream)
        {
            using Shape = GetIOShape_t<FragT>;
            using T     = GetDataType_t<FragT>;
            if(rows % Shape::BlockHeight != 0u || cols % Shape::BlockWidth != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            const uint32_t tr = rows / Shape::BlockHeight, tc = cols / Shape::BlockWidth;
            if(coop)
                hipLaunchKernelGGL((roundtripKernel<FragT, true>), dim3(tr, tc), dim3(256, 1), 0, stream, rows, cols,
                                   static_cast<const T*>(in), static_cast<T*>(out), ld);
            else
                hipLaunchKernelGGL((roundtripKernel<FragT, false>), dim3(ceilDiv(tr, 2u), ceilDiv(tc, 2u)), dim3(128, 2), 0,
                                   stream, rows, cols, static_cast<const T*>(in), static_cast<T*>(out), ld);
            return launchStatus();
        }

        // Block sizes follow the reference's unit-test matrix (test/unit/unit_test_params.hpp:89-141):
        // BlockM/N 16..256 against BlockK 8..256, thinned for the largest blocks to bound the
        // number of kernels.
        constexpr bool roundtripShape(uint32_t block, uint32_t blockk)
        {
            if(block == 16u)
                return blockk == 16u || blockk == 32u || blockk == 64u || blockk == 128u || blockk == 256u;
            if(block == 32u || block == 64u)
                return blockk == 8u || blockk == 16u || blockk == 32u || blockk == 64u || blockk == 128u;
            if(block == 128u || block == 256u)
                return blockk == 8u || blockk == 32u;
            return false;
        }

        template <typename MatrixT, typename T, typename Layout, uint32_t B, uint32_t K>
        int launchShape(int coop, uint32_t rows, uint32_t cols, const void* in, void* out, uint32_t ld, hipStream_t s)
        {
            // accumulator blocks above 64 x 64 would not fit a wave's registers
            constexpr bool tooBig = std::is_same<MatrixT, accumulator>::value && B > 64u;
            if constexpr(roundtripShape(B, K) && !tooBig)
                return launchRoundtrip<fragment<MatrixT, B, B, K, T, Layout>>(coop, rows, cols, in, out, ld, s);
            else
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        }

        template <typename MatrixT, typename T, typename Layout, uint32_t B>
        int pickBlockK(int blockk, int coop, uint32_t rows, uint32_t cols, const void* in, void* out, uint32_t ld, hipStream_t s)
        {
            switch(blockk)
            {
            case 8:
                return launchShape<MatrixT, T, Layout, B, 8>(coop, rows, cols, in, out, ld, s);
            case 16:
                return launchShape<MatrixT, T, Layout, B, 16>(coop, rows, cols, in, out, ld, s);
            case 32:
                return launchShape<MatrixT, T, Layout, B, 32>(coop, rows, cols, in, out, ld, s);
            case 64:
                return launchShape<MatrixT, T, Layout, B, 64>(coop, rows, cols, in, out, ld, s);
            case 128:
                return launchShape<MatrixT, T, Layout, B, 128>(coop, rows, cols, in, out, ld, s);
            case 256:
                return launchShape<MatrixT, T, Layout, B, 256>(coop, rows, cols, in, out, ld, s);
            default:
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            }
        }

        template <typename MatrixT, typename T, typename Layout>
        int pickBlock(int block, int blockk, int coop, uint32_t rows, uint32_t cols, const void* in, void* out, uint32_t ld, hipStream_t s)
        {
            switch(block)
            {
            case 16:
                return pickBlockK<MatrixT, T, Layout, 16>(blockk, coop, rows, cols, in, out, ld, s);
            case 32:
                return pickBlockK<MatrixT, T, Layout, 32>(blockk, coop, rows, cols, in, out, ld, s);
            case 64:
                return pickBlockK<MatrixT, T, Layout, 64>(blockk, coop, rows, cols, in, out, ld, s);
            case 128:
                return pickBlockK<MatrixT, T, Layout, 128>(blockk, coop, rows, cols, in, out, ld, s);
            case 256:
                return pickBlockK<MatrixT, T, Layout, 256>(blockk, coop, rows, cols, in, out, ld, s);
            default:
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            }
        }

        template <typename MatrixT, typename T>
        int pickLayout(int layout, int block, int blockk, int coop, uint32_t rows, uint32_t cols, const void* in, void* out,
                       uint32_t ld, hipStream_t s)
        {
            if(layout == ROCWMMA_AMD_ROW_MAJOR)
                return pickBlock<MatrixT, T, row_major>(block, blockk, coop, rows, cols, in, out, ld, s);
            return pickBlock<MatrixT, T, col_major>(block, blockk, coop, rows, cols, in, out, ld, s);
        }

        template <typename MatrixT>
        int pickType(int dtype, int layout, int block, int blockk, int coop, uint32_t rows, uint32_t cols, const void* in,
                     void* out, uint32_t ld, hipStream_t s)
        {
            switch(dtype)
            {
            case ROCWMMA_AMD_F16:
                return pickLayout<MatrixT, float16_t>(layout, block, blockk, coop, rows, cols, in, out, ld, s);
            case ROCWMMA_AMD_I8:
                return pickLayout<MatrixT, int8_t>(layout, block, blockk, coop, rows, cols, in, out, ld, s);
            case ROCWMMA_AMD_F32:
                return pickLayout<MatrixT, float32_t>(layout, block, blockk, coop, rows, cols, in, out, ld, s);
            default:
                return ROCWMMA_AMD_UNSUPPORTED_TYPE;
            }
        }

        // ---- perf_hgemm data flow through the public API only ---------------------------------
        namespace flow
        {
            constexpr uint32_t BM = 32, BN = 32, BK = 16;
            constexpr uint32_t BlocksX = 2, BlocksY = 2; // MFMA blocks per wave
            constexpr uint32_t WavesX = 2, WavesY = 2; // waves per workgroup: blockDim = (128, 2)
            constexpr uint32_t WaveTileX = BlocksX * BM, WaveTileY = BlocksY * BN;
            constexpr uint32_t MacroX = WavesX * WaveTileX, MacroY = WavesY * WaveTileY;
            constexpr uint32_t WaveCount = WavesX * WavesY;

            using LdsLayout = col_major;

            template <typename LA, typename LB>
            __global__ void __launch_bounds__(256) coopGemmKernel(uint32_t         m,
                                                                  uint32_t         n,
                                                                  uint32_t         k,
                                                                  const float16_t* a,
                                                                  const float16_t* b,
                                                                  const float*     c,
                                                                  float*           d,
                                                                  uint32_t         lda,
                                                                  uint32_t         ldb,
                                                                  uint32_t         ldc,
                                                                  uint32_t         ldd,
                                                                  float            alpha,
                                                                  float            beta)
            {
                using MfmaFragA   = fragment<matrix_a, BM, BN, BK, float16_t, LA>;
                using MfmaFragB   = fragment<matrix_b, BM, BN, BK, float16_t, LB>;
                using MfmaFragC   = fragment<accumulator, BM, BN, BK, float, row_major>;
                using MfmaFragAcc = fragment<accumulator, BM, BN, BK, float>;
                using GRBuffA     = fragment<matrix_a, MacroX, BN, BK, float16_t, LA>;
                using GRBuffB     = fragment<matrix_b, BM, MacroY, BK, float16_t, LB>;
                using LWBuffA     = ApplyDataLayout_t<GRBuffA, LdsLayout>;
                using LWBuffB     = ApplyDataLayout_t<ApplyTranspose_t<GRBuffB>, LdsLayout>;
                static_assert(std::is_same<GetDataLayout_t<LWBuffA>, GetDataLayout_t<LWBuffB>>::value,
                              "A and transposed-B slabs share the LDS layout");
                using LRFragA     = ApplyDataLayout_t<MfmaFragA, LdsLayout>;
                using LRFragB     = ApplyDataLayout_t<ApplyTranspose_t<MfmaFragB>, LdsLayout>;

                extern __shared__ __attribute__((aligned(16))) char ldsRaw[];
                float16_t* lds = reinterpret_cast<float16_t*>(ldsRaw);

                constexpr uint32_t ldsHeight = MacroX + MacroY; // A blocks stacked over transposed B blocks
                constexpr uint32_t ldsld     = ldsHeight; // col-major LDS, width BK

                const auto     waveCoord = make_coord2d(threadIdx.x / Constants::AMDGCN_WAVE_SIZE, threadIdx.y);
                const uint32_t waveIndex = get<0>(waveCoord) * WavesY + get<1>(waveCoord);
                const auto     macroCoord = make_coord2d(blockIdx.x * MacroX, blockIdx.y * MacroY);
                const auto     waveTile   = macroCoord + waveCoord * make_coord2d(WaveTileX, WaveTileY);
                if(get<0>(waveTile) + WaveTileX > m || get<1>(waveTile) + WaveTileY > n)
                    return;

                using MapA = GetDataLayout_t<GRBuffA>;
                using MapB = GetDataLayout_t<GRBuffB>;
                using MapL = GetDataLayout_t<LWBuffA>;

                uint32_t       offA  = MapA::fromMatrixCoord(make_coord2d(get<0>(macroCoord), 0u), lda);
                uint32_t       offB  = MapB::fromMatrixCoord(make_coord2d(0u, get<1>(macroCoord)), ldb);
                const uint32_t stepA = MapA::fromMatrixCoord(make_coord2d(0u, BK), lda);
                const uint32_t stepB = MapB::fromMatrixCoord(make_coord2d(BK, 0u), ldb);

                const uint32_t ldsOffB  = MapL::fromMatrixCoord(make_coord2d(MacroX, 0u), ldsld);
                const uint32_t ldsReadA = MapL::fromMatrixCoord(make_coord2d(get<0>(waveCoord) * WaveTileX, 0u), ldsld);
                const uint32_t ldsReadB
                    = ldsOffB + MapL::fromMatrixCoord(make_coord2d(get<1>(waveCoord) * WaveTileY, 0u), ldsld);
                const uint32_t blockStep = MapL::fromMatrixCoord(make_coord2d(BM, 0u), ldsld);

                MfmaFragAcc acc[BlocksX][BlocksY];
                for(uint32_t i = 0; i < BlocksX; ++i)
                    for(uint32_t j = 0; j < BlocksY; ++j)
                        fill_fragment(acc[i][j], 0.0f);

                for(uint32_t kk = 0; kk < k; kk += BK)
                {
                    GRBuffA grA;
                    GRBuffB grB;
                    load_matrix_coop_sync<WaveCount>(grA, a + offA, lda, waveIndex);
                    load_matrix_coop_sync<WaveCount>(grB, b + offB, ldb, waveIndex);
                    offA += stepA;
                    offB += stepB;

                    synchronize_workgroup(); // previous step's LDS reads are done
                    store_matrix_coop_sync<WaveCount>(lds, applyDataLayout<LdsLayout, WaveCount>(grA), ldsld, waveIndex);
                    store_matrix_coop_sync<WaveCount>(
                        lds + ldsOffB, applyDataLayout<LdsLayout, WaveCount>(applyTranspose(grB)), ldsld, waveIndex);
                    synchronize_workgroup();

                    MfmaFragA fa[BlocksX];
                    MfmaFragB fb[BlocksY];
                    for(uint32_t i = 0; i < BlocksX; ++i)
                    {
                        LRFragA tmp;
                        load_matrix_sync(tmp, lds + ldsReadA + i * blockStep, ldsld);
                        fa[i] = applyDataLayout<LA>(tmp);
                    }
                    for(uint32_t j = 0; j < BlocksY; ++j)
                    {
                        LRFragB tmp;
                        load_matrix_sync(tmp, lds + ldsReadB + j * blockStep, ldsld);
                        fb[j] = applyDataLayout<LB>(applyTranspose(tmp));
                    }
                    for(uint32_t i = 0; i < BlocksX; ++i)
                        for(uint32_t j = 0; j < BlocksY; ++j)
                            mma_sync(acc[i][j], fa[i], fb[j], acc[i][j]);
                }

                for(uint32_t i = 0; i < BlocksX; ++i)
                    for(uint32_t j = 0; j < BlocksY; ++j)
                    {
                        const uint32_t r = get<0>(waveTile) + i * BM, cc = get<1>(waveTile) + j * BN;
                        MfmaFragC      fc;
                        load_matrix_sync(fc, c + r * ldc + cc, ldc);
                        for(uint32_t e = 0; e < fc.num_elements; ++e)
                            fc.x[e] = alpha * acc[i][j].x[e] + beta * fc.x[e];
                        store_matrix_sync(d + r * ldd + cc, fc, ldd);
                    }
            }

            template <typename LA, typename LB>
            int launch(uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b, const float* c, float* d,
                       float alpha, float beta, hipStream_t stream)
            {
                const uint32_t lda = std::is_same<LA, row_major>::value ? k : m;
                const uint32_t ldb = std::is_same<LB, row_major>::value ? n : k;
                const uint32_t lds = (MacroX + MacroY) * BK * sizeof(float16_t);
                hipLaunchKernelGGL((coopGemmKernel<LA, LB>), dim3(m / MacroX, n / MacroY), dim3(64 * WavesX, WavesY), lds,
                                   stream, m, n, k, static_cast<const float16_t*>(a), static_cast<const float16_t*>(b), c, d,
                                   lda, ldb, n, n, alpha, beta);
                return launchStatus();
            }
        } // namespace flow
        // ---- a blocked GEMM for gfx950 through the public API only ------------------------------
        // What a kernel written against the fragment API gets when it is laid out for this device rather than
        // after perf_hgemm: 256 x 256 macro tile, eight waves (4 x 2) of 64 x 128, 16 x 16 x 32 blocks (the
        // full-rate f16 instruction), K stages of 64 in two LDS buffers with one barrier per stage, the next stage's
        // slabs fetched into registers with cooperative loads while this stage is multiplied.  LDS slabs are
        // K-contiguous rows (row-major A, transposed B) of 64 + 8 halves: the 16 rows a quarter-wave reads at one
        // K offset are 144 bytes apart, sixteen distinct 16-byte slots, and fragments are always held in the
        // order the matrix instruction takes them, so every LDS access is a conflict-free 16-byte one whatever
        // the layouts in global memory (applyDataLayout / applyTranspose are re-typings).  Without the padding
        // the same kernel runs at half the speed.
        namespace tiled
        {
            constexpr uint32_t BM = 16, BN = 16, BK = 32;
            constexpr uint32_t BlocksX = 4, BlocksY = 8;
            constexpr uint32_t WavesX = 4, WavesY = 2;
            constexpr uint32_t WaveTileX = BlocksX * BM, WaveTileY = BlocksY * BN;
            constexpr uint32_t MacroX = WavesX * WaveTileX, MacroY = WavesY * WaveTileY;
            constexpr uint32_t WaveCount = WavesX * WavesY;
            constexpr uint32_t StageK = 64, Steps = StageK / BK;
            constexpr uint32_t LdsLd   = StageK + 8; // halves per LDS row
            constexpr uint32_t BufElts = (MacroX + MacroY) * LdsLd;
            constexpr uint32_t LdsBytes = 2u * BufElts * sizeof(float16_t);

            template <typename LA, typename LB>
            __global__ void __launch_bounds__(64 * WaveCount) tiledGemmKernel(uint32_t         m,
                                                                             uint32_t         n,
                                                                             uint32_t         k,
                                                                             const float16_t* a,
                                                                             const float16_t* b,
                                                                             const float*     c,
                                                                             float*           d,
                                                                             uint32_t         lda,
                                                                             uint32_t         ldb,
                                                                             uint32_t         ldc,
                                                                             uint32_t         ldd,
                                                                             float            alpha,
                                                                             float            beta)
            {
                using FragA    = fragment<matrix_a, BM, BN, BK, float16_t, LA>;
                using FragB    = fragment<matrix_b, BM, BN, BK, float16_t, LB>;
                using FragC    = fragment<accumulator, BM, BN, BK, float, row_major>;
                using FragAcc  = fragment<accumulator, BM, BN, BK, float>;
                using LdsFragA = ApplyDataLayout_t<FragA, row_major>;
                using LdsFragB = ApplyDataLayout_t<ApplyTranspose_t<FragB>, row_major>;
                using SlabA    = fragment<matrix_a, MacroX, BN, StageK, float16_t, LA>;
                using SlabB    = fragment<matrix_b, BM, MacroY, StageK, float16_t, LB>;
                using MapA     = GetDataLayout_t<SlabA>;
                using MapB     = GetDataLayout_t<SlabB>;

                extern __shared__ __attribute__((aligned(16))) char ldsRaw[];
                float16_t* lds = reinterpret_cast<float16_t*>(ldsRaw);

                const uint32_t waveIndex = threadIdx.x / Constants::AMDGCN_WAVE_SIZE;
                const uint32_t wx = waveIndex / WavesY, wy = waveIndex % WavesY;
                const uint32_t row0 = blockIdx.x * MacroX, col0 = blockIdx.y * MacroY;

                const float16_t* aPtr  = a + MapA::fromMatrixCoord(make_coord2d(row0, 0u), lda);
                const float16_t* bPtr  = b + MapB::fromMatrixCoord(make_coord2d(0u, col0), ldb);
                const uint32_t   stepA = MapA::fromMatrixCoord(make_coord2d(0u, StageK), lda);
                const uint32_t   stepB = MapB::fromMatrixCoord(make_coord2d(StageK, 0u), ldb);

                FragAcc acc[BlocksX][BlocksY];
                for(uint32_t i = 0; i < BlocksX; ++i)
                    for(uint32_t j = 0; j < BlocksY; ++j)
                        fill_fragment(acc[i][j], 0.0f);

                SlabA grA;
                SlabB grB;
                load_matrix_coop_sync<WaveCount>(grA, aPtr, lda, waveIndex);
                load_matrix_coop_sync<WaveCount>(grB, bPtr, ldb, waveIndex);
                store_matrix_coop_sync<WaveCount>(lds, applyDataLayout<row_major, WaveCount>(grA), LdsLd, waveIndex);
                store_matrix_coop_sync<WaveCount>(lds + MacroX * LdsLd, applyDataLayout<row_major, WaveCount>(applyTranspose(grB)), LdsLd,
                                                  waveIndex);
                synchronize_workgroup();

                uint32_t cur = 0;
                for(uint32_t kk = 0; kk < k; kk += StageK)
                {
                    const bool more = kk + StageK < k;
                    if(more)
                    {
                        aPtr += stepA;
                        bPtr += stepB;
                        load_matrix_coop_sync<WaveCount>(grA, aPtr, lda, waveIndex);
                        load_matrix_coop_sync<WaveCount>(grB, bPtr, ldb, waveIndex);
                    }
                    const float16_t* ldsA = lds + cur * BufElts + wx * WaveTileX * LdsLd;
                    const float16_t* ldsB = lds + cur * BufElts + (MacroX + wy * WaveTileY) * LdsLd;
#pragma unroll
                    for(uint32_t s = 0; s < Steps; ++s)
                    {
                        FragA fa[BlocksX];
                        FragB fb[BlocksY];
#pragma unroll
                        for(uint32_t i = 0; i < BlocksX; ++i)
                        {
                            LdsFragA t;
                            load_matrix_sync(t, ldsA + i * BM * LdsLd + s * BK, LdsLd);
                            fa[i] = applyDataLayout<LA>(t);
                        }
#pragma unroll
                        for(uint32_t j = 0; j < BlocksY; ++j)
                        {
                            LdsFragB t;
                            load_matrix_sync(t, ldsB + j * BN * LdsLd + s * BK, LdsLd);
                            fb[j] = applyDataLayout<LB>(applyTranspose(t));
                        }
#pragma unroll
                        for(uint32_t i = 0; i < BlocksX; ++i)
#pragma unroll
                            for(uint32_t j = 0; j < BlocksY; ++j)
                                mma_sync(acc[i][j], fa[i], fb[j], acc[i][j]);
                    }
                    if(more)
                    {
                        float16_t* nxt = lds + (cur ^ 1u) * BufElts;
                        store_matrix_coop_sync<WaveCount>(nxt, applyDataLayout<row_major, WaveCount>(grA), LdsLd, waveIndex);
                        store_matrix_coop_sync<WaveCount>(nxt + MacroX * LdsLd, applyDataLayout<row_major, WaveCount>(applyTranspose(grB)),
                                                          LdsLd, waveIndex);
                    }
                    synchronize_workgroup();
                    cur ^= 1u;
                }

                for(uint32_t i = 0; i < BlocksX; ++i)
                    for(uint32_t j = 0; j < BlocksY; ++j)
                    {
                        const size_t r = row0 + wx * WaveTileX + i * BM, cc = col0 + wy * WaveTileY + j * BN;
                        FragC        fc;
                        load_matrix_sync(fc, c + r * ldc + cc, ldc);
                        for(uint32_t e = 0; e < fc.num_elements; ++e)
                            fc.x[e] = alpha * acc[i][j].x[e] + beta * fc.x[e];
                        store_matrix_sync(d + r * ldd + cc, fc, ldd);
                    }
            }

            template <typename LA, typename LB>
            int launch(uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b, const float* c, float* d, float alpha, float beta,
                       hipStream_t stream)
            {
                auto kernel = tiledGemmKernel<LA, LB>;
                if(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       static_cast<int>(LdsBytes))
                   != hipSuccess)
                    return ROCWMMA_AMD_LAUNCH_FAILED;
                const uint32_t lda = std::is_same<LA, row_major>::value ? k : m;
                const uint32_t ldb = std::is_same<LB, row_major>::value ? n : k;
                hipLaunchKernelGGL(kernel, dim3(m / MacroX, n / MacroY), dim3(64 * WaveCount), LdsBytes, stream, m, n, k,
                                   static_cast<const float16_t*>(a), static_cast<const float16_t*>(b), c, d, lda, ldb, n, n, alpha, beta);
                return launchStatus();
            }
        } // namespace tiled
    } // namespace

    int selftestTiledGemm(int layoutA, int layoutB, uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b, const float* c,
                          float* d, float alpha, float beta, hipStream_t stream)
    {
        if(m == 0u || n == 0u || k == 0u || m % tiled::MacroX != 0u || n % tiled::MacroY != 0u || k % tiled::StageK != 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const bool ar = layoutA == ROCWMMA_AMD_ROW_MAJOR, br = layoutB == ROCWMMA_AMD_ROW_MAJOR;
        if(ar && br)
            return tiled::launch<row_major, row_major>(m, n, k, a, b, c, d, alpha, beta, stream);
        if(ar && !br)
            return tiled::launch<row_major, col_major>(m, n, k, a, b, c, d, alpha, beta, stream);
        if(!ar && br)
            return tiled::launch<col_major, row_major>(m, n, k, a, b, c, d, alpha, beta, stream);
        return tiled::launch<col_major, col_major>(m, n, k, a, b, c, d, alpha, beta, stream);
    }

    int selftestRoundtrip(int context, int dtype, int layout, int block, int blockk, int coop, uint32_t rows, uint32_t cols,
                          const void* in, void* out, uint32_t ld, hipStream_t stream)
    {
        switch(context)
        {
        case 0:
            return pickType<matrix_a>(dtype, layout, block, blockk, coop, rows, cols, in, out, ld, stream);
        case 1:
            return pickType<matrix_b>(dtype, layout, block, blockk, coop, rows, cols, in, out, ld, stream);
        case 2:
            return pickType<accumulator>(dtype, layout, block, blockk, coop, rows, cols, in, out, ld, stream);
        default:
            return ROCWMMA_AMD_INVALID_ARGUMENT;
        }
    }

    int selftestCoopGemm(int layoutA, int layoutB, uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b,
                         const float* c, float* d, float alpha, float beta, hipStream_t stream)
    {
        if(m % flow::MacroX != 0u || n % flow::MacroY != 0u || k % flow::BK != 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const bool ar = layoutA == ROCWMMA_AMD_ROW_MAJOR, br = layoutB == ROCWMMA_AMD_ROW_MAJOR;
        if(ar && br)
            return flow::launch<row_major, row_major>(m, n, k, a, b, c, d, alpha, beta, stream);
        if(ar && !br)
            return flow::launch<row_major, col_major>(m, n, k, a, b, c, d, alpha, beta, stream);
        if(!ar && br)
            return flow::launch<col_major, row_major>(m, n, k, a, b, c, d, alpha, beta, stream);
        return flow::launch<col_major, col_major>(m, n, k, a, b, c, d, alpha, beta, stream);
    }

} // namespace rocwmma_amd
