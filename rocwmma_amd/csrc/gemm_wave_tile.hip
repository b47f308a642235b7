// Wave-tile GEMM: D = alpha * A * B + beta * C with one BM x BN output block per wave, operands
// loaded straight from global memory through the public fragment API (no LDS).
//
// This is the gfx950 counterpart of the reference's hgemm_rocwmma_d
// (samples/simple_hgemm.cpp:81-139): same decomposition (a workgroup of waves, each owning one
// block; K walked in BlockK steps; epilogue D = alpha*acc + beta*C element-wise on fragments),
// generalised over input type, A/B layout and run-time C/D layout.  It serves the small
// configuration, every shape that does not fill the blocked kernel's macro tiles, and the
// layouts the blocked kernel does not cover.
#include "common.hpp"

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        constexpr uint32_t kWavesX = 2; // along M  (blockDim.x = 64 * kWavesX)
        constexpr uint32_t kWavesY = 2; // along N  (blockDim.y = kWavesY)

        template <typename InT, typename OutT, typename CompT, typename LA, typename LB, uint32_t BM, uint32_t BN, uint32_t BK>
        __global__ void __launch_bounds__(64 * kWavesX * kWavesY) gemmWaveTileKernel(uint32_t     m,
                                                                                      uint32_t     n,
                                                                                      uint32_t     k,
                                                                                      InT const*   a,
                                                                                      InT const*   b,
                                                                                      OutT const*  c,
                                                                                      OutT*        d,
                                                                                      uint32_t     lda,
                                                                                      uint32_t     ldb,
                                                                                      uint32_t     ldc,
                                                                                      uint32_t     ldd,
                                                                                      CompT        alpha,
                                                                                      CompT        beta,
                                                                                      layout_t     layoutC,
                                                                                      const float* bias, // fused epilogue (float
                                                                                      int          activation) // compute types only)
        {
            using FragA   = fragment<matrix_a, BM, BN, BK, InT, LA>;
            using FragB   = fragment<matrix_b, BM, BN, BK, InT, LB>;
            using FragC   = fragment<accumulator, BM, BN, BK, OutT>;
            using FragAcc = fragment<accumulator, BM, BN, BK, CompT>;
            using MapA    = GetDataLayout_t<FragA>;
            using MapB    = GetDataLayout_t<FragB>;

            const uint32_t waveRow = (blockIdx.x * blockDim.x + threadIdx.x) / Constants::AMDGCN_WAVE_SIZE;
            const uint32_t waveCol = blockIdx.y * blockDim.y + threadIdx.y;
            const uint32_t cRow    = waveRow * BM;
            const uint32_t cCol    = waveCol * BN;
            if(cRow >= m || cCol >= n)
                return;

            FragAcc acc;
            fill_fragment(acc, static_cast<CompT>(0));

            // (64-bit offsets of the block's first element: operands of 2^32 elements and more)
            const InT*     aPtr  = a + (std::is_same<LA, row_major>::value ? static_cast<size_t>(cRow) * lda : cRow);
            const InT*     bPtr  = b + (std::is_same<LB, row_major>::value ? cCol : static_cast<size_t>(cCol) * ldb);
            const uint32_t aStep = MapA::fromMatrixCoord(make_coord2d(0u, BK), lda);
            const uint32_t bStep = MapB::fromMatrixCoord(make_coord2d(BK, 0u), ldb);


            for(uint32_t i = 0; i < k; i += BK)
            {
                FragA fa;
                FragB fb;
                load_matrix_sync(fa, aPtr, lda);
                load_matrix_sync(fb, bPtr, ldb);
                mma_sync(acc, fa, fb, acc);
                aPtr += aStep;
                bPtr += bStep;
            }

            // fused epilogue: the bias of each element's column is added and the activation applied
            // before the result is narrowed
            using MapAcc = typename detail::FragConfig<accumulator, BM, BN, BK, CompT>::Map;
            auto finish  = [&](uint32_t e, CompT v) -> CompT {
                if constexpr(std::is_same<CompT, float32_t>::value)
                {
                    if(bias)
                        v += bias[cCol + MapAcc::colOf(e, threadIdx.x % Constants::AMDGCN_WAVE_SIZE)];
                    return applyActivation(v, activation);
                }
                else
                {
                    (void)e;
                    return v;
                }
            };

            FragC          fc;
            const size_t   cOff = layoutC == mem_row_major ? static_cast<size_t>(cRow) * ldc + cCol
                                                           : static_cast<size_t>(cCol) * ldc + cRow;
            const size_t   dOff = layoutC == mem_row_major ? static_cast<size_t>(cRow) * ldd + cCol
                                                           : static_cast<size_t>(cCol) * ldd + cRow;
            if(beta != static_cast<CompT>(0))
            {
                load_matrix_sync(fc, c + cOff, ldc, layoutC);
#pragma unroll
                for(uint32_t i = 0; i < fc.num_elements; ++i)
                    fc.x[i] = static_cast<OutT>(finish(i, alpha * acc.x[i] + beta * static_cast<CompT>(fc.x[i])));
            }
            else
            {
#pragma unroll
                for(uint32_t i = 0; i < fc.num_elements; ++i)
                    fc.x[i] = static_cast<OutT>(finish(i, alpha * acc.x[i]));
            }
            store_matrix_sync(d + dOff, fc, ldd, layoutC);
        }

        template <typename InT, typename OutT, typename CompT, typename LA, typename LB, uint32_t B, uint32_t BK>
        int launchOne(GemmArgs const& g, hipStream_t stream)
        {
            dim3 block(64 * kWavesX, kWavesY);
            dim3 grid(ceilDiv(g.m, B * kWavesX), ceilDiv(g.n, B * kWavesY));
            hipLaunchKernelGGL((gemmWaveTileKernel<InT, OutT, CompT, LA, LB, B, B, BK>),
                               grid,
                               block,
                               0,
                               stream,
                               g.m,
                               g.n,
                               g.k,
                               static_cast<InT const*>(g.a),
                               static_cast<InT const*>(g.b),
                               static_cast<OutT const*>(g.c),
                               static_cast<OutT*>(g.d),
                               g.lda,
                               g.ldb,
                               g.ldc,
                               g.ldd,
                               static_cast<CompT>(g.alpha),
                               static_cast<CompT>(g.beta),
                               g.layoutC == ROCWMMA_AMD_ROW_MAJOR ? mem_row_major : mem_col_major,
                               g.bias,
                               g.activation);
            return launchStatus();
        }

        // KWide16 / KWide32: the widest BlockK with a single-instruction MFMA for 16- and
        // 32-wide blocks; KNarrow*: the legacy half-width shapes for K that is not a multiple.
        template <typename InT, typename OutT, typename CompT, typename LA, typename LB, uint32_t KWide16, uint32_t KWide32>
        int pickBlock(GemmArgs const& g, hipStream_t stream)
        {
            const bool block32 = (g.m % 32u == 0u) && (g.n % 32u == 0u);
            if(block32)
            {
                if(g.k % KWide32 == 0u)
                    return launchOne<InT, OutT, CompT, LA, LB, 32, KWide32>(g, stream);
                if(g.k % (KWide32 / 2u) == 0u && sizeof(InT) == 2)
                    return launchOne<InT, OutT, CompT, LA, LB, 32, (sizeof(InT) == 2 ? KWide32 / 2u : KWide32)>(g, stream);
            }
            if(g.m % 16u != 0u || g.n % 16u != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            if(g.k % KWide16 == 0u)
                return launchOne<InT, OutT, CompT, LA, LB, 16, KWide16>(g, stream);
            if(g.k % (KWide16 / 2u) == 0u && sizeof(InT) == 2)
                return launchOne<InT, OutT, CompT, LA, LB, 16, (sizeof(InT) == 2 ? KWide16 / 2u : KWide16)>(g, stream);
            if(g.k % 32u == 0u && sizeof(InT) == 1)
                return launchOne<InT, OutT, CompT, LA, LB, 16, (sizeof(InT) == 1 ? 32u : KWide16)>(g, stream);
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        }

        template <typename InT, typename OutT, typename CompT, uint32_t KWide16, uint32_t KWide32>
        int pickLayout(int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream)
        {
            const bool aRow = layoutA == ROCWMMA_AMD_ROW_MAJOR;
            const bool bRow = layoutB == ROCWMMA_AMD_ROW_MAJOR;
            if(aRow && !bRow)
                return pickBlock<InT, OutT, CompT, row_major, col_major, KWide16, KWide32>(g, stream);
            if(aRow && bRow)
                return pickBlock<InT, OutT, CompT, row_major, row_major, KWide16, KWide32>(g, stream);
            if(!aRow && !bRow)
                return pickBlock<InT, OutT, CompT, col_major, col_major, KWide16, KWide32>(g, stream);
            return pickBlock<InT, OutT, CompT, col_major, row_major, KWide16, KWide32>(g, stream);
        }
    } // namespace

    int launchGemmWaveTile(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream)
    {
        // the per-step pointer increments along K are 32-bit element counts (BlockK * ld at most)
        if(static_cast<uint64_t>(g.lda) * 256u >= (1ull << 32) || static_cast<uint64_t>(g.ldb) * 256u >= (1ull << 32))
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        if(dtypeIn == ROCWMMA_AMD_F16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout<float16_t, float32_t, float32_t, 32, 16>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_F16 && dtypeOut == ROCWMMA_AMD_F16)
            return pickLayout<float16_t, float16_t, float32_t, 32, 16>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_BF16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout<bfloat16_t, float32_t, float32_t, 32, 16>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_BF16 && dtypeOut == ROCWMMA_AMD_BF16)
            return pickLayout<bfloat16_t, bfloat16_t, float32_t, 32, 16>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_F32 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout<float32_t, float32_t, float32_t, 4, 2>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_E4M3 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout<float8_t, float32_t, float32_t, 128, 64>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_E5M2 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout<bfloat8_t, float32_t, float32_t, 128, 64>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_I8 && dtypeOut == ROCWMMA_AMD_I32)
            return pickLayout<int8_t, int32_t, int32_t, 64, 32>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_I8 && dtypeOut == ROCWMMA_AMD_I8)
            return pickLayout<int8_t, int8_t, int32_t, 64, 32>(layoutA, layoutB, g, stream);
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    }

} // namespace rocwmma_amd
