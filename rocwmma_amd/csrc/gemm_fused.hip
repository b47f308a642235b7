// Blocked GEMM with a fused epilogue, D = act(alpha * A * B + beta * C + bias[column]): the Fused
// configurations of the blocked kernel (gemm_blocked_core.hpp) and their dispatch.
//
// The reference's GEMM kernels end with D = alpha * acc + beta * C on fragments
// (samples/perf_hgemm.cpp:683-713); a bias and an activation behind them are two more passes over D.
// Here the accumulators take both on their way out: the lane's bias values (the same for every row of
// blocks) sit in registers, the activation is evaluated in f32 before the result is narrowed.
#include "gemm_blocked_launch.hpp"

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        // Two rungs: 256 x 256 tiles (with the last round cut into half tiles) for problems in whole large
        // tiles that occupy at least half of the compute units, else 128 x 128 tiles whose last row and
        // column of tiles may be partly filled (any m, n in multiples of 16).
        template <typename InT, typename OutT, bool AK, bool BK>
        int pickTile(GemmArgs const& g, hipStream_t stream)
        {
            static constexpr bool Edge16 = sizeof(InT) == 2u || (AK && BK);
            using Big     = std::conditional_t<Edge16,
                                               BlockedConfig<InT, OutT, float32_t, AK, BK, 4, 2, 4, 8, 2, 2, 16, false, false, true>,
                                               BlockedConfig<InT, OutT, float32_t, AK, BK, 4, 2, 2, 4, 2, 2, 32, false, false, true>>;
            using BigHalf = std::conditional_t<Edge16,
                                               BlockedConfig<InT, OutT, float32_t, AK, BK, 4, 2, 4, 4, 2, 2, 16, false, false, true>,
                                               BlockedConfig<InT, OutT, float32_t, AK, BK, 4, 2, 2, 2, 2, 2, 32, false, false, true>>;
            using Edge    = BlockedConfig<InT, OutT, float32_t, AK, BK, 2, 2, 2, 2, 4, 2, 32, true, false, true>;
            using Edge2   = BlockedConfig<InT, OutT, float32_t, AK, BK, 2, 2, 2, 2, 2, 2, 32, true, false, true>;
            TileExtras ex{};
            ex.fused = FusedEpilogue{g.bias, g.activation};
            if(g.m % Big::MacroM == 0u && g.n % Big::MacroN == 0u
               && 2u * (g.m / Big::MacroM) * (g.n / Big::MacroN) >= computeUnits())
            {
                int rc = launchSplitTail<Big, BigHalf>(g, stream, ex);
                if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                    return rc;
                rc = launchCfg<Big>(g, stream, ex);
                if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                    return rc;
            }
            return launchByRounds<Edge, Edge2>(g, stream, ex);
        }

        template <typename InT, typename OutT>
        int pickLayout(int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream)
        {
            const bool ak = layoutA == ROCWMMA_AMD_ROW_MAJOR;
            const bool bk = layoutB == ROCWMMA_AMD_COL_MAJOR;
            if(ak && bk)
                return pickTile<InT, OutT, true, true>(g, stream);
            if(ak && !bk)
                return pickTile<InT, OutT, true, false>(g, stream);
            if(!ak && bk)
                return pickTile<InT, OutT, false, true>(g, stream);
            return pickTile<InT, OutT, false, false>(g, stream);
        }
    } // namespace

    int launchGemmBlockedFused(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream)
    {
        if(g.layoutC != ROCWMMA_AMD_ROW_MAJOR)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE; // (the bias runs along the columns of a row-major D)
        if(dtypeIn == ROCWMMA_AMD_F16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout<float16_t, float32_t>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_BF16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout<bfloat16_t, float32_t>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_F16 && dtypeOut == ROCWMMA_AMD_F16)
            return pickLayout<float16_t, float16_t>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_BF16 && dtypeOut == ROCWMMA_AMD_BF16)
            return pickLayout<bfloat16_t, bfloat16_t>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_E4M3 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout<float8_t, float32_t>(layoutA, layoutB, g, stream);
        if(dtypeIn == ROCWMMA_AMD_E5M2 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout<bfloat8_t, float32_t>(layoutA, layoutB, g, stream);
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    }

} // namespace rocwmma_amd
