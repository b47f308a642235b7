// Benchmark support (librocwmma_amd_aux.so): the blocked GEMM's 256 x 256 kernel built with time stamps in
// its main loop.  ROCWMMA_AMD_PHASE_TRACE makes gemm_blocked_core.hpp read the shader clock at the phase
// boundaries of the ring-of-two loop and leave the sums per wave in a caller-provided buffer; everything
// else is the product kernel's code, compiled a second time in this translation unit (the product
// library is built without the macro and carries none of this).
#define ROCWMMA_AMD_PHASE_TRACE 1
#include "gemm_blocked_launch.hpp"

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        template <typename InT, bool AK, bool BK>
        int traced(GemmArgs const& g, unsigned long long* trace, hipStream_t stream)
        {
            // (the 256 x 256 configuration of gemm_blocked.hip for 16-bit types and int8)
            using Big = BlockedConfig<InT, std::conditional_t<std::is_same<InT, int8_t>::value, int32_t, float32_t>,
                                      std::conditional_t<std::is_same<InT, int8_t>::value, int32_t, float32_t>, AK, BK, 4, 2, 4, 8, 2, 2, 16>;
            TileExtras ex{};
            ex.trace = trace;
            return launchCfg<Big>(g, stream, ex);
        }

        template <typename InT>
        int tracedLayout(int layoutA, int layoutB, GemmArgs const& g, unsigned long long* trace, hipStream_t stream)
        {
            const bool ak = layoutA == ROCWMMA_AMD_ROW_MAJOR;
            const bool bk = layoutB == ROCWMMA_AMD_COL_MAJOR;
            if(ak && bk)
                return traced<InT, true, true>(g, trace, stream);
            if(ak && !bk)
                return traced<InT, true, false>(g, trace, stream);
            if(!ak && bk)
                return traced<InT, false, true>(g, trace, stream);
            return traced<InT, false, false>(g, trace, stream);
        }
    } // namespace

    // trace: (m / 256) * (n / 256) * 8 waves * 8 words of device memory
    int benchPhaseTrace(int dtypeIn, int layoutA, int layoutB, GemmArgs const& g, unsigned long long* trace, hipStream_t stream)
    {
        if(g.layoutC != ROCWMMA_AMD_ROW_MAJOR || g.m % 256u != 0u || g.n % 256u != 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        if(dtypeIn == ROCWMMA_AMD_F16)
            return tracedLayout<float16_t>(layoutA, layoutB, g, trace, stream);
        if(dtypeIn == ROCWMMA_AMD_BF16)
            return tracedLayout<bfloat16_t>(layoutA, layoutB, g, trace, stream);
        if(dtypeIn == ROCWMMA_AMD_I8)
            return tracedLayout<int8_t>(layoutA, layoutB, g, trace, stream);
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    }
} // namespace rocwmma_amd
