// Matrix pipes next to their operand streams (benchmark support, part of the auxiliary library).
//
// The ceiling of mfma_ceiling.hip is a loop of nothing but matrix instructions.  A blocked GEMM cannot run
// that loop: per 64 of K a 256 x 256 tile of 16-bit operands needs 64 KiB copied from the L2s into LDS and
// (with 64 x 128 wave tiles) 192 KiB read from LDS into registers, and on a power-managed part those bytes cost
// clock.  This probe runs the matrix instructions of such a tile next to exactly these streams and nothing else:
// one workgroup of eight waves per compute unit, every wave issuing per stage its 64 v_mfma_f32_16x16x32_f16 on
// fragments it reads from the LDS stages (24 conflict-free 16-byte reads, the K-major stage layout of
// rocwmma_lds.hpp), the first wave of each SIMD issuing the stage's 16 one-KiB global -> LDS copies of the A and
// B panels the tile order of an 8192 x 8192 x 8192 problem gives the workgroup.  There is no barrier, no tile
// bookkeeping and no epilogue, and nothing is computed that anybody checks: what it sustains is what
// the device delivers for the tile's instruction and byte mix, an upper bound for any kernel with that tiling.
// Each stream can be switched off, which prices it.
#include "common.hpp"
#include <rocwmma/rocwmma_lds.hpp>

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        typedef float    f32x4 __attribute__((ext_vector_type(4)));
        typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

        constexpr uint32_t kProbeDim     = 8192; // the problem whose panels and tile order are walked
        constexpr uint32_t kProbeTile    = 256;
        constexpr uint32_t kProbeStageKB = 128; // bytes of K per stage
        constexpr uint32_t kProbeStages  = kProbeDim * 2u / kProbeStageKB; // 128 stages per tile
        constexpr uint32_t kProbeWaves   = 8;

#if defined(__HIP_DEVICE_COMPILE__)
#define ROCWMMA_AMD_PROBE_MFMA(ACC, A, B) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(ACC) : "v"(A), "v"(B))
#else
#define ROCWMMA_AMD_PROBE_MFMA(ACC, A, B) (void)(A), (void)(B)
#endif

        template <bool Reads, bool Copies>
        __global__ void __launch_bounds__(kProbeWaves * 64u) __attribute__((amdgpu_waves_per_eu(2, 2)))
        mfmaStreamsKernel(const char* a, const char* b, const uint32_t* operands, float* out, uint32_t tilesPerWorkgroup)
        {
            using Tile = lds::KMajorTile<kProbeTile, kProbeStageKB>;
            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];
            constexpr uint32_t StageBytes = 2u * Tile::bytes; // A tile, B tile

            const uint32_t lane  = threadIdx.x & 63u;
            const uint32_t wave  = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t waveM = wave / 2u, waveN = wave % 2u; // 4 x 2 waves of 64 x 128

            // the LDS starts out holding operand bits of the caller's table (Reads without Copies reads these)
            for(uint32_t i = threadIdx.x; i < 2u * StageBytes / 4u; i += kProbeWaves * 64u)
                reinterpret_cast<uint32_t*>(ldsRaw)[i] = operands[i & 16383u];
            __syncthreads();

            f16x8 fa[2][4], fb[2][8];
#pragma unroll
            for(uint32_t s = 0; s < 2u; ++s)
            {
#pragma unroll
                for(uint32_t i = 0; i < 4u; ++i)
#pragma unroll
                    for(uint32_t w = 0; w < 4u; ++w)
                        reinterpret_cast<uint32_t*>(&fa[s][i])[w] = operands[(threadIdx.x * 8u + 2048u * i + 512u * s + w) & 16383u];
#pragma unroll
                for(uint32_t j = 0; j < 8u; ++j)
#pragma unroll
                    for(uint32_t w = 0; w < 4u; ++w)
                        reinterpret_cast<uint32_t*>(&fb[s][j])[w] = operands[(threadIdx.x * 24u + 7816u * j + 40u + 304u * s + w) & 16383u];
            }
            f32x4 acc[4][8];
#pragma unroll
            for(uint32_t i = 0; i < 4u; ++i)
#pragma unroll
                for(uint32_t j = 0; j < 8u; ++j)
                    acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

            auto readStep = [&](uint32_t set, uint32_t slot, uint32_t ks) {
                if constexpr(Reads)
                {
                    const char* ldsA = ldsRaw + slot * StageBytes;
                    const char* ldsB = ldsA + Tile::bytes;
#pragma unroll
                    for(uint32_t i = 0; i < 4u; ++i)
                        Tile::template readBlock16<16u>(&fa[set][i], ldsA, waveM * 64u + i * 16u, ks, lane);
#pragma unroll
                    for(uint32_t j = 0; j < 8u; ++j)
                        Tile::template readBlock16<16u>(&fb[set][j], ldsB, waveN * 128u + j * 16u, ks, lane);
                }
            };
            auto multiply = [&](uint32_t set) {
#pragma unroll
                for(uint32_t i = 0; i < 4u; ++i)
#pragma unroll
                    for(uint32_t j = 0; j < 8u; ++j)
                        ROCWMMA_AMD_PROBE_MFMA(acc[i][j], fb[set][j], fa[set][i]);
            };
            constexpr uint32_t ldBytes = kProbeDim * 2u; // row pitch of the K-contiguous operands
            const uint32_t     laneOff = Tile::laneSourceOffset(lane, wave % 4u, ldBytes);

            for(uint32_t t = 0; t < tilesPerWorkgroup; ++t)
            {
                // the tile the one-tile-per-workgroup launch would give this compute unit in round t
                const uint32_t tilesPerDim = kProbeDim / kProbeTile;
                const uint32_t wg          = t * gridDim.x + blockIdx.x;
                const uint32_t id          = (wg % 8u) * (tilesPerDim * tilesPerDim / 8u) + wg / 8u;
                const uint32_t panelIdx = id / (4u * tilesPerDim), inPanel = id % (4u * tilesPerDim);
                const uint32_t tm = panelIdx * 4u + inPanel % 4u, tn = inPanel / 4u;
                const char*    aSrc = a + static_cast<size_t>(tm) * kProbeTile * ldBytes;
                const char*    bSrc = b + static_cast<size_t>(tn) * kProbeTile * ldBytes;
                for(uint32_t s = 0; s < kProbeStages; ++s)
                {
                    readStep(1u, s % 2u, 1u);
                    multiply(0u);
                    __builtin_amdgcn_sched_barrier(0);
                    lds::waitCopiesAndReads<0u>();
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr(Copies)
                    {
                        if(wave < 4u) // the first wave of each SIMD, for itself and its partner
                        {
                            const lds::BufferRsrc srcA = lds::makeSource(aSrc + static_cast<size_t>(s) * kProbeStageKB);
                            const lds::BufferRsrc srcB = lds::makeSource(bSrc + static_cast<size_t>(s) * kProbeStageKB);
                            char* const           dstA = ldsRaw + (s % 2u) * StageBytes;
#pragma unroll
                            for(uint32_t i = 0; i < Tile::copies / 4u; ++i)
                            {
                                const uint32_t copy = i * 4u + wave;
                                lds::asyncCopy16(dstA + copy * 1024u, srcA, laneOff, Tile::copySourceOffset(copy, ldBytes));
                            }
#pragma unroll
                            for(uint32_t i = 0; i < Tile::copies / 4u; ++i)
                            {
                                const uint32_t copy = i * 4u + wave;
                                lds::asyncCopy16(dstA + Tile::bytes + copy * 1024u, srcB, laneOff, Tile::copySourceOffset(copy, ldBytes));
                            }
                        }
                    }
                    readStep(0u, (s + 1u) % 2u, 0u);
                    multiply(1u);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            lds::waitCopiesAndReads<0u>();
            float r = 0.0f;
#pragma unroll
            for(uint32_t i = 0; i < 4u; ++i)
#pragma unroll
                for(uint32_t j = 0; j < 8u; ++j)
                    r += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
            out[blockIdx.x * kProbeWaves * 64u + threadIdx.x] = r;
        }
#undef ROCWMMA_AMD_PROBE_MFMA

        template <bool Reads, bool Copies>
        int launchStreams(const void* a, const void* b, const void* operands, float* out, uint32_t tiles, hipStream_t stream)
        {
            auto               kernel = mfmaStreamsKernel<Reads, Copies>;
            constexpr uint32_t lds    = 2u * 2u * lds::KMajorTile<kProbeTile, kProbeStageKB>::bytes;
            if(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds))
               != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            hipLaunchKernelGGL(kernel, dim3(computeUnits()), dim3(kProbeWaves * 64u), lds, stream, static_cast<const char*>(a),
                               static_cast<const char*>(b), static_cast<const uint32_t*>(operands), out, tiles);
            return launchStatus();
        }
    } // namespace

    // streams: bit 0 = fragments read from LDS, bit 1 = panels copied from global memory into LDS (needs bit 0).
    // a, b: 8192 x 8192 halves each, K contiguous (the copies walk them as the GEMM's tile order would); operands: the
    // 64 KiB table of operand bits (as for the matrix-pipe ceiling probe); out: one float per launched lane.
    int benchMfmaStreams(int streams, uint32_t tilesPerWorkgroup, const void* a, const void* b, const void* operands, float* out,
                         double* ops, hipStream_t stream)
    {
        if(streams < 0 || streams > 3 || streams == 2 || tilesPerWorkgroup == 0u || !operands || !out || (streams == 3 && (!a || !b)))
            return ROCWMMA_AMD_INVALID_ARGUMENT;
        const uint32_t units = computeUnits();
        if(static_cast<uint64_t>(tilesPerWorkgroup) * units > (kProbeDim / kProbeTile) * (kProbeDim / kProbeTile) || units % 8u != 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        if(ops)
            *ops = 2.0 * kProbeTile * kProbeTile * kProbeDim * static_cast<double>(tilesPerWorkgroup) * units;
        switch(streams)
        {
        case 0:
            return launchStreams<false, false>(a, b, operands, out, tilesPerWorkgroup, stream);
        case 1:
            return launchStreams<true, false>(a, b, operands, out, tilesPerWorkgroup, stream);
        default:
            return launchStreams<true, true>(a, b, operands, out, tilesPerWorkgroup, stream);
        }
    }
} // namespace rocwmma_amd
