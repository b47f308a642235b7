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
//
// Three instruction kinds: v_mfma_f32_16x16x32_f16 (the 16-bit kernels), v_mfma_i32_16x16x64_i8 and
// v_mfma_f32_16x16x128_f8f6f4 (the 8-bit kernels).  The byte streams are the same for all three (128 bytes of K per
// row and stage, rows 16 KiB apart: for the 8-bit kinds the walked problem is 8192 x 8192 x 16384); per stage a wave
// issues 64 of the first two (two steps of 32) or 32 of the third, whose operands are the two 16-byte halves of a
// row's 128 bytes and whose B fragments stream through column buffers as in the kernel.
#include "common.hpp"
#include <rocwmma/rocwmma_lds.hpp>
#include <type_traits>

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        typedef float    f32x4 __attribute__((ext_vector_type(4)));

        constexpr uint32_t kProbeDim     = 8192; // the problem whose panels and tile order are walked
        constexpr uint32_t kProbeTile    = 256;
        constexpr uint32_t kProbeStageKB = 128; // bytes of K per stage
        constexpr uint32_t kProbeStages  = kProbeDim * 2u / kProbeStageKB; // 128 stages per tile
        constexpr uint32_t kProbeWaves   = 8;

        typedef int      i32x4 __attribute__((ext_vector_type(4)));
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));

        // Kind: 0 = f16 16x16x32, 1 = int8 16x16x64 (same operand shapes: 16 bytes per lane), 2 = fp8 16x16x128
        template <int Kind, typename Acc, typename Op>
        ROCWMMA_DEVICE ROCWMMA_INLINE void probeMfma(Acc& acc, Op const& x, Op const& y)
        {
#if defined(__HIP_DEVICE_COMPILE__)
            if constexpr(Kind == 0)
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(x), "v"(y));
            else if constexpr(Kind == 1)
                asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(acc) : "v"(x), "v"(y));
            else
                asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+v"(acc) : "v"(x), "v"(y));
#else
            (void)acc, (void)x, (void)y;
#endif
        }

        // the global -> LDS copies of one stage, spread over `Parts` calls (issuer waves only)
        template <uint32_t Parts, typename Tile>
        ROCWMMA_DEVICE ROCWMMA_INLINE void copyPart(uint32_t part, char* ldsStage, lds::BufferRsrc srcA, lds::BufferRsrc srcB,
                                                    uint32_t laneOff, uint32_t wave, uint32_t ldBytes)
        {
            constexpr uint32_t perOperand = Tile::copies / 4u; // per issuer wave
            constexpr uint32_t perPart    = 2u * perOperand / Parts;
#pragma unroll
            for(uint32_t c = 0; c < perPart; ++c)
            {
                const uint32_t idx  = part * perPart + c; // 0 .. 2 * perOperand - 1: A's copies, then B's
                const bool     isB  = idx >= perOperand;
                const uint32_t copy = (isB ? idx - perOperand : idx) * 4u + wave;
                lds::asyncCopy16(ldsStage + (isB ? Tile::bytes : 0u) + copy * 1024u, isB ? srcB : srcA, laneOff,
                                 Tile::copySourceOffset(copy, ldBytes));
            }
        }

        template <int Kind, bool Reads, bool Copies>
        __global__ void __launch_bounds__(kProbeWaves * 64u) __attribute__((amdgpu_waves_per_eu(2, 2)))
        mfmaStreamsKernel(const char* a, const char* b, const uint32_t* operands, float* out, uint32_t tilesPerWorkgroup)
        {
            using Tile = lds::KMajorTile<kProbeTile, kProbeStageKB>;
            using Acc  = std::conditional_t<Kind == 1, i32x4, f32x4>;
            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];
            constexpr uint32_t StageBytes = 2u * Tile::bytes; // A tile, B tile

            const uint32_t lane  = threadIdx.x & 63u;
            const uint32_t wave  = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t waveM = wave / 2u, waveN = wave % 2u; // 4 x 2 waves of 64 x 128

            // the LDS starts out holding operand bits of the caller's table (Reads without Copies reads these)
            for(uint32_t i = threadIdx.x; i < 2u * StageBytes / 4u; i += kProbeWaves * 64u)
                reinterpret_cast<uint32_t*>(ldsRaw)[i] = operands[i & 16383u];
            __syncthreads();

            Acc acc[4][8];
#pragma unroll
            for(uint32_t i = 0; i < 4u; ++i)
#pragma unroll
                for(uint32_t j = 0; j < 8u; ++j)
                    acc[i][j] = Acc{0, 0, 0, 0};

            constexpr uint32_t ldBytes = kProbeDim * 2u; // row pitch of the K-contiguous operands
            const uint32_t     laneOff = Tile::laneSourceOffset(lane, wave % 4u, ldBytes);
            // the tile the one-tile-per-workgroup launch would give this compute unit in round t
            auto panels = [&](uint32_t t, const char*& aSrc, const char*& bSrc) {
                const uint32_t tilesPerDim = kProbeDim / kProbeTile;
                const uint32_t wg          = t * gridDim.x + blockIdx.x;
                const uint32_t id          = (wg % 8u) * (tilesPerDim * tilesPerDim / 8u) + wg / 8u;
                const uint32_t panelIdx = id / (4u * tilesPerDim), inPanel = id % (4u * tilesPerDim);
                const uint32_t tm = panelIdx * 4u + inPanel % 4u, tn = inPanel / 4u;
                aSrc = a + static_cast<size_t>(tm) * kProbeTile * ldBytes;
                bSrc = b + static_cast<size_t>(tn) * kProbeTile * ldBytes;
            };

            if constexpr(Kind != 2)
            {
                // two steps per stage; the fragments of a step are read while the step before it is multiplied
                u32x4 fa[2][4], fb[2][8];
#pragma unroll
                for(uint32_t s = 0; s < 2u; ++s)
                {
#pragma unroll
                    for(uint32_t i = 0; i < 4u; ++i)
#pragma unroll
                        for(uint32_t w = 0; w < 4u; ++w)
                            fa[s][i][w] = operands[(threadIdx.x * 8u + 2048u * i + 512u * s + w) & 16383u];
#pragma unroll
                    for(uint32_t j = 0; j < 8u; ++j)
#pragma unroll
                        for(uint32_t w = 0; w < 4u; ++w)
                            fb[s][j][w] = operands[(threadIdx.x * 24u + 7816u * j + 40u + 304u * s + w) & 16383u];
                }
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
                            probeMfma<Kind>(acc[i][j], fb[set][j], fa[set][i]);
                };
                for(uint32_t t = 0; t < tilesPerWorkgroup; ++t)
                {
                    const char *aSrc, *bSrc;
                    panels(t, aSrc, bSrc);
                    for(uint32_t s = 0; s < kProbeStages; ++s)
                    {
                        readStep(1u, s % 2u, 1u);
                        multiply(0u);
                        __builtin_amdgcn_sched_barrier(0);
                        lds::waitCopiesAndReads<0u>(); // (the copies of the stage before: they have had a stage to land)
                        __builtin_amdgcn_sched_barrier(0);
                        if constexpr(Copies)
                        {
                            if(wave < 4u) // the first wave of each SIMD, for itself and its partner
                                copyPart<1u, Tile>(0u, ldsRaw + (s % 2u) * StageBytes,
                                                   lds::makeSource(aSrc + static_cast<size_t>(s) * kProbeStageKB),
                                                   lds::makeSource(bSrc + static_cast<size_t>(s) * kProbeStageKB), laneOff, wave, ldBytes);
                        }
                        readStep(0u, (s + 1u) % 2u, 0u);
                        multiply(1u);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            else
            {
                // one step per stage, operands of 32 bytes per lane (the two 16-byte halves of a row's 128 bytes).  The
                // A fragments of a stage are held whole and read a stage ahead into a second set; the B fragments
                // stream through three column buffers: while column j is multiplied, column j + 2 is read.
                u32x8 fa[2][4], fb[3];
#pragma unroll
                for(uint32_t w = 0; w < 8u; ++w)
                {
#pragma unroll
                    for(uint32_t s = 0; s < 2u; ++s)
#pragma unroll
                        for(uint32_t i = 0; i < 4u; ++i)
                            fa[s][i][w] = operands[(threadIdx.x * 8u + 2048u * i + 512u * s + w) & 16383u];
#pragma unroll
                    for(uint32_t j = 0; j < 3u; ++j)
                        fb[j][w] = operands[(threadIdx.x * 24u + 7816u * j + 40u + w) & 16383u];
                }
                auto readWide = [&](u32x8& f, const char* ldsTile, uint32_t row0) {
                    if constexpr(Reads)
                    {
                        Tile::template readBlock16<16u>(reinterpret_cast<u32x4*>(&f), ldsTile, row0, 0u, lane);
                        Tile::template readBlock16<16u>(reinterpret_cast<u32x4*>(&f) + 1, ldsTile, row0, 1u, lane);
                    }
                };
                auto stage = [&](auto parity, uint32_t s, const char* aSrc, const char* bSrc) {
                    constexpr uint32_t P    = decltype(parity)::value;
                    const char*        ldsB = ldsRaw + P * StageBytes + Tile::bytes;          // this stage's B tile
                    const char*        nxtA = ldsRaw + (1u - P) * StageBytes;                 // the next stage's tiles
                    const char*        nxtB = nxtA + Tile::bytes;
#pragma unroll
                    for(uint32_t j = 0; j < 8u; ++j)
                    {
                        const uint32_t ahead = j + 2u;
                        readWide(fb[ahead % 3u], ahead < 8u ? ldsB : nxtB, waveN * 128u + (ahead % 8u) * 16u);
                        if(j < 4u)
                            readWide(fa[1u - P][j], nxtA, waveM * 64u + j * 16u);
                        if constexpr(Copies)
                        {
                            if(j == 4u)
                                lds::waitCopiesAndReads<0u>(); // (the copies of the stage before)
                            if(j >= 4u && wave < 4u)
                                copyPart<4u, Tile>(j - 4u, ldsRaw + P * StageBytes,
                                                   lds::makeSource(aSrc + static_cast<size_t>(s) * kProbeStageKB),
                                                   lds::makeSource(bSrc + static_cast<size_t>(s) * kProbeStageKB), laneOff, wave, ldBytes);
                        }
#pragma unroll
                        for(uint32_t i = 0; i < 4u; ++i)
                            probeMfma<2>(acc[i][j], fb[j % 3u], fa[P][i]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                };
                for(uint32_t t = 0; t < tilesPerWorkgroup; ++t)
                {
                    const char *aSrc, *bSrc;
                    panels(t, aSrc, bSrc);
                    for(uint32_t s = 0; s < kProbeStages; s += 2u)
                    {
                        stage(std::integral_constant<uint32_t, 0u>{}, s, aSrc, bSrc);
                        stage(std::integral_constant<uint32_t, 1u>{}, s + 1u, aSrc, bSrc);
                    }
                }
            }
            lds::waitCopiesAndReads<0u>();
            float r = 0.0f;
#pragma unroll
            for(uint32_t i = 0; i < 4u; ++i)
#pragma unroll
                for(uint32_t j = 0; j < 8u; ++j)
                    r += static_cast<float>(acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3]);
            out[blockIdx.x * kProbeWaves * 64u + threadIdx.x] = r;
        }

        template <int Kind, bool Reads, bool Copies>
        int launchStreams(const void* a, const void* b, const void* operands, float* out, uint32_t tiles, hipStream_t stream)
        {
            auto               kernel = mfmaStreamsKernel<Kind, Reads, Copies>;
            constexpr uint32_t lds    = 2u * 2u * lds::KMajorTile<kProbeTile, kProbeStageKB>::bytes;
            if(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds))
               != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            hipLaunchKernelGGL(kernel, dim3(computeUnits()), dim3(kProbeWaves * 64u), lds, stream, static_cast<const char*>(a),
                               static_cast<const char*>(b), static_cast<const uint32_t*>(operands), out, tiles);
            return launchStatus();
        }

        template <int Kind>
        int launchKind(int streams, const void* a, const void* b, const void* operands, float* out, uint32_t tiles, hipStream_t stream)
        {
            switch(streams)
            {
            case 0:
                return launchStreams<Kind, false, false>(a, b, operands, out, tiles, stream);
            case 1:
                return launchStreams<Kind, true, false>(a, b, operands, out, tiles, stream);
            default:
                return launchStreams<Kind, true, true>(a, b, operands, out, tiles, stream);
            }
        }
    } // namespace

    // kind: 0 = f16 (16x16x32), 1 = int8 (16x16x64), 2 = fp8 e4m3 (16x16x128).
    // streams: bit 0 = fragments read from LDS, bit 1 = panels copied from global memory into LDS (needs bit 0).
    // a, b: 8192 rows of 16 KiB each, K contiguous (the copies walk them as the GEMM's tile order would: 8192 x 8192 halves,
    // or 8192 x 16384 bytes); operands: the 64 KiB table of operand bits (as for the matrix-pipe ceiling probe); out: one
    // float per launched lane.
    int benchMfmaStreams(int kind, int streams, uint32_t tilesPerWorkgroup, const void* a, const void* b, const void* operands,
                         float* out, double* ops, hipStream_t stream)
    {
        if(kind < 0 || kind > 2 || streams < 0 || streams > 3 || streams == 2 || tilesPerWorkgroup == 0u || !operands || !out
           || (streams == 3 && (!a || !b)))
            return ROCWMMA_AMD_INVALID_ARGUMENT;
        const uint32_t units = computeUnits();
        if(static_cast<uint64_t>(tilesPerWorkgroup) * units > (kProbeDim / kProbeTile) * (kProbeDim / kProbeTile) || units % 8u != 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        if(ops) // (K of the walked problem: 16 KiB per row)
            *ops = 2.0 * kProbeTile * kProbeTile * (kind == 0 ? kProbeDim : 2u * kProbeDim) * static_cast<double>(tilesPerWorkgroup) * units;
        switch(kind)
        {
        case 0:
            return launchKind<0>(streams, a, b, operands, out, tilesPerWorkgroup, stream);
        case 1:
            return launchKind<1>(streams, a, b, operands, out, tilesPerWorkgroup, stream);
        default:
            return launchKind<2>(streams, a, b, operands, out, tilesPerWorkgroup, stream);
        }
    }
} // namespace rocwmma_amd
