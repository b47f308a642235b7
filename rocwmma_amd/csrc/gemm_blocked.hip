// Blocked GEMM for gfx950, one macro tile per workgroup: tile ladder and dispatch.  The device side
// (configuration, LDS pipeline, epilogue) is in gemm_blocked_core.hpp, the kernels and launch helpers in
// gemm_blocked_launch.hpp.
#include "gemm_blocked_launch.hpp"

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        // Tile ladder: the 256 x 256 macro tile when the problem divides into enough of them to occupy
        // at least half of the compute units, else 128 x 128; when that gives at most one tile per two
        // compute units (few token rows against a wide weight matrix), 128 x 64 tiles double the
        // number of workgroups.
        template <typename InT, typename OutT, typename CompT, bool AK, bool BK>
        int pickTile(GemmArgs const& g, hipStream_t stream, bool forceLargeTile)
        {
            // 256 x 256 macro tile, 8 waves of 64 x 128.  16-bit and int8 operands use 16-wide blocks
            // (16x16x32 / 16x16x64 instructions: half the accumulator traffic per flop of the
            // 32-wide forms, which is worth 5-7 % under the power cap).
            // fp8 with both operands K-contiguous uses 16x16x128 (its fragments streamed column by column:
            // the matrix pipes sustain 6 % more on it than on 32x32x64, the kernel gains 1.5-3 %); the other fp8 layouts use 32x32x64.
            static constexpr bool Edge16 = sizeof(InT) == 2u || std::is_same<InT, int8_t>::value || (AK && BK);
            // Ring of two stages of 128 bytes of K: a copy instruction then requests whole 128-byte lines
            // of a K-contiguous operand (half as many requests to the L2 as with 64-byte stage rows);
            // against the ring of four 64-byte stages 8192^3 runs 1-5 % faster for f16 / bf16 in every
            // layout pair and 6 % faster for int8 and fp8.
            using Big    = std::conditional_t<Edge16,
                                              BlockedConfig<InT, OutT, CompT, AK, BK, 4, 2, 4, 8, 2, 2, 16>,
                                              BlockedConfig<InT, OutT, CompT, AK, BK, 4, 2, 2, 4, 2, 2, 32>>;
            // (the 4-wave configurations declare the occupancy their LDS use allows, two and three
            // workgroups per compute unit: the compiler pads the register count of a kernel that
            // declares one wave per SIMD so that no second workgroup fits, and problems with more
            // tiles than compute units then ran in whole rounds: 512 x 14336 x 4096 f16 90 -> 77 us,
            // 256 x 14336 x 4096 fp8 36 -> 30 us)
            using Small  = BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 2, 4, 2>;
            // the same tiles on the ring of two 128-byte stages, for more than one workgroup per
            // compute unit (see launchByRounds)
            using Small2 = BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 2, 2, 2>;
            // (a 256 x 256 tiling that covers less than half of the compute units loses to 128 x 128
            // tiles: 2048^3 f16 47 -> 24 us, 1024^3 30 -> 9 us, 512 x 14336 x 4096 int8 51 -> 42 us;
            // from 144 tiles on 256 units the large tile wins again)
            // the same rows and pipeline with half the columns, for the tiles of a last round that would be
            // at most half full (launchSplitTail)
            using BigHalf = std::conditional_t<Edge16,
                                               BlockedConfig<InT, OutT, CompT, AK, BK, 4, 2, 4, 4, 2, 2, 16>,
                                               BlockedConfig<InT, OutT, CompT, AK, BK, 4, 2, 2, 2, 2, 2, 32>>;
            if(g.m % Big::MacroM == 0u && g.n % Big::MacroN == 0u
               && (forceLargeTile || 2u * (g.m / Big::MacroM) * (g.n / Big::MacroN) >= computeUnits()))
            {
                int rc = forceLargeTile ? ROCWMMA_AMD_UNSUPPORTED_SHAPE : launchSplitTail<Big, BigHalf>(g, stream);
                if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                    return rc;
                rc = launchCfg<Big>(g, stream);
                if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                    return rc;
            }
            if(forceLargeTile)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            if constexpr(AK && BK)
            {
                // small problems, at most one 128 x 128 tile per four compute units: 64 x 64 tiles put
                // four times as many workgroups to work (512 x 512 x 4096 int8 13 -> 11 us,
                // 256 x 256 x 8192 f16 45 -> 40 us)
                using Tiny0 = BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 1, 1, 4, 4>;
                if(g.m % Small::MacroM == 0u && g.n % Small::MacroN == 0u
                   && 4u * (g.m / Small::MacroM) * (g.n / Small::MacroN) <= computeUnits())
                {
                    int rc = launchCfg<Tiny0>(g, stream);
                    if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                        return rc;
                }
                using Narrow = BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 1, 4, 3>;
                // The same 128 x 64 tile on a ring of four stages of 128 bytes of K (96 KiB of LDS, one
                // workgroup per compute unit): a copy requests whole lines, and three stages of 24 KiB are in
                // flight.  These launches are one round of workgroups that stream their operands from HBM:
                // 128 x 14336 x 4096 int8 25.1 -> 19.2 us, fp8 27.3 -> 19.5, 256 x 8192 x 8192 int8 41.5 -> 30.9,
                // f16 74 -> 56; f16 / bf16 128 x 14336 x 4096 within 3 %.  With little K the deeper prologue
                // costs more than it gains (128 x 14336 x 384 f16 7.0 -> 8.8 us), so from 2 KiB of K per row on.
                // 16-wide blocks (two MFMA steps per stage) except for fp8, whose 16 x 16 x 128 needs the ring of
                // two.  (A ring of five: the same.  128 x 128 tiles on this ring, one workgroup per compute
                // unit, lose to the two-workgroup configurations below: 2048^3 f16 +6 %, 128 x 28672 x 4096 +12 %.)
                constexpr bool Fp8 = sizeof(InT) == 1u && !std::is_same<InT, int8_t>::value;
                using NarrowLines = std::conditional_t<!Fp8,
                                                       BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 4, 2, 4, 1, 16, false, false, false, 128>,
                                                       BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 1, 4, 1, 32, false, false, false, 128>>;
                // (up to one 128 x 128 tile per two compute units; with two resident workgroups per
                // compute unit the 128 x 128 tiling wins from 144 tiles on, fewer bytes per compute
                // unit: 256 x 14336 x 4096 int8 30 -> 24 us, f16 73 -> 52 us)
                if(g.m % Small::MacroM == 0u && g.n % Small::MacroN == 0u
                   && 2u * (g.m / Small::MacroM) * (g.n / Small::MacroN) <= computeUnits())
                {
                    int rc = static_cast<size_t>(g.k) * sizeof(InT) >= 2048u ? launchCfg<NarrowLines>(g, stream) : ROCWMMA_AMD_UNSUPPORTED_SHAPE;
                    if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                        return rc;
                    rc = launchCfg<Narrow>(g, stream);
                    if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                        return rc;
                }
            }
            else if constexpr(AK != BK)
            {
                // one operand dim-major: its LDS tile is at least 128 wide, the other side may be 64
                // (128 x 64 tiles with a K-contiguous B, 64 x 128 with a K-contiguous A)
                using Half = std::conditional_t<BK, BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 1, 4, 3>,
                                                BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 1, 2, 4, 3>>;
                // The same tiles on the ring of four 128-byte stages (see NarrowLines above) for the 8-bit types with
                // at least 4 KiB of K per row: 128 x 14336 x 4096 int8 27.5 -> 24.8 us (A row / B row) and 24.8 -> 22.5
                // (A col / B col), fp8 28.6 -> 24.0 and 26.1 -> 18.6, 256 x 8192 x 8192 int8 41.8 -> 37.6 and 41.5 ->
                // 36.9.  (f16 / bf16: between 6 % faster and 11 % slower, left on the 64-byte ring; 2 KiB of K: up to
                // 9 % slower.)
                constexpr bool Fp8h = sizeof(InT) == 1u && !std::is_same<InT, int8_t>::value;
                using HalfLines = std::conditional_t<
                    BK,
                    std::conditional_t<!Fp8h, BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 4, 2, 4, 1, 16, false, false, false, 128>,
                                       BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 1, 4, 1, 32, false, false, false, 128>>,
                    std::conditional_t<!Fp8h, BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 4, 4, 1, 16, false, false, false, 128>,
                                       BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 1, 2, 4, 1, 32, false, false, false, 128>>>;
                if(g.m % Small::MacroM == 0u && g.n % Small::MacroN == 0u
                   && 2u * (g.m / Small::MacroM) * (g.n / Small::MacroN) <= computeUnits())
                {
                    if constexpr(sizeof(InT) == 1u)
                    {
                        const int rcl = g.k >= 4096u ? launchCfg<HalfLines>(g, stream) : ROCWMMA_AMD_UNSUPPORTED_SHAPE;
                        if(rcl != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                            return rcl;
                    }
                    int rc = launchCfg<Half>(g, stream);
                    if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                        return rc;
                }
            }
            // fp8, both operands K-contiguous, one round of more than half as many 128 x 128 tiles as there are
            // compute units, at least 4 KiB of K: the tile on the ring of four 128-byte stages (128 KiB of LDS, one
            // workgroup per compute unit).  256 x 14336 x 4096 30.9 -> 25.5 us, 2048 x 2048 x 4096 26.2 -> 23.0,
            // 256 x 16384 x 8192 53.7 -> 42.7, 128 x 28672 x 4096 27.0 -> 24.6; with more tiles than compute units it loses to
            // the two-workgroup ring of two, 512 x 14336 x 4096 43.6 -> 48.1.  (int8 and the 16-bit types, whose
            // 32-wide blocks would make four MFMA steps of such a stage, ran it with 16-wide blocks: int8 3 %
            // faster to 12 % slower, f16 6-12 % slower; they stay on the 64-byte ring.)
            if constexpr(AK && BK && sizeof(InT) == 1u && !std::is_same<InT, int8_t>::value)
            {
                using SmallLines = BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 2, 4, 1, 32, false, false, false, 128>;
                if(g.m % Small::MacroM == 0u && g.n % Small::MacroN == 0u && g.k >= 4096u
                   && (g.m / Small::MacroM) * (g.n / Small::MacroN) <= computeUnits()
                   && 2u * (g.m / Small::MacroM) * (g.n / Small::MacroN) > computeUnits())
                {
                    int rc = launchCfg<SmallLines>(g, stream);
                    if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                        return rc;
                }
            }
            {
                int rc = launchByRounds<Small, Small2>(g, stream);
                if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                    return rc;
            }
            // Fewer rows than a whole 128 x 64 tile (and other multiples of 16 that leave one partly filled row of
            // tiles): the same ring of four 128-byte stages with partly filled tiles, when that is one round of
            // workgroups with enough K to stream.  The rows that are not there cost matrix instructions, not
            // bytes: 64 x 14336 x 4096 int8 22.1 -> 18.2 us, fp8 24.3 -> 16.4; 96 rows int8 27.0 -> 18.7, fp8
            // 29.0 -> 17.1, f16 37.8 -> 30.1; 64 x 8192 x 8192 f16 69 -> 55.  Not below 4 KiB of K per row
            // (64 x 14336 x 2048 int8 9.2 -> 10.1 us), and 16-bit types with up to 64 rows only from 16 KiB
            // (64 x 14336 x 4096 f16 27.8 -> 31.7 us on it).
            if constexpr(AK && BK)
            {
                constexpr bool Fp8e = sizeof(InT) == 1u && !std::is_same<InT, int8_t>::value;
                using NarrowLinesEdge = std::conditional_t<!Fp8e,
                                                           BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 4, 2, 4, 1, 16, true, false, false, 128>,
                                                           BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 1, 4, 1, 32, true, false, false, 128>>;
                static_assert(NarrowLinesEdge::MacroM == 128u && NarrowLinesEdge::MacroN == 64u, "gemmBlockedTakesPartlyFilledLineTiles");
                if(gemmBlockedTakesPartlyFilledLineTiles(g.m, g.n, g.k, sizeof(InT)))
                {
                    int rc = launchCfg<NarrowLinesEdge>(g, stream);
                    if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                        return rc;
                }
            }
            // multiples of 64 that are not multiples of 128: 64 x 64 tiles, one 32 x 32 block per wave
            // (K-contiguous operands only: the dim-major LDS tile is at least 128 wide)
            if constexpr(AK && BK)
            {
                using Tiny  = BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 1, 1, 4, 4>;
                using Tiny2 = BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 1, 1, 2, 4>;
                int rc      = launchByRounds<Tiny, Tiny2>(g, stream);
                if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                    return rc;
            }
            // any other multiples of 16: 128 x 128 tiles, the last row and column of tiles partly
            // filled (the wave-tile kernel, which these shapes used to fall to, is 2-3x slower)
            using Edge  = BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 2, 4, 2, 32, true>;
            using Edge2 = BlockedConfig<InT, OutT, CompT, AK, BK, 2, 2, 2, 2, 2, 2, 32, true>;
            return launchByRounds<Edge, Edge2>(g, stream);
        }

        template <typename InT, typename OutT, typename CompT>
        int pickLayout16(int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream, bool big)
        {
            const bool ak = layoutA == ROCWMMA_AMD_ROW_MAJOR;
            const bool bk = layoutB == ROCWMMA_AMD_COL_MAJOR;
            if(ak && bk)
                return pickTile<InT, OutT, CompT, true, true>(g, stream, big);
            if(ak && !bk)
                return pickTile<InT, OutT, CompT, true, false>(g, stream, big);
            if(!ak && bk)
                return pickTile<InT, OutT, CompT, false, true>(g, stream, big);
            return pickTile<InT, OutT, CompT, false, false>(g, stream, big);
        }

        template <typename InT, typename OutT, typename CompT>
        int pickLayout8(int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream, bool big)
        {
            const bool ak = layoutA == ROCWMMA_AMD_ROW_MAJOR;
            const bool bk = layoutB == ROCWMMA_AMD_COL_MAJOR;
            if(ak && bk)
                return pickTile<InT, OutT, CompT, true, true>(g, stream, big);
            if(ak && !bk)
                return pickTile<InT, OutT, CompT, true, false>(g, stream, big);
            if(!ak && bk)
                return pickTile<InT, OutT, CompT, false, true>(g, stream, big);
            return pickTile<InT, OutT, CompT, false, false>(g, stream, big);
        }
    } // namespace

    namespace
    {
        template <typename InT>
        int launchMx(GemmArgs const& g, TileExtras const& ex, hipStream_t stream)
        {
            // 256 x 256 tiles of 16x16x128 blocks with block scales; the tiles of a last round at most half
            // full run as 256 x 128 half tiles, as in the unscaled kernel
            using Big     = BlockedConfig<InT, float32_t, float32_t, true, true, 4, 2, 4, 8, 2, 2, 16, false, true>;
            using BigHalf = BlockedConfig<InT, float32_t, float32_t, true, true, 4, 2, 4, 4, 2, 2, 16, false, true>;
            const int rc  = launchSplitTail<Big, BigHalf>(g, stream, ex);
            if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                return rc;
            return launchCfg<Big>(g, stream, ex);
        }
    } // namespace

    namespace
    {
        template <typename InT>
        int launchMxMid(GemmArgs const& g, TileExtras const& ex, hipStream_t stream)
        {
            // 128 x 128 tiles of 32x32x64 blocks with block scales, the last row and column of tiles partly
            // filled: any m, n in multiples of 16
            using Mid = BlockedConfig<InT, float32_t, float32_t, true, true, 2, 2, 2, 2, 2, 2, 32, true, true>;
            // at most one 128 x 128 tile per two compute units (few token rows against a wide weight matrix):
            // 128 x 64 tiles put twice as many workgroups to work
            using Narrow = BlockedConfig<InT, float32_t, float32_t, true, true, 2, 2, 2, 1, 2, 3, 32, true, true>;
            // One round of 128 x 64 tiles with at least 4 KiB of K per row: the tile on the ring of four 128-byte
            // stages (whole-line requests, three stages in flight), as for the unscaled types (NarrowLinesEdge
            // above): 128 x 14336 x 4096 31 -> 21 us on scales packed beforehand.
            using NarrowLines = BlockedConfig<InT, float32_t, float32_t, true, true, 2, 2, 2, 1, 4, 1, 32, true, true, false, 128>;
            if(gemmBlockedTakesPartlyFilledLineTiles(g.m, g.n, g.k, 1u))
            {
                const int rc = launchCfg<NarrowLines>(g, stream, ex);
                if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                    return rc;
            }
            if(2u * ceilDiv(g.m, 128u) * ceilDiv(g.n, 128u) <= computeUnits())
                return launchCfg<Narrow>(g, stream, ex);
            return launchCfg<Mid>(g, stream, ex);
        }
    } // namespace

    bool gemmBlockedTakesPartlyFilledLineTiles(uint32_t m, uint32_t n, uint32_t k, uint32_t elemBytes)
    {
        const uint32_t tiles  = ceilDiv(m, 128u) * ceilDiv(n, 64u);
        const size_t   kBytes = static_cast<size_t>(k) * elemBytes;
        const size_t   minK   = (elemBytes == 2u && m <= 64u) ? 16384u : 4096u;
        return kBytes % 128u == 0u && kBytes >= minK && tiles <= computeUnits() && 4u * tiles > computeUnits();
    }

    bool gemmMxBlockedUsesLargeTile(GemmArgs const& g)
    {
        return g.m % 256u == 0u && g.n % 256u == 0u && 2u * (g.m / 256u) * (g.n / 256u) >= computeUnits();
    }

    int launchGemmMxBlocked(int dtypeIn, GemmArgs const& g, const void* packedA, const void* packedB, hipStream_t stream)
    {
        if(g.layoutC != ROCWMMA_AMD_ROW_MAJOR || g.m % 16u != 0u || g.n % 16u != 0u || g.k % 128u != 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        TileExtras ex{};
        ex.mx = MxPacked{packedA, packedB, (g.k / 128u + 1u) / 2u};
        const bool large = gemmMxBlockedUsesLargeTile(g);
        if(dtypeIn == ROCWMMA_AMD_E4M3)
            return large ? launchMx<float8_t>(g, ex, stream) : launchMxMid<float8_t>(g, ex, stream);
        if(dtypeIn == ROCWMMA_AMD_E5M2)
            return large ? launchMx<bfloat8_t>(g, ex, stream) : launchMxMid<bfloat8_t>(g, ex, stream);
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    }

    int launchGemmBlocked(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream,
                          bool forceLargeTile)
    {
        if(g.layoutC != ROCWMMA_AMD_ROW_MAJOR)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE; // caller transposes the problem first
        if(dtypeIn == ROCWMMA_AMD_F16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout16<float16_t, float32_t, float32_t>(layoutA, layoutB, g, stream, forceLargeTile);
        if(dtypeIn == ROCWMMA_AMD_BF16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout16<bfloat16_t, float32_t, float32_t>(layoutA, layoutB, g, stream, forceLargeTile);
        if(dtypeIn == ROCWMMA_AMD_F16 && dtypeOut == ROCWMMA_AMD_F16)
            return pickLayout16<float16_t, float16_t, float32_t>(layoutA, layoutB, g, stream, forceLargeTile);
        if(dtypeIn == ROCWMMA_AMD_BF16 && dtypeOut == ROCWMMA_AMD_BF16)
            return pickLayout16<bfloat16_t, bfloat16_t, float32_t>(layoutA, layoutB, g, stream, forceLargeTile);
        if(dtypeIn == ROCWMMA_AMD_I8 && dtypeOut == ROCWMMA_AMD_I32)
            return pickLayout8<int8_t, int32_t, int32_t>(layoutA, layoutB, g, stream, forceLargeTile);
        if(dtypeIn == ROCWMMA_AMD_I8 && dtypeOut == ROCWMMA_AMD_I8)
            return pickLayout8<int8_t, int8_t, int32_t>(layoutA, layoutB, g, stream, forceLargeTile);
        if(dtypeIn == ROCWMMA_AMD_E4M3 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout8<float8_t, float32_t, float32_t>(layoutA, layoutB, g, stream, forceLargeTile);
        if(dtypeIn == ROCWMMA_AMD_E5M2 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayout8<bfloat8_t, float32_t, float32_t>(layoutA, layoutB, g, stream, forceLargeTile);
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    }

} // namespace rocwmma_amd
