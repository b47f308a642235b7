// Fragment-to-register maps for gfx950 (CDNA4) matrix cores.
//
// This header is plain constexpr C++ (no HIP) so the maps can be enumerated and checked on
// the host.  It answers one question: which matrix element does register element `e` of
// lane `l` hold, for each kind of fragment?
//
// Design (differs on purpose from rocWMMA's layout-dependent register formats,
// reference: library/include/rocwmma/internal/io_layout.hpp:39-308 and layout/*):
//
//  * The register layout of a fragment depends on (context, BlockM, BlockN, BlockK, element
//    size) only -- never on the in-memory data layout.  Fragments are always held in the
//    order the MFMA instruction consumes, so mma_sync needs no shuffles, applyDataLayout and
//    applyTranspose are free, and accumulator fragments of different element types or layout
//    tags agree element by element.
//
//  * Input fragments (matrix_a: BlockDim=BlockM rows x BlockK; matrix_b: BlockK x
//    BlockDim=BlockN columns; described here in the A orientation, "dim" index x k index):
//        tile   = 32 if BlockM and BlockN are multiples of 32, else 16   (MFMA edge)
//        groups = 64 / tile                                              (lane groups along K)
//        kpack  = elements each lane holds per MFMA (contiguous in K)
//        kstep  = kpack * groups                                         (K extent of one MFMA)
//      element e = (db * nk + ks) * kpack + j   holds
//        dim = db * tile + lane % tile
//        k   = ks * kstep + (lane / tile) * kpack + j
//    which is exactly the operand layout of v_mfma_*_16x16x{16,32,64} / v_mfma_*_32x32x{8,16,32}:
//    one lane = one row (column) and a contiguous run of K.  The fp8 wide-K instructions
//    (16x16x128 / 32x32x64) take two consecutive K steps of 16-byte runs in one go (mmaSteps = 2).
//
//  * Accumulators are held TRANSPOSED with respect to the MFMA result (mma_sync swaps the
//    two multiplicands), so that a lane owns runs of 4 consecutive columns of one row:
//        tile 16: e = (bi * nbj + bj) * 4 + i      row = bi*16 + lane%16
//                                                  col = bj*16 + (lane/16)*4 + i
//        tile 32: e = (bi * nbj + bj) * 16 + i     row = bi*32 + lane%32
//                                                  col = bj*32 + 8*(i/4) + (lane/32)*4 + i%4
//    Row-major C/D tiles therefore move with 16-byte vector accesses.  (64-bit accumulators differ:
//    see AccMapStrided.)
#ifndef ROCWMMA_FRAGMENT_MAP_HPP
#define ROCWMMA_FRAGMENT_MAP_HPP

#include <cstdint>

namespace rocwmma
{
    namespace detail
    {
        constexpr uint32_t kWaveSize = 64u;

        // Operand class as far as the K packing rules care.
        enum class PackClass : uint32_t
        {
            Bits16, // f16, bf16
            Fp8, // e4m3, e5m2
            Int8,
            Bits32, // f32 inputs
            Other // 64-bit etc: load / store only
        };

        constexpr uint32_t mmaTileDim(uint32_t blockM, uint32_t blockN)
        {
            return (blockM % 32u == 0u && blockN % 32u == 0u) ? 32u : 16u;
        }

        // Blocks with an edge of 8 have no matrix instruction; they exist for load / store / fill
        // only (the reference's unit tests move 32..256 x 8 blocks, test/unit/unit_test_params.hpp:
        // 104-141).  Inputs: the 64 lanes form 8 rows x 8 lane groups along K.  Accumulators:
        // 32-row x 8-column tiles, one 4-column run per lane.
        constexpr uint32_t inputTileDim(uint32_t blockM, uint32_t blockN, uint32_t blockDim)
        {
            return blockDim % 16u == 0u ? mmaTileDim(blockM, blockN) : 8u;
        }
        constexpr uint32_t accTileRows(uint32_t blockM, uint32_t blockN)
        {
            return blockN % 16u == 0u ? mmaTileDim(blockM, blockN) : 32u;
        }

        // Largest per-lane K run (elements) for which an MFMA exists, given the class.
        constexpr uint32_t maxKPack(PackClass c)
        {
            switch(c)
            {
            case PackClass::Bits16:
                return 8u; // v_mfma_f32_16x16x32_f16 / 32x32x16: 8 halves per lane
            case PackClass::Fp8:
                return 32u; // v_mfma_f32_16x16x128_f8f6f4 / 32x32x64: 32 bytes per lane (two runs of 16)
            case PackClass::Int8:
                return 16u; // v_mfma_i32_16x16x64_i8 / 32x32x32: 16 bytes per lane
            default:
                return 1u;
            }
        }

        // fp8: the wide-K instructions take their 32 bytes per lane as two runs of 16 bytes of K, one
        // from each half of the instruction's K range (lane group g holds k = 16 g + 0..15 and
        // k = 16 groups + 16 g + 0..15: the first four registers are the operand of one 16x16x64-shaped
        // half, the last four of the other; the block scales of the scaled forms go by this order).  So
        // the run is 16 bytes long, and it exists only where the K steps pair up into whole instructions;
        // elsewhere fp8 uses the 8-byte runs of the 16x16x32 / 32x32x16 instructions.
        constexpr bool kPackAllowed(PackClass c, uint32_t p, uint32_t groups, uint32_t blockK)
        {
            if(c != PackClass::Fp8)
                return true;
            return p <= 8u || (p == 16u && blockK % (32u * groups) == 0u);
        }

        constexpr uint32_t chooseKPack(PackClass c, uint32_t tile, uint32_t blockK)
        {
            uint32_t groups = kWaveSize / tile;
            uint32_t p      = maxKPack(c);
            while(p > 1u && !(kPackAllowed(c, p, groups, blockK) && blockK % (p * groups) == 0u))
                p >>= 1u;
            return p;
        }

        // Geometry of an input (matrix_a / matrix_b) fragment.
        template <uint32_t BlockDim, uint32_t BlockK, uint32_t Tile, PackClass Class>
        struct InputMap
        {
            static_assert(Tile == 8u || Tile == 16u || Tile == 32u, "tile edge is 16 or 32 (8: load / store only)");
            static_assert(BlockDim % Tile == 0u, "block dimension must be a multiple of the tile edge");

            static constexpr uint32_t tile    = Tile;
            static constexpr uint32_t groups  = kWaveSize / Tile;
            static constexpr uint32_t kpack   = chooseKPack(Class, Tile, BlockK);
            static constexpr uint32_t kstep   = kpack * groups;
            static constexpr uint32_t nk      = BlockK / kstep;
            static constexpr uint32_t ndim    = BlockDim / Tile;
            static constexpr uint32_t nchunks = ndim * nk; // MFMA operands held
            static constexpr uint32_t size    = nchunks * kpack; // elements per lane
            // consecutive K steps one instruction consumes (fp8 wide-K forms: two 16-byte runs)
            static constexpr uint32_t mmaSteps = (Class == PackClass::Fp8 && kpack == 16u) ? 2u : 1u;
            static constexpr uint32_t mmaKPack = kpack * mmaSteps; // elements per lane and instruction
            static constexpr uint32_t nmma     = nk / mmaSteps; // instructions along K

            static_assert(BlockK % kstep == 0u && nk >= 1u,
                          "BlockK must be a multiple of 64 / tile (4 for 16-wide, 2 for 32-wide blocks)");
            static_assert(size * kWaveSize == BlockDim * BlockK, "map must cover the block exactly");

            // chunk c (one MFMA operand) -> (dim block, k step)
            static constexpr uint32_t chunkDimBlock(uint32_t c)
            {
                return c / nk;
            }
            static constexpr uint32_t chunkKStep(uint32_t c)
            {
                return c % nk;
            }
            static constexpr uint32_t chunkIndex(uint32_t dimBlock, uint32_t kStep)
            {
                return dimBlock * nk + kStep;
            }
            // coordinates of the first element of chunk c held by `lane`
            static constexpr uint32_t chunkDim(uint32_t c, uint32_t lane)
            {
                return chunkDimBlock(c) * Tile + lane % Tile;
            }
            static constexpr uint32_t chunkK(uint32_t c, uint32_t lane)
            {
                return chunkKStep(c) * kstep + (lane / Tile) * kpack;
            }
            // coordinates of element e held by `lane`
            static constexpr uint32_t dimOf(uint32_t e, uint32_t lane)
            {
                return chunkDim(e / kpack, lane);
            }
            static constexpr uint32_t kOf(uint32_t e, uint32_t lane)
            {
                return chunkK(e / kpack, lane) + e % kpack;
            }
        };

        // Geometry of an accumulator fragment.  Tile = rows of a tile; a tile is Tile columns wide,
        // or 8 columns for blocks whose width is not a multiple of 16 (load / store only).
        template <uint32_t BlockM, uint32_t BlockN, uint32_t Tile>
        struct AccMap
        {
            static_assert(Tile == 16u || Tile == 32u, "MFMA tile edge is 16 or 32");
            static constexpr uint32_t tile  = Tile;
            static constexpr uint32_t tileN = BlockN % 16u == 0u ? Tile : 8u;
            static_assert(tileN == Tile || Tile == 32u, "8-column tiles are 32 rows high");
            static_assert(BlockM % Tile == 0u && BlockN % tileN == 0u,
                          "accumulator block must be a multiple of the MFMA tile (or 32 x 8 for load / store)");

            static constexpr uint32_t nbi      = BlockM / Tile;
            static constexpr uint32_t nbj      = BlockN / tileN;
            static constexpr uint32_t perBlock = Tile * tileN / kWaveSize; // 4 or 16
            static constexpr uint32_t runLen   = 4u; // consecutive columns a lane holds per run
            static constexpr uint32_t runs     = perBlock / 4u; // 4-column runs per block per lane
            static constexpr uint32_t nruns    = nbi * nbj * runs;
            static constexpr uint32_t size     = nbi * nbj * perBlock;

            static constexpr uint32_t blockIndex(uint32_t bi, uint32_t bj)
            {
                return bi * nbj + bj;
            }
            // run r = 4 consecutive columns of one row
            static constexpr uint32_t runRow(uint32_t r, uint32_t lane)
            {
                return ((r / runs) / nbj) * Tile + lane % Tile;
            }
            static constexpr uint32_t runCol(uint32_t r, uint32_t lane)
            {
                return ((r / runs) % nbj) * tileN + (Tile == 16u ? 0u : 8u * (r % runs))
                       + (lane / Tile) * 4u;
            }
            static constexpr uint32_t rowOf(uint32_t e, uint32_t lane)
            {
                return runRow(e / 4u, lane);
            }
            static constexpr uint32_t colOf(uint32_t e, uint32_t lane)
            {
                return runCol(e / 4u, lane) + e % 4u;
            }
        };

        // Accumulators of 64-bit elements.  v_mfma_f64_16x16x4_f64 spreads a lane's four results over
        // rows (lane / 16) + 4 i of the instruction's result, not over four consecutive ones, so with
        // the multiplicands swapped as for the other types a lane owns row lane % 16 and the columns
        // (lane / 16) + 4 i of each 16 x 16 tile: runs of one element.  Blocks of any multiple of 16 are
        // tiled with 16 x 16 tiles (there is no 32-wide f64 instruction).
        template <uint32_t BlockM, uint32_t BlockN>
        struct AccMapStrided
        {
            static constexpr uint32_t tile  = 16u;
            static constexpr uint32_t tileN = 16u;
            static_assert(BlockM % 16u == 0u && BlockN % 16u == 0u, "accumulator block must be a multiple of 16 x 16");

            static constexpr uint32_t nbi      = BlockM / 16u;
            static constexpr uint32_t nbj      = BlockN / 16u;
            static constexpr uint32_t perBlock = 4u;
            static constexpr uint32_t runLen   = 1u;
            static constexpr uint32_t runs     = 4u;
            static constexpr uint32_t nruns    = nbi * nbj * runs;
            static constexpr uint32_t size     = nbi * nbj * perBlock;

            static constexpr uint32_t blockIndex(uint32_t bi, uint32_t bj)
            {
                return bi * nbj + bj;
            }
            static constexpr uint32_t runRow(uint32_t r, uint32_t lane)
            {
                return ((r / runs) / nbj) * 16u + lane % 16u;
            }
            static constexpr uint32_t runCol(uint32_t r, uint32_t lane)
            {
                return ((r / runs) % nbj) * 16u + lane / 16u + 4u * (r % runs);
            }
            static constexpr uint32_t rowOf(uint32_t e, uint32_t lane)
            {
                return runRow(e, lane);
            }
            static constexpr uint32_t colOf(uint32_t e, uint32_t lane)
            {
                return runCol(e, lane);
            }
        };

    } // namespace detail
} // namespace rocwmma

#endif // ROCWMMA_FRAGMENT_MAP_HPP
