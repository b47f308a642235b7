// Register <-> memory movers for fragments (global memory or LDS, through generic pointers).
//
// A fragment is a sequence of "items": for input fragments an item is one MFMA operand
// (kpack elements contiguous in K, see fragment_map.hpp); for accumulators an item is a run
// of four consecutive columns of one row (a single element for 64-bit accumulators).  Items whose elements are contiguous in memory
// (K-contiguous operands; row-major accumulators) move as one 2..32-byte vector access,
// the others element by element.
//
// The same walk serves the cooperative API.  Wave w of a pool of W waves owns the fragment's
// register elements [w * size / W, (w + 1) * size / W) and keeps them at their ordinary
// positions; the rest of its fragment is untouched.  With Items % W == 0 that is a run of whole
// items; with more waves than items (W % Items == 0) an item is cut into W / Items equal
// pieces.  Because the share is a range of register elements, a cooperative fragment may be
// reinterpreted as another fragment type with the same element count (an LDS "register file"
// view, say) and stored cooperatively with the same (w, W): every wave then writes what it
// read, whatever the item sizes of the two types.  Other wave counts (3 waves, 4 items) fall
// back to ceil(Items / W) whole items per wave, which agrees only between types with equal
// item sizes.
// (rocWMMA's engines for the same job: reference library/include/rocwmma/internal/
// opaque_load.hpp:65-159, opaque_store.hpp:56-135, coop_load.hpp:43-218, coop_store.hpp:43-217.)
//
// Alignment contract: a vector access of B bytes needs its address aligned to min(B, 16).
// That holds when the tile origin and the leading dimension are multiples of 16 bytes.
#ifndef ROCWMMA_FRAGMENT_IO_HPP
#define ROCWMMA_FRAGMENT_IO_HPP

#include "fragment_map.hpp"
#include "types.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <uint32_t Bytes>
        ROCWMMA_DEVICE ROCWMMA_INLINE void copyBytes(void* dst, const void* src)
        {
            if constexpr(Bytes % 16u == 0u)
            {
#pragma unroll
                for(uint32_t i = 0; i < Bytes / 16u; ++i)
                    reinterpret_cast<u32x4*>(dst)[i] = reinterpret_cast<const u32x4*>(src)[i];
            }
            else if constexpr(Bytes == 8u)
                *reinterpret_cast<u32x2*>(dst) = *reinterpret_cast<const u32x2*>(src);
            else if constexpr(Bytes == 4u)
                *reinterpret_cast<u32x1*>(dst) = *reinterpret_cast<const u32x1*>(src);
            else if constexpr(Bytes == 2u)
                *reinterpret_cast<u16x1*>(dst) = *reinterpret_cast<const u16x1*>(src);
            else
            {
                static_assert(Bytes == 1u, "unsupported vector width");
                *reinterpret_cast<u8x1*>(dst) = *reinterpret_cast<const u8x1*>(src);
            }
        }

        // ---- input fragments -------------------------------------------------------------
        // KContiguous: memory offset of (dim, k) is dim * ld + k  (matrix_a row_major,
        // matrix_b col_major); otherwise k * ld + dim.
        template <typename Map, typename DataT, bool KContiguous>
        struct InputIO
        {
            static constexpr uint32_t Items     = Map::nchunks;
            static constexpr uint32_t ItemElems = Map::kpack;

            // Elements [first, first + Count) of item `item`; the whole item is <ItemElems>(.., 0u, ..).
            template <uint32_t Count>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadPart(DataT* x, uint32_t item, uint32_t first, const DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t dim = Map::chunkDim(item, lane);
                const uint32_t k   = Map::chunkK(item, lane) + first;
                DataT*         reg = x + item * ItemElems + first;
                if constexpr(KContiguous)
                    copyBytes<Count * sizeof(DataT)>(reg, data + dim * ld + k);
                else
                {
#pragma unroll
                    for(uint32_t j = 0; j < Count; ++j)
                        copyBytes<sizeof(DataT)>(reg + j, data + (k + j) * ld + dim);
                }
            }

            template <uint32_t Count>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storePart(const DataT* x, uint32_t item, uint32_t first, DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t dim = Map::chunkDim(item, lane);
                const uint32_t k   = Map::chunkK(item, lane) + first;
                const DataT*   reg = x + item * ItemElems + first;
                if constexpr(KContiguous)
                    copyBytes<Count * sizeof(DataT)>(data + dim * ld + k, reg);
                else
                {
#pragma unroll
                    for(uint32_t j = 0; j < Count; ++j)
                        copyBytes<sizeof(DataT)>(data + (k + j) * ld + dim, reg + j);
                }
            }
        };

        // ---- accumulator fragments -------------------------------------------------------
        template <typename Map, typename DataT, bool RowMajor>
        struct AccIO
        {
            static constexpr uint32_t Items     = Map::nruns;
            static constexpr uint32_t ItemElems = Map::runLen; // 4 (1 for 64-bit accumulators)

            template <uint32_t Count>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadPart(DataT* x, uint32_t item, uint32_t first, const DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t row = Map::runRow(item, lane);
                const uint32_t col = Map::runCol(item, lane) + first;
                DataT*         reg = x + item * ItemElems + first;
                if constexpr(RowMajor)
                    copyBytes<Count * sizeof(DataT)>(reg, data + row * ld + col);
                else
                {
#pragma unroll
                    for(uint32_t j = 0; j < Count; ++j)
                        copyBytes<sizeof(DataT)>(reg + j, data + (col + j) * ld + row);
                }
            }

            template <uint32_t Count>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storePart(const DataT* x, uint32_t item, uint32_t first, DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t row = Map::runRow(item, lane);
                const uint32_t col = Map::runCol(item, lane) + first;
                const DataT*   reg = x + item * ItemElems + first;
                if constexpr(RowMajor)
                    copyBytes<Count * sizeof(DataT)>(data + row * ld + col, reg);
                else
                {
#pragma unroll
                    for(uint32_t j = 0; j < Count; ++j)
                        copyBytes<sizeof(DataT)>(data + (col + j) * ld + row, reg + j);
                }
            }
        };

        // ---- whole-fragment and cooperative drivers --------------------------------------
        // `move(item, first, Count)` callbacks below receive a compile-time item and piece so that
        // register indices stay static; which of them run is decided by (waveIndex, waveCount).
        template <typename IO, typename DataT>
        struct FragmentMover
        {
            static constexpr uint32_t Items     = IO::Items; // work items of the whole fragment
            static constexpr uint32_t ItemElems = IO::ItemElems;
            static constexpr uint32_t MaxWaves  = 16u; // 1024 threads per workgroup

            template <bool Load, uint32_t Count, typename Ptr, typename Reg>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                part(Reg* x, uint32_t item, uint32_t first, Ptr* data, uint32_t ld, uint32_t lane)
            {
                if constexpr(Load)
                    IO::template loadPart<Count>(x, item, first, data, ld, lane);
                else
                    IO::template storePart<Count>(x, item, first, data, ld, lane);
            }

            template <bool Load, typename Ptr, typename Reg>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void whole(Reg* x, Ptr* data, uint32_t ld)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
#pragma unroll
                for(uint32_t item = 0; item < Items; ++item)
                    part<Load, ItemElems>(x, item, 0u, data, ld, lane);
            }

            // Wave count known at compile time.
            template <bool Load, uint32_t WaveCount, typename Ptr, typename Reg>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void shared(Reg* x, Ptr* data, uint32_t ld, uint32_t waveIndex)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
                if constexpr(WaveCount > Items && WaveCount % Items == 0u && ItemElems % (WaveCount / Items) == 0u)
                {
                    constexpr uint32_t pieces = WaveCount / Items, count = ItemElems / pieces;
#pragma unroll
                    for(uint32_t item = 0; item < Items; ++item)
#pragma unroll
                        for(uint32_t piece = 0; piece < pieces; ++piece)
                            if(waveIndex == item * pieces + piece)
                                part<Load, count>(x, item, piece * count, data, ld, lane);
                }
                else
                {
                    constexpr uint32_t per = (Items + WaveCount - 1u) / WaveCount;
#pragma unroll
                    for(uint32_t item = 0; item < Items; ++item)
                        if(waveIndex == item / per)
                            part<Load, ItemElems>(x, item, 0u, data, ld, lane);
                }
            }

            // Pieces of `Count` elements, for a wave count only known at run time: tried for every
            // piece size an item can be cut into with at most MaxWaves waves.
            template <bool Load, uint32_t Count, typename Ptr, typename Reg>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                pieces(Reg* x, Ptr* data, uint32_t ld, uint32_t lane, uint32_t waveIndex, uint32_t count)
            {
                if constexpr(Count >= 1u && Items * (ItemElems / (Count == 0u ? 1u : Count)) <= MaxWaves)
                {
                    constexpr uint32_t perItem = ItemElems / Count;
                    if(count == Count)
                    {
#pragma unroll
                        for(uint32_t item = 0; item < Items; ++item)
#pragma unroll
                            for(uint32_t piece = 0; piece < perItem; ++piece)
                                if(waveIndex == item * perItem + piece)
                                    part<Load, Count>(x, item, piece * Count, data, ld, lane);
                    }
                    else
                        pieces<Load, Count / 2u>(x, data, ld, lane, waveIndex, count);
                }
            }

            template <bool Load, typename Ptr, typename Reg>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                shared(Reg* x, Ptr* data, uint32_t ld, uint32_t waveIndex, uint32_t waveCount)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
                if(waveCount > Items && waveCount % Items == 0u && ItemElems % (waveCount / Items) == 0u)
                    pieces<Load, ItemElems / 2u>(x, data, ld, lane, waveIndex, ItemElems / (waveCount / Items));
                else
                {
                    const uint32_t per   = (Items + waveCount - 1u) / waveCount;
                    const uint32_t begin = waveIndex * per;
#pragma unroll
                    for(uint32_t item = 0; item < Items; ++item)
                        if(item >= begin && item - begin < per)
                            part<Load, ItemElems>(x, item, 0u, data, ld, lane);
                }
            }

            ROCWMMA_DEVICE static ROCWMMA_INLINE void load(DataT* x, const DataT* data, uint32_t ld)
            {
                whole<true>(x, data, ld);
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE void store(DataT* data, const DataT* x, uint32_t ld)
            {
                whole<false>(x, data, ld);
            }
            template <uint32_t WaveCount>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadCoop(DataT* x, const DataT* data, uint32_t ld, uint32_t waveIndex)
            {
                shared<true, WaveCount>(x, data, ld, waveIndex);
            }
            template <uint32_t WaveCount>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storeCoop(DataT* data, const DataT* x, uint32_t ld, uint32_t waveIndex)
            {
                shared<false, WaveCount>(x, data, ld, waveIndex);
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadCoop(DataT* x, const DataT* data, uint32_t ld, uint32_t waveIndex, uint32_t waveCount)
            {
                shared<true>(x, data, ld, waveIndex, waveCount);
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storeCoop(DataT* data, const DataT* x, uint32_t ld, uint32_t waveIndex, uint32_t waveCount)
            {
                shared<false>(x, data, ld, waveIndex, waveCount);
            }
        };

    } // namespace detail
} // namespace rocwmma

#endif // ROCWMMA_FRAGMENT_IO_HPP
