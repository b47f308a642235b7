// Register <-> memory movers for fragments (global memory or LDS, through generic pointers).
//
// A fragment is a sequence of "items": for input fragments an item is one MFMA operand
// (kpack elements contiguous in K, see fragment_map.hpp); for accumulators an item is a run
// of four consecutive columns of one row.  Items whose elements are contiguous in memory
// (K-contiguous operands; row-major accumulators) move as one 2..32-byte vector access,
// the others element by element.
//
// The same walk serves the cooperative API: wave w of a pool of W waves moves items
// w, w+W, w+2W, ... and keeps them in its first register slots.  A cooperative fragment is
// therefore only meaningful to the matching cooperative store with the same (w, W).
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

        // Walks items `first, first + stride, ...` (< Items) and calls fn(slot, item) with a
        // compile-time register slot and a (possibly run-time) item index.
        template <uint32_t Items, uint32_t Stride, typename Fn>
        ROCWMMA_DEVICE ROCWMMA_INLINE void forEachItemStatic(uint32_t first, Fn&& fn)
        {
            constexpr uint32_t slots = (Items + Stride - 1u) / Stride;
#pragma unroll
            for(uint32_t s = 0; s < slots; ++s)
            {
                uint32_t item = s * Stride + first;
                if constexpr(Items % Stride == 0u)
                    fn(s, item);
                else if(item < Items)
                    fn(s, item);
            }
        }

        template <uint32_t Items, typename Fn>
        ROCWMMA_DEVICE ROCWMMA_INLINE void forEachItemDynamic(uint32_t first, uint32_t stride, Fn&& fn)
        {
#pragma unroll
            for(uint32_t s = 0; s < Items; ++s)
            {
                uint32_t item = s * stride + first;
                if(item < Items)
                    fn(s, item);
            }
        }

        // ---- input fragments -------------------------------------------------------------
        // KContiguous: memory offset of (dim, k) is dim * ld + k  (matrix_a row_major,
        // matrix_b col_major); otherwise k * ld + dim.
        template <typename Map, typename DataT, bool KContiguous>
        struct InputIO
        {
            static constexpr uint32_t Items = Map::nchunks;

            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadItem(DataT* x, uint32_t slot, uint32_t item, const DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t dim = Map::chunkDim(item, lane);
                const uint32_t k   = Map::chunkK(item, lane);
                if constexpr(KContiguous)
                    copyBytes<Map::kpack * sizeof(DataT)>(x + slot * Map::kpack, data + dim * ld + k);
                else
                {
#pragma unroll
                    for(uint32_t j = 0; j < Map::kpack; ++j)
                        copyBytes<sizeof(DataT)>(x + slot * Map::kpack + j, data + (k + j) * ld + dim);
                }
            }

            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storeItem(const DataT* x, uint32_t slot, uint32_t item, DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t dim = Map::chunkDim(item, lane);
                const uint32_t k   = Map::chunkK(item, lane);
                if constexpr(KContiguous)
                    copyBytes<Map::kpack * sizeof(DataT)>(data + dim * ld + k, x + slot * Map::kpack);
                else
                {
#pragma unroll
                    for(uint32_t j = 0; j < Map::kpack; ++j)
                        copyBytes<sizeof(DataT)>(data + (k + j) * ld + dim, x + slot * Map::kpack + j);
                }
            }
        };

        // ---- accumulator fragments -------------------------------------------------------
        template <typename Map, typename DataT, bool RowMajor>
        struct AccIO
        {
            static constexpr uint32_t Items = Map::nruns;

            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadItem(DataT* x, uint32_t slot, uint32_t item, const DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t row = Map::runRow(item, lane);
                const uint32_t col = Map::runCol(item, lane);
                if constexpr(RowMajor)
                    copyBytes<4u * sizeof(DataT)>(x + slot * 4u, data + row * ld + col);
                else
                {
#pragma unroll
                    for(uint32_t j = 0; j < 4u; ++j)
                        copyBytes<sizeof(DataT)>(x + slot * 4u + j, data + (col + j) * ld + row);
                }
            }

            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storeItem(const DataT* x, uint32_t slot, uint32_t item, DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t row = Map::runRow(item, lane);
                const uint32_t col = Map::runCol(item, lane);
                if constexpr(RowMajor)
                    copyBytes<4u * sizeof(DataT)>(data + row * ld + col, x + slot * 4u);
                else
                {
#pragma unroll
                    for(uint32_t j = 0; j < 4u; ++j)
                        copyBytes<sizeof(DataT)>(data + (col + j) * ld + row, x + slot * 4u + j);
                }
            }
        };

        // ---- whole-fragment and cooperative drivers --------------------------------------
        template <typename IO, typename DataT>
        struct FragmentMover
        {
            static constexpr uint32_t Items = IO::Items; // work items of the whole fragment
            ROCWMMA_DEVICE static ROCWMMA_INLINE void load(DataT* x, const DataT* data, uint32_t ld)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
                forEachItemStatic<IO::Items, 1u>(
                    0u, [&](uint32_t slot, uint32_t item) { IO::loadItem(x, slot, item, data, ld, lane); });
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE void store(DataT* data, const DataT* x, uint32_t ld)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
                forEachItemStatic<IO::Items, 1u>(
                    0u, [&](uint32_t slot, uint32_t item) { IO::storeItem(x, slot, item, data, ld, lane); });
            }
            template <uint32_t WaveCount>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadCoop(DataT* x, const DataT* data, uint32_t ld, uint32_t waveIndex)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
                forEachItemStatic<IO::Items, WaveCount>(
                    waveIndex,
                    [&](uint32_t slot, uint32_t item) { IO::loadItem(x, slot, item, data, ld, lane); });
            }
            template <uint32_t WaveCount>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storeCoop(DataT* data, const DataT* x, uint32_t ld, uint32_t waveIndex)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
                forEachItemStatic<IO::Items, WaveCount>(
                    waveIndex,
                    [&](uint32_t slot, uint32_t item) { IO::storeItem(x, slot, item, data, ld, lane); });
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadCoop(DataT* x, const DataT* data, uint32_t ld, uint32_t waveIndex, uint32_t waveCount)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
                forEachItemDynamic<IO::Items>(
                    waveIndex, waveCount,
                    [&](uint32_t slot, uint32_t item) { IO::loadItem(x, slot, item, data, ld, lane); });
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storeCoop(DataT* data, const DataT* x, uint32_t ld, uint32_t waveIndex, uint32_t waveCount)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
                forEachItemDynamic<IO::Items>(
                    waveIndex, waveCount,
                    [&](uint32_t slot, uint32_t item) { IO::storeItem(x, slot, item, data, ld, lane); });
            }
        };

    } // namespace detail
} // namespace rocwmma

#endif // ROCWMMA_FRAGMENT_IO_HPP
