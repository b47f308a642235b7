// Wave -> block -> matrix -> memory coordinate helpers.
//
// Same contract as rocWMMA's MappingUtil (reference:
// library/include/rocwmma/internal/mapping_util.hpp:114-206, mapping_util_impl.hpp:46-149):
// a workgroup is shaped blockDim = (64 * wavesX, wavesY); the wave at (threadIdx.x / 64,
// threadIdx.y) owns the BlockHeight x BlockWidth block at that position of the global wave
// grid; coordinates are (row, col); a data layout turns (row, col) into an element offset.
#ifndef ROCWMMA_MAPPING_UTIL_HPP
#define ROCWMMA_MAPPING_UTIL_HPP

#include "constants.hpp"
#include "coord.hpp"
#include "types.hpp"

namespace rocwmma
{
    struct row_major;
    struct col_major;

    namespace detail
    {
        ROCWMMA_DEVICE ROCWMMA_INLINE uint32_t laneId()
        {
            return threadIdx.x & (Constants::AMDGCN_WAVE_SIZE - 1u);
        }

        // threads (x, y) -> waves (x / 64, y)
        ROCWMMA_HOST_DEVICE constexpr inline Coord2d waveCount(Coord2d const& threadCount)
        {
            return make_coord2d(threadCount.x / Constants::AMDGCN_WAVE_SIZE, threadCount.y);
        }

        ROCWMMA_HOST_DEVICE constexpr inline Coord2d threadCount(Coord2d const& waveCount)
        {
            return make_coord2d(waveCount.x * Constants::AMDGCN_WAVE_SIZE, waveCount.y);
        }

        template <uint32_t TBlockX = 0u, uint32_t TBlockY = 0u>
        struct WaveSpace
        {
            using WaveCoordT      = Coord2d;
            using WorkgroupCoordT = Coord2d;
            using WorkgroupDimT   = Coord2d;

            ROCWMMA_DEVICE static inline uint32_t localLaneId()
            {
                return laneId();
            }
            ROCWMMA_DEVICE static inline WaveCoordT localWaveCoord()
            {
                return waveCount(make_coord2d(threadIdx.x, threadIdx.y));
            }
            ROCWMMA_DEVICE static inline WaveCoordT globalWaveCoord()
            {
                if constexpr(TBlockX > 0u && TBlockY > 0u)
                    return waveCount(make_coord2d(blockIdx.x * TBlockX + threadIdx.x,
                                                  blockIdx.y * TBlockY + threadIdx.y));
                else
                    return waveCount(make_coord2d(blockIdx.x * blockDim.x + threadIdx.x,
                                                  blockIdx.y * blockDim.y + threadIdx.y));
            }
            ROCWMMA_DEVICE static inline WorkgroupCoordT workgroupCoord()
            {
                return make_coord2d(blockIdx.x, blockIdx.y);
            }
            // a constant expression when the thread-block shape is given at compile time
            ROCWMMA_DEVICE constexpr static inline WorkgroupDimT workgroupDim()
            {
                if constexpr(TBlockX > 0u && TBlockY > 0u)
                    return waveCount(make_coord2d(TBlockX, TBlockY));
                else
                    return waveCount(make_coord2d(blockDim.x, blockDim.y));
            }
        };

        template <uint32_t BlockHeight, uint32_t BlockWidth>
        struct MatrixSpace
        {
            using MatrixCoordT = Coord2d;
            using BlockCoordT  = Coord2d;

            ROCWMMA_HOST_DEVICE constexpr static inline MatrixCoordT
                fromBlockCoord(BlockCoordT const& blockCoord)
            {
                return make_coord2d(blockCoord.x * BlockHeight, blockCoord.y * BlockWidth);
            }
        };

        template <typename DataOrientation>
        struct DataSpace
        {
            using MatrixCoordT = Coord2d;
            using MatrixSizeT  = Coord2d;
            using Orientation  = DataOrientation;

            enum : uint32_t
            {
                MajorIndex = std::is_same<DataOrientation, row_major>::value ? 0 : 1,
                MinorIndex = std::is_same<DataOrientation, row_major>::value ? 1 : 0
            };

            ROCWMMA_HOST_DEVICE constexpr static inline auto leadingDim(MatrixSizeT const& matrixSize)
            {
                return get<MinorIndex>(matrixSize);
            }

            // (row, col) -> element offset
            ROCWMMA_HOST_DEVICE constexpr static inline auto
                fromMatrixCoord(MatrixCoordT const& matrixCoord, uint32_t leadingDim)
            {
                return get<MajorIndex>(matrixCoord) * leadingDim + get<MinorIndex>(matrixCoord);
            }
        };

        template <>
        struct DataSpace<void>;
    } // namespace detail

    // Names existing kernels use for the (row, col) -> element offset map of a row- or column-major
    // array (reference: library/include/rocwmma/internal/layout/layout.hpp, namespace DataLayout).
    namespace DataLayout
    {
        template <typename DataOrientation>
        using Array1d = detail::DataSpace<DataOrientation>;
        using RowMajor = Array1d<row_major>;
        using ColMajor = Array1d<col_major>;
    } // namespace DataLayout

    template <uint32_t BlockHeight, uint32_t BlockWidth, typename DataT, typename DataLayout>
    struct MappingUtil
    {
        using WaveSpace   = detail::WaveSpace<>;
        using MatrixSpace = detail::MatrixSpace<BlockHeight, BlockWidth>;
        using DataSpace   = detail::DataSpace<DataLayout>;

        using WaveCoordT    = typename WaveSpace::WaveCoordT;
        using BlockCoordT   = typename MatrixSpace::BlockCoordT;
        using MatrixCoordT  = typename MatrixSpace::MatrixCoordT;
        using WorkgroupDimT = typename WaveSpace::WorkgroupDimT;

        ROCWMMA_DEVICE static inline uint32_t laneId()
        {
            return WaveSpace::localLaneId();
        }
        ROCWMMA_DEVICE static inline WaveCoordT waveCoord()
        {
            return WaveSpace::localWaveCoord();
        }
        ROCWMMA_DEVICE static inline BlockCoordT blockCoord()
        {
            return WaveSpace::globalWaveCoord();
        }
        ROCWMMA_DEVICE static inline MatrixCoordT matrixCoord()
        {
            return MatrixSpace::fromBlockCoord(blockCoord());
        }
        ROCWMMA_DEVICE static inline DataT const* dataCoord(DataT const* baseAddr, uint32_t ldm)
        {
            return baseAddr + DataSpace::fromMatrixCoord(matrixCoord(), ldm);
        }
        ROCWMMA_DEVICE static inline DataT* dataCoord(DataT* baseAddr, uint32_t ldm)
        {
            return baseAddr + DataSpace::fromMatrixCoord(matrixCoord(), ldm);
        }
        ROCWMMA_DEVICE static inline WorkgroupDimT workgroupDim()
        {
            return WaveSpace::workgroupDim();
        }
        ROCWMMA_DEVICE static inline BlockCoordT blockCoordM(uint32_t m)
        {
            auto coord = blockCoord();
            coord.x    = m;
            return coord;
        }
        ROCWMMA_DEVICE static inline BlockCoordT blockCoordN(uint32_t n)
        {
            auto coord = blockCoord();
            coord.y    = n;
            return coord;
        }
        ROCWMMA_DEVICE static inline MatrixCoordT matrixCoordM(uint32_t m)
        {
            auto coord = matrixCoord();
            coord.x    = m;
            return coord;
        }
        ROCWMMA_DEVICE static inline MatrixCoordT matrixCoordN(uint32_t n)
        {
            auto coord = matrixCoord();
            coord.y    = n;
            return coord;
        }
        ROCWMMA_HOST_DEVICE static inline MatrixCoordT matrixCoord(BlockCoordT const& blockCoord)
        {
            return MatrixSpace::fromBlockCoord(blockCoord);
        }
        ROCWMMA_HOST_DEVICE static inline uint32_t dataOffset(MatrixCoordT const& matrixCoord,
                                                              uint32_t            ldm)
        {
            return DataSpace::fromMatrixCoord(matrixCoord, ldm);
        }
        ROCWMMA_HOST_DEVICE static inline DataT const*
            dataCoord(DataT const* baseAddr, MatrixCoordT const& matrixCoord, uint32_t ldm)
        {
            return baseAddr + DataSpace::fromMatrixCoord(matrixCoord, ldm);
        }
        ROCWMMA_HOST_DEVICE static inline DataT*
            dataCoord(DataT* baseAddr, MatrixCoordT const& matrixCoord, uint32_t ldm)
        {
            return baseAddr + DataSpace::fromMatrixCoord(matrixCoord, ldm);
        }
    };

} // namespace rocwmma

#endif // ROCWMMA_MAPPING_UTIL_HPP
