// Cooperative fragment load / store: a pool of waves moves one large fragment together,
// each wave a share of it.
//
// Same overload set and argument meaning as rocWMMA's cooperative API (reference:
// library/include/rocwmma/rocwmma_coop.hpp:78-412).  Wave `waveIndex` of `waveCount` moves
// the register elements [waveIndex * size / waveCount, (waveIndex + 1) * size / waveCount) of
// the fragment (whole items, or equal pieces of an item when there are more waves than items;
// see internal/fragment_io.hpp) and leaves the others alone.  A fragment filled by a
// cooperative load holds only that wave's share, at its ordinary register positions, and must
// be written back by a cooperative store with the same (waveIndex, waveCount), as the same
// fragment type or reinterpreted as another one with the same element count.  The deprecated
// splitCount arguments are accepted and ignored, as in the reference
// (rocwmma_coop_impl.hpp:44-53,116-132).
//
// Default wave order (overloads without waveIndex): row-major over the workgroup's wave
// grid, index = waveRow * wavesPerRow... i.e. (threadIdx.x / 64) * blockDim.y + threadIdx.y
// (reference: rocwmma_coop_impl.hpp:106-112).
#ifndef ROCWMMA_COOP_API_HPP
#define ROCWMMA_COOP_API_HPP

#include "rocwmma.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
        struct CoopMover
        {
            static_assert(!std::is_same<DataLayoutT, void>::value,
                          "cooperative load / store needs a fragment with a static data layout");
            using Config = FragConfig<MatrixT, BlockM, BlockN, BlockK, DataT>;
            using type   = FragmentMover<typename Config::template IO<DataLayoutT>, DataT>;
        };

        ROCWMMA_DEVICE ROCWMMA_INLINE uint32_t defaultWaveIndex()
        {
            return (threadIdx.x / Constants::AMDGCN_WAVE_SIZE) * blockDim.y + threadIdx.y;
        }
        ROCWMMA_DEVICE ROCWMMA_INLINE uint32_t defaultWaveCount()
        {
            return (blockDim.x / Constants::AMDGCN_WAVE_SIZE) * blockDim.y;
        }
    } // namespace detail

    // Cooperative I/O description of a fragment shared by WaveCount waves (reference:
    // library/include/rocwmma/internal/accessors.hpp:55-59).  IOTraits::IOCount is the number of
    // items one wave moves (at least 1); kernels use it only to derive the deprecated split
    // counts, which the loads and stores below ignore.
    template <typename FragT, uint32_t WaveCount>
    struct GetCoopIOConfig;

    template <uint32_t WaveCount,
              typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    struct GetCoopIOConfig<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>, WaveCount>
    {
        struct type
        {
            using Mover = typename detail::CoopMover<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>::type;
            struct IOTraits
            {
                enum : uint32_t
                {
                    IOCount = (Mover::Items + WaveCount - 1u) / WaveCount
                };
            };
        };
    };

    template <typename FragT, uint32_t WaveCount = 1u>
    using GetCoopIOConfig_t = typename GetCoopIOConfig<std::decay_t<FragT>, WaveCount>::type;

    // ---- loads -----------------------------------------------------------------------------
    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        load_matrix_coop_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                              const DataT*                                                   data,
                              uint32_t                                                       ldm,
                              uint32_t                                                       waveIndex,
                              uint32_t                                                       waveCount)
    {
        using Mover = typename detail::CoopMover<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>::type;
        Mover::loadCoop(frag.x, data, ldm, waveIndex, waveCount);
    }

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    [[deprecated("splitCount argument is deprecated and will be removed in a future release")]]
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        load_matrix_coop_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                              const DataT*                                                   data,
                              uint32_t                                                       ldm,
                              uint32_t                                                       waveIndex,
                              uint32_t                                                       waveCount,
                              uint32_t /*splitCount*/)
    {
        load_matrix_coop_sync(frag, data, ldm, waveIndex, waveCount);
    }

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        load_matrix_coop_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                              const DataT*                                                   data,
                              uint32_t                                                       ldm)
    {
        load_matrix_coop_sync(frag, data, ldm, detail::defaultWaveIndex(), detail::defaultWaveCount());
    }

    template <uint32_t WaveCount,
              typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        load_matrix_coop_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                              const DataT*                                                   data,
                              uint32_t                                                       ldm,
                              uint32_t                                                       waveIndex)
    {
        using Mover = typename detail::CoopMover<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>::type;
        Mover::template loadCoop<WaveCount>(frag.x, data, ldm, waveIndex);
    }

    template <uint32_t WaveCount,
              uint32_t SplitCount,
              typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    [[deprecated("SplitCount argument is deprecated and will be removed in a future release")]]
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        load_matrix_coop_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                              const DataT*                                                   data,
                              uint32_t                                                       ldm,
                              uint32_t                                                       waveIndex)
    {
        load_matrix_coop_sync<WaveCount>(frag, data, ldm, waveIndex);
    }

    // ---- stores ----------------------------------------------------------------------------
    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        store_matrix_coop_sync(DataT*                                                               data,
                               fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
                               uint32_t                                                             ldm,
                               uint32_t                                                             waveIndex,
                               uint32_t                                                             waveCount)
    {
        using Mover = typename detail::CoopMover<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>::type;
        Mover::storeCoop(data, frag.x, ldm, waveIndex, waveCount);
    }

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    [[deprecated("splitCount argument is deprecated and will be removed in a future release")]]
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        store_matrix_coop_sync(DataT*                                                               data,
                               fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
                               uint32_t                                                             ldm,
                               uint32_t                                                             waveIndex,
                               uint32_t                                                             waveCount,
                               uint32_t /*splitCount*/)
    {
        store_matrix_coop_sync(data, frag, ldm, waveIndex, waveCount);
    }

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        store_matrix_coop_sync(DataT*                                                               data,
                               fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
                               uint32_t                                                             ldm)
    {
        store_matrix_coop_sync(data, frag, ldm, detail::defaultWaveIndex(), detail::defaultWaveCount());
    }

    template <uint32_t WaveCount,
              typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        store_matrix_coop_sync(DataT*                                                               data,
                               fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
                               uint32_t                                                             ldm,
                               uint32_t                                                             waveIndex)
    {
        using Mover = typename detail::CoopMover<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>::type;
        Mover::template storeCoop<WaveCount>(data, frag.x, ldm, waveIndex);
    }

    template <uint32_t WaveCount,
              uint32_t SplitCount,
              typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    [[deprecated("SplitCount argument is deprecated and will be removed in a future release")]]
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        store_matrix_coop_sync(DataT*                                                               data,
                               fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
                               uint32_t                                                             ldm,
                               uint32_t                                                             waveIndex)
    {
        store_matrix_coop_sync<WaveCount>(data, frag, ldm, waveIndex);
    }

} // namespace rocwmma

#endif // ROCWMMA_COOP_API_HPP
