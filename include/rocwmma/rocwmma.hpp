// Wave-level matrix multiply-accumulate API for gfx950 (MI350X / MI355X, CDNA4).
//
// The public surface -- tags, fragment<>, fill_fragment, load_matrix_sync,
// store_matrix_sync, mma_sync, synchronize_workgroup -- has the names, template parameters
// and argument meaning of rocWMMA (reference: library/include/rocwmma/rocwmma.hpp:74-317),
// so kernels written for it compile unchanged.  Everything underneath is written for the
// CDNA4 matrix cores only: see internal/fragment_map.hpp for the register layouts and
// internal/mfma_gfx950.hpp for the instruction table.
//
// Rules of use (same as the reference):
//   * every function is called by all 64 lanes of a wave with wave-uniform arguments;
//   * workgroups are shaped blockDim = (64 * wavesX, wavesY);
//   * pointers may address global memory or LDS; the caller synchronises LDS use;
//   * `data` points at the top-left element of the tile, `ldm` is the leading dimension in
//     elements; vector accesses need 16-byte aligned tile origins and leading dimensions;
//   * accumulator fragments may leave the data layout `void` and pick it at run time;
//   * element i of two accumulator fragments of equal block size is the same matrix element,
//     whatever their element types or layout tags.
#ifndef ROCWMMA_API_HPP
#define ROCWMMA_API_HPP

#include "internal/config.hpp"
#include "internal/constants.hpp"
#include "internal/coord.hpp"
#include "internal/flow_control.hpp"
#include "internal/fragment_io.hpp"
#include "internal/fragment_map.hpp"
#include "internal/mapping_util.hpp"
#include "internal/mfma_gfx950.hpp"
#include "internal/type_traits.hpp"
#include "internal/types.hpp"
#include "internal/utils.hpp"

namespace rocwmma
{
    // In-memory layout tags
    struct row_major
    {
    };
    struct col_major
    {
    };

    // Fragment context tags
    struct matrix_a
    {
    };
    struct matrix_b
    {
    };
    struct accumulator
    {
    };

    // Run-time layout selector for accumulator load / store
    enum layout_t : uint32_t
    {
        mem_row_major,
        mem_col_major
    };

    // Geometry of a fragment (reference: library/include/rocwmma/internal/io_shape.hpp:43-80)
    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK>
    struct IOShape;

    template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK>
    struct IOShape<matrix_a, BlockM, BlockN, BlockK>
    {
        enum : uint32_t
        {
            BlockHeight = BlockM,
            BlockWidth  = BlockK,
            BlockDim    = BlockM,
            KDim        = BlockK,
        };
    };
    template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK>
    struct IOShape<matrix_b, BlockM, BlockN, BlockK>
    {
        enum : uint32_t
        {
            BlockHeight = BlockK,
            BlockWidth  = BlockN,
            BlockDim    = BlockN,
            KDim        = BlockK,
        };
    };
    template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK>
    struct IOShape<accumulator, BlockM, BlockN, BlockK>
    {
        enum : uint32_t
        {
            BlockHeight = BlockM,
            BlockWidth  = BlockN,
            BlockDim    = BlockN,
            KDim        = BlockM,
        };
    };

    namespace detail
    {
        template <typename DataT>
        constexpr PackClass packClassOf()
        {
            switch(TypeInfo<DataT>::cls)
            {
            case MmaClass::F16:
            case MmaClass::BF16:
                return PackClass::Bits16;
            case MmaClass::F8:
            case MmaClass::BF8:
                return PackClass::Fp8;
            case MmaClass::I8:
                return PackClass::Int8;
            case MmaClass::F32:
                return PackClass::Bits32;
            default:
                return sizeof(DataT) == 2 ? PackClass::Bits16
                                          : (sizeof(DataT) == 4 ? PackClass::Bits32 : PackClass::Other);
            }
        }

        // MFMA tile edge of an input fragment: 64-bit elements only have the 16 x 16 x 4 instruction
        template <typename DataT>
        constexpr uint32_t fragTileDim(uint32_t blockM, uint32_t blockN, uint32_t blockDim)
        {
            const uint32_t t = inputTileDim(blockM, blockN, blockDim);
            return sizeof(DataT) == 8u && t == 32u ? 16u : t;
        }

        // Binds fragment template parameters to a register map and its movers.
        template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
        struct FragConfig;

        template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
        struct FragConfig<matrix_a, BlockM, BlockN, BlockK, DataT>
        {
            using Map = InputMap<BlockM, BlockK, fragTileDim<DataT>(BlockM, BlockN, BlockM), packClassOf<DataT>()>;
            // K runs along a row of A
            template <typename Layout>
            using IO = InputIO<Map, DataT, std::is_same<Layout, row_major>::value>;
        };
        template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
        struct FragConfig<matrix_b, BlockM, BlockN, BlockK, DataT>
        {
            using Map = InputMap<BlockN, BlockK, fragTileDim<DataT>(BlockM, BlockN, BlockN), packClassOf<DataT>()>;
            // K runs along a column of B
            template <typename Layout>
            using IO = InputIO<Map, DataT, std::is_same<Layout, col_major>::value>;
        };
        template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
        struct FragConfig<accumulator, BlockM, BlockN, BlockK, DataT>
        {
            // 64-bit accumulators in blocks of whole 16 x 16 tiles use the layout of the f64 instruction
            using Map = std::conditional_t<sizeof(DataT) == 8u && BlockM % 16u == 0u && BlockN % 16u == 0u,
                                           AccMapStrided<BlockM % 16u == 0u ? BlockM : 16u, BlockN % 16u == 0u ? BlockN : 16u>,
                                           AccMap<BlockM, BlockN, accTileRows(BlockM, BlockN)>>;
            template <typename Layout>
            using IO = AccIO<Map, DataT, std::is_same<Layout, row_major>::value>;
        };

        template <typename MatrixT, typename DataLayoutT>
        struct LayoutCheck
        {
            static_assert(std::is_same<DataLayoutT, row_major>::value
                              || std::is_same<DataLayoutT, col_major>::value
                              || (std::is_same<DataLayoutT, void>::value
                                  && std::is_same<MatrixT, accumulator>::value),
                          "fragment data layout must be row_major or col_major (void only for accumulators)");
        };
    } // namespace detail

    // Per-fragment counts (subset of reference library/include/rocwmma/internal/io_traits.hpp:43-82)
    template <uint32_t BlockDim, uint32_t BlockK, typename DataT>
    struct IOTraits
    {
        enum : uint32_t
        {
            ThreadsPerIO      = Constants::AMDGCN_WAVE_SIZE,
            ElementCount      = BlockDim * BlockK,
            UnpackedSize      = ElementCount / ThreadsPerIO,
            PackedSize        = (UnpackedSize + PackTraits<DataT>::PackRatio - 1u) / PackTraits<DataT>::PackRatio,
            PackedVRegCount   = PackedSize,
            UnpackedVRegCount = UnpackedSize
        };
        static_assert(ElementCount % ThreadsPerIO == 0u, "Element count must be divisible by threads per wave");
    };

    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT = void>
    class alignas(16) fragment : detail::LayoutCheck<MatrixT, DataLayoutT>
    {
        using Shape  = IOShape<MatrixT, BlockM, BlockN, BlockK>;
        using Config = detail::FragConfig<MatrixT, BlockM, BlockN, BlockK, DataT>;

    public:
        using IOTraits = ::rocwmma::IOTraits<Shape::BlockDim, Shape::KDim, DataT>;

        struct Traits
        {
            using AccessT  = VecT<typename PackTraits<DataT>::UnpackedT, IOTraits::UnpackedSize>;
            using StorageT = VecT<typename PackTraits<DataT>::PackedT, IOTraits::PackedSize>;
            constexpr static uint32_t Size = IOTraits::UnpackedSize;
            static_assert(IOTraits::PackedVRegCount >= 1, "Fragments must occupy at least one packed register");
            static_assert(IOTraits::UnpackedSize % IOTraits::PackedSize == 0, "Unable to pack fragment elements");
        };
        static_assert(Config::Map::size == Traits::Size, "register map and fragment size disagree");

        ROCWMMA_DEVICE fragment()                      = default;
        ROCWMMA_DEVICE fragment(const fragment& other) = default;
        ROCWMMA_DEVICE fragment& operator=(const fragment& other) = default;

        ROCWMMA_DEVICE inline DataT& operator[](uint32_t index)
        {
            return x[index];
        }
        ROCWMMA_DEVICE inline DataT const& operator[](uint32_t index) const
        {
            return x[index];
        }
        ROCWMMA_DEVICE inline typename Traits::StorageT& operator*()
        {
            return mStorage;
        }
        ROCWMMA_DEVICE inline typename Traits::StorageT const& operator*() const
        {
            return mStorage;
        }

        ROCWMMA_HOST_DEVICE constexpr static inline uint32_t height()
        {
            return Shape::BlockHeight;
        }
        ROCWMMA_HOST_DEVICE constexpr static inline uint32_t width()
        {
            return Shape::BlockWidth;
        }
        ROCWMMA_HOST_DEVICE constexpr static inline uint32_t blockDim()
        {
            return Shape::BlockDim;
        }
        ROCWMMA_HOST_DEVICE constexpr static inline uint32_t kDim()
        {
            return Shape::KDim;
        }
        ROCWMMA_HOST_DEVICE constexpr static inline uint32_t size()
        {
            return Traits::Size;
        }

        // Three views of the same registers
        union
        {
            typename Traits::StorageT mStorage; // packed 32-bit words
            typename Traits::AccessT  mAccess; // element vector
            DataT                     x[Traits::Size]; // element array
        };
        static_assert(sizeof(typename Traits::AccessT) == sizeof(typename Traits::StorageT),
                      "the packed register view and the element array of a fragment must have the same size");

        constexpr static uint32_t num_elements = Traits::Size;
        using element_type                     = DataT;
    };

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        fill_fragment(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag, DataT value)
    {
#pragma unroll
        for(uint32_t i = 0; i < frag.num_elements; ++i)
            frag.x[i] = value;
    }

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        load_matrix_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                         const DataT*                                                   data,
                         uint32_t                                                       ldm)
    {
        static_assert(!std::is_same<DataLayoutT, void>::value,
                      "this fragment type has no data layout: name one in the fragment's template arguments, or call the "
                      "overload that takes the layout at run time");
        using Config = detail::FragConfig<MatrixT, BlockM, BlockN, BlockK, DataT>;
        using IO     = typename Config::template IO<DataLayoutT>;
        detail::FragmentMover<IO, DataT>::load(frag.x, data, ldm);
    }

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
    ROCWMMA_DEVICE ROCWMMA_INLINE void load_matrix_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT>& frag,
                                                        const DataT*                                      data,
                                                        uint32_t                                          ldm,
                                                        layout_t                                          layout)
    {
        using Config = detail::FragConfig<MatrixT, BlockM, BlockN, BlockK, DataT>;
        if(layout == layout_t::mem_row_major)
            detail::FragmentMover<typename Config::template IO<row_major>, DataT>::load(frag.x, data, ldm);
        else
            detail::FragmentMover<typename Config::template IO<col_major>, DataT>::load(frag.x, data, ldm);
    }

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        store_matrix_sync(DataT*                                                               data,
                          fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
                          uint32_t                                                             ldm)
    {
        static_assert(!std::is_same<DataLayoutT, void>::value,
                      "this fragment type has no data layout: name one in the fragment's template arguments, or call the "
                      "overload that takes the layout at run time");
        using Config = detail::FragConfig<MatrixT, BlockM, BlockN, BlockK, DataT>;
        using IO     = typename Config::template IO<DataLayoutT>;
        detail::FragmentMover<IO, DataT>::store(data, frag.x, ldm);
    }

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
    ROCWMMA_DEVICE ROCWMMA_INLINE void store_matrix_sync(DataT*                                                  data,
                                                         fragment<MatrixT, BlockM, BlockN, BlockK, DataT> const& frag,
                                                         uint32_t                                                ldm,
                                                         layout_t                                                layout)
    {
        using Config = detail::FragConfig<MatrixT, BlockM, BlockN, BlockK, DataT>;
        if(layout == layout_t::mem_row_major)
            detail::FragmentMover<typename Config::template IO<row_major>, DataT>::store(data, frag.x, ldm);
        else
            detail::FragmentMover<typename Config::template IO<col_major>, DataT>::store(data, frag.x, ldm);
    }

    // D = A * B + C on fragments.  c may alias d.
    template <uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename InputTA,
              typename InputTB,
              typename ComputeT,
              typename LayoutA,
              typename LayoutB,
              typename LayoutC,
              typename LayoutD>
    ROCWMMA_DEVICE ROCWMMA_INLINE void
        mma_sync(fragment<accumulator, BlockM, BlockN, BlockK, ComputeT, LayoutD>&       d,
                 fragment<matrix_a, BlockM, BlockN, BlockK, InputTA, LayoutA> const&     a,
                 fragment<matrix_b, BlockM, BlockN, BlockK, InputTB, LayoutB> const&     b,
                 fragment<accumulator, BlockM, BlockN, BlockK, ComputeT, LayoutC> const& c)
    {
#if ROCWMMA_ARCH_GFX950 // device pass only: the host pass sees an empty body
        using MapA   = typename detail::FragConfig<matrix_a, BlockM, BlockN, BlockK, InputTA>::Map;
        using MapB   = typename detail::FragConfig<matrix_b, BlockM, BlockN, BlockK, InputTB>::Map;
        using MapAcc = typename detail::FragConfig<accumulator, BlockM, BlockN, BlockK, ComputeT>::Map;
        static_assert(sizeof(InputTA) == sizeof(InputTB) && MapA::kpack == MapB::kpack,
                      "A and B fragments must use the same K packing");
        static_assert(MapA::tile == MapAcc::tile && MapB::tile == MapAcc::tile && MapAcc::tileN == MapAcc::tile,
                      "blocks with an edge of 8 can be loaded, stored and filled but not multiplied");
        // The accumulator is kept transposed: the instruction's row operand is B, its column
        // operand is A (see fragment_map.hpp).
        // Compute types narrower than 32 bits (f16, bf16, __half accumulators): the matrix cores
        // accumulate in f32 only, so the accumulator is widened, multiplied and narrowed again in
        // every call, as the reference does (library/include/rocwmma/internal/mfma_impl.hpp:108-155).
        constexpr bool NarrowCompute = sizeof(ComputeT) < 4u;
        using NativeT                = std::conditional_t<NarrowCompute, float32_t, ComputeT>;
        using Op = detail::Mfma<detail::TypeInfo<InputTB>::cls,
                                detail::TypeInfo<InputTA>::cls,
                                NativeT,
                                MapAcc::tile,
                                MapA::mmaKPack>;
        static_assert(Op::supported,
                      "no gfx950 MFMA instruction for this combination of input types, "
                      "accumulator type, block size and BlockK");
        using Acc = typename Op::Acc;
        static_assert(sizeof(Acc) == MapAcc::perBlock * sizeof(NativeT), "accumulator block size mismatch");

        Acc acc[MapAcc::nbi][MapAcc::nbj];
#pragma unroll
        for(uint32_t bi = 0; bi < MapAcc::nbi; ++bi)
#pragma unroll
            for(uint32_t bj = 0; bj < MapAcc::nbj; ++bj)
            {
                if constexpr(NarrowCompute)
                {
#pragma unroll
                    for(uint32_t e = 0; e < MapAcc::perBlock; ++e)
                        acc[bi][bj][e] = static_cast<float32_t>(c.x[MapAcc::blockIndex(bi, bj) * MapAcc::perBlock + e]);
                }
                else
                    acc[bi][bj] = *reinterpret_cast<const Acc*>(&c.x[MapAcc::blockIndex(bi, bj) * MapAcc::perBlock]);
            }

            // K outermost so consecutive instructions write different accumulators
#pragma unroll
        // (an fp8 wide-K instruction takes the registers of two consecutive K steps)
        for(uint32_t ks = 0; ks < MapA::nmma; ++ks)
#pragma unroll
            for(uint32_t bi = 0; bi < MapAcc::nbi; ++bi)
#pragma unroll
                for(uint32_t bj = 0; bj < MapAcc::nbj; ++bj)
                    acc[bi][bj] = Op::exec(&b.x[MapB::chunkIndex(bj, ks * MapB::mmaSteps) * MapB::kpack],
                                           &a.x[MapA::chunkIndex(bi, ks * MapA::mmaSteps) * MapA::kpack],
                                           acc[bi][bj]);

#pragma unroll
        for(uint32_t bi = 0; bi < MapAcc::nbi; ++bi)
#pragma unroll
            for(uint32_t bj = 0; bj < MapAcc::nbj; ++bj)
            {
                if constexpr(NarrowCompute)
                {
#pragma unroll
                    for(uint32_t e = 0; e < MapAcc::perBlock; ++e)
                        d.x[MapAcc::blockIndex(bi, bj) * MapAcc::perBlock + e] = static_cast<ComputeT>(acc[bi][bj][e]);
                }
                else
                    *reinterpret_cast<Acc*>(&d.x[MapAcc::blockIndex(bi, bj) * MapAcc::perBlock]) = acc[bi][bj];
            }
#else
        (void)d, (void)a, (void)b, (void)c;
#endif // ROCWMMA_ARCH_GFX950
    }

    // Workgroup barrier that also orders LDS traffic.
    ROCWMMA_DEVICE ROCWMMA_INLINE void synchronize_workgroup()
    {
        __syncthreads();
    }

    // ---- accessors (reference: library/include/rocwmma/internal/accessors.hpp:35-89) --------
    template <typename FragT>
    struct GetDataType;
    template <typename FragT>
    struct GetIOShape;
    template <typename FragT>
    struct GetDataLayout;
    template <typename FragT>
    struct GetMappingUtil;
    template <typename FragT>
    struct GetIOTraits;

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    struct GetDataType<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
    {
        using type = DataT;
    };
    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    struct GetIOShape<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
    {
        using type = IOShape<MatrixT, BlockM, BlockN, BlockK>;
    };
    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    struct GetDataLayout<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
    {
        using type = detail::DataSpace<DataLayoutT>;
    };
    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    struct GetMappingUtil<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
    {
        using IOShapeT = IOShape<MatrixT, BlockM, BlockN, BlockK>;
        using type     = MappingUtil<IOShapeT::BlockHeight, IOShapeT::BlockWidth, DataT, DataLayoutT>;
    };
    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    struct GetIOTraits<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
    {
        using type = typename fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>::IOTraits;
    };

    // I/O description of a fragment (reference: accessors.hpp:43-49): here only its traits
    template <typename FragT>
    struct GetIOConfig;
    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
    struct GetIOConfig<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
    {
        struct type
        {
            using IOTraits = typename fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>::IOTraits;
            using IOShape  = rocwmma::IOShape<MatrixT, BlockM, BlockN, BlockK>;
        };
    };
    template <typename FragT>
    using GetIOConfig_t = typename GetIOConfig<std::decay_t<FragT>>::type;

    template <typename FragT>
    using GetDataType_t = typename GetDataType<std::decay_t<FragT>>::type;
    template <typename FragT>
    using GetIOShape_t = typename GetIOShape<std::decay_t<FragT>>::type;
    template <typename FragT>
    using GetDataLayout_t = typename GetDataLayout<std::decay_t<FragT>>::type;
    template <typename FragT>
    using GetMappingUtil_t = typename GetMappingUtil<std::decay_t<FragT>>::type;
    template <typename FragT>
    using GetIOTraits_t = typename GetIOTraits<std::decay_t<FragT>>::type;

} // namespace rocwmma

#endif // ROCWMMA_API_HPP
