// Fragment transforms: transpose and data-layout change.
//
// Same names and meaning as rocWMMA's transforms API (reference:
// library/include/rocwmma/rocwmma_transforms.hpp:36-66, rocwmma_transforms_impl.hpp:56-255).
// In this library the register layout of a fragment does not depend on its in-memory data
// layout, and matrix_a / matrix_b fragments of mirrored shape hold mirrored elements in the
// same registers (lane = row of A = column of B, registers = run of K).  Both transforms
// are therefore pure re-typing of the same registers -- no cross-lane traffic at all, where
// the reference needs AOS<->SOA shuffles for applyDataLayout.
//
//   applyTranspose:  fragment<matrix_a, M, N, K, T, L>  <->  fragment<matrix_b, N, M, K, T, ortho(L)>
//   applyDataLayout<L2, WaveCount>:  fragment<Ctx, M, N, K, T, L>  ->  fragment<Ctx, M, N, K, T, L2>
//
// WaveCount (cooperative fragments) is accepted and not needed: a wave's share of a
// cooperative fragment is layout independent too.
#ifndef ROCWMMA_TRANSFORMS_API_HPP
#define ROCWMMA_TRANSFORMS_API_HPP

#include "rocwmma.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <typename Layout>
        struct OrthoLayout;
        template <>
        struct OrthoLayout<row_major>
        {
            using type = col_major;
        };
        template <>
        struct OrthoLayout<col_major>
        {
            using type = row_major;
        };

        template <typename FragT>
        struct ApplyTranspose;

        template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
        struct ApplyTranspose<fragment<matrix_a, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
        {
            using Type = fragment<matrix_b, BlockN, BlockM, BlockK, DataT, typename OrthoLayout<DataLayoutT>::type>;
        };
        template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
        struct ApplyTranspose<fragment<matrix_b, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
        {
            using Type = fragment<matrix_a, BlockN, BlockM, BlockK, DataT, typename OrthoLayout<DataLayoutT>::type>;
        };

        template <typename FragT, typename NewDataLayoutT>
        struct ApplyDataLayout;

        template <typename MatrixT,
                  uint32_t BlockM,
                  uint32_t BlockN,
                  uint32_t BlockK,
                  typename DataT,
                  typename DataLayoutT,
                  typename NewDataLayoutT>
        struct ApplyDataLayout<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>, NewDataLayoutT>
        {
            using Type = fragment<MatrixT, BlockM, BlockN, BlockK, DataT, NewDataLayoutT>;
        };

        // A fragment seen as a plain register file: 64 lanes x (registers) elements.
        template <typename FragT>
        struct ApplyRegisterFile;

        template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
        struct ApplyRegisterFile<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
        {
        private:
            using FragT = fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>;

        public:
            using Type = fragment<matrix_b, 1u, Constants::AMDGCN_WAVE_SIZE, FragT::num_elements, DataT, row_major>;
        };

        // Re-types a fragment reference, keeping const-ness and value category.
        template <typename To, typename From>
        ROCWMMA_DEVICE ROCWMMA_INLINE decltype(auto) retype(From&& frag)
        {
            using Plain = std::remove_reference_t<From>;
            static_assert(sizeof(To) == sizeof(std::remove_cv_t<Plain>), "re-typed fragments must be the same size");
            if constexpr(std::is_lvalue_reference<From&&>::value)
            {
                if constexpr(std::is_const<Plain>::value)
                    return reinterpret_cast<To const&>(frag);
                else
                    return reinterpret_cast<To&>(frag);
            }
            else
            {
                // temporaries are returned by value
                To out;
#pragma unroll
                for(uint32_t i = 0; i < To::num_elements; ++i)
                    out.x[i] = frag.x[i];
                return out;
            }
        }
    } // namespace detail

    template <typename FragT>
    using ApplyTranspose_t = typename detail::ApplyTranspose<std::decay_t<FragT>>::Type;

    template <typename FragT, typename NewDataLayoutT>
    using ApplyDataLayout_t = typename detail::ApplyDataLayout<std::decay_t<FragT>, NewDataLayoutT>::Type;

    template <typename FragT>
    using ApplyRegisterFile_t = typename detail::ApplyRegisterFile<std::decay_t<FragT>>::Type;

    template <typename FragT>
    ROCWMMA_DEVICE static ROCWMMA_INLINE decltype(auto) applyTranspose(FragT&& frag)
    {
        return detail::retype<ApplyTranspose_t<FragT>>(std::forward<FragT>(frag));
    }

    template <typename DataLayoutT, uint32_t WaveCount = 1, typename FragT>
    ROCWMMA_DEVICE static ROCWMMA_INLINE decltype(auto) applyDataLayout(FragT&& frag)
    {
        return detail::retype<ApplyDataLayout_t<FragT, DataLayoutT>>(std::forward<FragT>(frag));
    }

} // namespace rocwmma

#endif // ROCWMMA_TRANSFORMS_API_HPP
