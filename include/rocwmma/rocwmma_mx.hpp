// Block-scaled (OCP microscaling, "MX") multiply-accumulate for fp8 / bf8 fragments on gfx950.
//
// Extension of the rocWMMA-style API: the reference has no counterpart (its fp8 path multiplies
// unscaled operands, library/include/rocwmma/internal/mfma_impl.hpp).  In the MX formats every 32
// consecutive elements along K of an operand share one E8M0 scale, a biased power-of-two exponent:
//
//     value(row, k) = element(row, k) * 2^(scale(row, k / 32) - 127)          (scale = 255: NaN)
//
// The CDNA4 wide-K instructions (v_mfma_scale_f32_16x16x128_f8f6f4 / _32x32x64_) apply both
// operands' scales inside the matrix core: next to its 32 bytes of operand, every lane passes one
// scale byte per multiplicand.  The scale of lane l belongs to row (column) l % tile and K block
// l / tile of the instruction's K range (four blocks of 32 for 16-wide, two for 32-wide blocks) --
// not to the lane's own operand bytes, which come as two runs of 16 from the two halves of that
// range (see internal/fragment_map.hpp).  A scale fragment therefore holds one byte per lane and
// instruction.
//
//   fragment<matrix_a, 16, 16, 128, float8_t, row_major> a;     // K a multiple of 128 (16-wide blocks)
//   mx::scale_fragment<decltype(a)>                      sa;    // or of 64 (32-wide blocks)
//   load_matrix_sync(a, aPtr, lda);
//   mx::load_scale_sync(sa, scaleA + row0 * ldsa + k0 / 32, ldsa);
//   mx::mma_sync(acc, a, sa, b, sb, acc);
//
// Scales live in memory as a (rows of A) x (K / 32) byte matrix for A and a (columns of B) x (K / 32)
// byte matrix for B, K blocks contiguous, whatever the data layout of the operand itself.
#ifndef ROCWMMA_MX_HPP
#define ROCWMMA_MX_HPP

#include "rocwmma.hpp"

namespace rocwmma
{
    namespace mx
    {
        // Elements along K that share one scale.
        constexpr uint32_t BLOCK_SIZE = 32u;

        // E8M0: eight exponent bits, bias 127, no sign, no mantissa.
        using scale_t = uint8_t;
        constexpr scale_t SCALE_ONE = 127u;

        namespace detail
        {
            template <typename FragT>
            struct ScaleConfig;

            template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename LayoutT>
            struct ScaleConfig<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, LayoutT>>
            {
                static_assert(std::is_same<MatrixT, matrix_a>::value || std::is_same<MatrixT, matrix_b>::value,
                              "scales belong to matrix_a / matrix_b fragments");
                static_assert(std::is_same<DataT, float8_t>::value || std::is_same<DataT, bfloat8_t>::value,
                              "block scales: fp8 / bf8 fragments");
                using Map = typename ::rocwmma::detail::FragConfig<MatrixT, BlockM, BlockN, BlockK, DataT>::Map;
                static_assert(Map::mmaSteps == 2u && Map::mmaKPack == BLOCK_SIZE,
                              "scaled instructions are the wide-K ones: BlockK a multiple of 128 for 16-wide "
                              "blocks, of 64 for 32-wide blocks");
            };
        } // namespace detail

        // One E8M0 scale per lane and instruction of the fragment it belongs to (low byte of x[i]; the
        // other bytes are ignored by mma_sync): x[db * nmma + s] is the scale of row (column)
        // db * tile + lane % tile and K block s * groups + lane / tile.
        template <typename FragT>
        struct scale_fragment
        {
            using Map                              = typename detail::ScaleConfig<FragT>::Map;
            constexpr static uint32_t num_elements = Map::ndim * Map::nmma;
            uint32_t                  x[num_elements];
        };

        template <typename FragT>
        ROCWMMA_DEVICE ROCWMMA_INLINE void fill_scale(scale_fragment<FragT>& s, scale_t value)
        {
#pragma unroll
            for(uint32_t c = 0; c < s.num_elements; ++c)
                s.x[c] = value;
        }

        // `scales` points at the scale of the fragment's first row (matrix_a) or column (matrix_b)
        // and first K block; the scale of row r, K block kb is scales[r * ld + kb].
        template <typename FragT>
        ROCWMMA_DEVICE ROCWMMA_INLINE void load_scale_sync(scale_fragment<FragT>& s, const scale_t* scales, uint32_t ld)
        {
            using Map           = typename scale_fragment<FragT>::Map;
            const uint32_t lane = threadIdx.x % Constants::AMDGCN_WAVE_SIZE;
#pragma unroll
            for(uint32_t db = 0; db < Map::ndim; ++db)
#pragma unroll
                for(uint32_t i = 0; i < Map::nmma; ++i)
                    s.x[db * Map::nmma + i]
                        = scales[static_cast<size_t>(db * Map::tile + lane % Map::tile) * ld + i * Map::groups + lane / Map::tile];
        }

        // d = a * b + c with a and b scaled block-wise.
        template <uint32_t BlockM,
                  uint32_t BlockN,
                  uint32_t BlockK,
                  typename InputTA,
                  typename InputTB,
                  typename LayoutA,
                  typename LayoutB,
                  typename LayoutC,
                  typename LayoutD>
        ROCWMMA_DEVICE ROCWMMA_INLINE void
            mma_sync(fragment<accumulator, BlockM, BlockN, BlockK, float32_t, LayoutD>&                       d,
                     fragment<matrix_a, BlockM, BlockN, BlockK, InputTA, LayoutA> const&                      a,
                     scale_fragment<fragment<matrix_a, BlockM, BlockN, BlockK, InputTA, LayoutA>> const&      sa,
                     fragment<matrix_b, BlockM, BlockN, BlockK, InputTB, LayoutB> const&                      b,
                     scale_fragment<fragment<matrix_b, BlockM, BlockN, BlockK, InputTB, LayoutB>> const&      sb,
                     fragment<accumulator, BlockM, BlockN, BlockK, float32_t, LayoutC> const&                 c)
        {
#if ROCWMMA_ARCH_GFX950 // device pass only: the host pass sees an empty body
            using MapA   = typename ::rocwmma::detail::FragConfig<matrix_a, BlockM, BlockN, BlockK, InputTA>::Map;
            using MapB   = typename ::rocwmma::detail::FragConfig<matrix_b, BlockM, BlockN, BlockK, InputTB>::Map;
            using MapAcc = typename ::rocwmma::detail::FragConfig<accumulator, BlockM, BlockN, BlockK, float32_t>::Map;
            static_assert(MapA::tile == MapAcc::tile && MapB::tile == MapAcc::tile && MapAcc::tileN == MapAcc::tile,
                          "blocks with an edge of 8 cannot be multiplied");
            // (the accumulator is kept transposed: the instruction's first multiplicand is B)
            using Op = ::rocwmma::detail::MfmaScaled<::rocwmma::detail::TypeInfo<InputTB>::cls,
                                                     ::rocwmma::detail::TypeInfo<InputTA>::cls,
                                                     MapAcc::tile>;
            static_assert(Op::supported, "no scaled gfx950 MFMA instruction for these types and block size");
            using Acc = typename Op::Acc;

#pragma unroll
            for(uint32_t bi = 0; bi < MapAcc::nbi; ++bi)
#pragma unroll
                for(uint32_t bj = 0; bj < MapAcc::nbj; ++bj)
                {
                    const uint32_t at  = MapAcc::blockIndex(bi, bj) * MapAcc::perBlock;
                    Acc            acc = *reinterpret_cast<const Acc*>(&c.x[at]);
#pragma unroll
                    for(uint32_t ks = 0; ks < MapA::nmma; ++ks)
                        acc = Op::template exec<0, 0>(&b.x[MapB::chunkIndex(bj, ks * MapB::mmaSteps) * MapB::kpack],
                                                      &a.x[MapA::chunkIndex(bi, ks * MapA::mmaSteps) * MapA::kpack],
                                                      acc,
                                                      sb.x[bj * MapB::nmma + ks],
                                                      sa.x[bi * MapA::nmma + ks]);
                    *reinterpret_cast<Acc*>(&d.x[at]) = acc;
                }
#else
            (void)d, (void)a, (void)sa, (void)b, (void)sb, (void)c;
#endif // ROCWMMA_ARCH_GFX950
        }
    } // namespace mx
} // namespace rocwmma

#endif // ROCWMMA_MX_HPP
