// Block-scaled (OCP microscaling) fp8 / bf8 GEMM: D = alpha * (A . 2^(SA - 127)) * (B . 2^(SB - 127)) + beta * C,
// one E8M0 scale per 32 elements along K of every row of A and every column of B.
//
// The reference has no block-scaled path (its fp8 GEMM tests multiply unscaled operands,
// test/gemm/gemm_common_test_params.hpp:170-196); this is the CDNA4 form of the same GEMM for
// quantised inference, where the scales are applied inside the matrix cores
// (v_mfma_scale_f32_*_f8f6f4) at no cost in instructions.
//
// Kernels here: one output block per wave, operands and scales straight from global memory through the
// fragment API (rocwmma_mx.hpp) -- every layout pair, every shape in whole blocks; and the kernel that
// re-orders the scales for the blocked kernel (gemm_blocked.hip, Scaled configurations).
#include "common.hpp"

#include <rocwmma/rocwmma_mx.hpp>

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        constexpr uint32_t kWavesX = 2; // along M  (blockDim.x = 64 * kWavesX)
        constexpr uint32_t kWavesY = 2; // along N  (blockDim.y = kWavesY)

        template <typename InT, typename LA, typename LB, uint32_t B, uint32_t BK>
        __global__ void __launch_bounds__(64 * kWavesX * kWavesY) gemmMxWaveTileKernel(GemmArgs g, MxScales s)
        {
            using FragA   = fragment<matrix_a, B, B, BK, InT, LA>;
            using FragB   = fragment<matrix_b, B, B, BK, InT, LB>;
            using FragAcc = fragment<accumulator, B, B, BK, float32_t>;
            using MapA    = GetDataLayout_t<FragA>;
            using MapB    = GetDataLayout_t<FragB>;

            const uint32_t waveRow = (blockIdx.x * blockDim.x + threadIdx.x) / Constants::AMDGCN_WAVE_SIZE;
            const uint32_t waveCol = blockIdx.y * blockDim.y + threadIdx.y;
            const uint32_t cRow    = waveRow * B;
            const uint32_t cCol    = waveCol * B;
            if(cRow >= g.m || cCol >= g.n)
                return;

            FragAcc acc;
            fill_fragment(acc, 0.0f);

            const InT* aPtr = static_cast<const InT*>(g.a) + (std::is_same<LA, row_major>::value ? static_cast<size_t>(cRow) * g.lda : cRow);
            const InT* bPtr = static_cast<const InT*>(g.b) + (std::is_same<LB, row_major>::value ? cCol : static_cast<size_t>(cCol) * g.ldb);
            const mx::scale_t* saPtr = s.a + static_cast<size_t>(cRow) * s.lda;
            const mx::scale_t* sbPtr = s.b + static_cast<size_t>(cCol) * s.ldb;
            const uint32_t     aStep = MapA::fromMatrixCoord(make_coord2d(0u, BK), g.lda);
            const uint32_t     bStep = MapB::fromMatrixCoord(make_coord2d(BK, 0u), g.ldb);

            for(uint32_t i = 0; i < g.k; i += BK)
            {
                FragA                     fa;
                FragB                     fb;
                mx::scale_fragment<FragA> sa;
                mx::scale_fragment<FragB> sb;
                load_matrix_sync(fa, aPtr, g.lda);
                load_matrix_sync(fb, bPtr, g.ldb);
                mx::load_scale_sync(sa, saPtr, s.lda);
                mx::load_scale_sync(sb, sbPtr, s.ldb);
                mx::mma_sync(acc, fa, sa, fb, sb, acc);
                aPtr += aStep;
                bPtr += bStep;
                saPtr += BK / mx::BLOCK_SIZE;
                sbPtr += BK / mx::BLOCK_SIZE;
            }

            const layout_t layoutC = g.layoutC == ROCWMMA_AMD_ROW_MAJOR ? mem_row_major : mem_col_major;
            const float*   c       = static_cast<const float*>(g.c);
            float*         d       = static_cast<float*>(g.d);
            const size_t   cOff = layoutC == mem_row_major ? static_cast<size_t>(cRow) * g.ldc + cCol : static_cast<size_t>(cCol) * g.ldc + cRow;
            const size_t   dOff = layoutC == mem_row_major ? static_cast<size_t>(cRow) * g.ldd + cCol : static_cast<size_t>(cCol) * g.ldd + cRow;
            FragAcc        fc;
            if(g.beta != 0.0f)
            {
                load_matrix_sync(fc, c + cOff, g.ldc, layoutC);
#pragma unroll
                for(uint32_t i = 0; i < fc.num_elements; ++i)
                    fc.x[i] = g.alpha * acc.x[i] + g.beta * fc.x[i];
            }
            else
            {
#pragma unroll
                for(uint32_t i = 0; i < fc.num_elements; ++i)
                    fc.x[i] = g.alpha * acc.x[i];
            }
            store_matrix_sync(d + dOff, fc, g.ldd, layoutC);
        }

        template <typename InT, typename LA, typename LB, uint32_t B, uint32_t BK>
        int launchOne(GemmArgs const& g, MxScales const& s, hipStream_t stream)
        {
            dim3 block(64 * kWavesX, kWavesY);
            dim3 grid((g.m + B * kWavesX - 1u) / (B * kWavesX), (g.n + B * kWavesY - 1u) / (B * kWavesY));
            hipLaunchKernelGGL((gemmMxWaveTileKernel<InT, LA, LB, B, BK>), grid, block, 0, stream, g, s);
            return launchStatus();
        }

        // 16-wide blocks walk K in steps of 128 (v_mfma_scale_f32_16x16x128_f8f6f4), 32-wide blocks in steps
        // of 64 (32x32x64): K that is a multiple of 64 only needs m and n in whole 32-wide blocks.
        template <typename InT, typename LA, typename LB>
        int pickBlock(GemmArgs const& g, MxScales const& s, hipStream_t stream)
        {
            if(g.m % 16u != 0u || g.n % 16u != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            if(g.k % 128u == 0u)
                return launchOne<InT, LA, LB, 16, 128>(g, s, stream);
            if(g.k % 64u == 0u && g.m % 32u == 0u && g.n % 32u == 0u)
                return launchOne<InT, LA, LB, 32, 64>(g, s, stream);
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        }

        template <typename InT>
        int pickLayout(int layoutA, int layoutB, GemmArgs const& g, MxScales const& s, hipStream_t stream)
        {
            const bool aRow = layoutA == ROCWMMA_AMD_ROW_MAJOR;
            const bool bRow = layoutB == ROCWMMA_AMD_ROW_MAJOR;
            if(aRow && !bRow)
                return pickBlock<InT, row_major, col_major>(g, s, stream);
            if(aRow && bRow)
                return pickBlock<InT, row_major, row_major>(g, s, stream);
            if(!aRow && !bRow)
                return pickBlock<InT, col_major, col_major>(g, s, stream);
            return pickBlock<InT, col_major, row_major>(g, s, stream);
        }

        // Re-orders the scales of both operands for the blocked kernels.  One workgroup per (operand, group
        // of 64 rows): it reads the group's scale rows in pieces of 128 bytes (4096 elements of K) with
        // coalesced accesses, each line once, into LDS, and writes from there the 8 bytes every lane of the
        // GEMM loads per pair of K stages (256 bytes of K):
        //   16-wide blocks: lane l = row l % 16 of a block, K block l / 16 of a stage; bytes [block 0..3][stage 0..1]
        //   32-wide blocks: lane l = row l % 32 of a block, K block l / 32 of a step;  bytes [block 0..1][step 0..3]
        // Rows and K blocks beyond the operand get the scale 1 (they only ever meet zero operands).
        // (A first version gathered 8 bytes from 8 different scale rows per thread straight from global
        // memory, one workgroup per group and pair: every 128-byte line was fetched by 16 workgroups on
        // different XCDs, 7 us for the 1.9 MB of scales of a 4096 x 14336 x 4096 problem.)
        constexpr uint32_t kPackRowBytes = 128u; // scale bytes of a row per piece
        constexpr uint32_t kPackRowPitch = 132u; // LDS pitch of a row (byte reads down a column spread over the banks)

        template <bool Wide32>
        __global__ void __launch_bounds__(256) mxPackScalesKernel(MxScales s, uint32_t m, uint32_t n, uint32_t kBlocks, uint32_t pairs,
                                                                  uint32_t groupsA, uint2* packedA, uint2* packedB)
        {
            __shared__ uint8_t tile[64u * kPackRowPitch];
            const bool     isA    = blockIdx.x < groupsA;
            const uint32_t group  = isA ? blockIdx.x : blockIdx.x - groupsA;
            const uint8_t* scales = isA ? s.a : s.b;
            const uint32_t ld     = isA ? s.lda : s.ldb;
            const uint32_t rows   = isA ? m : n;
            uint2*         packed = isA ? packedA : packedB;
            const bool     dwords = (reinterpret_cast<uintptr_t>(scales) & 3u) == 0u && ld % 4u == 0u;

            for(uint32_t kb0 = 0; kb0 < pairs * 8u; kb0 += kPackRowBytes)
            {
                // 64 rows x 128 bytes -> LDS, consecutive threads along a row
                for(uint32_t idx = threadIdx.x; idx < 64u * (kPackRowBytes / 4u); idx += 256u)
                {
                    const uint32_t r   = idx / (kPackRowBytes / 4u);
                    const uint32_t kb  = kb0 + (idx % (kPackRowBytes / 4u)) * 4u;
                    const uint32_t row = group * 64u + r;
                    uint32_t       v   = 0x7f7f7f7fu;
                    if(row < rows && kb < kBlocks)
                    {
                        const uint8_t* src = scales + static_cast<size_t>(row) * ld + kb;
                        if(dwords && kb + 4u <= kBlocks)
                            v = *reinterpret_cast<const uint32_t*>(src);
                        else
                        {
                            v = 0u;
#pragma unroll
                            for(uint32_t j = 0; j < 4u; ++j)
                                v |= static_cast<uint32_t>(kb + j < kBlocks ? src[j] : 127u) << (8u * j);
                        }
                    }
                    // (pitch 132: 4-byte aligned)
                    *reinterpret_cast<uint32_t*>(tile + r * kPackRowPitch + (kb - kb0)) = v;
                }
                __syncthreads();
                // 16 pairs of stages x 64 lanes x 8 bytes
                for(uint32_t o = threadIdx.x; o < (kPackRowBytes / 8u) * 64u; o += 256u)
                {
                    const uint32_t pairHere = o / 64u, lane = o % 64u;
                    const uint32_t pair     = kb0 / 8u + pairHere;
                    if(pair >= pairs)
                        continue;
                    uint32_t word[2] = {0u, 0u};
                    if constexpr(Wide32)
                    {
#pragma unroll
                        for(uint32_t blk = 0; blk < 2u; ++blk)
#pragma unroll
                            for(uint32_t step = 0; step < 4u; ++step)
                                word[blk] |= static_cast<uint32_t>(tile[(blk * 32u + lane % 32u) * kPackRowPitch + pairHere * 8u + step * 2u + lane / 32u])
                                             << (8u * step);
                    }
                    else
                    {
#pragma unroll
                        for(uint32_t blk = 0; blk < 4u; ++blk)
#pragma unroll
                            for(uint32_t st = 0; st < 2u; ++st)
                                word[blk / 2u] |= static_cast<uint32_t>(tile[(blk * 16u + lane % 16u) * kPackRowPitch + pairHere * 8u + st * 4u + lane / 16u])
                                                  << (8u * ((blk % 2u) * 2u + st));
                    }
                    packed[(static_cast<size_t>(group) * pairs + pair) * 64u + lane] = make_uint2(word[0], word[1]);
                }
                __syncthreads();
            }
        }
    } // namespace

    int launchMxPackScales(MxScales const& s, uint32_t m, uint32_t n, uint32_t k, void* packedA, void* packedB, bool wide32,
                           hipStream_t stream)
    {
        // (an operand without scales is left as it is in the workspace: a caller with fixed weights packs
        // those once and the tokens' scales per call)
        const uint32_t pairs   = (k + 255u) / 256u;
        const uint32_t groupsA = s.a ? (m + 63u) / 64u : 0u;
        const uint32_t groupsB = s.b ? (n + 63u) / 64u : 0u;
        if(groupsA + groupsB == 0u)
            return ROCWMMA_AMD_OK;
        const dim3     grid(groupsA + groupsB);
        if(wide32)
            hipLaunchKernelGGL(mxPackScalesKernel<true>, grid, dim3(256), 0, stream, s, m, n, k / 32u, pairs, groupsA,
                               static_cast<uint2*>(packedA), static_cast<uint2*>(packedB));
        else
            hipLaunchKernelGGL(mxPackScalesKernel<false>, grid, dim3(256), 0, stream, s, m, n, k / 32u, pairs, groupsA,
                               static_cast<uint2*>(packedA), static_cast<uint2*>(packedB));
        return launchStatus();
    }

    int launchGemmMxWaveTile(int dtypeIn, int layoutA, int layoutB, GemmArgs const& g, MxScales const& s, hipStream_t stream)
    {
        if(static_cast<uint64_t>(g.lda) * 256u >= (1ull << 32) || static_cast<uint64_t>(g.ldb) * 256u >= (1ull << 32))
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        if(dtypeIn == ROCWMMA_AMD_E4M3)
            return pickLayout<float8_t>(layoutA, layoutB, g, s, stream);
        if(dtypeIn == ROCWMMA_AMD_E5M2)
            return pickLayout<bfloat8_t>(layoutA, layoutB, g, s, stream);
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    }

} // namespace rocwmma_amd
