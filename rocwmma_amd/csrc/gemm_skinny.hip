// Skinny quantised GEMM: D = alpha * A * B + beta * C for M <= 32 token rows against an
// N x K weight matrix (8-bit A row-major, B col-major, C/D row-major).
//
// At these shapes (the reference's GEMM kernels, samples/perf_hgemm.cpp:518-714, need whole
// 128-wide macro tiles in M and would leave most of the chip idle) the job is streaming the
// weights from HBM exactly once, so the kernel is built for memory-level parallelism, written
// with the public fragment API only:
//   * a workgroup of four waves owns 16*NBlocks weight rows and ALL token rows;
//   * the four waves split K; each wave walks its quarter in 128-byte steps with
//     16 x 16 x 128 fragments (one v_mfma_f32_16x16x128_f8f6f4, or two v_mfma_i32_16x16x64_i8),
//     so a weight row is read as whole 128-byte lines and many lines are in flight per wave;
//   * the four partial accumulators meet in LDS; the sum is formed in a fixed order, so the
//     result is deterministic (and bit-exact for int8).
#include "common.hpp"

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        constexpr uint32_t kSkinnyWaves = 4;
        constexpr uint32_t kSkinnyK     = 128; // K elements (= bytes) per fragment step

        template <typename InT, typename OutT, typename CompT, uint32_t MBlocks, uint32_t NBlocks>
        __global__ void __launch_bounds__(64 * kSkinnyWaves) gemmSkinnyKernel(uint32_t    m,
                                                                              uint32_t    n,
                                                                              uint32_t    k,
                                                                              InT const*  a,
                                                                              InT const*  b,
                                                                              OutT const* c,
                                                                              OutT*       d,
                                                                              uint32_t    lda,
                                                                              uint32_t    ldb,
                                                                              uint32_t    ldc,
                                                                              uint32_t    ldd,
                                                                              CompT       alpha,
                                                                              CompT       beta)
        {
            using FragA   = fragment<matrix_a, 16, 16, kSkinnyK, InT, row_major>;
            using FragB   = fragment<matrix_b, 16, 16, kSkinnyK, InT, col_major>;
            using FragAcc = fragment<accumulator, 16, 16, kSkinnyK, CompT>;
            using FragC   = fragment<accumulator, 16, 16, kSkinnyK, OutT, row_major>;
            constexpr uint32_t Blocks = MBlocks * NBlocks;

            extern __shared__ __attribute__((aligned(16))) char ldsRaw[];
            // partial[wave][block][lane] : the 4 accumulator registers of a lane as one 16-byte unit
            using Quad    = CompT __attribute__((ext_vector_type(4)));
            Quad* partial = reinterpret_cast<Quad*>(ldsRaw);

            const uint32_t lane = threadIdx.x & 63u;
            const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t n0   = blockIdx.x * NBlocks * 16u;
            const uint32_t kLen = k / kSkinnyWaves;
            const uint32_t kBeg = wave * kLen;

            FragAcc acc[MBlocks][NBlocks];
#pragma unroll
            for(uint32_t i = 0; i < MBlocks; ++i)
#pragma unroll
                for(uint32_t j = 0; j < NBlocks; ++j)
                    fill_fragment(acc[i][j], static_cast<CompT>(0));

            const InT* bPtr = b + static_cast<size_t>(n0) * ldb + kBeg;
            const InT* aPtr = a + kBeg;
#pragma unroll 8
            for(uint32_t kk = 0; kk < kLen; kk += kSkinnyK)
            {
                FragB fb[NBlocks];
#pragma unroll
                for(uint32_t j = 0; j < NBlocks; ++j)
                    load_matrix_sync(fb[j], bPtr + static_cast<size_t>(j * 16u) * ldb + kk, ldb);
#pragma unroll
                for(uint32_t i = 0; i < MBlocks; ++i)
                {
                    FragA fa;
                    load_matrix_sync(fa, aPtr + static_cast<size_t>(i * 16u) * lda + kk, lda);
#pragma unroll
                    for(uint32_t j = 0; j < NBlocks; ++j)
                        mma_sync(acc[i][j], fa, fb[j], acc[i][j]);
                }
            }

            // meet in LDS
#pragma unroll
            for(uint32_t i = 0; i < MBlocks; ++i)
#pragma unroll
                for(uint32_t j = 0; j < NBlocks; ++j)
                    partial[(wave * Blocks + i * NBlocks + j) * 64u + lane] = *reinterpret_cast<Quad*>(acc[i][j].x);
            __syncthreads();

            // block q is finished by wave q % 4: fixed summation order wave 0, 1, 2, 3
#pragma unroll
            for(uint32_t i = 0; i < MBlocks; ++i)
#pragma unroll
                for(uint32_t j = 0; j < NBlocks; ++j)
                {
                    const uint32_t q = i * NBlocks + j;
                    if(q % kSkinnyWaves != wave)
                        continue;
                    Quad sum = partial[(0u * Blocks + q) * 64u + lane];
#pragma unroll
                    for(uint32_t w = 1; w < kSkinnyWaves; ++w)
                        sum += partial[(w * Blocks + q) * 64u + lane];
                    const size_t row = i * 16u;
                    const size_t col = n0 + j * 16u;
                    FragC        fc;
                    if(beta != static_cast<CompT>(0))
                    {
                        load_matrix_sync(fc, c + row * ldc + col, ldc);
#pragma unroll
                        for(uint32_t e = 0; e < 4u; ++e)
                            fc.x[e] = static_cast<OutT>(alpha * sum[e] + beta * static_cast<CompT>(fc.x[e]));
                    }
                    else
                    {
#pragma unroll
                        for(uint32_t e = 0; e < 4u; ++e)
                            fc.x[e] = static_cast<OutT>(alpha * sum[e]);
                    }
                    store_matrix_sync(d + row * ldd + col, fc, ldd);
                }
        }

        template <typename InT, typename OutT, typename CompT, uint32_t MBlocks, uint32_t NBlocks>
        int launchOne(GemmArgs const& g, hipStream_t stream)
        {
            constexpr uint32_t lds    = kSkinnyWaves * MBlocks * NBlocks * 1024u;
            auto               kernel = gemmSkinnyKernel<InT, OutT, CompT, MBlocks, NBlocks>;
            if(lds > 65536u
               && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(lds))
                      != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            hipLaunchKernelGGL(kernel, dim3(g.n / (NBlocks * 16u)), dim3(64u * kSkinnyWaves), lds, stream, g.m, g.n, g.k,
                               static_cast<InT const*>(g.a), static_cast<InT const*>(g.b), static_cast<OutT const*>(g.c),
                               static_cast<OutT*>(g.d), g.lda, g.ldb, g.ldc, g.ldd, static_cast<CompT>(g.alpha),
                               static_cast<CompT>(g.beta));
            return launchStatus();
        }

        template <typename InT, typename OutT, typename CompT>
        int pickShape(GemmArgs const& g, hipStream_t stream)
        {
            if(g.m % 16u != 0u || g.m > 32u || g.k % (kSkinnyWaves * kSkinnyK) != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            const uint32_t mBlocks = g.m / 16u;
            // 16 weight rows per workgroup: the most workgroups and the most loads in flight
            if(g.n % 16u != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            if(mBlocks == 1u)
                return launchOne<InT, OutT, CompT, 1, 1>(g, stream);
            return launchOne<InT, OutT, CompT, 2, 1>(g, stream);
        }
    } // namespace

    int launchGemmSkinny(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream)
    {
        if(layoutA != ROCWMMA_AMD_ROW_MAJOR || layoutB != ROCWMMA_AMD_COL_MAJOR || g.layoutC != ROCWMMA_AMD_ROW_MAJOR)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        if(dtypeIn == ROCWMMA_AMD_I8 && dtypeOut == ROCWMMA_AMD_I32)
            return pickShape<int8_t, int32_t, int32_t>(g, stream);
        if(dtypeIn == ROCWMMA_AMD_E4M3 && dtypeOut == ROCWMMA_AMD_F32)
            return pickShape<float8_t, float32_t, float32_t>(g, stream);
        if(dtypeIn == ROCWMMA_AMD_E5M2 && dtypeOut == ROCWMMA_AMD_F32)
            return pickShape<bfloat8_t, float32_t, float32_t>(g, stream);
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    }

} // namespace rocwmma_amd
