// DLRM dot-interaction forward and backward for gfx950 (f16 storage, f32 accumulate).
//
// Semantics follow the reference's CPU reference dlrm_fwd_CPU / dlrm_bwd_CPU
// (test/reference_impl.hpp:83-179).  The reference GPU kernels (dlrmDotFwd, trilReconstruct,
// dlrmDotBwd: samples/simple_dlrm.cpp:184-441) tile the m x m Gram matrix in 16 x 16 blocks
// over a 3-D grid, bounce the f32 result through a global scratch matrix, scatter the lower
// triangle with 2-byte stores and need m % 16 == 0.  Here instead:
//
//   * one wave owns a whole sample: the m <= 32 feature rows are one 32-row MFMA operand, so
//     Z = F F^T is K/16 v_mfma_f32_32x32x16_f16 with the SAME registers as both multiplicands
//     (applyTranspose of the A fragment is the B fragment);
//   * a workgroup of 4 waves owns 8 consecutive samples, whose outputs are contiguous in
//     memory: results are assembled in LDS and leave as 16-byte coalesced stores;
//   * backward rebuilds the symmetric matrix G in registers from the LDS-staged upstream
//     gradient (no global m x m scratch, no second launch), reads F^T operands with the
//     transposing LDS load, and writes grad through LDS the same way.
//
// Both kernels are judged on bytes moved: forward reads m*k and writes k + m(m-1)/2 halves per
// sample; backward reads m*k + k + m(m-1)/2 and writes m*k + k.
#include "common.hpp"
#include <rocwmma/rocwmma_lds.hpp>
#include <rocwmma/rocwmma_transforms.hpp>

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        constexpr uint32_t kSamplesPerWg   = 8;
        constexpr uint32_t kWavesPerWg     = 4;
        constexpr uint32_t kSamplesPerWave = kSamplesPerWg / kWavesPerWg;
        constexpr uint32_t kMaxM           = 32;

        typedef uint32_t u32x4_t __attribute__((ext_vector_type(4), may_alias));
        typedef uint16_t u16_alias __attribute__((may_alias));

        ROCWMMA_DEVICE inline uint32_t trilIndex(uint32_t row, uint32_t col) // row > col
        {
            return (row * (row - 1u)) / 2u + col;
        }

        // Copies `halves` f16 values from LDS (16-byte aligned) to global (16-byte aligned),
        // whole workgroup, 16-byte accesses with a 2-byte tail.
        ROCWMMA_DEVICE inline void copyOut(float16_t* dst, const float16_t* ldsSrc, uint32_t halves)
        {
            const uint32_t vecs = halves / 8u;
            for(uint32_t i = threadIdx.x; i < vecs; i += blockDim.x)
                reinterpret_cast<u32x4_t*>(dst)[i] = reinterpret_cast<const u32x4_t*>(ldsSrc)[i];
            for(uint32_t i = vecs * 8u + threadIdx.x; i < halves; i += blockDim.x)
                dst[i] = ldsSrc[i];
        }

        ROCWMMA_DEVICE inline void copyIn(float16_t* ldsDst, const float16_t* src, uint32_t halves)
        {
            const uint32_t vecs = halves / 8u;
            for(uint32_t i = threadIdx.x; i < vecs; i += blockDim.x)
                reinterpret_cast<u32x4_t*>(ldsDst)[i] = reinterpret_cast<const u32x4_t*>(src)[i];
            for(uint32_t i = vecs * 8u + threadIdx.x; i < halves; i += blockDim.x)
                ldsDst[i] = src[i];
        }

        // ------------------------------------------------------------------ forward
        template <uint32_t K>
        __global__ void __launch_bounds__(64 * kWavesPerWg)
            dlrmFwdKernel(const float16_t* __restrict__ input, float16_t* __restrict__ output, uint32_t m, uint32_t batch)
        {
            constexpr uint32_t KSteps = K / 16u;
            using FragA               = fragment<matrix_a, 32, 32, 16, float16_t, row_major>;
            using FragAcc             = fragment<accumulator, 32, 32, 16, float32_t>;
            using AccMap              = detail::AccMap<32, 32, 32>;

            extern __shared__ __attribute__((aligned(16))) char ldsRaw[];
            float16_t* ldsOut = reinterpret_cast<float16_t*>(ldsRaw);

            const uint32_t width   = K + (m * (m - 1u)) / 2u;
            const uint32_t lane    = threadIdx.x & 63u;
            const uint32_t wave    = threadIdx.x >> 6;
            const uint32_t sample0 = blockIdx.x * kSamplesPerWg;
            const uint32_t nHere   = min(kSamplesPerWg, batch - sample0);
            const uint32_t row     = lane & 31u;
            const uint32_t kGroup  = lane >> 5;

#pragma unroll
            for(uint32_t s = 0; s < kSamplesPerWave; ++s)
            {
                const uint32_t local = wave * kSamplesPerWave + s;
                if(local >= nHere)
                    break;
                const float16_t* F = input + static_cast<size_t>(sample0 + local) * m * K;

                // operand registers: row `row`, k = ks*16 + kGroup*8 .. +7 ; rows >= m are zero
                FragA fa[KSteps];
#pragma unroll
                for(uint32_t ks = 0; ks < KSteps; ++ks)
                {
                    u32x4_t v = {0u, 0u, 0u, 0u};
                    if(row < m)
                        v = *reinterpret_cast<const u32x4_t*>(F + row * K + ks * 16u + kGroup * 8u);
                    *reinterpret_cast<u32x4_t*>(fa[ks].x) = v;
                }

                FragAcc acc;
                fill_fragment(acc, 0.0f);
#pragma unroll
                for(uint32_t ks = 0; ks < KSteps; ++ks)
                    mma_sync(acc, fa[ks], applyTranspose(fa[ks]), acc);

                float16_t* out = ldsOut + local * width;
                // bottom-MLP row: the lanes holding row 0 copy their operand registers
                if(row == 0u)
                {
#pragma unroll
                    for(uint32_t ks = 0; ks < KSteps; ++ks)
#pragma unroll
                        for(uint32_t j = 0; j < 8u; ++j)
                            out[ks * 16u + kGroup * 8u + j] = fa[ks].x[j];
                }
                // strict lower triangle, row by row
#pragma unroll
                for(uint32_t e = 0; e < FragAcc::num_elements; ++e)
                {
                    const uint32_t r = AccMap::rowOf(e, lane);
                    const uint32_t c = AccMap::colOf(e, lane);
                    if(r < m && c < r)
                        out[K + trilIndex(r, c)] = static_cast<float16_t>(acc.x[e]);
                }
            }
            __syncthreads();
            copyOut(output + static_cast<size_t>(sample0) * width, ldsOut, nHere * width);
        }

        // ------------------------------------------------------------------ backward
        template <uint32_t K>
        __global__ void __launch_bounds__(64 * kWavesPerWg) dlrmBwdKernel(const float16_t* __restrict__ input,
                                                                           const float16_t* __restrict__ upstream,
                                                                           float16_t* __restrict__ grad,
                                                                           float16_t* __restrict__ mlpGrad,
                                                                           uint32_t m,
                                                                           uint32_t batch)
        {
            constexpr uint32_t NBlocks = K / 32u; // 32-column blocks of the m x K result
            using FragG                = fragment<matrix_a, 32, 32, 16, float16_t, row_major>;
            using FragF                = fragment<matrix_b, 32, 32, 16, float16_t, row_major>;
            using FragAcc              = fragment<accumulator, 32, 32, 16, float32_t>;
            using AccMap               = detail::AccMap<32, 32, 32>;
            using FTile                = lds::DimMajorTile<(K < 128u ? 128u : K)>; // [feature row][K] with swizzled segments

            // LDS: per workgroup the contiguous upstream rows of its samples, then one
            // 32 x K feature tile per sample (rows m..31 stay zero).
            constexpr uint32_t tileBytes = kMaxM * FTile::rowBytes;
            extern __shared__ __attribute__((aligned(16))) char ldsRaw[];

            const uint32_t width    = K + (m * (m - 1u)) / 2u;
            const uint32_t upBytes  = ((kSamplesPerWg * width * 2u + 15u) / 16u) * 16u;
            float16_t*     ldsUp    = reinterpret_cast<float16_t*>(ldsRaw);
            char*          ldsTiles = ldsRaw + upBytes;

            const uint32_t lane    = threadIdx.x & 63u;
            const uint32_t wave    = threadIdx.x >> 6;
            const uint32_t sample0 = blockIdx.x * kSamplesPerWg;
            const uint32_t nHere   = min(kSamplesPerWg, batch - sample0);

            // stage upstream gradients (contiguous for the workgroup's samples)
            copyIn(ldsUp, upstream + static_cast<size_t>(sample0) * width, nHere * width);

            // stage features: 16-byte chunks, segment-swizzled rows; zero the padding rows
            constexpr uint32_t chunksPerRow = K / 8u;
            for(uint32_t s = 0; s < nHere; ++s)
            {
                const float16_t* F    = input + static_cast<size_t>(sample0 + s) * m * K;
                char*            tile = ldsTiles + s * tileBytes;
                for(uint32_t i = threadIdx.x; i < kMaxM * chunksPerRow; i += blockDim.x)
                {
                    const uint32_t r     = i / chunksPerRow;
                    const uint32_t chunk = i % chunksPerRow;
                    u32x4_t        v     = {0u, 0u, 0u, 0u};
                    if(r < m)
                        v = *reinterpret_cast<const u32x4_t*>(F + r * K + chunk * 8u);
                    *reinterpret_cast<u32x4_t*>(tile + FTile::offset(r, chunk >> 1) + ((chunk & 1u) << 4)) = v;
                }
            }
            __syncthreads();

            const uint32_t row    = lane & 31u;
            const uint32_t kGroup = lane >> 5;
#pragma unroll
            for(uint32_t s = 0; s < kSamplesPerWave; ++s)
            {
                const uint32_t local = wave * kSamplesPerWave + s;
                if(local >= nHere)
                    break;
                const float16_t* up   = ldsUp + local * width;
                char*            tile = ldsTiles + local * tileBytes;

                // G operand: row `row`, columns ks*16 + kGroup*8 + j, rebuilt from the packed triangle
                FragG fg[2];
#pragma unroll
                for(uint32_t ks = 0; ks < 2u; ++ks)
#pragma unroll
                    for(uint32_t j = 0; j < 8u; ++j)
                    {
                        const uint32_t c  = ks * 16u + kGroup * 8u + j;
                        const uint32_t hi = row > c ? row : c;
                        const uint32_t lo = row > c ? c : row;
                        float16_t      g  = static_cast<float16_t>(0);
                        if(hi < m && hi != lo)
                            g = up[K + trilIndex(hi, lo)];
                        fg[ks].x[j] = g;
                    }

                FragAcc acc[NBlocks];
#pragma unroll
                for(uint32_t nb = 0; nb < NBlocks; ++nb)
                {
                    fill_fragment(acc[nb], 0.0f);
#pragma unroll
                    for(uint32_t ks = 0; ks < 2u; ++ks)
                    {
                        FragF ff;
                        FTile::readBlock32(ff.x, tile, nb * 32u, ks, lane);
                        lds::waitReads();
                        __builtin_amdgcn_sched_barrier(0);
                        mma_sync(acc[nb], fg[ks], ff, acc[nb]);
                    }
                }

                // all of this wave's reads of the tile are done (same wave, in order): reuse it,
                // un-swizzled, as the staging buffer of grad[sample] (m x K, row-major)
                float16_t* stage = reinterpret_cast<float16_t*>(tile);
#pragma unroll
                for(uint32_t nb = 0; nb < NBlocks; ++nb)
#pragma unroll
                    for(uint32_t r4 = 0; r4 < AccMap::runs; ++r4)
                    {
                        const uint32_t e0 = r4 * 4u;
                        const uint32_t r  = AccMap::rowOf(e0, lane);
                        const uint32_t c  = nb * 32u + AccMap::colOf(e0, lane);
                        if(r < m)
                        {
                            float16_t* p = stage + r * K + c;
#pragma unroll
                            for(uint32_t j = 0; j < 4u; ++j)
                                p[j] = static_cast<float16_t>(acc[nb].x[e0 + j]);
                        }
                    }
            }
            __syncthreads();

            // coalesced write-out: grad (m*K halves per sample) and the bottom-MLP gradient
            for(uint32_t s = 0; s < nHere; ++s)
            {
                copyOut(grad + static_cast<size_t>(sample0 + s) * m * K,
                        reinterpret_cast<const float16_t*>(ldsTiles + s * tileBytes),
                        m * K);
                const float16_t* up  = ldsUp + s * width;
                float16_t*       dst = mlpGrad + static_cast<size_t>(sample0 + s) * K;
                for(uint32_t i = threadIdx.x; i < K; i += blockDim.x)
                    dst[i] = up[i];
            }
        }

        template <uint32_t K>
        int launchFwd(const void* input, void* output, uint32_t m, uint32_t batch, hipStream_t stream)
        {
            const uint32_t width = K + (m * (m - 1u)) / 2u;
            const uint32_t lds   = kSamplesPerWg * width * 2u;
            const uint32_t grid  = (batch + kSamplesPerWg - 1u) / kSamplesPerWg;
            hipLaunchKernelGGL((dlrmFwdKernel<K>),
                               dim3(grid),
                               dim3(64u * kWavesPerWg),
                               lds,
                               stream,
                               static_cast<const float16_t*>(input),
                               static_cast<float16_t*>(output),
                               m,
                               batch);
            return launchStatus();
        }

        template <uint32_t K>
        int launchBwd(const void* input, const void* upstream, void* grad, void* mlpGrad, uint32_t m, uint32_t batch,
                      hipStream_t stream)
        {
            using FTile           = lds::DimMajorTile<(K < 128u ? 128u : K)>;
            const uint32_t width  = K + (m * (m - 1u)) / 2u;
            const uint32_t upB    = ((kSamplesPerWg * width * 2u + 15u) / 16u) * 16u;
            const uint32_t lds    = upB + kSamplesPerWg * kMaxM * FTile::rowBytes;
            const uint32_t grid   = (batch + kSamplesPerWg - 1u) / kSamplesPerWg;
            auto           kernel = dlrmBwdKernel<K>;
            if(lds > 65536u
               && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(lds))
                      != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            hipLaunchKernelGGL(kernel,
                               dim3(grid),
                               dim3(64u * kWavesPerWg),
                               lds,
                               stream,
                               static_cast<const float16_t*>(input),
                               static_cast<const float16_t*>(upstream),
                               static_cast<float16_t*>(grad),
                               static_cast<float16_t*>(mlpGrad),
                               m,
                               batch);
            return launchStatus();
        }
    } // namespace

    int launchDlrmFwd(const void* input, void* output, uint32_t m, uint32_t k, uint32_t batch, hipStream_t stream)
    {
        switch(k)
        {
        case 32:
            return launchFwd<32>(input, output, m, batch, stream);
        case 64:
            return launchFwd<64>(input, output, m, batch, stream);
        case 128:
            return launchFwd<128>(input, output, m, batch, stream);
        case 256:
            return launchFwd<256>(input, output, m, batch, stream);
        default:
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        }
    }

    int launchDlrmBwd(const void* input, const void* upstream, void* grad, void* mlpGrad, uint32_t m, uint32_t k,
                      uint32_t batch, hipStream_t stream)
    {
        switch(k)
        {
        case 32:
            return launchBwd<32>(input, upstream, grad, mlpGrad, m, batch, stream);
        case 64:
            return launchBwd<64>(input, upstream, grad, mlpGrad, m, batch, stream);
        case 128:
            return launchBwd<128>(input, upstream, grad, mlpGrad, m, batch, stream);
        case 256:
            return launchBwd<256>(input, upstream, grad, mlpGrad, m, batch, stream);
        default:
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        }
    }

} // namespace rocwmma_amd
