// DLRM dot-interaction forward and backward in float32 for gfx950.
//
// The reference's DLRM kernels and tests are templates over the element type and are instantiated for
// float32_t as well as float16_t (test/dlrm/test/dlrm_test_params.hpp:51; fp32 data files next to the fp16
// ones under test/dlrm/data).  Semantics: dlrm_fwd_CPU / dlrm_bwd_CPU with DataT = float
// (test/reference_impl.hpp:83-179).  The f16 kernels (dlrm.hip) are the benchmarked ones; these follow the same
// plan -- one wave owns a sample, no m x m scratch in global memory, one launch for backward -- written for
// parity rather than for the last byte per second:
//
//   * operands come straight from global memory (a sample is read by one wave only, so there is nothing to share
//     through LDS, and without LDS five waves per SIMD are resident); rows and contraction indices from m on are
//     never read: their lanes multiply zeros, so nothing of a neighbouring sample can leak (0 * Inf);
//   * the products run on v_mfma_f32_32x32x2_f32 through the fragment API.  Forward: block (I, J), J <= I, of
//     Z = F F^T from the 32-row tiles I and J; a lane loads 16 bytes of K of its row at a time and feeds four
//     instructions from them (the order in which K is contracted is free as long as both multiplicands
//     agree: instruction t of a group contracts k = 8 g + t and 8 g + 4 + t).  Backward: row tile I of the
//     gradient is the sum over contraction tiles J of G_IJ F_J, G rebuilt from the packed triangle of the
//     upstream gradient, 32 columns at a time (32 lanes read 128 contiguous bytes of a feature row), stored
//     from the accumulators as 16-byte pieces;
//   * nothing is shared between the waves of a workgroup: no barrier; LDS only to put a sample's forward output
//     row together before it is written out.
#include "common.hpp"
#include <rocwmma/rocwmma_transforms.hpp>

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        typedef float f32x4_t __attribute__((ext_vector_type(4), may_alias));

        constexpr uint32_t kMaxM32   = 128;

        template <uint32_t K, uint32_t Samples>
        __global__ void __launch_bounds__(64 * Samples)
            dlrmFwdF32Kernel(const float* __restrict__ input, float* __restrict__ output, uint32_t m, uint32_t batch)
        {
            using FragA   = fragment<matrix_a, 32, 32, 2, float32_t, row_major>;
            using FragAcc = fragment<accumulator, 32, 32, 2, float32_t>;
            using AccMap  = detail::AccMap<32, 32, 32>;
            static_assert(FragA::num_elements == 1u && FragAcc::num_elements == 16u, "one float per lane and instruction");

            const uint32_t lane   = threadIdx.x & 63u;
            const uint32_t wave   = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t sample = blockIdx.x * Samples + wave;
            const uint32_t tiles  = (m + 31u) / 32u;
            if(sample >= batch)
                return; // (no workgroup barrier anywhere below)
            const uint32_t width = K + (m * (m - 1u)) / 2u;
            const float*   feat  = input + static_cast<size_t>(sample) * m * K;
            // the sample's output row is put together in LDS (the triangle leaves the accumulators as single floats
            // all over the row) and written out in whole-wave pieces of 256 contiguous bytes
            extern __shared__ __attribute__((aligned(16))) float ldsOut[];
            float* out = ldsOut + wave * width;

            // bottom-MLP row: the sample's first feature row
            for(uint32_t e = lane; e < K; e += 64u)
                out[e] = feat[e];

            const uint32_t row = lane & 31u, half = lane >> 5;
#pragma unroll 1
            for(uint32_t I = 0; I < tiles; ++I)
#pragma unroll 1
                for(uint32_t J = 0; J <= I; ++J)
                {
                    // (rows from m on do not exist: their lanes multiply zeros and read nothing)
                    const bool     liveI = I * 32u + row < m, liveJ = J * 32u + row < m;
                    const f32x4_t* fI    = reinterpret_cast<const f32x4_t*>(feat + static_cast<size_t>(I * 32u + row) * K) + half;
                    const f32x4_t* fJ    = reinterpret_cast<const f32x4_t*>(feat + static_cast<size_t>(J * 32u + row) * K) + half;
                    FragAcc        acc;
                    fill_fragment(acc, 0.0f);
                    constexpr uint32_t Groups = K / 8u, Batch = Groups < 8u ? Groups : 8u; // loads in flight per operand
#pragma unroll 1
                    for(uint32_t g0 = 0; g0 < Groups; g0 += Batch)
                    {
                        f32x4_t vi[Batch], vj[Batch];
#pragma unroll
                        for(uint32_t g = 0; g < Batch; ++g)
                        {
                            vi[g] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                            if(liveI)
                                vi[g] = fI[2u * (g0 + g)];
                        }
                        if(I != J) // (wave uniform)
                        {
#pragma unroll
                            for(uint32_t g = 0; g < Batch; ++g)
                            {
                                vj[g] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                                if(liveJ)
                                    vj[g] = fJ[2u * (g0 + g)];
                            }
                        }
                        else
                        {
#pragma unroll
                            for(uint32_t g = 0; g < Batch; ++g)
                                vj[g] = vi[g];
                        }
#pragma unroll
                        for(uint32_t g = 0; g < Batch; ++g)
#pragma unroll
                            for(uint32_t t = 0; t < 4u; ++t)
                            {
                                FragA a, b;
                                a.x[0] = vi[g][t];
                                b.x[0] = vj[g][t];
                                mma_sync(acc, a, applyTranspose(b), acc);
                            }
                    }
                    // strict lower triangle, row by row
#pragma unroll
                    for(uint32_t e = 0; e < FragAcc::num_elements; ++e)
                    {
                        const uint32_t Rg = I * 32u + AccMap::rowOf(e, lane);
                        const uint32_t Cg = J * 32u + AccMap::colOf(e, lane);
                        if(Rg < m && Cg < Rg)
                            out[K + (Rg * (Rg - 1u)) / 2u + Cg] = acc.x[e];
                    }
                }
            // (the wave's own LDS writes, read back by other lanes of the same wave: the LDS serves a wave's accesses in order)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            float* dst = output + static_cast<size_t>(sample) * width;
            for(uint32_t e = lane; e < width; e += 64u)
                dst[e] = out[e];
        }

        // MaxTiles: contraction tiles of 32 the kernel is built for (1, 2 or 4: the G values of a row tile against
        // every contraction tile are held in registers, 16 per tile)
        template <uint32_t K, uint32_t Samples, uint32_t MaxTiles>
        __global__ void __launch_bounds__(64 * Samples) dlrmBwdF32Kernel(const float* __restrict__ input,
                                                                            const float* __restrict__ upstream,
                                                                            float* __restrict__ grad,
                                                                            float* __restrict__ mlpGrad,
                                                                            uint32_t m,
                                                                            uint32_t batch)
        {
            using FragG   = fragment<matrix_a, 32, 32, 2, float32_t, row_major>;
            using FragF   = fragment<matrix_b, 32, 32, 2, float32_t, row_major>;
            using FragAcc = fragment<accumulator, 32, 32, 2, float32_t>;
            using AccMap  = detail::AccMap<32, 32, 32>;
            static_assert(FragG::num_elements == 1u && FragF::num_elements == 1u, "one float per lane and instruction");
            constexpr uint32_t NBlocks = K / 32u;

            const uint32_t lane   = threadIdx.x & 63u;
            const uint32_t wave   = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t sample = blockIdx.x * Samples + wave;
            const uint32_t tiles  = (m + 31u) / 32u;
            if(sample >= batch)
                return;
            const uint32_t width = K + (m * (m - 1u)) / 2u;
            const float*   feat  = input + static_cast<size_t>(sample) * m * K;
            const float*   up    = upstream + static_cast<size_t>(sample) * width;
            float*         dst   = grad + static_cast<size_t>(sample) * m * K;

            // bottom-MLP gradient = the first K entries of the upstream row
            for(uint32_t e = lane; e < K; e += 64u)
                mlpGrad[static_cast<size_t>(sample) * K + e] = up[e];

            const uint32_t row = lane & 31u, half = lane >> 5;
#pragma unroll 1
            for(uint32_t I = 0; I < tiles; ++I)
            {
                // G(Rg, c) for this lane's row and its contraction indices c = J * 32 + 2 s + half: below the
                // diagonal the row's entries are consecutive in the packed triangle (tri(Rg) + c), above it entry
                // (c, Rg) sits at tri(c) + Rg; zero on the diagonal and beyond m.
                const uint32_t Rg    = I * 32u + row;
                const uint32_t below = K + (Rg * (Rg - 1u)) / 2u;
                float          g[MaxTiles][16];
#pragma unroll
                for(uint32_t J = 0; J < MaxTiles; ++J)
#pragma unroll
                    for(uint32_t s = 0; s < 16u; ++s)
                    {
                        const uint32_t c     = J * 32u + 2u * s + half;
                        const bool     there = (c > Rg ? c : Rg) < m && c != Rg;
                        g[J][s]              = there ? up[c < Rg ? below + c : K + (c * (c - 1u)) / 2u + Rg] : 0.0f;
                    }
#pragma unroll 1
                for(uint32_t nb = 0; nb < NBlocks; ++nb)
                {
                    FragAcc acc;
                    fill_fragment(acc, 0.0f);
#pragma unroll
                    for(uint32_t J = 0; J < MaxTiles; ++J)
                    {
                        if(J < tiles) // (wave uniform)
                        {
                            // F(c, column) for the lane's contraction indices c = J * 32 + 2 s + half and its column:
                            // 32 lanes read 128 contiguous bytes of a row; rows from m on do not exist (zeros, not
                            // another sample's values: 0 * Inf would leak)
                            const float* f = feat + static_cast<size_t>(J * 32u + half) * K + nb * 32u + row;
                            float        fv[16];
#pragma unroll
                            for(uint32_t s = 0; s < 16u; ++s)
                                fv[s] = J * 32u + 2u * s + half < m ? f[static_cast<size_t>(2u * s) * K] : 0.0f;
#pragma unroll
                            for(uint32_t s = 0; s < 16u; ++s)
                            {
                                FragG a;
                                FragF b;
                                a.x[0] = g[J][s];
                                b.x[0] = fv[s];
                                mma_sync(acc, a, b, acc);
                            }
                        }
                    }
                    // a lane owns runs of four consecutive columns of one row
#pragma unroll
                    for(uint32_t r4 = 0; r4 < AccMap::runs; ++r4)
                    {
                        const uint32_t e0 = r4 * 4u;
                        const uint32_t r  = I * 32u + AccMap::rowOf(e0, lane);
                        const uint32_t c  = nb * 32u + AccMap::colOf(e0, lane);
                        if(r < m)
                            *reinterpret_cast<f32x4_t*>(dst + static_cast<size_t>(r) * K + c)
                                = f32x4_t{acc.x[e0], acc.x[e0 + 1u], acc.x[e0 + 2u], acc.x[e0 + 3u]};
                    }
                }
            }
        }

        // Four samples (waves) per workgroup; nothing is shared between them.
        constexpr uint32_t kSamples = 4;

        template <uint32_t K>
        int launchFwd32(const float* input, float* output, uint32_t m, uint32_t batch, hipStream_t stream)
        {
            const uint32_t lds    = kSamples * (K + (m * (m - 1u)) / 2u) * static_cast<uint32_t>(sizeof(float));
            auto           kernel = dlrmFwdF32Kernel<K, kSamples>;
            if(lds > 65536u
               && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(lds))
                      != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            hipLaunchKernelGGL(kernel, dim3((batch + kSamples - 1u) / kSamples), dim3(64u * kSamples), lds, stream, input, output, m, batch);
            return launchStatus();
        }

        template <uint32_t K>
        int launchBwd32(const float* input, const float* upstream, float* grad, float* mlpGrad, uint32_t m, uint32_t batch,
                        hipStream_t stream)
        {
            const dim3 grid((batch + kSamples - 1u) / kSamples), block(64u * kSamples);
            if(m <= 32u)
                hipLaunchKernelGGL((dlrmBwdF32Kernel<K, kSamples, 1>), grid, block, 0, stream, input, upstream, grad, mlpGrad, m, batch);
            else if(m <= 64u)
                hipLaunchKernelGGL((dlrmBwdF32Kernel<K, kSamples, 2>), grid, block, 0, stream, input, upstream, grad, mlpGrad, m, batch);
            else
                hipLaunchKernelGGL((dlrmBwdF32Kernel<K, kSamples, 4>), grid, block, 0, stream, input, upstream, grad, mlpGrad, m, batch);
            return launchStatus();
        }
    } // namespace

    int launchDlrmFwdF32(const void* input, void* output, uint32_t m, uint32_t k, uint32_t batch, hipStream_t stream)
    {
        if(m > kMaxM32)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const float* in  = static_cast<const float*>(input);
        float*       out = static_cast<float*>(output);
        switch(k)
        {
        case 32:
            return launchFwd32<32>(in, out, m, batch, stream);
        case 64:
            return launchFwd32<64>(in, out, m, batch, stream);
        case 128:
            return launchFwd32<128>(in, out, m, batch, stream);
        case 256:
            return launchFwd32<256>(in, out, m, batch, stream);
        default:
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        }
    }

    int launchDlrmBwdF32(const void* input, const void* upstream, void* grad, void* mlpGrad, uint32_t m, uint32_t k, uint32_t batch,
                         hipStream_t stream)
    {
        if(m > kMaxM32)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const float* in = static_cast<const float*>(input);
        const float* up = static_cast<const float*>(upstream);
        float*       g  = static_cast<float*>(grad);
        float*       mg = static_cast<float*>(mlpGrad);
        switch(k)
        {
        case 32:
            return launchBwd32<32>(in, up, g, mg, m, batch, stream);
        case 64:
            return launchBwd32<64>(in, up, g, mg, m, batch, stream);
        case 128:
            return launchBwd32<128>(in, up, g, mg, m, batch, stream);
        case 256:
            return launchBwd32<256>(in, up, g, mg, m, batch, stream);
        default:
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        }
    }
} // namespace rocwmma_amd
