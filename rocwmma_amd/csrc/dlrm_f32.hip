// DLRM dot-interaction forward and backward in float32 for gfx950.
//
// The reference's DLRM kernels and tests are templates over the element type and are instantiated for
// float32_t as well as float16_t (test/dlrm/test/dlrm_test_params.hpp:51; fp32 data files next to the fp16
// ones under test/dlrm/data).  Semantics: dlrm_fwd_CPU / dlrm_bwd_CPU with DataT = float
// (test/reference_impl.hpp:83-179).  The f16 kernels (dlrm.hip) are the benchmarked ones; these follow the same
// plan -- one wave owns a sample, no m x m scratch in global memory, one launch for backward -- written for
// parity rather than for the last byte per second:
//
//   * a wave copies its sample's m x K features into LDS rows of K + 4 floats (16-byte global loads; rows from m
//     to the next multiple of 32 are zeros, so no lane ever reads another sample or past the end of the input);
//   * the products run on v_mfma_f32_32x32x2_f32 through the fragment API.  Forward: block (I, J), J <= I, of
//     Z = F F^T from the 32-row tiles I and J; a lane reads 16 bytes of K per row and LDS instruction and feeds
//     four instructions from them (the order in which K is contracted is free as long as both multiplicands
//     agree: instruction t of a group contracts k = 8 g + t and 8 g + 4 + t).  Backward: row tile I of the
//     gradient is the sum over contraction tiles J of G_IJ F_J, G rebuilt from the packed triangle of the
//     upstream gradient (read straight from global memory), 32 columns at a time, stored from the accumulators
//     as 16-byte pieces;
//   * nothing is shared between the waves of a workgroup: no barrier.
#include "common.hpp"
#include <rocwmma/rocwmma_transforms.hpp>

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        typedef float f32x4_t __attribute__((ext_vector_type(4), may_alias));

        constexpr uint32_t kMaxM32   = 128;
        constexpr uint32_t kMaxTiles = kMaxM32 / 32u;
        constexpr uint32_t kRowPad   = 4; // floats: 16 consecutive rows at one column offset fall into 16 distinct 16-byte slots
        constexpr uint32_t kLdsBytes = 160u * 1024u;

        template <uint32_t K>
        ROCWMMA_DEVICE inline void stageFeatures(float* ldsF, const float* src, uint32_t m, uint32_t rowsPad, uint32_t lane)
        {
            constexpr uint32_t pitch  = K + kRowPad;
            constexpr uint32_t perRow = K / 4u;
            for(uint32_t i = lane; i < rowsPad * perRow; i += 64u)
            {
                const uint32_t r = i / perRow, c4 = i % perRow;
                f32x4_t        v = {0.0f, 0.0f, 0.0f, 0.0f};
                if(r < m)
                    v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(src + static_cast<size_t>(r) * K) + c4);
                *reinterpret_cast<f32x4_t*>(ldsF + r * pitch + 4u * c4) = v;
            }
            // (the wave's own LDS writes are visible to its later LDS reads: the LDS serves a wave's accesses in order)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }

        template <uint32_t K, uint32_t Samples>
        __global__ void __launch_bounds__(64 * Samples)
            dlrmFwdF32Kernel(const float* __restrict__ input, float* __restrict__ output, uint32_t m, uint32_t batch)
        {
            using FragA   = fragment<matrix_a, 32, 32, 2, float32_t, row_major>;
            using FragAcc = fragment<accumulator, 32, 32, 2, float32_t>;
            using AccMap  = detail::AccMap<32, 32, 32>;
            static_assert(FragA::num_elements == 1u && FragAcc::num_elements == 16u, "one float per lane and instruction");
            constexpr uint32_t pitch = K + kRowPad;

            extern __shared__ __attribute__((aligned(16))) float ldsAll[];
            const uint32_t lane    = threadIdx.x & 63u;
            const uint32_t wave    = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t sample  = blockIdx.x * Samples + wave;
            const uint32_t tiles   = (m + 31u) / 32u;
            const uint32_t rowsPad = tiles * 32u;
            if(sample >= batch)
                return; // (no workgroup barrier anywhere below)
            float*         ldsF  = ldsAll + wave * rowsPad * pitch;
            const uint32_t width = K + (m * (m - 1u)) / 2u;
            float*         out   = output + static_cast<size_t>(sample) * width;

            stageFeatures<K>(ldsF, input + static_cast<size_t>(sample) * m * K, m, rowsPad, lane);

            // bottom-MLP row: the sample's first feature row
            for(uint32_t e = lane; e < K; e += 64u)
                out[e] = ldsF[e];

            const uint32_t row = lane & 31u, half = lane >> 5;
#pragma unroll 1
            for(uint32_t I = 0; I < tiles; ++I)
#pragma unroll 1
                for(uint32_t J = 0; J <= I; ++J)
                {
                    const float* fI = ldsF + (I * 32u + row) * pitch + 4u * half;
                    const float* fJ = ldsF + (J * 32u + row) * pitch + 4u * half;
                    FragAcc      acc;
                    fill_fragment(acc, 0.0f);
#pragma unroll 4
                    for(uint32_t g = 0; g < K / 8u; ++g)
                    {
                        const f32x4_t vi = *reinterpret_cast<const f32x4_t*>(fI + 8u * g);
                        const f32x4_t vj = *reinterpret_cast<const f32x4_t*>(fJ + 8u * g);
#pragma unroll
                        for(uint32_t t = 0; t < 4u; ++t)
                        {
                            FragA a, b;
                            a.x[0] = vi[t];
                            b.x[0] = vj[t];
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
        }

        template <uint32_t K, uint32_t Samples>
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
            constexpr uint32_t pitch   = K + kRowPad;
            constexpr uint32_t NBlocks = K / 32u;

            extern __shared__ __attribute__((aligned(16))) float ldsAll[];
            const uint32_t lane    = threadIdx.x & 63u;
            const uint32_t wave    = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t sample  = blockIdx.x * Samples + wave;
            const uint32_t tiles   = (m + 31u) / 32u;
            const uint32_t rowsPad = tiles * 32u;
            if(sample >= batch)
                return;
            float*         ldsF  = ldsAll + wave * rowsPad * pitch;
            const uint32_t width = K + (m * (m - 1u)) / 2u;
            const float*   up    = upstream + static_cast<size_t>(sample) * width;
            float*         dst   = grad + static_cast<size_t>(sample) * m * K;

            stageFeatures<K>(ldsF, input + static_cast<size_t>(sample) * m * K, m, rowsPad, lane);

            // bottom-MLP gradient = the first K entries of the upstream row
            for(uint32_t e = lane; e < K; e += 64u)
                mlpGrad[static_cast<size_t>(sample) * K + e] = up[e];

            const uint32_t row = lane & 31u, half = lane >> 5;
#pragma unroll 1
            for(uint32_t I = 0; I < tiles; ++I)
            {
                // G(Rg, c) for this lane's row and its contraction indices c = J * 32 + 2 s + half: below the
                // diagonal the row's entries are consecutive in the packed triangle (tri(Rg) + c), above it entry
                // (c, Rg) sits at tri(c) + Rg; zero on the diagonal and beyond m.  (Rows and contraction indices
                // >= m meet zeros on both sides: the staged feature rows there are zeros.)
                const uint32_t Rg    = I * 32u + row;
                const uint32_t below = K + (Rg * (Rg - 1u)) / 2u;
                float          g[kMaxTiles][16];
#pragma unroll
                for(uint32_t J = 0; J < kMaxTiles; ++J)
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
                    for(uint32_t J = 0; J < kMaxTiles; ++J)
                    {
                        if(J < tiles) // (wave uniform)
                        {
                            const float* f = ldsF + (J * 32u + half) * pitch + nb * 32u + row;
#pragma unroll
                            for(uint32_t s = 0; s < 16u; ++s)
                            {
                                FragG a;
                                FragF b;
                                a.x[0] = g[J][s];
                                b.x[0] = f[2u * s * pitch];
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

        template <typename Kernel, typename... Args>
        int launchWithLds(Kernel kernel, uint32_t grid, uint32_t threads, uint32_t lds, hipStream_t stream, Args... args)
        {
            if(lds > kLdsBytes)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            if(lds > 65536u
               && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(lds))
                      != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), lds, stream, args...);
            return launchStatus();
        }

        // Samples (waves) per workgroup: as many of 4, 2, 1 as keep a workgroup's feature tiles within 64 KiB
        // (several workgroups per compute unit), one where a single sample needs more.
        template <uint32_t K>
        uint32_t samplesFor(uint32_t m)
        {
            const uint32_t perSample = ((m + 31u) / 32u) * 32u * (K + kRowPad) * 4u;
            return 4u * perSample <= 65536u ? 4u : (2u * perSample <= 65536u ? 2u : 1u);
        }

        template <uint32_t K>
        int launchFwd32(const float* input, float* output, uint32_t m, uint32_t batch, hipStream_t stream)
        {
            const uint32_t perSample = ((m + 31u) / 32u) * 32u * (K + kRowPad) * 4u;
            switch(samplesFor<K>(m))
            {
            case 4:
                return launchWithLds(dlrmFwdF32Kernel<K, 4>, (batch + 3u) / 4u, 256u, 4u * perSample, stream, input, output, m, batch);
            case 2:
                return launchWithLds(dlrmFwdF32Kernel<K, 2>, (batch + 1u) / 2u, 128u, 2u * perSample, stream, input, output, m, batch);
            default:
                return launchWithLds(dlrmFwdF32Kernel<K, 1>, batch, 64u, perSample, stream, input, output, m, batch);
            }
        }

        template <uint32_t K>
        int launchBwd32(const float* input, const float* upstream, float* grad, float* mlpGrad, uint32_t m, uint32_t batch,
                        hipStream_t stream)
        {
            const uint32_t perSample = ((m + 31u) / 32u) * 32u * (K + kRowPad) * 4u;
            switch(samplesFor<K>(m))
            {
            case 4:
                return launchWithLds(dlrmBwdF32Kernel<K, 4>, (batch + 3u) / 4u, 256u, 4u * perSample, stream, input, upstream, grad,
                                     mlpGrad, m, batch);
            case 2:
                return launchWithLds(dlrmBwdF32Kernel<K, 2>, (batch + 1u) / 2u, 128u, 2u * perSample, stream, input, upstream, grad,
                                     mlpGrad, m, batch);
            default:
                return launchWithLds(dlrmBwdF32Kernel<K, 1>, batch, 64u, perSample, stream, input, upstream, grad, mlpGrad, m, batch);
            }
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
