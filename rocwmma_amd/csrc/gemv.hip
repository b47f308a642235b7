// Skinny GEMV / GEMM:  Y = alpha * A * X + beta * Y  for f16 A (row-major) and 1..8 right-hand
// sides.  A pure HBM-bandwidth kernel: every byte of A is read exactly once with 16-byte
// loads, the dot products run on the vector ALU (v_dot2_f32_f16, f32 accumulate).
//
// The reference's GEMV sample (sgemv_rocwmma_d, samples/simple_sgemv.cpp:103-155) pads the
// vector to a 16-column MFMA operand and so wastes 15/16 of the matrix-core work and reads
// past its buffers; its CPU twin sgemv_cpu_h (samples/simple_sgemv.cpp:46-66) defines the
// semantics kept here.
//
// Work split: one wave owns RowsPerWave consecutive rows and walks K in steps of 512 elements
// (64 lanes x 8 halves = 1 KiB contiguous per row per step); the four waves of a workgroup
// walk K together on neighbouring rows so the X chunk they share stays in the CU's L1.
#include "common.hpp"

namespace rocwmma_amd
{
    namespace
    {
        typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
        typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

        ROCWMMA_DEVICE inline float dot8(u32x4_t a, u32x4_t x, float acc)
        {
#pragma unroll
            for(int i = 0; i < 4; ++i)
            {
                // copy the lanes out first: a bit cast applied directly to a vector element
                // reads the vector's first word
                const uint32_t ai = a[i];
                const uint32_t xi = x[i];
                acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, ai), __builtin_bit_cast(half2_t, xi), acc, false);
            }
            return acc;
        }

        ROCWMMA_DEVICE inline float waveSum(float v)
        {
#pragma unroll
            for(int off = 32; off >= 1; off >>= 1)
                v += __shfl_xor(v, off, 64);
            return v;
        }

        template <uint32_t NCols, uint32_t RowsPerWave>
        __global__ void __launch_bounds__(256) gemvKernel(uint32_t        m,
                                                          uint32_t        k,
                                                          const _Float16* a,
                                                          uint32_t        lda,
                                                          const _Float16* x,
                                                          uint32_t        ldx,
                                                          float*          y,
                                                          uint32_t        ldy,
                                                          float           alpha,
                                                          float           beta)
        {
            const uint32_t lane = threadIdx.x & 63u;
            const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
            const uint32_t row0 = wave * RowsPerWave;
            if(row0 >= m)
                return;

            // rows past the end are clamped for loads and dropped at the store
            const _Float16* aRow[RowsPerWave];
#pragma unroll
            for(uint32_t r = 0; r < RowsPerWave; ++r)
            {
                const uint32_t row = (row0 + r < m) ? row0 + r : m - 1u;
                aRow[r]            = a + static_cast<size_t>(row) * lda;
            }

            float acc[RowsPerWave][NCols];
#pragma unroll
            for(uint32_t r = 0; r < RowsPerWave; ++r)
#pragma unroll
                for(uint32_t c = 0; c < NCols; ++c)
                    acc[r][c] = 0.0f;

#pragma unroll 2
            for(uint32_t k0 = lane * 8u; k0 < k; k0 += 512u)
            {
                u32x4_t av[RowsPerWave];
                u32x4_t xv[NCols];
#pragma unroll
                for(uint32_t r = 0; r < RowsPerWave; ++r)
                    av[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(aRow[r] + k0));
#pragma unroll
                for(uint32_t c = 0; c < NCols; ++c)
                    xv[c] = *reinterpret_cast<const u32x4_t*>(x + static_cast<size_t>(c) * ldx + k0);
#pragma unroll
                for(uint32_t r = 0; r < RowsPerWave; ++r)
#pragma unroll
                    for(uint32_t c = 0; c < NCols; ++c)
                        acc[r][c] = dot8(av[r], xv[c], acc[r][c]);
            }

#pragma unroll
            for(uint32_t r = 0; r < RowsPerWave; ++r)
#pragma unroll
                for(uint32_t c = 0; c < NCols; ++c)
                    acc[r][c] = waveSum(acc[r][c]);

            // lane (r * NCols + c) writes result (r, c)
#pragma unroll
            for(uint32_t r = 0; r < RowsPerWave; ++r)
#pragma unroll
                for(uint32_t c = 0; c < NCols; ++c)
                {
                    if(lane == r * NCols + c && row0 + r < m)
                    {
                        float*      dst = y + static_cast<size_t>(c) * ldy + row0 + r;
                        const float v   = alpha * acc[r][c];
                        *dst            = (beta != 0.0f) ? v + beta * *dst : v;
                    }
                }
        }

        template <uint32_t NCols>
        int launch(uint32_t m, uint32_t k, const void* a, uint32_t lda, const void* x, uint32_t ldx, float* y,
                   uint32_t ldy, float alpha, float beta, hipStream_t stream)
        {
            constexpr uint32_t rowsPerWave = NCols >= 8 ? 4u : 4u;
            constexpr uint32_t wavesPerWg  = 4u;
            const uint32_t     waves       = (m + rowsPerWave - 1u) / rowsPerWave;
            const uint32_t     grid        = (waves + wavesPerWg - 1u) / wavesPerWg;
            hipLaunchKernelGGL((gemvKernel<NCols, rowsPerWave>),
                               dim3(grid),
                               dim3(64u * wavesPerWg),
                               0,
                               stream,
                               m,
                               k,
                               static_cast<const _Float16*>(a),
                               lda,
                               static_cast<const _Float16*>(x),
                               ldx,
                               y,
                               ldy,
                               alpha,
                               beta);
            return launchStatus();
        }
    } // namespace

    int launchGemv(uint32_t m, uint32_t k, uint32_t ncols, const void* a, uint32_t lda, const void* x, uint32_t ldx,
                   float* y, uint32_t ldy, float alpha, float beta, hipStream_t stream)
    {
        switch(ncols)
        {
        case 1:
            return launch<1>(m, k, a, lda, x, ldx, y, ldy, alpha, beta, stream);
        case 2:
            return launch<2>(m, k, a, lda, x, ldx, y, ldy, alpha, beta, stream);
        case 4:
            return launch<4>(m, k, a, lda, x, ldx, y, ldy, alpha, beta, stream);
        case 8:
            return launch<8>(m, k, a, lda, x, ldx, y, ldy, alpha, beta, stream);
        default:
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        }
    }

} // namespace rocwmma_amd
