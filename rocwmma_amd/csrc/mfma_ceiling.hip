// Matrix-pipe ceiling probe (benchmark support, part of the auxiliary library).
//
// A loop of nothing but matrix instructions on operands held in registers: no LDS, no global
// memory, no barriers.  What it sustains is what the matrix pipes of the whole chip deliver under
// the board's power management for a given instruction shape and a given operand bit pattern
// (the part lowers its clock under load, and how far depends on how much the operand bits toggle:
// all-zero operands and uniform random operands give different rates for the same instruction
// stream).  The GEMM benchmark reports its kernels against this figure next to the nominal peak.
//
// Every workgroup has four waves (one per SIMD); wavesPerSimd workgroups are launched per compute
// unit.  A wave keeps 32 (16-wide shapes) or 8 (32-wide shapes) independent accumulator blocks and
// rotates over four A and four B operand register sets, as a GEMM wave tile does.
#include "common.hpp"

namespace rocwmma_amd
{
    namespace
    {
        typedef float    f32x4 __attribute__((ext_vector_type(4)));
        typedef float    f32x16 __attribute__((ext_vector_type(16)));
        typedef int      i32x4 __attribute__((ext_vector_type(4)));
        typedef int      i32x8 __attribute__((ext_vector_type(8)));
        typedef int      i32x16 __attribute__((ext_vector_type(16)));

        enum Shape : int
        {
            F16_16x16x32 = 0,
            F16_32x32x16,
            BF16_16x16x32,
            BF16_32x32x16,
            I8_16x16x64,
            I8_32x32x32,
            F8_16x16x128,
            F8_32x32x64,
            F8_16x16x128_SCALED, // v_mfma_scale_f32_16x16x128_f8f6f4 with per-lane block scales
        };

        // flops (or integer ops) of one instruction of the shape
        constexpr double opsPerInstruction(int shape)
        {
            switch(shape)
            {
            case F16_16x16x32:
            case BF16_16x16x32:
                return 2.0 * 16 * 16 * 32;
            case F16_32x32x16:
            case BF16_32x32x16:
                return 2.0 * 32 * 32 * 16;
            case I8_16x16x64:
                return 2.0 * 16 * 16 * 64;
            case I8_32x32x32:
                return 2.0 * 32 * 32 * 32;
            case F8_16x16x128:
            case F8_16x16x128_SCALED:
                return 2.0 * 16 * 16 * 128;
            default:
                return 2.0 * 32 * 32 * 64;
            }
        }

        // 32-wide shapes: 8 blocks x 4 operand rotations; 16-wide shapes: 32 blocks once
        constexpr uint32_t kInstructionsPerTrip = 32u;

        // (the host pass only needs the kernel's signature: it cannot parse the register constraints)
#if defined(__HIP_DEVICE_COMPILE__)
#define ROCWMMA_AMD_MFMA(NAME, ACC, A, B) asm volatile(NAME " %0, %1, %2, %0" : "+v"(ACC) : "v"(A), "v"(B))
#else
#define ROCWMMA_AMD_MFMA(NAME, ACC, A, B) (void)(A), (void)(B)
#endif

        template <int S>
        __global__ void __launch_bounds__(256) mfmaCeilingKernel(const uint32_t* operands, float* out, uint32_t trips)
        {
            // 16 bytes (four dwords) per lane and operand for the 16-bit and int8 shapes, 32 bytes for fp8
            constexpr bool     Fp8     = S == F8_16x16x128 || S == F8_32x32x64 || S == F8_16x16x128_SCALED;
            constexpr bool     Wide    = S == F16_32x32x16 || S == BF16_32x32x16 || S == I8_32x32x32 || S == F8_32x32x64;
            constexpr bool     Integer = S == I8_16x16x64 || S == I8_32x32x32;
            constexpr uint32_t Words   = Fp8 ? 8u : 4u;
            using Operand = std::conditional_t<Fp8, i32x8, i32x4>;
            using Acc     = std::conditional_t<Wide, std::conditional_t<Integer, i32x16, f32x16>,
                                               std::conditional_t<Integer, i32x4, f32x4>>;
            Operand a[4], b[4];
#pragma unroll
            for(uint32_t i = 0; i < 4u; ++i)
#pragma unroll
                for(uint32_t w = 0; w < Words; ++w)
                {
                    // operand words taken from the caller's 64 KiB table at lane-dependent places
                    a[i][w] = static_cast<int>(operands[(threadIdx.x * 8u + 2048u * i + w) & 16383u]);
                    b[i][w] = static_cast<int>(operands[(threadIdx.x * 24u + 7816u * i + 40u + w) & 16383u]);
                }
            constexpr uint32_t Blocks = Wide ? 8u : 32u;
            Acc                acc[Blocks];
#pragma unroll
            for(uint32_t q = 0; q < Blocks; ++q)
                acc[q] = Acc{};
            for(uint32_t t = 0; t < trips; ++t)
            {
                if constexpr(Wide)
                {
#pragma unroll
                    for(uint32_t s = 0; s < 4u; ++s) // four K steps with different operand registers
#pragma unroll
                        for(uint32_t q = 0; q < 8u; ++q)
                        {
                            auto& ra = a[((q >> 1) + s) & 3u];
                            auto& rb = b[((q & 1u) + s) & 3u];
                            if constexpr(S == F16_32x32x16)
                                ROCWMMA_AMD_MFMA("v_mfma_f32_32x32x16_f16", acc[q], ra, rb);
                            else if constexpr(S == BF16_32x32x16)
                                ROCWMMA_AMD_MFMA("v_mfma_f32_32x32x16_bf16", acc[q], ra, rb);
                            else if constexpr(S == I8_32x32x32)
                                ROCWMMA_AMD_MFMA("v_mfma_i32_32x32x32_i8", acc[q], ra, rb);
                            else
                                ROCWMMA_AMD_MFMA("v_mfma_f32_32x32x64_f8f6f4", acc[q], ra, rb);
                        }
                }
                else
                {
#pragma unroll
                    for(uint32_t q = 0; q < 32u; ++q) // a 4 x 8 grid of blocks
                    {
                        auto& ra = a[(q >> 3) & 3u];
                        auto& rb = b[q & 3u];
                        if constexpr(S == F16_16x16x32)
                            ROCWMMA_AMD_MFMA("v_mfma_f32_16x16x32_f16", acc[q], ra, rb);
                        else if constexpr(S == BF16_16x16x32)
                            ROCWMMA_AMD_MFMA("v_mfma_f32_16x16x32_bf16", acc[q], ra, rb);
                        else if constexpr(S == I8_16x16x64)
                            ROCWMMA_AMD_MFMA("v_mfma_i32_16x16x64_i8", acc[q], ra, rb);
                        else if constexpr(S == F8_16x16x128_SCALED)
                        {
#if defined(__HIP_DEVICE_COMPILE__)
                            // scales near one (E8M0 124..131), different per lane and operand set
                            acc[q] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ra, rb, acc[q], 0, 0, 0, 124 + (ra[0] & 7), 0,
                                                                                     124 + (rb[0] & 7));
#endif
                        }
                        else
                            ROCWMMA_AMD_MFMA("v_mfma_f32_16x16x128_f8f6f4", acc[q], ra, rb);
                    }
                }
            }
            float r = 0.0f;
#pragma unroll
            for(uint32_t q = 0; q < Blocks; ++q)
#pragma unroll
                for(uint32_t e = 0; e < sizeof(Acc) / 4u; ++e)
                    r += static_cast<float>(acc[q][e]);
            out[blockIdx.x * 256u + threadIdx.x] = r;
        }
#undef ROCWMMA_AMD_MFMA

        template <int S>
        int launchShape(const uint32_t* operands, float* out, uint32_t trips, uint32_t workgroups, hipStream_t stream)
        {
            hipLaunchKernelGGL(mfmaCeilingKernel<S>, dim3(workgroups), dim3(256), 0, stream, operands, out, trips);
            return launchStatus();
        }
    } // namespace

    int benchMfmaCeiling(int shape, uint32_t trips, uint32_t wavesPerSimd, const void* operands, float* out, double* ops,
                         hipStream_t stream)
    {
        if(shape < F16_16x16x32 || shape > F8_16x16x128_SCALED || trips == 0u || wavesPerSimd == 0u || wavesPerSimd > 2u)
            return ROCWMMA_AMD_INVALID_ARGUMENT;
        const uint32_t workgroups = computeUnits() * wavesPerSimd;
        if(ops)
            *ops = opsPerInstruction(shape) * kInstructionsPerTrip * static_cast<double>(trips) * 4.0 * workgroups;
        const uint32_t* src = static_cast<const uint32_t*>(operands);
        switch(shape)
        {
        case F16_16x16x32:
            return launchShape<F16_16x16x32>(src, out, trips, workgroups, stream);
        case F16_32x32x16:
            return launchShape<F16_32x32x16>(src, out, trips, workgroups, stream);
        case BF16_16x16x32:
            return launchShape<BF16_16x16x32>(src, out, trips, workgroups, stream);
        case BF16_32x32x16:
            return launchShape<BF16_32x32x16>(src, out, trips, workgroups, stream);
        case I8_16x16x64:
            return launchShape<I8_16x16x64>(src, out, trips, workgroups, stream);
        case I8_32x32x32:
            return launchShape<I8_32x32x32>(src, out, trips, workgroups, stream);
        case F8_16x16x128:
            return launchShape<F8_16x16x128>(src, out, trips, workgroups, stream);
        case F8_16x16x128_SCALED:
            return launchShape<F8_16x16x128_SCALED>(src, out, trips, workgroups, stream);
        default:
            return launchShape<F8_32x32x64>(src, out, trips, workgroups, stream);
        }
    }

} // namespace rocwmma_amd
