// Skinny GEMV / GEMM:  Y = alpha * A * X + beta * Y  for f16 A (row-major) and 1..8 right-hand
// sides.  A pure HBM-bandwidth kernel: every byte of A is read exactly once with 16-byte
// loads, the dot products run on the vector ALU (v_dot2_f32_f16, f32 accumulate).
//
// The reference's GEMV sample (sgemv_rocwmma_d, samples/simple_sgemv.cpp:103-155) pads the
// vector to a 16-column MFMA operand and so wastes 15/16 of the matrix-core work and reads
// past its buffers; its CPU twin sgemv_cpu_h (samples/simple_sgemv.cpp:46-66) defines the
// semantics kept here.
//
// Two kernels, picked by the number of right-hand sides:
//   * split kernel (1 column): a workgroup of four waves owns two rows and splits K four ways;
//     every wave keeps four 1 KiB row segments in flight, partial sums meet in LDS.  Many
//     short waves keep all HBM channels busy.
//   * staged kernel (2..8 columns): X (ncols x K halves, at most 128 KiB) is copied into LDS
//     once per workgroup; persistent waves then stream rows of A, one row per wave at a time,
//     reading X from LDS so the extra columns cost no L1/L2 traffic.
//   If X does not fit the LDS the split kernel reads X through the caches instead.
#include "common.hpp"
#include <rocwmma/rocwmma_lds.hpp>

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

        // Sum over the 16 lanes that share lane % 4 (the 16 blocks of v_mfma_f32_4x4x4_16B), left in every
        // lane: two rotations inside the rows of 16 lanes (DPP), then the rows of a half and the two halves
        // exchanged with v_permlane16_swap / v_permlane32_swap.  All on the vector ALU: the same sum with
        // four ds_bpermute steps per value kept the LDS pipe busy for microseconds per workgroup.
        ROCWMMA_DEVICE inline float sumOverBlocks(float v)
        {
#if defined(__HIP_DEVICE_COMPILE__)
            const auto bits = [](float f) { return __builtin_bit_cast(uint32_t, f); };
            const auto flt  = [](uint32_t u) { return __builtin_bit_cast(float, u); };
            v += flt(static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(bits(v)), 0x124 /* row_ror:4 */, 0xF, 0xF, true)));
            v += flt(static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(bits(v)), 0x128 /* row_ror:8 */, 0xF, 0xF, true)));
            // (x, x) -> (rows 0 0 2 2, rows 1 1 3 3) of x
            const auto rows = __builtin_amdgcn_permlane16_swap(bits(v), bits(v), false, false);
            v               = flt(rows[0]) + flt(rows[1]);
            // (x, x) -> (lower half twice, upper half twice)
            const auto halves = __builtin_amdgcn_permlane32_swap(bits(v), bits(v), false, false);
            v                 = flt(halves[0]) + flt(halves[1]);
#endif
            return v;
        }

        // Sum over the 64 lanes, left in every lane: inside the quads with two DPP quad permutes, then
        // over the 16 quads as above.
        ROCWMMA_DEVICE inline float waveSum(float v)
        {
#if defined(__HIP_DEVICE_COMPILE__)
            const auto bits = [](float f) { return static_cast<int>(__builtin_bit_cast(uint32_t, f)); };
            const auto flt  = [](int u) { return __builtin_bit_cast(float, static_cast<uint32_t>(u)); };
            v += flt(__builtin_amdgcn_update_dpp(0, bits(v), 0xB1 /* quad_perm:[1,0,3,2] */, 0xF, 0xF, true));
            v += flt(__builtin_amdgcn_update_dpp(0, bits(v), 0x4E /* quad_perm:[2,3,0,1] */, 0xF, 0xF, true));
#endif
            return sumOverBlocks(v);
        }

        // Split kernel: workgroup = 4 waves = (4 / KSplit) row groups x KSplit slices of K.
        template <uint32_t NCols, uint32_t RowsPerWave, uint32_t KSplit>
        __global__ void __launch_bounds__(256) gemvSplitKernel(uint32_t        m,
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
            __shared__ float partial[4][RowsPerWave * NCols];
            const uint32_t   lane     = threadIdx.x & 63u;
            const uint32_t   wave     = threadIdx.x >> 6;
            const uint32_t   rowGroup = (blockIdx.x * 4u + wave) / KSplit;
            const uint32_t   slice    = wave % KSplit;
            const uint32_t   row0     = rowGroup * RowsPerWave;
            // K slices in whole 16-byte chunks; the last slice takes the remainder
            const uint32_t chunks   = k / 8u;
            const uint32_t perSlice = (chunks + KSplit - 1u) / KSplit;
            const uint32_t cBeg     = slice * perSlice;
            const uint32_t cEnd     = (cBeg + perSlice < chunks) ? cBeg + perSlice : chunks;

            // rows past the end are clamped for loads and dropped at the store
            const u32x4_t* aRow[RowsPerWave];
#pragma unroll
            for(uint32_t r = 0; r < RowsPerWave; ++r)
            {
                const uint32_t row = (row0 + r < m) ? row0 + r : m - 1u;
                aRow[r]            = reinterpret_cast<const u32x4_t*>(a + static_cast<size_t>(row) * lda);
            }

            float acc[RowsPerWave][NCols];
#pragma unroll
            for(uint32_t r = 0; r < RowsPerWave; ++r)
#pragma unroll
                for(uint32_t c = 0; c < NCols; ++c)
                    acc[r][c] = 0.0f;

#pragma unroll 4
            for(uint32_t ch = cBeg + lane; ch < cEnd; ch += 64u)
            {
                u32x4_t av[RowsPerWave];
                u32x4_t xv[NCols];
#pragma unroll
                for(uint32_t r = 0; r < RowsPerWave; ++r)
                    av[r] = __builtin_nontemporal_load(aRow[r] + ch);
#pragma unroll
                for(uint32_t c = 0; c < NCols; ++c)
                    xv[c] = reinterpret_cast<const u32x4_t*>(x + static_cast<size_t>(c) * ldx)[ch];
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

            if constexpr(KSplit > 1u)
            {
                if(lane == 0u)
                {
#pragma unroll
                    for(uint32_t r = 0; r < RowsPerWave; ++r)
#pragma unroll
                        for(uint32_t c = 0; c < NCols; ++c)
                            partial[wave][r * NCols + c] = acc[r][c];
                }
                __syncthreads();
                if(slice == 0u)
                {
#pragma unroll
                    for(uint32_t r = 0; r < RowsPerWave; ++r)
#pragma unroll
                        for(uint32_t c = 0; c < NCols; ++c)
#pragma unroll
                            for(uint32_t j = 1; j < KSplit; ++j)
                                acc[r][c] += partial[wave + j][r * NCols + c];
                }
            }
            if(slice != 0u)
                return;
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

        // Staged kernel: X in LDS, persistent waves, one row per wave at a time.
        template <uint32_t NCols, uint32_t Waves>
        __global__ void __launch_bounds__(Waves * 64u) gemvStagedKernel(uint32_t        m,
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
            extern __shared__ __attribute__((aligned(16))) char ldsRaw[];
            u32x4_t*       xs     = reinterpret_cast<u32x4_t*>(ldsRaw); // [NCols][k / 8] 16-byte chunks
            const uint32_t chunks = k / 8u;
#pragma unroll
            for(uint32_t c = 0; c < NCols; ++c)
                for(uint32_t i = threadIdx.x; i < chunks; i += Waves * 64u)
                    xs[c * chunks + i] = reinterpret_cast<const u32x4_t*>(x + static_cast<size_t>(c) * ldx)[i];
            __syncthreads();

            const uint32_t lane   = threadIdx.x & 63u;
            const uint32_t gwave  = blockIdx.x * Waves + (threadIdx.x >> 6);
            const uint32_t nwaves = gridDim.x * Waves;
            for(uint32_t row = gwave; row < m; row += nwaves)
            {
                const u32x4_t* aRow = reinterpret_cast<const u32x4_t*>(a + static_cast<size_t>(row) * lda);
                float          acc[NCols];
#pragma unroll
                for(uint32_t c = 0; c < NCols; ++c)
                    acc[c] = 0.0f;
#pragma unroll 4
                for(uint32_t ch = lane; ch < chunks; ch += 64u)
                {
                    const u32x4_t av = __builtin_nontemporal_load(aRow + ch);
#pragma unroll
                    for(uint32_t c = 0; c < NCols; ++c)
                        acc[c] = dot8(av, xs[c * chunks + ch], acc[c]);
                }
#pragma unroll
                for(uint32_t c = 0; c < NCols; ++c)
                    acc[c] = waveSum(acc[c]);
#pragma unroll
                for(uint32_t c = 0; c < NCols; ++c)
                {
                    if(lane == c)
                    {
                        float*      dst = y + static_cast<size_t>(c) * ldy + row;
                        const float v   = alpha * acc[c];
                        *dst            = (beta != 0.0f) ? v + beta * *dst : v;
                    }
                }
            }
        }

        // Quad kernel for 4 and 8 right-hand sides: the dot products run on the matrix core's
        // small-block instruction v_mfma_f32_4x4x4_16B_f16 (16 independent 4 x 4 x 4 blocks per
        // wave), which fits a row stream: a lane fetches 16 bytes, lanes 4b..4b+3 hold the same
        // 16-byte K chunk of 4 consecutive rows of A (block b of the instruction), so one load
        // instruction reads 4 rows x 256 contiguous bytes and feeds two instructions per group of 4
        // columns.  Against the v_dot2 kernels this is 8x fewer arithmetic instructions, 4x fewer
        // LDS reads of X and 6x fewer cross-lane reduction steps (8192 x 8192, 8 columns:
        // 30 -> 24.6 us; 14336 x 4096: 30 -> 20.9 us).
        //   * workgroup = 16 waves = 4 row-quad lanes x 4 slices of K; X is copied into LDS once
        //     (direct-to-LDS, the chunks of column c XOR-swizzled by (c % 4) * 4 so the 16 lanes
        //     of a quarter-wave, 4 chunks x 4 columns, read 16 distinct bank groups);
        //   * a wave walks its K slice of its 4 rows, `Unroll` 1 KiB loads in flight;
        //   * block b accumulates the products of its own K chunks; at the end of a row quad the
        //     16 blocks are summed on the vector ALU (sumOverBlocks), the K-slice partial sums meet in
        //     LDS and are added in slice order (deterministic).
        constexpr uint32_t kQuadWaves = 16, kQuadSlices = 4;

        template <uint32_t NCols, uint32_t Unroll>
        __global__ void __launch_bounds__(kQuadWaves * 64u) gemvQuadKernel(uint32_t        m,
                                                                           uint32_t        k,
                                                                           const _Float16* a,
                                                                           uint32_t        lda,
                                                                           const _Float16* x,
                                                                           uint32_t        ldx,
                                                                           float*          y,
                                                                           uint32_t        ldy,
                                                                           float           alpha,
                                                                           float           beta,
                                                                           uint32_t        quadsPerWg)
        {
            typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
            typedef float    float4_t __attribute__((ext_vector_type(4)));
            typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
            constexpr uint32_t Groups = NCols / 4u;

            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];
            const uint32_t chunks  = k / 8u; // 16-byte chunks per row of A / column of X
            u32x4_t*       xs      = reinterpret_cast<u32x4_t*>(ldsRaw); // [NCols][chunks]
            float*         partial = reinterpret_cast<float*>(ldsRaw + static_cast<size_t>(NCols) * k * 2u);
            // partial[row quad of the workgroup][K slice][row in quad][column]

            const uint32_t lane = threadIdx.x & 63u;
            const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            {
                const uint32_t perCol = chunks / 64u;
                for(uint32_t j = wave; j < NCols * perCol; j += kQuadWaves)
                {
                    const uint32_t c   = j / perCol;
                    const uint32_t pos = (j % perCol) * 64u + lane;
                    rocwmma::lds::asyncCopy16(xs + c * chunks + (j % perCol) * 64u,
                                              reinterpret_cast<const u32x4_t*>(x + static_cast<size_t>(c) * ldx)
                                                  + (pos ^ ((c & 3u) << 2)));
                }
                rocwmma::lds::waitCopiesAndReads<0>();
            }
            __syncthreads();

            const uint32_t r4     = lane & 3u; // row of the quad (A operand) = column of the group (X operand)
            const uint32_t blk    = lane >> 2; // block of the instruction = K chunk within a step
            const uint32_t slice  = wave % kQuadSlices;
            const uint32_t qLane  = wave / kQuadSlices;
            const uint32_t quads  = m / 4u;
            const uint32_t q0     = blockIdx.x * quadsPerWg;
            const uint32_t sliceChunks = chunks / kQuadSlices;
            const uint32_t cBeg   = slice * sliceChunks;
            const uint32_t steps  = sliceChunks / 16u; // a multiple of Unroll (checked by the host)

            for(uint32_t ql = qLane; ql < quadsPerWg && q0 + ql < quads; ql += kQuadWaves / kQuadSlices)
            {
                const uint32_t  row  = (q0 + ql) * 4u + r4;
                const u32x4_t*  aRow = reinterpret_cast<const u32x4_t*>(a + static_cast<size_t>(row) * lda) + cBeg + blk;
                float4_t        acc[Groups];
#pragma unroll
                for(uint32_t g = 0; g < Groups; ++g)
                    acc[g] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
                for(uint32_t s0 = 0; s0 < steps; s0 += Unroll)
                {
                    u32x4_t av[Unroll];
#pragma unroll
                    for(uint32_t u = 0; u < Unroll; ++u)
                        av[u] = __builtin_nontemporal_load(aRow + 16u * (s0 + u));
#pragma unroll
                    for(uint32_t u = 0; u < Unroll; ++u)
                    {
                        const uint32_t ch  = cBeg + blk + 16u * (s0 + u);
                        const u32x2_t  alo = {av[u][0], av[u][1]}, ahi = {av[u][2], av[u][3]};
#pragma unroll
                        for(uint32_t g = 0; g < Groups; ++g)
                        {
                            const u32x4_t xv  = xs[(g * 4u + r4) * chunks + (ch ^ (r4 << 2))];
                            const u32x2_t xlo = {xv[0], xv[1]}, xhi = {xv[2], xv[3]};
                            // D[i][j] += sum_k X[column i][k] * A[row j][k]
                            acc[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, xlo),
                                                                        __builtin_bit_cast(half4_t, alo), acc[g], 0, 0, 0);
                            acc[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, xhi),
                                                                        __builtin_bit_cast(half4_t, ahi), acc[g], 0, 0, 0);
                        }
                    }
                }
                // lane (b, j) holds D[0..3][j] of block b: sum the 16 blocks
#pragma unroll
                for(uint32_t g = 0; g < Groups; ++g)
#pragma unroll
                    for(uint32_t i = 0; i < 4u; ++i)
                    {
                        acc[g][i] = sumOverBlocks(acc[g][i]);
                    }
                if(blk == 0u)
                {
#pragma unroll
                    for(uint32_t g = 0; g < Groups; ++g)
#pragma unroll
                        for(uint32_t i = 0; i < 4u; ++i)
                            partial[((ql * kQuadSlices + slice) * 4u + r4) * NCols + g * 4u + i] = acc[g][i];
                }
            }
            __syncthreads();
            const uint32_t quadsHere = q0 < quads ? (quads - q0 < quadsPerWg ? quads - q0 : quadsPerWg) : 0u;
            const uint32_t rowsHere  = quadsHere * 4u;
            for(uint32_t i = threadIdx.x; i < rowsHere * NCols; i += kQuadWaves * 64u)
            {
                const uint32_t r = i % rowsHere, c = i / rowsHere; // consecutive threads: consecutive rows of a column of Y
                const float*   p = partial + ((r / 4u) * kQuadSlices * 4u + (r & 3u)) * NCols + c;
                float          sum = p[0];
#pragma unroll
                for(uint32_t h = 1; h < kQuadSlices; ++h)
                    sum += p[h * 4u * NCols];
                float*      dst = y + static_cast<size_t>(c) * ldy + q0 * 4u + r;
                const float v   = alpha * sum;
                *dst            = (beta != 0.0f) ? v + beta * *dst : v;
            }
        }

        struct GemvArgs
        {
            uint32_t    m, k;
            const void* a;
            uint32_t    lda;
            const void* x;
            uint32_t    ldx;
            float*      y;
            uint32_t    ldy;
            float       alpha, beta;
        };

        template <uint32_t NCols, uint32_t RowsPerWave, uint32_t KSplit>
        int launchSplit(GemvArgs const& g, hipStream_t stream)
        {
            const uint32_t groups = (g.m + RowsPerWave - 1u) / RowsPerWave;
            const uint32_t waves  = groups * KSplit;
            hipLaunchKernelGGL((gemvSplitKernel<NCols, RowsPerWave, KSplit>), dim3((waves + 3u) / 4u), dim3(256), 0, stream,
                               g.m, g.k, static_cast<const _Float16*>(g.a), g.lda, static_cast<const _Float16*>(g.x), g.ldx,
                               g.y, g.ldy, g.alpha, g.beta);
            return launchStatus();
        }

        template <uint32_t NCols, uint32_t Waves>
        int launchStaged(GemvArgs const& g, uint32_t workgroups, hipStream_t stream)
        {
            const uint32_t ldsBytes = NCols * g.k * 2u;
            auto           kernel   = gemvStagedKernel<NCols, Waves>;
            if(ldsBytes > 65536u
               && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(ldsBytes))
                      != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            const uint32_t needed = (g.m + Waves - 1u) / Waves;
            hipLaunchKernelGGL(kernel, dim3(needed < workgroups ? needed : workgroups), dim3(Waves * 64u), ldsBytes, stream,
                               g.m, g.k, static_cast<const _Float16*>(g.a), g.lda, static_cast<const _Float16*>(g.x), g.ldx,
                               g.y, g.ldy, g.alpha, g.beta);
            return launchStatus();
        }

        template <uint32_t NCols, uint32_t Unroll>
        int launchQuadU(GemvArgs const& g, uint32_t workgroups, uint32_t quadsPerWg, uint32_t ldsBytes, hipStream_t stream)
        {
            auto kernel = gemvQuadKernel<NCols, Unroll>;
            if(ldsBytes > 65536u
               && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(ldsBytes))
                      != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(kQuadWaves * 64u), ldsBytes, stream, g.m, g.k,
                               static_cast<const _Float16*>(g.a), g.lda, static_cast<const _Float16*>(g.x), g.ldx, g.y, g.ldy,
                               g.alpha, g.beta, quadsPerWg);
            return launchStatus();
        }

        template <uint32_t NCols>
        int launchQuad(GemvArgs const& g, hipStream_t stream)
        {
            // whole row quads; whole 1 KiB copies per column of X; whole steps of 16 chunks per K slice
            if(g.m % 4u != 0u || g.k % (8u * 16u * kQuadSlices * 2u) != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            const uint32_t quads      = g.m / 4u;
            const uint32_t cus        = computeUnits();
            const uint32_t workgroups = quads < cus ? quads : cus;
            const uint32_t quadsPerWg = (quads + workgroups - 1u) / workgroups;
            const uint32_t ldsBytes   = NCols * g.k * 2u + quadsPerWg * kQuadSlices * 4u * NCols * 4u;
            if(ldsBytes > 160u * 1024u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            const uint32_t steps = g.k / (8u * 16u * kQuadSlices);
            if(steps % 16u == 0u)
                return launchQuadU<NCols, 16>(g, workgroups, quadsPerWg, ldsBytes, stream);
            if(steps % 8u == 0u)
                return launchQuadU<NCols, 8>(g, workgroups, quadsPerWg, ldsBytes, stream);
            return launchQuadU<NCols, 2>(g, workgroups, quadsPerWg, ldsBytes, stream);
        }

        constexpr uint32_t kStagedLdsLimit = 131072u; // X must leave room in the 160 KiB LDS
    } // namespace

    int launchGemv(uint32_t m, uint32_t k, uint32_t ncols, const void* a, uint32_t lda, const void* x, uint32_t ldx,
                   float* y, uint32_t ldy, float alpha, float beta, hipStream_t stream)
    {
        const GemvArgs g{m, k, a, lda, x, ldx, y, ldy, alpha, beta};
        const uint32_t cus    = computeUnits();
        const bool     staged = ncols * k * 2u <= kStagedLdsLimit;
        // 4 and 8 columns: the quad kernel where the shape allows it
        if(ncols == 4u || ncols == 8u)
        {
            const int rc = ncols == 4u ? launchQuad<4>(g, stream) : launchQuad<8>(g, stream);
            if(rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE)
                return rc;
        }
        switch(ncols)
        {
        case 1:
            return launchSplit<1, 2, 4>(g, stream);
        case 2:
            return staged ? launchStaged<2, 8>(g, 2u * cus, stream) : launchSplit<2, 2, 4>(g, stream);
        case 4:
            // two 512-thread workgroups per CU while X is at most 64 KiB, else one
            return staged ? launchStaged<4, 8>(g, (4u * k * 2u <= 65536u ? 2u : 1u) * cus, stream)
                          : launchSplit<4, 4, 2>(g, stream);
        case 8:
            return staged ? launchStaged<8, 16>(g, cus, stream) : launchSplit<8, 4, 2>(g, stream);
        default:
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        }
    }

} // namespace rocwmma_amd
