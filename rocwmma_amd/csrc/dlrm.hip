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
//   * a workgroup of 2, 4 or 8 waves owns as many consecutive samples, whose inputs and outputs are
//     contiguous in memory: features arrive as whole-wave 1 KiB direct-to-LDS copies, results
//     are assembled in LDS and leave as 16-byte coalesced stores;
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
        // A workgroup owns `Samples` consecutive samples, one per wave: 8 for large batches (longest
        // contiguous stores), 4 or 2 when the batch would otherwise not give every compute unit
        // several workgroups (batch 2048: 7 us with 4 samples per workgroup against 19 us with 8).
        constexpr uint32_t kMaxM         = 32;

        typedef uint32_t u32x4_t __attribute__((ext_vector_type(4), may_alias));
        typedef short    s16x4_t __attribute__((ext_vector_type(4)));

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

        // The feature rows of a workgroup's samples are contiguous in global memory
        // (samples x m rows of K halves).  They are copied into LDS as one matrix of
        // RowBytes-wide rows with whole-wave 1 KiB direct copies; inside a row the 16-byte
        // chunks (forward) or 32-byte segments (backward) are XOR-swizzled by the row index so
        // that the MFMA operand reads are bank-conflict free.  The swizzle is applied to the
        // source address of each lane's 16 bytes.
        template <uint32_t K>
        struct FeatureTile
        {
            static constexpr uint32_t rowBytes  = K * 2u;
            static constexpr uint32_t chunks    = rowBytes / 16u;
            static constexpr uint32_t segments  = rowBytes / 32u;
            static constexpr uint32_t rowsPer256 = rowBytes >= 256u ? 1u : 256u / rowBytes;

            // forward: 16 consecutive rows reading the same logical chunk hit 16 distinct banks groups
            ROCWMMA_DEVICE static inline uint32_t chunkSwizzle(uint32_t row)
            {
                return (row / rowsPer256) & ((chunks < 16u ? chunks : 16u) - 1u);
            }
            // backward: the 4 rows x 2 segments of one transposing read hit 8 distinct bank groups
            ROCWMMA_DEVICE static inline uint32_t segmentSwizzle(uint32_t row)
            {
                return ((row & 3u) << 1) & (segments - 1u);
            }

            // Issues this wave's share of the copies of `bytes` (multiple of 16) from `src` into
            // `ldsTile`.  Lanes past `bytes` read nothing (buffer bounds) and store zeros.
            template <bool BySegment>
            ROCWMMA_DEVICE static inline void
                asyncLoad(char* ldsTile, const void* src, uint32_t bytes, uint32_t wave, uint32_t waves, uint32_t lane)
            {
                const lds::BufferRsrc rsrc   = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(src), 0, static_cast<int>(bytes), 0x00020000);
                const uint32_t        copies = (bytes + 1023u) / 1024u;
                for(uint32_t copy = wave; copy < copies; copy += waves)
                {
                    const uint32_t o   = copy * 1024u + lane * 16u; // LDS byte offset of this lane's 16 bytes
                    const uint32_t row = o / rowBytes;
                    const uint32_t pos = (o % rowBytes) / 16u;
                    uint32_t       srcOff;
                    if constexpr(BySegment)
                        srcOff = row * rowBytes + ((((pos >> 1) ^ segmentSwizzle(row)) << 5) | ((pos & 1u) << 4));
                    else
                        srcOff = row * rowBytes + ((pos ^ chunkSwizzle(row)) << 4);
                    lds::asyncCopy16Streaming(ldsTile + copy * 1024u, rsrc, srcOff, 0u);
                }
            }
        };

        // ------------------------------------------------------------------ forward
        template <uint32_t K, uint32_t Samples>
        __global__ void __launch_bounds__(64 * Samples)
            dlrmFwdKernel(const float16_t* __restrict__ input, float16_t* __restrict__ output, uint32_t m, uint32_t batch)
        {
            constexpr uint32_t KSteps = K / 16u;
            using Tile                = FeatureTile<K>;
            using FragA               = fragment<matrix_a, 32, 32, 16, float16_t, row_major>;
            using FragAcc             = fragment<accumulator, 32, 32, 16, float32_t>;
            using AccMap              = detail::AccMap<32, 32, 32>;

            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];
            const uint32_t width     = K + (m * (m - 1u)) / 2u;
            const uint32_t tileBytes = (((Samples - 1u) * m + kMaxM) * Tile::rowBytes + 1023u) & ~1023u;
            char*          ldsIn     = ldsRaw;
            float16_t*     ldsOut    = reinterpret_cast<float16_t*>(ldsRaw + tileBytes);

            const uint32_t lane    = threadIdx.x & 63u;
            const uint32_t wave    = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t sample0 = blockIdx.x * Samples;
            const uint32_t nHere   = min(Samples, batch - sample0);

            // all feature rows of the workgroup's samples: one contiguous block
            Tile::template asyncLoad<false>(ldsIn, input + static_cast<size_t>(sample0) * m * K, nHere * m * Tile::rowBytes,
                                            wave, Samples, lane);
            lds::waitCopiesAndReads<0>();
            __syncthreads();

            if(wave < nHere)
            {
                // operand: matrix row = lane % 32 (rows >= m belong to the next sample or are
                // stale LDS: they only reach Gram entries with an index >= m, which are dropped)
                const uint32_t row    = lane & 31u;
                const uint32_t kGroup = lane >> 5;
                const uint32_t R      = wave * m + row;
                const uint32_t swz    = Tile::chunkSwizzle(R);
                FragA          fa[KSteps];
#pragma unroll
                for(uint32_t ks = 0; ks < KSteps; ++ks)
                    *reinterpret_cast<u32x4_t*>(fa[ks].x)
                        = *reinterpret_cast<const u32x4_t*>(ldsIn + R * Tile::rowBytes + (((ks * 2u + kGroup) ^ swz) << 4));

                FragAcc acc;
                fill_fragment(acc, 0.0f);
#pragma unroll
                for(uint32_t ks = 0; ks < KSteps; ++ks)
                    mma_sync(acc, fa[ks], applyTranspose(fa[ks]), acc);

                float16_t* out = ldsOut + wave * width;
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
        template <uint32_t K, uint32_t Samples>
        __global__ void __launch_bounds__(64 * Samples) dlrmBwdKernel(const float16_t* __restrict__ input,
                                                                           const float16_t* __restrict__ upstream,
                                                                           float16_t* __restrict__ grad,
                                                                           float16_t* __restrict__ mlpGrad,
                                                                           uint32_t m,
                                                                           uint32_t batch)
        {
            constexpr uint32_t NBlocks = K / 32u; // 32-column blocks of the m x K result
            using Tile                 = FeatureTile<K>;
            using FragG                = fragment<matrix_a, 32, 32, 16, float16_t, row_major>;
            using FragF                = fragment<matrix_b, 32, 32, 16, float16_t, row_major>;
            using FragAcc              = fragment<accumulator, 32, 32, 16, float32_t>;
            using AccMap               = detail::AccMap<32, 32, 32>;

            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];
            const uint32_t width     = K + (m * (m - 1u)) / 2u;
            const uint32_t tileBytes = (((Samples - 1u) * m + kMaxM) * Tile::rowBytes + 1023u) & ~1023u;
            char*          ldsF      = ldsRaw; // features in, gradients out
            float16_t*     ldsUp     = reinterpret_cast<float16_t*>(ldsRaw + tileBytes);

            const uint32_t lane    = threadIdx.x & 63u;
            const uint32_t wave    = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t sample0 = blockIdx.x * Samples;
            const uint32_t nHere   = min(Samples, batch - sample0);

            // Rows past the last sample are read as contraction rows >= m (multiplied by the zero
            // columns of G): they must hold finite values, so clear everything behind the features
            // first (the tail of the last partial copy is out of the buffer's bounds and reads zeros).
            const uint32_t featBytes = nHere * m * Tile::rowBytes;
            for(uint32_t i = featBytes / 16u + threadIdx.x; i < tileBytes / 16u; i += blockDim.x)
                reinterpret_cast<u32x4_t*>(ldsF)[i] = u32x4_t{0u, 0u, 0u, 0u};
            // features: direct copies, segment-swizzled for the transposing reads
            Tile::template asyncLoad<true>(ldsF, input + static_cast<size_t>(sample0) * m * K, featBytes, wave, Samples, lane);
            // upstream gradients (contiguous for the workgroup's samples)
            copyIn(ldsUp, upstream + static_cast<size_t>(sample0) * width, nHere * width);
            lds::waitCopiesAndReads<0>();
            __syncthreads();

            FragAcc acc[NBlocks];
            if(wave < nHere)
            {
                const uint32_t   row    = lane & 31u;
                const uint32_t   kGroup = lane >> 5;
                const float16_t* up     = ldsUp + wave * width;

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

                // F operands: transposing reads, lane l gets column nb*32 + l%32 and contraction
                // rows ks*16 + (l/32)*8 + 0..7 of this sample
                const uint32_t group   = lane >> 4;
                const uint32_t s16     = lane & 15u;
                const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds::LdsPtr)ldsF));
                FragF          ff[NBlocks][2];
#pragma unroll
                for(uint32_t nb = 0; nb < NBlocks; ++nb)
#pragma unroll
                    for(uint32_t ks = 0; ks < 2u; ++ks)
#pragma unroll
                        for(uint32_t kk = 0; kk < 2u; ++kk)
                        {
                            const uint32_t c    = ks * 16u + (group >> 1) * 8u + kk * 4u + (s16 >> 2);
                            const uint32_t R    = wave * m + c;
                            const uint32_t seg  = nb * 2u + (group & 1u);
                            const uint32_t addr = ldsBase + R * Tile::rowBytes + ((seg ^ Tile::segmentSwizzle(R)) << 5)
                                                  + ((s16 & 3u) << 3);
                            s16x4_t v;
                            asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(addr) : "memory");
                            reinterpret_cast<s16x4_t*>(ff[nb][ks].x)[kk] = v;
                        }
                lds::waitReads();
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(uint32_t nb = 0; nb < NBlocks; ++nb)
                {
                    fill_fragment(acc[nb], 0.0f);
#pragma unroll
                    for(uint32_t ks = 0; ks < 2u; ++ks)
                        mma_sync(acc[nb], fg[ks], ff[nb][ks], acc[nb]);
                }
            }
            __syncthreads(); // every wave is done reading features (its own and its neighbour's rows)

            if(wave < nHere)
            {
                // this sample's feature rows become the staging buffer of its gradient (m x K, row-major)
                float16_t* stage = reinterpret_cast<float16_t*>(ldsF) + wave * m * K;
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

            // coalesced write-out: gradients of all samples are one contiguous block
            copyOut(grad + static_cast<size_t>(sample0) * m * K, reinterpret_cast<const float16_t*>(ldsF), nHere * m * K);
            for(uint32_t i = threadIdx.x; i < nHere * (K / 8u); i += blockDim.x)
            {
                const uint32_t   s   = i / (K / 8u);
                const uint32_t   c8  = i % (K / 8u);
                const float16_t* src = ldsUp + s * width + c8 * 8u; // only 2-byte aligned in general
                float16_t        tmp[8];
#pragma unroll
                for(uint32_t j = 0; j < 8u; ++j)
                    tmp[j] = src[j];
                reinterpret_cast<u32x4_t*>(mlpGrad + static_cast<size_t>(sample0 + s) * K)[c8] = *reinterpret_cast<u32x4_t*>(tmp);
            }
        }

        template <uint32_t K, uint32_t Samples>
        uint32_t tileBytesFor(uint32_t m)
        {
            return (((Samples - 1u) * m + kMaxM) * K * 2u + 1023u) & ~1023u;
        }

        template <typename Kernel>
        int optInLds(Kernel kernel, uint32_t lds)
        {
            if(lds > 65536u
               && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(lds))
                      != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            return ROCWMMA_AMD_OK;
        }

        template <uint32_t K, uint32_t Samples>
        int launchFwdS(const void* input, void* output, uint32_t m, uint32_t batch, hipStream_t stream)
        {
            const uint32_t width  = K + (m * (m - 1u)) / 2u;
            const uint32_t lds    = tileBytesFor<K, Samples>(m) + ((Samples * width * 2u + 15u) & ~15u);
            const uint32_t grid   = (batch + Samples - 1u) / Samples;
            auto           kernel = dlrmFwdKernel<K, Samples>;
            if(int rc = optInLds(kernel, lds))
                return rc;
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(64u * Samples), lds, stream, static_cast<const float16_t*>(input),
                               static_cast<float16_t*>(output), m, batch);
            return launchStatus();
        }

        template <uint32_t K, uint32_t Samples>
        int launchBwdS(const void* input, const void* upstream, void* grad, void* mlpGrad, uint32_t m, uint32_t batch,
                       hipStream_t stream)
        {
            const uint32_t width  = K + (m * (m - 1u)) / 2u;
            const uint32_t lds    = tileBytesFor<K, Samples>(m) + ((Samples * width * 2u + 15u) & ~15u);
            const uint32_t grid   = (batch + Samples - 1u) / Samples;
            auto           kernel = dlrmBwdKernel<K, Samples>;
            if(int rc = optInLds(kernel, lds))
                return rc;
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(64u * Samples), lds, stream, static_cast<const float16_t*>(input),
                               static_cast<const float16_t*>(upstream), static_cast<float16_t*>(grad),
                               static_cast<float16_t*>(mlpGrad), m, batch);
            return launchStatus();
        }
        // samples per workgroup for a batch: 8 once that still leaves >= 8 workgroups per compute unit
        inline uint32_t samplesFor(uint32_t batch)
        {
            const uint32_t cus = computeUnits();
            if(batch >= 64u * cus)
                return 8u;
            return batch >= 8u * cus ? 4u : 2u;
        }

        template <uint32_t K>
        int launchFwd(const void* input, void* output, uint32_t m, uint32_t batch, hipStream_t stream)
        {
            switch(samplesFor(batch))
            {
            case 8:
                return launchFwdS<K, 8>(input, output, m, batch, stream);
            case 4:
                return launchFwdS<K, 4>(input, output, m, batch, stream);
            default:
                return launchFwdS<K, 2>(input, output, m, batch, stream);
            }
        }

        template <uint32_t K>
        int launchBwd(const void* input, const void* upstream, void* grad, void* mlpGrad, uint32_t m, uint32_t batch,
                      hipStream_t stream)
        {
            switch(samplesFor(batch))
            {
            case 8:
                return launchBwdS<K, 8>(input, upstream, grad, mlpGrad, m, batch, stream);
            case 4:
                return launchBwdS<K, 4>(input, upstream, grad, mlpGrad, m, batch, stream);
            default:
                return launchBwdS<K, 2>(input, upstream, grad, mlpGrad, m, batch, stream);
            }
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
