// Skinny GEMM: D = alpha * A * B + beta * C for M <= 32 token rows against an N x K weight
// matrix (8-bit or 16-bit A row-major, B col-major, 32-bit C/D row-major), and a K-sliced variant
// further down for 48 token rows or when A does not fit the LDS whole.
//
// At these shapes (the reference's GEMM kernels, samples/perf_hgemm.cpp:518-714, need whole
// 128-wide macro tiles in M and would leave most of the chip idle) the job is streaming the
// weights from HBM exactly once, so the kernel is built for memory-level parallelism:
//   * a workgroup of 16 waves = 4 blocks of 16 weight rows x 4 slices of K; every wave walks
//     its K slice of its weight rows in 128-byte steps with 16 x 16 x 128 (16-bit: x 64) fragments loaded
//     straight from global memory (one v_mfma_f32_16x16x128_f8f6f4, or two
//     v_mfma_i32_16x16x64_i8, per step), several steps in flight;
//   * the token matrix A is copied into LDS once per workgroup (direct-to-LDS copies, 16-byte
//     chunks XOR-swizzled by row so the operand reads are bank-conflict free) and read from
//     there: fetched from the L2 by every wave, the same few KiB of A cost as much time as
//     the whole weight stream (17 us against 9 us at M = 16, N = 14336, K = 4096);
//   * the four K-slice partial accumulators of a block meet in LDS; the sum is formed in a
//     fixed order, so the result is deterministic (and bit-exact for int8).
#include "common.hpp"
#include <rocwmma/rocwmma_lds.hpp>

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        constexpr uint32_t kSkinnySlices = 4;   // K slices per block of weight rows
        constexpr uint32_t kSkinnyBlocks = 4;   // blocks of 16 weight rows per workgroup
        constexpr uint32_t kSkinnyWaves  = kSkinnySlices * kSkinnyBlocks;
        constexpr uint32_t kSkinnyKBytes = 128; // bytes of K per fragment step (128 8-bit or 64 16-bit elements)
        constexpr uint32_t kSkinnyMaxA   = 131072; // bytes of LDS the token matrix may take

        // Scaled: fp8 operands with one E8M0 scale per 32 elements of K (block-scaled / MX); a fragment step
        // is then one v_mfma_scale_f32_16x16x128_f8f6f4, whose scale operand of lane l belongs to row
        // l % 16 and K block l / 16 of the step.  The scales of the weights are fetched with the weight
        // fragments (one dword per lane and step: the four K blocks of the step, shifted down by the lane's
        // own), the scales of the tokens wait in LDS next to A.
        template <typename InT, typename OutT, typename CompT, uint32_t MBlocks, uint32_t Ahead, bool Scaled = false>
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
                                                                              CompT       beta,
                                                                              uint32_t    rowsPerWg,
                                                                              MxScales    scales)
        {
            constexpr uint32_t E       = sizeof(InT); // bytes per element
            static_assert(!Scaled || (sizeof(InT) == 1u && std::is_same<CompT, float>::value), "block scales: fp8 operands");
            constexpr uint32_t kSkinnyK = kSkinnyKBytes / E; // K elements per fragment step
            using FragA   = fragment<matrix_a, 16, 16, kSkinnyK, InT, row_major>;
            using FragB   = fragment<matrix_b, 16, 16, kSkinnyK, InT, col_major>;
            using FragAcc = fragment<accumulator, 16, 16, kSkinnyK, CompT>;
            using FragC   = fragment<accumulator, 16, 16, kSkinnyK, OutT, row_major>;
            using MapA    = detail::InputMap<16, kSkinnyK, 16, detail::packClassOf<InT>()>;
            static_assert(sizeof(InT) <= 2, "8- and 16-bit operands");

            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];
            char* aTile = ldsRaw; // [m][k * E] bytes, chunk c of row r at chunk position c ^ (r % 16)
            // partial[wave][mblock][lane] : the 4 accumulator registers of a lane as one 16-byte unit
            using Quad    = CompT __attribute__((ext_vector_type(4)));
            Quad* partial = reinterpret_cast<Quad*>(ldsRaw + m * k * E);
            // (Scaled) the tokens' scales, [k / 128][m] dwords (the four K blocks of a step), in the space of the
            // partial sums until those are due
            uint8_t* aScales = reinterpret_cast<uint8_t*>(partial);

            const uint32_t lane   = threadIdx.x & 63u;
            const uint32_t wave   = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t slice  = wave % kSkinnySlices;
            const uint32_t blk    = wave / kSkinnySlices;
            // A workgroup owns rowsPerWg weight rows (a multiple of 8, at most 64: the host picks the count
            // that spreads the rows most evenly over the compute units); block `blk` covers the next 16 of
            // them, of which the last block of a workgroup may hold only 8 (its other lanes load and store
            // nothing) or none.
            const uint32_t first    = blockIdx.x * rowsPerWg + blk * 16u; // first weight row of this block
            const uint32_t wgEnd    = min(blockIdx.x * rowsPerWg + rowsPerWg, n);
            const uint32_t liveRows = first < wgEnd ? min(16u, wgEnd - first) : 0u;
            const bool     live     = liveRows != 0u;
            const uint32_t n0       = live ? first : 0u; // idle waves shadow block 0, store nothing
            const bool     rowLive  = !live || (lane & 15u) < liveRows; // this lane's weight row exists
            const uint32_t kLen   = k / kSkinnySlices;
            const uint32_t kBeg   = slice * kLen;

            // A -> LDS: whole-wave 1 KiB copies, k / 1024 per row
            {
                const uint32_t perRow = k * E / 1024u;
                const uint32_t copies = m * perRow;
                for(uint32_t j = wave; j < copies; j += kSkinnyWaves)
                {
                    const uint32_t r   = j / perRow;
                    const uint32_t pos = (j % perRow) * 64u + lane; // chunk position inside the LDS row
                    lds::asyncCopy16(aTile + r * k * E + (j % perRow) * 1024u,
                                     reinterpret_cast<const char*>(a) + static_cast<size_t>(r) * lda * E
                                         + ((pos ^ (r & 15u)) << 4));
                }
            }

            // (Scaled) the tokens' scales: at most 32 x 128 bytes, one dword per thread (k / 32 is a multiple of 4
            // and the scale rows are 4-byte aligned: checked by the host).  Fetched here, stored to LDS only
            // after the first weight loads have gone out: the store has to wait for the fetch, and a wait in
            // front of the weight loads would hold them back until A has landed.
            uint32_t       myScalesA  = 0u;
            const uint32_t scaleWords = Scaled ? m * (k / 128u) : 0u; // <= 1024 = threads of the workgroup
            if constexpr(Scaled)
            {
                const uint32_t perRow = k / 128u;
                if(threadIdx.x < scaleWords)
                    myScalesA = *reinterpret_cast<const uint32_t*>(scales.a + static_cast<size_t>(threadIdx.x / perRow) * scales.lda
                                                                   + (threadIdx.x % perRow) * 4u);
            }

            FragAcc acc[MBlocks];
#pragma unroll
            for(uint32_t i = 0; i < MBlocks; ++i)
                fill_fragment(acc[i], static_cast<CompT>(0));

            // this lane's A operand rows in LDS and its swizzle
            const uint32_t aRow = lane & 15u;
            const InT*     bPtr = b + static_cast<size_t>(n0) * ldb + kBeg;

            // (Scaled) this lane's weight row of scales, at the first K block of the wave's K slice
            const uint8_t* sbPtr = nullptr;
            uint32_t       sb[Scaled ? Ahead : 1u] = {};
            if constexpr(Scaled)
                sbPtr = scales.b + static_cast<size_t>(n0 + (lane & 15u)) * scales.ldb + kBeg / 32u;
            const uint32_t myShift = 8u * (lane >> 4); // the lane's K block of a step inside the step's dword
            auto loadB = [&](FragB(&fb)[Ahead], uint32_t kk) {
                if(rowLive) // (lanes of rows beyond a half-filled block keep their zeros)
                {
                    if constexpr(Scaled)
                    {
                        // The dwords of up to four consecutive steps in one load (16-byte aligned: checked by the
                        // host), in front of the fragments: loads return in order, and behind them the first
                        // MFMA of a batch would wait for the whole batch.
                        constexpr uint32_t Vec = Ahead < 4u ? Ahead : 4u;
                        typedef uint32_t   Dwords __attribute__((ext_vector_type(Vec)));
#pragma unroll
                        for(uint32_t u = 0; u < Ahead; u += Vec)
                        {
                            const Dwords q = *reinterpret_cast<const Dwords*>(sbPtr + (kk + u * kSkinnyK) / 32u);
#pragma unroll
                            for(uint32_t j = 0; j < Vec; ++j)
                                sb[u + j] = q[j];
                        }
                    }
#pragma unroll
                    for(uint32_t u = 0; u < Ahead; ++u)
                        load_matrix_sync(fb[u], bPtr + kk + u * kSkinnyK, ldb);
                }
            };
            auto multiply = [&](FragB(&fb)[Ahead], uint32_t kk) {
#pragma unroll
                for(uint32_t u = 0; u < Ahead; ++u)
#pragma unroll
                    for(uint32_t i = 0; i < MBlocks; ++i)
                    {
                        FragA          fa;
                        const uint32_t row = i * 16u + aRow;
#pragma unroll
                        for(uint32_t ch = 0; ch < MapA::nchunks; ++ch)
#pragma unroll
                            for(uint32_t piece = 0; piece < MapA::kpack * E / 16u; ++piece)
                            {
                                const uint32_t kByte
                                    = (kBeg + kk + u * kSkinnyK + MapA::chunkK(ch, lane)) * E + piece * 16u;
                                detail::copyBytes<16u>(fa.x + ch * MapA::kpack + piece * (16u / E),
                                                       aTile + row * k * E + (((kByte >> 4) ^ (row & 15u)) << 4));
                            }
                        if constexpr(Scaled)
                        {
#if ROCWMMA_ARCH_GFX950 // (the instruction table exists in the device pass only)
                            using Op  = detail::MfmaScaled<detail::TypeInfo<InT>::cls, detail::TypeInfo<InT>::cls, 16u>;
                            using Acc = typename Op::Acc;
                            // (dword of step s of row r at [s][r]: the 16 rows a quarter-wave reads are 16 consecutive
                            // dwords; row-major, 128 bytes apart, they all fell into one bank)
                            const uint32_t sa = reinterpret_cast<const uint32_t*>(aScales)[((kBeg + kk + u * kSkinnyK) / kSkinnyK) * m + row];
                            Acc&           v  = *reinterpret_cast<Acc*>(acc[i].x);
                            // (the accumulator is kept transposed: the instruction's first multiplicand is B)
                            v = Op::template exec<0, 0>(fb[u].x, fa.x, v, sb[u] >> myShift, sa >> myShift);
#endif
                        }
                        else
                            mma_sync(acc[i], fa, fb[u], acc[i]);
                    }
            };

            // the first batch of weight fragments is requested before waiting for A
            FragB fb[Ahead];
#pragma unroll
            for(uint32_t u = 0; u < Ahead; ++u)
                fill_fragment(fb[u], static_cast<InT>(0));
            loadB(fb, 0u);
            if constexpr(Scaled)
            {
                if(threadIdx.x < scaleWords)
                    reinterpret_cast<uint32_t*>(aScales)[(threadIdx.x % (k / 128u)) * m + threadIdx.x / (k / 128u)] = myScalesA;
            }
            lds::waitCopiesAndReads<0>();
            __syncthreads();
            multiply(fb, 0u);
            for(uint32_t kk = Ahead * kSkinnyK; kk < kLen; kk += Ahead * kSkinnyK)
            {
                loadB(fb, kk);
                multiply(fb, kk);
            }

            // meet in LDS
            if constexpr(Scaled)
                __syncthreads(); // (everybody is done with the scales that sit where the partial sums go)
#pragma unroll
            for(uint32_t i = 0; i < MBlocks; ++i)
                partial[(wave * MBlocks + i) * 64u + lane] = *reinterpret_cast<Quad*>(acc[i].x);
            __syncthreads();

            // token block i of a weight block is finished by the wave of slice i % 4: fixed
            // summation order slice 0, 1, 2, 3
#pragma unroll
            for(uint32_t i = 0; i < MBlocks; ++i)
            {
                if(i % kSkinnySlices != slice || !live)
                    continue;
                const uint32_t first = blk * kSkinnySlices;
                Quad           sum   = partial[((first + 0u) * MBlocks + i) * 64u + lane];
#pragma unroll
                for(uint32_t w = 1; w < kSkinnySlices; ++w)
                    sum += partial[((first + w) * MBlocks + i) * 64u + lane];
                const size_t row = i * 16u;
                const size_t col = n0;
                FragC        fc;
                // (accumulator layout: a lane owns output columns 4 (lane / 16) .. + 3 of the block)
                if(4u * (lane >> 4) >= liveRows)
                    continue;
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

        template <typename InT, typename OutT, typename CompT, uint32_t MBlocks, uint32_t Ahead, bool Scaled = false>
        int launchOne(GemmArgs const& g, hipStream_t stream, MxScales const& scales = MxScales{})
        {
            const uint32_t lds    = g.m * g.k * static_cast<uint32_t>(sizeof(InT)) + kSkinnyWaves * MBlocks * 1024u;
            auto           kernel = gemmSkinnyKernel<InT, OutT, CompT, MBlocks, Ahead, Scaled>;
            if(lds > 65536u
               && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(lds))
                      != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            // Weight rows per workgroup: 64, or fewer (a multiple of 8) when that spreads the rows more evenly:
            // the kernel is bound by what one compute unit's L1 can request, so the busiest unit sets the time
            // (14336 rows on 256 units: 224 workgroups of 64 rows leave 32 units idle, 256 of 56 rows do not).
            const uint32_t units = computeUnits();
            uint32_t       rows  = 16u * kSkinnyBlocks;
            uint32_t       best  = ((g.n + rows - 1u) / rows + units - 1u) / units * rows;
            for(uint32_t r = 16u * kSkinnyBlocks - 8u; r >= 32u; r -= 8u)
            {
                const uint32_t cost = ((g.n + r - 1u) / r + units - 1u) / units * r;
                if(cost < best)
                    best = cost, rows = r;
            }
            hipLaunchKernelGGL(kernel, dim3((g.n + rows - 1u) / rows), dim3(64u * kSkinnyWaves), lds,
                               stream, g.m, g.n, g.k, static_cast<InT const*>(g.a), static_cast<InT const*>(g.b),
                               static_cast<OutT const*>(g.c), static_cast<OutT*>(g.d), g.lda, g.ldb, g.ldc, g.ldd,
                               static_cast<CompT>(g.alpha), static_cast<CompT>(g.beta), rows, scales);
            return launchStatus();
        }


        // ---- 48 token rows (and A too large for the LDS): K slices over workgroups ------------------
        // With more than 32 token rows A no longer fits the LDS whole, and the blocked kernel needs
        // whole 128-row tiles.  Here a workgroup keeps one K slice of A (at most 128 KiB)
        // in LDS and its 8 waves stream the same K slice of 32 weight rows each, so a compute
        // unit reads its slice of A once.  The K slices of a block of outputs belong to different
        // workgroups: D is first set to beta * C by a small kernel, then every workgroup adds
        // alpha * (its partial product) with atomic adds.  The partial tile goes through LDS
        // (the A slice is no longer needed) so that an atomic instruction covers 256 contiguous
        // bytes of one output row.  int32 sums are exact in any order; f32 sums of more than two
        // slices depend on the order the workgroups arrive in (last-bit differences between runs).
        // The atomic adds set the pace (about 3 ns per output element and slice over the whole
        // chip: 64 x 14336 x 4096 takes 24 us, 128 rows would take 36 us against 25 us on the
        // blocked kernel, which therefore keeps the multiples of 128).
        constexpr uint32_t kSlicedWaves = 8;
        constexpr uint32_t kSlicedNB    = 2; // blocks of 16 weight rows per wave
        constexpr uint32_t kSlicedCols  = kSlicedWaves * kSlicedNB * 16u; // output columns per workgroup
        constexpr uint32_t kSlicedAhead = 4;
        constexpr uint32_t kSlicedMaxM  = 128;

        template <typename OutT, typename CompT>
        __global__ void __launch_bounds__(256)
            initOutputKernel(uint32_t m, uint32_t n, OutT const* c, uint32_t ldc, OutT* d, uint32_t ldd, CompT beta)
        {
            typedef OutT Vec __attribute__((ext_vector_type(4)));
            const uint32_t perRow = n / 4u;
            const uint32_t idx    = blockIdx.x * 256u + threadIdx.x;
            if(idx >= m * perRow)
                return;
            const uint32_t row = idx / perRow, col = (idx % perRow) * 4u;
            Vec            v   = {0, 0, 0, 0};
            if(beta != static_cast<CompT>(0))
            {
                const Vec cv = *reinterpret_cast<const Vec*>(c + static_cast<size_t>(row) * ldc + col);
#pragma unroll
                for(uint32_t e = 0; e < 4u; ++e)
                    v[e] = static_cast<OutT>(beta * static_cast<CompT>(cv[e]));
            }
            *reinterpret_cast<Vec*>(d + static_cast<size_t>(row) * ldd + col) = v;
        }

        ROCWMMA_DEVICE inline void addTo(int32_t* p, int32_t v)
        {
            __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        ROCWMMA_DEVICE inline void addTo(float* p, float v)
        {
            unsafeAtomicAdd(p, v);
        }

        template <typename InT, typename OutT, typename CompT, uint32_t MBlocks>
        __global__ void __launch_bounds__(64 * kSlicedWaves) gemmSlicedKernel(uint32_t   m,
                                                                              uint32_t   n,
                                                                              uint32_t   k,
                                                                              InT const* a,
                                                                              InT const* b,
                                                                              OutT*      d,
                                                                              uint32_t   lda,
                                                                              uint32_t   ldb,
                                                                              uint32_t   ldd,
                                                                              CompT      alpha)
        {
            constexpr uint32_t E       = sizeof(InT); // bytes per element
            constexpr uint32_t kSkinnyK = kSkinnyKBytes / E; // K elements per fragment step
            using FragA   = fragment<matrix_a, 16, 16, kSkinnyK, InT, row_major>;
            using FragB   = fragment<matrix_b, 16, 16, kSkinnyK, InT, col_major>;
            using FragAcc = fragment<accumulator, 16, 16, kSkinnyK, CompT>;
            using MapA    = detail::InputMap<16, kSkinnyK, 16, detail::packClassOf<InT>()>;
            static_assert(sizeof(InT) <= 2 && std::is_same<OutT, CompT>::value, "8- or 16-bit operands, 32-bit results");
            constexpr uint32_t Ahead = kSlicedAhead;

            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];
            char* aTile = ldsRaw; // [m][kLen * E] bytes, chunk c of row r at chunk position c ^ (r % 16)

            const uint32_t lane   = threadIdx.x & 63u;
            const uint32_t wave   = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t kLen   = k / gridDim.y;
            const uint32_t kBeg   = blockIdx.y * kLen;
            constexpr uint32_t NB = kSlicedNB;
            const InT*         bPtr[NB];
#pragma unroll
            for(uint32_t j = 0; j < NB; ++j)
            {
                const uint32_t nBlock = (blockIdx.x * kSlicedWaves + wave) * NB + j; // block of 16 weight rows
                const uint32_t n0     = (nBlock * 16u < n ? nBlock : 0u) * 16u; // idle blocks shadow block 0
                bPtr[j]               = b + static_cast<size_t>(n0) * ldb + kBeg;
            }

            // this lane's A operand rows in LDS and its swizzle
            const uint32_t aRow = lane & 15u;
            auto           loadB = [&](FragB(&fb)[Ahead][NB], uint32_t kk) {
#pragma unroll
                for(uint32_t u = 0; u < Ahead; ++u)
#pragma unroll
                    for(uint32_t j = 0; j < NB; ++j)
                        load_matrix_sync(fb[u][j], bPtr[j] + kk + u * kSkinnyK, ldb);
            };
            // the first batch of weight fragments is requested before anything else
            FragB fb[Ahead][NB];
            loadB(fb, 0u);

            // A slice -> LDS: whole-wave 1 KiB copies, kLen / 1024 per row
            {
                const uint32_t perRow = kLen * E / 1024u;
                const uint32_t copies = m * perRow;
                for(uint32_t j = wave; j < copies; j += kSlicedWaves)
                {
                    const uint32_t r   = j / perRow;
                    const uint32_t pos = (j % perRow) * 64u + lane; // chunk position inside the LDS row
                    lds::asyncCopy16(aTile + r * kLen * E + (j % perRow) * 1024u,
                                     reinterpret_cast<const char*>(a) + (static_cast<size_t>(r) * lda + kBeg) * E
                                         + ((pos ^ (r & 15u)) << 4));
                }
            }

            FragAcc acc[MBlocks][NB];
#pragma unroll
            for(uint32_t i = 0; i < MBlocks; ++i)
#pragma unroll
                for(uint32_t j = 0; j < NB; ++j)
                    fill_fragment(acc[i][j], static_cast<CompT>(0));

            auto multiply = [&](FragB(&fb)[Ahead][NB], uint32_t kk) {
#pragma unroll
                for(uint32_t u = 0; u < Ahead; ++u)
#pragma unroll
                    for(uint32_t i = 0; i < MBlocks; ++i)
                    {
                        FragA          fa;
                        const uint32_t row = i * 16u + aRow;
#pragma unroll
                        for(uint32_t ch = 0; ch < MapA::nchunks; ++ch)
#pragma unroll
                            for(uint32_t piece = 0; piece < MapA::kpack * E / 16u; ++piece)
                            {
                                const uint32_t kByte = (kk + u * kSkinnyK + MapA::chunkK(ch, lane)) * E + piece * 16u;
                                detail::copyBytes<16u>(fa.x + ch * MapA::kpack + piece * (16u / E),
                                                       aTile + row * kLen * E + (((kByte >> 4) ^ (row & 15u)) << 4));
                            }
#pragma unroll
                        for(uint32_t j = 0; j < NB; ++j)
                            mma_sync(acc[i][j], fa, fb[u][j], acc[i][j]);
                    }
            };

            lds::waitCopiesAndReads<0>();
            __syncthreads();
            multiply(fb, 0u);
            for(uint32_t kk = Ahead * kSkinnyK; kk < kLen; kk += Ahead * kSkinnyK)
            {
                loadB(fb, kk);
                multiply(fb, kk);
            }

            // The partial tile (m x 256 results) replaces the A slice in LDS: rows of 64 16-byte
            // chunks, chunk c of row r at position c ^ (r % 16) (conflict-free for the 16 rows a
            // quarter-wave writes and for the 64 consecutive columns a wave reads back).
            __syncthreads();
            using Quad     = CompT __attribute__((ext_vector_type(4)));
            Quad* outTile  = reinterpret_cast<Quad*>(ldsRaw);
            constexpr uint32_t RowChunks = kSlicedCols / 4u;
#pragma unroll
            for(uint32_t i = 0; i < MBlocks; ++i)
#pragma unroll
                for(uint32_t j = 0; j < NB; ++j)
                {
                    const uint32_t row   = i * 16u + (lane & 15u);
                    const uint32_t chunk = (wave * NB + j) * 4u + (lane >> 4);
                    Quad           v     = *reinterpret_cast<Quad*>(acc[i][j].x);
                    outTile[row * RowChunks + (chunk ^ (row & 15u))] = alpha * v;
                }
            __syncthreads();
            const CompT* outFlat = reinterpret_cast<const CompT*>(ldsRaw);
            for(uint32_t row = wave; row < m; row += kSlicedWaves)
            {
#pragma unroll
                for(uint32_t q = 0; q < kSlicedCols / 64u; ++q)
                {
                    const uint32_t col  = q * 64u + lane;
                    const uint32_t gcol = blockIdx.x * kSlicedCols + col;
                    const CompT    v    = outFlat[(row * RowChunks + ((col >> 2) ^ (row & 15u))) * 4u + (col & 3u)];
                    if(gcol < n)
                        addTo(d + static_cast<size_t>(row) * ldd + gcol, v);
                }
            }
        }

        template <typename InT, typename OutT, typename CompT, uint32_t MBlocks>
        int launchSliced(GemmArgs const& g, hipStream_t stream, uint32_t slices)
        {
            const uint32_t slice  = g.m * (g.k / slices) * static_cast<uint32_t>(sizeof(InT)); // bytes of A per slice
            const uint32_t tile   = g.m * kSlicedCols * static_cast<uint32_t>(sizeof(CompT));
            const uint32_t lds    = slice > tile ? slice : tile;
            auto           kernel = gemmSlicedKernel<InT, OutT, CompT, MBlocks>;
            if(lds > 65536u
               && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(lds))
                      != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            const uint32_t quads = g.m * (g.n / 4u);
            hipLaunchKernelGGL((initOutputKernel<OutT, CompT>), dim3((quads + 255u) / 256u), dim3(256), 0, stream, g.m, g.n,
                               static_cast<OutT const*>(g.c), g.ldc, static_cast<OutT*>(g.d), g.ldd,
                               static_cast<CompT>(g.beta));
            hipLaunchKernelGGL(kernel, dim3((g.n + kSlicedCols - 1u) / kSlicedCols, slices), dim3(64u * kSlicedWaves), lds,
                               stream, g.m, g.n, g.k, static_cast<InT const*>(g.a), static_cast<InT const*>(g.b),
                               static_cast<OutT*>(g.d), g.lda, g.ldb, g.ldd, static_cast<CompT>(g.alpha));
            return launchStatus();
        }

        template <typename InT, typename OutT, typename CompT>
        int pickSliced(GemmArgs const& g, hipStream_t stream)
        {
            constexpr uint32_t E = sizeof(InT);
            // (n: the kernel that initialises D counts 4-element groups in 32 bits)
            if(g.m % 16u != 0u || g.m >= kSlicedMaxM || g.n % 16u != 0u || g.n > (1u << 24) || (g.k * E) % 1024u != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            // From 64 rows on the blocked kernel is as fast or faster, in one launch and without atomic adds
            // (its 64 x 64 tiles at 64 rows: 21 against 21 us; its partly filled 128 x 128 tiles at 80, 96,
            // 112 rows of int8 against 14336 x 4096: 25.5, 25.4, 26.4 us against 26.8, 29.0, 32.3 us here);
            // 48 rows stayed (20.8 against 24.6 us) until the blocked kernel got partly filled 128 x 64 tiles on
            // whole-line stages: where it runs those (one round of workgroups, 4 KiB of K and more) it takes 48
            // rows as well, 17.7 / 16.9 us int8 / fp8 against 20.9 / 22.5 us here.
            if(g.m >= 64u || gemmBlockedTakesPartlyFilledLineTiles(g.m, g.n, g.k, E))
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            // K slices: whole 1 KiB copies per row and whole batches of fragment steps per slice, the
            // A slice within 128 KiB of LDS; as few slices as fill the compute units
            const uint32_t groups = (g.n + kSlicedCols - 1u) / kSlicedCols;
            const uint32_t units  = g.k * E / 1024u;
            uint32_t       slices = 0;
            for(uint32_t s = 1; s <= units; ++s)
            {
                if(units % s != 0u || g.m * (g.k / s) * E > kSkinnyMaxA)
                    continue;
                slices = s;
                if(groups * s >= computeUnits() * 3u / 4u)
                    break;
            }
            if(slices == 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            switch(g.m / 16u)
            {
            case 1: // (16 and 32 rows come here only when all of A does not fit the LDS)
                return launchSliced<InT, OutT, CompT, 1>(g, stream, slices);
            case 2:
                return launchSliced<InT, OutT, CompT, 2>(g, stream, slices);
            case 3:
                return launchSliced<InT, OutT, CompT, 3>(g, stream, slices);
            default:
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            }
        }

        template <typename InT, typename OutT, typename CompT>
        int pickShape(GemmArgs const& g, hipStream_t stream)
        {
            constexpr uint32_t E = sizeof(InT);
            if(g.m > 32u || g.m * g.k * E > kSkinnyMaxA)
                return pickSliced<InT, OutT, CompT>(g, stream);
            // whole 1 KiB copies per row of A, whole fragment steps per K slice, A resident in LDS
            if(g.m % 16u != 0u || g.n % 16u != 0u || (g.k * E) % 1024u != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            // K steps of a wave's slice fetched together: as many as divide the slice, up to 8
            const uint32_t steps = g.k * E / (kSkinnySlices * kSkinnyKBytes);
            if(g.m == 16u)
            {
                if(steps % 8u == 0u)
                    return launchOne<InT, OutT, CompT, 1, 8>(g, stream);
                if(steps % 4u == 0u)
                    return launchOne<InT, OutT, CompT, 1, 4>(g, stream);
                return launchOne<InT, OutT, CompT, 1, 2>(g, stream);
            }
            if(steps % 8u == 0u)
                return launchOne<InT, OutT, CompT, 2, 8>(g, stream);
            if(steps % 4u == 0u)
                return launchOne<InT, OutT, CompT, 2, 4>(g, stream);
            return launchOne<InT, OutT, CompT, 2, 2>(g, stream);
        }
    } // namespace

    namespace
    {
        template <typename InT>
        int pickShapeMx(GemmArgs const& g, MxScales const& s, hipStream_t stream)
        {
            // as pickShape, for up to 32 token rows whose A fits the LDS; scale rows of A readable as dwords, of B
            // as 16-byte vectors
            if(g.m > 32u || g.m * g.k > kSkinnyMaxA)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            if(g.m % 16u != 0u || g.n % 16u != 0u || g.k % 1024u != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            if((reinterpret_cast<uintptr_t>(s.a) & 3u) || (reinterpret_cast<uintptr_t>(s.b) & 15u) || s.lda % 4u != 0u || s.ldb % 16u != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            const uint32_t steps = g.k / (kSkinnySlices * kSkinnyKBytes);
            if(g.m == 16u)
            {
                if(steps % 8u == 0u)
                    return launchOne<InT, float32_t, float32_t, 1, 8, true>(g, stream, s);
                if(steps % 4u == 0u)
                    return launchOne<InT, float32_t, float32_t, 1, 4, true>(g, stream, s);
                return launchOne<InT, float32_t, float32_t, 1, 2, true>(g, stream, s);
            }
            if(steps % 8u == 0u)
                return launchOne<InT, float32_t, float32_t, 2, 8, true>(g, stream, s);
            if(steps % 4u == 0u)
                return launchOne<InT, float32_t, float32_t, 2, 4, true>(g, stream, s);
            return launchOne<InT, float32_t, float32_t, 2, 2, true>(g, stream, s);
        }
    } // namespace

    int launchGemmMxSkinny(int dtypeIn, int layoutA, int layoutB, GemmArgs const& g, MxScales const& s, hipStream_t stream)
    {
        if(layoutA != ROCWMMA_AMD_ROW_MAJOR || layoutB != ROCWMMA_AMD_COL_MAJOR || g.layoutC != ROCWMMA_AMD_ROW_MAJOR)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        if(dtypeIn == ROCWMMA_AMD_E4M3)
            return pickShapeMx<float8_t>(g, s, stream);
        if(dtypeIn == ROCWMMA_AMD_E5M2)
            return pickShapeMx<bfloat8_t>(g, s, stream);
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    }

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
        if(dtypeIn == ROCWMMA_AMD_F16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickShape<float16_t, float32_t, float32_t>(g, stream);
        if(dtypeIn == ROCWMMA_AMD_BF16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickShape<bfloat16_t, float32_t, float32_t>(g, stream);
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    }

} // namespace rocwmma_amd
