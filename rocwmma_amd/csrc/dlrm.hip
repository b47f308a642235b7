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

        // Copies `halves` f16 values from LDS to global, whole workgroup.  `dst` is 2-byte aligned in
        // general (rows of odd width); the caller stages the data at an LDS address congruent to `dst`
        // modulo 16, so the 16-byte pieces are aligned on both sides and only the few halves in
        // front of the first and behind the last whole piece move one by one.
        ROCWMMA_DEVICE inline void copyOut(float16_t* dst, const float16_t* ldsSrc, uint32_t halves)
        {
            const uint32_t misalign = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(dst) & 15u) / 2u;
            const uint32_t head     = min(halves, (8u - misalign) & 7u);
            const uint32_t vecs     = (halves - head) / 8u;
            for(uint32_t i = threadIdx.x; i < vecs; i += blockDim.x)
                reinterpret_cast<u32x4_t*>(dst + head)[i] = reinterpret_cast<const u32x4_t*>(ldsSrc + head)[i];
            for(uint32_t i = threadIdx.x; i < head; i += blockDim.x)
                dst[i] = ldsSrc[i];
            for(uint32_t i = head + vecs * 8u + threadIdx.x; i < halves; i += blockDim.x)
                dst[i] = ldsSrc[i];
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
            const uint32_t sample0   = blockIdx.x * Samples;
            // the output block of the workgroup's samples, staged at an LDS address congruent to its
            // global address modulo 16 (see copyOut)
            float16_t* const outBlock = output + static_cast<size_t>(sample0) * width;
            float16_t*       ldsOut   = reinterpret_cast<float16_t*>(ldsRaw + tileBytes + (reinterpret_cast<uintptr_t>(outBlock) & 15u));

            const uint32_t lane    = threadIdx.x & 63u;
            const uint32_t wave    = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
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
                // bottom-MLP row: the sample's first feature row, copied from the LDS tile by the whole
                // wave (the output row starts on a 2-byte boundary only, so halves move one by one)
                {
                    const uint32_t   R0   = wave * m;
                    const float16_t* row0 = reinterpret_cast<const float16_t*>(ldsIn + R0 * Tile::rowBytes);
                    const uint32_t   swz0 = Tile::chunkSwizzle(R0);
#pragma unroll
                    for(uint32_t e = lane; e < K; e += 64u)
                        out[e] = row0[(((e / 8u) ^ swz0) << 3) + e % 8u];
                }
                // strict lower triangle, row by row.  Every lane writes all of its 16 values, those
                // outside the triangle into a spare half behind the output block, so the writes issue
                // back to back instead of one per branch.
                const uint32_t rowStart = K + (row * (row - 1u)) / 2u;
                const uint32_t spare    = (Samples - wave) * width + wave; // behind the last sample's row
#pragma unroll
                for(uint32_t e = 0; e < FragAcc::num_elements; ++e)
                {
                    const uint32_t c = AccMap::colOf(e, lane);
                    out[(row < m && c < row) ? rowStart + c : spare] = static_cast<float16_t>(acc.x[e]);
                }
            }
            __syncthreads();
            copyOut(outBlock, ldsOut, nHere * width);
        }

        // ------------------------------------------------------------------ backward
        // LDS staging of the gradient: the m x K result of a sample replaces its feature rows.  A lane
        // writes runs of four columns of one row (8 bytes); the 32 lanes of a half-wave hold 32
        // consecutive rows at the same column, which in a plain row-major stage are 32 addresses
        // one row pitch apart: one bank.  The 8-byte units of LDS row R are therefore stored at unit
        // position u ^ (R % units), and the write-out, which moves 16 bytes (two units whose positions
        // differ in bit 0 only), reads them back and swaps the pair where R is odd.
        template <uint32_t K>
        struct GradStage
        {
            static constexpr uint32_t rowBytes = K * 2u;
            static constexpr uint32_t units    = K / 4u; // 8-byte units per row
            static constexpr uint32_t mask     = (units < 32u ? units : 32u) - 1u;

            ROCWMMA_DEVICE static inline uint32_t unitOffset(uint32_t R, uint32_t unit)
            {
                return R * rowBytes + ((unit ^ (R & mask)) << 3);
            }
        };

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
            using Stage                = GradStage<K>;
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

            // features: direct copies, segment-swizzled for the transposing reads.  (Rows behind the
            // last sample are never copied: whatever the LDS holds there only meets contraction indices
            // >= m, which are masked out of the operand registers below.)
            const uint32_t featBytes = nHere * m * Tile::rowBytes;
            Tile::template asyncLoad<true>(ldsF, input + static_cast<size_t>(sample0) * m * K, featBytes, wave, Samples, lane);
            // upstream gradients (contiguous for the workgroup's samples): direct copies of 4 bytes per
            // lane (the first sample of a workgroup has an even index, so the block starts on a 4-byte
            // boundary whatever the row width).  An odd number of samples of odd width leaves two bytes
            // behind the last whole word: no lane copies that word (nothing is read past the end of the
            // caller's array), one lane moves the last half by hand.
            {
                const uint32_t        upBytes = nHere * width * 2u;
                const uint32_t        whole   = upBytes & ~3u;
                const float16_t*      upBlock = upstream + static_cast<size_t>(sample0) * width;
                const lds::BufferRsrc rsrc
                    = __builtin_amdgcn_make_buffer_rsrc(const_cast<float16_t*>(upBlock), 0, static_cast<int>(whole), 0x00020000);
                for(uint32_t copy = wave; copy * 256u < whole; copy += Samples)
                    if(copy * 256u + lane * 4u < whole)
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds::LdsPtr)(reinterpret_cast<char*>(ldsUp) + copy * 256u), 4,
                                                                 static_cast<int>(copy * 256u + lane * 4u), 0, 0, 2 /* nt */);
                if(whole != upBytes && threadIdx.x == 0u)
                    ldsUp[whole / 2u] = upBlock[whole / 2u];
            }
            lds::waitCopiesAndReads<0>();
            __syncthreads();

            // bottom-MLP gradient = the first K entries of every upstream row; a row starts on a 2-byte
            // boundary only, so it is read as halves.  Issued first: the stores drain under the arithmetic.
            for(uint32_t i = threadIdx.x; i < nHere * (K / 8u); i += blockDim.x)
            {
                const uint32_t   s   = i / (K / 8u);
                const uint32_t   c8  = i % (K / 8u);
                const float16_t* src = ldsUp + s * width + c8 * 8u;
                float16_t        tmp[8];
#pragma unroll
                for(uint32_t j = 0; j < 8u; ++j)
                    tmp[j] = src[j];
                reinterpret_cast<u32x4_t*>(mlpGrad + static_cast<size_t>(sample0 + s) * K)[c8] = *reinterpret_cast<u32x4_t*>(tmp);
            }

            FragAcc acc[NBlocks];
            if(wave < nHere)
            {
                const uint32_t   row    = lane & 31u;
                const uint32_t   kGroup = lane >> 5;
                const float16_t* up     = ldsUp + wave * width;

                // G operand: row `row`, columns ks*16 + kGroup*8 + j, rebuilt from the packed triangle.
                // Every lane reads all of its 16 entries (a harmless address where there is none) and
                // selects afterwards, so the reads issue back to back instead of one per branch.
                FragG fg[2];
                // packed position of G(row, c): below the diagonal the row's entries are consecutive
                // (tri(row) + c); above it entry (c, row) sits at tri(c) + row with tri(c + 1) = tri(c) + c
                const uint32_t below = K + (row * (row - 1u)) / 2u;
#pragma unroll
                for(uint32_t ks = 0; ks < 2u; ++ks)
                {
                    const uint32_t c0    = ks * 16u + kGroup * 8u;
                    uint32_t       above = K + (c0 * (c0 - 1u)) / 2u + row; // (c0 = 0: the product wraps to 0)
#pragma unroll
                    for(uint32_t j = 0; j < 8u; ++j)
                    {
                        const uint32_t c     = c0 + j;
                        const bool     there = (c > row ? c : row) < m && c != row;
                        const float16_t g    = up[there ? (c < row ? below + c : above) : 0u];
                        fg[ks].x[j]          = there ? g : static_cast<float16_t>(0);
                        above += c;
                    }
                }

                // F operands: transposing reads, lane l gets column nb*32 + l%32 and contraction
                // rows ks*16 + (l/32)*8 + 0..7 of this sample
                const uint32_t group   = lane >> 4;
                const uint32_t s16     = lane & 15u;
                const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds::LdsPtr)ldsF));
                uint32_t       ff[NBlocks][2][4]; // [block][k step][two halves per word]
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
                            typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
                            u32x2_t v;
                            asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(addr) : "memory");
                            ff[nb][ks][2u * kk]      = v[0];
                            ff[nb][ks][2u * kk + 1u] = v[1];
                        }
                // Contraction rows >= m are the next sample's features (or stale LDS): G is zero there,
                // but 0 * Inf and 0 * NaN are NaN, so those operand halves are cleared, which keeps
                // the samples independent of one another as in the reference's CPU loops
                // (test/reference_impl.hpp:121-179).  Word w of step ks holds contraction indices
                // ks*16 + (l/32)*8 + 2w, + 1.
                uint32_t keep[2][4];
#pragma unroll
                for(uint32_t ks = 0; ks < 2u; ++ks)
#pragma unroll
                    for(uint32_t w = 0; w < 4u; ++w)
                    {
                        const uint32_t c0 = ks * 16u + kGroup * 8u + 2u * w;
                        keep[ks][w]       = (c0 < m ? 0x0000FFFFu : 0u) | (c0 + 1u < m ? 0xFFFF0000u : 0u);
                    }
                // the wait also makes the registers written by the inline assembly valid for what follows
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
                for(uint32_t nb = 0; nb < NBlocks; ++nb)
                {
                    fill_fragment(acc[nb], 0.0f);
#pragma unroll
                    for(uint32_t ks = 0; ks < 2u; ++ks)
                    {
                        FragF f;
#pragma unroll
                        for(uint32_t w = 0; w < 4u; ++w)
                        {
                            // (the "+v" ties each operand word to a point behind the wait)
                            asm volatile("" : "+v"(ff[nb][ks][w]));
                            reinterpret_cast<uint32_t*>(f.x)[w] = ff[nb][ks][w] & keep[ks][w];
                        }
                        mma_sync(acc[nb], fg[ks], f, acc[nb]);
                    }
                }
            }
            __syncthreads(); // every wave is done reading features (its own and its neighbour's rows)

            if(wave < nHere)
            {
                // this sample's feature rows become the staging buffer of its gradient (m x K)
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
                            float16_t h[4];
#pragma unroll
                            for(uint32_t j = 0; j < 4u; ++j)
                                h[j] = static_cast<float16_t>(acc[nb].x[e0 + j]);
                            typedef uint32_t u32x2_t __attribute__((ext_vector_type(2), may_alias));
                            *reinterpret_cast<u32x2_t*>(ldsF + Stage::unitOffset(wave * m + r, c / 4u)) = *reinterpret_cast<u32x2_t*>(h);
                        }
                    }
            }
            __syncthreads();

            // coalesced write-out: gradients of all samples are one contiguous block of 16-byte pieces
            {
                constexpr uint32_t chunksPerRow = K / 8u;
                u32x4_t*           dst          = reinterpret_cast<u32x4_t*>(grad + static_cast<size_t>(sample0) * m * K);
                for(uint32_t q = threadIdx.x; q < nHere * m * chunksPerRow; q += blockDim.x)
                {
                    const uint32_t R = q / chunksPerRow, ch = q % chunksPerRow;
                    const uint32_t s = R & Stage::mask;
                    u32x4_t        v = *reinterpret_cast<const u32x4_t*>(ldsF + R * Stage::rowBytes + ((ch ^ (s >> 1)) << 4));
                    if(s & 1u)
                        v = u32x4_t{v[2], v[3], v[0], v[1]};
                    dst[q] = v;
                }
            }
        }

        // ------------------------------------------------------------------ more than 32 feature rows
        // 32 < m <= 128 (the reference's DLRM tests also run m = 128, test/dlrm/test/dlrm_test_params.hpp:51-58): the
        // same wave-per-sample structure with the sample's rows cut into tiles of 32.  Forward: Z block (I, J), J <= I,
        // is F_I F_J^T, one 32 x 32 accumulator at a time.  Backward: row tile I of the gradient is the sum over
        // contraction tiles J of G_IJ F_J, with the G fragments of a row tile rebuilt once from the packed triangle
        // and the result staged per wave.  One or two samples per workgroup, whatever fits the LDS.  These shapes
        // are not a benchmark configuration; the kernels are written for parity, with the data paths of the ones above.
        constexpr uint32_t kMaxTiledM = 128;

        template <uint32_t K, uint32_t Samples>
        __global__ void __launch_bounds__(64 * Samples)
            dlrmFwdTiledKernel(const float16_t* __restrict__ input, float16_t* __restrict__ output, uint32_t m, uint32_t batch)
        {
            constexpr uint32_t KSteps = K / 16u;
            using Tile                = FeatureTile<K>;
            using FragA               = fragment<matrix_a, 32, 32, 16, float16_t, row_major>;
            using FragAcc             = fragment<accumulator, 32, 32, 16, float32_t>;
            using AccMap              = detail::AccMap<32, 32, 32>;

            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];
            const uint32_t width     = K + (m * (m - 1u)) / 2u;
            const uint32_t tiles     = (m + 31u) / 32u;
            const uint32_t tileBytes = (((Samples - 1u) * m + tiles * 32u) * Tile::rowBytes + 1023u) & ~1023u;
            char*          ldsIn     = ldsRaw;
            const uint32_t sample0   = blockIdx.x * Samples;
            float16_t* const outBlock = output + static_cast<size_t>(sample0) * width;
            float16_t*       ldsOut   = reinterpret_cast<float16_t*>(ldsRaw + tileBytes + (reinterpret_cast<uintptr_t>(outBlock) & 15u));

            const uint32_t lane  = threadIdx.x & 63u;
            const uint32_t wave  = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t nHere = min(Samples, batch - sample0);

            Tile::template asyncLoad<false>(ldsIn, input + static_cast<size_t>(sample0) * m * K, nHere * m * Tile::rowBytes,
                                            wave, Samples, lane);
            lds::waitCopiesAndReads<0>();
            __syncthreads();

            if(wave < nHere)
            {
                const uint32_t row    = lane & 31u;
                const uint32_t kGroup = lane >> 5;
                float16_t*     out    = ldsOut + wave * width;
                {
                    const uint32_t   R0   = wave * m;
                    const float16_t* row0 = reinterpret_cast<const float16_t*>(ldsIn + R0 * Tile::rowBytes);
                    const uint32_t   swz0 = Tile::chunkSwizzle(R0);
#pragma unroll
                    for(uint32_t e = lane; e < K; e += 64u)
                        out[e] = row0[(((e / 8u) ^ swz0) << 3) + e % 8u];
                }
                const uint32_t spare = (Samples - wave) * width + wave; // behind the last sample's row
                // operand of tile T: matrix row = lane % 32 (rows >= m belong to the next sample or are stale LDS:
                // they only reach Gram entries with an index >= m, which are dropped)
                auto loadTile = [&](FragA(&f)[KSteps], uint32_t T) {
                    const uint32_t R   = wave * m + T * 32u + row;
                    const uint32_t swz = Tile::chunkSwizzle(R);
#pragma unroll
                    for(uint32_t ks = 0; ks < KSteps; ++ks)
                        *reinterpret_cast<u32x4_t*>(f[ks].x)
                            = *reinterpret_cast<const u32x4_t*>(ldsIn + R * Tile::rowBytes + (((ks * 2u + kGroup) ^ swz) << 4));
                };
#pragma unroll 1
                for(uint32_t I = 0; I < tiles; ++I)
                {
                    FragA fI[KSteps];
                    loadTile(fI, I);
                    const uint32_t Rg       = I * 32u + row; // row of Z
                    const uint32_t rowStart = K + (Rg * (Rg - 1u)) / 2u;
#pragma unroll 1
                    for(uint32_t J = 0; J <= I; ++J)
                    {
                        FragA fJ[KSteps];
                        loadTile(fJ, J);
                        FragAcc acc;
                        fill_fragment(acc, 0.0f);
#pragma unroll
                        for(uint32_t ks = 0; ks < KSteps; ++ks)
                            mma_sync(acc, fI[ks], applyTranspose(fJ[ks]), acc);
#pragma unroll
                        for(uint32_t e = 0; e < FragAcc::num_elements; ++e)
                        {
                            const uint32_t Cg = J * 32u + AccMap::colOf(e, lane);
                            out[(Rg < m && Cg < Rg) ? rowStart + Cg : spare] = static_cast<float16_t>(acc.x[e]);
                        }
                    }
                }
            }
            __syncthreads();
            copyOut(outBlock, ldsOut, nHere * width);
        }

        template <uint32_t K, uint32_t Samples>
        __global__ void __launch_bounds__(64 * Samples) dlrmBwdTiledKernel(const float16_t* __restrict__ input,
                                                                                const float16_t* __restrict__ upstream,
                                                                                float16_t* __restrict__ grad,
                                                                                float16_t* __restrict__ mlpGrad,
                                                                                uint32_t m,
                                                                                uint32_t batch)
        {
            constexpr uint32_t NBlocks  = K / 32u; // 32-column blocks of the m x K result
            constexpr uint32_t MaxTiles = kMaxTiledM / 32u;
            using Tile                  = FeatureTile<K>;
            using Stage                 = GradStage<K>;
            using FragG                 = fragment<matrix_a, 32, 32, 16, float16_t, row_major>;
            using FragF                 = fragment<matrix_b, 32, 32, 16, float16_t, row_major>;
            using FragAcc               = fragment<accumulator, 32, 32, 16, float32_t>;
            using AccMap                = detail::AccMap<32, 32, 32>;

            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];
            const uint32_t width     = K + (m * (m - 1u)) / 2u;
            const uint32_t tiles     = (m + 31u) / 32u;
            const uint32_t tileBytes = (((Samples - 1u) * m + tiles * 32u) * Tile::rowBytes + 1023u) & ~1023u;
            const uint32_t upBytesLds = (Samples * width * 2u + 2u + 255u) & ~255u;
            char*          ldsF      = ldsRaw;
            float16_t*     ldsUp     = reinterpret_cast<float16_t*>(ldsRaw + tileBytes);
            char*          ldsStage  = ldsRaw + tileBytes + upBytesLds; // per wave: 32 rows of the gradient

            const uint32_t lane    = threadIdx.x & 63u;
            const uint32_t wave    = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t sample0 = blockIdx.x * Samples;
            const uint32_t nHere   = min(Samples, batch - sample0);

            Tile::template asyncLoad<true>(ldsF, input + static_cast<size_t>(sample0) * m * K, nHere * m * Tile::rowBytes, wave, Samples,
                                           lane);
            // upstream gradients: 4-byte direct copies.  With one sample per workgroup and an odd row width a
            // block can start on an odd half: it is then copied from the half in front of it (the previous
            // sample's last) and read one half on.
            const float16_t* upBlock = upstream + static_cast<size_t>(sample0) * width;
            const uint32_t   upSkew  = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(upBlock) & 2u) / 2u; // 0 or 1 halves
            {
                const float16_t*      from    = upBlock - upSkew;
                const uint32_t        upBytes = (nHere * width + upSkew) * 2u;
                const uint32_t        whole   = upBytes & ~3u;
                const lds::BufferRsrc rsrc
                    = __builtin_amdgcn_make_buffer_rsrc(const_cast<float16_t*>(from), 0, static_cast<int>(whole), 0x00020000);
                for(uint32_t copy = wave; copy * 256u < whole; copy += Samples)
                    if(copy * 256u + lane * 4u < whole)
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds::LdsPtr)(reinterpret_cast<char*>(ldsUp) + copy * 256u), 4,
                                                                 static_cast<int>(copy * 256u + lane * 4u), 0, 0, 2 /* nt */);
                if(whole != upBytes && threadIdx.x == 0u)
                    ldsUp[whole / 2u] = from[whole / 2u];
            }
            lds::waitCopiesAndReads<0>();
            __syncthreads();
            const float16_t* upLds = ldsUp + upSkew;

            for(uint32_t i = threadIdx.x; i < nHere * (K / 8u); i += blockDim.x)
            {
                const uint32_t   s   = i / (K / 8u);
                const uint32_t   c8  = i % (K / 8u);
                const float16_t* src = upLds + s * width + c8 * 8u;
                float16_t        tmp[8];
#pragma unroll
                for(uint32_t j = 0; j < 8u; ++j)
                    tmp[j] = src[j];
                reinterpret_cast<u32x4_t*>(mlpGrad + static_cast<size_t>(sample0 + s) * K)[c8] = *reinterpret_cast<u32x4_t*>(tmp);
            }

            if(wave < nHere)
            {
                const uint32_t   row     = lane & 31u;
                const uint32_t   kGroup  = lane >> 5;
                const uint32_t   group   = lane >> 4;
                const uint32_t   s16     = lane & 15u;
                const float16_t* up      = upLds + wave * width;
                const uint32_t   ldsBase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds::LdsPtr)ldsF));
                char*            stage   = ldsStage + wave * (32u * Stage::rowBytes);
                u32x4_t*         dstSample = reinterpret_cast<u32x4_t*>(grad + static_cast<size_t>(sample0 + wave) * m * K);
#pragma unroll 1
                for(uint32_t I = 0; I < tiles; ++I)
                {
                    // G operands of row tile I against every contraction tile J: row Rg, columns J*32 + ks*16 +
                    // kGroup*8 + j, rebuilt from the packed triangle (every lane reads all of its entries, a harmless
                    // address where there is none, and selects afterwards)
                    const uint32_t Rg    = I * 32u + row;
                    const uint32_t below = K + (Rg * (Rg - 1u)) / 2u;
                    FragG          fg[MaxTiles][2];
#pragma unroll
                    for(uint32_t J = 0; J < MaxTiles; ++J)
#pragma unroll
                        for(uint32_t ks = 0; ks < 2u; ++ks)
                        {
                            const uint32_t c0    = J * 32u + ks * 16u + kGroup * 8u;
                            uint32_t       above = K + (c0 * (c0 - 1u)) / 2u + Rg; // (c0 = 0: the product wraps to 0)
#pragma unroll
                            for(uint32_t j = 0; j < 8u; ++j)
                            {
                                const uint32_t  c     = c0 + j;
                                const bool      there = (c > Rg ? c : Rg) < m && c != Rg;
                                const float16_t g     = up[there ? (c < Rg ? below + c : above) : 0u];
                                fg[J][ks].x[j]        = there ? g : static_cast<float16_t>(0);
                                above += c;
                            }
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
                                // F operands: transposing reads, lane l gets column nb*32 + l%32 and contraction rows
                                // J*32 + ks*16 + (l/32)*8 + 0..7 of this sample
                                uint32_t ff[2][4];
#pragma unroll
                                for(uint32_t ks = 0; ks < 2u; ++ks)
#pragma unroll
                                    for(uint32_t kk = 0; kk < 2u; ++kk)
                                    {
                                        const uint32_t c    = J * 32u + ks * 16u + (group >> 1) * 8u + kk * 4u + (s16 >> 2);
                                        const uint32_t R    = wave * m + c;
                                        const uint32_t seg  = nb * 2u + (group & 1u);
                                        const uint32_t addr = ldsBase + R * Tile::rowBytes + ((seg ^ Tile::segmentSwizzle(R)) << 5)
                                                              + ((s16 & 3u) << 3);
                                        typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
                                        u32x2_t v;
                                        asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(addr) : "memory");
                                        ff[ks][2u * kk]      = v[0];
                                        ff[ks][2u * kk + 1u] = v[1];
                                    }
                                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
                                for(uint32_t ks = 0; ks < 2u; ++ks)
                                {
                                    FragF f;
#pragma unroll
                                    for(uint32_t w = 0; w < 4u; ++w)
                                    {
                                        // contraction rows >= m are the next sample's features or stale LDS: cleared, so
                                        // that 0 * Inf and 0 * NaN cannot leak between samples
                                        const uint32_t c0   = J * 32u + ks * 16u + kGroup * 8u + 2u * w;
                                        const uint32_t keep = (c0 < m ? 0x0000FFFFu : 0u) | (c0 + 1u < m ? 0xFFFF0000u : 0u);
                                        asm volatile("" : "+v"(ff[ks][w]));
                                        reinterpret_cast<uint32_t*>(f.x)[w] = ff[ks][w] & keep;
                                    }
                                    mma_sync(acc, fg[J][ks], f, acc);
                                }
                            }
                        }
                        // into this wave's staging rows (8-byte units XOR-swizzled by the row)
#pragma unroll
                        for(uint32_t r4 = 0; r4 < AccMap::runs; ++r4)
                        {
                            const uint32_t e0 = r4 * 4u;
                            const uint32_t r  = AccMap::rowOf(e0, lane);
                            const uint32_t c  = nb * 32u + AccMap::colOf(e0, lane);
                            float16_t      h[4];
#pragma unroll
                            for(uint32_t j = 0; j < 4u; ++j)
                                h[j] = static_cast<float16_t>(acc.x[e0 + j]);
                            typedef uint32_t u32x2_t __attribute__((ext_vector_type(2), may_alias));
                            *reinterpret_cast<u32x2_t*>(stage + Stage::unitOffset(r, c / 4u)) = *reinterpret_cast<u32x2_t*>(h);
                        }
                    }
                    // rows I*32 .. of this sample's gradient: one contiguous block of 16-byte pieces
                    {
                        constexpr uint32_t chunksPerRow = K / 8u;
                        const uint32_t     rowsHere     = min(32u, m - I * 32u);
                        u32x4_t*           dst          = dstSample + static_cast<size_t>(I) * 32u * chunksPerRow;
                        for(uint32_t q = lane; q < rowsHere * chunksPerRow; q += 64u)
                        {
                            const uint32_t R = q / chunksPerRow, ch = q % chunksPerRow;
                            const uint32_t s = R & Stage::mask;
                            u32x4_t        v = *reinterpret_cast<const u32x4_t*>(stage + R * Stage::rowBytes + ((ch ^ (s >> 1)) << 4));
                            if(s & 1u)
                                v = u32x4_t{v[2], v[3], v[0], v[1]};
                            dst[q] = v;
                        }
                    }
                }
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
            // (+ 32: the output staging starts at the output block's global address modulo 16, and a spare
            // half per wave follows the block)
            const uint32_t lds    = tileBytesFor<K, Samples>(m) + ((Samples * width * 2u + 15u) & ~15u) + 32u;
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
            // (the upstream block arrives as whole 256-byte copies)
            const uint32_t lds    = tileBytesFor<K, Samples>(m) + ((Samples * width * 2u + 255u) & ~255u);
            const uint32_t grid   = (batch + Samples - 1u) / Samples;
            auto           kernel = dlrmBwdKernel<K, Samples>;
            if(int rc = optInLds(kernel, lds))
                return rc;
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(64u * Samples), lds, stream, static_cast<const float16_t*>(input),
                               static_cast<const float16_t*>(upstream), static_cast<float16_t*>(grad),
                               static_cast<float16_t*>(mlpGrad), m, batch);
            return launchStatus();
        }
        // Samples per workgroup for a batch.  Backward: 8 once that still leaves >= 8 workgroups per compute
        // unit (the longest contiguous stores; batch 262144: 706 us against 722 us with 4).  Forward: 4 at
        // most -- four workgroups of 33 KiB of LDS per compute unit overlap their load, multiply and store phases
        // better than two of 65 KiB (batch 262144: 328 us against 347 us with 8, 6.28 against 5.94 TB/s).  2 for
        // small batches, so that every compute unit still gets several workgroups.  (Non-temporal stores in the
        // write-outs: no difference, 707 against 706 us backward.)
        inline uint32_t samplesFor(uint32_t batch, bool forward)
        {
            const uint32_t cus = computeUnits();
            if(batch >= 64u * cus && !forward)
                return 8u;
            return batch >= 8u * cus ? 4u : 2u;
        }

        constexpr uint32_t kLdsBytes = 160u * 1024u;

        template <uint32_t K, uint32_t Samples>
        int launchFwdTiledS(const void* input, void* output, uint32_t m, uint32_t batch, hipStream_t stream)
        {
            const uint32_t width = K + (m * (m - 1u)) / 2u, tiles = (m + 31u) / 32u;
            const uint32_t lds   = ((((Samples - 1u) * m + tiles * 32u) * K * 2u + 1023u) & ~1023u) + ((Samples * width * 2u + 15u) & ~15u) + 32u;
            if(lds > kLdsBytes)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            auto kernel = dlrmFwdTiledKernel<K, Samples>;
            if(int rc = optInLds(kernel, lds))
                return rc;
            hipLaunchKernelGGL(kernel, dim3((batch + Samples - 1u) / Samples), dim3(64u * Samples), lds, stream,
                               static_cast<const float16_t*>(input), static_cast<float16_t*>(output), m, batch);
            return launchStatus();
        }

        template <uint32_t K, uint32_t Samples>
        int launchBwdTiledS(const void* input, const void* upstream, void* grad, void* mlpGrad, uint32_t m, uint32_t batch,
                            hipStream_t stream)
        {
            const uint32_t width = K + (m * (m - 1u)) / 2u, tiles = (m + 31u) / 32u;
            const uint32_t lds   = ((((Samples - 1u) * m + tiles * 32u) * K * 2u + 1023u) & ~1023u) + ((Samples * width * 2u + 2u + 255u) & ~255u)
                                 + Samples * 32u * K * 2u;
            if(lds > kLdsBytes)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            auto kernel = dlrmBwdTiledKernel<K, Samples>;
            if(int rc = optInLds(kernel, lds))
                return rc;
            hipLaunchKernelGGL(kernel, dim3((batch + Samples - 1u) / Samples), dim3(64u * Samples), lds, stream,
                               static_cast<const float16_t*>(input), static_cast<const float16_t*>(upstream),
                               static_cast<float16_t*>(grad), static_cast<float16_t*>(mlpGrad), m, batch);
            return launchStatus();
        }

        template <uint32_t K>
        int launchFwd(const void* input, void* output, uint32_t m, uint32_t batch, hipStream_t stream)
        {
            if(m > kMaxM)
            {
                // two samples per workgroup where the LDS holds them, else one
                const int rc = launchFwdTiledS<K, 2>(input, output, m, batch, stream);
                return rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE ? rc : launchFwdTiledS<K, 1>(input, output, m, batch, stream);
            }
            switch(samplesFor(batch, true))
            {
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
            if(m > kMaxM)
            {
                const int rc = launchBwdTiledS<K, 2>(input, upstream, grad, mlpGrad, m, batch, stream);
                return rc != ROCWMMA_AMD_UNSUPPORTED_SHAPE ? rc : launchBwdTiledS<K, 1>(input, upstream, grad, mlpGrad, m, batch, stream);
            }
            switch(samplesFor(batch, false))
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
