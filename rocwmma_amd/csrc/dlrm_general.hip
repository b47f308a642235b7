// DLRM dot interaction for the shapes the one-wave-per-sample kernels (dlrm.hip, dlrm_f32.hip) do not take:
// more than 128 feature rows, or a feature width other than 32 / 64 / 128 / 256.  The reference's tests run
// (m, k) = (1024, 1024) among others (test/dlrm/test/dlrm_test_params.hpp:51-68); semantics = dlrm_fwd_CPU /
// dlrm_bwd_CPU (test/reference_impl.hpp:83-179).
//
// A sample of that size is a matrix product of its own (1024 x 1024 x 1024), so a sample's work is cut into tiles
// of 128 x 128 over workgroups of four waves (2 x 2, 64 x 64 each, 32 x 32 blocks), one grid for the whole batch:
//
//   * forward: tile (I, J), J <= I, of Z = F F^T; both operands are rows of F with K contiguous.  The strict lower
//     triangle leaves through a 32 x 32 LDS block per wave as row pieces, which are contiguous in the packed
//     output.  No m x m scratch in global memory.
//   * backward: tile (I, N) of grad = S F, S = the symmetric matrix with zero diagonal whose strict lower triangle
//     is the packed upstream gradient, never materialised: where the contraction index lies below the tile's rows
//     the packed triangle holds S row by row, where it lies above them it holds the transpose, and only the
//     stages that meet the diagonal are gathered element by element.
//
// Operands go through LDS (coalesced 16-byte pieces into registers one stage ahead, then LDS, then fragments).
// Rows from m on and columns from k on are never read: their lanes multiply zeros.  These shapes are no benchmark
// configuration; the kernels are written for parity and reasonable speed, not tuned to the last tenth.
#include "common.hpp"
#include <rocwmma/rocwmma_lds.hpp>
#include <rocwmma/rocwmma_transforms.hpp>

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        typedef uint32_t u32x4_t __attribute__((ext_vector_type(4), may_alias));
        typedef uint32_t u32x2_t __attribute__((ext_vector_type(2), may_alias));
        typedef float    f32x4_t __attribute__((ext_vector_type(4), may_alias));

        constexpr uint32_t kTile       = 128; // workgroup tile edge
        constexpr uint32_t kWaveTile   = 64;
        constexpr uint32_t kMaxRows    = 32768; // m * (m - 1) stays below 2^32
        constexpr uint32_t kNowhere    = 0x80000000u; // beyond every sample: a bounds-checked load there returns zero

        // offset of Z(row, 0) in a sample's packed output / upstream row
        ROCWMMA_DEVICE inline size_t packedRow(uint32_t k, uint32_t row)
        {
            return static_cast<size_t>(k) + (static_cast<size_t>(row) * (row - (row != 0u))) / 2u;
        }

        ROCWMMA_DEVICE inline void waveSync()
        {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }

        // Which (sample, tile) a workgroup takes.  Workgroups are handed to the device's 8 XCDs in turn (workgroup w
        // runs on XCD w % 8), and every XCD has an L2 of its own: all tiles of a sample go to one XCD, sample s to XCD
        // s % 8, so that a sample's operands are fetched into one L2 once instead of into all eight (measured at
        // (1024, 1024, 64) in f16: 955 MiB fetched per forward launch for 128 MiB of features with the tiles of a
        // sample dealt out over the XCDs).  The grid is 8 * ceil(batch / 8) * tiles workgroups.
        constexpr uint32_t kXcds = 8;
        ROCWMMA_DEVICE inline void sampleAndTile(uint32_t tiles, uint32_t& sample, uint32_t& tile)
        {
            const uint32_t slot = blockIdx.x / kXcds;
            sample              = (slot / tiles) * kXcds + blockIdx.x % kXcds;
            tile                = slot % tiles;
        }

        // ------------------------------------------------------------------ operands through LDS
        // In the fragment layout consecutive lanes hold different rows, and a global load whose lanes touch 32
        // different cache lines is served at a fraction of the rate of one whose lanes read consecutive addresses
        // (with operands straight from global memory the f16 kernels ran at half (forward) and at 0.4 (backward) of
        // the rate at (1024, 1024, 64)).  So a thread fetches consecutive 16-byte pieces of a tile row into registers (one
        // stage ahead of the multiplication), the pieces go to LDS, and the fragments come from there.
        //
        // Two LDS layouts for float16, 64 contraction indices per stage (float32 below):
        //   "rows":    128 tile rows of 64 halves of K (row pitch 144 bytes: 16-byte aligned, rows spread over the
        //              banks); a fragment is one 16-byte read per lane.  Forward: both operands.  Backward: S where
        //              the packed triangle holds it row by row (contraction index below the tile's rows).
        //   "columns": 64 contraction rows of 128 halves (the 32-byte segments of a row XOR-ed with 2 * (row % 4),
        //              which spreads the 4 rows x 2 segments of one transposing read over 8 bank groups); a fragment
        //              is two transposing 8-byte reads per lane.  Backward: F, and S where the packed triangle holds
        //              its transpose (contraction index above the tile's rows).
        constexpr uint32_t kStageK    = 64;
        constexpr uint32_t kRowPitch  = 144;
        constexpr uint32_t kRowsBytes = kTile * kRowPitch; // 18432
        constexpr uint32_t kColBytes  = kTile * 2u; // bytes per contraction row of the "columns" layout
        constexpr uint32_t kColsBytes = kStageK * kColBytes; // 16384

        ROCWMMA_DEVICE inline uint32_t segmentSwizzle(uint32_t row)
        {
            return (row & 3u) << 1;
        }

        // byte offset of 16-byte piece `pos` of contraction row `row` in the "columns" layout
        ROCWMMA_DEVICE inline uint32_t columnsOffset(uint32_t row, uint32_t pos)
        {
            return row * kColBytes + ((((pos >> 1) ^ segmentSwizzle(row)) << 5) | ((pos & 1u) << 4));
        }

        // 16 bytes at a 2-byte aligned address (rows of the packed triangle start anywhere)
        struct __attribute__((packed, aligned(2))) UnalignedPiece
        {
            uint32_t w[4];
        };
        ROCWMMA_DEVICE inline u32x4_t loadUnaligned(const float16_t* from)
        {
            const UnalignedPiece p = *reinterpret_cast<const UnalignedPiece*>(from);
            return u32x4_t{p.w[0], p.w[1], p.w[2], p.w[3]};
        }

        using FragK16   = fragment<matrix_a, 32, 32, 16, float16_t, row_major>;
        using FragAcc16 = fragment<accumulator, 32, 32, 16, float32_t>;

        // fragment words of 32-row block `block32` (of the tile's 128 rows) at K step `ks` (16 halves) of a "rows" tile
        ROCWMMA_DEVICE inline u32x4_t rowsFragment(const char* tile, uint32_t block32, uint32_t ks, uint32_t lane)
        {
            return *reinterpret_cast<const u32x4_t*>(tile + (block32 * 32u + (lane & 31u)) * kRowPitch + ks * 32u + (lane >> 5) * 16u);
        }

        // fragment words of 32-column block `block32` at K step `ks` of a "columns" tile: lane l gets column
        // block32 * 32 + l % 32 and contraction rows ks * 16 + (l / 32) * 8 + 0..7, as two transposing 8-byte reads
        // (through the compiler's builtin, so that it keeps the wait counters and schedules the reads itself)
        typedef short s16x4_t __attribute__((ext_vector_type(4)));
        ROCWMMA_DEVICE inline u32x4_t columnsFragment(const char* tile, uint32_t block32, uint32_t ks, uint32_t lane)
        {
            const uint32_t group = lane >> 4, s16 = lane & 15u;
            u32x4_t        words;
#pragma unroll
            for(uint32_t kk = 0; kk < 2u; ++kk)
            {
                const uint32_t row = ks * 16u + (group >> 1) * 8u + kk * 4u + (s16 >> 2);
                const uint32_t seg = block32 * 2u + (group & 1u);
                const char*    at  = tile + row * kColBytes + ((seg ^ segmentSwizzle(row)) << 5) + ((s16 & 3u) << 3);
                const s16x4_t  v   = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)at);
                const u32x2_t  w   = __builtin_bit_cast(u32x2_t, v);
                words[2u * kk]      = w[0];
                words[2u * kk + 1u] = w[1];
            }
            return words;
        }

        template <typename Frag>
        ROCWMMA_DEVICE inline Frag fragmentOf(const u32x4_t& words)
        {
            Frag f;
            *reinterpret_cast<u32x4_t*>(f.x) = words;
            return f;
        }

        // the fragment instruction `w` of a 16-byte piece takes: all of it (eight halves) or its word w (one float)
        template <typename Frag>
        ROCWMMA_DEVICE inline Frag pieceFragment(const u32x4_t& piece, uint32_t w)
        {
            Frag f;
            if constexpr(Frag::num_elements == 8u)
                *reinterpret_cast<u32x4_t*>(f.x) = piece;
            else
            {
                // (through a named scalar: __builtin_bit_cast applied to the element expression itself reads element 0)
                const uint32_t word = piece[w];
                f.x[0]              = __builtin_bit_cast(float, word);
            }
            return f;
        }

        // T = float16_t: 64 of K per stage, one v_mfma_f32_32x32x16_f16 per 16-byte piece and block; T = float: 32 of K
        // per stage, four v_mfma_f32_32x32x2_f32 per piece and block, one per word (the order in which K is contracted
        // is free as long as both multiplicands agree: instruction t of a piece contracts word t of both lane halves)
        template <typename T>
        __global__ void __launch_bounds__(256, sizeof(T) == 2u ? 4 : 3) // (waves per SIMD that fit without spills)
            dlrmFwdStagedKernel(const T* __restrict__ input, T* __restrict__ output, uint32_t m, uint32_t k, uint32_t batch, uint32_t tiles)
        {
            constexpr uint32_t KI = sizeof(T) == 2u ? 16u : 2u;
            using FragK           = fragment<matrix_a, 32, 32, KI, T, row_major>;
            using FragAcc         = fragment<accumulator, 32, 32, KI, float32_t>;
            using AccMap          = detail::AccMap<32, 32, 32>;
            constexpr uint32_t Size     = static_cast<uint32_t>(sizeof(T));
            constexpr uint32_t PerPiece = 16u / Size; // elements of a 16-byte piece
            constexpr uint32_t StageK   = 128u / Size; // a tile row of a stage is 128 bytes
            constexpr uint32_t InstrPerPiece = PerPiece / FragK::num_elements; // 1 or 4
            __shared__ __attribute__((aligned(16))) char lds[2u * kRowsBytes];
            char* const ldsA = lds;
            char* const ldsB = lds + kRowsBytes;

            uint32_t sample, t; // t: tiles of the lower triangle, row by row
            sampleAndTile(tiles, sample, t);
            if(sample >= batch) // (the whole workgroup)
                return;
            const uint32_t tid  = threadIdx.x;
            const uint32_t lane = tid & 63u;
            const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);

            uint32_t       I = static_cast<uint32_t>((__builtin_sqrtf(8.0f * static_cast<float>(t) + 1.0f) - 1.0f) * 0.5f);
            while(I * (I + 1u) / 2u > t)
                --I;
            while((I + 1u) * (I + 2u) / 2u <= t)
                ++I;
            const uint32_t J  = t - I * (I + 1u) / 2u;
            const uint32_t I0 = I * kTile, J0 = J * kTile;

            const size_t     width = packedRow(k, m);
            const T* feat = input + static_cast<size_t>(sample) * m * k;
            T*       out  = output + static_cast<size_t>(sample) * width;

            if(t == 0u) // bottom-MLP row: the sample's first feature row
                for(uint32_t e = tid; e < k; e += 256u)
                    out[e] = feat[e];

            const uint32_t wr = wave >> 1, wc = wave & 1u;
            const uint32_t R0 = I0 + wr * kWaveTile, C0 = J0 + wc * kWaveTile;
            // the wave's 64 x 64 holds entries below the diagonal and inside the matrix (every wave stages and meets
            // the barriers all the same)
            const bool waveLive = R0 < m && C0 < min(R0 + kWaveTile - 1u, m - 1u);

            // this thread's pieces of a stage: tile rows tid / 8 + 32 i, piece tid % 8 of the row's 128 bytes.  A row
            // from m on starts at the end of the sample, where a bounds-checked load returns zero.
            const lds::BufferRsrc rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(feat), 0, static_cast<int>(m * k * Size), 0x00020000);
            const uint32_t        pos  = tid & 7u;
            uint32_t              offA[4], offB[4], offLds[4];
#pragma unroll
            for(uint32_t i = 0; i < 4u; ++i)
            {
                const uint32_t r = (tid >> 3) + 32u * i;
                offA[i]          = (min(I0 + r, m) * k + pos * PerPiece) * Size;
                offB[i]          = (min(J0 + r, m) * k + pos * PerPiece) * Size;
                offLds[i]        = r * kRowPitch + pos * 16u;
            }
            u32x4_t ra[4], rb[4];
            auto    fetch = [&](uint32_t k0) {
                const bool inK = k0 + pos * PerPiece < k;
#pragma unroll
                for(uint32_t i = 0; i < 4u; ++i)
                {
                    ra[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(inK ? offA[i] + k0 * Size : kNowhere), 0, 0);
                    rb[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(inK ? offB[i] + k0 * Size : kNowhere), 0, 0);
                }
            };

            FragAcc acc[2][2];
#pragma unroll
            for(uint32_t i = 0; i < 2u; ++i)
#pragma unroll
                for(uint32_t j = 0; j < 2u; ++j)
                    fill_fragment(acc[i][j], 0.0f);

            fetch(0u);
#pragma unroll 1
            for(uint32_t k0 = 0; k0 < k; k0 += StageK)
            {
#pragma unroll
                for(uint32_t i = 0; i < 4u; ++i)
                {
                    *reinterpret_cast<u32x4_t*>(ldsA + offLds[i]) = ra[i];
                    *reinterpret_cast<u32x4_t*>(ldsB + offLds[i]) = rb[i];
                }
                __syncthreads();
                // the next stage's pieces fly while this one is multiplied (a stage from k on loads nothing)
                fetch(k0 + StageK);
                __builtin_amdgcn_sched_barrier(0);
                if(waveLive)
                {
#pragma unroll
                    for(uint32_t ks = 0; ks < 4u; ++ks) // a row's 128 bytes: 32 per step, 16 per lane half
                    {
                        u32x4_t pa[2], pb[2];
#pragma unroll
                        for(uint32_t i = 0; i < 2u; ++i)
                        {
                            pa[i] = rowsFragment(ldsA, wr * 2u + i, ks, lane);
                            pb[i] = rowsFragment(ldsB, wc * 2u + i, ks, lane);
                        }
#pragma unroll
                        for(uint32_t w = 0; w < InstrPerPiece; ++w)
                        {
                            FragK a[2], b[2];
#pragma unroll
                            for(uint32_t i = 0; i < 2u; ++i)
                            {
                                a[i] = pieceFragment<FragK>(pa[i], w);
                                b[i] = pieceFragment<FragK>(pb[i], w);
                            }
#pragma unroll
                            for(uint32_t i = 0; i < 2u; ++i)
#pragma unroll
                                for(uint32_t j = 0; j < 2u; ++j)
                                    mma_sync(acc[i][j], a[i], applyTranspose(b[j]), acc[i][j]);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
            }

            if(!waveLive)
                return;
            // strict lower triangle: block by block through LDS (the operand tiles are done with), then pieces of rows,
            // which are contiguous in the packed output
            T(*st)[33] = reinterpret_cast<T(*)[33]>(lds + wave * (32u * 33u * Size));
            const uint32_t row = lane & 31u, half = lane >> 5;
#pragma unroll
            for(uint32_t i = 0; i < 2u; ++i)
#pragma unroll
                for(uint32_t j = 0; j < 2u; ++j)
                {
                    if(C0 + j * 32u >= min(R0 + i * 32u + 31u, m - 1u)) // (wave uniform: nothing of the block is below the diagonal)
                        continue;
#pragma unroll
                    for(uint32_t e = 0; e < 16u; ++e)
                        st[AccMap::rowOf(e, lane)][AccMap::colOf(e, lane)] = static_cast<T>(acc[i][j].x[e]);
                    waveSync();
#pragma unroll 4
                    for(uint32_t rr = 0; rr < 16u; ++rr)
                    {
                        const uint32_t r = rr * 2u + half, Rg = R0 + i * 32u + r, Cg = C0 + j * 32u + row;
                        if(Rg < m && Cg < Rg)
                            out[packedRow(k, Rg) + Cg] = st[r][row];
                    }
                    waveSync();
                }
        }

        __global__ void __launch_bounds__(256, 3) dlrmBwdStagedF16Kernel(const float16_t* __restrict__ input,
                                                                         const float16_t* __restrict__ upstream,
                                                                         float16_t* __restrict__ grad,
                                                                         float16_t* __restrict__ mlpGrad,
                                                                         uint32_t m,
                                                                         uint32_t k,
                                                                         uint32_t batch,
                                                                         uint32_t colTiles)
        {
            using FragF  = fragment<matrix_b, 32, 32, 16, float16_t, row_major>;
            using AccMap = detail::AccMap<32, 32, 32>;

            __shared__ __attribute__((aligned(16))) char ldsS[kRowsBytes]; // "rows" or "columns" layout, by stage
            __shared__ __attribute__((aligned(16))) char ldsF[kColsBytes]; // "columns" layout

            uint32_t sample, t;
            sampleAndTile(((m + kTile - 1u) / kTile) * colTiles, sample, t);
            if(sample >= batch) // (the whole workgroup)
                return;
            const uint32_t tid  = threadIdx.x;
            const uint32_t lane = tid & 63u;
            const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
            const uint32_t I = t / colTiles, N = t % colTiles;
            const uint32_t I0 = I * kTile, N0 = N * kTile;

            const size_t     width = packedRow(k, m);
            const float16_t* feat  = input + static_cast<size_t>(sample) * m * k;
            const float16_t* up    = upstream + static_cast<size_t>(sample) * width;
            float16_t*       dst   = grad + static_cast<size_t>(sample) * m * k;

            if(t == 0u) // bottom-MLP gradient = the first k entries of the upstream row
                for(uint32_t e = tid; e < k; e += 256u)
                    mlpGrad[static_cast<size_t>(sample) * k + e] = up[e];

            const uint32_t wr = wave >> 1, wc = wave & 1u;
            const bool     waveLive = I0 + wr * kWaveTile < m && N0 + wc * kWaveTile < k; // (every wave stages and meets the barriers)

            // Where a stage of 64 contraction indices c0 .. lies against the tile's rows I0 .. I0 + 127 decides how S
            // arrives (workgroup uniform):
            //   Below:  c0 + 63 < I0: S(r, c) = up[packedRow(r) + c], 128 contiguous bytes per tile row -> "rows"
            //   Above:  c0 >= I0 + 128: S(r, c) = up[packedRow(c) + r], 256 contiguous bytes per contraction row
            //           -> "columns"
            //   Across: the stage meets the diagonal: element by element into "rows" (zero diagonal, both triangles)
            enum Where : uint32_t { Below, Above, Across };
            auto whereOf = [&](uint32_t c0) { return c0 + kStageK <= I0 ? Below : (c0 >= I0 + kTile ? Above : Across); };

            // this thread's pieces.  "rows": tile rows tid / 8 + 32 i, piece tid % 8; "columns": contraction rows
            // tid / 16 + 16 i, piece tid % 16.
            const lds::BufferRsrc rsrcF = __builtin_amdgcn_make_buffer_rsrc(const_cast<float16_t*>(feat), 0, static_cast<int>(m * k * 2u), 0x00020000);
            const uint32_t        posR = tid & 7u, posC = tid & 15u;
            const bool            colInK = N0 + posC * 8u < k;
            // (rows from m on are clamped to the last one: they only reach results that are never written)
            size_t belowStart[4]; // of the thread's tile rows in the packed triangle
#pragma unroll
            for(uint32_t i = 0; i < 4u; ++i)
                belowStart[i] = packedRow(k, min(I0 + (tid >> 3) + 32u * i, m - 1u));

            u32x4_t rs[4], rf[4];
            auto    fetch = [&](uint32_t c0) { // (c0 < m)
                const Where where = whereOf(c0);
#pragma unroll
                for(uint32_t i = 0; i < 4u; ++i)
                {
                    const uint32_t cr = (tid >> 4) + 16u * i; // contraction row of the stage ("columns" pieces)
                    rf[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrcF, static_cast<int>(colInK ? (min(c0 + cr, m) * k + N0 + posC * 8u) * 2u : kNowhere), 0, 0);
                    if(where == Below)
                        rs[i] = loadUnaligned(up + belowStart[i] + c0 + posR * 8u);
                    else if(where == Above) // (contraction rows from m on: clamped here, cleared before they reach LDS)
                        rs[i] = loadUnaligned(up + packedRow(k, min(c0 + cr, m - 1u)) + I0 + posC * 8u);
                }
            };

            FragAcc16 acc[2][2];
#pragma unroll
            for(uint32_t i = 0; i < 2u; ++i)
#pragma unroll
                for(uint32_t j = 0; j < 2u; ++j)
                    fill_fragment(acc[i][j], 0.0f);

            fetch(0u);
#pragma unroll 1
            for(uint32_t c0 = 0; c0 < m; c0 += kStageK)
            {
                const Where where = whereOf(c0);
#pragma unroll
                for(uint32_t i = 0; i < 4u; ++i)
                {
                    const uint32_t cr = (tid >> 4) + 16u * i;
                    *reinterpret_cast<u32x4_t*>(ldsF + columnsOffset(cr, posC)) = rf[i];
                    if(where == Below)
                        *reinterpret_cast<u32x4_t*>(ldsS + ((tid >> 3) + 32u * i) * kRowPitch + posR * 16u) = rs[i];
                    else if(where == Above)
                        *reinterpret_cast<u32x4_t*>(ldsS + columnsOffset(cr, posC)) = c0 + cr < m ? rs[i] : u32x4_t{0u, 0u, 0u, 0u};
                }
                if(where == Across)
                {
                    // consecutive threads along the contraction index (consecutive in the packed row below the diagonal)
#pragma unroll 4
                    for(uint32_t i = 0; i < 32u; ++i)
                    {
                        const uint32_t r  = (tid >> 6) + 4u * i, c = tid & 63u;
                        const uint32_t Rg = I0 + r, cg = c0 + c;
                        const uint32_t hi = Rg > cg ? Rg : cg, lo = Rg > cg ? cg : Rg;
                        float16_t      v  = static_cast<float16_t>(0);
                        if(hi < m && Rg != cg)
                            v = up[packedRow(k, hi) + lo];
                        *reinterpret_cast<float16_t*>(ldsS + r * kRowPitch + c * 2u) = v;
                    }
                }
                __syncthreads();
                // the next stage's pieces fly while this one is multiplied
                if(c0 + kStageK < m)
                    fetch(c0 + kStageK);
                __builtin_amdgcn_sched_barrier(0);
                if(waveLive)
                {
#pragma unroll
                    for(uint32_t ks = 0; ks < kStageK / 16u; ++ks)
                    {
                        FragK16 a[2];
                        FragF   b[2];
#pragma unroll
                        for(uint32_t j = 0; j < 2u; ++j)
                            b[j] = fragmentOf<FragF>(columnsFragment(ldsF, wc * 2u + j, ks, lane));
#pragma unroll
                        for(uint32_t i = 0; i < 2u; ++i)
                            a[i] = fragmentOf<FragK16>(where == Above ? columnsFragment(ldsS, wr * 2u + i, ks, lane)
                                                                      : rowsFragment(ldsS, wr * 2u + i, ks, lane));
#pragma unroll
                        for(uint32_t i = 0; i < 2u; ++i)
#pragma unroll
                            for(uint32_t j = 0; j < 2u; ++j)
                                mma_sync(acc[i][j], a[i], b[j], acc[i][j]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
            }

            if(!waveLive)
                return;
            // a lane owns runs of four consecutive columns of one row (k is a multiple of 8)
#pragma unroll
            for(uint32_t i = 0; i < 2u; ++i)
#pragma unroll
                for(uint32_t j = 0; j < 2u; ++j)
#pragma unroll
                    for(uint32_t r4 = 0; r4 < AccMap::runs; ++r4)
                    {
                        const uint32_t e0 = r4 * 4u;
                        const uint32_t r  = I0 + wr * kWaveTile + i * 32u + AccMap::rowOf(e0, lane);
                        const uint32_t c  = N0 + wc * kWaveTile + j * 32u + AccMap::colOf(e0, lane);
                        float16_t      h[4];
#pragma unroll
                        for(uint32_t e = 0; e < 4u; ++e)
                            h[e] = static_cast<float16_t>(acc[i][j].x[e0 + e]);
                        if(r < m && c < k)
                            *reinterpret_cast<u32x2_t*>(dst + static_cast<size_t>(r) * k + c) = *reinterpret_cast<u32x2_t*>(h);
                    }
        }

        // float32 backward through LDS.  32 contraction indices per stage; an instruction takes one float per lane,
        // so no transposing reads: "rows" as above (128 tile rows of 32 floats, 16-byte reads, instruction w of a
        // piece takes word w), "columns" = 32 contraction rows of 128 floats, row pitch 544 bytes (the two lane
        // halves of an instruction read rows four apart: 4 x 544 bytes puts them on different banks), 4-byte reads.
        constexpr uint32_t kStageK32   = 32;
        constexpr uint32_t kColPitch32 = 544;
        constexpr uint32_t kColsBytes32 = kStageK32 * kColPitch32; // 17408

        __global__ void __launch_bounds__(256, 3) dlrmBwdStagedF32Kernel(const float* __restrict__ input,
                                                                         const float* __restrict__ upstream,
                                                                         float* __restrict__ grad,
                                                                         float* __restrict__ mlpGrad,
                                                                         uint32_t m,
                                                                         uint32_t k,
                                                                         uint32_t batch,
                                                                         uint32_t colTiles)
        {
            using FragS   = fragment<matrix_a, 32, 32, 2, float32_t, row_major>;
            using FragF   = fragment<matrix_b, 32, 32, 2, float32_t, row_major>;
            using FragAcc = fragment<accumulator, 32, 32, 2, float32_t>;
            using AccMap  = detail::AccMap<32, 32, 32>;

            __shared__ __attribute__((aligned(16))) char ldsS[kRowsBytes]; // "rows" or "columns" layout, by stage
            __shared__ __attribute__((aligned(16))) char ldsF[kColsBytes32]; // "columns" layout

            uint32_t sample, t;
            sampleAndTile(((m + kTile - 1u) / kTile) * colTiles, sample, t);
            if(sample >= batch) // (the whole workgroup)
                return;
            const uint32_t tid  = threadIdx.x;
            const uint32_t lane = tid & 63u;
            const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
            const uint32_t I = t / colTiles, N = t % colTiles;
            const uint32_t I0 = I * kTile, N0 = N * kTile;

            const size_t width = packedRow(k, m);
            const float* feat  = input + static_cast<size_t>(sample) * m * k;
            const float* up    = upstream + static_cast<size_t>(sample) * width;
            float*       dst   = grad + static_cast<size_t>(sample) * m * k;

            if(t == 0u) // bottom-MLP gradient = the first k entries of the upstream row
                for(uint32_t e = tid; e < k; e += 256u)
                    mlpGrad[static_cast<size_t>(sample) * k + e] = up[e];

            const uint32_t wr = wave >> 1, wc = wave & 1u;
            const bool     waveLive = I0 + wr * kWaveTile < m && N0 + wc * kWaveTile < k; // (every wave stages and meets the barriers)

            // (as in the float16 kernel) where a stage lies against the tile's rows decides how S arrives
            enum Where : uint32_t { Below, Above, Across };
            auto whereOf = [&](uint32_t c0) { return c0 + kStageK32 <= I0 ? Below : (c0 >= I0 + kTile ? Above : Across); };

            // this thread's pieces.  "rows": tile rows tid / 8 + 32 i, piece tid % 8; "columns": contraction rows
            // tid / 32 + 8 i, piece tid % 32.
            const lds::BufferRsrc rsrcF = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(feat), 0, static_cast<int>(m * k * 4u), 0x00020000);
            const uint32_t        posR = tid & 7u, posC = tid & 31u;
            const bool            colInK = N0 + posC * 4u < k;
            size_t                belowStart[4];
#pragma unroll
            for(uint32_t i = 0; i < 4u; ++i)
                belowStart[i] = packedRow(k, min(I0 + (tid >> 3) + 32u * i, m - 1u));

            u32x4_t rs[4], rf[4];
            auto    fetch = [&](uint32_t c0) { // (c0 < m)
                const Where where = whereOf(c0);
#pragma unroll
                for(uint32_t i = 0; i < 4u; ++i)
                {
                    const uint32_t cr = (tid >> 5) + 8u * i;
                    rf[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrcF, static_cast<int>(colInK ? (min(c0 + cr, m) * k + N0 + posC * 4u) * 4u : kNowhere), 0, 0);
                    // (rows of the packed triangle start at any float: 4-byte aligned 16-byte loads)
                    if(where == Below)
                        rs[i] = *reinterpret_cast<const u32x4_t __attribute__((aligned(4)))*>(up + belowStart[i] + c0 + posR * 4u);
                    else if(where == Above)
                        rs[i] = *reinterpret_cast<const u32x4_t __attribute__((aligned(4)))*>(up + packedRow(k, min(c0 + cr, m - 1u)) + I0 + posC * 4u);
                }
            };

            FragAcc acc[2][2];
#pragma unroll
            for(uint32_t i = 0; i < 2u; ++i)
#pragma unroll
                for(uint32_t j = 0; j < 2u; ++j)
                    fill_fragment(acc[i][j], 0.0f);

            const uint32_t row = lane & 31u, half = lane >> 5;
            fetch(0u);
#pragma unroll 1
            for(uint32_t c0 = 0; c0 < m; c0 += kStageK32)
            {
                const Where where = whereOf(c0);
#pragma unroll
                for(uint32_t i = 0; i < 4u; ++i)
                {
                    const uint32_t cr = (tid >> 5) + 8u * i;
                    *reinterpret_cast<u32x4_t*>(ldsF + cr * kColPitch32 + posC * 16u) = rf[i];
                    if(where == Below)
                        *reinterpret_cast<u32x4_t*>(ldsS + ((tid >> 3) + 32u * i) * kRowPitch + posR * 16u) = rs[i];
                    else if(where == Above)
                        *reinterpret_cast<u32x4_t*>(ldsS + cr * kColPitch32 + posC * 16u) = c0 + cr < m ? rs[i] : u32x4_t{0u, 0u, 0u, 0u};
                }
                if(where == Across)
                {
#pragma unroll 4
                    for(uint32_t i = 0; i < 16u; ++i)
                    {
                        const uint32_t r  = (tid >> 5) + 8u * i, c = tid & 31u;
                        const uint32_t Rg = I0 + r, cg = c0 + c;
                        const uint32_t hi = Rg > cg ? Rg : cg, lo = Rg > cg ? cg : Rg;
                        float          v  = 0.0f;
                        if(hi < m && Rg != cg)
                            v = up[packedRow(k, hi) + lo];
                        *reinterpret_cast<float*>(ldsS + r * kRowPitch + c * 4u) = v;
                    }
                }
                __syncthreads();
                if(c0 + kStageK32 < m)
                    fetch(c0 + kStageK32);
                __builtin_amdgcn_sched_barrier(0);
                if(waveLive)
                {
                    // instruction (ks, w) contracts c = ks * 8 + half * 4 + w of the stage
#pragma unroll
                    for(uint32_t ks = 0; ks < 4u; ++ks)
                    {
                        u32x4_t sp[2];
                        if(where != Above)
                        {
#pragma unroll
                            for(uint32_t i = 0; i < 2u; ++i)
                                sp[i] = rowsFragment(ldsS, wr * 2u + i, ks, lane);
                        }
#pragma unroll
                        for(uint32_t w = 0; w < 4u; ++w)
                        {
                            const uint32_t cr = ks * 8u + half * 4u + w;
                            FragS          a[2];
                            FragF          b[2];
#pragma unroll
                            for(uint32_t j = 0; j < 2u; ++j)
                                b[j].x[0] = *reinterpret_cast<const float*>(ldsF + cr * kColPitch32 + ((wc * 2u + j) * 32u + row) * 4u);
                            if(where == Above)
                            {
#pragma unroll
                                for(uint32_t i = 0; i < 2u; ++i)
                                    a[i].x[0] = *reinterpret_cast<const float*>(ldsS + cr * kColPitch32 + ((wr * 2u + i) * 32u + row) * 4u);
                            }
                            else
                            {
#pragma unroll
                                for(uint32_t i = 0; i < 2u; ++i)
                                    a[i] = pieceFragment<FragS>(sp[i], w);
                            }
#pragma unroll
                            for(uint32_t i = 0; i < 2u; ++i)
#pragma unroll
                                for(uint32_t j = 0; j < 2u; ++j)
                                    mma_sync(acc[i][j], a[i], b[j], acc[i][j]);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
            }

            if(!waveLive)
                return;
            // a lane owns runs of four consecutive columns of one row (k is a multiple of 4)
#pragma unroll
            for(uint32_t i = 0; i < 2u; ++i)
#pragma unroll
                for(uint32_t j = 0; j < 2u; ++j)
#pragma unroll
                    for(uint32_t r4 = 0; r4 < AccMap::runs; ++r4)
                    {
                        const uint32_t e0 = r4 * 4u;
                        const uint32_t r  = I0 + wr * kWaveTile + i * 32u + AccMap::rowOf(e0, lane);
                        const uint32_t c  = N0 + wc * kWaveTile + j * 32u + AccMap::colOf(e0, lane);
                        if(r < m && c < k)
                            *reinterpret_cast<f32x4_t*>(dst + static_cast<size_t>(r) * k + c)
                                = f32x4_t{acc[i][j].x[e0], acc[i][j].x[e0 + 1u], acc[i][j].x[e0 + 2u], acc[i][j].x[e0 + 3u]};
                    }
        }

        // workgroups of a launch (see sampleAndTile), 0 if they do not fit a grid dimension
        inline uint32_t gridFor(uint32_t tiles, uint32_t batch)
        {
            const uint64_t workgroups = static_cast<uint64_t>((batch + kXcds - 1u) / kXcds) * kXcds * tiles;
            return workgroups <= 0x7FFFFFFFull ? static_cast<uint32_t>(workgroups) : 0u;
        }
    } // namespace

    // Shapes: 1 <= m <= 32768; k a multiple of 8 (f16) or 4 (f32), so that a row's 16-byte pieces are whole; a sample's
    // features below 2 GiB (32-bit byte offsets into a bounds-checked buffer).
    int launchDlrmFwdGeneral(int dtype, const void* input, void* output, uint32_t m, uint32_t k, uint32_t batch, hipStream_t stream)
    {
        const uint32_t size = dtype == ROCWMMA_AMD_F16 ? 2u : 4u;
        if(m > kMaxRows || k == 0u || k % (16u / size) != 0u || static_cast<uint64_t>(m) * k * size >= (1ull << 31))
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const uint32_t side = (m + kTile - 1u) / kTile, tiles = side * (side + 1u) / 2u;
        const uint32_t grid = gridFor(tiles, batch);
        if(grid == 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        if(dtype == ROCWMMA_AMD_F16)
            hipLaunchKernelGGL(dlrmFwdStagedKernel<float16_t>, dim3(grid), dim3(256), 0, stream, static_cast<const float16_t*>(input),
                               static_cast<float16_t*>(output), m, k, batch, tiles);
        else
            hipLaunchKernelGGL(dlrmFwdStagedKernel<float>, dim3(grid), dim3(256), 0, stream, static_cast<const float*>(input),
                               static_cast<float*>(output), m, k, batch, tiles);
        return launchStatus();
    }

    int launchDlrmBwdGeneral(int dtype, const void* input, const void* upstream, void* grad, void* mlpGrad, uint32_t m, uint32_t k,
                             uint32_t batch, hipStream_t stream)
    {
        const uint32_t size = dtype == ROCWMMA_AMD_F16 ? 2u : 4u;
        if(m > kMaxRows || k == 0u || k % (16u / size) != 0u || static_cast<uint64_t>(m) * k * size >= (1ull << 31))
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const uint32_t rowTiles = (m + kTile - 1u) / kTile, colTiles = (k + kTile - 1u) / kTile;
        if(static_cast<uint64_t>(rowTiles) * colTiles > 0x7FFFFFFFull)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const uint32_t grid = gridFor(rowTiles * colTiles, batch);
        if(grid == 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        if(dtype == ROCWMMA_AMD_F16)
            hipLaunchKernelGGL(dlrmBwdStagedF16Kernel, dim3(grid), dim3(256), 0, stream, static_cast<const float16_t*>(input),
                               static_cast<const float16_t*>(upstream), static_cast<float16_t*>(grad), static_cast<float16_t*>(mlpGrad), m,
                               k, batch, colTiles);
        else
            hipLaunchKernelGGL(dlrmBwdStagedF32Kernel, dim3(grid), dim3(256), 0, stream, static_cast<const float*>(input),
                               static_cast<const float*>(upstream), static_cast<float*>(grad), static_cast<float*>(mlpGrad), m, k, batch,
                               colTiles);
        return launchStatus();
    }
} // namespace rocwmma_amd
