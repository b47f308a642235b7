// DLRM dot interaction for the shapes the one-wave-per-sample kernels (dlrm.hip, dlrm_f32.hip) do not take:
// more than 128 feature rows, or a feature width other than 32 / 64 / 128 / 256.  The reference's tests run
// (m, k) = (1024, 1024) among others (test/dlrm/test/dlrm_test_params.hpp:51-68); semantics = dlrm_fwd_CPU /
// dlrm_bwd_CPU (test/reference_impl.hpp:83-179).
//
// A sample of that size is a matrix product of its own (1024 x 1024 x 1024), so a sample's work is cut into tiles
// of 128 x 128 over workgroups of four waves (2 x 2, 64 x 64 each, 32 x 32 blocks), one grid for the whole batch:
//
//   * forward: tile (I, J), J <= I, of Z = F F^T.  Both operands are rows of F with K contiguous, read straight
//     from global memory (a sample's F stays in the L2): a lane reads 64 contiguous bytes of its row per step
//     and feeds them to the instructions one 16-byte piece after the other -- the order in which K is contracted
//     is free as long as both multiplicands agree.  The strict lower triangle leaves through a 32 x 32 LDS block
//     per wave as row pieces, which are contiguous in the packed output.  No m x m scratch in global memory.
//   * backward: tile (I, N) of grad = S F, S = the symmetric matrix with zero diagonal whose strict lower triangle
//     is the packed upstream gradient, never materialised: float32 operands are single elements per lane and
//     instruction (v_mfma_f32_32x32x2_f32) and come straight from global memory; float16 goes through LDS per
//     32 contraction rows, S gathered element by element with the thread order that follows the memory order
//     (along the row below the diagonal, along the column above it), F as 16-byte pieces read back with the
//     transposing LDS load.
//
// Rows from m on and columns from k on are never read: their lanes multiply zeros.  These shapes are no benchmark
// configuration; the kernels are written for parity and reasonable speed, not tuned.
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
        constexpr uint32_t kMaxGridY   = 32768;
        constexpr uint32_t kMaxRows    = 32768; // m * (m - 1) stays below 2^32

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

        ROCWMMA_DEVICE inline uint32_t sampleOfBlock()
        {
            return blockIdx.z * gridDim.y + blockIdx.y;
        }

        // ------------------------------------------------------------------ forward
        template <typename T, uint32_t Pieces> // Pieces: 16-byte pieces of its row a lane reads per step
        __global__ void __launch_bounds__(256)
            dlrmFwdGeneralKernel(const T* __restrict__ input, T* __restrict__ output, uint32_t m, uint32_t k, uint32_t batch)
        {
            constexpr uint32_t KI = sizeof(T) == 2u ? 16u : 2u;
            using FragA           = fragment<matrix_a, 32, 32, KI, T, row_major>;
            using FragAcc         = fragment<accumulator, 32, 32, KI, float32_t>;
            using AccMap          = detail::AccMap<32, 32, 32>;
            constexpr uint32_t PerPiece      = 16u / sizeof(T); // elements of a 16-byte piece
            constexpr uint32_t InstrPerPiece = PerPiece / FragA::num_elements; // 1 (f16) or 4 (f32)
            constexpr uint32_t Chunk         = Pieces * PerPiece;
            constexpr uint32_t Step          = 2u * Chunk; // K per step: the two lane halves read neighbouring chunks
            static_assert(FragAcc::num_elements == 16u, "32 x 32 accumulator");

            __shared__ T stage[4][32][33];

            const uint32_t sample = sampleOfBlock();
            if(sample >= batch)
                return;
            const uint32_t lane = threadIdx.x & 63u;
            const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

            // blockIdx.x counts the tiles of the lower triangle row by row
            const uint32_t t = blockIdx.x;
            uint32_t       I = static_cast<uint32_t>((__builtin_sqrtf(8.0f * static_cast<float>(t) + 1.0f) - 1.0f) * 0.5f);
            while(I * (I + 1u) / 2u > t)
                --I;
            while((I + 1u) * (I + 2u) / 2u <= t)
                ++I;
            const uint32_t J = t - I * (I + 1u) / 2u;

            const size_t width = packedRow(k, m);
            const T*     feat  = input + static_cast<size_t>(sample) * m * k;
            T*           out   = output + static_cast<size_t>(sample) * width;

            if(t == 0u) // bottom-MLP row: the sample's first feature row
                for(uint32_t e = threadIdx.x; e < k; e += 256u)
                    out[e] = feat[e];

            const uint32_t R0 = I * kTile + (wave >> 1) * kWaveTile, C0 = J * kTile + (wave & 1u) * kWaveTile;
            // no entry of this wave's 64 x 64 below the diagonal and inside the matrix (nothing below is shared
            // between waves: no workgroup barrier)
            if(R0 >= m || C0 >= min(R0 + kWaveTile - 1u, m - 1u))
                return;
            // 32 x 32 block (rb, cb) holds such entries
            auto blockLive = [&](uint32_t rb, uint32_t cb) { return C0 + cb * 32u < min(R0 + rb * 32u + 31u, m - 1u); };

            const uint32_t row = lane & 31u, half = lane >> 5;
            // bounds-checked loads: a row from m on starts at the end of the sample, where every read returns zero;
            // so does the offset given to a piece from k on
            const lds::BufferRsrc rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(feat), 0, static_cast<int>(m * k * sizeof(T)), 0x00020000);
            constexpr uint32_t    kNowhere = 0x80000000u;
            uint32_t              offA[2], offB[2];
#pragma unroll
            for(uint32_t b = 0; b < 2u; ++b)
            {
                offA[b] = (min(R0 + b * 32u + row, m) * k + half * Chunk) * static_cast<uint32_t>(sizeof(T));
                offB[b] = (min(C0 + b * 32u + row, m) * k + half * Chunk) * static_cast<uint32_t>(sizeof(T));
            }

            struct Operands
            {
                u32x4_t a[2][Pieces], b[2][Pieces];
            };
            auto load = [&](Operands& o, uint32_t k0) {
#pragma unroll
                for(uint32_t q = 0; q < Pieces; ++q)
                {
                    const bool     inK = k0 + half * Chunk + q * PerPiece < k;
                    const uint32_t at  = (k0 + q * PerPiece) * static_cast<uint32_t>(sizeof(T));
#pragma unroll
                    for(uint32_t blk = 0; blk < 2u; ++blk)
                    {
                        o.a[blk][q] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(inK ? offA[blk] + at : kNowhere), 0, 0);
                        o.b[blk][q] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(inK ? offB[blk] + at : kNowhere), 0, 0);
                    }
                }
            };
            auto asFragment = [](const u32x4_t& piece, uint32_t i) {
                FragA f;
                if constexpr(sizeof(T) == 2u)
                    *reinterpret_cast<u32x4_t*>(f.x) = piece;
                else
                    {
                    // (through a named scalar: __builtin_bit_cast applied to the element expression itself reads element 0)
                    const uint32_t word = piece[i];
                    f.x[0]              = __builtin_bit_cast(float, word);
                }
                return f;
            };

            FragAcc acc[2][2];
#pragma unroll
            for(uint32_t rb = 0; rb < 2u; ++rb)
#pragma unroll
                for(uint32_t cb = 0; cb < 2u; ++cb)
                    fill_fragment(acc[rb][cb], 0.0f);
            // (block (0, 1) of a wave tile on the diagonal lies above it: multiplied all the same, never written)
            auto multiply = [&](const Operands& o) {
#pragma unroll
                for(uint32_t q = 0; q < Pieces; ++q)
#pragma unroll
                    for(uint32_t i = 0; i < InstrPerPiece; ++i)
                    {
                        const FragA a0 = asFragment(o.a[0][q], i), a1 = asFragment(o.a[1][q], i);
                        const FragA b0 = asFragment(o.b[0][q], i), b1 = asFragment(o.b[1][q], i);
                        mma_sync(acc[0][0], a0, applyTranspose(b0), acc[0][0]);
                        mma_sync(acc[0][1], a0, applyTranspose(b1), acc[0][1]);
                        mma_sync(acc[1][0], a1, applyTranspose(b0), acc[1][0]);
                        mma_sync(acc[1][1], a1, applyTranspose(b1), acc[1][1]);
                    }
            };

            // two operand sets in turn: the loads of one step fly while the other is multiplied (a step from k on
            // loads nothing and returns zeros)
            const uint32_t steps = (k + Step - 1u) / Step;
            Operands       o0, o1;
            load(o0, 0u);
            uint32_t s = 0;
#pragma unroll 1
            for(; s + 2u <= steps; s += 2u)
            {
                // (the fences keep the compiler from sinking a step's loads to just in front of their use)
                load(o1, (s + 1u) * Step);
                __builtin_amdgcn_sched_barrier(0);
                multiply(o0);
                __builtin_amdgcn_sched_barrier(0);
                load(o0, (s + 2u) * Step);
                __builtin_amdgcn_sched_barrier(0);
                multiply(o1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if(s < steps)
                multiply(o0);

            // strict lower triangle: block by block through LDS, then pieces of rows (contiguous in the packed output)
            T(*st)[33] = stage[wave];
#pragma unroll
            for(uint32_t rb = 0; rb < 2u; ++rb)
#pragma unroll
                for(uint32_t cb = 0; cb < 2u; ++cb)
                {
                    if(!blockLive(rb, cb))
                        continue;
#pragma unroll
                    for(uint32_t e = 0; e < 16u; ++e)
                        st[AccMap::rowOf(e, lane)][AccMap::colOf(e, lane)] = static_cast<T>(acc[rb][cb].x[e]);
                    waveSync();
#pragma unroll 4
                    for(uint32_t rr = 0; rr < 16u; ++rr)
                    {
                        const uint32_t r = rr * 2u + half, Rg = R0 + rb * 32u + r, Cg = C0 + cb * 32u + row;
                        if(Rg < m && Cg < Rg)
                            out[packedRow(k, Rg) + Cg] = st[r][row];
                    }
                    waveSync();
                }
        }

        // ------------------------------------------------------------------ backward, float32
        __global__ void __launch_bounds__(256) dlrmBwdGeneralF32Kernel(const float* __restrict__ input,
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
            static_assert(FragS::num_elements == 1u && FragF::num_elements == 1u, "one float per lane and instruction");
            constexpr uint32_t Pairs = 8u; // contraction pairs (instructions per block) between two rounds of loads

            const uint32_t sample = sampleOfBlock();
            if(sample >= batch)
                return;
            const uint32_t lane = threadIdx.x & 63u;
            const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            const uint32_t I = blockIdx.x / colTiles, N = blockIdx.x % colTiles;

            const size_t width = packedRow(k, m);
            const float* feat  = input + static_cast<size_t>(sample) * m * k;
            const float* up    = upstream + static_cast<size_t>(sample) * width;
            float*       dst   = grad + static_cast<size_t>(sample) * m * k;

            if(blockIdx.x == 0u) // bottom-MLP gradient = the first k entries of the upstream row
                for(uint32_t e = threadIdx.x; e < k; e += 256u)
                    mlpGrad[static_cast<size_t>(sample) * k + e] = up[e];

            const uint32_t R0 = I * kTile + (wave >> 1) * kWaveTile, N0 = N * kTile + (wave & 1u) * kWaveTile;
            if(R0 >= m || N0 >= k) // (no workgroup barrier below)
                return;

            const uint32_t row = lane & 31u, half = lane >> 5;
            uint32_t       Rg[2], col[2];
            size_t         below[2];
#pragma unroll
            for(uint32_t b = 0; b < 2u; ++b)
            {
                Rg[b]    = R0 + b * 32u + row;
                col[b]   = N0 + b * 32u + row;
                below[b] = packedRow(k, Rg[b]);
            }

            FragAcc acc[2][2];
#pragma unroll
            for(uint32_t rb = 0; rb < 2u; ++rb)
#pragma unroll
                for(uint32_t cb = 0; cb < 2u; ++cb)
                    fill_fragment(acc[rb][cb], 0.0f);

#pragma unroll 1
            for(uint32_t c0 = 0; c0 < m; c0 += 2u * Pairs)
            {
                // S(Rg, c) for the lane's rows and F(c, col) for its columns, c = c0 + 2 p + half: below the diagonal
                // S(Rg, c) sits at packedRow(Rg) + c, above it entry (c, Rg) sits at packedRow(c) + Rg
                float s[2][Pairs], f[2][Pairs];
#pragma unroll
                for(uint32_t p = 0; p < Pairs; ++p)
                {
                    const uint32_t c      = c0 + 2u * p + half;
                    const size_t   cStart = packedRow(k, c);
#pragma unroll
                    for(uint32_t b = 0; b < 2u; ++b)
                    {
                        const bool there = (c > Rg[b] ? c : Rg[b]) < m && c != Rg[b];
                        s[b][p]          = 0.0f;
                        if(there)
                            s[b][p] = up[c < Rg[b] ? below[b] + c : cStart + Rg[b]];
                        f[b][p] = 0.0f;
                        if(c < m && col[b] < k)
                            f[b][p] = feat[static_cast<size_t>(c) * k + col[b]];
                    }
                }
#pragma unroll
                for(uint32_t p = 0; p < Pairs; ++p)
#pragma unroll
                    for(uint32_t rb = 0; rb < 2u; ++rb)
#pragma unroll
                        for(uint32_t cb = 0; cb < 2u; ++cb)
                        {
                            FragS a;
                            FragF b;
                            a.x[0] = s[rb][p];
                            b.x[0] = f[cb][p];
                            mma_sync(acc[rb][cb], a, b, acc[rb][cb]);
                        }
            }

            // a lane owns runs of four consecutive columns of one row (k is a multiple of 4)
#pragma unroll
            for(uint32_t rb = 0; rb < 2u; ++rb)
#pragma unroll
                for(uint32_t cb = 0; cb < 2u; ++cb)
#pragma unroll
                    for(uint32_t r4 = 0; r4 < AccMap::runs; ++r4)
                    {
                        const uint32_t e0 = r4 * 4u;
                        const uint32_t r  = R0 + rb * 32u + AccMap::rowOf(e0, lane);
                        const uint32_t c  = N0 + cb * 32u + AccMap::colOf(e0, lane);
                        if(r < m && c < k)
                            *reinterpret_cast<f32x4_t*>(dst + static_cast<size_t>(r) * k + c)
                                = f32x4_t{acc[rb][cb].x[e0], acc[rb][cb].x[e0 + 1u], acc[rb][cb].x[e0 + 2u], acc[rb][cb].x[e0 + 3u]};
                    }
        }

        // ------------------------------------------------------------------ backward, float16
        // LDS per stage of 32 contraction rows: the S tile (128 rows of 32 halves, row pitch 40 halves so that a
        // lane's 16 bytes stay aligned and neighbouring rows spread over the banks) and the F tile (32 rows of
        // 128 halves; the 32-byte segments of a row XOR-ed with 2 * (row % 4), which spreads the 4 rows x 2 segments
        // of one transposing read over 8 bank groups).
        constexpr uint32_t kStageRows = 32;
        constexpr uint32_t kSPitch    = 40;
        constexpr uint32_t kFRowBytes = kTile * 2u;

        ROCWMMA_DEVICE inline uint32_t segmentSwizzle(uint32_t row)
        {
            return (row & 3u) << 1;
        }

        __global__ void __launch_bounds__(256) dlrmBwdGeneralF16Kernel(const float16_t* __restrict__ input,
                                                                          const float16_t* __restrict__ upstream,
                                                                          float16_t* __restrict__ grad,
                                                                          float16_t* __restrict__ mlpGrad,
                                                                          uint32_t m,
                                                                          uint32_t k,
                                                                          uint32_t batch,
                                                                          uint32_t colTiles)
        {
            using FragS   = fragment<matrix_a, 32, 32, 16, float16_t, row_major>;
            using FragF   = fragment<matrix_b, 32, 32, 16, float16_t, row_major>;
            using FragAcc = fragment<accumulator, 32, 32, 16, float32_t>;
            using AccMap  = detail::AccMap<32, 32, 32>;

            __shared__ __attribute__((aligned(16))) float16_t ldsS[kTile * kSPitch];
            __shared__ __attribute__((aligned(16))) char      ldsF[kStageRows * kFRowBytes];

            const uint32_t sample = sampleOfBlock();
            if(sample >= batch) // (the whole workgroup)
                return;
            const uint32_t tid  = threadIdx.x;
            const uint32_t lane = tid & 63u;
            const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
            const uint32_t I = blockIdx.x / colTiles, N = blockIdx.x % colTiles;
            const uint32_t I0 = I * kTile, N0 = N * kTile;

            const size_t     width = packedRow(k, m);
            const float16_t* feat  = input + static_cast<size_t>(sample) * m * k;
            const float16_t* up    = upstream + static_cast<size_t>(sample) * width;
            float16_t*       dst   = grad + static_cast<size_t>(sample) * m * k;

            if(blockIdx.x == 0u)
                for(uint32_t e = tid; e < k; e += 256u)
                    mlpGrad[static_cast<size_t>(sample) * k + e] = up[e];

            const uint32_t wr = wave >> 1, wc = wave & 1u;
            const bool     waveLive = I0 + wr * kWaveTile < m && N0 + wc * kWaveTile < k; // (every wave stages and meets the barriers)
            const uint32_t row = lane & 31u, half = lane >> 5, group = lane >> 4, s16 = lane & 15u;
            const uint32_t ldsFBase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds::LdsPtr)ldsF));

            FragAcc acc[2][2];
#pragma unroll
            for(uint32_t rb = 0; rb < 2u; ++rb)
#pragma unroll
                for(uint32_t cb = 0; cb < 2u; ++cb)
                    fill_fragment(acc[rb][cb], 0.0f);

#pragma unroll 1
            for(uint32_t c0 = 0; c0 < m; c0 += kStageRows)
            {
                // S tile: rows I0 .., contraction c0 ..; consecutive threads along the contraction index where the
                // tile reaches below the diagonal (consecutive in the packed row), along the row where it lies above
                const bool above = c0 >= I0 + kTile; // (workgroup uniform)
#pragma unroll 4
                for(uint32_t i = 0; i < 16u; ++i)
                {
                    const uint32_t r  = above ? (tid & 127u) : (tid >> 5) + 8u * i;
                    const uint32_t c  = above ? (tid >> 7) + 2u * i : (tid & 31u);
                    const uint32_t Rg = I0 + r, cg = c0 + c;
                    const uint32_t hi = Rg > cg ? Rg : cg, lo = Rg > cg ? cg : Rg;
                    float16_t      v  = static_cast<float16_t>(0);
                    if(hi < m && Rg != cg)
                        v = up[packedRow(k, hi) + lo];
                    ldsS[r * kSPitch + c] = v;
                }
                // F tile: contraction rows c0 .., columns N0 ..: 32 rows of 16 pieces of 16 bytes
#pragma unroll
                for(uint32_t i = 0; i < 2u; ++i)
                {
                    const uint32_t q = tid + 256u * i, fr = q >> 4, pos = q & 15u;
                    const uint32_t cg = c0 + fr, cn = N0 + pos * 8u;
                    u32x4_t        v  = u32x4_t{0u, 0u, 0u, 0u};
                    if(cg < m && cn < k)
                        v = *reinterpret_cast<const u32x4_t*>(feat + static_cast<size_t>(cg) * k + cn);
                    *reinterpret_cast<u32x4_t*>(ldsF + fr * kFRowBytes + ((((pos >> 1) ^ segmentSwizzle(fr)) << 5) | ((pos & 1u) << 4))) = v;
                }
                __syncthreads();
                if(waveLive)
                {
#pragma unroll
                    for(uint32_t ks = 0; ks < 2u; ++ks)
                    {
                        FragS a[2];
#pragma unroll
                        for(uint32_t rb = 0; rb < 2u; ++rb)
                            *reinterpret_cast<u32x4_t*>(a[rb].x) = *reinterpret_cast<const u32x4_t*>(
                                ldsS + (wr * kWaveTile + rb * 32u + row) * kSPitch + ks * 16u + half * 8u);
                        // F operands: lane l gets column (wc * 2 + cb) * 32 + l % 32 and contraction rows
                        // ks * 16 + (l / 32) * 8 + 0..7 of the stage
                        uint32_t ff[2][4];
#pragma unroll
                        for(uint32_t cb = 0; cb < 2u; ++cb)
#pragma unroll
                            for(uint32_t kk = 0; kk < 2u; ++kk)
                            {
                                const uint32_t fr   = ks * 16u + (group >> 1) * 8u + kk * 4u + (s16 >> 2);
                                const uint32_t seg  = (wc * 2u + cb) * 2u + (group & 1u);
                                const uint32_t addr = ldsFBase + fr * kFRowBytes + ((seg ^ segmentSwizzle(fr)) << 5) + ((s16 & 3u) << 3);
                                u32x2_t        v;
                                asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(addr) : "memory");
                                ff[cb][2u * kk]      = v[0];
                                ff[cb][2u * kk + 1u] = v[1];
                            }
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        FragF b[2];
#pragma unroll
                        for(uint32_t cb = 0; cb < 2u; ++cb)
#pragma unroll
                            for(uint32_t w = 0; w < 4u; ++w)
                            {
                                asm volatile("" : "+v"(ff[cb][w]));
                                reinterpret_cast<uint32_t*>(b[cb].x)[w] = ff[cb][w];
                            }
#pragma unroll
                        for(uint32_t rb = 0; rb < 2u; ++rb)
#pragma unroll
                            for(uint32_t cb = 0; cb < 2u; ++cb)
                                mma_sync(acc[rb][cb], a[rb], b[cb], acc[rb][cb]);
                    }
                }
                __syncthreads();
            }

            if(!waveLive)
                return;
            // a lane owns runs of four consecutive columns of one row (k is a multiple of 8)
#pragma unroll
            for(uint32_t rb = 0; rb < 2u; ++rb)
#pragma unroll
                for(uint32_t cb = 0; cb < 2u; ++cb)
#pragma unroll
                    for(uint32_t r4 = 0; r4 < AccMap::runs; ++r4)
                    {
                        const uint32_t e0 = r4 * 4u;
                        const uint32_t r  = I0 + wr * kWaveTile + rb * 32u + AccMap::rowOf(e0, lane);
                        const uint32_t c  = N0 + wc * kWaveTile + cb * 32u + AccMap::colOf(e0, lane);
                        float16_t      h[4];
#pragma unroll
                        for(uint32_t j = 0; j < 4u; ++j)
                            h[j] = static_cast<float16_t>(acc[rb][cb].x[e0 + j]);
                        if(r < m && c < k)
                            *reinterpret_cast<u32x2_t*>(dst + static_cast<size_t>(r) * k + c) = *reinterpret_cast<u32x2_t*>(h);
                    }
        }

        constexpr uint32_t kFwdPieces = 2;

        inline dim3 gridFor(uint32_t tiles, uint32_t batch)
        {
            const uint32_t y = batch < kMaxGridY ? batch : kMaxGridY;
            return dim3(tiles, y, (batch + y - 1u) / y);
        }
    } // namespace

    // Shapes: 1 <= m <= 32768; k a multiple of 8 (f16) or 4 (f32), so that a row's 16-byte pieces are whole.
    int launchDlrmFwdGeneral(int dtype, const void* input, void* output, uint32_t m, uint32_t k, uint32_t batch, hipStream_t stream)
    {
        const uint32_t perPiece = dtype == ROCWMMA_AMD_F16 ? 8u : 4u;
        if(m > kMaxRows || k == 0u || k % perPiece != 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const uint32_t side = (m + kTile - 1u) / kTile;
        const dim3     grid = gridFor(side * (side + 1u) / 2u, batch);
        if(dtype == ROCWMMA_AMD_F16)
            hipLaunchKernelGGL((dlrmFwdGeneralKernel<float16_t, kFwdPieces>), grid, dim3(256), 0, stream, static_cast<const float16_t*>(input),
                               static_cast<float16_t*>(output), m, k, batch);
        else
            hipLaunchKernelGGL((dlrmFwdGeneralKernel<float, kFwdPieces>), grid, dim3(256), 0, stream, static_cast<const float*>(input),
                               static_cast<float*>(output), m, k, batch);
        return launchStatus();
    }

    int launchDlrmBwdGeneral(int dtype, const void* input, const void* upstream, void* grad, void* mlpGrad, uint32_t m, uint32_t k,
                             uint32_t batch, hipStream_t stream)
    {
        const uint32_t perPiece = dtype == ROCWMMA_AMD_F16 ? 8u : 4u;
        if(m > kMaxRows || k == 0u || k % perPiece != 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const uint32_t rowTiles = (m + kTile - 1u) / kTile, colTiles = (k + kTile - 1u) / kTile;
        if(static_cast<uint64_t>(rowTiles) * colTiles > 0x7FFFFFFFull)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const dim3 grid = gridFor(rowTiles * colTiles, batch);
        if(dtype == ROCWMMA_AMD_F16)
            hipLaunchKernelGGL(dlrmBwdGeneralF16Kernel, grid, dim3(256), 0, stream, static_cast<const float16_t*>(input),
                               static_cast<const float16_t*>(upstream), static_cast<float16_t*>(grad), static_cast<float16_t*>(mlpGrad), m,
                               k, batch, colTiles);
        else
            hipLaunchKernelGGL(dlrmBwdGeneralF32Kernel, grid, dim3(256), 0, stream, static_cast<const float*>(input),
                               static_cast<const float*>(upstream), static_cast<float*>(grad), static_cast<float*>(mlpGrad), m, k, batch,
                               colTiles);
        return launchStatus();
    }
} // namespace rocwmma_amd
