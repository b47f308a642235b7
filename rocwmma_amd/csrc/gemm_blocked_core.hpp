// Blocked GEMM for gfx950, device side: D = alpha * A * B + beta * C, C/D row-major.  Shared by the
// one-tile-per-workgroup kernel (gemm_blocked.hip) and the persistent stream-K kernel
// (gemm_streamk.hip).
//
// The workload of the reference's perf_hgemm sample (gemm_rocwmma_d,
// samples/perf_hgemm.cpp:518-714: macro tile per workgroup, wave tile of MFMA blocks per wave,
// two LDS buffers, next K slab prefetched while the current one is multiplied), re-tiled and
// re-plumbed for CDNA4:
//
//   reference (gfx9 params)                      this kernel (256 x 256 configuration)
//   macro tile 128 x 128 x 16, 4 waves           256 x 256 x (128 bytes of K) x ring of two LDS stages, 8 waves
//                                                (two per SIMD: one keeps the matrix pipe fed while the
//                                                other issues the stage's copies or waits at the barrier)
//   wave tile 2 x 2 blocks of 32x32x16 (2 MFMA)  4 x 8 blocks of 16x16, wide-K MFMAs (16x16x32 f16 / bf16,
//                                                16x16x64 int8, 16x16x128 fp8), 64 per wave and stage
//   global -> VGPR -> shuffle -> LDS             global -> LDS directly (buffer_load_dwordx4 ... lds), issued by
//                                                the first wave of each SIMD for itself and its partner
//   LDS -> VGPR -> shuffle (AOS<->SOA)           swizzled ds_read_b128, or ds_read_b64_tr_b16 / _b8
//                                                for operands whose K is not contiguous
//   2 LDS buffers, wait + barrier per step       copies one stage ahead, one barrier per 128-byte stage
//   8 MFMA between barriers                      64 MFMA (1024 clocks of matrix-pipe work) per wave between barriers
//   C read / D written in fragment layout       C staged through LDS (full-row non-temporal
//                                                copies), D written in fragment layout
//   grid (m/128, n/128)                          1-D grid, tiles dealt to XCDs in L2-friendly patches
//                                                (9 % faster than the plain order at 8192^3)
//
// The smaller configurations (128 x 128, 128 x 64, 64 x 64 tiles of 4 waves) come with a ring of four stages
// of 64 bytes of K (copies three stages ahead), a ring of four stages of 128 bytes, or the ring of two.
//
// Column-major C/D is handled by the caller as the transposed problem (D^T = B^T A^T).
#ifndef ROCWMMA_AMD_CSRC_GEMM_BLOCKED_CORE_HPP
#define ROCWMMA_AMD_CSRC_GEMM_BLOCKED_CORE_HPP

#include "common.hpp"
#include <rocwmma/rocwmma_lds.hpp>

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        constexpr uint32_t kXcds = 8; // MI355X: 8 accelerator complex dies, one L2 each

        template <typename InT_,
                  typename OutT_,
                  typename CompT_,
                  bool     AKMajor_, // A row-major  (K contiguous)
                  bool     BKMajor_, // B col-major  (K contiguous)
                  uint32_t WavesM_,
                  uint32_t WavesN_,
                  uint32_t BlocksM_,
                  uint32_t BlocksN_,
                  uint32_t Stages_       = 4u, // LDS ring depth
                  uint32_t WavesPerSimd_ = 1u, // waves per SIMD: sizes the register budget, and no more become resident
                  uint32_t BlockEdge_    = 32u, // MFMA block edge: 32 (32x32xK) or 16 (16x16x2K)
                  bool     Edges_        = false, // M and N need not fill whole macro tiles (multiples of 16 do)
                  bool     Scaled_       = false, // fp8 operands with one E8M0 scale per 32 elements of K (MX)
                  bool     Fused_        = false, // epilogue adds a per-column bias and applies an activation
                  uint32_t StageKB_      = 0u> // bytes of K per stage (0: 128 in the ring of two, else 64)
        struct BlockedConfig
        {
            using InT   = InT_;
            using OutT  = OutT_;
            using CompT = CompT_;

            static constexpr bool     AKMajor = AKMajor_;
            static constexpr bool     BKMajor = BKMajor_;
            // Partly filled tiles at the lower and right edges of C/D: operand reads past a matrix end
            // are cut off by the buffer bounds (rows and columns beyond the problem only ever meet
            // results beyond it), C reads and D stores are masked lane by lane.
            static constexpr bool     Edges   = Edges_;
            // Block-scaled operands: the scaled instruction's K order decides which bytes a lane holds
            // (two runs of 16 from the two halves of the stage, see rocwmma/internal/fragment_map.hpp),
            // so the fragments are read like two steps of a 16-bytes-per-lane operand.
            static constexpr bool     Scaled  = Scaled_;
            // D = act(alpha * A * B + beta * C + bias[column]): see FusedEpilogue
            static constexpr bool     Fused   = Fused_;
            static constexpr uint32_t WavesM  = WavesM_;
            static constexpr uint32_t WavesN  = WavesN_;
            static constexpr uint32_t BlocksM = BlocksM_;
            static constexpr uint32_t BlocksN = BlocksN_;
            static constexpr uint32_t Waves   = WavesM * WavesN;
            static constexpr uint32_t Threads = Waves * 64u;
            static constexpr uint32_t Block   = BlockEdge_; // MFMA edge
            static constexpr uint32_t WaveM   = BlocksM * Block;
            static constexpr uint32_t WaveN   = BlocksN * Block;
            static constexpr uint32_t MacroM  = WavesM * WaveM;
            static constexpr uint32_t MacroN  = WavesN * WaveN;
            // bytes of K per pipeline stage: 64 in the ring of four, 128 (whole lines of a K-contiguous
            // operand) in the ring of two
            static constexpr uint32_t StageKB = StageKB_ != 0u ? StageKB_ : (Stages_ == 2u ? 128u : 64u);
            static constexpr uint32_t MacroK  = StageKB / sizeof(InT); // K elements per stage

            // Fragments of one MFMA step.  BlockK = K of the widest single instruction.
            static constexpr uint32_t KPack      = detail::maxKPack(detail::packClassOf<InT>());
            static constexpr uint32_t BlockK     = KPack * (64u / Block); // 2 (32-wide) or 4 (16-wide) lane groups along K
            static constexpr uint32_t KPackBytes = KPack * sizeof(InT);
            static constexpr uint32_t KSteps     = MacroK / BlockK; // MFMA steps per stage (1 or 2)

            using FragA   = fragment<matrix_a, Block, Block, BlockK, InT, row_major>;
            using FragB   = fragment<matrix_b, Block, Block, BlockK, InT, col_major>;
            using FragAcc = fragment<accumulator, Block, Block, BlockK, CompT>;
            using FragC   = fragment<accumulator, Block, Block, BlockK, OutT, row_major>;

            // (a dim-major tile holds one K index per LDS row: StageKB / sizeof(InT) rows)
            template <uint32_t Dim>
            using DimTile = std::conditional_t<sizeof(InT) == 2u, lds::DimMajorTile<Dim, StageKB / 2u>,
                                               lds::DimMajorTile8<(Dim == 128u || Dim == 256u) ? Dim : 128u, StageKB>>;
            // (16-wide blocks with 32 bytes of K per lane, fp8 16x16x128: the K-major tile's pair reader)
            static constexpr bool PairReads = Block == 16u && KPackBytes == 32u && !Scaled;
            using TileA = std::conditional_t<AKMajor, lds::KMajorTile<MacroM, StageKB, PairReads>, DimTile<MacroM>>;
            using TileB = std::conditional_t<BKMajor, lds::KMajorTile<MacroN, StageKB, PairReads>, DimTile<MacroN>>;

            static constexpr uint32_t BytesA     = MacroM * StageKB;
            static constexpr uint32_t BytesB     = MacroN * StageKB;
            static constexpr uint32_t StageBytes = BytesA + BytesB;
            static constexpr uint32_t Stages     = Stages_; // ring of K stages in LDS
            static constexpr uint32_t WavesPerSimd = WavesPerSimd_;
            static constexpr uint32_t LdsBytes   = Stages * StageBytes;
            static constexpr uint32_t CopiesA    = BytesA / 1024u / Waves; // direct copies per wave per stage
            static constexpr uint32_t CopiesB    = BytesB / 1024u / Waves;
            static constexpr uint32_t Copies     = CopiesA + CopiesB;
            // With two waves per SIMD only the first wave of each SIMD issues the copies of the main loop, for
            // itself and for its partner (wave + CopyWaves).  A copy holds its wave's instruction issue for a
            // dozen cycles; when both waves of a SIMD issue theirs at the same point of the same phase
            // nothing feeds the matrix pipe meanwhile, with one issuer the partner's MFMAs fill that time
            // (8192^3, A row-major / B col-major: f16 0.845 -> 0.798 ms, bf16 0.821 -> 0.765; both row-major
            // 0.906 -> 0.884, both col-major 0.883 -> 0.853; with the second wave of each SIMD as the issuer
            // 1-5 % slower than that).  A col-major / B row-major (neither K-contiguous: every fragment comes
            // from transposing reads) is left as it was: 5 % slower with one issuer.  So are the kernels with
            // block scales: their main loop loads scales into registers, and behind a branch that only some
            // waves take the compiler waits for every copy in flight before it uses them (five times slower).
            static constexpr uint32_t CopyWaves
                = (Waves == 8u && WavesPerSimd_ == 2u && Stages_ == 2u && (AKMajor || BKMajor) && !Scaled_) ? 4u : Waves;
            // LDS read instructions per MFMA step: b128 reads per block (K-major) or two transposing b64 reads
            static constexpr uint32_t TrReads      = KPackBytes / 8u; // transposing 8-byte reads per operand
            static constexpr uint32_t ReadsA       = BlocksM * (AKMajor ? KPackBytes / 16u : TrReads);
            static constexpr uint32_t ReadsB       = BlocksN * (BKMajor ? KPackBytes / 16u : TrReads);
            static constexpr uint32_t ReadsPerStep = ReadsA + ReadsB;
            static constexpr uint32_t MfmasPerStep = BlocksM * BlocksN;
            // beta * C operand staged through LDS in the epilogue, in groups of Block rows by
            // GroupBlocks blocks (256- or 512-byte rows), two group buffers per wave
            static constexpr uint32_t GroupBlocks
                = (WaveN == 128u && 2u * Block * 128u * sizeof(OutT) * Waves <= LdsBytes) ? 128u / Block : 64u / Block;
            static constexpr bool StagedC = !Edges && sizeof(OutT) == 4u && WaveN % 64u == 0u
                                            && BlocksM * (BlocksN / GroupBlocks) >= 2u
                                            && 2u * Block * GroupBlocks * Block * sizeof(OutT) * Waves <= LdsBytes;

            static_assert(Block == 32u || Block == 16u, "MFMA blocks are 32 or 16 wide");
            static_assert(!Scaled
                              || (KPackBytes == 32u && AKMajor && BKMajor && (Block == 32u || !Edges_)
                                  && (Stages_ == 2u || (Stages_ == 4u && StageKB == 128u && Block == 32u))),
                          "block scales: fp8 on K-contiguous operands in the ring of two (16x16x128 on whole tiles, or 32x32x64), "
                          "or 32x32x64 in the ring of four 128-byte stages");
            static_assert(Block == 32u || KPackBytes == 16u || ((PairReads || Scaled) && AKMajor && BKMajor && Stages_ == 2u),
                          "16-wide blocks: 16 bytes of K per lane (16-bit types, int8), or fp8 16x16x128 on K-contiguous "
                          "operands in the ring of two");
            static_assert(sizeof(InT) == 2u || sizeof(InT) == 1u, "16-bit and 8-bit operands");
            static_assert(sizeof(InT) == 2u || ((AKMajor || MacroM == 128u || MacroM == 256u) && (BKMajor || MacroN == 128u || MacroN == 256u)),
                          "dim-major tiles of 8-bit operands are 128 or 256 wide");
            static_assert(TileA::bytes == BytesA && TileB::bytes == BytesB, "stage geometry mismatch");
            static_assert(BytesA % (1024u * Waves) == 0u && BytesB % (1024u * Waves) == 0u,
                          "a stage must split into whole-wave copies evenly");
            static_assert((Stages - 1u) * Copies < 64u, "too many copies in flight for vmcnt");
            static_assert(Stages != 2u || KSteps == 2u || KSteps == 4u || (KSteps == 1u && BlocksN % 2u == 0u),
                          "the ring of two runs one (fragments streamed by columns), two or four MFMA steps per stage");
            static_assert(LdsBytes <= Constants::AMDGCN_LDS_MAX_SIZE_BYTES, "macro tile does not fit the LDS");
            // the dim-major tile's swizzle looks at K row bits 0..3: a wave's copies must all start
            // on the same K row modulo 16
            // (the 8-bit tile's looks at K row bit 4 as well)
            static_assert((AKMajor || (Waves * TileA::rowsPerCopy) % (sizeof(InT) == 2u ? 16u : 32u) == 0u)
                              && (BKMajor || (Waves * TileB::rowsPerCopy) % (sizeof(InT) == 2u ? 16u : 32u) == 0u),
                          "wave pool too small for the dim-major tile");
            // the K-major tile's swizzle looks at row bits 0..3 likewise
            static_assert((!AKMajor || (Waves * TileA::rowsPerCopy) % 16u == 0u)
                              && (!BKMajor || (Waves * TileB::rowsPerCopy) % 16u == 0u),
                          "wave pool too small for the K-major tile");
        };

        // Deals the 1-D grid to tiles so that the workgroups resident on one XCD (ids congruent
        // mod 8 land on the same XCD) form a compact patch of the tile grid and share A / B
        // panels through that XCD's L2.
        ROCWMMA_DEVICE inline void tileOfWorkgroup(uint32_t wg, uint32_t tilesM, uint32_t tilesN, uint32_t& tm, uint32_t& tn)
        {
            const uint32_t total = tilesM * tilesN;
            uint32_t       id    = wg;
            if(total % kXcds == 0u)
                id = (wg % kXcds) * (total / kXcds) + wg / kXcds;
            // panels of 4 tile rows, walked column by column: the 32 workgroups an XCD runs at a
            // time cover 4 x 8 tiles (measured: 1 % faster than 8 x 4, 5 % faster than 16 x 2)
            constexpr uint32_t panel    = 4u;
            const uint32_t     perPanel = panel * tilesN;
            const uint32_t     panelIdx = id / perPanel;
            const uint32_t     firstRow = panelIdx * panel;
            const uint32_t     rowsHere = (tilesM - firstRow) < panel ? (tilesM - firstRow) : panel;
            const uint32_t     inPanel  = id - panelIdx * perPanel;
            tm                          = firstRow + inPanel % rowsHere;
            tn                          = inPanel / rowsHere;
        }

        // Scheduling hint: within the current scheduling region, issue `Mfmas` matrix instructions
        // with `Reads` LDS reads and `Copies` global -> LDS copies spread evenly between them.
        template <uint32_t Mfmas, uint32_t Reads, uint32_t Copies>
        ROCWMMA_DEVICE ROCWMMA_INLINE void scheduleInterleaved()
        {
            constexpr uint32_t Div = Mfmas > 0u ? Mfmas : 1u; // (an empty group: the loop does not run)
#pragma unroll
            for(uint32_t j = 0; j < Mfmas; ++j)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // 1 MFMA
                const uint32_t r = ((j + 1u) * Reads) / Div - (j * Reads) / Div;
                const uint32_t c = ((j + 1u) * Copies) / Div - (j * Copies) / Div;
                if(r == 1u)
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // DS read
                else if(r == 2u)
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                else if(r > 2u)
                    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
                if(c == 1u)
                    __builtin_amdgcn_sched_group_barrier(0x010, 1, 0); // VMEM
                else if(c >= 2u)
                    __builtin_amdgcn_sched_group_barrier(0x010, 2, 0);
            }
        }


        // Compile-time loop: f(std::integral_constant<uint32_t, 0>{}), ..., f(<N - 1>) -- for bodies whose
        // iteration index must be a constant expression (instruction immediates).
        template <typename F, uint32_t... I>
        ROCWMMA_DEVICE ROCWMMA_INLINE void staticForImpl(F&& f, std::integer_sequence<uint32_t, I...>)
        {
            (f(std::integral_constant<uint32_t, I>{}), ...);
        }
        template <uint32_t N, typename F>
        ROCWMMA_DEVICE ROCWMMA_INLINE void staticFor(F&& f)
        {
            staticForImpl(f, std::make_integer_sequence<uint32_t, N>{});
        }

        // Block scales of a Scaled configuration, in the order the lanes load them (written by the
        // re-ordering kernel in gemm_mx.hip): per operand, group of 64 rows of A (columns of B) and pair
        // of K stages, 8 bytes per lane = [block of 16 rows 0..3][stage of the pair 0..1]; lane l's bytes
        // are the scales of row l % 16 of each block and K block l / 16 of each stage.
        struct MxPacked
        {
            const void* a;
            const void* b;
            uint32_t    pairs; // pairs of stages along K (the last one padded when the stage count is odd)
        };

        // What a Fused configuration's epilogue does beyond alpha * acc + beta * C.
        struct FusedEpilogue
        {
            const float* bias; // one value per column of D (n floats), or nullptr
            int          activation; // rocwmma_amd_activation
        };

        // Per-launch arguments beyond the GEMM's own, for the configurations that use them.
        struct TileExtras
        {
            MxPacked      mx;
            FusedEpilogue fused;
        };

        // ---- stream-K support ------------------------------------------------------------------
        // Which part of a tile's K range a call of gemmTile computes.
        enum class TilePart
        {
            Whole, // all of K: the result goes through the epilogue
            Contributor, // a part that does not start at K = 0: the raw accumulators go to a workspace slot
            Owner // the part that starts at K = 0 of a tile other workgroups contribute to
        };

        // Workspace of the stream-K kernel: one slot of raw accumulators (MacroM x MacroN x 4 bytes, in
        // register order) and one flag per workgroup, then one word that records a wait that ran out
        // (kStreamKTimedOut; never cleared by a launch, only by the query that reports it) and the ticket
        // counter the workgroups of a launch draw their ranges from.
        constexpr uint32_t kStreamKTimedOut = 0x54494D45u; // "TIME": a value, not a bit, so that an uninitialised workspace does not read as a time-out
        struct StreamKPart
        {
            char*     slots; // slot i at slots + i * slotBytes
            uint32_t* flags; // flag i set to 1 once slot i is complete; [workgroups] = time-out marker, [workgroups + 1] = tickets
            uint32_t  slotBytes;
            uint32_t  mySlot; // contributor: where the accumulators go
            uint32_t  firstSlot, slotCount; // owner: the slots to add, in this order
            uint32_t  timeoutWord; // index of the time-out marker in flags
        };

        // Returns true when the caller is done with the tile (contributor).
        template <typename Cfg, TilePart Part, typename Acc>
        ROCWMMA_DEVICE ROCWMMA_INLINE bool streamKHandOver(Acc (&acc)[Cfg::BlocksM][Cfg::BlocksN], StreamKPart const& sk)
        {
            typedef uint32_t Words __attribute__((ext_vector_type(4)));
            constexpr uint32_t PerBlock = sizeof(acc[0][0].x) / 16u; // 16-byte pieces per accumulator block
            if constexpr(Part == TilePart::Contributor)
            {
                Words* slot = reinterpret_cast<Words*>(sk.slots + static_cast<size_t>(sk.mySlot) * sk.slotBytes);
#pragma unroll
                for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
#pragma unroll
                    for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
#pragma unroll
                        for(uint32_t p = 0; p < PerBlock; ++p)
                        {
                            Words v;
                            __builtin_memcpy(&v, reinterpret_cast<const char*>(acc[i][j].x) + 16u * p, 16);
                            slot[((i * Cfg::BlocksN + j) * PerBlock + p) * Cfg::Threads + threadIdx.x] = v;
                        }
                // Every thread's stores are visible device-wide before the flag is.  The barrier orders
                // the workgroup's stores before thread 0's releasing store, whose write-back of this L2
                // covers them all (the eight XCDs have an L2 each; one write-back per workgroup, not one
                // per wave: they are served one at a time and cost microseconds each).
                __syncthreads();
                if(threadIdx.x == 0u)
                    __hip_atomic_store(sk.flags + sk.mySlot, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
                return true;
            }
            else
            {
                for(uint32_t c = 0; c < sk.slotCount; ++c)
                {
                    const uint32_t s = sk.firstSlot + c;
                    if(threadIdx.x == 0u)
                    {
                        // bounded wait: the contributors run their parts first, so the flag is normally
                        // up long before; a wait that runs out is recorded and the result is wrong
                        // rather than the device hung
                        // (relaxed polls: an acquiring load would invalidate this L2 on every poll and
                        // take the operand panels of the workgroups next door with it; the one fence
                        // that orders the slot reads follows below)
                        uint32_t spins = 0;
                        while(__hip_atomic_load(sk.flags + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u)
                        {
                            __builtin_amdgcn_s_sleep(8);
                            if(++spins > (1u << 22))
                            {
                                __hip_atomic_store(sk.flags + sk.timeoutWord, kStreamKTimedOut, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                break;
                            }
                        }
                        // one invalidation of this compute unit's L1 and this XCD's L2 for the workgroup
                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
                    }
                    __syncthreads();
                    const Words* slot = reinterpret_cast<const Words*>(sk.slots + static_cast<size_t>(s) * sk.slotBytes);
#pragma unroll
                    for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
#pragma unroll
                        for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
#pragma unroll
                            for(uint32_t p = 0; p < PerBlock; ++p)
                            {
                                const Words v = slot[((i * Cfg::BlocksN + j) * PerBlock + p) * Cfg::Threads + threadIdx.x];
                                typename Cfg::CompT part[4];
                                __builtin_memcpy(part, &v, 16);
#pragma unroll
                                for(uint32_t e = 0; e < 4u; ++e)
                                    acc[i][j].x[4u * p + e] += part[e];
                            }
                    __syncthreads();
                    if(threadIdx.x == 0u) // taken: the next launch finds the flag down
                        __hip_atomic_store(sk.flags + s, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                return false;
            }
        }

        // Main loop schedules (per wave), by ring:
        //
        //   ring of two stages of 128 bytes of K (the 256 x 256 tile; N = 2 or 4 MFMA steps per stage):
        //     prologue : copies of stages 0 and 1 in flight; wait for stage 0; barrier; read F(0, step 0)
        //     stage i  : steps 0 .. N-2: read the next step's fragments while this step's MFMAs run
        //                wait: stage i+1 landed and own LDS reads returned;  barrier
        //                issue the copies of stage i+2 into stage i's slot, read F(i+1, step 0) while the
        //                  MFMAs of step N-1 run
        //     (fp8 16x16x128, one step per stage: the A fragments of a stage are held whole, the B fragments
        //     stream through column buffers; see that branch)
        //
        //   ring of S = 4 stages (64 or 128 bytes of K; F0 / F1 = fragment sets of a stage's two steps):
        //     prologue : copies for stages 0..2 in flight; wait for stage 0; barrier; read F0(0)
        //     stage i  : issue copies of stage i+3 (into the slot everybody finished reading at the
        //                  barrier of stage i-1); read F1(i) while the MFMAs of F0(i) run
        //                wait: stage i+1 landed (stages i+2, i+3 may stay in flight) and own LDS reads
        //                  returned;  barrier
        //                read F0(i+1) while the MFMAs of F1(i) run
        //
        // Every LDS read has a full MFMA step to return, and the barrier is the only synchronisation per
        // stage.
        // One macro tile (or, with Part != Whole, a part of its K range): tile (tm, tn) of the tile grid,
        // `stages` pipeline stages of K starting at stage `stage0`.
        template <typename Cfg, TilePart Part = TilePart::Whole>
        ROCWMMA_DEVICE ROCWMMA_INLINE void gemmTile(uint32_t                   tm,
                                                    uint32_t                   tn,
                                                    uint32_t                   stage0,
                                                    uint32_t                   stages,
                                                    uint32_t                   m, // problem size: used by
                                                    uint32_t                   n, // configurations with edge
                                                    uint32_t                   k, // tiles only
                                                    typename Cfg::InT const*   a,
                                                    typename Cfg::InT const*   b,
                                                    typename Cfg::OutT const*  c,
                                                    typename Cfg::OutT*        d,
                                                    uint32_t                   lda,
                                                    uint32_t                   ldb,
                                                    uint32_t                   ldc,
                                                    uint32_t                   ldd,
                                                    typename Cfg::CompT        alpha,
                                                    typename Cfg::CompT        beta,
                                                    StreamKPart const&         sk,
                                                    TileExtras const&          ex = TileExtras{})
        {
            const MxPacked& mx = ex.mx;
            using InT   = typename Cfg::InT;
            using OutT  = typename Cfg::OutT;
            using CompT = typename Cfg::CompT;
            using TileA = typename Cfg::TileA;
            using TileB = typename Cfg::TileB;

            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];

            // (The thread index passes through an empty asm statement: in the persistent kernel, which
            // runs this function once per tile, everything derived from it would otherwise be hoisted
            // out of the tile loop and kept in registers across tiles, and the epilogue, which has none
            // to spare, would spill.)
            uint32_t tid = threadIdx.x;
            asm volatile("" : "+v"(tid));
            const uint32_t lane  = tid & 63u;
            const uint32_t wave  = __builtin_amdgcn_readfirstlane(tid >> 6); // wave uniform
            const uint32_t waveM = wave / Cfg::WavesN;
            const uint32_t waveN = wave % Cfg::WavesN;

            const uint32_t row0 = tm * Cfg::MacroM;
            const uint32_t col0 = tn * Cfg::MacroN;

            // Global sources: uniform tile pointer + uniform per-copy offset + per-lane offset
            const uint32_t ldaB = lda * sizeof(InT);
            const uint32_t ldbB = ldb * sizeof(InT);
            const char*    aSrc = reinterpret_cast<const char*>(a)
                               + static_cast<size_t>(row0) * (Cfg::AKMajor ? ldaB : static_cast<uint32_t>(sizeof(InT)));
            const char* bSrc = reinterpret_cast<const char*>(b)
                               + static_cast<size_t>(col0) * (Cfg::BKMajor ? ldbB : static_cast<uint32_t>(sizeof(InT)));
            // one past the last byte of each operand (edge tiles: the buffer bounds end there)
            const char* const aEnd = reinterpret_cast<const char*>(a)
                                     + (static_cast<size_t>((Cfg::AKMajor ? m : k) - 1u) * lda + (Cfg::AKMajor ? k : m)) * sizeof(InT);
            const char* const bEnd = reinterpret_cast<const char*>(b)
                                     + (static_cast<size_t>((Cfg::BKMajor ? n : k) - 1u) * ldb + (Cfg::BKMajor ? k : n)) * sizeof(InT);
            const size_t   aStep    = TileA::stageStep(ldaB);
            const size_t   bStep    = TileB::stageStep(ldbB);
            aSrc += aStep * stage0; // (the whole K range starts at stage 0)
            bSrc += bStep * stage0;
            // Issuers of the main loop's copies (Cfg::CopyWaves).  The partial tiles of the stream-K kernel keep
            // every wave issuing its own: with the issuer branch their instances, which already spill, ran
            // two to five times slower.
            constexpr uint32_t CopyWaves  = Part == TilePart::Whole ? Cfg::CopyWaves : Cfg::Waves;
            constexpr uint32_t CopyShares = Cfg::Waves / CopyWaves; // waves whose copies one issuer carries
            // (the lane offset of a copy depends on the wave it is issued for through the tile's swizzle: the
            // K-major tile's is the same for a wave and its partner, the dim-major tiles' are not)
            uint32_t aLaneOff[CopyShares], bLaneOff[CopyShares];
#pragma unroll
            for(uint32_t j = 0; j < CopyShares; ++j)
            {
                aLaneOff[j] = TileA::laneSourceOffset(lane, wave % CopyWaves + (Cfg::AKMajor ? 0u : j * CopyWaves), ldaB);
                bLaneOff[j] = TileB::laneSourceOffset(lane, wave % CopyWaves + (Cfg::BKMajor ? 0u : j * CopyWaves), ldbB);
            }

            // A stage is copied in two halves (the A operand, then the B operand) so that each
            // MFMA phase of an iteration carries half of the copy instructions.
            // advance == false leaves the source on the stage just copied (used to re-copy the last
            // stage instead of running past the end of the operand)
            auto issueA = [&](uint32_t slot, bool advance = true) {
                char*                 ldsA = ldsRaw + slot * Cfg::StageBytes;
                const lds::BufferRsrc src  = Cfg::Edges ? lds::makeSource(aSrc, aEnd) : lds::makeSource(aSrc);
                if constexpr(CopyWaves < Cfg::Waves)
                {
                    if(wave < CopyWaves)
                    {
#pragma unroll
                        for(uint32_t i = 0; i < Cfg::CopiesA * CopyShares; ++i)
                        {
                            // (copy i * CopyWaves + wave = copy i / CopyShares of wave + (i % CopyShares) * CopyWaves)
                            const uint32_t copy = i * CopyWaves + wave;
                            lds::asyncCopy16(ldsA + copy * 1024u, src, aLaneOff[i % CopyShares], TileA::copySourceOffset(copy, ldaB));
                        }
                    }
                }
                else
                {
#pragma unroll
                    for(uint32_t i = 0; i < Cfg::CopiesA; ++i)
                    {
                        const uint32_t copy = i * Cfg::Waves + wave;
                        lds::asyncCopy16(ldsA + copy * 1024u, src, aLaneOff[0], TileA::copySourceOffset(copy, ldaB));
                    }
                }
                aSrc += advance ? aStep : size_t{0};
            };
            auto issueB = [&](uint32_t slot, bool advance = true) {
                char*                 ldsB = ldsRaw + slot * Cfg::StageBytes + Cfg::BytesA;
                const lds::BufferRsrc src  = Cfg::Edges ? lds::makeSource(bSrc, bEnd) : lds::makeSource(bSrc);
                if constexpr(CopyWaves < Cfg::Waves)
                {
                    if(wave < CopyWaves)
                    {
#pragma unroll
                        for(uint32_t i = 0; i < Cfg::CopiesB * CopyShares; ++i)
                        {
                            // (copy i * CopyWaves + wave = copy i / CopyShares of wave + (i % CopyShares) * CopyWaves)
                            const uint32_t copy = i * CopyWaves + wave;
                            lds::asyncCopy16(ldsB + copy * 1024u, src, bLaneOff[i % CopyShares], TileB::copySourceOffset(copy, ldbB));
                        }
                    }
                }
                else
                {
#pragma unroll
                    for(uint32_t i = 0; i < Cfg::CopiesB; ++i)
                    {
                        const uint32_t copy = i * Cfg::Waves + wave;
                        lds::asyncCopy16(ldsB + copy * 1024u, src, bLaneOff[0], TileB::copySourceOffset(copy, ldbB));
                    }
                }
                bSrc += advance ? bStep : size_t{0};
            };
            auto issueStage = [&](uint32_t slot, bool advance = true) {
                issueA(slot, advance);
                issueB(slot, advance);
            };

            struct Frags
            {
                typename Cfg::FragA a[Cfg::BlocksM];
                typename Cfg::FragB b[Cfg::BlocksN];
            };

            auto readFrags = [&](Frags& f, uint32_t slot, uint32_t ks) {
                const char* ldsA = ldsRaw + slot * Cfg::StageBytes;
                const char* ldsB = ldsA + Cfg::BytesA;
                if constexpr(Cfg::Scaled && Cfg::Block == 16u) // (has a reader of its own in its loop)
                    return;
                else if constexpr(Cfg::Scaled)
                {
                    // 32x32x64 with block scales: the instruction's own K order, two runs of 16 bytes per lane from
                    // the two halves of the 64-byte step (chunks h and 2 + h of the step's four)
#pragma unroll
                    for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
                    {
                        TileA::template readBlock32<16u>(f.a[i].x, ldsA, waveM * Cfg::WaveM + i * Cfg::Block, 2u * ks, lane);
                        TileA::template readBlock32<16u>(f.a[i].x + 16, ldsA, waveM * Cfg::WaveM + i * Cfg::Block, 2u * ks + 1u, lane);
                    }
#pragma unroll
                    for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
                    {
                        TileB::template readBlock32<16u>(f.b[j].x, ldsB, waveN * Cfg::WaveN + j * Cfg::Block, 2u * ks, lane);
                        TileB::template readBlock32<16u>(f.b[j].x + 16, ldsB, waveN * Cfg::WaveN + j * Cfg::Block, 2u * ks + 1u, lane);
                    }
                }
                else
                {
#pragma unroll
                for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
                {
                    if constexpr(Cfg::Block == 32u)
                        TileA::template readBlock32<Cfg::KPackBytes>(f.a[i].x, ldsA, waveM * Cfg::WaveM + i * Cfg::Block, ks, lane);
                    else
                        TileA::template readBlock16<Cfg::KPackBytes>(f.a[i].x, ldsA, waveM * Cfg::WaveM + i * Cfg::Block, ks, lane);
                }
#pragma unroll
                for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
                {
                    if constexpr(Cfg::Block == 32u)
                        TileB::template readBlock32<Cfg::KPackBytes>(f.b[j].x, ldsB, waveN * Cfg::WaveN + j * Cfg::Block, ks, lane);
                    else
                        TileB::template readBlock16<Cfg::KPackBytes>(f.b[j].x, ldsB, waveN * Cfg::WaveN + j * Cfg::Block, ks, lane);
                }
                }
            };

            // Fragments of a dim-major operand come from inline-assembly transposing reads: after the wait
            // that covers those reads, their registers are tied to that point of the program.
            auto pinFrags = [&](Frags& f) {
                if constexpr(!Cfg::AKMajor)
                {
#pragma unroll
                    for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
                        lds::pinRegisters(f.a[i].x);
                }
                if constexpr(!Cfg::BKMajor)
                {
#pragma unroll
                    for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
                        lds::pinRegisters(f.b[j].x);
                }
                (void)f;
            };

            typename Cfg::FragAcc acc[Cfg::BlocksM][Cfg::BlocksN];
#pragma unroll
            for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
#pragma unroll
                for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
                    fill_fragment(acc[i][j], static_cast<CompT>(0));

            auto multiply = [&](Frags const& f) {
#pragma unroll
                for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
#pragma unroll
                    for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
                        mma_sync(acc[i][j], f.a[i], f.b[j], acc[i][j]);
            };

            constexpr uint32_t S      = Cfg::Stages;
            // `stages` stages of K from stage0 on: >= S - 1 of them (checked by the host)

            if constexpr(S == 2u && Cfg::KSteps == 1u)
            {
                // Ring of two stages, one MFMA step per stage whose fragments would not fit the register
                // file twice (fp8 16x16x128: 8 registers per block and operand).  The A fragments of a
                // stage are held whole (and read one stage ahead into a second set); the B fragments
                // stream through column buffers: while column j is multiplied, column j + Ahead is read.
                // The barrier sits in front of the last Ahead columns: by then the wave has read everything
                // it needs from stage i (the last columns' fragments arrived with the wait), stage i + 1 has
                // landed, and the copies of stage i + 2 go out into stage i's slot.
                static_assert(Cfg::AKMajor && Cfg::BKMajor, "streamed columns: K-contiguous operands");
                static_assert(!Cfg::Scaled || Part == TilePart::Whole, "block scales: whole K ranges from stage 0");
                // Block scales (Scaled only): per lane, pair of stages and group of four blocks, two
                // registers: byte (block % 2) * 2 + stage parity of register (block % 4) / 2.  The next
                // pair's are loaded while the first stage of a pair is multiplied and take over after the
                // second.
                typedef uint32_t   Scales __attribute__((ext_vector_type(2)));
                constexpr uint32_t GroupsN = Cfg::BlocksN / 4u;
                static_assert(!Cfg::Scaled || (Cfg::BlocksM == 4u && Cfg::BlocksN % 4u == 0u), "packed scales: groups of four blocks");
                Scales        sA = {}, sAnext = {};
                Scales        sB[GroupsN > 0u ? GroupsN : 1u] = {}, sBnext[GroupsN > 0u ? GroupsN : 1u] = {};
                const Scales* mxA = nullptr;
                const Scales* mxB = nullptr;
                auto loadScales = [&](Scales& a_, Scales(&b_)[GroupsN > 0u ? GroupsN : 1u], uint32_t pair) {
                    a_ = mxA[static_cast<size_t>(pair) * 64u];
#pragma unroll
                    for(uint32_t gN = 0; gN < GroupsN; ++gN)
                        b_[gN] = mxB[(static_cast<size_t>(gN) * mx.pairs + pair) * 64u];
                };
                if constexpr(Cfg::Scaled)
                {
                    mxA = static_cast<const Scales*>(mx.a) + static_cast<size_t>(row0 / 64u + waveM) * mx.pairs * 64u + lane;
                    mxB = static_cast<const Scales*>(mx.b) + static_cast<size_t>(col0 / 64u + waveN * GroupsN) * mx.pairs * 64u + lane;
                    // (in front of the first copies: the wait for stage 0 below then covers these loads, and the
                    // loop is entered with none of them in flight)
                    loadScales(sA, sB, 0u);
                    __builtin_amdgcn_sched_barrier(0); // (and stay in front of them)
                }
                issueStage(0u, 1u < stages);
                issueStage(1u, 2u < stages);
                lds::waitCopiesAndReads<(CopyWaves == Cfg::Waves ? Cfg::Copies : 0u)>(); // stage 0 has landed
                lds::barrier();
                // B column buffers: `Ahead` columns are read in advance.  With three (four buffers, whose indices
                // repeat every stage of four or eight columns) the barrier moves in front of the last three
                // columns, so that what follows it (the copies, the next stage's A fragments and first B columns)
                // has twelve MFMAs to hide behind instead of four: 252 registers, no spills, fp8
                // 4096 x 14336 x 4096 194.0 -> 190.3 us.  The kernel with block scales keeps one column ahead
                // (its scale registers take the room).
                constexpr uint32_t Ahead = (!Cfg::Scaled && Cfg::BlocksN % 4u == 0u) ? 3u : 1u;
                constexpr uint32_t NB    = Ahead + 1u;
                static_assert(Cfg::BlocksN % NB == 0u && Cfg::BlocksN > Ahead, "the buffer of a column must not depend on the stage");
                typename Cfg::FragA fa[2][Cfg::BlocksM];
                typename Cfg::FragB fb[NB];
                auto readA = [&](typename Cfg::FragA(&dst)[Cfg::BlocksM], uint32_t slot) {
                    const char* ldsA = ldsRaw + slot * Cfg::StageBytes;
#pragma unroll
                    for(uint32_t bi = 0; bi < Cfg::BlocksM; ++bi)
                    {
                        const uint32_t r0 = waveM * Cfg::WaveM + bi * Cfg::Block;
                        if constexpr(Cfg::Scaled)
                        {
                            TileA::template readBlock16<16u>(dst[bi].x, ldsA, r0, 0u, lane);
                            TileA::template readBlock16<16u>(dst[bi].x + 16, ldsA, r0, 1u, lane);
                        }
                        else
                            TileA::template readBlock16<Cfg::KPackBytes>(dst[bi].x, ldsA, r0, 0u, lane);
                    }
                };
                auto readB = [&](typename Cfg::FragB& dst, uint32_t slot, uint32_t bj) {
                    const char*    ldsB = ldsRaw + slot * Cfg::StageBytes + Cfg::BytesA;
                    const uint32_t c0   = waveN * Cfg::WaveN + bj * Cfg::Block;
                    if constexpr(Cfg::Scaled)
                    {
                        TileB::template readBlock16<16u>(dst.x, ldsB, c0, 0u, lane);
                        TileB::template readBlock16<16u>(dst.x + 16, ldsB, c0, 1u, lane);
                    }
                    else
                        TileB::template readBlock16<Cfg::KPackBytes>(dst.x, ldsB, c0, 0u, lane);
                };
                auto column = [&](typename Cfg::FragA const(&a_)[Cfg::BlocksM], typename Cfg::FragB const& b_, auto bjC, auto stC) {
                    constexpr uint32_t bj = decltype(bjC)::value, st = decltype(stC)::value;
                    if constexpr(Cfg::Scaled)
                    {
#if ROCWMMA_ARCH_GFX950 // (the instruction table exists in the device pass only)
                        using Op  = detail::MfmaScaled<detail::TypeInfo<InT>::cls, detail::TypeInfo<InT>::cls, 16u>;
                        using Acc = typename Op::Acc;
                        staticFor<Cfg::BlocksM>([&](auto biC) {
                            constexpr uint32_t bi = decltype(biC)::value;
                            Acc&               v  = *reinterpret_cast<Acc*>(acc[bi][bj].x);
                            // (the accumulator is kept transposed: the instruction's first multiplicand is B)
                            v = Op::template exec<(bj % 2u) * 2u + st, (bi % 2u) * 2u + st>(b_.x, a_[bi].x, v, sB[bj / 4u][(bj % 4u) / 2u],
                                                                                           sA[bi / 2u]);
                        });
#else
                        (void)a_, (void)b_, (void)bj, (void)st;
#endif
                    }
                    else
                    {
#pragma unroll
                        for(uint32_t bi = 0; bi < Cfg::BlocksM; ++bi)
                            mma_sync(acc[bi][bj], a_[bi], b_, acc[bi][bj]);
                    }
                };
                constexpr uint32_t RB = Cfg::KPackBytes / 16u; // LDS reads per block
                readA(fa[0], 0u);
#pragma unroll
                for(uint32_t j = 0; j < Ahead; ++j)
                    readB(fb[j], 0u, j);
                // (the A sets alternate with the stage parity; two stages per trip keep the indices static)
                auto stage = [&](typename Cfg::FragA(&cur)[Cfg::BlocksM], typename Cfg::FragA(&nxt)[Cfg::BlocksM], auto slotC,
                                 uint32_t ii) {
                        constexpr uint32_t slot = decltype(slotC)::value;
                        staticFor<Cfg::BlocksN - Ahead>([&](auto bjC) {
                            constexpr uint32_t bj = decltype(bjC)::value;
                            readB(fb[(bj + Ahead) % NB], slot, bj + Ahead);
                            column(cur, fb[bj % NB], bjC, slotC);
                            scheduleInterleaved<Cfg::BlocksM, RB, 0u>();
                            __builtin_amdgcn_sched_barrier(0);
                        });
                        lds::waitCopiesAndReads<0u>(); // stage ii + 1 has landed, stage ii is in registers
                        lds::barrier();
                        __builtin_amdgcn_sched_barrier(0);
                        issueStage(slot, ii + 3u < stages);
                        if constexpr(Cfg::Scaled && slot == 0u)
                        {
                            // scales of the next pair of stages (the last pair again past the end of K)
                            loadScales(sAnext, sBnext, ii / 2u + 1u < mx.pairs ? ii / 2u + 1u : mx.pairs - 1u);
                        }
                        readA(nxt, slot ^ 1u);
                        staticFor<Ahead>([&](auto tC) {
                            constexpr uint32_t t  = decltype(tC)::value;
                            constexpr uint32_t bj = Cfg::BlocksN - Ahead + t;
                            readB(fb[(bj + Ahead) % NB], slot ^ 1u, t);
                            column(cur, fb[bj % NB], std::integral_constant<uint32_t, bj>{}, slotC);
                            if constexpr(Ahead > 1u)
                                __builtin_amdgcn_sched_barrier(0);
                        });
                        __builtin_amdgcn_sched_barrier(0);
                        if constexpr(Cfg::Scaled && slot == 1u)
                        {
                            sA = sAnext;
#pragma unroll
                            for(uint32_t gN = 0; gN < GroupsN; ++gN)
                                sB[gN] = sBnext[gN];
                        }
                };
                const std::integral_constant<uint32_t, 0u> even{};
                const std::integral_constant<uint32_t, 1u> odd{};
                uint32_t i = 0;
                for(; i + 1u < stages; i += 2u)
                {
                    stage(fa[0], fa[1], even, i);
                    stage(fa[1], fa[0], odd, i + 1u);
                }
                if(i < stages)
                    stage(fa[0], fa[1], even, i);
                lds::waitCopiesAndReads<0u>(); // the surplus copies still target this workgroup's LDS
                lds::barrier();
            }
            else if constexpr(S == 2u)
            {
                // Ring of two stages of 128 bytes of K (two or four MFMA steps each).  A phase multiplies
                // one step while it reads the fragments of the next; the barrier in front of a stage's
                // last phase is where stage i has been read completely and stage i+1 has landed, so
                // the copies of stage i+2 go out right behind it, into stage i's slot, and have the
                // phases up to the next barrier to land.  Past the end of K the loop copies the
                // last stage again and reads fragments nobody multiplies, so its body is uniform.
                // Block scales (Scaled, 32-wide blocks): per lane and pair of stages (256 bytes of K = four
                // instruction steps), one dword per block of 32 rows, byte = step; the step's byte is shifted
                // down at run time.  The next pair's are loaded behind the barrier of a pair's first stage.
                static_assert(!Cfg::Scaled || Cfg::KSteps == 2u, "packed scales: two instruction steps per stage");
                uint32_t        sA[Cfg::BlocksM] = {}, sB[Cfg::BlocksN] = {}, sAnext[Cfg::BlocksM] = {}, sBnext[Cfg::BlocksN] = {};
                const uint32_t* mxA = nullptr; // dword of (this wave's first block, pair of stages 0, this lane)
                const uint32_t* mxB = nullptr;
                // (dword of block b of an operand, pair p, lane l: (((b / 2) * pairs + p) * 64 + l) * 2 + b % 2)
                auto scalePtr = [&](const void* base, uint32_t firstBlock) {
                    return static_cast<const uint32_t*>(base) + (static_cast<size_t>(firstBlock / 2u) * mx.pairs * 64u + lane) * 2u + firstBlock % 2u;
                };
                auto loadScales32 = [&](uint32_t(&a_)[Cfg::BlocksM], uint32_t(&b_)[Cfg::BlocksN], uint32_t pair) {
                    // (a wave's blocks start at an even block or are a single one: block i sits i % 2 dwords and
                    // i / 2 groups on)
#pragma unroll
                    for(uint32_t bi = 0; bi < Cfg::BlocksM; ++bi)
                        a_[bi] = mxA[(static_cast<size_t>(bi / 2u) * mx.pairs + pair) * 128u + bi % 2u];
#pragma unroll
                    for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                        b_[bj] = mxB[(static_cast<size_t>(bj / 2u) * mx.pairs + pair) * 128u + bj % 2u];
                };
                if constexpr(Cfg::Scaled)
                {
                    static_assert(Cfg::BlocksM == 1u || Cfg::BlocksM % 2u == 0u, "a wave's row blocks: one, or whole groups of two");
                    static_assert(Cfg::BlocksN == 1u || Cfg::BlocksN % 2u == 0u, "a wave's column blocks: one, or whole groups of two");
                    mxA = scalePtr(mx.a, (row0 + waveM * Cfg::WaveM) / 32u);
                    mxB = scalePtr(mx.b, (col0 + waveN * Cfg::WaveN) / 32u);
                    // (in front of the first copies and kept there: the wait for stage 0 then covers these loads,
                    // and the loop is entered with none of them in flight)
                    loadScales32(sA, sB, 0u);
                    __builtin_amdgcn_sched_barrier(0);
                }
                issueStage(0u, 1u < stages);
                issueStage(1u, 2u < stages);
                lds::waitCopiesAndReads<(CopyWaves == Cfg::Waves ? Cfg::Copies : 0u)>(); // stage 0 has landed
                lds::barrier();
                constexpr uint32_t N = Cfg::KSteps; // MFMA steps per stage: 2 or 4 (even: the fragment sets alternate)
                Frags              f[2];
                auto multiplyStep = [&](Frags const& fr, uint32_t i, uint32_t ks) {
                    if constexpr(Cfg::Scaled)
                    {
#if ROCWMMA_ARCH_GFX950 // (the instruction table exists in the device pass only)
                        using Op  = detail::MfmaScaled<detail::TypeInfo<InT>::cls, detail::TypeInfo<InT>::cls, 32u>;
                        using Acc = typename Op::Acc;
                        const uint32_t shift = 8u * ((i % 2u) * N + ks); // the step's byte within the pair of stages
#pragma unroll
                        for(uint32_t bi = 0; bi < Cfg::BlocksM; ++bi)
#pragma unroll
                            for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                            {
                                Acc& v = *reinterpret_cast<Acc*>(acc[bi][bj].x);
                                // (the accumulator is kept transposed: the instruction's first multiplicand is B)
                                v = Op::template exec<0, 0>(fr.b[bj].x, fr.a[bi].x, v, sB[bj] >> shift, sA[bi] >> shift);
                            }
#else
                        (void)fr, (void)i, (void)ks;
#endif
                    }
                    else
                    {
                        (void)i, (void)ks;
                        multiply(fr);
                    }
                };
                readFrags(f[0], 0u, 0u);
                for(uint32_t i = 0; i < stages; ++i)
                {
#pragma unroll
                    for(uint32_t ks = 0; ks + 1u < N; ++ks)
                    {
                        if constexpr(!Cfg::AKMajor || !Cfg::BKMajor)
                        {
                            lds::waitReads(); // transposing reads of the previous phase
                            pinFrags(f[ks & 1u]);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                        readFrags(f[(ks + 1u) & 1u], i % 2u, ks + 1u);
                        multiplyStep(f[ks & 1u], i, ks);
                        scheduleInterleaved<Cfg::MfmasPerStep / 2u, Cfg::ReadsPerStep, 0u>();
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    lds::waitCopiesAndReads<0u>(); // stage i+1 has landed, stage i is in registers
                    pinFrags(f[(N - 1u) & 1u]);
                    lds::barrier();
                    __builtin_amdgcn_sched_barrier(0);
                    issueStage(i % 2u, i + 3u < stages);
                    if constexpr(Cfg::Scaled)
                    {
                        if(i % 2u == 0u)
                            loadScales32(sAnext, sBnext, i / 2u + 1u < mx.pairs ? i / 2u + 1u : mx.pairs - 1u);
                    }
                    readFrags(f[0], (i + 1u) % 2u, 0u);
                    multiplyStep(f[(N - 1u) & 1u], i, N - 1u);
                    if constexpr(Cfg::Scaled)
                    {
                        if(i % 2u == 1u)
                        {
#pragma unroll
                            for(uint32_t bi = 0; bi < Cfg::BlocksM; ++bi)
                                sA[bi] = sAnext[bi];
#pragma unroll
                            for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                                sB[bj] = sBnext[bj];
                        }
                    }
                    scheduleInterleaved<Cfg::MfmasPerStep / 2u, Cfg::ReadsPerStep, 0u>();
                    scheduleInterleaved<Cfg::MfmasPerStep - Cfg::MfmasPerStep / 2u, 0u, Cfg::Copies>();
                    __builtin_amdgcn_sched_barrier(0);
                }
                lds::waitCopiesAndReads<0u>(); // the surplus copies still target this workgroup's LDS
                lds::barrier();
            }
            else if constexpr(Cfg::KSteps == 2u && Cfg::Scaled)
            {
                // Ring of four stages of 128 bytes of K with block scales (32-wide blocks, two instruction steps per
                // stage): the loop below with the scale loads joining its count of vector-memory operations in
                // flight.  Two stages per trip, so that a trip is one pair of stages of the packed scales (one dword
                // per block and lane, byte = step of the pair) and everything that depends on a stage's parity is a
                // constant: the next pair's scales are requested at the head of a trip, two stages before they take
                // over.  Every trip issues its stages (past the end of K the last stage again, into a slot nobody
                // reads), so the body and its counts are uniform.
                static_assert(S == 4u && Cfg::StageKB == 128u && Cfg::Block == 32u && Part == TilePart::Whole, "scaled ring of four: 128-byte stages of 32-wide blocks");
                uint32_t        sA[Cfg::BlocksM] = {}, sB[Cfg::BlocksN] = {}, sAnext[Cfg::BlocksM] = {}, sBnext[Cfg::BlocksN] = {};
                // (dword of block b of an operand, pair p, lane l: (((b / 2) * pairs + p) * 64 + l) * 2 + b % 2)
                const uint32_t* mxA = static_cast<const uint32_t*>(mx.a)
                                      + (static_cast<size_t>((row0 + waveM * Cfg::WaveM) / 64u) * mx.pairs * 64u + lane) * 2u
                                      + ((row0 + waveM * Cfg::WaveM) / 32u) % 2u;
                const uint32_t* mxB = static_cast<const uint32_t*>(mx.b)
                                      + (static_cast<size_t>((col0 + waveN * Cfg::WaveN) / 64u) * mx.pairs * 64u + lane) * 2u
                                      + ((col0 + waveN * Cfg::WaveN) / 32u) % 2u;
                static_assert(Cfg::BlocksM == 1u || Cfg::BlocksM % 2u == 0u, "a wave's row blocks: one, or whole groups of two");
                static_assert(Cfg::BlocksN == 1u || Cfg::BlocksN % 2u == 0u, "a wave's column blocks: one, or whole groups of two");
                auto loadScales32 = [&](uint32_t(&a_)[Cfg::BlocksM], uint32_t(&b_)[Cfg::BlocksN], uint32_t pair) {
#pragma unroll
                    for(uint32_t bi = 0; bi < Cfg::BlocksM; ++bi)
                        a_[bi] = mxA[(static_cast<size_t>(bi / 2u) * mx.pairs + pair) * 128u + bi % 2u];
#pragma unroll
                    for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                        b_[bj] = mxB[(static_cast<size_t>(bj / 2u) * mx.pairs + pair) * 128u + bj % 2u];
                };
                auto multiplyScaled = [&](Frags const& fr, auto stepC) {
#if ROCWMMA_ARCH_GFX950 // (the instruction table exists in the device pass only)
                    using Op  = detail::MfmaScaled<detail::TypeInfo<InT>::cls, detail::TypeInfo<InT>::cls, 32u>;
                    using Acc = typename Op::Acc;
                    constexpr uint32_t shift = 8u * decltype(stepC)::value; // the step's byte within the pair of stages
#pragma unroll
                    for(uint32_t bi = 0; bi < Cfg::BlocksM; ++bi)
#pragma unroll
                        for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                        {
                            Acc& v = *reinterpret_cast<Acc*>(acc[bi][bj].x);
                            // (the accumulator is kept transposed: the instruction's first multiplicand is B)
                            v = Op::template exec<0, 0>(fr.b[bj].x, fr.a[bi].x, v, sB[bj] >> shift, sA[bi] >> shift);
                        }
#else
                    (void)fr, (void)stepC;
#endif
                };
                // (in front of the first copies and kept there: the wait for stage 0 covers them)
                loadScales32(sA, sB, 0u);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(uint32_t st = 0; st < S - 1u; ++st)
                    issueStage(st, st + 1u < stages);
                lds::waitCopiesAndReads<(S - 2u) * Cfg::Copies>();
                lds::barrier();
                Frags f0, f1;
                readFrags(f0, 0u, 0u);
                auto stage = [&](uint32_t i, auto parityC) {
                    constexpr uint32_t parity = decltype(parityC)::value;
                    const uint32_t     slot   = (i + S - 1u) % S;
                    const bool         adv    = i + S < stages;
                    issueA(slot, adv);
                    readFrags(f1, i % S, 1u);
                    multiplyScaled(f0, std::integral_constant<uint32_t, parity * 2u>{});
                    scheduleInterleaved<Cfg::MfmasPerStep / 2u, Cfg::ReadsPerStep, 0u>();
                    scheduleInterleaved<Cfg::MfmasPerStep - Cfg::MfmasPerStep / 2u, 0u, Cfg::CopiesA>();
                    __builtin_amdgcn_sched_barrier(0);
                    // Stage i+1 has landed once only stage i+2 and the A half of stage i+3 are in flight.  The scale
                    // loads of a trip's head sit between those two in issue order, but loads into registers do not
                    // complete in order with copies into LDS (counting them as in flight let a wait pass with a copy of
                    // stage i+1 outstanding whenever they had returned first: wrong results on a cold cache), so they
                    // are not counted: with them outstanding the wait holds a little longer, never too short.
                    lds::waitCopiesAndReads<(S - 3u) * Cfg::Copies + Cfg::CopiesA>();
                    lds::barrier();
                    __builtin_amdgcn_sched_barrier(0);
                    issueB(slot, adv);
                    readFrags(f0, (i + 1u) % S, 0u);
                    multiplyScaled(f1, std::integral_constant<uint32_t, parity * 2u + 1u>{});
                    scheduleInterleaved<Cfg::MfmasPerStep / 2u, Cfg::ReadsPerStep, 0u>();
                    scheduleInterleaved<Cfg::MfmasPerStep - Cfg::MfmasPerStep / 2u, 0u, Cfg::CopiesB>();
                    __builtin_amdgcn_sched_barrier(0);
                };
                for(uint32_t i = 0; i < stages; i += 2u)
                {
                    loadScales32(sAnext, sBnext, i / 2u + 1u < mx.pairs ? i / 2u + 1u : mx.pairs - 1u);
                    __builtin_amdgcn_sched_barrier(0);
                    stage(i, std::integral_constant<uint32_t, 0u>{});
                    if(i + 1u < stages)
                        stage(i + 1u, std::integral_constant<uint32_t, 1u>{});
#pragma unroll
                    for(uint32_t bi = 0; bi < Cfg::BlocksM; ++bi)
                        sA[bi] = sAnext[bi];
#pragma unroll
                    for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                        sB[bj] = sBnext[bj];
                }
                lds::waitCopiesAndReads<0u>(); // the surplus copies still target this workgroup's LDS
                lds::barrier();
            }
            else if constexpr(Cfg::KSteps == 2u)
            {
                // Prologue
#pragma unroll
                for(uint32_t s = 0; s < S - 1u; ++s)
                    issueStage(s);
                lds::waitCopiesAndReads<(S - 2u) * Cfg::Copies>();
                lds::barrier();
                Frags f0, f1;
                readFrags(f0, 0u, 0u);

                // Steady state: a new stage is issued every iteration
                uint32_t i = 0;
                for(; i + (S - 1u) < stages; ++i)
                {
                    if constexpr(!Cfg::AKMajor || !Cfg::BKMajor)
                    {
                        lds::waitReads(); // fragments read during the previous phase
                        pinFrags(f0);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    issueA((i + S - 1u) % S);
                    readFrags(f1, i % S, 1u);
                    multiply(f0);
                    // LDS reads ride on the first half of the MFMAs (so they are back at the
                    // barrier), the copies on the second half, two MFMAs per copy
                    scheduleInterleaved<Cfg::MfmasPerStep / 2u, Cfg::ReadsPerStep, 0u>();
                    scheduleInterleaved<Cfg::MfmasPerStep - Cfg::MfmasPerStep / 2u, 0u, Cfg::CopiesA>();
                    __builtin_amdgcn_sched_barrier(0); // nothing moves across the synchronisation point
                    // stage i+1 has landed once only stage i+2 and the A half of stage i+3 are in flight
                    lds::waitCopiesAndReads<(S - 3u) * Cfg::Copies + Cfg::CopiesA>();
                    pinFrags(f1);
                    lds::barrier();
                    __builtin_amdgcn_sched_barrier(0);
                    issueB((i + S - 1u) % S);
                    readFrags(f0, (i + 1u) % S, 0u);
                    multiply(f1);
                    scheduleInterleaved<Cfg::MfmasPerStep / 2u, Cfg::ReadsPerStep, 0u>();
                    scheduleInterleaved<Cfg::MfmasPerStep - Cfg::MfmasPerStep / 2u, 0u, Cfg::CopiesB>();
                    __builtin_amdgcn_sched_barrier(0);
                }
                // Drain: nothing left to issue; the remaining stages are already in flight
                for(; i < stages; ++i)
                {
                    const bool more = i + 1u < stages;
                    if constexpr(!Cfg::AKMajor || !Cfg::BKMajor)
                    {
                        lds::waitReads();
                        pinFrags(f0);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    readFrags(f1, i % S, 1u);
                    multiply(f0);
                    __builtin_amdgcn_sched_barrier(0);
                    lds::waitCopiesAndReads<0u>();
                    pinFrags(f1);
                    lds::barrier();
                    __builtin_amdgcn_sched_barrier(0);
                    if(more)
                        readFrags(f0, (i + 1u) % S, 0u);
                    multiply(f1);
                }
            }
            else
            {
                // One MFMA step per stage (wide fp8): a phase multiplies stage s (fragments read
                // during the previous phase) while it reads the fragments of stage s+1 and issues
                // the copies of stage s+3; the wait + barrier closing the phase makes stage s+2
                // visible.  Two phases per loop trip so the fragment sets swap without copies.
                // Every phase issues a stage, so the loop body and its wait counts are uniform:
                // past the end of K the last stage is copied again into a ring slot nobody reads.
                static_assert(Cfg::KSteps == 1u, "one MFMA step per stage");
                Frags f0, f1;
                // Transposing LDS reads are inline assembly, which the scheduling hints cannot
                // place: with a dim-major B (two such reads for each of its 8 blocks) the phase is laid
                // out by hand, one column of blocks at a time (the reads of that column of the next
                // stage, then its MFMAs): 5 % faster than leaving the reads in front of the MFMAs.  With
                // only A dim-major (4 blocks) the compiler's placement is 1 % better and is kept.
                auto phaseByColumns = [&](Frags const& cur, Frags& nxt, uint32_t slot) {
                    const char* ldsA = ldsRaw + slot * Cfg::StageBytes;
                    const char* ldsB = ldsA + Cfg::BytesA;
                    if constexpr(Cfg::Block == 16u)
                    {
                        static_assert(Cfg::BlocksM <= Cfg::BlocksN, "the A blocks are read along with the first B columns");
#pragma unroll
                        for(uint32_t j = 0; j < Cfg::BlocksN; ++j)
                        {
                            TileB::template readBlock16<Cfg::KPackBytes>(nxt.b[j].x, ldsB, waveN * Cfg::WaveN + j * Cfg::Block, 0u, lane);
                            if(j < Cfg::BlocksM)
                                TileA::template readBlock16<Cfg::KPackBytes>(nxt.a[j].x, ldsA, waveM * Cfg::WaveM + j * Cfg::Block, 0u, lane);
#pragma unroll
                            for(uint32_t i = 0; i < Cfg::BlocksM; ++i)
                                mma_sync(acc[i][j], cur.a[i], cur.b[j], acc[i][j]);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                };
#define ROCWMMA_AMD_PHASE(STAGE, CUR, NXT, READ)                                                         \
    do                                                                                                  \
    {                                                                                                   \
        issueStage(((STAGE) + S - 1u) % S, (STAGE) + S < stages);                                       \
        if constexpr(Cfg::BKMajor || Cfg::Block != 16u)                                                 \
        {                                                                                               \
            if(READ)                                                                                    \
                readFrags(NXT, ((STAGE) + 1u) % S, 0u);                                                 \
            multiply(CUR);                                                                              \
            scheduleInterleaved<Cfg::MfmasPerStep / 2u, Cfg::ReadsPerStep, 0u>();                       \
            scheduleInterleaved<Cfg::MfmasPerStep - Cfg::MfmasPerStep / 2u, 0u, Cfg::Copies>();         \
        }                                                                                               \
        else                                                                                            \
            phaseByColumns(CUR, NXT, ((STAGE) + 1u) % S);                                               \
        __builtin_amdgcn_sched_barrier(0);                                                              \
        lds::waitCopiesAndReads<(S - 3u) * Cfg::Copies>();                                              \
        pinFrags(NXT);                                                                                  \
        lds::barrier();                                                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                              \
    } while(0)

#pragma unroll
                for(uint32_t s = 0; s < S - 1u; ++s)
                    issueStage(s, s + 1u < stages);
                lds::waitCopiesAndReads<(S - 3u) * Cfg::Copies>(); // stages 0 and 1 have landed
                lds::barrier();
                readFrags(f0, 0u, 0u);
                if constexpr(!Cfg::AKMajor || !Cfg::BKMajor)
                {
                    lds::waitReads(); // the transposing reads are outside the compiler's tracking
                    pinFrags(f0);
                    __builtin_amdgcn_sched_barrier(0);
                }
                uint32_t s = 0;
                for(; s + 1u < stages; s += 2u)
                {
                    ROCWMMA_AMD_PHASE(s, f0, f1, true);
                    // (past the last stage this reads a ring slot whose content nobody multiplies:
                    // an unconditional phase body keeps the instruction interleave intact)
                    ROCWMMA_AMD_PHASE(s + 1u, f1, f0, true);
                }
                if(s < stages)
                    multiply(f0);
                lds::waitCopiesAndReads<0u>(); // the surplus copies still target this workgroup's LDS
                lds::barrier();
#undef ROCWMMA_AMD_PHASE
            }

            if constexpr(Part != TilePart::Whole)
            {
                // Part of a tile's K range (stream-K).  A contributor hands its raw accumulators over
                // through its workspace slot and is done; the owner (the part that starts at K = 0)
                // adds the slots of the parts behind it, in order, and goes on to the epilogue.
                if(streamKHandOver<Cfg, Part>(acc, sk))
                    return;
            }

            // Epilogue: D = alpha * acc + beta * C, one row of blocks (BlocksN blocks) at a time,
            // 16-byte accesses per lane.  Every block of a group has registers of its own, so
            // the stores of a group issue back to back (a store whose data registers are about
            // to be overwritten holds up the instruction stream until it has read them), and
            // the C blocks of the next two groups are in flight while a group is finished.
            const uint32_t wRow        = row0 + waveM * Cfg::WaveM;
            const uint32_t wCol        = col0 + waveN * Cfg::WaveN;
            // Plain stores: the 32-byte pieces a store instruction writes per row are merged into
            // full lines in the L2.  Non-temporal stores bypass that merge and were 3-5x slower
            // (4096 x 14336 x 256 int8: 157-277 us against 58 us).
            // (accumulator layout: lane l owns runs of 4 consecutive columns of row l % Block;
            // 32-wide blocks: 4 runs at columns 8 r + 4 (l / 32); 16-wide blocks: 1 run at 4 (l / 16))
            constexpr uint32_t Runs     = Cfg::Block == 32u ? 4u : 1u; // runs per block per lane
            const uint32_t     accRow   = lane & (Cfg::Block - 1u);
            const uint32_t     accGroup = lane / Cfg::Block; // 0..1 or 0..3
            // (edge tiles: a lane's run of four columns of one row is inside the problem or outside it
            // as a whole, N being a multiple of 16)
            auto inside = [&](uint32_t bi, uint32_t bj, uint32_t r) {
                return wRow + bi * Cfg::Block + accRow < m && wCol + bj * Cfg::Block + 8u * r + 4u * accGroup < n;
            };
            auto storeBlock = [&](uint32_t bi, uint32_t bj, auto const& f) {
                typedef uint32_t Words __attribute__((ext_vector_type(sizeof(OutT))));
                OutT* dst = d + static_cast<size_t>(wRow + bi * Cfg::Block) * ldd + wCol + bj * Cfg::Block;
#pragma unroll
                for(uint32_t r = 0; r < Runs; ++r)
                {
                    Words v;
                    __builtin_memcpy(&v, f.x + 4u * r, sizeof(v));
                    if(!Cfg::Edges || inside(bi, bj, r))
                        *reinterpret_cast<Words*>(dst + static_cast<size_t>(accRow) * ldd + 8u * r + 4u * accGroup) = v;
                }
            };
            auto loadBlockC = [&](uint32_t bi, uint32_t bj, auto& f) {
                const OutT* src = c + static_cast<size_t>(wRow + bi * Cfg::Block) * ldc + wCol + bj * Cfg::Block;
                if constexpr(!Cfg::Edges)
                    load_matrix_sync(f, src, ldc);
                else
                {
                    typedef uint32_t Words __attribute__((ext_vector_type(sizeof(OutT))));
#pragma unroll
                    for(uint32_t r = 0; r < Runs; ++r)
                    {
                        Words v = {};
                        if(inside(bi, bj, r))
                            v = *reinterpret_cast<const Words*>(src + static_cast<size_t>(accRow) * ldc + 8u * r + 4u * accGroup);
                        __builtin_memcpy(f.x + 4u * r, &v, sizeof(v));
                    }
                }
            };
            // 16-bit outputs with 16-wide blocks: a lane's run is only 8 bytes, a store instruction would
            // write 32-byte pieces.  Two neighbouring blocks are handled together: v_permlane16_swap
            // exchanges the second block's run of a lane in an even 16-lane row with the first block's
            // run of its partner in the next row, after which every lane owns 8 consecutive columns
            // (even rows: of the first block, odd rows: of the second) and moves 16 bytes; an
            // instruction then covers 64 contiguous bytes per matrix row.  The exchange is its own
            // inverse, so C is read the same way.
            constexpr bool PairIO = !Cfg::Edges && Cfg::Block == 16u && sizeof(OutT) == 2u && Cfg::BlocksN % 2u == 0u;
            const uint32_t pairCol = (accGroup & 1u) * 16u + 4u * (accGroup & 2u);
            auto           swapPair = [](auto& fx, auto& fy) {
                uint32_t x[2], y[2];
                __builtin_memcpy(x, fx.x, 8);
                __builtin_memcpy(y, fy.x, 8);
#pragma unroll
                for(uint32_t w = 0; w < 2u; ++w)
                {
                    auto r = __builtin_amdgcn_permlane16_swap(x[w], y[w], false, false);
                    x[w]   = r[0];
                    y[w]   = r[1];
                }
                __builtin_memcpy(fx.x, x, 8);
                __builtin_memcpy(fy.x, y, 8);
            };
            auto storePair = [&](OutT* dst, auto& fx, auto& fy, uint32_t ld) {
                swapPair(fx, fy);
                typedef uint32_t Words __attribute__((ext_vector_type(4)));
                Words            v;
                __builtin_memcpy(&v, fx.x, 8);
                __builtin_memcpy(reinterpret_cast<char*>(&v) + 8, fy.x, 8);
                *reinterpret_cast<Words*>(dst + static_cast<size_t>(accRow) * ld + pairCol) = v;
            };
            auto loadPair = [&](auto& fx, auto& fy, const OutT* src, uint32_t ld) {
                typedef uint32_t Words __attribute__((ext_vector_type(4)));
                const Words      v = *reinterpret_cast<const Words*>(src + static_cast<size_t>(accRow) * ld + pairCol);
                __builtin_memcpy(fx.x, &v, 8);
                __builtin_memcpy(fy.x, reinterpret_cast<const char*>(&v) + 8, 8);
                swapPair(fx, fy);
            };
            auto           blockOffset = [&](uint32_t bi, uint32_t bj, uint32_t ld) {
                return static_cast<size_t>(wRow + bi * Cfg::Block) * ld + wCol + bj * Cfg::Block;
            };
            // Fused configurations: the bias values of a lane's columns of one block are fetched (four
            // consecutive floats per run, cache hits after the first row of blocks) just before the
            // block's results go out; finish() is what every result passes through.
            static_assert(!Cfg::Fused || std::is_same<CompT, float>::value, "fused epilogue: f32 compute");
            struct BiasOfBlock
            {
                float v[Cfg::Fused ? 4u * Runs : 1u];
            };
            auto loadBias = [&](uint32_t bj) {
                BiasOfBlock bv = {};
                if constexpr(Cfg::Fused)
                {
                    if(ex.fused.bias)
                    {
#pragma unroll
                        for(uint32_t r = 0; r < Runs; ++r)
                        {
                            const uint32_t col = wCol + bj * Cfg::Block + 8u * r + 4u * accGroup;
                            if(!Cfg::Edges || col < n)
                                __builtin_memcpy(&bv.v[4u * r], ex.fused.bias + col, 16);
                        }
                    }
                }
                return bv;
            };
            // With 16-wide blocks a wave's bias values (four per block and lane) are few enough to be fetched once,
            // in front of everything else the epilogue requests, and kept for every row of blocks; fetched per
            // block, each load's latency sat in front of that block's stores (8192^3 f16 with a bias: +26 us,
            // hoisted: +3 us).  The 32-wide blocks (16 values per block and lane) keep the per-block loads: held
            // for all blocks they spilled.
            constexpr bool HoistBias = Cfg::Fused && 4u * Runs * Cfg::BlocksN <= 32u;
            BiasOfBlock    biasRow[HoistBias ? Cfg::BlocksN : 1u];
            if constexpr(HoistBias)
            {
#pragma unroll
                for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                    biasRow[bj] = loadBias(bj);
                __builtin_amdgcn_sched_barrier(0);
            }
            auto biasOf = [&](uint32_t bj) {
                if constexpr(HoistBias)
                    return biasRow[bj];
                else
                    return loadBias(bj);
            };
            auto finish = [&](BiasOfBlock const& bv, uint32_t e, CompT v) -> CompT {
                if constexpr(Cfg::Fused)
                    return applyActivation(v + bv.v[e], ex.fused.activation);
                else
                {
                    (void)bv, (void)e;
                    return v;
                }
            };
            if(beta != static_cast<CompT>(0))
            {
                if constexpr(Cfg::StagedC)
                {
                    // C reaches the accumulator layout through LDS: whole-wave direct copies
                    // fetch full rows of a 32-row group of GroupBlocks blocks (read in the
                    // accumulator layout straight from global memory, an instruction would touch
                    // 32 rows for 32 bytes each, at half the rate).  Row r is stored with its
                    // 16-byte chunks XOR-swizzled by r % 16 so that the 16 rows a quarter-wave
                    // reads at one chunk position fall into distinct bank groups.  The main-loop
                    // ring is free by now and every wave owns two group buffers in it.
                    constexpr uint32_t GB          = Cfg::GroupBlocks;
                    constexpr uint32_t RowBytes    = GB * Cfg::Block * sizeof(OutT); // 256 or 512
                    constexpr uint32_t GroupBytes  = Cfg::Block * RowBytes;
                    constexpr uint32_t RowChunks   = RowBytes / 16u;
                    constexpr uint32_t RowsPerCopy = 1024u / RowBytes;
                    constexpr uint32_t CopiesC     = GroupBytes / 1024u;
                    constexpr uint32_t StoresD     = GB * Runs; // 16-byte stores per group
                    constexpr uint32_t GroupsPerRow = Cfg::BlocksN / GB;
                    constexpr uint32_t NG          = Cfg::BlocksM * GroupsPerRow;
                    static_assert((RowBytes == 256u || RowBytes == 512u) && 2u * GroupBytes * Cfg::Waves <= Cfg::LdsBytes
                                      && NG >= 2u,
                                  "C staging geometry");
                    char*          myLds  = ldsRaw + wave * (2u * GroupBytes);
                    const char*    cWave  = reinterpret_cast<const char*>(c + static_cast<size_t>(wRow) * ldc + wCol);
                    const size_t   ldcB   = static_cast<size_t>(ldc) * sizeof(OutT);
                    const uint32_t cpRow  = lane / RowChunks; // row inside a copy
                    const uint32_t chunk  = lane % RowChunks; // chunk position inside the LDS row
                    auto           copyGroup = [&](uint32_t gi) {
                        const uint32_t bi = gi / GroupsPerRow, bj0 = (gi % GroupsPerRow) * GB;
#pragma unroll
                        for(uint32_t i = 0; i < CopiesC; ++i)
                        {
                            const uint32_t r = RowsPerCopy * i + cpRow;
                            lds::asyncCopy16Streaming(myLds + (gi % 2u) * GroupBytes + i * 1024u,
                                                      cWave + (bi * Cfg::Block + r) * ldcB + bj0 * Cfg::Block * sizeof(OutT)
                                                          + ((chunk ^ (r & 15u)) << 4));
                        }
                    };
                    const uint32_t rdRow  = accRow;
                    const uint32_t rdBase = rdRow * RowBytes;
                    copyGroup(0u);
                    copyGroup(1u);
#pragma unroll
                    for(uint32_t gi = 0; gi < NG; ++gi)
                    {
                        const uint32_t bi = gi / GroupsPerRow, bj0 = (gi % GroupsPerRow) * GB;
                        // vector-memory operations younger than this group's copies: the next
                        // group's copies and the stores of the two previous groups
                        if(gi == 0u)
                            lds::waitCopiesAndReads<CopiesC>();
                        else if(gi == 1u)
                            lds::waitCopiesAndReads<(NG > 2u ? CopiesC : 0u) + StoresD>();
                        else if(gi + 1u < NG)
                            lds::waitCopiesAndReads<CopiesC + 2u * StoresD>();
                        else
                            lds::waitCopiesAndReads<2u * StoresD>();
                        asm volatile("" ::: "memory");
                        typename Cfg::FragC io[GB];
#pragma unroll
                        for(uint32_t bj = 0; bj < GB; ++bj)
#pragma unroll
                            for(uint32_t r = 0; r < Runs; ++r)
                            {
                                // logical chunk of this run: block bj holds Block / 4 chunks per row
                                const uint32_t g = bj * (Cfg::Block / 4u) + 2u * r + accGroup;
                                detail::copyBytes<16u>(io[bj].x + 4u * r,
                                                       myLds + (gi % 2u) * GroupBytes + rdBase + ((g ^ (rdRow & 15u)) << 4));
                            }
                        if(gi + 2u < NG)
                        {
                            lds::waitReads(); // the buffer is overwritten next
                            asm volatile("" ::: "memory");
                            copyGroup(gi + 2u);
                        }
#pragma unroll
                        for(uint32_t bj = 0; bj < GB; ++bj)
                        {
                            const BiasOfBlock bv = biasOf(bj0 + bj);
#pragma unroll
                            for(uint32_t e = 0; e < io[bj].num_elements; ++e)
                                acc[bi][bj0 + bj].x[e]
                                    = finish(bv, e, alpha * acc[bi][bj0 + bj].x[e] + beta * static_cast<CompT>(io[bj].x[e]));
                        }
                        // (results replace the accumulators: every store has registers of its own)
#pragma unroll
                        for(uint32_t bj = 0; bj < GB; ++bj)
                            storeBlock(bi, bj0 + bj, acc[bi][bj0 + bj]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                else
                {
                typename Cfg::FragC fc[2][Cfg::BlocksN];
                auto                loadGroup = [&](uint32_t bi) {
                    if constexpr(PairIO)
                    {
#pragma unroll
                        for(uint32_t bj = 0; bj < Cfg::BlocksN; bj += 2u)
                            loadPair(fc[bi % 2u][bj], fc[bi % 2u][bj + 1u], c + blockOffset(bi, bj, ldc), ldc);
                    }
                    else
                    {
#pragma unroll
                        for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                            loadBlockC(bi, bj, fc[bi % 2u][bj]);
                    }
                };
                loadGroup(0u);
                if constexpr(Cfg::BlocksM > 1u)
                    loadGroup(1u);
#pragma unroll
                for(uint32_t bi = 0; bi < Cfg::BlocksM; ++bi)
                {
#pragma unroll
                    for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                    {
                        auto& io = fc[bi % 2u][bj];
                        const BiasOfBlock bv = biasOf(bj);
#pragma unroll
                        for(uint32_t e = 0; e < io.num_elements; ++e)
                            io.x[e] = static_cast<OutT>(finish(bv, e, alpha * acc[bi][bj].x[e] + beta * static_cast<CompT>(io.x[e])));
                    }
                    if constexpr(PairIO)
                    {
#pragma unroll
                        for(uint32_t bj = 0; bj < Cfg::BlocksN; bj += 2u)
                            storePair(d + blockOffset(bi, bj, ldd), fc[bi % 2u][bj], fc[bi % 2u][bj + 1u], ldd);
                    }
                    else
                    {
#pragma unroll
                        for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                            storeBlock(bi, bj, fc[bi % 2u][bj]);
                    }
                    if(bi + 2u < Cfg::BlocksM)
                        loadGroup(bi + 2u);
                    __builtin_amdgcn_sched_barrier(0);
                }
                }
            }
            else
            {
#pragma unroll
                for(uint32_t bi = 0; bi < Cfg::BlocksM; ++bi)
                {
                    if constexpr(std::is_same<OutT, CompT>::value)
                    {
                        // results replace the accumulators, so no two stores share data registers
                        // (with alpha = 1 they go out as they are: a 32-bit integer multiply runs at a quarter of the
                        // rate of the other vector instructions, 128 of them per lane and tile)
                        if(Cfg::Fused || alpha != static_cast<CompT>(1))
                        {
#pragma unroll
                            for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                            {
                                const BiasOfBlock bv = biasOf(bj);
#pragma unroll
                                for(uint32_t e = 0; e < acc[bi][bj].num_elements; ++e)
                                    acc[bi][bj].x[e] = finish(bv, e, alpha * acc[bi][bj].x[e]);
                            }
                        }
#pragma unroll
                        for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                            storeBlock(bi, bj, acc[bi][bj]);
                    }
                    else
                    {
                        typename Cfg::FragC fd[Cfg::BlocksN];
#pragma unroll
                        for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                        {
                            const BiasOfBlock bv = biasOf(bj);
#pragma unroll
                            for(uint32_t e = 0; e < fd[bj].num_elements; ++e)
                                fd[bj].x[e] = static_cast<OutT>(finish(bv, e, alpha * acc[bi][bj].x[e]));
                        }
                        if constexpr(PairIO)
                        {
#pragma unroll
                            for(uint32_t bj = 0; bj < Cfg::BlocksN; bj += 2u)
                                storePair(d + blockOffset(bi, bj, ldd), fd[bj], fd[bj + 1u], ldd);
                        }
                        else
                        {
#pragma unroll
                            for(uint32_t bj = 0; bj < Cfg::BlocksN; ++bj)
                                storeBlock(bi, bj, fd[bj]);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }

    } // namespace
} // namespace rocwmma_amd

#endif // ROCWMMA_AMD_CSRC_GEMM_BLOCKED_CORE_HPP
