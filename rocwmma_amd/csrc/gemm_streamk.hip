// Blocked GEMM for gfx950 with the tile count balanced over the compute units ("stream-K").
//
// The one-tile-per-workgroup kernel (gemm_blocked.hip) runs its tiles in rounds of one tile per
// compute unit; a tile count that is not a multiple of the unit count leaves part of the machine
// idle in the last round (896 tiles on 256 units: 3.5 rounds run as 4; 144 tiles: 0.56 rounds run
// as 1).  Here one persistent workgroup per compute unit takes
//
//   * its share of the whole rounds, tile by tile in the same L2-friendly order, and
//   * an equal share of the K iterations of the remaining tiles, as a contiguous range of the
//     (tile, K stage) sequence: at most one part of a tile that starts behind K = 0 (run first:
//     the raw accumulators go to the workgroup's workspace slot and a flag goes up), whole tiles,
//     and at most one part that starts at K = 0 (run last: it waits for the flags of the parts
//     behind it, adds their slots in order and runs the epilogue).
//
// The sums are taken in a fixed order, so results do not change from run to run (int32 results are
// exact, f32 results differ from the one-tile kernel's only in the rounding of the partial sums).
// Deadlock freedom does not lean on the dispatcher's order: a workgroup draws a ticket from a counter
// in the workspace when it starts, and ranges are numbered against the tickets.  A part that waits
// looks only at ranges of workgroups with earlier tickets, which are therefore resident, and which
// compute the awaited part before anything else and without waiting for anyone: no workgroup waits for
// one that cannot run, whatever order the workgroups start in and whatever else occupies the device.
// (The whole rounds are dealt by workgroup id, which is what places a tile on an XCD.)  The owner's
// wait is bounded all the same; a wait that runs out leaves kStreamKTimedOut in the workspace, which
// rocwmma_amd_gemm_streamk_timed_out reports to the caller.  The reference's GEMM hosts have no
// counterpart (plain 2-D grids, samples/perf_hgemm.cpp:810-812).
#include "gemm_blocked_core.hpp"

using namespace rocwmma;

namespace rocwmma_amd
{
    namespace
    {
        template <typename Cfg>
        __global__ void __launch_bounds__(Cfg::Threads) __attribute__((amdgpu_waves_per_eu(Cfg::WavesPerSimd, Cfg::WavesPerSimd)))
        gemmStreamKKernel(uint32_t                   m,
                          uint32_t                   n,
                          uint32_t                   k,
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
                          char*                      slots,
                          uint32_t*                  flags,
                          uint32_t                   wholeRounds)
        {
            const uint32_t workgroups = gridDim.x;
            const uint32_t tilesM = m / Cfg::MacroM, tilesN = n / Cfg::MacroN; // (whole tiles: checked by the host)
            const uint32_t stagesPerTile = k / Cfg::MacroK;
            const uint32_t roundTiles    = wholeRounds * workgroups; // tile ids [0, roundTiles): one per workgroup and round
            const uint32_t splitTiles    = tilesM * tilesN - roundTiles; // tile ids behind them: shared by K range

            // this workgroup's range of the (split tile, stage) sequence; ranges are numbered against
            // the order the workgroups start in (a ticket drawn here), so the parts a range waits for
            // belong to workgroups that are already running
            extern __shared__ __attribute__((aligned(1024))) char ldsRaw[];
            if(threadIdx.x == 0u)
                *reinterpret_cast<uint32_t*>(ldsRaw)
                    = __hip_atomic_fetch_add(flags + workgroups + 1u, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            const uint32_t ticket = __builtin_amdgcn_readfirstlane(*reinterpret_cast<const uint32_t*>(ldsRaw));
            __syncthreads(); // (the first copies overwrite the word)
            const uint32_t range = workgroups - 1u - ticket;
            const uint64_t units = static_cast<uint64_t>(splitTiles) * stagesPerTile;
            auto           rangeStart = [&](uint32_t r) { return static_cast<uint32_t>(units * r / workgroups); };
            uint32_t       u    = rangeStart(range);
            const uint32_t uEnd = rangeStart(range + 1u);

            StreamKPart sk{};
            sk.slots       = slots;
            sk.flags       = flags;
            sk.slotBytes   = Cfg::MacroM * Cfg::MacroN * static_cast<uint32_t>(sizeof(typename Cfg::CompT));
            sk.timeoutWord = workgroups;

            auto tileOf = [&](uint32_t id, uint32_t& tm, uint32_t& tn) { tileOfWorkgroup(id, tilesM, tilesN, tm, tn); };
            uint32_t tm, tn;

            // 1. a part that starts behind K = 0: first, so that its owner finds it ready
            if(u < uEnd && u % stagesPerTile != 0u)
            {
                const uint32_t stage0 = u % stagesPerTile;
                const uint32_t count  = min(stagesPerTile - stage0, uEnd - u);
                tileOf(roundTiles + u / stagesPerTile, tm, tn);
                sk.mySlot = range;
                gemmTile<Cfg, TilePart::Contributor>(tm, tn, stage0, count, m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta, sk);
                u += count;
                __syncthreads(); // the next tile's copies reuse the LDS
            }
            // 2. the whole rounds
            for(uint32_t r = 0; r < wholeRounds; ++r)
            {
                tileOf(r * workgroups + blockIdx.x, tm, tn);
                gemmTile<Cfg>(tm, tn, 0u, stagesPerTile, m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta, sk);
                __syncthreads();
            }
            // 3. the rest of the range: whole split tiles, then a part that starts at K = 0
            while(u < uEnd)
            {
                const uint32_t count = min(stagesPerTile, uEnd - u);
                tileOf(roundTiles + u / stagesPerTile, tm, tn);
                if(count == stagesPerTile)
                    gemmTile<Cfg>(tm, tn, 0u, stagesPerTile, m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta, sk);
                else
                {
                    // the parts behind this one: the ranges that start before the tile ends
                    const uint32_t tileEnd = u + stagesPerTile;
                    sk.firstSlot           = range + 1u;
                    sk.slotCount           = 0u;
                    while(sk.firstSlot + sk.slotCount < workgroups && rangeStart(sk.firstSlot + sk.slotCount) < tileEnd)
                        ++sk.slotCount;
                    gemmTile<Cfg, TilePart::Owner>(tm, tn, 0u, count, m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta, sk);
                }
                u += count;
                __syncthreads();
            }
        }

        // Clears the flags and the ticket counter of a launch, not the time-out marker between them (a later
        // launch must not hide an earlier failure: the query clears it).  A kernel, not a memset: the
        // entry points may be recorded into a HIP graph.
        __global__ void clearFlagsKernel(uint32_t* flags, uint32_t workgroups)
        {
            for(uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < workgroups + 2u; i += gridDim.x * blockDim.x)
                if(i != workgroups)
                    flags[i] = 0u;
        }

        // The 256 x 256 configurations of the one-tile kernel (ring of two 128-byte K stages).
        template <typename InT, typename OutT, typename CompT, bool AK, bool BK>
        using BigConfig = std::conditional_t<sizeof(InT) == 2u || std::is_same<InT, int8_t>::value,
                                             BlockedConfig<InT, OutT, CompT, AK, BK, 4, 2, 4, 8, 2, 2, 16>,
                                             BlockedConfig<InT, OutT, CompT, AK, BK, 4, 2, 2, 4, 2, 2, 32>>;

        template <typename Cfg>
        int launchStreamK(GemmArgs const& g, void* workspace, size_t workspaceBytes, hipStream_t stream)
        {
            if(g.m % Cfg::MacroM != 0u || g.n % Cfg::MacroN != 0u || g.k % Cfg::MacroK != 0u)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            {
                const uint64_t spanA = static_cast<uint64_t>(g.lda) * sizeof(typename Cfg::InT) * (Cfg::AKMajor ? Cfg::MacroM : Cfg::MacroK);
                const uint64_t spanB = static_cast<uint64_t>(g.ldb) * sizeof(typename Cfg::InT) * (Cfg::BKMajor ? Cfg::MacroN : Cfg::MacroK);
                if(spanA >= 0x7FFF0000ull || spanB >= 0x7FFF0000ull)
                    return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            }
            const uint32_t tiles      = (g.m / Cfg::MacroM) * (g.n / Cfg::MacroN);
            const uint32_t stages     = g.k / Cfg::MacroK;
            const uint32_t workgroups = computeUnits(); // one persistent workgroup per compute unit
            uint32_t       wholeRounds = tiles / workgroups;
            // few tiles left over: a whole round joins them, so that a tile is shared by two or three
            // workgroups rather than by many
            if(wholeRounds > 0u && 2u * (tiles % workgroups) < workgroups)
                --wholeRounds;
            // every workgroup needs at least one stage of the shared tiles (a range without stages
            // would be waited for and never report)
            if(static_cast<uint64_t>(tiles - wholeRounds * workgroups) * stages < workgroups)
                return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
            const size_t need = streamKWorkspaceBytes(workgroups);
            if(!workspace || workspaceBytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0u)
                return ROCWMMA_AMD_INVALID_ARGUMENT;
            char*     slots = static_cast<char*>(workspace);
            uint32_t* flags = reinterpret_cast<uint32_t*>(slots + static_cast<size_t>(workgroups) * kStreamKSlotBytes);

            auto kernel = gemmStreamKKernel<Cfg>;
            if(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   static_cast<int>(Cfg::LdsBytes))
               != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
            hipLaunchKernelGGL(clearFlagsKernel, dim3(1), dim3(256), 0, stream, flags, workgroups);
            hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(Cfg::Threads), Cfg::LdsBytes, stream, g.m, g.n, g.k,
                               static_cast<typename Cfg::InT const*>(g.a), static_cast<typename Cfg::InT const*>(g.b),
                               static_cast<typename Cfg::OutT const*>(g.c), static_cast<typename Cfg::OutT*>(g.d), g.lda, g.ldb,
                               g.ldc, g.ldd, static_cast<typename Cfg::CompT>(g.alpha), static_cast<typename Cfg::CompT>(g.beta),
                               slots, flags, wholeRounds);
            return launchStatus();
        }

        template <typename InT, typename OutT, typename CompT>
        int pickLayouts(int layoutA, int layoutB, GemmArgs const& g, void* ws, size_t wsBytes, hipStream_t stream)
        {
            const bool ak = layoutA == ROCWMMA_AMD_ROW_MAJOR;
            const bool bk = layoutB == ROCWMMA_AMD_COL_MAJOR;
            if(ak && !bk)
                return launchStreamK<BigConfig<InT, OutT, CompT, true, false>>(g, ws, wsBytes, stream);
            if(!ak && bk)
                return launchStreamK<BigConfig<InT, OutT, CompT, false, true>>(g, ws, wsBytes, stream);
            if(!ak && !bk)
                return launchStreamK<BigConfig<InT, OutT, CompT, false, false>>(g, ws, wsBytes, stream);
            return launchStreamK<BigConfig<InT, OutT, CompT, true, true>>(g, ws, wsBytes, stream);
        }
    } // namespace

    // ---- the library's own scratch, for callers that cannot allocate ---------------------------
    // A workspace for devices of up to 256 compute units, held by every device the library runs on
    // until the process ends.  Host code never uses the array's name as an address: the device
    // address is asked for once per device (hipGetSymbolAddress) and kept.
    namespace
    {
        constexpr uint32_t kScratchWorkgroups = 256u;
        constexpr size_t   kScratchBytes = static_cast<size_t>(kScratchWorkgroups) * kStreamKSlotBytes + 1280u; // slots + 258 words (flags, marker, tickets)
        __device__ __align__(256) unsigned char scratch[kScratchBytes];

        void* scratchOfCurrentDevice()
        {
            constexpr int             kMaxDevices = 64;
            static std::atomic<void*> known[kMaxDevices];
            int                       dev = 0;
            if(hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
                return nullptr;
            void* ptr = known[dev].load(std::memory_order_acquire);
            if(ptr)
                return ptr;
            if(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr)
                return nullptr;
            known[dev].store(ptr, std::memory_order_release);
            return ptr;
        }
    } // namespace

    int launchGemmStreamKStatic(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& g, hipStream_t stream)
    {
        if(streamKWorkspaceBytes(computeUnits()) > kScratchBytes)
            return ROCWMMA_AMD_SCRATCH_TOO_SMALL;
        void* ptr = scratchOfCurrentDevice();
        if(!ptr)
            return ROCWMMA_AMD_LAUNCH_FAILED;
        return launchGemmStreamK(dtypeIn, dtypeOut, layoutA, layoutB, g, ptr, kScratchBytes, stream);
    }

    size_t streamKWorkspaceBytes(uint32_t workgroups)
    {
        // slots, then the flags, the time-out marker and the ticket counter, rounded to 256 bytes
        return static_cast<size_t>(workgroups) * kStreamKSlotBytes + ((static_cast<size_t>(workgroups) + 2u) * 4u + 255u) / 256u * 256u;
    }

    int streamKTimedOut(void* workspace, size_t workspaceBytes, hipStream_t stream, int* timedOut)
    {
        const uint32_t workgroups = computeUnits();
        if(!workspace)
        {
            if(streamKWorkspaceBytes(workgroups) > kScratchBytes)
                return ROCWMMA_AMD_SCRATCH_TOO_SMALL;
            workspace      = scratchOfCurrentDevice();
            workspaceBytes = kScratchBytes;
            if(!workspace)
                return ROCWMMA_AMD_LAUNCH_FAILED;
        }
        if(workspaceBytes < streamKWorkspaceBytes(workgroups))
            return ROCWMMA_AMD_INVALID_ARGUMENT;
        uint32_t* marker = reinterpret_cast<uint32_t*>(static_cast<char*>(workspace) + static_cast<size_t>(workgroups) * kStreamKSlotBytes)
                           + workgroups;
        uint32_t word = 0u;
        if(hipStreamSynchronize(stream) != hipSuccess || hipMemcpy(&word, marker, sizeof(word), hipMemcpyDeviceToHost) != hipSuccess)
            return ROCWMMA_AMD_LAUNCH_FAILED;
        *timedOut = word == kStreamKTimedOut ? 1 : 0;
        if(word == kStreamKTimedOut) // reported once
        {
            const uint32_t zero = 0u;
            if(hipMemcpy(marker, &zero, sizeof(zero), hipMemcpyHostToDevice) != hipSuccess)
                return ROCWMMA_AMD_LAUNCH_FAILED;
        }
        return ROCWMMA_AMD_OK;
    }

    int launchGemmStreamK(int dtypeIn, int dtypeOut, int layoutA, int layoutB, GemmArgs const& g, void* workspace,
                          size_t workspaceBytes, hipStream_t stream)
    {
        if(g.layoutC != ROCWMMA_AMD_ROW_MAJOR)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE; // caller transposes the problem first
        if(dtypeIn == ROCWMMA_AMD_F16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayouts<float16_t, float32_t, float32_t>(layoutA, layoutB, g, workspace, workspaceBytes, stream);
        if(dtypeIn == ROCWMMA_AMD_BF16 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayouts<bfloat16_t, float32_t, float32_t>(layoutA, layoutB, g, workspace, workspaceBytes, stream);
        if(dtypeIn == ROCWMMA_AMD_I8 && dtypeOut == ROCWMMA_AMD_I32)
            return pickLayouts<int8_t, int32_t, int32_t>(layoutA, layoutB, g, workspace, workspaceBytes, stream);
        if(dtypeIn == ROCWMMA_AMD_E4M3 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayouts<float8_t, float32_t, float32_t>(layoutA, layoutB, g, workspace, workspaceBytes, stream);
        if(dtypeIn == ROCWMMA_AMD_E5M2 && dtypeOut == ROCWMMA_AMD_F32)
            return pickLayouts<bfloat8_t, float32_t, float32_t>(layoutA, layoutB, g, workspace, workspaceBytes, stream);
        return ROCWMMA_AMD_UNSUPPORTED_TYPE;
    }

} // namespace rocwmma_amd
