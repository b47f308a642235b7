// Memory-stream ceiling probe of librocwmma_amd_aux.so: plain kernels that only read, only write, or
// copy a buffer with 16-byte non-temporal accesses, several in flight per lane.  The bandwidth-bound
// workloads (GEMV, DLRM, the weight-streaming GEMMs) are priced against what these reach on the same
// device for the same number of bytes, next to the nominal HBM peak: at tens of megabytes a launch is
// over before the memory system reaches the rate of a long stream.
#include "common.hpp"

namespace rocwmma_amd
{
    namespace
    {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        constexpr uint32_t kStreamThreads = 256;
        constexpr uint32_t kStreamUnroll  = 8; // 16-byte accesses in flight per lane

        __global__ void __launch_bounds__(kStreamThreads) streamReadKernel(const u32x4* __restrict__ src, size_t vecs, uint32_t* sink)
        {
            size_t       i      = static_cast<size_t>(blockIdx.x) * kStreamThreads * kStreamUnroll + threadIdx.x;
            const size_t stride = static_cast<size_t>(gridDim.x) * kStreamThreads * kStreamUnroll;
            uint32_t     acc    = 0;
            for(; i + kStreamThreads * (kStreamUnroll - 1u) < vecs; i += stride)
            {
                u32x4 v[kStreamUnroll];
#pragma unroll
                for(uint32_t u = 0; u < kStreamUnroll; ++u)
                    v[u] = __builtin_nontemporal_load(src + i + u * kStreamThreads);
#pragma unroll
                for(uint32_t u = 0; u < kStreamUnroll; ++u)
                    acc += v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
            }
            if(acc == 0x12345678u) // (keeps the loads alive; practically never true)
                sink[0] = acc;
        }

        // Write and copy: workgroups of 1024 threads, four 16-byte accesses per lane and trip.  The variants were
        // swept over 1-16 accesses per lane, 256-1024 threads, 2-64 workgroups per compute unit and plain /
        // non-temporal accesses on 1.75 GiB: the write reaches most with plain stores and one workgroup per
        // compute unit (5.9 TB/s; one access per lane on 16 workgroups of 256 threads per unit: 4.0), the copy
        // with non-temporal loads and stores on 8 workgroups per unit (5.75 TB/s; plain stores, 256 threads: 5.0).
        constexpr uint32_t kWideThreads = 1024;
        constexpr uint32_t kWideUnroll  = 4;

        __global__ void __launch_bounds__(kWideThreads) streamWriteKernel(u32x4* __restrict__ dst, size_t vecs)
        {
            size_t       i      = static_cast<size_t>(blockIdx.x) * kWideThreads * kWideUnroll + threadIdx.x;
            const size_t stride = static_cast<size_t>(gridDim.x) * kWideThreads * kWideUnroll;
            const u32x4  v      = {1u, 2u, 3u, 4u};
            for(; i + kWideThreads * (kWideUnroll - 1u) < vecs; i += stride)
#pragma unroll
                for(uint32_t u = 0; u < kWideUnroll; ++u)
                    dst[i + u * kWideThreads] = v;
        }

        // ExtraReads: every tenth trip also reads a trip's worth of data that is not written anywhere (from the
        // `vecs` vectors behind the copied ones): 1.1 bytes read per byte written, the mix of the DLRM backward
        // pass (7870 bytes read, 7168 written per sample), which a plain 1 : 1 copy slightly under-prices because
        // reads are the cheaper half.
        template <bool ExtraReads>
        __global__ void __launch_bounds__(kWideThreads)
            streamCopyKernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t vecs, uint32_t* sink)
        {
            size_t       i      = static_cast<size_t>(blockIdx.x) * kWideThreads * kWideUnroll + threadIdx.x;
            const size_t stride = static_cast<size_t>(gridDim.x) * kWideThreads * kWideUnroll;
            uint32_t     acc    = 0;
            for(uint32_t trip = blockIdx.x; i + kWideThreads * (kWideUnroll - 1u) < vecs; i += stride, ++trip)
            {
                u32x4 v[kWideUnroll];
#pragma unroll
                for(uint32_t u = 0; u < kWideUnroll; ++u)
                    v[u] = __builtin_nontemporal_load(src + i + u * kWideThreads);
                if(ExtraReads && trip % 10u == 0u)
                {
#pragma unroll
                    for(uint32_t u = 0; u < kWideUnroll; ++u)
                    {
                        const u32x4 x = __builtin_nontemporal_load(src + vecs + i + u * kWideThreads);
                        acc += x[0] ^ x[1] ^ x[2] ^ x[3];
                    }
                }
#pragma unroll
                for(uint32_t u = 0; u < kWideUnroll; ++u)
                    __builtin_nontemporal_store(v[u], dst + i + u * kWideThreads);
            }
            if(ExtraReads && acc == 0x12345678u) // (keeps the extra loads alive; practically never true)
                sink[0] = acc;
        }

        // What a compute unit can draw from its XCD's L2: one workgroup of 1024 threads per 64 KiB chunk reads its own
        // chunk kResidentPasses times with plain 16-byte loads, all of the chunk in flight at once.  A chunk is twice
        // the vector L1, read cyclically, so every pass misses the L1; workgroup w runs on XCD w % 8, so with 16 MiB
        // (one workgroup per compute unit) every L2 holds 2 MiB of its 4: every pass after the first hits the L2.
        // The operand streams of the tiled kernels (GEMM, the tiled DLRM kernels, the M = 128 weight-streaming case)
        // are priced against this.
        constexpr uint32_t kResidentPasses = 256;
        constexpr size_t   kResidentChunkVecs = 65536u / 16u;

        __global__ void __launch_bounds__(kWideThreads) streamResidentReadKernel(const u32x4* __restrict__ src, uint32_t* sink)
        {
            const u32x4* mine = src + static_cast<size_t>(blockIdx.x) * kResidentChunkVecs + threadIdx.x;
            uint32_t     acc  = 0;
#pragma unroll 1
            for(uint32_t pass = 0; pass < kResidentPasses; ++pass)
            {
                const u32x4* from = mine;
                asm volatile("" : "+v"(from)); // (the same addresses every pass: keeps the loads inside the loop)
                u32x4 v[kWideUnroll];
#pragma unroll
                for(uint32_t u = 0; u < kWideUnroll; ++u)
                    v[u] = from[u * kWideThreads];
#pragma unroll
                for(uint32_t u = 0; u < kWideUnroll; ++u)
                    acc += v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
            }
            if(acc == 0x12345678u) // (keeps the loads alive; practically never true)
                sink[0] = acc;
        }
    } // namespace

    // mode 0: read `bytes` from src; 1: write `bytes` to dst; 2: copy `bytes` from src to dst; 3: copy with a tenth more reads;
    // 4: read `bytes` 256 times, cache resident.
    // bytes must be a multiple of 64 KiB (whole trips of the unrolled loops for every workgroup size used).
    int benchStream(int mode, const void* src, void* dst, size_t bytes, hipStream_t stream)
    {
        if(bytes == 0u || bytes % 65536u != 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const size_t   vecs = bytes / 16u;
        const uint32_t cus  = computeUnits();
        // enough workgroups to keep every compute unit's request queues full, but no more trips than data
        const size_t   perTrip = mode == 0 ? static_cast<size_t>(kStreamThreads) * kStreamUnroll : static_cast<size_t>(kWideThreads) * kWideUnroll;
        size_t         grid    = static_cast<size_t>(cus) * (mode == 0 ? 16u : (mode >= 2 ? 8u : 1u));
        if(grid > vecs / perTrip)
            grid = vecs / perTrip;
        if(grid == 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        switch(mode)
        {
        case 0:
            if(!src || !dst)
                return ROCWMMA_AMD_INVALID_ARGUMENT; // (dst: 4 bytes for the sink)
            hipLaunchKernelGGL(streamReadKernel, dim3(static_cast<uint32_t>(grid)), dim3(kStreamThreads), 0, stream,
                               static_cast<const u32x4*>(src), vecs, static_cast<uint32_t*>(dst));
            break;
        case 1:
            if(!dst)
                return ROCWMMA_AMD_INVALID_ARGUMENT;
            hipLaunchKernelGGL(streamWriteKernel, dim3(static_cast<uint32_t>(grid)), dim3(kWideThreads), 0, stream,
                               static_cast<u32x4*>(dst), vecs);
            break;
        case 2:
            if(!src || !dst)
                return ROCWMMA_AMD_INVALID_ARGUMENT;
            hipLaunchKernelGGL(streamCopyKernel<false>, dim3(static_cast<uint32_t>(grid)), dim3(kWideThreads), 0, stream,
                               static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), vecs, static_cast<uint32_t*>(nullptr));
            break;
        case 3: // copy `bytes` and read a tenth as much again from behind them (src holds 2 * bytes; 4 bytes of dst + bytes are the sink)
            if(!src || !dst)
                return ROCWMMA_AMD_INVALID_ARGUMENT;
            hipLaunchKernelGGL(streamCopyKernel<true>, dim3(static_cast<uint32_t>(grid)), dim3(kWideThreads), 0, stream,
                               static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), vecs,
                               reinterpret_cast<uint32_t*>(static_cast<char*>(dst) + bytes));
            break;
        case 4: // read every 64 KiB chunk of `bytes` kResidentPasses times, one workgroup per chunk (4 bytes of dst are the sink)
            if(!src || !dst)
                return ROCWMMA_AMD_INVALID_ARGUMENT;
            hipLaunchKernelGGL(streamResidentReadKernel, dim3(static_cast<uint32_t>(bytes / 65536u)), dim3(kWideThreads), 0, stream,
                               static_cast<const u32x4*>(src), static_cast<uint32_t*>(dst));
            break;
        default:
            return ROCWMMA_AMD_INVALID_ARGUMENT;
        }
        return launchStatus();
    }
} // namespace rocwmma_amd
