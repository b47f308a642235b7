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

        __global__ void __launch_bounds__(kStreamThreads) streamWriteKernel(u32x4* __restrict__ dst, size_t vecs)
        {
            size_t       i      = static_cast<size_t>(blockIdx.x) * kStreamThreads + threadIdx.x;
            const size_t stride = static_cast<size_t>(gridDim.x) * kStreamThreads;
            const u32x4  v      = {1u, 2u, 3u, 4u};
            for(; i < vecs; i += stride)
                dst[i] = v;
        }

        __global__ void __launch_bounds__(kStreamThreads)
            streamCopyKernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t vecs)
        {
            constexpr uint32_t U      = 4;
            size_t             i      = static_cast<size_t>(blockIdx.x) * kStreamThreads * U + threadIdx.x;
            const size_t       stride = static_cast<size_t>(gridDim.x) * kStreamThreads * U;
            for(; i + kStreamThreads * (U - 1u) < vecs; i += stride)
            {
                u32x4 v[U];
#pragma unroll
                for(uint32_t u = 0; u < U; ++u)
                    v[u] = __builtin_nontemporal_load(src + i + u * kStreamThreads);
#pragma unroll
                for(uint32_t u = 0; u < U; ++u)
                    dst[i + u * kStreamThreads] = v[u];
            }
        }
    } // namespace

    // mode 0: read `bytes` from src; 1: write `bytes` to dst; 2: copy `bytes` from src to dst.
    // bytes must be a multiple of 32 KiB (whole trips of the unrolled loops for every workgroup size used).
    int benchStream(int mode, const void* src, void* dst, size_t bytes, hipStream_t stream)
    {
        if(bytes == 0u || bytes % 32768u != 0u)
            return ROCWMMA_AMD_UNSUPPORTED_SHAPE;
        const size_t   vecs = bytes / 16u;
        const uint32_t cus  = computeUnits();
        // enough workgroups to keep every compute unit's request queues full, but no more trips than data
        const size_t   perTrip = static_cast<size_t>(kStreamThreads) * (mode == 0 ? kStreamUnroll : (mode == 2 ? 4u : 1u));
        size_t         grid    = static_cast<size_t>(cus) * 16u;
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
            hipLaunchKernelGGL(streamWriteKernel, dim3(static_cast<uint32_t>(grid)), dim3(kStreamThreads), 0, stream,
                               static_cast<u32x4*>(dst), vecs);
            break;
        case 2:
            if(!src || !dst)
                return ROCWMMA_AMD_INVALID_ARGUMENT;
            hipLaunchKernelGGL(streamCopyKernel, dim3(static_cast<uint32_t>(grid)), dim3(kStreamThreads), 0, stream,
                               static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), vecs);
            break;
        default:
            return ROCWMMA_AMD_INVALID_ARGUMENT;
        }
        return launchStatus();
    }
} // namespace rocwmma_amd
