// extern "C" entry points of librocwmma_amd_aux.so (test and benchmark support; declarations in
// include/rocwmma_amd_aux.h).
#include "common.hpp"
#include <rocwmma_amd_aux.h>

#include <cstring>

namespace rocwmma_amd
{
    int selftestRoundtrip(int context, int dtype, int layout, int block, int blockk, int coop, uint32_t rows, uint32_t cols,
                          const void* in, void* out, uint32_t ld, hipStream_t stream);
    int selftestTiledGemm(int layoutA, int layoutB, uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b, const float* c,
                          float* d, float alpha, float beta, hipStream_t stream);
    int selftestCoopGemm(int layoutA, int layoutB, uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b,
                         const float* c, float* d, float alpha, float beta, hipStream_t stream);
    int benchMfmaCeiling(int shape, uint32_t trips, uint32_t wavesPerSimd, const void* operands, float* out, double* ops,
                         hipStream_t stream);
    int benchStream(int mode, const void* src, void* dst, size_t bytes, hipStream_t stream);
    int benchMfmaStreams(int kind, int streams, uint32_t tilesPerWorkgroup, const void* a, const void* b, const void* operands, float* out,
                         double* ops, hipStream_t stream);

    namespace
    {
        bool validLayout(int l)
        {
            return l == ROCWMMA_AMD_ROW_MAJOR || l == ROCWMMA_AMD_COL_MAJOR;
        }

        bool isGfx950Current()
        {
            // (asked once per call: these entry points are not on anyone's hot path)
            int dev = 0;
            if(hipGetDevice(&dev) != hipSuccess)
                return false;
            hipDeviceProp_t props;
            if(hipGetDeviceProperties(&props, dev) != hipSuccess)
                return false;
            return std::strncmp(props.gcnArchName, "gfx950", 6) == 0;
        }
    } // namespace
} // namespace rocwmma_amd

using namespace rocwmma_amd;

extern "C" {

int rocwmma_amd_selftest_roundtrip(int         context,
                                   int         dtype,
                                   int         layout,
                                   int         block,
                                   int         blockk,
                                   int         coop,
                                   uint32_t    rows,
                                   uint32_t    cols,
                                   const void* in,
                                   void*       out,
                                   uint32_t    ld,
                                   void*       stream)
{
    if(!in || !out || rows == 0u || cols == 0u || !validLayout(layout))
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(!aligned16(in) || !aligned16(out) || (ld * dtypeSize(dtype)) % 16u != 0u)
        return ROCWMMA_AMD_BAD_ALIGNMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    return selftestRoundtrip(context, dtype, layout, block, blockk, coop, rows, cols, in, out, ld, asStream(stream));
}

int rocwmma_amd_selftest_coop_gemm(int          layout_a,
                                   int          layout_b,
                                   uint32_t     m,
                                   uint32_t     n,
                                   uint32_t     k,
                                   const void*  a,
                                   const void*  b,
                                   const float* c,
                                   float*       d,
                                   float        alpha,
                                   float        beta,
                                   void*        stream)
{
    if(!a || !b || !c || !d || !validLayout(layout_a) || !validLayout(layout_b))
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    return selftestCoopGemm(layout_a, layout_b, m, n, k, a, b, c, d, alpha, beta, asStream(stream));
}

int rocwmma_amd_selftest_tiled_gemm(int          layout_a,
                                    int          layout_b,
                                    uint32_t     m,
                                    uint32_t     n,
                                    uint32_t     k,
                                    const void*  a,
                                    const void*  b,
                                    const float* c,
                                    float*       d,
                                    float        alpha,
                                    float        beta,
                                    void*        stream)
{
    if(!a || !b || !c || !d || !validLayout(layout_a) || !validLayout(layout_b))
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(!aligned16(a) || !aligned16(b) || !aligned16(c) || !aligned16(d))
        return ROCWMMA_AMD_BAD_ALIGNMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    return selftestTiledGemm(layout_a, layout_b, m, n, k, a, b, c, d, alpha, beta, asStream(stream));
}

int rocwmma_amd_bench_mfma_ceiling(int         shape,
                                   uint32_t    trips,
                                   uint32_t    waves_per_simd,
                                   const void* operands,
                                   float*      out,
                                   double*     ops,
                                   void*       stream)
{
    if(!operands || !out)
        return ROCWMMA_AMD_INVALID_ARGUMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    return benchMfmaCeiling(shape, trips, waves_per_simd, operands, out, ops, asStream(stream));
}

int rocwmma_amd_bench_mfma_streams(int         kind,
                                   int         streams,
                                   uint32_t    tiles_per_workgroup,
                                   const void* a,
                                   const void* b,
                                   const void* operands,
                                   float*      out,
                                   double*     ops,
                                   void*       stream)
{
    if((a && !aligned16(a)) || (b && !aligned16(b)) || !aligned16(operands) || !aligned16(out))
        return ROCWMMA_AMD_BAD_ALIGNMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    return benchMfmaStreams(kind, streams, tiles_per_workgroup, a, b, operands, out, ops, asStream(stream));
}

int rocwmma_amd_bench_stream(int mode, const void* src, void* dst, size_t bytes, void* stream)
{
    if((src && !aligned16(src)) || (dst && !aligned16(dst)))
        return ROCWMMA_AMD_BAD_ALIGNMENT;
    if(!isGfx950Current())
        return ROCWMMA_AMD_NO_DEVICE;
    return benchStream(mode, src, dst, bytes, asStream(stream));
}

} // extern "C"
