/*
 * rocwmma_amd_aux.h -- C ABI of librocwmma_amd_aux.so: test and benchmark support that is not part
 * of the product library (librocwmma_amd.so, rocwmma_amd.h).
 *
 *   - the device side of the fragment-API semantics tests: tiny kernels written only against the
 *     public rocwmma:: device API, launched from the host tests;
 *   - measurement probes the benchmark reports beside its kernels: a loop of nothing but matrix
 *     instructions (what the matrix pipes sustain under the board's power management), and a
 *     blocked GEMM written with the public fragment API only.
 *
 * Same conventions as rocwmma_amd.h: device pointers owned by the caller, work enqueued on
 * `stream`, a rocwmma_amd_status is returned.
 */
#ifndef ROCWMMA_AMD_AUX_H
#define ROCWMMA_AMD_AUX_H

#include "rocwmma_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Fragment API self-tests (device side of the API-semantics tests; each launches a tiny kernel
 * written only with the public rocwmma:: API and returns a status).
 *
 * rocwmma_amd_selftest_roundtrip: out = store(load(in)) for one fragment kind; mirrors the
 * reference unit test test/unit/load_store_matrix_sync_test/device/load_store_matrix_sync.hpp:35-117
 * (and, with coop != 0, the cooperative twin load_store_matrix_coop_sync_test).
 *   context : 0 matrix_a, 1 matrix_b, 2 accumulator
 *   `in`/`out` are rows x cols matrices of `dtype` in `layout` with leading dimension ld; the
 *   grid covers the matrix with one fragment per wave (or per workgroup of 4 waves when coop).
 *   block   : 16 or 32 (BlockM = BlockN), blockk : K extent of the fragment.
 */
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
                                   void*       stream);

/* Runs the reference's perf_hgemm data flow (cooperative global read -> applyDataLayout /
 * applyTranspose -> cooperative LDS write -> LDS read -> mma_sync) written only against the
 * public API, f16 in / f32 out, for the four A/B layout combinations.  Used to test the
 * cooperative and transform API end to end. */
int rocwmma_amd_selftest_coop_gemm(int         layout_a,
                                   int         layout_b,
                                   uint32_t    m,
                                   uint32_t    n,
                                   uint32_t    k,
                                   const void* a,
                                   const void* b,
                                   const float* c,
                                   float*      d,
                                   float       alpha,
                                   float       beta,
                                   void*       stream);

/* A blocked GEMM written only against the public API and laid out for gfx950 instead of after perf_hgemm
 * (256 x 256 macro tile, eight waves of 64 x 128, 16 x 16 x 32 blocks, K stages of 64 in two padded LDS buffers,
 * the next stage prefetched with cooperative loads), f16 in / f32 out, the four A/B layout combinations, row-major
 * C / D with leading dimension n; m, n multiples of 256, k a multiple of 64.  What a kernel ported to this device
 * reaches through the fragment API alone; the benchmark reports it next to the perf_hgemm data flow above. */
int rocwmma_amd_selftest_tiled_gemm(int         layout_a,
                                    int         layout_b,
                                    uint32_t    m,
                                    uint32_t    n,
                                    uint32_t    k,
                                    const void* a,
                                    const void* b,
                                    const float* c,
                                    float*      d,
                                    float       alpha,
                                    float       beta,
                                    void*       stream);

/* Instruction shapes of rocwmma_amd_bench_mfma_ceiling. */
typedef enum rocwmma_amd_mfma_shape
{
    ROCWMMA_AMD_MFMA_F16_16X16X32  = 0,
    ROCWMMA_AMD_MFMA_F16_32X32X16  = 1,
    ROCWMMA_AMD_MFMA_BF16_16X16X32 = 2,
    ROCWMMA_AMD_MFMA_BF16_32X32X16 = 3,
    ROCWMMA_AMD_MFMA_I8_16X16X64   = 4,
    ROCWMMA_AMD_MFMA_I8_32X32X32   = 5,
    ROCWMMA_AMD_MFMA_F8_16X16X128  = 6, /* v_mfma_f32_16x16x128_f8f6f4 on e4m3 operands */
    ROCWMMA_AMD_MFMA_F8_32X32X64   = 7,
    ROCWMMA_AMD_MFMA_F8_16X16X128_SCALED = 8 /* the same instruction with per-lane block scales */
} rocwmma_amd_mfma_shape;

/*
 * Matrix-pipe ceiling probe: every SIMD of the device runs `waves_per_simd` (1 or 2) waves that
 * issue nothing but matrix instructions of `shape` on operands held in registers, 32 instructions
 * per trip, `trips` trips.  The operand registers are filled from `operands`, a 64 KiB table of
 * operand bits the caller chooses (all zero, or the bit patterns of the data distribution of
 * interest): the sustained rate depends on them because the part is power managed.
 * `out` receives one float per launched lane (256 x waves_per_simd x compute units).  *ops is set
 * to the number of floating-point (integer) operations of the launch (2 per multiply-add).
 * Has no counterpart in the reference, whose efficiency figure divides by a nominal peak
 * (test/performance.hpp:435-442).
 */
int rocwmma_amd_bench_mfma_ceiling(int         shape,
                                   uint32_t    trips,
                                   uint32_t    waves_per_simd,
                                   const void* operands,
                                   float*      out,
                                   double*     ops,
                                   void*       stream);

/*
 * Matrix pipes next to their operand streams: what the device sustains when the matrix instructions of a
 * 256 x 256 tile (eight waves of 64 x 128 per compute unit) run next to the byte streams such a tile needs per
 * 128 bytes of K, and nothing else: no barrier, no tile bookkeeping, no epilogue.  kind = 0: 16-bit operands
 * (v_mfma_f32_16x16x32_f16), 1: int8 (v_mfma_i32_16x16x64_i8), 2: fp8 (v_mfma_f32_16x16x128_f8f6f4, B fragments
 * streamed through column buffers as in the kernel).  streams = 0: matrix instructions only; 1: with the
 * 192 KiB of fragment reads from LDS per stage; 3: with those and the 64 KiB of global -> LDS copies per stage,
 * walking the A / B panels in the tile order of an 8192 x 8192 problem with 16 KiB of K per row (K = 8192 halves or
 * 16384 bytes).  `a`, `b`: 8192 rows of 16 KiB each, K contiguous (needed for streams = 3); `operands`: a
 * 64 KiB table of operand bits as for rocwmma_amd_bench_mfma_ceiling; `out`: 512 floats per compute unit;
 * tiles_per_workgroup: tiles (of 128 stages) each compute unit walks, at most 1024 / compute units; *ops: the
 * operations of the launch.  On a power-managed part each stream costs clock: the blocked GEMM is priced against
 * this figure next to the matrix-pipe ceiling and the nominal peak.  Has no counterpart in the reference.
 */
int rocwmma_amd_bench_mfma_streams(int         kind,
                                   int         streams,
                                   uint32_t    tiles_per_workgroup,
                                   const void* a,
                                   const void* b,
                                   const void* operands,
                                   float*      out,
                                   double*     ops,
                                   void*       stream);

/*
 * Memory-stream ceiling probe: one plain kernel that reads (mode 0), writes (mode 1) or copies (mode 2)
 * `bytes` bytes (a multiple of 64 KiB) with 16-byte accesses (reads: 16 workgroups of 256 threads per compute
 * unit; writes and copies: workgroups of 1024 threads; each tuned by a sweep over accesses per lane, workgroup
 * size and count, plain / non-temporal accesses).  mode 0 reads `src` (and needs 4 writable bytes at `dst`),
 * mode 1 writes `dst`, mode 2 copies `src` to `dst`, mode 3 copies `src` to `dst` and reads a tenth as much again
 * from the `bytes` bytes behind `src`'s first `bytes` (so `src` holds 2 * bytes; 4 writable bytes behind `dst`'s
 * `bytes`): 1.1 bytes read per byte written, the mix of the DLRM backward pass.  The bandwidth-bound workloads
 * are priced against what this reaches for their byte counts on the same device.  mode 4 reads `src`'s `bytes`
 * ROCWMMA_AMD_STREAM_RESIDENT_PASSES times over, one workgroup of 1024 threads per 64 KiB chunk re-reading its own
 * chunk (4 writable bytes at `dst`): with 16 MiB (one workgroup per compute unit, 2 MiB per XCD) every pass after the
 * first is served by the L2s, which is the rate the operand streams of the tiled kernels are priced against.
 * Has no counterpart in the reference.
 */
#define ROCWMMA_AMD_STREAM_RESIDENT_PASSES 256
int rocwmma_amd_bench_stream(int mode, const void* src, void* dst, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* ROCWMMA_AMD_AUX_H */
