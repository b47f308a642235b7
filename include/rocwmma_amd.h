/*
 * rocwmma_amd.h -- C ABI of librocwmma_amd.so: the GEMM / GEMV / DLRM workloads built on the
 * gfx950 wave-level MMA headers in include/rocwmma/.
 *
 * The reference (rocWMMA) is a header-only device library with no host library; what a caller
 * of its workloads binds to today are the kernel launches inside its sample / test hosts.  Each
 * entry point below names the reference launch it stands in for.
 *
 * Conventions (all entry points):
 *   - every pointer is a DEVICE pointer owned by the caller; nothing is allocated or freed;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the null stream) and
 *     the call returns without waiting for it; a call enqueues kernels only (no memset or copy
 *     nodes), so it may be recorded into a HIP graph and replayed
 *     (tests/test_gpu_graph_replay.py);
 *   - leading dimensions are in elements;
 *   - the return value is a rocwmma_amd_status (0 = success); a non-zero status means nothing
 *     was launched.  The reference's hosts exit() on HIP errors (samples/common.hpp:34-46) and
 *     print "Unsupported size!" for shapes they reject (samples/simple_hgemm.cpp:144-149);
 *     here both become status codes;
 *   - calls are re-entrant and thread safe; the only state the library keeps is a per-device cache
 *     of immutable device properties (compute-unit count, architecture).
 */
#ifndef ROCWMMA_AMD_H
#define ROCWMMA_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum rocwmma_amd_dtype
{
    ROCWMMA_AMD_F16  = 0, /* IEEE binary16                       */
    ROCWMMA_AMD_BF16 = 1, /* bfloat16                            */
    ROCWMMA_AMD_E4M3 = 2, /* OCP FP8 E4M3 (rocwmma::float8_t)    */
    ROCWMMA_AMD_E5M2 = 3, /* OCP FP8 E5M2 (rocwmma::bfloat8_t)   */
    ROCWMMA_AMD_I8   = 4,
    ROCWMMA_AMD_F32  = 5,
    ROCWMMA_AMD_I32  = 6
} rocwmma_amd_dtype;

typedef enum rocwmma_amd_layout
{
    ROCWMMA_AMD_ROW_MAJOR = 0,
    ROCWMMA_AMD_COL_MAJOR = 1
} rocwmma_amd_layout;

typedef enum rocwmma_amd_status
{
    ROCWMMA_AMD_OK                = 0,
    ROCWMMA_AMD_INVALID_ARGUMENT  = 1, /* null pointer, zero size, bad enum                  */
    ROCWMMA_AMD_UNSUPPORTED_TYPE  = 2, /* dtype combination has no kernel                    */
    ROCWMMA_AMD_UNSUPPORTED_SHAPE = 3, /* size not a multiple of the block the kernel needs  */
    ROCWMMA_AMD_BAD_ALIGNMENT     = 4, /* pointer or leading dimension not 16-byte aligned   */
    ROCWMMA_AMD_BAD_LEADING_DIM   = 5, /* leading dimension smaller than the matrix extent   */
    ROCWMMA_AMD_NO_DEVICE         = 6, /* no gfx950 device is current                        */
    ROCWMMA_AMD_LAUNCH_FAILED     = 7, /* hipGetLastError() reported a launch failure        */
    ROCWMMA_AMD_SCRATCH_TOO_SMALL = 8  /* the library's static scratch cannot hold what this
                                          device needs (rocwmma_amd_gemm_streamk_static)     */
} rocwmma_amd_status;

/* Which GEMM kernel family rocwmma_amd_gemm_ex runs. */
typedef enum rocwmma_amd_gemm_algo
{
    ROCWMMA_AMD_GEMM_AUTO      = 0, /* blocked kernel when the shape allows, else wave-tile */
    ROCWMMA_AMD_GEMM_WAVE_TILE = 1, /* one block per wave, operands straight from global    */
    ROCWMMA_AMD_GEMM_BLOCKED   = 2, /* LDS multi-buffered macro-tile kernel                 */
    ROCWMMA_AMD_GEMM_BLOCKED_256 = 3 /* the same with its 256 x 256 tile forced, however few
                                        compute units that tiling occupies (AUTO and BLOCKED
                                        fall back to 128 x 128 tiles below half occupancy)  */
} rocwmma_amd_gemm_algo;

/* Activation applied by rocwmma_amd_gemm_bias_act. */
typedef enum rocwmma_amd_activation
{
    ROCWMMA_AMD_ACT_NONE = 0,
    ROCWMMA_AMD_ACT_RELU = 1, /* max(x, 0)                          */
    ROCWMMA_AMD_ACT_GELU = 2  /* x * (1 + erf(x / sqrt(2))) / 2     */
} rocwmma_amd_activation;

/* Library identification: returns 10000*major + 100*minor + patch. */
int rocwmma_amd_version(void);

/* Static, human readable text for a status code. */
const char* rocwmma_amd_status_string(int status);

/* Properties of the current device the benchmarks report next to their numbers:
 * compute-unit count, peak engine clock in MHz, and whether it is gfx950. */
int rocwmma_amd_device_info(int* compute_units, int* clock_mhz, int* is_gfx950);

/*
 * D = alpha * A * B + beta * C.
 *
 * Stands in for the kernel launches of the reference's GEMM hosts, whose kernels all take
 * (m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta):
 *   samples/simple_hgemm.cpp:81-93,202      (hgemm_rocwmma_d: one block per wave)
 *   samples/perf_hgemm.cpp:518-530,848-870  (gemm_rocwmma_d: LDS double-buffered macro tile)
 *   test/gemm/gemm_kernel_base.hpp          (KernelFunc, the test-suite generalisation)
 *
 * A is m x k, B is k x n, C and D are m x n; C and D share `layout_c`.
 * dtype_in  : element type of A and B (F16, BF16, E4M3, E5M2, I8, F32).
 * dtype_out : element type of C and D: F32 for the float inputs (F16 also allowed with F16
 *             inputs, BF16 with BF16 inputs), I32 or I8 for I8.  These are the Input/Output/Compute
 *             triples of the reference's GEMM tests (test/gemm/gemm_common_test_params.hpp:51-111).
 *             The compute type is f32 (i32 for I8); alpha and beta are converted to it (for I8
 *             they must be integers).  I8 results keep the low eight bits of the 32-bit result, as
 *             the reference's static_cast<int8_t> does (test/reference_impl.hpp:77-78).
 * c may be NULL when beta == 0.  c may equal d.
 * Shapes: m and n multiples of 16, k a multiple of 32 bytes' worth of elements per row is the
 * minimum every kernel accepts (k % 16 == 0 for 16-bit types, k % 32 == 0 for 8-bit types);
 * the blocked kernel additionally needs k in whole 64-byte stages and at least three of them, takes every
 * type in all four A/B layout pairs (m, n that do not fill whole tiles run on partly filled edge tiles)
 * and is chosen automatically, as are the weight-streaming kernels for up to 48 rows of A against a
 * col-major B.
 * One of those (48 rows against few columns or little K, or a 16-bit A of 16 / 32 rows too large for the
 * LDS; wide 48-row problems run on the blocked kernel) runs as two launches on the
 * stream and adds its K slices into D with atomic adds: I32 results are exact, F32 results can differ
 * in the last bit from run to run.
 * Alignment: base pointers and leading dimensions must be multiples of 16 bytes.
 */
int rocwmma_amd_gemm(int         dtype_in,
                     int         dtype_out,
                     int         layout_a,
                     int         layout_b,
                     int         layout_c,
                     uint32_t    m,
                     uint32_t    n,
                     uint32_t    k,
                     const void* a,
                     uint32_t    lda,
                     const void* b,
                     uint32_t    ldb,
                     const void* c,
                     uint32_t    ldc,
                     void*       d,
                     uint32_t    ldd,
                     float       alpha,
                     float       beta,
                     void*       stream);

/* Same as rocwmma_amd_gemm with the kernel family forced (`algo` is a rocwmma_amd_gemm_algo).
 * ROCWMMA_AMD_GEMM_BLOCKED returns ROCWMMA_AMD_UNSUPPORTED_SHAPE when k is not in whole stages, and
 * _BLOCKED_256 when the shape does not fill whole 256 x 256 tiles, like the reference's perf_hgemm host
 * (samples/perf_hgemm.cpp:735-765). */
int rocwmma_amd_gemm_ex(int         algo,
                        int         dtype_in,
                        int         dtype_out,
                        int         layout_a,
                        int         layout_b,
                        int         layout_c,
                        uint32_t    m,
                        uint32_t    n,
                        uint32_t    k,
                        const void* a,
                        uint32_t    lda,
                        const void* b,
                        uint32_t    ldb,
                        const void* c,
                        uint32_t    ldc,
                        void*       d,
                        uint32_t    ldd,
                        float       alpha,
                        float       beta,
                        void*       stream);

/*
 * D = alpha * A * B + beta * C with the tile count balanced over the compute units ("stream-K").
 *
 * Same arguments and semantics as rocwmma_amd_gemm.  The plain kernel runs one 256 x 256 tile per
 * workgroup, in rounds of one tile per compute unit, so a tile count that is not a multiple of the
 * unit count leaves units idle in the last round (m = 4096, n = 14336: 896 tiles = 3.5 rounds on
 * 256 units; 3072^3: 144 tiles).  Here one persistent workgroup per unit takes whole tiles plus an
 * equal share of the K range of the remaining ones; tiles shared by several workgroups are summed
 * through `workspace`, in a fixed order (results are reproducible; I32 results are exact, F32 results
 * differ from rocwmma_amd_gemm's only in how partial sums are rounded).
 * The reference has no counterpart: its GEMM hosts launch plain 2-D grids
 * (samples/perf_hgemm.cpp:810-812).
 *
 * Types: F16 / BF16 inputs with F32 C/D, I8 -> I32 and E4M3 / E5M2 -> F32, each in every layout
 * pair.  m and n multiples of 256, k a multiple of 128 bytes' worth of
 * elements; other shapes return ROCWMMA_AMD_UNSUPPORTED_SHAPE (use rocwmma_amd_gemm).
 * workspace: device memory, 256-byte aligned, at least rocwmma_amd_gemm_streamk_workspace_size()
 * bytes (64 MiB + 1.25 KiB on a 256-unit device); contents need not be initialised and are not
 * preserved.  Two calls that use the same workspace must not overlap in time.
 * The call enqueues two kernels on `stream` (a small one that clears the flags, then the GEMM).
 */
size_t rocwmma_amd_gemm_streamk_workspace_size(void);

int rocwmma_amd_gemm_streamk(int         dtype_in,
                             int         dtype_out,
                             int         layout_a,
                             int         layout_b,
                             int         layout_c,
                             uint32_t    m,
                             uint32_t    n,
                             uint32_t    k,
                             const void* a,
                             uint32_t    lda,
                             const void* b,
                             uint32_t    ldb,
                             const void* c,
                             uint32_t    ldc,
                             void*       d,
                             uint32_t    ldd,
                             float       alpha,
                             float       beta,
                             void*       workspace,
                             size_t      workspace_bytes,
                             void*       stream);

/*
 * Reports whether a stream-K launch on `workspace` (NULL: the static scratch of
 * rocwmma_amd_gemm_streamk_static on the current device) gave up waiting since the last query.
 *
 * In the stream-K kernel the workgroup that owns a shared tile waits for the workgroups that computed the
 * other parts of its K range.  Workgroups draw their ranges in the order they start (a ticket counter in
 * the workspace), and a range only ever waits for ranges of earlier tickets, which compute the awaited
 * part first and without waiting themselves, so the wait ends whatever order the device starts workgroups
 * in.  It is bounded all the same (2^22 polls): should it run out, the owner stops waiting, D holds wrong
 * values for that tile, and the kernel leaves the value 0x54494D45 in the word at byte offset
 * units * (65536 * 4) + units * 4 of the workspace (units = compute units of the device; the flags
 * start at units * 65536 * 4).  Launches never clear that word; this call does, after reporting it, so a later launch
 * cannot hide an earlier failure.  A workspace that has never been written reads as "no time-out" unless
 * it happens to hold that value.
 *
 * Waits for `stream` (the launches to be checked must have been enqueued there or be complete), copies four
 * bytes to the host, allocates nothing; not for use under graph capture.  *timed_out receives 0 or 1.
 * Has no counterpart in the reference (its kernels never wait for one another).
 */
int rocwmma_amd_gemm_streamk_timed_out(void* workspace, size_t workspace_bytes, void* stream, int* timed_out);

/*
 * rocwmma_amd_gemm_streamk without a workspace argument and without any allocation: for callers that
 * cannot allocate device memory (code under HIP graph capture, tight serving loops, harnesses that
 * forbid it).  It has no counterpart in the reference.  The workspace is a static device array inside
 * the library: 64 MiB + 1.25 KiB, enough for devices of up to 256 compute units
 * (ROCWMMA_AMD_SCRATCH_TOO_SMALL on larger ones), which every GPU the library runs on holds until
 * the process ends.  The entry point calls no hipMalloc / hipFree and no allocating library routine;
 * the first call on a device for a type and layout pair resolves the array's device address and sets the
 * kernel's LDS attribute (host-side queries, no allocation): make that call outside a graph capture;
 * the flags in the scratch are cleared by a small kernel on `stream` in front of the GEMM.  All calls
 * on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two
 * threads) race, so serialise them, or give the overlapping ones workspaces of their own through
 * rocwmma_amd_gemm_streamk.
 */
int rocwmma_amd_gemm_streamk_static(int         dtype_in,
                                    int         dtype_out,
                                    int         layout_a,
                                    int         layout_b,
                                    int         layout_c,
                                    uint32_t    m,
                                    uint32_t    n,
                                    uint32_t    k,
                                    const void* a,
                                    uint32_t    lda,
                                    const void* b,
                                    uint32_t    ldb,
                                    const void* c,
                                    uint32_t    ldc,
                                    void*       d,
                                    uint32_t    ldd,
                                    float       alpha,
                                    float       beta,
                                    void*       stream);

/*
 * GEMM with a fused epilogue:  D = act(alpha * A * B + beta * C + bias[j])  for column j of D.
 *
 * The reference's GEMM kernels end with D = alpha * acc + beta * C on fragments
 * (samples/perf_hgemm.cpp:683-713) and leave bias and activation to further kernels, i.e. to two more
 * passes over D; here they are applied to the accumulators on their way out.  Arguments and limits are
 * those of rocwmma_amd_gemm with
 *   dtype_in / dtype_out : the float triples only (F16, BF16, E4M3, E5M2 inputs; F32, or F16 / BF16 with
 *                          inputs of the same type); the sum and the activation are computed in f32;
 *   bias       : n floats (device memory, 16-byte aligned), or NULL for none;
 *   activation : a rocwmma_amd_activation.
 * Row-major C/D with k in whole 64-byte stages (at least three) runs on the blocked kernel, everything
 * else one block per wave.
 */
int rocwmma_amd_gemm_bias_act(int          dtype_in,
                              int          dtype_out,
                              int          layout_a,
                              int          layout_b,
                              int          layout_c,
                              uint32_t     m,
                              uint32_t     n,
                              uint32_t     k,
                              const void*  a,
                              uint32_t     lda,
                              const void*  b,
                              uint32_t     ldb,
                              const void*  c,
                              uint32_t     ldc,
                              void*        d,
                              uint32_t     ldd,
                              float        alpha,
                              float        beta,
                              const float* bias,
                              int          activation,
                              void*        stream);

/*
 * Block-scaled ("microscaled", MX) fp8 GEMM:
 *     D = alpha * (A . 2^(scale_a - 127)) * (B . 2^(scale_b - 127)) + beta * C.
 *
 * A and B hold E4M3 or E5M2 elements (dtype_in); every 32 consecutive elements along K of a row of A
 * and of a column of B share one E8M0 scale, a biased power-of-two exponent (the MXFP8 formats of the
 * OCP Microscaling Formats specification v1.0; scale 255 encodes NaN).  C and D are F32.  On gfx950 the
 * scales are applied inside the matrix cores (v_mfma_scale_f32_*_f8f6f4).
 * The reference has no counterpart: its fp8 GEMMs multiply unscaled operands
 * (test/gemm/gemm_common_test_params.hpp:170-196).  Arguments are those of rocwmma_amd_gemm plus
 *   scale_a : m x (k / 32) bytes, K blocks of a row contiguous, leading dimension ld_scale_a >= k / 32;
 *   scale_b : n x (k / 32) bytes, K blocks of a column of B contiguous, ld_scale_b >= k / 32;
 * whatever the layouts of A and B themselves.
 * Shapes: m, n multiples of 16 and k a multiple of 128, or m, n multiples of 32 and k a multiple of 64.
 * workspace: NULL, or device memory (256-byte aligned) of at least
 * rocwmma_amd_gemm_mx_workspace_size(m, n, k) bytes.  With a workspace, row-major A / col-major B
 * (for a col-major C: col-major A / row-major B) with k a multiple of 128 run on the blocked kernels
 * (256 x 256 tiles of v_mfma_scale_f32_16x16x128_f8f6f4 blocks when m and n are multiples of 256 and the
 * tiles occupy at least half of the compute units, else 128 x 128 or 128 x 64 tiles of 32x32x64 blocks with
 * partly filled edge tiles): the call then
 * enqueues a small kernel that re-orders the scales into the workspace, and the GEMM (two launches).  Everything else
 * runs one block per wave straight from global memory, except up to 32 rows of a row-major A against a
 * col-major B with k a multiple of 1024 (few tokens against a wide weight matrix), which run on the
 * weight-streaming kernel with or without a workspace (m * k <= 128 KiB; scale_a 4-byte aligned with
 * ld_scale_a a multiple of 4, scale_b 16-byte aligned with ld_scale_b a multiple of 16).  Two calls
 * that use the same workspace must not overlap in time.
 */
size_t rocwmma_amd_gemm_mx_workspace_size(uint32_t m, uint32_t n, uint32_t k);

int rocwmma_amd_gemm_mx(int         dtype_in,
                        int         layout_a,
                        int         layout_b,
                        int         layout_c,
                        uint32_t    m,
                        uint32_t    n,
                        uint32_t    k,
                        const void* a,
                        uint32_t    lda,
                        const void* scale_a,
                        uint32_t    ld_scale_a,
                        const void* b,
                        uint32_t    ldb,
                        const void* scale_b,
                        uint32_t    ld_scale_b,
                        const void* c,
                        uint32_t    ldc,
                        void*       d,
                        uint32_t    ldd,
                        float       alpha,
                        float       beta,
                        void*       workspace,
                        size_t      workspace_bytes,
                        void*       stream);

/*
 * The two halves of rocwmma_amd_gemm_mx's blocked path as calls of their own, for callers whose scales
 * outlive a call (a weight matrix multiplied again and again): re-ordering the scales takes a launch of
 * its own (6-7 us for the 1.9 MB of scales of a 4096 x 14336 x 4096 problem), a fifth of the time of a
 * 128-row problem.  They have no counterpart in the reference.
 *
 * rocwmma_amd_gemm_mx_pack_scales re-orders the scales of a problem of this shape and these layouts into
 * `workspace` (as for rocwmma_amd_gemm_mx: 256-byte aligned, at least rocwmma_amd_gemm_mx_workspace_size
 * bytes).  scale_a or scale_b may be NULL: that operand's part of the workspace is left as it is (pack the
 * weights' scales once, the tokens' scales per call).  The packed order depends on m, n and k (which tile
 * the GEMM will run on), so a workspace serves calls with the shape it was packed for.
 * ROCWMMA_AMD_UNSUPPORTED_SHAPE for problems the blocked kernels do not take (see rocwmma_amd_gemm_mx:
 * row-major A / col-major B, or the transposed pairing for a col-major C; m, n multiples of 16; k a
 * multiple of 128).
 *
 * rocwmma_amd_gemm_mx_packed is rocwmma_amd_gemm_mx on a workspace filled by rocwmma_amd_gemm_mx_pack_scales
 * for the same m, n, k and layouts: one launch, the GEMM.  It does not write the workspace, so calls that
 * share one may overlap.  Same shape rule; it never falls back to another kernel.
 */
int rocwmma_amd_gemm_mx_pack_scales(int         layout_a,
                                    int         layout_b,
                                    int         layout_c,
                                    uint32_t    m,
                                    uint32_t    n,
                                    uint32_t    k,
                                    const void* scale_a,
                                    uint32_t    ld_scale_a,
                                    const void* scale_b,
                                    uint32_t    ld_scale_b,
                                    void*       workspace,
                                    size_t      workspace_bytes,
                                    void*       stream);

int rocwmma_amd_gemm_mx_packed(int         dtype_in,
                               int         layout_a,
                               int         layout_b,
                               int         layout_c,
                               uint32_t    m,
                               uint32_t    n,
                               uint32_t    k,
                               const void* a,
                               uint32_t    lda,
                               const void* b,
                               uint32_t    ldb,
                               const void* c,
                               uint32_t    ldc,
                               void*       d,
                               uint32_t    ldd,
                               float       alpha,
                               float       beta,
                               const void* workspace,
                               size_t      workspace_bytes,
                               void*       stream);

/*
 * Skinny GEMV / GEMM:  Y = alpha * A * X + beta * Y,  in place on Y.
 *
 * Stands in for sgemv_rocwmma_d and its host (samples/simple_sgemv.cpp:103-155,207-227), whose
 * semantics are those of its CPU twin sgemv_cpu_h (samples/simple_sgemv.cpp:46-66); here for
 * f16 A and up to 8 right-hand sides, as a pure bandwidth kernel (no MFMA).
 *
 * A : m x k, f16, row-major, leading dimension lda >= k.
 * X : k x ncols, f16, column-major (each right-hand side contiguous), ldx >= k.
 * Y : m x ncols, f32, column-major, ldy >= m.  Read only when beta != 0.
 * ncols in {1, 2, 4, 8}; k a multiple of 8; A, X 16-byte aligned with lda, ldx multiples of 8.
 */
int rocwmma_amd_gemv(uint32_t    m,
                     uint32_t    k,
                     uint32_t    ncols,
                     const void* a,
                     uint32_t    lda,
                     const void* x,
                     uint32_t    ldx,
                     float*      y,
                     uint32_t    ldy,
                     float       alpha,
                     float       beta,
                     void*       stream);

/*
 * DLRM dot-interaction, forward.  f16 in / out, f32 accumulate.
 *
 * Stands in for dlrmDotFwd and its launch (samples/simple_dlrm.cpp:184-284,504-529;
 * test/dlrm/device/dlrm_dot_fwd.hpp:38).  Semantics = dlrm_fwd_CPU
 * (test/reference_impl.hpp:83-119):
 *   input  : batch x m x k   (row 0 of every sample is the bottom-MLP output)
 *   output : batch x (k + m(m-1)/2):  [ input[b,0,:] , Z[1,0], Z[2,0], Z[2,1], Z[3,0], ... ]
 *            with Z = input[b] * input[b]^T.
 * Unlike the reference kernel this one needs no f32 m x m scratch (`acc`) and accepts any m up to 32768
 * (the reference GPU kernels need m % 16 == 0, test/dlrm/dlrm_kernel_base_impl.hpp:146-150; its tests run
 * (m, k) = (32, 32), (32, 128), (128, 128) and (1024, 1024), test/dlrm/test/dlrm_test_params.hpp:51-68).  Up to 32 rows
 * with k in {32, 64, 128, 256} are one matrix-instruction operand per sample (the benchmark configuration, m = 27), up
 * to 128 rows run as tiles of 32 inside one wave per sample; every other shape runs as 128 x 128 tiles per workgroup
 * and needs k % 8 == 0 and a sample's features (m * k * 2 bytes) below 2 GiB, ROCWMMA_AMD_UNSUPPORTED_SHAPE otherwise.
 * input and output must be 16-byte aligned.
 */
int rocwmma_amd_dlrm_fwd(const void* input,
                         void*       output,
                         uint32_t    m,
                         uint32_t    k,
                         uint32_t    batch,
                         void*       stream);

/*
 * DLRM dot-interaction, backward.
 *
 * Stands in for trilReconstruct + dlrmDotBwd and their launches
 * (samples/simple_dlrm.cpp:290-441,534-587; test/dlrm/device/dlrm_dot_bwd.hpp:36,80) in ONE
 * launch with no m x m scratch and no host synchronisation in between.  Semantics =
 * dlrm_bwd_CPU (test/reference_impl.hpp:121-179):
 *   upstream_grad   : batch x (k + m(m-1)/2)
 *   bottom_mlp_grad : batch x k        = upstream_grad[b, 0:k]
 *   grad            : batch x m x k    = G * input[b],  G = symmetric matrix rebuilt from the
 *                     packed strict lower triangle upstream_grad[b, k:], zero diagonal.
 * The bottom-MLP gradient is NOT added into grad row 0 (neither does the reference).
 * Same shape limits as the forward pass.
 */
int rocwmma_amd_dlrm_bwd(const void* input,
                         const void* upstream_grad,
                         void*       grad,
                         void*       bottom_mlp_grad,
                         uint32_t    m,
                         uint32_t    k,
                         uint32_t    batch,
                         void*       stream);

/*
 * The two DLRM passes with the element type as an argument: ROCWMMA_AMD_F16 (the entry points above) or
 * ROCWMMA_AMD_F32.  The reference's DLRM kernels and tests are templates over the element type and are
 * instantiated for float32_t as well (test/dlrm/test/dlrm_test_params.hpp:51; fp32 data files under
 * test/dlrm/data); semantics = dlrm_fwd_CPU / dlrm_bwd_CPU with DataT = float (test/reference_impl.hpp:83-179).
 * Same shapes, limits and alignment as above (float32: k % 4 == 0 for the shapes that run as 128 x 128 tiles,
 * m * k * 4 bytes below 2 GiB; 16-byte aligned pointers); the float32 kernels multiply with v_mfma_f32_32x32x2_f32
 * and are written for parity, not tuned.  Other element
 * types: ROCWMMA_AMD_UNSUPPORTED_TYPE.
 */
int rocwmma_amd_dlrm_fwd_ex(int         dtype,
                            const void* input,
                            void*       output,
                            uint32_t    m,
                            uint32_t    k,
                            uint32_t    batch,
                            void*       stream);

int rocwmma_amd_dlrm_bwd_ex(int         dtype,
                            const void* input,
                            const void* upstream_grad,
                            void*       grad,
                            void*       bottom_mlp_grad,
                            uint32_t    m,
                            uint32_t    k,
                            uint32_t    batch,
                            void*       stream);

#ifdef __cplusplus
}
#endif

#endif /* ROCWMMA_AMD_H */
