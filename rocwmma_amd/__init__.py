"""rocwmma_amd: host-side front end of librocwmma_amd.so, the GEMM / GEMV / DLRM workloads built
on the gfx950 wave-level MMA headers under include/rocwmma/.

Everything here calls the HIP library through its C ABI (include/rocwmma_amd.h); there is no
CPU fallback: a missing library or a non-gfx950 device raises."""
from .api import (  # noqa: F401
    ACT_GELU, ACT_NONE, ACT_RELU, BF16, COL_MAJOR, E4M3, E5M2, F16, F32, GEMM_AUTO, GEMM_BLOCKED, GEMM_BLOCKED_256, GEMM_WAVE_TILE, I8, I32, ROW_MAJOR,
    MFMA_BF16_16X16X32, MFMA_BF16_32X32X16, MFMA_F8_16X16X128, MFMA_F8_16X16X128_SCALED, MFMA_F8_32X32X64, MFMA_F16_16X16X32, MFMA_F16_32X32X16,
    MFMA_I8_16X16X64, MFMA_I8_32X32X32,
    RocwmmaError, STREAM_COPY, STREAM_COPY_READ_MORE, STREAM_READ, STREAM_READ_RESIDENT, STREAM_RESIDENT_PASSES, STREAM_WRITE, STREAMS_F16, STREAMS_FP8, STREAMS_I8, aux_library, aux_library_path, bench_mfma_ceiling, bench_mfma_streams, bench_stream, device_info, dlrm_bwd, dlrm_fwd, gemm, gemm_bias_act, gemm_mx, gemm_mx_pack_scales, gemm_mx_packed, gemm_mx_workspace_size, gemm_raw, gemm_streamk, gemm_streamk_static, gemm_streamk_timed_out, gemm_streamk_workspace_size, gemv,
    library, library_path, selftest_coop_gemm, selftest_roundtrip, selftest_tiled_gemm, status_string, version,
)
