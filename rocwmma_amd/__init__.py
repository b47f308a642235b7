"""rocwmma_amd: host-side front end of librocwmma_amd.so, the GEMM / GEMV / DLRM workloads built
on the gfx950 wave-level MMA headers under include/rocwmma/.

Everything here calls the HIP library through its C ABI (include/rocwmma_amd.h); there is no
CPU fallback: a missing library or a non-gfx950 device raises."""
from .api import (  # noqa: F401
    BF16, COL_MAJOR, E4M3, E5M2, F16, F32, GEMM_AUTO, GEMM_BLOCKED, GEMM_BLOCKED_256, GEMM_WAVE_TILE, I8, I32, ROW_MAJOR,
    RocwmmaError, device_info, dlrm_bwd, dlrm_fwd, gemm, gemm_raw, gemv, library, library_path,
    selftest_coop_gemm, selftest_roundtrip, status_string, version,
)
