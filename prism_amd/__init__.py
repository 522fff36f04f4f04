"""prism_amd: MI355X (gfx950) kernels for the data-parallel path of manya-bansal/prism.

Hand-written HIP kernels (add_m, single-pass look-back scan, the fp32 SGEMM
progression, a bf16 MFMA GEMM) behind a C-ABI shared library
(include/prism_amd.h), with this package as the ctypes-level host mirror of the
reference's launchers. Importing the package does not touch the GPU; the first
call loads (and, if the file is absent, builds) libprism_amd.so.
"""
from .ops import (  # noqa: F401
    PrismError,
    ScanOrderError,
    ScanWorkspaceError,
    SGEMM_KERNELS,
    add_m,
    device_info,
    gemm_bf16,
    get_workspace_size,
    launch_scan,
    new_scan_workspace,
    run_my_kernel,
    runmyh100,
    scan,
    scan_status,
    scan_workspace_init,
    segmented_scan,
    sgemm,
    sgemm_workspace_plan,
    sgemm_workspace_size,
    tile_coords,
    wave_regroup,
)

__version__ = "0.1.0"
