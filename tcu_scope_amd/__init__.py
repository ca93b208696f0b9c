"""tcu_scope_amd — MI355X (gfx950) implementation of the tcu_scope hot path.

The product is ``libtcu_scope_amd.so`` (C ABI in ``include/tcu_scope.h``, HIP sources in
``tcu_scope_amd/csrc``) and the C++ benchmark harness in ``tcu_scope_amd/host``.  This
module is a thin ctypes view of the C ABI for Python callers: torch is used only to own
device memory and streams.  There is no CPU fallback: if the shared library is missing,
importing a function from here raises.
"""
from .binding import (  # noqa: F401
    TcuError,
    VARIANTS,
    Variant,
    FullStrategy,
    FULL_MFMA,
    Dist,
    add_partial_sums,
    build,
    device_info,
    fill,
    convert_f32_to_f16,
    full_reduce,
    full_scan,
    gemm,
    gemv,
    gemv_col_major,
    generate,
    init,
    lane_probe,
    lib,
    library_path,
    seg_reduce,
    seg_reduce_offsets,
    seg_scan_offsets,
    seg_scan,
    seg_scan_noalloc,
    seg_scan_by_key,
    seg_reduce_by_key,
    set_option,
    stream_probe,
    temporary_allocations,
    time_next_launch,
)
