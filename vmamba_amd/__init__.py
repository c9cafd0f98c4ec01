"""vmamba_amd -- MI355X-native SS2D inference hot path (CrossScan -> selective scan -> CrossMerge).

Host code is Python and mirrors the reference's operator API; the kernels are hand-written HIP
for gfx950 behind a C ABI (include/ss2d_hip.h, libss2d_hip.so).
"""
from .csm import cross_scan_fn, cross_merge_fn  # noqa: F401
from .csms6s import selective_scan_bwd, selective_scan_fn, selective_scan_fwd  # noqa: F401

__all__ = ["cross_scan_fn", "cross_merge_fn", "selective_scan_fn", "selective_scan_fwd", "selective_scan_bwd"]
