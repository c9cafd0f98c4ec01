"""ctypes binding of libss2d_hip.so (the C ABI declared in include/ss2d_hip.h).

There is no CPU fallback: if the library has not been built, loading fails loudly.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libss2d_hip.so")

SS2D_F32, SS2D_BF16, SS2D_F16 = 0, 1, 2
SS2D_OK, SS2D_EINVAL, SS2D_ENOTSUP, SS2D_ELAUNCH, SS2D_ENOMEM = 0, -22, -95, -5, -12
MERGE_PAIRWISE, MERGE_LEFT_TO_RIGHT = 0, 1
SCAN_CHUNK = 2048
STATIC_STAGING_BYTES = 80 << 20
ABI_VERSION = 1

SCAN_KERNEL_NONE, SCAN_KERNEL_ROW, SCAN_KERNEL_ROW4, SCAN_KERNEL_FLAT, SCAN_KERNEL_SMALL, SCAN_KERNEL_CHAN = range(6)
SCAN_KERNEL_NAMES = ("none", "row", "row4", "flat", "small", "chan")

EXPORTS = ("ss2d_abi_version", "ss2d_strerror", "ss2d_cross_scan", "ss2d_cross_merge", "ss2d_selective_scan_fwd",
           "ss2d_selective_scan_kernel", "ss2d_selective_scan_fwd_maps",
           "ss2d_layer_norm", "ss2d_add_layer_norm", "ss2d_bias_layer_norm", "ss2d_layer_norm_cf", "ss2d_dwconv3x3_silu", "ss2d_cross_scan_1b1", "ss2d_core_fwd",
           "ss2d_core_workspace_bytes", "ss2d_core_fwd_ws", "ss2d_core_mask_pads", "ss2d_core_embed_maps",
           "ss2d_dt_proj", "ss2d_dt_proj_masked", "ss2d_cross_scan_flex", "ss2d_cross_scan_flex_ws", "ss2d_cross_scan_flex_static", "ss2d_cross_merge_flex",
           "ss2d_selective_scan_bwd", "ss2d_transpose_bcl", "ss2d_mlp_fused", "ss2d_linear_cl", "ss2d_linear_cf_ln", "ss2d_stem_conv_ln_gelu", "ss2d_mean_pool_cl")


class ScanParams(ctypes.Structure):
    """struct ss2d_scan_params (include/ss2d_hip.h)."""
    _fields_ = (
        [(n, ctypes.c_int32) for n in ("batch", "dim", "seqlen", "dstate", "n_groups", "delta_dim",
                                       "in_dtype", "out_dtype", "delta_softplus", "reserved")]
        + [(n, ctypes.c_void_p) for n in ("u", "delta", "A", "B", "C", "D", "delta_bias", "out", "x")]
        + [(n, ctypes.c_int64) for n in ("u_batch_stride", "u_d_stride", "delta_batch_stride", "delta_d_stride",
                                         "A_d_stride", "A_dstate_stride",
                                         "B_batch_stride", "B_group_stride", "B_dstate_stride",
                                         "C_batch_stride", "C_group_stride", "C_dstate_stride",
                                         "out_batch_stride", "out_d_stride")]
    )


class ScanBwdParams(ctypes.Structure):
    """struct ss2d_scan_bwd_params (include/ss2d_hip.h)."""
    _fields_ = (
        [(n, ctypes.c_int32) for n in ("batch", "dim", "seqlen", "dstate", "n_groups", "delta_dim",
                                       "in_dtype", "dout_dtype", "delta_softplus", "reserved")]
        + [(n, ctypes.c_void_p) for n in ("u", "delta", "A", "B", "C", "D", "delta_bias", "dout",
                                          "du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias")]
        + [(n, ctypes.c_int64) for n in ("u_batch_stride", "u_d_stride", "delta_batch_stride", "delta_d_stride",
                                         "A_d_stride", "A_dstate_stride",
                                         "B_batch_stride", "B_group_stride", "B_dstate_stride",
                                         "C_batch_stride", "C_group_stride", "C_dstate_stride",
                                         "dout_batch_stride", "dout_d_stride")]
    )


class CoreParams(ctypes.Structure):
    """struct ss2d_core_params (include/ss2d_hip.h)."""
    _fields_ = (
        [(n, ctypes.c_int32) for n in ("batch", "dim", "height", "width", "in_dtype", "delta_softplus")]
        + [(n, ctypes.c_void_p) for n in ("x", "delta", "A", "B", "C", "D", "delta_bias", "y")]
        + [(n, ctypes.c_int64) for n in ("delta_dir_stride", "delta_dim_stride", "delta_batch_stride",
                                         "B_dir_stride", "B_batch_stride", "C_dir_stride", "C_batch_stride")]
    )


class Ss2dError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__(f"{what}: {strerror(code)} (ss2d status {code})")


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build the HIP library first (python -m vmamba_amd.build). "
                "vmamba_amd has no CPU or PyTorch fallback for its kernels.")
        L = ctypes.CDLL(LIB_PATH)
        L.ss2d_abi_version.restype = ctypes.c_int
        L.ss2d_strerror.restype = ctypes.c_char_p
        L.ss2d_strerror.argtypes = [ctypes.c_int]
        L.ss2d_cross_scan.restype = ctypes.c_int
        L.ss2d_cross_scan.argtypes = [ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 5 + [ctypes.c_void_p]
        L.ss2d_cross_merge.restype = ctypes.c_int
        L.ss2d_cross_merge.argtypes = [ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 6 + [ctypes.c_void_p]
        L.ss2d_selective_scan_fwd.restype = ctypes.c_int
        L.ss2d_selective_scan_fwd.argtypes = [ctypes.POINTER(ScanParams), ctypes.c_void_p]
        L.ss2d_selective_scan_fwd_maps.restype = ctypes.c_int
        L.ss2d_selective_scan_fwd_maps.argtypes = [ctypes.POINTER(ScanParams), ctypes.c_void_p, ctypes.c_void_p]
        L.ss2d_selective_scan_kernel.restype = ctypes.c_int
        L.ss2d_selective_scan_kernel.argtypes = [ctypes.POINTER(ScanParams)]
        L.ss2d_layer_norm.restype = ctypes.c_int
        L.ss2d_layer_norm.argtypes = ([ctypes.c_void_p] * 4 + [ctypes.c_int64, ctypes.c_int, ctypes.c_float]
                                      + [ctypes.c_int] * 3 + [ctypes.c_void_p])
        L.ss2d_add_layer_norm.restype = ctypes.c_int
        L.ss2d_add_layer_norm.argtypes = ([ctypes.c_void_p] * 6 + [ctypes.c_int64, ctypes.c_int, ctypes.c_float]
                                          + [ctypes.c_int] * 3 + [ctypes.c_void_p])
        L.ss2d_stem_conv_ln_gelu.restype = ctypes.c_int
        L.ss2d_stem_conv_ln_gelu.argtypes = ([ctypes.c_void_p] * 2 + [ctypes.POINTER(ctypes.c_int64)] + [ctypes.c_void_p] * 3
                                             + [ctypes.c_float, ctypes.c_void_p] + [ctypes.c_int] * 5 + [ctypes.c_void_p])
        L.ss2d_bias_layer_norm.restype = ctypes.c_int
        L.ss2d_bias_layer_norm.argtypes = ([ctypes.c_void_p] * 5 + [ctypes.c_int64, ctypes.c_int, ctypes.c_float]
                                           + [ctypes.c_int] * 3 + [ctypes.c_void_p])
        L.ss2d_layer_norm_cf.restype = ctypes.c_int
        L.ss2d_layer_norm_cf.argtypes = ([ctypes.c_void_p] * 4 + [ctypes.c_int] * 3 + [ctypes.c_float]
                                         + [ctypes.c_int] * 4 + [ctypes.c_void_p])
        L.ss2d_dwconv3x3_silu.restype = ctypes.c_int
        L.ss2d_dwconv3x3_silu.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 7 + [ctypes.c_void_p]
        L.ss2d_cross_scan_1b1.restype = ctypes.c_int
        L.ss2d_cross_scan_1b1.argtypes = ([ctypes.c_void_p] * 2 + [ctypes.c_int] * 5 + [ctypes.c_int64] * 3
                                          + [ctypes.c_void_p])
        L.ss2d_core_fwd.restype = ctypes.c_int
        L.ss2d_core_fwd.argtypes = [ctypes.POINTER(CoreParams), ctypes.c_void_p]
        L.ss2d_core_workspace_bytes.restype = ctypes.c_int64
        L.ss2d_core_workspace_bytes.argtypes = [ctypes.POINTER(CoreParams)]
        L.ss2d_core_fwd_ws.restype = ctypes.c_int
        L.ss2d_core_fwd_ws.argtypes = [ctypes.POINTER(CoreParams), ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        L.ss2d_core_embed_maps.restype = ctypes.c_int
        L.ss2d_core_embed_maps.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                           ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
        L.ss2d_core_mask_pads.restype = ctypes.c_int
        L.ss2d_core_mask_pads.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 6 + [ctypes.c_int64] * 3 + [ctypes.c_int, ctypes.c_void_p]
        L.ss2d_dt_proj.restype = ctypes.c_int
        L.ss2d_dt_proj.argtypes = ([ctypes.c_void_p] * 3 + [ctypes.c_int] * 3 + [ctypes.c_int64] * 3 + [ctypes.c_int]
                                   + [ctypes.c_void_p])
        L.ss2d_dt_proj_masked.restype = ctypes.c_int
        L.ss2d_dt_proj_masked.argtypes = ([ctypes.c_void_p] * 3 + [ctypes.c_float, ctypes.c_void_p] + [ctypes.c_int] * 3
                                          + [ctypes.c_int64] * 3 + [ctypes.c_int, ctypes.c_void_p])
        L.ss2d_cross_scan_flex.restype = ctypes.c_int
        L.ss2d_cross_scan_flex.argtypes = [ctypes.c_void_p] * 2 + [ctypes.c_int] * 9 + [ctypes.c_void_p]
        L.ss2d_cross_scan_flex_ws.restype = ctypes.c_int
        L.ss2d_cross_scan_flex_ws.argtypes = ([ctypes.c_void_p] * 2 + [ctypes.c_int] * 9 + [ctypes.c_void_p, ctypes.c_int64]
                                              + [ctypes.c_void_p])
        L.ss2d_cross_scan_flex_static.restype = ctypes.c_int
        L.ss2d_cross_scan_flex_static.argtypes = [ctypes.c_void_p] * 2 + [ctypes.c_int] * 9 + [ctypes.c_void_p]
        L.ss2d_cross_merge_flex.restype = ctypes.c_int
        L.ss2d_cross_merge_flex.argtypes = [ctypes.c_void_p] * 2 + [ctypes.c_int] * 10 + [ctypes.c_void_p]
        L.ss2d_selective_scan_bwd.restype = ctypes.c_int
        L.ss2d_selective_scan_bwd.argtypes = [ctypes.POINTER(ScanBwdParams), ctypes.c_void_p]
        L.ss2d_transpose_bcl.restype = ctypes.c_int
        L.ss2d_transpose_bcl.argtypes = [ctypes.c_void_p] * 2 + [ctypes.c_int] * 4 + [ctypes.c_void_p]
        L.ss2d_mlp_fused.restype = ctypes.c_int
        L.ss2d_mlp_fused.argtypes = ([ctypes.c_void_p] * 3 + [ctypes.c_float] + [ctypes.c_void_p] * 6 +
                                     [ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p])
        L.ss2d_linear_cl.restype = ctypes.c_int
        L.ss2d_linear_cl.argtypes = ([ctypes.c_void_p] * 3 + [ctypes.c_float] + [ctypes.c_void_p] * 4 +
                                     [ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p])
        L.ss2d_linear_cf_ln.restype = ctypes.c_int
        L.ss2d_linear_cf_ln.argtypes = ([ctypes.c_void_p] * 3 + [ctypes.c_float] + [ctypes.c_void_p] * 4 +
                                        [ctypes.c_int] * 5 + [ctypes.c_void_p])
        L.ss2d_mean_pool_cl.restype = ctypes.c_int
        L.ss2d_mean_pool_cl.argtypes = [ctypes.c_void_p] * 2 + [ctypes.c_int] * 4 + [ctypes.c_void_p]
        if L.ss2d_abi_version() != ABI_VERSION:
            raise ImportError(f"{LIB_PATH}: ABI version {L.ss2d_abi_version()} != expected {ABI_VERSION}; rebuild")
        _lib = L
    return _lib


def strerror(code):
    return lib().ss2d_strerror(int(code)).decode()


def check(code, what):
    if code != SS2D_OK:
        raise Ss2dError(code, what)
